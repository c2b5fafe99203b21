"""Reading and writing the safetensors container.

Layout (as the reference reads it, ginfer/model/loader/safetensor_loader.cc:13-42): 8 bytes
little-endian header length, a JSON header mapping tensor name to {dtype, shape, data_offsets}
(offsets relative to the first byte after the header; `__metadata__` is skipped), then raw
little-endian data.  The file is memory-mapped and tensors are zero-copy views of the mapping.
Unlike the reference, offsets and sizes are checked against the file before anything is read.
"""
import json
import mmap
import os
import struct

import torch

_DTYPES = {
    "F64": torch.float64, "F32": torch.float32, "F16": torch.float16, "BF16": torch.bfloat16,
    "I64": torch.int64, "I32": torch.int32, "I16": torch.int16, "I8": torch.int8, "U8": torch.uint8,
    "BOOL": torch.bool,
}
_NAMES = {v: k for k, v in _DTYPES.items()}


class SafetensorsError(ValueError):
    pass


class SafetensorsFile:
    def __init__(self, path):
        self.path = path
        size = os.path.getsize(path)
        if size < 8:
            raise SafetensorsError("%s: too short to be a safetensors file (%d bytes)" % (path, size))
        self._f = open(path, "rb")
        self._map = mmap.mmap(self._f.fileno(), 0, access=mmap.ACCESS_READ)
        (hlen,) = struct.unpack("<Q", self._map[:8])
        if hlen > size - 8:
            raise SafetensorsError("%s: header length %d exceeds the file (%d bytes)" % (path, hlen, size))
        try:
            header = json.loads(self._map[8:8 + hlen].decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise SafetensorsError("%s: header is not valid JSON: %s" % (path, e))
        self._base = 8 + hlen
        self.metadata = header.pop("__metadata__", None)
        self.entries = {}
        for name, e in header.items():
            dt = e.get("dtype")
            if dt not in _DTYPES:
                raise SafetensorsError("%s: tensor %r has unsupported dtype %r" % (path, name, dt))
            shape = tuple(int(s) for s in e["shape"])
            begin, end = (int(x) for x in e["data_offsets"])
            numel = 1
            for s in shape:
                numel *= s
            item = torch.empty(0, dtype=_DTYPES[dt]).element_size()
            if end - begin != numel * item:
                raise SafetensorsError("%s: tensor %r: data size mismatch (%d bytes for shape %s %s)"
                                       % (path, name, end - begin, list(shape), dt))
            if begin < 0 or self._base + end > size:
                raise SafetensorsError("%s: tensor %r lies outside the file" % (path, name))
            self.entries[name] = (_DTYPES[dt], shape, begin, end)

    def names(self):
        return list(self.entries)

    def info(self, name):
        dtype, shape, _, _ = self.entries[name]
        return dtype, shape

    def tensor(self, name):
        """A read-only CPU view of the mapping (copy before changing it)."""
        if name not in self.entries:
            raise SafetensorsError("%s: tensor not found: %s" % (self.path, name))
        dtype, shape, begin, end = self.entries[name]
        if end == begin:
            return torch.empty(shape, dtype=dtype)
        import warnings
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")   # the mapping is read-only by design
            flat = torch.frombuffer(self._map, dtype=dtype, count=(end - begin) // max(
                torch.empty(0, dtype=dtype).element_size(), 1), offset=self._base + begin)
        return flat.view(shape)

    def close(self):
        # views handed out keep the mapping alive through torch's buffer reference
        try:
            self._map.close()
        except BufferError:
            pass
        self._f.close()


def write_safetensors(path, tensors, metadata=None):
    """tensors: name -> CPU tensor.  Written in the given order, 8-byte aligned header."""
    header = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    offset = 0
    for name, t in tensors.items():
        if t.dtype not in _NAMES:
            raise SafetensorsError("tensor %r has dtype %s, which safetensors cannot hold" % (name, t.dtype))
        n = t.numel() * t.element_size()
        header[name] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape),
                        "data_offsets": [offset, offset + n]}
        offset += n
    blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
    blob += b" " * ((8 - len(blob) % 8) % 8)
    tmp = path + ".tmp"
    with open(tmp, "wb") as f:
        f.write(struct.pack("<Q", len(blob)))
        f.write(blob)
        for name, t in tensors.items():
            t = t.detach().contiguous().cpu()
            if t.numel():
                f.write(t.view(torch.uint8).numpy().tobytes() if t.dim() else
                        t.reshape(1).view(torch.uint8).numpy().tobytes())
    os.replace(tmp, path)


def open_model_files(folder):
    """name -> SafetensorsFile for a model folder: `model.safetensors`, or the shards that
    `model.safetensors.index.json` names (the reference reads the single file only,
    ginfer/model/qwen2.cc:32)."""
    single = os.path.join(folder, "model.safetensors")
    index = os.path.join(folder, "model.safetensors.index.json")
    files = {}
    if os.path.isfile(single):
        f = SafetensorsFile(single)
        return {n: f for n in f.names()}
    if os.path.isfile(index):
        with open(index) as fh:
            weight_map = json.load(fh)["weight_map"]
        for name, shard in weight_map.items():
            if shard not in files:
                files[shard] = SafetensorsFile(os.path.join(folder, shard))
        return {name: files[shard] for name, shard in weight_map.items()}
    raise SafetensorsError("no model.safetensors (or model.safetensors.index.json) in %s" % folder)
