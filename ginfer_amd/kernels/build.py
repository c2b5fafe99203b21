"""Compiling and loading the HIP kernels.

Each source under `ginfer_amd/csrc/` becomes one shared library, built with hipcc for gfx950 and
loaded with ctypes (the entry points are `extern "C"`; tensors cross as raw device pointers and the
launches go to the stream the caller names).  A library is built when it is first asked for and its
source (or common header, or flags) has changed since the last build; the build goes into
`csrc/_build/` inside the package, or, when that folder cannot be written, into a per-user folder
under the system's temporary directory.  There is no fallback: if a library can neither be found nor
built, loading raises.
"""
import ctypes
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import threading
import time

CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "csrc")
ARCH = "gfx950"
# packed 32-bit float instructions are switched off for all device code
FLAGS = ["--offload-arch=" + ARCH, "-O3", "-std=c++17", "-shared", "-fPIC",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument"]
MODULES = ("embedding", "norm", "rope_kv", "attention_generic", "attention_mfma", "gemm", "gemm_skinny",
           "activation", "sampling", "random_fill")
# flags of single modules: the random-weights generator must round every operation by itself, as the host's twin does
MODULE_FLAGS = {"random_fill": ["-ffp-contract=off"], "attention_generic": ["-ffp-contract=off"]}
# headers beside common.h that a module includes (they enter its digest)
MODULE_HEADERS = {"random_fill": ["random_normal.h"]}
# plain C++ libraries for the host (no GPU runtime), built with the host compiler from csrc/host/
HOST_MODULES = ("random_fill_host",)
HOST_FLAGS = ["-O2", "-std=c++17", "-shared", "-fPIC", "-pthread", "-ffp-contract=off"]
HOST_HEADERS = {"random_fill_host": ["random_normal.h"]}
# Modules that are compiled for one value of a parameter (a macro) at a time; build_all() without a
# list compiles these values, and any other value a model needs is compiled when it is first asked for.
VARIANTS = {"attention_mfma": [{"HEAD_DIM": hd} for hd in range(16, 257, 16)]}

_loaded = {}
_lock = threading.Lock()


class KernelBuildError(RuntimeError):
    pass


def available_modules():
    return [m for m in MODULES if os.path.isfile(os.path.join(CSRC, m + ".hip"))]


def _hipcc():
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand):
            return cand
    return None


def _split(module):
    """A module is named "source" or ("source", {macro: value}); returns (source, defines, library stem)."""
    if isinstance(module, str):
        return module, {}, module
    src, defines = module
    defines = dict(defines or {})
    stem = src + "".join("_%s%s" % (k, defines[k]) for k in sorted(defines))
    return src, defines, stem


def _digest(module):
    src, defines, _ = _split(module)
    h = hashlib.sha256()
    for name in [src + ".hip", "common.h", "ginfer_amd.h"] + MODULE_HEADERS.get(src, []):
        with open(os.path.join(CSRC, name), "rb") as f:
            h.update(f.read())
    h.update(" ".join(FLAGS + MODULE_FLAGS.get(src, [])).encode())
    h.update(repr(sorted(defines.items())).encode())
    return h.hexdigest()[:16]


def _build_dirs():
    dirs = [os.path.join(CSRC, "_build")]
    tmp = os.path.join(tempfile.gettempdir(), "ginfer_amd_build_%d" % os.getuid())
    dirs.append(tmp)
    return dirs


def _writable_dir():
    for d in _build_dirs():
        try:
            os.makedirs(d, exist_ok=True)
            probe = os.path.join(d, ".probe_%d_%d" % (os.getpid(), threading.get_ident()))
            with open(probe, "w"):
                pass
            os.remove(probe)
            return d
        except OSError:
            continue
    raise KernelBuildError("no writable folder for built kernels (tried %s)" % ", ".join(_build_dirs()))


def _find_built(module, digest):
    stem = _split(module)[2]
    for d in _build_dirs():
        so = os.path.join(d, "lib%s.so" % stem)
        stamp = os.path.join(d, "%s.stamp" % stem)
        try:
            with open(stamp) as f:
                if f.read().strip() == digest and os.path.isfile(so):
                    return so
        except OSError:
            pass
    return None


def _say(msg):
    sys.stderr.write("[ginfer_amd] %s\n" % msg)
    sys.stderr.flush()


def compile_module(module, out_dir=None, quiet=False):
    """Runs hipcc for one module; returns the library's path."""
    hipcc = _hipcc()
    if hipcc is None:
        raise KernelBuildError("hipcc not found: cannot build kernel library %r" % module)
    out_dir = out_dir or _writable_dir()
    src, defines, stem = _split(module)
    so = os.path.join(out_dir, "lib%s.so" % stem)
    tmp = so + ".%d.tmp" % os.getpid()
    cmd = ([hipcc] + FLAGS + MODULE_FLAGS.get(src, []) + ["-D%s=%s" % kv for kv in sorted(defines.items())]
           + ["-I", CSRC, "-o", tmp, os.path.join(CSRC, src + ".hip")])
    module = stem
    env = dict(os.environ)
    if not env.get("HOME"):
        env["HOME"] = tempfile.gettempdir()          # hipcc wants a home for its caches
    t0 = time.time()
    proc = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, env=env, text=True)
    # a line now and then while a long compile runs
    out = []
    reader = threading.Thread(target=lambda: out.append(proc.stdout.read()), daemon=True)
    reader.start()
    while proc.poll() is None:
        try:
            proc.wait(timeout=20)
        except subprocess.TimeoutExpired:
            if not quiet:
                _say("still compiling %s (%.0f s)" % (module, time.time() - t0))
    reader.join()
    log = "".join(out)
    if proc.returncode != 0:
        if os.path.exists(tmp):
            os.remove(tmp)
        raise KernelBuildError("hipcc failed for %s:\n%s" % (module, log))
    os.replace(tmp, so)
    with open(os.path.join(out_dir, "%s.stamp" % stem), "w") as f:
        f.write(_digest((src, defines) if defines else src))
    return so


def _host_compiler():
    for cand in (os.environ.get("CXX"), shutil.which("g++"), shutil.which("c++"), shutil.which("clang++"),
                 "/opt/rocm/llvm/bin/clang++"):
        if cand and os.path.isfile(cand if os.path.isabs(cand) else (shutil.which(cand) or "")):
            return cand if os.path.isabs(cand) else shutil.which(cand)
    return None


def _host_digest(name):
    h = hashlib.sha256()
    for path in [os.path.join(CSRC, "host", name + ".cpp")] + [os.path.join(CSRC, x) for x in HOST_HEADERS.get(name, [])]:
        with open(path, "rb") as f:
            h.update(f.read())
    h.update(" ".join(HOST_FLAGS).encode())
    return h.hexdigest()[:16]


def compile_host_module(name, out_dir=None):
    """Runs the host compiler for one plain C++ library; returns its path."""
    cxx = _host_compiler()
    if cxx is None:
        raise KernelBuildError("no C++ compiler found: cannot build host library %r" % name)
    out_dir = out_dir or _writable_dir()
    so = os.path.join(out_dir, "lib%s.so" % name)
    tmp = so + ".%d.tmp" % os.getpid()
    proc = subprocess.run([cxx] + HOST_FLAGS + ["-o", tmp, os.path.join(CSRC, "host", name + ".cpp")],
                          stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        if os.path.exists(tmp):
            os.remove(tmp)
        raise KernelBuildError("%s failed for %s:\n%s" % (cxx, name, proc.stdout))
    os.replace(tmp, so)
    with open(os.path.join(out_dir, "%s.stamp" % name), "w") as f:
        f.write(_host_digest(name))
    return so


def load_host(name):
    """The ctypes library of a plain C++ host module, built first if it is missing or stale.  Needs no GPU."""
    with _lock:
        if name in _loaded:
            return _loaded[name]
        if name not in HOST_MODULES:
            raise KernelBuildError("no host library %r" % name)
        digest, so = _host_digest(name), None
        for d in _build_dirs():
            try:
                with open(os.path.join(d, "%s.stamp" % name)) as f:
                    if f.read().strip() == digest and os.path.isfile(os.path.join(d, "lib%s.so" % name)):
                        so = os.path.join(d, "lib%s.so" % name)
                        break
            except OSError:
                pass
        if so is None:
            so = compile_host_module(name)
        try:
            lib = ctypes.CDLL(so)
        except OSError as e:
            raise KernelBuildError("cannot load host library %s: %s" % (so, e))
        _loaded[name] = lib
        return lib


def build_all(force=False, modules=None, quiet=False):
    """Builds every module (in parallel); with force, also those already built.  Without a list of modules the
    host libraries are built too."""
    from concurrent.futures import ThreadPoolExecutor
    if modules is None:
        for name in HOST_MODULES:
            if force:
                compile_host_module(name)
                if not quiet:
                    _say("compiled host library %s" % name)
            else:
                load_host(name)
        modules = []
        for m in available_modules():
            modules.extend([(m, v) for v in VARIANTS[m]] if m in VARIANTS else [m])
    modules = [m for m in modules if os.path.isfile(os.path.join(CSRC, _split(m)[0] + ".hip"))]
    todo = [m for m in modules if force or _find_built(m, _digest(m)) is None]
    if not todo:
        return
    out_dir = _writable_dir()
    if not quiet:
        _say("compiling %d kernel librar%s for %s: %s" % (len(todo), "y" if len(todo) == 1 else "ies",
                                                        ARCH, ", ".join(_split(m)[2] for m in todo)))
    done = []

    def one(m):
        compile_module(m, out_dir, quiet=quiet)
        done.append(m)
        if not quiet:
            _say("compiled %s (%d/%d)" % (_split(m)[2], len(done), len(todo)))
    workers = max(1, min(len(todo), (os.cpu_count() or 4), 8))
    with ThreadPoolExecutor(workers) as ex:
        list(ex.map(one, todo))


def load(module, defines=None):
    """The ctypes library of a module (for one set of macro values), building it first if it is
    missing or stale."""
    if defines:
        module = (module, dict(defines))
    src, _, stem = _split(module)
    with _lock:
        if stem in _loaded:
            return _loaded[stem]
        if not os.path.isfile(os.path.join(CSRC, src + ".hip")):
            raise KernelBuildError("no kernel source for module %r in %s" % (src, CSRC))
        digest = _digest(module)
        so = _find_built(module, digest)
        if so is None:
            _say("kernel library %r is not built yet; compiling it for %s" % (stem, ARCH))
            so = compile_module(module)
            _say("compiled %s" % stem)
        import torch  # noqa: F401  the HIP runtime that torch loaded is the one the library binds to
        try:
            lib = ctypes.CDLL(so)
        except OSError as e:
            raise KernelBuildError("cannot load kernel library %s: %s" % (so, e))
        _loaded[stem] = lib
        return lib
