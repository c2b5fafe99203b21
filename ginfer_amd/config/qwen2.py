"""Typed configuration of the Qwen2 dense decoder, read from its own config.json keys.

Required keys and defaults follow ginfer/model/loader/model_loader.cc:38-52 (layers, vocabulary,
positions, heads, head_dim 0 -> hidden/heads, eos scalar or list defaulting to vocab-1) and :95-106
(hidden, intermediate, rms_norm_eps 1e-6, rope_theta 10000, tie_word_embeddings false).  The
reference fixes biases on q/k/v and none on o (ginfer/model/qwen2.cc:15-17) and SiLU as activation
(ginfer/core/layer/transformer/feedforward.cc:24); it never reads the window keys
(`use_sliding_window`, `sliding_window`, `max_window_layers`), which here choose a windowed mixer
for the layers from `max_window_layers` on.
"""
from dataclasses import dataclass, field, asdict
from typing import List, Optional

from .registry import register_architecture, ConfigError
from .spec import PartSpec, prenorm_layer, ScheduleEntry, ModelSpec

# How this architecture's checkpoints spell the prefixes of a layer's parts and of the parts outside the layers
# (ginfer/model/qwen2.cc:34-46 and ginfer/model/loader/model_loader.cc:108-119 bind the same names)
LAYER_TENSOR_NAMES = dict(mixer="self_attn", feed_forward="mlp", mixer_norm="input_layernorm",
                          feed_forward_norm="post_attention_layernorm")
MODEL_TENSOR_NAMES = dict(embedding="model.embed_tokens", final_norm="model.norm", head="lm_head")

_REQUIRED = ("num_hidden_layers", "vocab_size", "max_position_embeddings", "num_attention_heads",
             "num_key_value_heads", "hidden_size", "intermediate_size")


def _int(d, key, minimum=1):
    v = d[key]
    if isinstance(v, bool) or not isinstance(v, int) or v < minimum:
        raise ConfigError("config.json: %r must be an integer >= %d, got %r" % (key, minimum, v))
    return v


@register_architecture("Qwen2ForCausalLM", "qwen2")
@dataclass
class Qwen2Config:
    num_hidden_layers: int
    vocab_size: int
    max_position_embeddings: int
    num_attention_heads: int
    num_key_value_heads: int
    hidden_size: int
    intermediate_size: int
    head_dim: int
    rms_norm_eps: float = 1e-6
    rope_theta: float = 10000.0
    tie_word_embeddings: bool = False
    eos_token_ids: List[int] = field(default_factory=list)
    torch_dtype: str = "float16"
    use_sliding_window: bool = False
    sliding_window: Optional[int] = None
    max_window_layers: Optional[int] = None

    architecture = "Qwen2ForCausalLM"

    @classmethod
    def from_dict(cls, d):
        missing = [k for k in _REQUIRED if k not in d]
        if missing:
            raise ConfigError("config.json lacks required key(s): %s" % ", ".join(missing))
        hidden = _int(d, "hidden_size")
        nh = _int(d, "num_attention_heads")
        head_dim = d.get("head_dim") or 0
        if head_dim == 0:
            if hidden % nh:
                raise ConfigError("config.json: hidden_size %d is not a multiple of "
                                  "num_attention_heads %d and no head_dim is given" % (hidden, nh))
            head_dim = hidden // nh
        vocab = _int(d, "vocab_size")
        eos = d.get("eos_token_id", vocab - 1)
        if eos is None:
            eos = vocab - 1
        eos = [int(e) for e in eos] if isinstance(eos, (list, tuple)) else [int(eos)]
        if d.get("rope_scaling") is not None:
            raise ConfigError("config.json: rope_scaling %r is not supported (only null)"
                              % (d["rope_scaling"],))
        if d.get("hidden_act", "silu") != "silu":
            raise ConfigError("config.json: hidden_act %r is not supported (only 'silu')"
                              % d["hidden_act"])
        cfg = cls(
            num_hidden_layers=_int(d, "num_hidden_layers"),
            vocab_size=vocab,
            max_position_embeddings=_int(d, "max_position_embeddings"),
            num_attention_heads=nh,
            num_key_value_heads=_int(d, "num_key_value_heads"),
            hidden_size=hidden,
            intermediate_size=_int(d, "intermediate_size"),
            head_dim=int(head_dim),
            rms_norm_eps=float(d.get("rms_norm_eps", 1e-6)),
            rope_theta=float(d.get("rope_theta", 10000.0)),
            tie_word_embeddings=bool(d.get("tie_word_embeddings", False)),
            eos_token_ids=eos,
            torch_dtype=str(d.get("torch_dtype", "float16")),
            use_sliding_window=bool(d.get("use_sliding_window", False)),
            sliding_window=d.get("sliding_window"),
            max_window_layers=d.get("max_window_layers"),
        )
        cfg.validate()
        return cfg

    def validate(self):
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError("config.json: num_attention_heads %d is not a multiple of "
                              "num_key_value_heads %d"
                              % (self.num_attention_heads, self.num_key_value_heads))
        if self.head_dim % 2:
            raise ConfigError("config.json: head_dim %d must be even for rotary pairs" % self.head_dim)
        if not self.rms_norm_eps > 0 or not self.rope_theta > 0:
            raise ConfigError("config.json: rms_norm_eps and rope_theta must be positive")
        if self.torch_dtype not in ("bfloat16", "float16", "float32"):
            raise ConfigError("config.json: unsupported torch_dtype %r" % self.torch_dtype)
        if self.use_sliding_window:
            if not isinstance(self.sliding_window, int) or self.sliding_window < 1:
                raise ConfigError("config.json: use_sliding_window needs a positive integer "
                                  "sliding_window, got %r" % (self.sliding_window,))

    def to_dict(self):
        d = asdict(self)
        eos = d.pop("eos_token_ids")
        d["eos_token_id"] = eos[0] if len(eos) == 1 else eos
        d["architectures"] = [self.architecture]
        d["model_type"] = "qwen2"
        d["hidden_act"] = "silu"
        return d

    def layer_window(self, i):
        """Window of layer i, or None for all keys."""
        if not self.use_sliding_window:
            return None
        first = self.num_hidden_layers if self.max_window_layers is None else self.max_window_layers
        return self.sliding_window if i >= first else None

    def model_spec(self):
        position = PartSpec("rope_neox", dict(theta=self.rope_theta, rotary_dim=self.head_dim,
                                              max_positions=self.max_position_embeddings))
        norm = PartSpec("rmsnorm", dict(size=self.hidden_size, eps=self.rms_norm_eps))
        layers = []
        for i in range(self.num_hidden_layers):
            mixer = PartSpec("attention", dict(
                hidden_size=self.hidden_size, num_heads=self.num_attention_heads,
                num_kv_heads=self.num_key_value_heads, head_dim=self.head_dim,
                qkv_bias=True, out_bias=False, window=self.layer_window(i), position=position,
                scale=None))
            ffn = PartSpec("swiglu", dict(hidden_size=self.hidden_size,
                                          intermediate_size=self.intermediate_size))
            layers.append(prenorm_layer("model.layers.%d" % i, mixer=mixer, feed_forward=ffn,
                                        mixer_norm=norm, feed_forward_norm=norm, names=LAYER_TENSOR_NAMES))
        spec = ModelSpec(
            hidden_size=self.hidden_size, vocab_size=self.vocab_size, layers=layers,
            schedule=[ScheduleEntry(i) for i in range(self.num_hidden_layers)],
            embedding=PartSpec("embedding", dict(vocab_size=self.vocab_size,
                                                 hidden_size=self.hidden_size)),
            final_norm=norm,
            head=PartSpec("lm_head", dict(vocab_size=self.vocab_size, hidden_size=self.hidden_size,
                                          tied=self.tie_word_embeddings)),
            max_positions=self.max_position_embeddings,
            eos_token_ids=list(self.eos_token_ids), names=dict(MODEL_TENSOR_NAMES))
        spec.validate()
        return spec
