"""A plain, slow statement of the Qwen2 decoder: whole sequences, no cache, one function per part.

Everything here is written from the reference's formulas (11Aln0/ginfer, paths relative to its root)
and shares no code with the product package: it reads model folders with the `safetensors` package,
keeps every tensor on the CPU, and recomputes attention over the whole sequence for every call.

The compute dtype is a parameter (float64 by default).  Rotation angles are the one exception: the
reference builds its sine/cosine tables in 32-bit (position cast to float, times a 32-bit inverse
frequency), and at positions in the thousands that rounding is visible, so the tables are built in
32-bit exactly as the reference's formula says and then cast to the compute dtype.
"""
import json
import math
import os

import numpy as np
import torch


# ----------------------------------------------------------------------------- configuration

def read_config(folder):
    """Keys and defaults of ginfer/model/loader/model_loader.cc:38-52 and :95-106."""
    with open(os.path.join(folder, "config.json")) as f:
        c = json.load(f)
    out = {
        "num_hidden_layers": c["num_hidden_layers"],
        "vocab_size": c["vocab_size"],
        "max_position_embeddings": c["max_position_embeddings"],
        "num_attention_heads": c["num_attention_heads"],
        "num_key_value_heads": c["num_key_value_heads"],
        "hidden_size": c["hidden_size"],
        "intermediate_size": c["intermediate_size"],
        "rms_norm_eps": c.get("rms_norm_eps", 1e-6),
        "rope_theta": c.get("rope_theta", 10000.0),
        "tie_word_embeddings": c.get("tie_word_embeddings", False),
        "head_dim": c.get("head_dim", 0) or c["hidden_size"] // c["num_attention_heads"],
    }
    eos = c.get("eos_token_id", c["vocab_size"] - 1)
    out["eos_token_ids"] = list(eos) if isinstance(eos, (list, tuple)) else [eos]
    # The reference never reads the window keys; they are part of the architecture's config.json
    # (layers with index >= max_window_layers attend to the last `sliding_window` positions when
    # use_sliding_window is set).
    if c.get("use_sliding_window", False):
        first = c.get("max_window_layers", c["num_hidden_layers"])
        out["windows"] = [c["sliding_window"] if i >= first else None
                          for i in range(c["num_hidden_layers"])]
    else:
        out["windows"] = [None] * c["num_hidden_layers"]
    return out


def read_weights(folder, dtype=torch.float64):
    from safetensors import safe_open
    tensors = {}
    with safe_open(os.path.join(folder, "model.safetensors"), framework="pt") as f:
        for name in f.keys():
            tensors[name] = f.get_tensor(name).to(dtype)
    return tensors


# ----------------------------------------------------------------------------- parts

def embedding(weight, ids):
    """out[t,:] = W[ids[t],:]; ginfer/core/op/kernels/cuda/embedding_kernel.cu:16-24."""
    return weight[torch.as_tensor(ids, dtype=torch.long)]


def rms_norm(x, gain, eps):
    """rms = sqrt(sum(x^2)/H + eps); y = (x*g)/rms; ginfer/core/op/kernels/cuda/rmsnorm_kernel.cu:27-66
    (sum :31-44, rms :54, scaling :63).  Plain gain, no mean subtraction."""
    ss = (x * x).sum(dim=-1, keepdim=True)
    rms = torch.sqrt(ss / x.shape[-1] + eps)
    return (x * gain) / rms


def linear(x, weight, bias=None):
    """y = x . W^T (+ b) with W stored [out, in]; ginfer/core/layer/linear.cc:9-20,
    ginfer/core/op/kernels/cuda/gemm_kernel/gemm_kernel.cu:100-121 (bias in the epilogue)."""
    y = x @ weight.t()
    if bias is not None:
        y = y + bias
    return y


def rope_tables(theta, rotary_dim, num_positions):
    """inv_freq[j] = 1/powf(theta, j/half); angle = (float)p * inv_freq[j]; sinf, cosf: all in 32-bit.
    ginfer/core/op/kernels/cuda/rope_kernel.cu:13-16 (frequency), :61-72 (table)."""
    half = rotary_dim // 2
    j = torch.arange(half, dtype=torch.float32)
    inv_freq = 1.0 / torch.pow(torch.tensor(theta, dtype=torch.float32), j / float(half))
    p = torch.arange(num_positions, dtype=torch.float32)
    ang = p[:, None] * inv_freq[None, :]
    return torch.sin(ang), torch.cos(ang)


def apply_rope(x, positions, sin, cos):
    """x: [T, heads, hd].  NeoX pairing (j, j+half):
    o[j] = x[j]*cos - x[j+half]*sin ; o[j+half] = x[j]*sin + x[j+half]*cos.
    ginfer/core/op/kernels/cuda/rope_kernel.cu:83-102 (the pair :93-101)."""
    half = sin.shape[1]
    pos = torch.as_tensor(positions, dtype=torch.long)
    s = sin[pos].to(x.dtype)[:, None, :]
    c = cos[pos].to(x.dtype)[:, None, :]
    lo, hi, rest = x[..., :half], x[..., half:2 * half], x[..., 2 * half:]
    return torch.cat([lo * c - hi * s, lo * s + hi * c, rest], dim=-1)


def attention(q, k, v, q_positions, window=None):
    """q: [Tq, nh, hd]; k, v: [Tk, nkv, hd] for key positions 0..Tk-1; q_positions: absolute
    position of every query row.  Head h reads kv head h // (nh/nkv).  score = (q.k) * 1/sqrt(hd);
    key c is allowed for a query at position p iff c <= p (the reference's
    `global_c <= global_r + kv_len - q_len && global_c < kv_len`), softmax over allowed keys.
    ginfer/core/op/kernels/cuda/page_attn_kernel/flash_gqa_varlen_kernel.cu:202-222 (mask and scale),
    :439-450 (head -> kv head).  With a window w only keys with p - c < w are allowed."""
    Tq, nh, hd = q.shape
    Tk, nkv, _ = k.shape
    group = nh // nkv
    scale = 1.0 / math.sqrt(hd)
    out = torch.empty_like(q)
    p = torch.as_tensor(q_positions, dtype=torch.long)[:, None]
    c = torch.arange(Tk)[None, :]
    allowed = c <= p
    if window is not None:
        allowed &= (p - c) < window
    for h in range(nh):
        g = h // group
        s = (q[:, h, :] @ k[:, g, :].t()) * scale
        s = s.masked_fill(~allowed, float("-inf"))
        m = s.max(dim=-1, keepdim=True).values
        e = torch.exp(s - m)
        out[:, h, :] = (e / e.sum(dim=-1, keepdim=True)) @ v[:, g, :]
    return out


def swiglu(gate, up):
    """(g * (1/(1+exp(-g)))) * u; ginfer/core/op/kernels/cuda/swiglu_kernel.cu:24-27."""
    return (gate * (1.0 / (1.0 + torch.exp(-gate)))) * up


def attention_block(n, w, prefix, cfg, positions, sin, cos, window, kv_from=None):
    """q/k/v projections with bias, view as heads, rotate q and k, attend, output projection
    without bias; ginfer/core/layer/transformer/attention.cc:61-81, biases ginfer/model/qwen2.cc:15-17.
    Returns (output, (k, v)); with `kv_from` the keys and values of another layer are used."""
    nh, nkv, hd = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    T = n.shape[0]
    q = linear(n, w[prefix + ".q_proj.weight"], w[prefix + ".q_proj.bias"]).view(T, nh, hd)
    q = apply_rope(q, positions, sin, cos)
    if kv_from is None:
        k = linear(n, w[prefix + ".k_proj.weight"], w[prefix + ".k_proj.bias"]).view(T, nkv, hd)
        v = linear(n, w[prefix + ".v_proj.weight"], w[prefix + ".v_proj.bias"]).view(T, nkv, hd)
        k = apply_rope(k, positions, sin, cos)
    else:
        k, v = kv_from
    a = attention(q, k, v, positions, window)
    return linear(a.reshape(T, nh * hd), w[prefix + ".o_proj.weight"]), (k, v)


def feed_forward(n, w, prefix):
    """gate, up, SwiGLU, down, no biases; ginfer/core/layer/transformer/feedforward.cc:22-25."""
    g = linear(n, w[prefix + ".gate_proj.weight"])
    u = linear(n, w[prefix + ".up_proj.weight"])
    return linear(swiglu(g, u), w[prefix + ".down_proj.weight"])


def forward(cfg, w, ids, schedule=None, rows=None):
    """Logits [T, V] for one whole sequence at positions 0..T-1 (with `rows`, a list of positions: the
    logits [len(rows), V] at those alone; the final norm and the head act on every row by itself).
    Block order ginfer/core/layer/transformer/encoder.cc:33-39: n = norm1(x); h = x + attn(n);
    n = norm2(h); x = h + mlp(n).  Then the final norm and the output head (tied to the embedding
    or `lm_head.weight`), ginfer/model/model.cc:158-165, ginfer/model/qwen2.cc:41-46.
    `schedule` is a list of (layer, cache_of) pairs: the order in which layers run; `cache_of` names
    an earlier entry of the list whose keys and values this run reads instead of making its own."""
    dtype = w["model.embed_tokens.weight"].dtype
    T = len(ids)
    positions = list(range(T))
    sin, cos = rope_tables(cfg["rope_theta"], cfg["head_dim"], max(T, 1))
    x = embedding(w["model.embed_tokens.weight"], ids).to(dtype)
    eps = cfg["rms_norm_eps"]
    if schedule is None:
        schedule = [(i, None) for i in range(cfg["num_hidden_layers"])]
    kept = []
    for layer, cache_of in schedule:
        p = "model.layers.%d" % layer
        n = rms_norm(x, w[p + ".input_layernorm.weight"], eps)
        a, kv = attention_block(n, w, p + ".self_attn", cfg, positions, sin, cos,
                                cfg["windows"][layer],
                                kv_from=None if cache_of is None else kept[cache_of])
        kept.append(kv)
        h = x + a
        n = rms_norm(h, w[p + ".post_attention_layernorm.weight"], eps)
        x = h + feed_forward(n, w, p + ".mlp")
    if rows is not None:
        x = x[torch.as_tensor(rows, dtype=torch.long)]
    n = rms_norm(x, w["model.norm.weight"], eps)
    head = w["model.embed_tokens.weight"] if cfg["tie_word_embeddings"] else w["lm_head.weight"]
    return linear(n, head)


# ----------------------------------------------------------------------------- sampling

def argmax_token(logits_row):
    """Greedy choice, lowest index among equals (ginfer/model/model.cc:219-220 takes the argmax)."""
    return int(np.argmax(logits_row.detach().cpu().numpy()))


def sample_token(logits_row, temperature, uniform):
    """Temperature sampling by inverse CDF with a given uniform number in [0,1):
    p = softmax(logits / temperature); the first index whose running sum exceeds uniform * total."""
    if temperature <= 0.0:
        return argmax_token(logits_row)
    x = logits_row.detach().double().cpu().numpy() / temperature
    e = np.exp(x - x.max())
    c = np.cumsum(e)
    return int(min(np.searchsorted(c, uniform * c[-1], side="right"), len(c) - 1))


def generate(cfg, w, prompt, max_tokens, temperature=0.0, uniforms=None, ignore_eos=False,
             schedule=None):
    """Token by token, recomputing the whole sequence every time.  Stops on an end-of-sequence id
    unless ignore_eos, or after max_tokens (ginfer/engine/scheduler.cc:91-92)."""
    ids = list(prompt)
    out = []
    for n in range(max_tokens):
        row = forward(cfg, w, ids, schedule)[-1]
        tok = sample_token(row, temperature, None if uniforms is None else uniforms[n])
        ids.append(tok)
        out.append(tok)
        if not ignore_eos and tok in cfg["eos_token_ids"]:
            break
    return out
