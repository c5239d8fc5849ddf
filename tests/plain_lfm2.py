"""A plain, slow, whole-sequence implementation of the LFM2 dense decoder.

It is the yardstick of the tests: no cache, no pages, no batching, no portions,
one function for each part, float64 arithmetic (except where the reference fixes
a 32-bit intermediate, which is then rounded the same way).  It shares no code
with ``celeg_amd``: it reads ``config.json`` as a dictionary and the tensors
through the ``safetensors`` package, and it is written from the formulas of the
reference's CPU backend.  Every function cites the reference lines it follows
(paths relative to the reference checkout).
"""
from __future__ import annotations

import json
import math
import os
from typing import Dict, List, Optional, Sequence

import numpy as np
import torch

F64 = torch.float64


# --------------------------------------------------------------------------- sizes

def ff_dim(intermediate_size: int, auto_adjust: bool, multiple_of: int = 256,
           multiplier: Optional[float] = 1.0) -> int:
    """Width of the feed-forward.

    The reference reads it off the rows of ``feed_forward.w1.weight``
    (src/model/inference/global_facts.cpp:127-152) and never evaluates
    ``block_multiple_of`` / ``block_ffn_dim_multiplier``; the arithmetic is the
    one the published shapes obey: 6656 -> 4608, 12288 -> 8192, 10752 -> 7168
    (multiple_of 256) and 512 -> 352 (multiple_of 32).
    """
    if not auto_adjust:
        return int(intermediate_size)
    ff = int(2 * intermediate_size / 3)
    if multiplier is not None:
        ff = int(multiplier * ff)
    return multiple_of * ((ff + multiple_of - 1) // multiple_of)


# --------------------------------------------------------------------------- parts

def embedding(table: torch.Tensor, tokens: Sequence[int]) -> torch.Tensor:
    """h0[t] = E[token[t]]; multiplier 1, nothing added
    (src/backend/cpu/model_forward_token.cpp:28-60)."""
    idx = torch.as_tensor(list(tokens), dtype=torch.long)
    if idx.numel() and (int(idx.min()) < 0 or int(idx.max()) >= table.shape[0]):
        raise ValueError("token id out of range")  # src/backend/cuda/model/prefill.cpp:41-70
    return table.to(F64)[idx]


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """y = x * 1/sqrt(mean(x^2) + eps) * w over the last axis; eps inside the root,
    added to the mean; weight is a plain scale (not 1+w)
    (src/backend/cpu/kernels/elementwise.cpp:56-76)."""
    x = x.to(F64)
    inv = 1.0 / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)
    return x * inv * weight.to(F64)


def rope_inverse_frequencies(theta: float, rotary_dim: int) -> np.ndarray:
    """f_i = theta^(-2 i / rotary_dim), i < rotary_dim/2, in double
    (include/celeg/model/position.hpp:77-78)."""
    half = rotary_dim // 2
    return np.array([math.pow(theta, -2.0 * i / rotary_dim) for i in range(half)],
                    dtype=np.float64)


def rope_cos_sin(positions: Sequence[int], theta: float, rotary_dim: int):
    """angle = float(position) * float(frequency), a 32-bit product, then cos/sin
    (src/backend/cpu/kernels/rope.cpp:30-36 of cpu_qk_norm_rope: lines 76-82)."""
    freq32 = rope_inverse_frequencies(theta, rotary_dim).astype(np.float32)
    pos32 = np.asarray(list(positions), dtype=np.float32)
    angle32 = (pos32[:, None] * freq32[None, :]).astype(np.float32)
    angle = torch.from_numpy(angle32.astype(np.float64))
    return torch.cos(angle), torch.sin(angle)


def rope_apply(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """Split-half pairing: for i < half, a = x[i], b = x[i+half];
    out[i] = a cos - b sin, out[i+half] = b cos + a sin
    (src/backend/cpu/kernels/rope.cpp:95-108, 141-152).  x is [T, heads, hd],
    cos/sin are [T, half]; dims beyond 2*half pass through."""
    x = x.to(F64)
    half = cos.shape[-1]
    a = x[..., :half]
    b = x[..., half:2 * half]
    c = cos[:, None, :]
    s = sin[:, None, :]
    out = x.clone()
    out[..., :half] = a * c - b * s
    out[..., half:2 * half] = b * c + a * s
    return out


def head_rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """RMSNorm over head_dim for every (row, head), one weight [hd] for all heads
    (src/backend/cpu/kernels/rope.cpp:84-94; granularity:
    src/model/inference/rules_attention.cpp:115-134)."""
    return rmsnorm(x, weight, eps)


def causal_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                     window: Optional[int] = None,
                     scale: Optional[float] = None) -> torch.Tensor:
    """Grouped-query causal attention over a whole sequence.

    q [T, Hq, hd]; k, v [T, Hkv, hd].  For row t and head j:
    s[u] = (q_j . k_g(j),u) / sqrt(hd) for u <= t (and u > t - window if a window
    is given), g(j) = j / (Hq/Hkv); softmax over u; o = sum p[u] v[u]
    (src/backend/cpu/attention/paged_attention.cpp:229-283; scale applied once,
    include/celeg/backend/cuda/attention_norm.hpp:13-23)."""
    q, k, v = q.to(F64), k.to(F64), v.to(F64)
    T, Hq, hd = q.shape
    Hkv = k.shape[1]
    if Hq % Hkv:
        raise ValueError("query heads must be a multiple of key/value heads")
    group = Hq // Hkv
    if scale is None:
        scale = 1.0 / math.sqrt(hd)
    out = torch.zeros(T, Hq, v.shape[-1], dtype=F64)
    for j in range(Hq):
        g = j // group
        for t in range(T):
            first = 0 if window is None else max(0, t - window + 1)
            s = (k[first:t + 1, g] @ q[t, j]) * scale
            p = torch.softmax(s, dim=0)
            out[t, j] = p @ v[first:t + 1, g]
    return out


def short_conv(bcx: torch.Tensor, weight: torch.Tensor,
               conv_bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Double-gated short causal convolution over a whole sequence.

    bcx [T, 3H] splits in this order: B = [0,H), C = [H,2H), x = [2H,3H)
    (src/backend/cpu/kernels/convolution.cpp:16-18).  bx[t] = B[t]*x[t];
    conv[t,ch] = sum_tap w[ch,tap] * bx[t-(L-1-tap), ch], zero before position 0:
    tap L-1 multiplies the current token (convolution.cpp:19-26 with the state
    ring, weight channel-major [H, L] as in src/model/reference.cpp:249-252);
    y = C[t] * conv[t].  A convolution bias, which the reference never reads
    (include/celeg/model/graph.hpp:316-320), is added to conv before the C gate.
    """
    bcx = bcx.to(F64)
    T, H3 = bcx.shape
    H = H3 // 3
    w = weight.to(F64).reshape(H, -1)
    L = w.shape[1]
    B, C, x = bcx[:, :H], bcx[:, H:2 * H], bcx[:, 2 * H:]
    bx = B * x
    y = torch.zeros(T, H, dtype=F64)
    for t in range(T):
        conv = torch.zeros(H, dtype=F64)
        for tap in range(L):
            src = t - (L - 1 - tap)
            if src >= 0:
                conv = conv + w[:, tap] * bx[src]
        if conv_bias is not None:
            conv = conv + conv_bias.to(F64)
        y[t] = C[t] * conv
    return y


def silu(g: torch.Tensor) -> torch.Tensor:
    """silu(g) = g / (1 + exp(-g)) (src/backend/cpu/kernels/elementwise.cpp:112-118)."""
    return g / (1.0 + torch.exp(-g))


def swiglu_ffn(x: torch.Tensor, w1: torch.Tensor, w3: torch.Tensor,
               w2: torch.Tensor) -> torch.Tensor:
    """(silu(x W1^T) * (x W3^T)) W2^T: w1 gate, w3 up, w2 down
    (src/backend/cpu/model_forward_token.cpp:163-172;
    src/model/inference/layer_bindings.cpp:439-473)."""
    x = x.to(F64)
    g = x @ w1.to(F64).T
    u = x @ w3.to(F64).T
    return (silu(g) * u) @ w2.to(F64).T


def linear(x: torch.Tensor, w: torch.Tensor, b: Optional[torch.Tensor] = None) -> torch.Tensor:
    """y = x W^T (+ b); weights are [out, in] row-major
    (src/model/weight_plan.cpp:82-130)."""
    y = x.to(F64) @ w.to(F64).T
    if b is not None:
        y = y + b.to(F64)
    return y


# --------------------------------------------------------------------------- blocks

def conv_mixer(n: torch.Tensor, W: Dict[str, torch.Tensor], prefix: str,
               conv_bias: bool) -> torch.Tensor:
    """in_proj -> short_conv -> out_proj
    (src/backend/cpu/operators/recurrent.cpp:212-240)."""
    bcx = linear(n, W[prefix + "conv.in_proj.weight"],
                 W.get(prefix + "conv.in_proj.bias") if conv_bias else None)
    y = short_conv(bcx, W[prefix + "conv.conv.weight"],
                   W.get(prefix + "conv.conv.bias") if conv_bias else None)
    return linear(y, W[prefix + "conv.out_proj.weight"],
                  W.get(prefix + "conv.out_proj.bias") if conv_bias else None)


def attention_project(n, W, prefix, cfg, positions):
    """q/k/v projections, per-head norm of q and k, then rotation of q and k
    (src/backend/cpu/model_forward_token.cpp:100-120; kernels/rope.cpp:61-111)."""
    Hq, Hkv, hd = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    eps = cfg["norm_eps"]
    T = n.shape[0]
    q = linear(n, W[prefix + "self_attn.q_proj.weight"]).reshape(T, Hq, hd)
    q = head_rmsnorm(q, W[prefix + "self_attn.q_layernorm.weight"], eps)
    cos, sin = rope_cos_sin(positions, cfg["rope_theta"], hd)
    q = rope_apply(q, cos, sin)
    k = v = None
    if prefix + "self_attn.k_proj.weight" in W:
        k = linear(n, W[prefix + "self_attn.k_proj.weight"]).reshape(T, Hkv, hd)
        v = linear(n, W[prefix + "self_attn.v_proj.weight"]).reshape(T, Hkv, hd)
        k = head_rmsnorm(k, W[prefix + "self_attn.k_layernorm.weight"], eps)
        k = rope_apply(k, cos, sin)
    return q, k, v


def attention_mixer(n, W, prefix, cfg, positions, shared_kv=None, window=None):
    q, k, v = attention_project(n, W, prefix, cfg, positions)
    if shared_kv is not None:
        k, v = shared_kv
    o = causal_attention(q, k, v, window=window)
    T = n.shape[0]
    return linear(o.reshape(T, -1), W[prefix + "self_attn.out_proj.weight"]), (k, v)


def normalise_config(cfg: dict) -> dict:
    """Fill the defaults the reference applies
    (src/model/inference/metadata.cpp:364-370, 407-409, 643)."""
    c = dict(cfg)
    c.setdefault("num_key_value_heads", c["num_attention_heads"])
    c.setdefault("head_dim", c["hidden_size"] // c["num_attention_heads"])
    if "norm_eps" not in c:
        c["norm_eps"] = c.get("rms_norm_eps", 1e-6)
    c.setdefault("conv_bias", False)
    if "tie_word_embeddings" not in c:
        c["tie_word_embeddings"] = c.get("tie_embedding", True)
    return c


def model_logits(cfg: dict, W: Dict[str, torch.Tensor], tokens: Sequence[int],
                 order: Optional[List[int]] = None,
                 kv_from: Optional[Dict[int, int]] = None,
                 first_position: int = 0, hidden: Optional[list] = None) -> torch.Tensor:
    """Logits [T, V] of a whole sequence.

    Every layer is pre-norm, mixer, add, pre-norm, feed-forward, add
    (src/backend/cpu/model_forward_token.cpp:93-172); the output is
    RMSNorm(h, embedding_norm) . E_out^T with E_out = E when tied
    (model_forward_token.cpp:213-218).  ``order`` lists the layers in the order
    they run (default 0..N-1) and ``kv_from[i] = j`` lets the i-th entry of the
    order attend over the keys and values that the j-th entry computed; both are
    generalisations used by tests of the engine's layer list, not LFM2 features.
    ``first_position`` shifts all positions (for the shift invariance test).  ``hidden``, a
    list, receives the residual stream [T, H] after every entry of the order.
    """
    cfg = normalise_config(cfg)
    T = len(tokens)
    positions = [first_position + t for t in range(T)]
    h = embedding(W["model.embed_tokens.weight"], tokens)
    kinds = cfg["layer_types"]
    order = list(range(len(kinds))) if order is None else order
    kv_from = kv_from or {}
    kv_of_step = {}
    for step, layer in enumerate(order):
        prefix = f"model.layers.{layer}."
        n = rmsnorm(h, W[prefix + "operator_norm.weight"], cfg["norm_eps"])
        if kinds[layer] == "conv":
            m = conv_mixer(n, W, prefix, cfg["conv_bias"])
        else:
            shared = kv_of_step[kv_from[step]] if step in kv_from else None
            m, kv = attention_mixer(n, W, prefix, cfg, positions, shared_kv=shared)
            kv_of_step[step] = kv
        h = h + m
        n2 = rmsnorm(h, W[prefix + "ffn_norm.weight"], cfg["norm_eps"])
        h = h + swiglu_ffn(n2, W[prefix + "feed_forward.w1.weight"],
                           W[prefix + "feed_forward.w3.weight"],
                           W[prefix + "feed_forward.w2.weight"])
        if hidden is not None:
            hidden.append(h.clone())
    n = rmsnorm(h, W["model.embedding_norm.weight"], cfg["norm_eps"])
    head = W["model.embed_tokens.weight"] if cfg["tie_word_embeddings"] else W["lm_head.weight"]
    return linear(n, head)


def load_model_folder(folder: str):
    """config.json as a dict and the tensors as float64, read with the
    safetensors package (not with the engine's own reader)."""
    from safetensors import safe_open
    with open(os.path.join(folder, "config.json")) as fh:
        cfg = json.load(fh)
    W = {}
    with safe_open(os.path.join(folder, "model.safetensors"), framework="pt") as fh:
        for name in fh.keys():
            W[name] = fh.get_tensor(name).to(F64)
    return cfg, W


# --------------------------------------------------------------------------- sampling

MASK64 = (1 << 64) - 1


def xorshift64star(state: int):
    """s ^= s>>12; s ^= s<<25; s ^= s>>27; bits = s * 2685821657736338717
    (src/backend/cpu/sampler.cpp:10-15).  Returns (new_state, bits)."""
    state ^= state >> 12
    state ^= (state << 25) & MASK64
    state ^= state >> 27
    return state, (state * 2685821657736338717) & MASK64


def random_unit(state: int):
    """u = float(((bits >> 11) + 0.5) / 2^53) (sampler.cpp:17-22)."""
    state, bits = xorshift64star(state)
    unit = (float(bits >> 11) + 0.5) * (1.0 / 9007199254740992.0)
    return state, float(np.float32(unit))


def sample(logits: Sequence[float], temperature: float, top_k: int, top_p: float,
           repetition_penalty: float, seen: Sequence[bool], rng_state: int):
    """The reference's sampler in 32-bit floats (src/backend/cpu/sampler.cpp:26-101).

    Returns (token, new_rng_state).  Greedy when temperature <= 0 or top_k == 1:
    argmax of the penalised logits, lowest index wins ties.  Otherwise
    score = penalised / temperature; keep the top_k by (score desc, id asc);
    p = exp(score - max) / sum; with top_p < 1 keep the shortest prefix whose
    cumulative mass reaches top_p (at least one); draw u * mass and walk the list.
    """
    f32 = np.float32
    logits = np.asarray(logits, dtype=np.float32)
    V = logits.shape[0]
    pen = logits.copy()
    if repetition_penalty > 1.0:
        s = np.asarray(seen, dtype=bool)
        rp = f32(repetition_penalty)
        pen = np.where(s, np.where(pen >= 0, pen / rp, pen * rp), pen).astype(np.float32)
    if temperature <= 0.0 or top_k == 1:
        best, best_v = 0, pen[0]
        for t in range(1, V):
            if pen[t] > best_v:
                best, best_v = t, pen[t]
        return int(best), rng_state
    k = min(top_k, V)
    score = (pen / f32(temperature)).astype(np.float32)
    idx = sorted(range(V), key=lambda t: (-float(score[t]), t))[:k]
    maximum = score[idx[0]]
    probs = np.exp((score[idx] - maximum).astype(np.float32)).astype(np.float32)
    total = f32(0)
    for p in probs:
        total = f32(total + p)
    probs = (probs / total).astype(np.float32)
    active = len(probs)
    if top_p < 1.0:
        cumulative = f32(0)
        active = 0
        while True:
            cumulative = f32(cumulative + probs[active])
            active += 1
            if not (active < len(probs) and cumulative < f32(top_p)):
                break
        total = f32(0)
        for i in range(active):
            total = f32(total + probs[i])
    else:
        total = f32(1)
    rng_state, u = random_unit(rng_state)
    target = f32(f32(u) * total)
    for i in range(active):
        target = f32(target - probs[i])
        if target <= 0:
            return int(idx[i]), rng_state
    return int(idx[active - 1]), rng_state
