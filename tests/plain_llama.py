"""A plain, slow Llama decoder written from the reference's formulas: whole sequences,
no cache, one function for each part, float64 arithmetic, no code shared with the engine.

Every function cites the reference lines (relative to the reference's root) it transcribes.
``rnd`` is the rounding applied where the engine's bfloat16 path stores activations in
bfloat16 (identity for the 32-bit path); the formulas themselves do not change.
"""

from __future__ import annotations

import math
import struct
from typing import Callable, Dict, List, Mapping, Optional, Sequence

import numpy as np
import torch

F64 = torch.float64


def identity(x: torch.Tensor) -> torch.Tensor:
    return x


def round_bf16(x: torch.Tensor) -> torch.Tensor:
    """Round to nearest even bfloat16 and widen again (src/model.cpp:69-74)."""
    return x.to(torch.float32).to(torch.bfloat16).to(F64)


def read_config(cfg: Mapping[str, object]) -> Dict[str, object]:
    """Keys and defaults of tools/convert.py:55-80."""
    heads = cfg["num_attention_heads"]
    eos = cfg.get("eos_token_id", -1)
    if isinstance(eos, list):
        eos = eos[0]
    return dict(
        vocab=cfg["vocab_size"], hidden=cfg["hidden_size"], layers=cfg["num_hidden_layers"], heads=heads,
        kv_heads=cfg.get("num_key_value_heads", heads),
        head_dim=cfg.get("head_dim") or cfg["hidden_size"] // heads,
        inter=cfg["intermediate_size"], theta=cfg.get("rope_theta", 10000.0), eps=cfg.get("rms_norm_eps", 1e-6),
        tied=bool(cfg.get("tie_word_embeddings", False)), eos=-1 if eos is None else eos)


# ----------------------------------------------------------------------------- parts

def embed(tokens: Sequence[int], table: torch.Tensor) -> torch.Tensor:
    """x[r,:] = float(E[token_r,:]) (src/model.cpp:274, :233-239)."""
    return table.to(F64)[torch.as_tensor(list(tokens), dtype=torch.long)]


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """inv = 1/sqrt(sumsq/dim + eps); y = (x*inv)*w (src/kernels.cpp:264-271): eps is added
    to the mean of squares inside the root, and the weight multiplies last."""
    dim = x.shape[-1]
    inv = 1.0 / torch.sqrt((x * x).sum(-1, keepdim=True) / dim + eps)
    return (x * inv) * weight.to(F64)


def linear(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """y[m,n] = sum_k x[m,k] * W[n,k], W stored [out, in], no bias (src/kernels.cpp:236-244)."""
    return x @ w.to(F64).T


def rope_inv_freq(theta: float, head_dim: int) -> np.ndarray:
    """inv_freq[i] = 1.0f / powf(theta, float(2i)/float(hd)), in 32-bit (src/model.cpp:220-225)."""
    i = np.arange(head_dim // 2, dtype=np.float32)
    expo = (np.float32(2.0) * i) / np.float32(head_dim)
    return (np.float32(1.0) / np.power(np.float32(theta), expo, dtype=np.float32)).astype(np.float32)


def rope(v: torch.Tensor, positions: Sequence[int], inv_freq: np.ndarray) -> torch.Tensor:
    """Rotate-half rotary embedding (src/kernels.cpp:273-289).  v: [rows, heads, hd].
    angle = float(pos) * inv_freq[i] as a 32-bit product; pairs are (i, i + hd/2):
    out[i] = x1*c - x2*s, out[i+hd/2] = x2*c + x1*s."""
    half = v.shape[-1] // 2
    pos = np.asarray(list(positions), dtype=np.float32)[:, None]
    angle = (pos * inv_freq[None, :]).astype(np.float32).astype(np.float64)
    c = torch.from_numpy(np.cos(angle))[:, None, :]
    s = torch.from_numpy(np.sin(angle))[:, None, :]
    x1, x2 = v[..., :half], v[..., half:]
    return torch.cat([x1 * c - x2 * s, x2 * c + x1 * s], dim=-1)


def attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, rnd: Callable = identity,
              window: Optional[int] = None, partition: Optional[int] = None, first_position: int = 0) -> torch.Tensor:
    """Causal grouped-query attention over one whole sequence (src/kernels.cpp:312-368).
    q: [T, heads, hd]; k, v: [T, kv_heads, hd].  Head h reads kv head h // group; the score
    is dot(q, k) * (1/sqrt(hd)) (scale after the dot); the query at position p sees keys
    0..p; weights are exp(s - max) and the output is sum(e*v) * (1/sum(e)).

    ``partition`` (with a rounding ``rnd``; the reference has neither): where a weight is rounded.  The engine's
    bfloat16 path cuts the keys at absolute positions into partitions of that many and rounds a weight against
    the maximum of its own partition's visible scores, rnd(exp(s - m_partition)); the partitions are then
    weighed against each other by exp(m_partition - max) unrounded.  Without rounding this is the formula
    above, term for term."""
    T, heads, hd = q.shape
    group = heads // k.shape[1]
    scale = 1.0 / math.sqrt(hd)
    out = torch.zeros(T, heads, hd, dtype=F64)
    for h in range(heads):
        kh, vh = k[:, h // group], v[:, h // group]
        for p in range(T):
            lo = 0 if window is None else max(0, p - window + 1)
            s = (kh[lo:p + 1] @ q[p, h]) * scale
            if partition is None:
                e = rnd(torch.exp(s - s.max()))
            else:
                part = (torch.arange(lo, p + 1) + first_position) // partition
                part = part - part[0]
                maxima = torch.full((int(part[-1]) + 1,), -math.inf, dtype=F64).scatter_reduce(0, part, s, "amax")
                local = maxima[part]                                                   # each key's partition's maximum
                e = rnd(torch.exp(s - local)) * torch.exp(local - s.max())
            out[p, h] = (e[:, None] * vh[lo:p + 1]).sum(0) * (1.0 / e.sum())
    return out


def swiglu(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """h = g * (1/(1+exp(-g))) * u (src/kernels.cpp:291-298)."""
    return gate * (1.0 / (1.0 + torch.exp(-gate))) * up


def attention_block(x, w, pre, c, positions, rnd, window=None, partition=None):
    """Steps 3-8 of the layer (src/model.cpp:281-300): norm, q/k/v projections (the engine's
    stacked QKV GEMM is the three projections side by side, src/model.cpp:150-153), rotary
    on q and k, attention, output projection."""
    T = x.shape[0]
    xn = rnd(rmsnorm(x, w[pre + "input_layernorm.weight"], c["eps"]))
    q = linear(xn, w[pre + "self_attn.q_proj.weight"]).view(T, c["heads"], c["head_dim"])
    k = linear(xn, w[pre + "self_attn.k_proj.weight"]).view(T, c["kv_heads"], c["head_dim"])
    v = linear(xn, w[pre + "self_attn.v_proj.weight"]).view(T, c["kv_heads"], c["head_dim"])
    inv_freq = rope_inv_freq(c["theta"], c["head_dim"])
    q, k, v = rnd(rope(q, positions, inv_freq)), rnd(rope(k, positions, inv_freq)), rnd(v)
    a = rnd(attention(q, k, v, rnd, window, partition, positions[0])).reshape(T, -1)
    return linear(a, w[pre + "self_attn.o_proj.weight"])


def mlp_block(x, w, pre, c, rnd):
    """Steps 9-12 (src/model.cpp:301-305): norm, gate and up projections, SwiGLU, down."""
    xn = rnd(rmsnorm(x, w[pre + "post_attention_layernorm.weight"], c["eps"]))
    h = rnd(swiglu(linear(xn, w[pre + "mlp.gate_proj.weight"]), linear(xn, w[pre + "mlp.up_proj.weight"])))
    return linear(h, w[pre + "mlp.down_proj.weight"])


def forward(config: Mapping[str, object], w: Mapping[str, torch.Tensor], tokens: Sequence[int],
            rnd: Callable = identity, first_position: int = 0, windows: Optional[Sequence[Optional[int]]] = None,
            partition: Optional[int] = None) -> torch.Tensor:
    """Logits [T, vocab] (float64) at every position of one whole sequence
    (src/model.cpp:267-322 with every row wanted, as python/bindings.cpp:35-52 does).
    ``first_position`` shifts all positions (only distances matter to rotary attention).
    ``windows``: per layer, how many keys a query sees (None: all; the reference has no window).
    ``partition``: see ``attention``."""
    c = read_config(config)
    positions = [first_position + i for i in range(len(tokens))]
    x = embed(tokens, w["model.embed_tokens.weight"])
    for layer in range(c["layers"]):
        pre = f"model.layers.{layer}."
        x = x + attention_block(x, w, pre, c, positions, rnd, None if windows is None else windows[layer], partition)
        x = x + mlp_block(x, w, pre, c, rnd)
    x = rnd(rmsnorm(x, w["model.norm.weight"], c["eps"]))
    head = w["model.embed_tokens.weight"] if c["tied"] else w["lm_head.weight"]
    return linear(x, head)


# ----------------------------------------------------------------------------- sampling

_M64 = (1 << 64) - 1


def mix64(z: int) -> int:
    """splitmix64 finaliser (src/engine.cpp:12-16)."""
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _M64
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _M64
    return z ^ (z >> 31)


def counter_uniform(seed: int, position: int, stream: int = 0) -> float:
    """(z >> 11) * 2**-53 with z = mix64(mix64(seed ^ C) ^ mix64(position*4 + stream))
    (src/engine.cpp:35-38)."""
    z = mix64(mix64((seed ^ 0x6A09E667F3BCC909) & _M64) ^ mix64((position * 4 + stream) & _M64))
    return (z >> 11) * 2.0 ** -53


def argmax_row(logits: np.ndarray) -> int:
    """Strict '>' scan: the first maximum wins (src/engine.cpp:40-45)."""
    best = 0
    for i in range(1, len(logits)):
        if logits[i] > logits[best]:
            best = i
    return best


def sample_row(logits: np.ndarray, temperature: float, u: float, expf=np.exp) -> int:
    """w[i] = expf((l[i]-max)/T) in 32-bit, total and running sum in double, first i with
    cum > u*total, else the last index with positive weight (src/engine.cpp:50-80).  ``expf``: the
    32-bit exponential (the library's, or the engine's own definition)."""
    l32 = np.asarray(logits, dtype=np.float32)
    w = np.asarray(expf((l32 - l32.max()) / np.float32(temperature)), dtype=np.float32)
    total = 0.0
    for x in w.tolist():
        total += x
    target = u * total
    cum, last = 0.0, 0
    for i, x in enumerate(w.tolist()):
        if x <= 0.0:
            continue
        cum += x
        last = i
        if cum > target:
            return last
    return last


def hash_floats(h: int, row: np.ndarray) -> int:
    """FNV-style chain over the 8-byte words of the raw 32-bit floats, then mix64
    (src/engine.cpp:18-29); the chain starts from 1469598103934665603 (src/engine.h:68)."""
    raw = np.asarray(row, dtype="<f4").tobytes()
    n8 = len(raw) // 8 * 8
    for (wd,) in struct.iter_unpack("<Q", raw[:n8]):
        h = ((h ^ wd) * 1099511628211) & _M64
    for b in raw[n8:]:
        h = ((h ^ b) * 1099511628211) & _M64
    return mix64(h)


def block_hash(parent: int, tokens: Sequence[int]) -> int:
    """FNV-1a over parent ^ basis and the page's tokens, then a 64-bit mixer
    (src/block_manager.cpp:8-19)."""
    h = 1469598103934665603 ^ parent
    for t in tokens:
        h ^= t & 0xFFFFFFFF
        h = (h * 1099511628211) & _M64
    h ^= h >> 33
    h = (h * 0xff51afd7ed558ccd) & _M64
    h ^= h >> 33
    return h


def generate(config, w, prompt: List[int], max_new_tokens: int, temperature: float = 0.0, seed: int = 0,
             ignore_eos: bool = False, rnd: Callable = identity, partition: Optional[int] = None) -> List[int]:
    """Whole-sequence recomputation for every new token; sampling position is the number of
    tokens held before the new one (src/engine.cpp:467-476), stop rules of :250-254."""
    c = read_config(config)
    toks = list(prompt)
    out: List[int] = []
    for _ in range(max_new_tokens):
        row = forward(config, w, toks, rnd, partition=partition)[-1].to(torch.float32).numpy()
        if temperature <= 0:
            t = argmax_row(row)
        else:
            t = sample_row(row, temperature, counter_uniform(seed, len(toks), 0))
        toks.append(t)
        out.append(t)
        if not ignore_eos and t == c["eos"]:
            break
    return out
