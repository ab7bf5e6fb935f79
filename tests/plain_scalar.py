"""Python face of the plain scalar 32-bit decoder (plain_scalar.cpp): compiles it for the CPU
with g++ into a temporary folder at first use and calls it through ctypes.  It is what the
engine's 32-bit path must equal bit for bit; the float64 model in plain_llama.py stays the
independent check at a tolerance."""

from __future__ import annotations

import ctypes
import os
import subprocess
import tempfile
from ctypes import c_float, c_int, c_longlong, c_void_p
from pathlib import Path
from typing import Mapping, Optional, Sequence

import numpy as np

HERE = Path(__file__).resolve().parent
_lib: Optional[ctypes.CDLL] = None


def library() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        src = HERE / "plain_scalar.cpp"
        out_dir = Path(tempfile.gettempdir()) / f"bitwise_amd_plain_{os.getuid()}"
        out_dir.mkdir(exist_ok=True)
        so = out_dir / f"plain_scalar_{int(src.stat().st_mtime)}_{src.stat().st_size}.so"
        if not so.exists():
            flags = ["-O2", "-ffp-contract=off", "-fno-fast-math", "-std=c++17", "-shared", "-fPIC"]
            try:
                if " fma " in open("/proc/cpuinfo").read():
                    flags.append("-mfma")            # std::fma as one instruction; the software one gives the same bits
            except OSError:
                pass
            tmp = so.with_suffix(f".tmp{os.getpid()}")
            subprocess.run(["g++", *flags, str(src), "-o", str(tmp)], check=True)
            os.replace(tmp, so)
        _lib = ctypes.CDLL(str(so))
        _lib.plain_dot_canonical.restype = c_float
    return _lib


def _f32(a) -> np.ndarray:
    return np.ascontiguousarray(np.asarray(a, dtype=np.float32))


def _p(a: np.ndarray) -> c_void_p:
    return a.ctypes.data_as(c_void_p)


def expf(x) -> np.ndarray:
    x = _f32(x)
    y = np.empty_like(x)
    library().plain_expf(_p(x), _p(y), c_longlong(x.size))
    return y


def swiglu(gate, up) -> np.ndarray:
    g, u = _f32(gate), _f32(up)
    h = np.empty_like(g)
    library().plain_swiglu(_p(g), _p(u), _p(h), c_longlong(g.size))
    return h


def linear(x, w) -> np.ndarray:
    x, w = _f32(x), _f32(w)
    M, K = x.shape
    N = w.shape[0]
    y = np.empty((M, N), np.float32)
    library().plain_linear(_p(x), _p(w), _p(y), c_int(M), c_int(N), c_int(K))
    return y


def rmsnorm(x, w, eps: float) -> np.ndarray:
    x, w = _f32(x), _f32(w)
    y = np.empty_like(x)
    library().plain_rmsnorm(_p(x), _p(w), _p(y), c_int(x.shape[0]), c_int(x.shape[1]), c_float(eps))
    return y


def dot_canonical(a, b) -> np.float32:
    a, b = _f32(a), _f32(b)
    return np.float32(library().plain_dot_canonical(_p(a), _p(b), c_int(a.size)))


def attention(q, k, v, window: int = 0) -> np.ndarray:
    """q [T, heads, hd], k and v [T, kv_heads, hd], rotated already; out [T, heads, hd]."""
    q, k, v = _f32(q), _f32(k), _f32(v)
    T, heads, hd = q.shape
    out = np.empty_like(q)
    library().plain_attention(_p(q), _p(k), _p(v), _p(out), c_int(T), c_int(heads), c_int(k.shape[1]), c_int(hd),
                              c_int(window))
    return out


def rope_tables(theta: float, head_dim: int, positions: Sequence[int]):
    """inv_freq[i] = 1.0f / powf(theta, float(2i)/float(hd)) (src/model.cpp:220-225) and
    angle = float(pos) * inv_freq[i] in 32-bit (src/kernels.cpp:277-279); cosine and sine of that
    32-bit angle evaluated in double and rounded once (the reference calls libm's cosf and sinf,
    whose bits differ between machines)."""
    i = np.arange(head_dim // 2, dtype=np.float32)
    inv = (np.float32(1.0) / np.power(np.float32(theta), (np.float32(2.0) * i) / np.float32(head_dim),
                                      dtype=np.float32)).astype(np.float32)
    pos = np.asarray(list(positions), dtype=np.float32)[:, None]
    angle = (pos * inv[None, :]).astype(np.float32).astype(np.float64)
    return np.cos(angle).astype(np.float32), np.sin(angle).astype(np.float32)


def forward(config: Mapping[str, object], w: Mapping[str, object], tokens: Sequence[int], window=0,
            first_position: int = 0) -> np.ndarray:
    """Logits [T, vocab] (float32) of one whole sequence.  ``w``: tensors by checkpoint name (torch or
    numpy; bfloat16 is widened exactly).  Keys and defaults of tools/convert.py:55-80.  ``window``: keys a
    query sees, one number for all layers or a list with one per layer (0 or None: all keys)."""
    import torch

    heads = int(config["num_attention_heads"])
    H, L, V, I = int(config["hidden_size"]), int(config["num_hidden_layers"]), int(config["vocab_size"]), int(config["intermediate_size"])
    kvh = int(config.get("num_key_value_heads", heads))
    hd = int(config.get("head_dim") or H // heads)
    eps = float(config.get("rms_norm_eps", 1e-6))
    theta = float(config.get("rope_theta", 10000.0))
    tied = bool(config.get("tie_word_embeddings", False))

    def t(name):
        x = w[name]
        if isinstance(x, torch.Tensor):
            x = x.to(torch.float32).cpu().numpy()
        return np.ascontiguousarray(x, dtype=np.float32).reshape(-1)

    parts = [t("model.embed_tokens.weight")]
    for l in range(L):
        pre = f"model.layers.{l}."
        parts += [t(pre + "input_layernorm.weight"), t(pre + "self_attn.q_proj.weight"), t(pre + "self_attn.k_proj.weight"),
                  t(pre + "self_attn.v_proj.weight"), t(pre + "self_attn.o_proj.weight"),
                  t(pre + "post_attention_layernorm.weight"), t(pre + "mlp.gate_proj.weight"),
                  t(pre + "mlp.up_proj.weight"), t(pre + "mlp.down_proj.weight")]
    parts += [t("model.norm.weight"), t("model.embed_tokens.weight" if tied else "lm_head.weight")]
    blob = np.concatenate(parts)
    T = len(tokens)
    toks = np.ascontiguousarray(np.asarray(list(tokens), dtype=np.int32))
    cos, sin = rope_tables(theta, hd, range(first_position, first_position + T))
    cos, sin = np.ascontiguousarray(cos), np.ascontiguousarray(sin)
    wins = list(window) if isinstance(window, (list, tuple)) else [window] * L
    wins = np.ascontiguousarray(np.asarray([int(x or 0) for x in wins], dtype=np.int32))
    assert wins.size == L
    out = np.empty((T, V), np.float32)
    library().plain_forward(_p(blob), _p(toks), c_int(T), c_int(V), c_int(H), c_int(L), c_int(heads), c_int(kvh),
                            c_int(hd), c_int(I), c_float(eps), _p(wins), _p(cos), _p(sin), _p(out))
    return out
