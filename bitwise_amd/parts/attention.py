"""Causal grouped-query attention over the paged cache (src/model.cpp:281-300).

One stacked projection [q; k; v] (src/model.cpp:150-153), rotary encoding of q and k and the
cache write in one kernel, attention over keys lo..p of the row's own sequence, output
projection added into the residual stream.  The part knows its sizes and nothing else: which
cache it reads, which block table belongs to it and where its rows sit arrive with the call.
"""

from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Dict, Optional

import numpy as np
import torch

from ..csrc import ops
from .base import CacheSpec, Mixer, TensorSpec, lookup, register_mixer, POSITION_ENCODINGS
from .linear import Linear

# A decoded token's attention goes to the kernel that gives every 64-key partition a wave of its
# own once its context is at least this long (same bits either way; this only buys parallelism).
DECODE_MIN_CONTEXT = 128


@dataclass
class AttentionPlan:
    """Which rows of a step the attention kernels treat together: tiles (first row, rows, request, 0)."""
    fold_tiles: Optional[torch.Tensor]
    fold_count: int
    decode_tiles: Optional[torch.Tensor]      # None with a positive count: tile t is row t of request t
    decode_count: int


def plan_tiles(ctx, tokens_per_tile: int, group_tiles: int = 1) -> AttentionPlan:
    """Cut a step's segments into tiles of up to ``tokens_per_tile`` consecutive rows of one request; every
    request's run of tiles is padded with empty tiles to a multiple of ``group_tiles`` (the tiles one wave owns
    must belong to one request).  Single decoded tokens with a long context go to the decode kernel (a wave per
    64-key partition).  A step of nothing but one row per request (``ctx.one_row_per_request``, the shape of a
    captured decode step) needs no tile list: tile t is row t of request t.  The plan is made once per step
    and kept in the context for the other layers."""
    if getattr(ctx, "one_row_per_request", False):
        return AttentionPlan(None, 0, None, ctx.rows)

    def make() -> AttentionPlan:
        fold, split = [], []
        for i, s in enumerate(ctx.segments):
            n, r0 = len(s.tokens), ctx.seq_start[i]
            if n == 1 and s.pos0 + 1 >= DECODE_MIN_CONTEXT:
                split.append((r0, 1, i, 0))
                continue
            for off in range(0, n, tokens_per_tile):
                fold.append((r0 + off, min(tokens_per_tile, n - off), i, 0))
            while len(fold) % group_tiles:
                fold.append((r0, 0, i, 0))
        both = np.asarray(fold + split, np.int32).reshape(-1, 4)
        dev = torch.from_numpy(both).to(ctx.device)
        return AttentionPlan(dev[:len(fold)].contiguous() if fold else None, len(fold),
                             dev[len(fold):].contiguous() if split else None, len(split))

    return ctx.memo(("attention_tiles", tokens_per_tile, group_tiles), make)


@register_mixer("attention")
class Attention(Mixer):
    """params: width, heads, kv_heads, head_dim, window (None = all keys), position (PartSpec
    of the position encoding).  tensors: q_proj/k_proj/v_proj/o_proj .weight."""

    launches_through_ops = True

    def __init__(self, params, runtime):
        super().__init__(params, runtime)
        p = params
        self.width, self.heads, self.kv_heads, self.head_dim = int(p["width"]), int(p["heads"]), int(p["kv_heads"]), int(p["head_dim"])
        self.window: Optional[int] = p.get("window")
        if self.heads % self.kv_heads:
            raise ValueError(f"attention: {self.heads} heads are no multiple of {self.kv_heads} kv heads")
        if self.head_dim not in ops.HEAD_DIMS:
            raise ValueError(f"attention: head size {self.head_dim} is not supported by the kernels; "
                             f"supported: {ops.HEAD_DIMS}")
        self.q_dim, self.kv_dim = self.heads * self.head_dim, self.kv_heads * self.head_dim
        self.scale = 1.0 / math.sqrt(float(self.head_dim))     # 1.0f / sqrtf(float(hd)), src/kernels.cpp:347
        pos = p["position"]
        self.position = lookup(POSITION_ENCODINGS, "position encoding", pos.kind).shared(pos.params, runtime)
        if int(getattr(self.position, "rotary_dim", 0)) != self.head_dim:
            raise ValueError(f"attention: this part rotates whole heads of {self.head_dim}; position encoding '{pos.kind}' "
                             f"rotates {getattr(self.position, 'rotary_dim', 0)} elements of a head and needs a mixer of its own")
        self.graph_safe = bool(getattr(self.position, "graph_safe", False))    # the tables must be device tensors
        self.cos = self.sin = None
        self.qkv: Optional[Linear] = None
        self.o: Optional[Linear] = None
        group = self.heads // self.kv_heads
        self.heads_per_tile = min(group, 16)
        self.tokens_per_tile = 16 // self.heads_per_tile

    def tensors(self) -> Dict[str, TensorSpec]:
        return {
            "q_proj.weight": TensorSpec((self.q_dim, self.width)),
            "k_proj.weight": TensorSpec((self.kv_dim, self.width)),
            "v_proj.weight": TensorSpec((self.kv_dim, self.width)),
            "o_proj.weight": TensorSpec((self.width, self.q_dim)),
        }

    def _tables(self):
        """The position encoding's tables, checked once against what the kernels index: [positions, head size / 2],
        32-bit, contiguous, on the device."""
        if self.cos is None:
            cos, sin = self.position.tables()
            for name, t in (("cos", cos), ("sin", sin)):
                if (not isinstance(t, torch.Tensor) or t.dtype != torch.float32 or t.dim() != 2 or t.shape[1] != self.head_dim // 2
                        or not t.is_contiguous() or t.device != self.rt.device or t.shape != cos.shape):
                    raise ValueError(f"attention: the position encoding's {name} table must be a contiguous float32 "
                                     f"[positions, {self.head_dim // 2}] tensor on {self.rt.device}")
            self.cos, self.sin = cos, sin
        return self.cos, self.sin

    def page_sizes(self):
        return ops.PAGE_SIZES

    def bind(self, tensors) -> None:
        self._tables()
        q, k, v = tensors["q_proj.weight"], tensors["k_proj.weight"], tensors["v_proj.weight"]
        if not (q.dtype == k.dtype == v.dtype):
            raise ValueError("q, k and v projections must be stored in one dtype to be stacked")
        self.qkv = Linear(torch.cat([q, k, v], dim=0), self.rt)
        self.o = Linear(tensors["o_proj.weight"], self.rt)

    def weight_bytes(self) -> int:
        return self.qkv.nbytes() + self.o.nbytes()

    def cache_spec(self) -> CacheSpec:
        return CacheSpec(self.kv_heads, self.head_dim, self.window)

    def page_elements(self, page_size: int) -> int:
        """Elements of one page of keys (and likewise of values) of one cache."""
        return self.kv_heads * page_size * self.head_dim

    def forward_with_norm(self, ctx, call, x, norm, residual) -> bool:
        """Decode steps of few rows: norm, q|k|v product, rotation and cache write are one kernel."""
        from .norm import RMSNorm
        rt, ws = self.rt, ctx.ws
        inner = self.qkv.weight.shape[1]
        # (rows wider than a segment of K: only the kernel with a workgroup per half head takes them)
        takes_width = inner <= 2048 or ops.qkv_rope_gemm_ok(ctx.rows, self.head_dim, inner, self.heads + 2 * self.kv_heads)
        if not (rt.bf16 and isinstance(norm, RMSNorm) and self.qkv.mfma and takes_width
                and ops.qkv_rope_head_dim_ok(self.head_dim, inner)
                and ops.can_fuse_norm(ctx.rows, self.qkv.weight, x)):
            return False
        q = ws.buffer("q_rot", self.q_dim, torch.bfloat16)
        ops.norm_qkv_rope_bf16(x, norm.weight, norm.eps, self.qkv.weight, q, ctx.positions, ctx.row_seq,
                               ctx.block_tables[call.group], self.cos, self.sin, call.k_cache,
                               call.v_cache, ctx.rows, self.heads, self.kv_heads, self.head_dim, ws.page_size,
                               call.writes_cache)
        self._attend(ctx, call, q, residual)
        return True

    def forward(self, ctx, call, h, residual) -> None:
        rt, ws, rows = self.rt, ctx.ws, ctx.rows
        table = ctx.block_tables[call.group]
        window = int(self.window or 0)
        if rt.bf16 and self.qkv.mfma and ops.qkv_rope_gemm_ok(rows, self.head_dim, self.qkv.weight.shape[1],
                                                              self.heads + 2 * self.kv_heads):
            # rotation and cache write ride in the product's epilogue
            q = ws.buffer("q_rot", self.q_dim, torch.bfloat16)
            ops.gemm_qkv_rope_bf16(h, self.qkv.weight, q, ctx.positions, ctx.row_seq, table, self.cos,
                                   self.sin, call.k_cache, call.v_cache, rows, self.heads, self.kv_heads,
                                   self.head_dim, ws.page_size, call.writes_cache)
            self._attend(ctx, call, q, residual)
            return
        qkv = ws.buffer("qkv", self.q_dim + 2 * self.kv_dim, torch.float32)
        self.qkv.store(ws, h, qkv, rows)
        if rt.bf16:
            q = ws.buffer("q_rot", self.q_dim, torch.bfloat16)
            ops.rope_kvwrite(qkv, q, ctx.positions, ctx.row_seq, table, self.cos, self.sin,
                             call.k_cache, call.v_cache, rows, self.heads, self.kv_heads, self.head_dim,
                             ws.page_size, call.writes_cache)
            self._attend(ctx, call, q, residual)
        else:
            ops.rope_kvwrite(qkv, None, ctx.positions, ctx.row_seq, table, self.cos, self.sin,
                             call.k_cache, call.v_cache, rows, self.heads, self.kv_heads, self.head_dim,
                             ws.page_size, call.writes_cache)
            out = ws.buffer("attn_out", self.q_dim, torch.float32)
            # prompt portions: tiles of 32 rows, a wave a tile, both products on the matrix cores; for head sizes
            # that fill the second product's blocks badly (80 to 112) tiles of 16 rows on the vector units
            on_matrix_cores = self.head_dim <= 64 or self.head_dim == 128
            plan = plan_tiles(ctx, 32 if on_matrix_cores else 16, 1)
            common = (call.k_cache, call.v_cache, out, self.heads, self.kv_heads, self.head_dim, ws.page_size,
                      window, self.scale)
            if plan.fold_count and self.head_dim > 128 or (plan.decode_count and plan.decode_tiles is None):
                # every row by itself (also: a batch of nothing but decoded tokens, row t of request t)
                ops.attention_f32(qkv, ctx.positions, ctx.row_seq, table, call.k_cache, call.v_cache, out, rows,
                                  self.heads, self.kv_heads, self.head_dim, ws.page_size, window, self.scale)
            else:
                if plan.fold_count:      # prompt portions: a tile's rows share the keys and values they load
                    ops.attention_f32_tiles(qkv, ctx.positions, table, plan.fold_tiles, plan.fold_count,
                                            2 if on_matrix_cores else 1, *common)
                if plan.decode_count:
                    ops.attention_f32_tiles(qkv, ctx.positions, table, plan.decode_tiles, plan.decode_count, False, *common)
            self.o.add_into(ws, out, residual, rows)

    def _split_scratch(self, ws, tiles: int, table_width: int):
        """(floats, counters) of the split decode's scratch for this workspace: the worst case over the launches it
        can see, or (0, 0) if this launch would not split."""
        if not ops.attention_decode_scratch(tiles, self.heads, self.kv_heads, self.head_dim, table_width, ws.page_size)[0]:
            return 0, 0
        width = max(table_width, ws.max_table_width or 0)
        key = ("attn_split_size", self.heads, self.kv_heads, self.head_dim, width)
        sizes = ws.notes.get(key)
        if sizes is None:
            floats = counters = 0
            for t in range(1, min(ws.max_rows, 256) + 1):            # (from 256 workgroups on nothing splits)
                f, c = ops.attention_decode_scratch(t, self.heads, self.kv_heads, self.head_dim, width, ws.page_size)
                floats, counters = max(floats, f), max(counters, c)
            sizes = ws.notes[key] = (floats, counters)
        return sizes

    def _attend(self, ctx, call, q, residual) -> None:
        """bfloat16 attention over the cache for rotated queries ``q``, then the output projection."""
        ws, rows = ctx.ws, ctx.rows
        table = ctx.block_tables[call.group]
        window = int(self.window or 0)
        out = ws.buffer("attn_out", self.q_dim, torch.bfloat16)
        plan = plan_tiles(ctx, self.tokens_per_tile, ops.fold_group_tiles(self.head_dim))
        common = (call.k_cache, call.v_cache, out, self.heads, self.kv_heads, self.head_dim, ws.page_size,
                  window, self.scale)
        if plan.fold_count:
            ops.attention_bf16(q, ctx.positions, table, plan.fold_tiles, plan.fold_count, *common)
        if plan.decode_count:
            # few decoded tokens: several workgroups a tile, meeting in device scratch.  One buffer a workspace, sized
            # for the worst launch it can see (the most tiles that still split, the widest table), whatever this
            # step's shape: tables grow by a page every few steps, and a buffer per width would pile up.
            floats, counters = self._split_scratch(ws, plan.decode_count, table.stride(0))
            scratch = None
            if floats:
                scratch = (ws.buffer("attn_split", floats, torch.float32, rows=1),
                           ws.buffer("attn_split_count", counters, torch.int32, rows=1))
            ops.attention_bf16(q, ctx.positions, table, plan.decode_tiles, plan.decode_count, *common, decode=True,
                               scratch=scratch)
        self.o.add_into(ws, out, residual, rows)
