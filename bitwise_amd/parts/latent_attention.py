"""Causal attention over a compressed cache: per token one latent vector (RMS-normed) and one rotated key
part shared by all heads are cached; a head's key is [W_uk c | rotated part], its value W_uv c.

The scores are taken in the cache's own space: q_unrotated . (W_uk c) = (W_uk^T q_unrotated) . c, so a head's
query becomes [W_uk^T q_unrotated | q_rotated] and one dot product with the cached vector is the score; the
softmax-weighted sum of cached latents is projected to the head's values by W_uv afterwards.  The softmax has
a sink: one learned number per head that enters the denominator as exp(sink) beside the keys' terms (nothing is
looked up for it, nothing is added to the output for it, and the score scale does not apply to it).

Rotations, the latent's norm, scores and softmax weights are 32-bit in both modes; the cache holds the mode's
activation dtype.
"""

from __future__ import annotations

from typing import Dict, Optional

import numpy as np
import torch

from ..csrc import ops
from .base import CacheSpec, Mixer, TensorSpec, lookup, register_mixer, POSITION_ENCODINGS
from .linear import Linear

ROWS_PER_PROMPT_TILE = 4        # the 32-bit kernel: 16 query vectors a workgroup, 4 rows x 4 heads or a single token's 16 heads
MAX_SPLITS = 64                 # pieces a single token's keys are cut into at most (each a multiple of 64 keys)


def _tiles(ctx, rows_per_tile: int):
    """(prompt tiles, count, single-token tiles, count): tiles (first row, rows, request, 0) of up to ``rows_per_tile``
    consecutive rows of a request; single tokens apart (their workgroups take 16 heads each).  None with a positive
    count: tile t is row t of request t (a step of one row per request)."""
    if getattr(ctx, "one_row_per_request", False):
        return None, 0, None, ctx.rows

    def make():
        many, single = [], []
        for i, s in enumerate(ctx.segments):
            n, r0 = len(s.tokens), ctx.seq_start[i]
            if n == 1:
                single.append((r0, 1, i, 0))
                continue
            for off in range(0, n, rows_per_tile):
                many.append((r0 + off, min(rows_per_tile, n - off), i, 0))
        both = torch.from_numpy(np.asarray(many + single, np.int32).reshape(-1, 4)).to(ctx.device)
        return (both[:len(many)].contiguous() if many else None, len(many),
                both[len(many):].contiguous() if single else None, len(single))

    return ctx.memo(("shared_key_tiles", rows_per_tile), make)


@register_mixer("latent_attention")
class LatentAttention(Mixer):
    """params: width, heads, dim (unrotated query/key elements a head), rot_dim (rotated ones), vdim, kv_rank, scale, eps
    (of the latent's norm), window (None: all keys), position (PartSpec of the rotary tables; it may rotate fewer than
    rot_dim elements, the rest of the rotated part passes unchanged).
    tensors: q [heads*(dim+rot_dim), width]; dkv [kv_rank+rot_dim, width]; dkv.norm [kv_rank]; uk [heads*dim, kv_rank];
    uv [heads*vdim, kv_rank]; sink [heads]; o [width, heads*vdim]."""

    launches_through_ops = True

    def __init__(self, params, runtime):
        super().__init__(params, runtime)
        p = params
        self.width, self.heads = int(p["width"]), int(p["heads"])
        self.dim, self.rot, self.vdim, self.rank = int(p["dim"]), int(p["rot_dim"]), int(p["vdim"]), int(p["kv_rank"])
        self.scale, self.eps = float(p["scale"]), float(p["eps"])
        self.window: Optional[int] = p.get("window")
        self.key_width = self.rank + self.rot
        if self.rank > 512:
            raise ValueError(f"latent_attention: a latent of {self.rank} elements; the kernel takes up to 512")
        pos = p["position"]
        self.position = lookup(POSITION_ENCODINGS, "position encoding", pos.kind).shared(pos.params, runtime)
        self.rotary = int(getattr(self.position, "rotary_dim", 0))
        if self.rotary % 2 or self.rotary > self.rot:
            raise ValueError(f"latent_attention: the position encoding rotates {self.rotary} elements, the rotated part has {self.rot}")
        self.graph_safe = bool(getattr(self.position, "graph_safe", False))
        self.cos = self.sin = None
        self.proj: Optional[Linear] = None
        self.o: Optional[Linear] = None
        # bfloat16 mode: the attention runs on the matrix cores and keeps the latents a second time, transposed within
        # their pages, as the values (the page sizes it takes: multiples of 4); the 32-bit mode reads values and keys
        # from the one copy
        self.on_matrix_cores = bool(runtime.bf16) and self.key_width % 8 == 0
        # heads that share a wave's 16 query vectors in prompt portions: the power of two from the number of heads up
        self.heads_per_group = 1
        while self.heads_per_group < min(self.heads, 16):
            self.heads_per_group *= 2

    def tensors(self) -> Dict[str, TensorSpec]:
        return {
            "q": TensorSpec((self.heads * (self.dim + self.rot), self.width)),
            "dkv": TensorSpec((self.key_width, self.width)),
            "dkv.norm": TensorSpec((self.rank,), "norm"),
            "uk": TensorSpec((self.heads * self.dim, self.rank)),
            "uv": TensorSpec((self.heads * self.vdim, self.rank)),
            "sink": TensorSpec((self.heads,), "bias"),
            "o": TensorSpec((self.width, self.heads * self.vdim)),
        }

    def bind(self, tensors) -> None:
        self.cos, self.sin = self.position.tables()
        q, dkv = tensors["q"], tensors["dkv"]
        if q.dtype != dkv.dtype:
            raise ValueError("q and dkv projections must be stored in one dtype to be stacked")
        self.q_off, self.dkv_off = 0, q.shape[0]
        self.proj = Linear(torch.cat([q, dkv], dim=0), self.rt)
        self.o = Linear(tensors["o"], self.rt)
        dev = self.rt.device
        self.latent_norm = tensors["dkv.norm"].to(dev).float().contiguous()
        self.sink = tensors["sink"].to(dev).float().contiguous()
        # input-major per head: uk as stored is [head][dim][rank] (the transposed product wants exactly that);
        # uv [head][vdim][rank] is turned to [head][rank][vdim]
        self.uk_t = tensors["uk"].to(dev).view(self.heads, self.dim, self.rank).contiguous()
        self.uv_t = tensors["uv"].to(dev).view(self.heads, self.vdim, self.rank).transpose(1, 2).contiguous()

    def weight_bytes(self) -> int:
        small = self.uk_t.numel() * self.uk_t.element_size() + self.uv_t.numel() * self.uv_t.element_size()
        return self.proj.nbytes() + self.o.nbytes() + small + 4 * (self.rank + self.heads)

    def cache_spec(self) -> CacheSpec:
        return CacheSpec(1, self.key_width, self.window, key_width=self.key_width,
                         value_width=self.rank if self.on_matrix_cores else 0)

    def page_sizes(self):
        return (4, 8, 16, 32, 64, 128) if self.on_matrix_cores else None

    def forward(self, ctx, call, h, residual) -> None:
        ws, rows = ctx.ws, ctx.rows
        table = ctx.block_tables[call.group]
        y = ws.buffer("latent_proj", self.proj.out_features, torch.float32)
        self.proj.store(ws, h, y, rows)
        mfma = self.on_matrix_cores
        # (the matrix-core kernel takes its queries rounded to bfloat16, so they are stored that way at once)
        qa = ws.buffer("latent_q", self.heads * self.key_width, torch.bfloat16 if mfma else torch.float32)
        ops.latent_prep(y, self.q_off, self.dkv_off, self.latent_norm, self.eps, self.cos, self.sin, ctx.positions, ctx.row_seq,
                        table, call.k_cache, qa, rows, self.heads, self.dim, self.rot, self.rotary, self.rank, ws.page_size,
                        call.writes_cache, latent_t=call.v_cache if mfma else None)
        # the unrotated query parts into the latent's space
        ops.headwise_linear(y, self.q_off, self.dim + self.rot, self.uk_t, qa, 0, self.key_width, rows)
        lat = ws.buffer("latent_out", self.heads * self.rank, torch.float32)
        if mfma:
            self._attend_on_matrix_cores(ctx, call, qa, lat, table)
        else:
            many, n_many, single, n_single = _tiles(ctx, ROWS_PER_PROMPT_TILE)
            common = (call.k_cache, self.sink, lat, self.heads, self.key_width, self.rank, ws.page_size, int(self.window or 0),
                      self.scale)
            if n_many:
                ops.shared_key_attention(qa, ctx.positions, table, many, n_many, *common, 16 // ROWS_PER_PROMPT_TILE)
            if n_single:
                ops.shared_key_attention(qa, ctx.positions, table, single, n_single, *common, 16)
        vals = ws.buffer("latent_values", self.heads * self.vdim, self.rt.act_dtype)
        ops.headwise_linear(lat, 0, self.rank, self.uv_t, vals, 0, self.vdim, rows)
        self.o.add_into(ws, vals, residual, rows)

    def _attend_on_matrix_cores(self, ctx, call, qa, lat, table) -> None:
        ws = ctx.ws
        hg = self.heads_per_group
        many, n_many, single, n_single = _tiles(ctx, 16 // hg)
        common = (call.k_cache, call.v_cache, self.sink, lat, self.heads, self.key_width, self.rank, ws.page_size,
                  int(self.window or 0), self.scale)
        if n_many:
            ops.shared_key_attention_mfma(qa, ctx.positions, table, many, n_many, *common, hg)
        if n_single:
            # Single tokens: the keys a token can have (what its block table spans) are cut into pieces of a multiple of
            # 64, at most MAX_SPLITS of them, a wave each; few tokens with long contexts still fill the chip.  The cut
            # depends on the table's width alone, which a captured step fixes.
            # The pieces are joined in another order than a wave walks its blocks of keys, so a position's last bits would depend
            # on whether it came alone or inside a portion: an engine that promises bits under any cut (Workspace.exact_cuts)
            # keeps single tokens on one wave per 16 heads.
            span = table.shape[1] * ws.page_size
            kchunk = 64 * max(1, -(-span // (64 * MAX_SPLITS)))
            nsplit = 1 if getattr(ws, "exact_cuts", True) else max(1, -(-span // kchunk))
            partial = None
            if nsplit > 1:
                # (room for the most pieces, for the power of two from this step's single tokens up: a few sizes at most)
                tokens = 1 << max(0, n_single - 1).bit_length()
                partial = ws.buffer("latent_split", tokens * MAX_SPLITS * self.heads * (self.rank + 2), torch.float32, rows=1)
            ops.shared_key_attention_mfma(qa, ctx.positions, table, single, n_single, *common, 16, nsplit, kchunk, partial)
