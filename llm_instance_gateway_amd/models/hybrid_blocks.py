"""Building blocks for hybrid stacks: layers whose sequence mixer is either
paged attention or a recurrence with a per-sequence state slot.

Every block works on the engine's flat token batch (prompt portions and
single decoded tokens side by side) and takes its constants as constructor
arguments, so another model family can assemble them differently.

  * `GatedAttention` — grouped-query attention with independent key and
    value head sizes, projection biases, a configurable score scale, an
    optional logarithmic query temperature and an optional sigmoid output
    gate; K/V live in the paged cache.
  * `MinGRU` — the minimal gated recurrent unit: gates read only the current
    token, the state is an fp32 vector per sequence in a slot pool.
  * `XieluMLP` — two-matrix feed-forward with the xIELU activation.

Projections are library GEMMs over fused weights (one GEMM in, one out per
block); everything between them is one HIP kernel each (ops layer).
"""

from __future__ import annotations

import math
from typing import Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from .. import ops


def _param(shape, device, dtype, scale: Optional[float] = None) -> nn.Parameter:
    t = torch.empty(*shape, device=device, dtype=dtype)
    with torch.no_grad():
        if scale is None:
            t.zero_()
        else:
            t.uniform_(-scale, scale)
    return nn.Parameter(t, requires_grad=False)


def softplus64(x: float) -> float:
    return math.log1p(math.exp(-abs(x))) + max(x, 0.0)


class GatedAttention(nn.Module):
    def __init__(
        self, hidden: int, heads: int, kv_heads: int, dim: int, vdim: int,
        scale: float, temp_coef: float = 0.0, temp_every: float = 1.0,
        out_gate: bool = True, device="cpu", dtype=torch.bfloat16,
    ) -> None:
        super().__init__()
        assert heads % kv_heads == 0
        self.heads, self.kv_heads, self.dim, self.vdim = heads, kv_heads, dim, vdim
        self.scale = float(scale)
        self.temp_coef, self.temp_every = float(temp_coef), float(temp_every)
        self.out_gate = out_gate
        self.nq, self.nk, self.nv = heads * dim, kv_heads * dim, kv_heads * vdim
        self.ng = heads * vdim if out_gate else 0
        n_in = self.nq + self.nk + self.nv + self.ng
        s = 1.0 / math.sqrt(hidden)
        # rows: q | k | v | gate
        self.w_in = _param((n_in, hidden), device, dtype, s)
        self.b_in = _param((n_in,), device, dtype, 0.1)
        with torch.no_grad():
            self.b_in[self.nq + self.nk + self.nv :].zero_()  # the gate has no bias
        self.w_o = _param((hidden, heads * vdim), device, dtype, 1.0 / math.sqrt(heads * vdim))

    def cache_spec(self) -> dict:
        return {"kind": "kv", "kv_heads": self.kv_heads, "k_dim": self.dim, "v_dim": self.vdim}

    def load(self, get, prefix: str) -> None:
        """Copy q/k/v(/g) and o from a checkpoint (`get(name)` returns the
        tensor in this module's dtype/device)."""
        parts = [get(prefix + "q"), get(prefix + "k"), get(prefix + "v")]
        bias = [get(prefix + "q.b"), get(prefix + "k.b"), get(prefix + "v.b")]
        if self.out_gate:
            parts.append(get(prefix + "g"))
            bias.append(torch.zeros(self.ng, device=self.b_in.device, dtype=self.b_in.dtype))
        with torch.no_grad():
            self.w_in.copy_(torch.cat(parts, dim=0))
            self.b_in.copy_(torch.cat(bias, dim=0))
            self.w_o.copy_(get(prefix + "o"))

    def forward(self, h, positions, cache, meta):
        k_cache, v_cache = cache
        proj = F.linear(h, self.w_in, self.b_in)
        a, b, c = self.nq, self.nq + self.nk, self.nq + self.nk + self.nv
        q, k, v = proj[:, :a], proj[:, a:b], proj[:, b:c]
        gate = proj[:, c:] if self.out_gate else None
        ops.kv_scatter(k, v, k_cache, v_cache, meta.slot_mapping)
        if ops.mfma_attention_supported(
            proj.dtype, self.dim, self.vdim, proj.is_cuda, self.heads // self.kv_heads
        ):
            o = self._attend_mfma(q, gate, positions, k_cache, v_cache, meta)
        elif (
            meta.num_prefill_tokens > 0
            and meta.prefill_tile_seq is not None
            and ops.tiled_prefill_supported(proj.dtype, self.dim, self.vdim, proj.is_cuda)
        ):
            # prompt portions on MFMA tiles (temperature and gate fused), the
            # step's single tokens (and pad rows) through the any-shape kernel
            np_, rows = meta.num_prefill_tokens, proj.shape[0]
            o = torch.empty(rows, self.heads * self.vdim, dtype=proj.dtype, device=proj.device)
            ops.paged_attention_prefill_tiles(
                q[:np_], k_cache, v_cache, meta.prefill_block_tables,
                meta.prefill_query_start_locs, meta.prefill_context_lens,
                meta.prefill_tile_seq, meta.prefill_tile_qstart, self.scale, self.heads,
                gate=None if gate is None else gate[:np_], temp_coef=self.temp_coef,
                temp_every=self.temp_every, out=o[:np_],
            )
            if rows > np_:
                ops.paged_attention_general(
                    q[np_:], k_cache, v_cache, meta.seq_block_tables, meta.tok_seq[np_:],
                    positions[np_:], self.scale, self.heads,
                    gate=None if gate is None else gate[np_:], temp_coef=self.temp_coef,
                    temp_every=self.temp_every, out=o[np_:],
                )
        else:
            o = ops.paged_attention_general(
                q, k_cache, v_cache, meta.seq_block_tables, meta.tok_seq, positions,
                self.scale, self.heads, gate=gate, temp_coef=self.temp_coef,
                temp_every=self.temp_every,
            )
        return F.linear(o, self.w_o)

    def _attend_mfma(self, q, gate, positions, k_cache, v_cache, meta):
        """bf16, key size == value size in {64, 128}: the MFMA flash-prefill
        and paged-decode kernels do the softmax(QK^T)V; the temperature is
        folded into q beforehand and the gate applied afterwards."""
        qh = ops.temperature_scale_rows(q, positions, self.temp_coef, self.temp_every)
        qh = qh.view(-1, self.heads, self.dim)
        np_, nd = meta.num_prefill_tokens, meta.num_decode_tokens
        out = torch.zeros_like(qh) if np_ + nd < qh.shape[0] else torch.empty_like(qh)
        if np_ > 0:
            out[:np_] = ops.paged_attention_prefill(
                qh[:np_], k_cache, v_cache, meta.prefill_block_tables,
                meta.prefill_query_start_locs, meta.prefill_context_lens, self.scale,
                tile_seq=meta.prefill_tile_seq, tile_qstart=meta.prefill_tile_qstart,
            )
        if nd > 0:
            out[np_ : np_ + nd] = ops.paged_attention_decode(
                qh[np_ : np_ + nd], k_cache, v_cache, meta.decode_block_tables,
                meta.decode_context_lens, self.scale, max_ctx=meta.max_decode_ctx,
                nsplits=meta.decode_nsplits,
            )
        o = out.view(-1, self.heads * self.vdim)
        if gate is not None:
            ops.sigmoid_gate_mul(o, gate)
        return o


class MinGRU(nn.Module):
    def __init__(self, hidden: int, width: int, device="cpu", dtype=torch.bfloat16) -> None:
        super().__init__()
        self.width = width
        s = 1.0 / math.sqrt(hidden)
        # rows: update gate z | candidate x | output gate g
        self.w_in = _param((3 * width, hidden), device, dtype, s)
        self.b_in = _param((3 * width,), device, dtype, 0.1)
        with torch.no_grad():
            self.b_in[2 * width :].zero_()
        self.w_o = _param((hidden, width), device, dtype, 1.0 / math.sqrt(width))

    def cache_spec(self) -> dict:
        return {"kind": "state", "width": self.width}

    def load(self, get, prefix: str) -> None:
        zero = torch.zeros(self.width, device=self.b_in.device, dtype=self.b_in.dtype)
        with torch.no_grad():
            self.w_in.copy_(torch.cat([get(prefix + "z"), get(prefix + "x"), get(prefix + "g")], dim=0))
            self.b_in.copy_(torch.cat([get(prefix + "z.b"), get(prefix + "x.b"), zero], dim=0))
            self.w_o.copy_(get(prefix + "o"))

    def forward(self, h, positions, cache, meta):
        (state,) = cache
        zxg = F.linear(h, self.w_in, self.b_in)
        s = ops.mingru_scan(
            zxg, state, meta.seg_start, meta.seg_len, meta.seg_slot,
            meta.seg_fresh, meta.max_seg_len,
        )
        covered = meta.num_prefill_tokens + meta.num_decode_tokens
        if covered < s.shape[0]:
            s[covered:].zero_()  # GEMM-bucketing pad rows belong to no segment
        return F.linear(s, self.w_o)


class XieluMLP(nn.Module):
    def __init__(self, hidden: int, ff: int, device="cpu", dtype=torch.bfloat16) -> None:
        super().__init__()
        self.w_up = _param((ff, hidden), device, dtype, 1.0 / math.sqrt(hidden))
        self.w_down = _param((hidden, ff), device, dtype, 1.0 / math.sqrt(ff))
        self.set_act(0.0, 0.0)

    def set_act(self, p: float, q: float) -> None:
        """The activation's two learnable scalars enter through softplus."""
        self.a_pos = softplus64(float(p))
        self.a_neg = 0.5 + softplus64(float(q))

    def load(self, get, prefix: str) -> None:
        with torch.no_grad():
            self.w_up.copy_(get(prefix + "up"))
            self.w_down.copy_(get(prefix + "down"))
        act = get(prefix + "act").float().cpu().tolist()
        self.set_act(act[0], act[1])

    def forward(self, h):
        return F.linear(ops.xielu(F.linear(h, self.w_up), self.a_pos, self.a_neg), self.w_down)
