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


def _mm(a: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    return F.linear(a, w)


class LatentAttention(nn.Module):
    """Attention whose keys and values are up-projections of one low-rank
    latent per token; only the normalised latent and one rotated key part
    shared by all heads are cached (one paged row of kv_rank + rot_dim
    entries).

    Per head a query has `dim` unrotated and `rot_dim` rotated entries; the
    score is (q_un . W_uk c + q_rot . k_rot) * scale.  The up-projections are
    absorbed so that attention runs in latent space as multi-query attention
    over the cache rows themselves:

        q_lat = W_uk^T q_un        (batched GEMM, per head)
        score = ([q_lat | q_rot] . [c | k_rot]) * scale
        o_lat = sum_j p_j c_j      (values = the leading kv_rank entries of the key rows)
        o     = W_uv o_lat         (batched GEMM, per head)

    which is exact because a softmax with a sink is still linear in the
    values.  Optional per-head sink in the softmax denominator, optional
    sigmoid output gate on the concatenated heads.  Rotation is interleaved
    pairs over the first `rot_dims` entries of the rotated part.
    """

    def __init__(
        self, hidden: int, heads: int, dim: int, rot_dim: int, vdim: int, q_rank: int,
        kv_rank: int, scale: float, rot_base: float, rot_dims: int, eps: float,
        sink: bool = True, out_gate: bool = True, device="cpu", dtype=torch.bfloat16,
    ) -> None:
        super().__init__()
        assert 0 <= rot_dims <= rot_dim and rot_dims % 2 == 0
        self.heads, self.dim, self.rot_dim, self.vdim = heads, dim, rot_dim, vdim
        self.q_rank, self.kv_rank = q_rank, kv_rank
        self.scale, self.eps = float(scale), float(eps)
        self.out_gate = out_gate
        self.row = kv_rank + rot_dim  # one cache row
        s = 1.0 / math.sqrt(hidden)
        self.n_in = q_rank + kv_rank + rot_dim
        self.ng = heads * vdim if out_gate else 0
        # rows: query latent | key/value latent | shared rotated key part | gate
        self.w_in = _param((self.n_in + self.ng, hidden), device, dtype, s)
        self.q_norm = _param((q_rank,), device, dtype, None)
        self.kv_norm = _param((kv_rank,), device, dtype, None)
        with torch.no_grad():
            self.q_norm.fill_(1.0)
            self.kv_norm.fill_(1.0)
        self.w_uq = _param((heads * (dim + rot_dim), q_rank), device, dtype, 1.0 / math.sqrt(q_rank))
        # per head, laid out for batched GEMMs: [H, dim, kv_rank] and [H, kv_rank, vdim]
        self.w_uk = _param((heads, dim, kv_rank), device, dtype, 1.0 / math.sqrt(kv_rank))
        self.w_uv = _param((heads, kv_rank, vdim), device, dtype, 1.0 / math.sqrt(kv_rank))
        self.sink = (
            nn.Parameter(torch.zeros(heads, device=device, dtype=torch.float32), requires_grad=False)
            if sink else None
        )
        self.w_o = _param((hidden, heads * vdim), device, dtype, 1.0 / math.sqrt(heads * vdim))
        self.register_buffer(
            "inv_freq", ops.rotary_inv_freq(rot_base, rot_dims, device), persistent=False
        )

    def cache_spec(self) -> dict:
        return {"kind": "latent", "row": self.row}

    def load(self, get, prefix: str) -> None:
        H, D, R = self.heads, self.dim, self.kv_rank
        parts = [get(prefix + "dq"), get(prefix + "dkv")]
        if self.out_gate:
            parts.append(get(prefix + "g"))
        with torch.no_grad():
            self.w_in.copy_(torch.cat(parts, dim=0))
            self.q_norm.copy_(get(prefix + "dq.norm"))
            self.kv_norm.copy_(get(prefix + "dkv.norm"))
            self.w_uq.copy_(get(prefix + "uq"))
            self.w_uk.copy_(get(prefix + "uk").view(H, D, R))
            self.w_uv.copy_(get(prefix + "uv").view(H, self.vdim, R).transpose(1, 2))
            if self.sink is not None:
                self.sink.copy_(get(prefix + "sink").float())
            self.w_o.copy_(get(prefix + "o"))

    def mfma_rows(self, dtype, on_gpu: bool) -> bool:
        return ops.latent_rows_supported(dtype, self.row, self.kv_rank, on_gpu)


    def forward(self, h, positions, cache, meta):
        lat_cache = cache[0]
        H, D, Rr, Rk = self.heads, self.dim, self.rot_dim, self.kv_rank
        rows = h.shape[0]
        proj = _mm(h, self.w_in)
        cq = ops.latent_kv_prep(
            proj, self.q_rank, Rk, Rr, self.q_norm, self.kv_norm, self.eps, self.inv_freq,
            positions, meta.slot_mapping, lat_cache,
        )
        q = _mm(cq, self.w_uq)  # [rows, H*(D+Rr)]
        qa = torch.empty(rows, H, self.row, dtype=q.dtype, device=q.device)
        # latent-space query part: per head q_un @ W_uk, written in place
        torch.bmm(
            q.view(rows, H, D + Rr)[:, :, :D].transpose(0, 1), self.w_uk,
            out=qa[:, :, :Rk].transpose(0, 1),
        )
        ops.rotate_pack_queries(q, H, D, Rr, self.inv_freq, positions, qa, Rk)
        qa = qa.view(rows, H * self.row)
        v_view = lat_cache[..., :Rk]
        np_ = meta.num_prefill_tokens
        if self.mfma_rows(q.dtype, q.is_cuda) and meta.seg_ctx is not None:
            # every row of the step in one launch: (token, head) row tiles
            # that share each key tile across the heads
            covered = np_ + meta.num_decode_tokens
            o = (torch.zeros if covered < rows else torch.empty)(
                rows, H * Rk, dtype=q.dtype, device=q.device
            )
            ops.latent_attention_rows(
                qa, lat_cache, Rk, meta.seq_block_tables, meta.seg_start, meta.seg_len,
                meta.seg_ctx, meta.max_seg_len, self.scale, H, sink=self.sink, out=o,
            )
        else:
            o = ops.paged_attention_general(
                qa, lat_cache, v_view, meta.seq_block_tables, meta.tok_seq, positions,
                self.scale, H, sink=self.sink,
            )
        # values: per head o_lat @ W_uv, heads concatenated in place
        ov = torch.empty(rows, H, self.vdim, dtype=q.dtype, device=q.device)
        torch.bmm(o.view(rows, H, Rk).transpose(0, 1), self.w_uv, out=ov.transpose(0, 1))
        ov = ov.view(rows, H * self.vdim)
        if self.out_gate:
            ops.sigmoid_gate_mul(ov, proj[:, self.n_in :])
        return _mm(ov, self.w_o)


class ReluSquaredMLP(nn.Module):
    """down(relu(up h)^2)."""

    def __init__(self, hidden: int, ff: int, device="cpu", dtype=torch.bfloat16) -> None:
        super().__init__()
        self.w_up = _param((ff, hidden), device, dtype, 1.0 / math.sqrt(hidden))
        self.w_down = _param((hidden, ff), device, dtype, 1.0 / math.sqrt(ff))

    def load(self, get, prefix: str) -> None:
        with torch.no_grad():
            self.w_up.copy_(get(prefix + "up"))
            self.w_down.copy_(get(prefix + "down"))

    def forward(self, h, meta=None):
        return _mm(ops.relu_squared(_mm(h, self.w_up)), self.w_down)


class ScoredExpertsMLP(nn.Module):
    """Routed gated-SiLU experts whose router scores are independent
    logistics: z = W_r h in fp32, s = sigmoid(z), the `top` largest scores
    pick the experts.  The chosen scores are used as they are (no
    renormalisation) and scale each expert's INPUT: out = sum_e expert_e(s_e h).

    Dispatch: (token, expert) pairs sorted by expert into a capacity-padded
    [E, cap, hidden] batch, gathered and scaled in one kernel, then one
    batched GEMM pair over all experts.  Steps made of single tokens only use
    a dense dispatch (every expert sees every token, unchosen pairs scaled by
    zero, which a bias-free expert maps to exactly zero): static shapes and
    no host round trip, so the step can be replayed from a hipGraph.
    """

    def __init__(
        self, hidden: int, ff: int, experts: int, top: int, device="cpu", dtype=torch.bfloat16
    ) -> None:
        super().__init__()
        assert 1 <= top <= experts
        self.experts, self.top, self.ff = experts, top, ff
        # the router runs in fp32 whatever the activation dtype
        self.w_router = nn.Parameter(
            torch.empty(experts, hidden, device=device, dtype=torch.float32).uniform_(
                -1.0 / math.sqrt(hidden), 1.0 / math.sqrt(hidden)
            ),
            requires_grad=False,
        )
        # pre-transposed for bmm: [E, hidden, gate | up] and [E, ff, hidden]
        self.w13 = _param((experts, hidden, 2 * ff), device, dtype, 1.0 / math.sqrt(hidden))
        self.w2 = _param((experts, ff, hidden), device, dtype, 1.0 / math.sqrt(ff))

    def load(self, get, prefix: str) -> None:
        with torch.no_grad():
            self.w_router.copy_(get(prefix + "router").float())
            for e in range(self.experts):
                p = f"{prefix}e{e}."
                self.w13[e].copy_(torch.cat([get(p + "gate"), get(p + "up")], dim=0).t())
                self.w2[e].copy_(get(p + "down").t())

    def route(self, h: torch.Tensor):
        z = F.linear(h.float(), self.w_router)
        w, idx = torch.topk(torch.sigmoid(z), self.top, dim=-1)
        return w, idx  # fp32 [T, top], int64 [T, top]

    def forward(self, h, meta=None):
        T, hidden = h.shape
        E = self.experts
        w, idx = self.route(h)
        if meta is not None and meta.num_prefill_tokens == 0:
            wd = torch.zeros(T, E, dtype=torch.float32, device=h.device).scatter_(1, idx, w)
            src = torch.arange(T, device=h.device).repeat(E)
            xe = ops.scale_gather_rows(h, src, wd.t().contiguous().view(-1))  # [E*T, hidden]
            act = ops.silu_mul(torch.bmm(xe.view(E, T, hidden), self.w13).view(E * T, -1))
            ye = torch.bmm(act.view(E, T, self.ff), self.w2)
            return ye.float().sum(dim=0).to(h.dtype)
        flat_e = idx.reshape(-1)
        flat_t = torch.arange(T, device=h.device).unsqueeze(1).expand(T, self.top).reshape(-1)
        order = torch.argsort(flat_e, stable=True)
        se, stok, sw = flat_e[order], flat_t[order], w.reshape(-1)[order]
        counts = torch.bincount(se, minlength=E)
        cap = int(counts.max())  # one host round trip per block; such steps run eager
        starts = torch.cumsum(counts, 0) - counts
        pos_in_e = torch.arange(se.numel(), device=h.device) - starts.index_select(0, se)
        dest = se * cap + pos_in_e
        gather = torch.full((E * cap,), -1, dtype=torch.int64, device=h.device)
        gather.index_copy_(0, dest, stok)
        wpad = torch.zeros(E * cap, dtype=torch.float32, device=h.device)
        wpad.index_copy_(0, dest, sw)
        xe = ops.scale_gather_rows(h, gather, wpad)
        act = ops.silu_mul(torch.bmm(xe.view(E, cap, hidden), self.w13).view(E * cap, -1))
        ye = torch.bmm(act.view(E, cap, self.ff), self.w2).view(E * cap, hidden)
        # every token owns exactly `top` rows of ye: gather them back in pair
        # order and sum in fp32 (no atomics, the same order every time)
        back = torch.empty_like(dest)
        back[order] = dest
        return ye.index_select(0, back).view(T, self.top, hidden).float().sum(dim=1).to(h.dtype)
