"""The mechanisms Lopovik added to the ops layer, each alone, against the slow
float64 functions in lopovik_oracle.py: CPU execution path and (marked gpu)
the HIP kernels in fp32 and bf16 storage.  Inputs are constructed where
random ones would hide a fault: one dominating key far back, at a page
border, at the query's own position and one past the causal edge; a sink
that dominates or vanishes; stale state in a reused slot.
"""

import math

import pytest
import torch

from llm_instance_gateway_amd import ops
from llm_instance_gateway_amd.models.hybrid_blocks import ScoredExpertsMLP

import lopovik_oracle as O

DEVICES = ["cpu", pytest.param("cuda:0", marks=pytest.mark.gpu)]
DTYPES = [torch.float32, torch.bfloat16]
F64 = torch.float64


def skip_cpu_bf16(device, dtype):
    if device == "cpu" and dtype == torch.bfloat16:
        pytest.skip("bf16 is the GPU serving precision")


def close(got, want, dtype, scale=None, tol32=2e-5):
    want = want.to(F64)
    s = scale if scale is not None else max(want.abs().max().item(), 1e-6)
    e = (got.detach().double().cpu() - want).abs().max().item() / s
    assert e < (tol32 if dtype == torch.float32 else 2e-2), e


def i32(v, device):
    return torch.tensor(v, dtype=torch.int32, device=device)


# -- norms with token shift ----------------------------------------------------

@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H", [20, 257, 1028, 2560, 5000])  # scalar and 4-wide paths, 1..8 vectors per thread
@pytest.mark.parametrize("adds", [0, 1, 2])
def test_offset_norm_shift_over_portions(device, dtype, H, adds):
    """Two sequences fed in portions of 1, 2 and more tokens through reused
    slots; the blended rows equal the whole-sequence computation.  With
    `adds` the rows arrive as a residual plus one or two branch outputs that
    the kernel adds on its way in."""
    skip_cpu_bf16(device, dtype)
    g = torch.Generator().manual_seed(H)
    eps = 1e-4
    w1 = (0.3 * torch.randn(H, generator=g)).to(dtype)
    w2 = (0.3 * torch.randn(H, generator=g)).to(dtype)
    mu = torch.rand(H, generator=g).to(dtype)
    xa, xb = 3 * torch.randn(11, H, generator=g), torch.randn(7, H, generator=g)
    want = {}
    for k, x in (("a", xa), ("b", xb)):
        h = O.offset_norm(x.to(F64), w1.to(F64), eps)
        want[k] = (O.token_shift(h, mu.to(F64)), O.offset_norm(x.to(F64), w2.to(F64), eps))
    state = torch.full((3, H), 7.0, device=device)  # stale values everywhere
    # steps: [(seq, slot, rows)], b starts later in a's old neighbourhood
    plan = [[("a", 1, 0, 4)], [("a", 1, 4, 5), ("b", 0, 0, 2)], [("a", 1, 5, 7), ("b", 0, 2, 3)],
            [("b", 0, 3, 7), ("a", 1, 7, 11)]]
    xs = {"a": xa, "b": xb}
    for step in plan:
        rows, tok_seq, s0, sl, slot, fresh = [], [], [], [], [], []
        for si, (k, sslot, lo, hi) in enumerate(step):
            s0.append(len(tok_seq))
            sl.append(hi - lo)
            slot.append(sslot)
            fresh.append(1 if lo == 0 else 0)
            tok_seq += [si] * (hi - lo)
            rows.append(xs[k][lo:hi])
        tok_seq.append(-1)  # a padding row
        rows.append(torch.randn(1, H, generator=g))
        x = torch.cat(rows).to(device)
        extra = []
        if adds:
            extra = [torch.randn(x.shape, generator=g).to(dtype).to(device) for _ in range(adds)]
            x_eff, before = x, None
            x = x_eff - sum(t.float() for t in extra)
            before = x.clone()
        hm, hf, x_new = ops.offset_norm_shift(
            x, w1.to(device), w2.to(device), mu.to(device), state, i32(tok_seq, device),
            i32(s0, device), i32(sl, device), i32(slot, device), i32(fresh, device), eps, *extra,
        )
        if adds:
            assert torch.equal(x, before), "the incoming residual is left as it was"
            n_live = len(tok_seq) - 1
            close(x_new[:n_live], x_eff[:n_live].double().cpu(), torch.float32)
        else:
            assert x_new is x
        assert hm.dtype == dtype and hf.dtype == dtype
        at = 0
        for k, _, lo, hi in step:
            close(hm[at : at + hi - lo], want[k][0][lo:hi], dtype, scale=want[k][0].abs().max().item())
            close(hf[at : at + hi - lo], want[k][1][lo:hi], dtype, scale=want[k][1].abs().max().item())
            at += hi - lo
        assert float(hm[at].abs().max()) == 0.0 and float(hf[at].abs().max()) == 0.0
    assert float((state[2] - 7.0).abs().max()) == 0.0, "an unused slot is left alone"


@pytest.mark.parametrize("device", DEVICES)
def test_offset_norm_without_feed_forward_branch(device):
    g = torch.Generator().manual_seed(3)
    H = 12
    x = torch.randn(5, H, generator=g).to(device)
    w1, mu = torch.randn(H, generator=g).to(device), torch.rand(H, generator=g).to(device)
    state = torch.zeros(1, H, device=device)
    hm, hf, _ = ops.offset_norm_shift(
        x, w1, None, mu, state, i32([0] * 5, device), i32([0], device), i32([5], device),
        i32([0], device), i32([1], device), 1e-5,
    )
    assert hf is None
    want = O.token_shift(O.offset_norm(x.double().cpu(), w1.double().cpu(), 1e-5), mu.double().cpu())
    close(hm, want, torch.float32)
    close(state[0], O.offset_norm(x.double().cpu(), w1.double().cpu(), 1e-5)[-1], torch.float32)
    close(ops.offset_rms_norm(x, w1, 1e-5), O.offset_norm(x.double().cpu(), w1.double().cpu(), 1e-5), torch.float32)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n", [7 * 9, 8 * 12])
def test_residual_add_and_activations(device, dtype, n):
    skip_cpu_bf16(device, dtype)
    g = torch.Generator().manual_seed(n)
    rows, H = (7, 9) if n == 63 else (8, 12)
    x = torch.randn(rows, H, generator=g)
    a = torch.randn(rows, H, generator=g).to(dtype)
    b = torch.randn(rows, H, generator=g).to(dtype)
    x1 = ops.residual_add(x.clone().to(device), a.to(device), b.to(device))
    assert x1.dtype == torch.float32
    close(x1, x.double() + a.double() + b.double(), torch.float32)
    x2 = ops.residual_add(x.clone().to(device), a.to(device))
    close(x2, x.double() + a.double(), torch.float32)
    z = (2 * torch.randn(rows, H, generator=g)).to(dtype)
    close(ops.relu_squared(z.to(device)), torch.relu(z.double()) ** 2, dtype)
    gu = torch.randn(rows, 2 * H, generator=g).to(dtype)
    gd, ud = gu[:, :H].double(), gu[:, H:].double()
    close(ops.silu_mul(gu.to(device)), gd * torch.sigmoid(gd) * ud, dtype)
    idx = torch.tensor([3, -1, 0, 3, rows - 1], dtype=torch.int64)
    w = torch.tensor([0.5, 9.0, 1.0, 0.25, 0.0])
    want = z.double()[idx.clamp(min=0)] * (w.double() * (idx >= 0))[:, None]
    close(ops.scale_gather_rows(z.to(device), idx.to(device), w.to(device)), want, dtype)


# -- latent prep and query rotation ----------------------------------------------

@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("sizes", [(10, 6, 4, 4), (24, 16, 8, 4), (5, 3, 2, 0), (300, 260, 6, 6), (1544, 72, 16, 16)])
def test_latent_prep_writes_normed_latent_and_rotated_key(device, dtype, sizes):
    skip_cpu_bf16(device, dtype)
    q_rank, kv_rank, rot_dim, rot_dims = sizes
    g = torch.Generator().manual_seed(sum(sizes))
    R, bs, nblk, eps, base = 6, 4, 5, 1e-5, 300.0
    # columns after the three parts (an output gate in the model); rows stay
    # 16-byte aligned when every size is a multiple of 8 (the wave-per-row path)
    extra = 8 if all(v % 8 == 0 for v in sizes) else 7
    proj = torch.randn(R, q_rank + kv_rank + rot_dim + extra, generator=g).to(dtype)
    wq = (1 + 0.2 * torch.randn(q_rank, generator=g)).to(dtype)
    wkv = (1 + 0.2 * torch.randn(kv_rank, generator=g)).to(dtype)
    pos = torch.tensor([0, 1, 2, 977, 15, 16], dtype=torch.int64)
    slots = torch.tensor([4, 5, 19, 0, 11, -1], dtype=torch.int64)  # the last row is not cached
    cache = torch.full((nblk, 1, bs, kv_rank + rot_dim), 5.0, dtype=dtype, device=device)
    inv = ops.rotary_inv_freq(base, rot_dims, device)
    cq = ops.latent_kv_prep(
        proj.to(device), q_rank, kv_rank, rot_dim, wq.to(device), wkv.to(device), eps, inv,
        pos.to(device), slots.to(device), cache,
    )
    pd = proj.double()
    close(cq, O.plain_norm(pd[:, :q_rank], wq.double(), eps), dtype)
    c = O.plain_norm(pd[:, q_rank : q_rank + kv_rank], wkv.double(), eps)
    kr = pd[:, q_rank + kv_rank : q_rank + kv_rank + rot_dim]
    if rot_dims:
        kr = O.rotate_interleaved(kr, pos, base, rot_dims)
    flat = cache.view(-1, kv_rank + rot_dim)
    for r in range(R - 1):
        close(flat[slots[r]], torch.cat([c[r], kr[r]]), dtype, scale=4.0)
    untouched = [s for s in range(nblk * bs) if s not in slots.tolist()]
    assert float((flat[untouched].float() - 5.0).abs().max()) == 0.0


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(6, 8, 6, 10), (8, 16, 16, 24), (16, 24, 10, 8)])
def test_rotate_pack_queries(device, dtype, shape):
    skip_cpu_bf16(device, dtype)
    g = torch.Generator().manual_seed(5)
    D, Rr, dims, lead = shape
    R, H, base = 5, 3, 1000.0
    q = torch.randn(R, H * (D + Rr), generator=g).to(dtype)
    pos = torch.tensor([0, 3, 64, 1500, 7], dtype=torch.int64)
    out = torch.zeros(R, H, lead + Rr, dtype=dtype, device=device)
    ops.rotate_pack_queries(q.to(device), H, D, Rr, ops.rotary_inv_freq(base, dims, device), pos.to(device), out, lead)
    want = O.rotate_interleaved(q.double().view(R, H, D + Rr)[..., D:], pos, base, dims)
    # angles are fp32 products: at position 1500 their rounding alone is 1e-4 rad
    close(out[..., lead:], want, dtype, tol32=2e-4)
    assert float(out[..., :lead].abs().max()) == 0.0
    # the last rot_dim - dims entries pass unchanged
    assert torch.equal(out[..., lead + dims :].cpu(), q.view(R, H, D + Rr)[..., D + dims :])


# -- softmax with a sink over a latent cache --------------------------------------

def paged(keys, bs, device, dtype, seed=0):
    """Scatter keys [L, D] of one sequence over shuffled pages; returns the
    cache [blocks, 1, bs, D] and the block table."""
    L, D = keys.shape
    nb = (L + bs - 1) // bs
    perm = torch.randperm(nb + 2, generator=torch.Generator().manual_seed(seed))[:nb]
    cache = torch.randn(nb + 2, 1, bs, D, generator=torch.Generator().manual_seed(seed + 1)).to(dtype)
    for j in range(L):
        cache[perm[j // bs], 0, j % bs] = keys[j].to(dtype)
    return cache.to(device), perm.to(torch.int32)


def run_general(q, cache, Dv, table, positions, scale, H, sink, device):
    R = q.shape[0]
    return ops.paged_attention_general(
        q.to(device), cache, cache[..., :Dv], table[None].contiguous().to(device),
        i32([0] * R, device), positions.to(device), scale, H, sink=None if sink is None else sink.to(device),
    )


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("D,Dv,bs", [(24, 16, 16), (10, 7, 8), (80, 64, 16)])
def test_sink_softmax_random(device, dtype, D, Dv, bs):
    """Values are the leading Dv entries of the key rows; prompt rows and a
    late single token in one launch."""
    skip_cpu_bf16(device, dtype)
    g = torch.Generator().manual_seed(D)
    L, H, scale = 150, 3, 0.4
    keys = torch.randn(L, D, generator=g).to(dtype)
    pos = torch.tensor([0, 1, bs - 1, bs, 63, 64, 65, L - 1], dtype=torch.int64)
    q = torch.randn(len(pos), H * D, generator=g).to(dtype)
    sink = torch.tensor([-1.0, 0.7, 3.0])
    cache, table = paged(keys, bs, device, dtype)
    got = run_general(q, cache, Dv, table, pos, scale, H, sink, device)
    kd = keys.double()
    for r, p in enumerate(pos.tolist()):
        n = p + 1
        qf = q[r].double().view(1, H, D).expand(n, H, D).clone()
        k = kd[:n, None, :].expand(n, H, D)
        want = O.sink_softmax_attention(qf, k, k[..., :Dv], scale, sink.double())[-1]
        close(got[r].view(H, Dv), want, dtype, scale=1.0)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("where", ["far", "page_edge", "own", "past_edge"])
def test_sink_softmax_one_key_stands_out(device, where):
    """One key scores far above the rest: the output is that key's value
    row (scaled by what the sink leaves) when the key is visible, wherever it
    lies, and unaffected when it is one past the query's position."""
    D, Dv, bs, L, H = 16, 12, 16, 400, 2
    g = torch.Generator().manual_seed(9)
    keys = 0.1 * torch.randn(L, D, generator=g)
    p = 350
    j = {"far": 3, "page_edge": 16 * 7, "own": p, "past_edge": p + 1}[where]
    keys[j] = 0.0
    keys[j, 0] = 6.0
    keys[j, 1:Dv] = torch.arange(1, Dv).float()
    q = torch.zeros(1, H * D)
    q[0, 0] = q[0, D] = 5.0  # score 30 on key j
    sink = torch.tensor([0.0, 30.0])
    cache, table = paged(keys, bs, device, torch.float32, seed=4)
    got = run_general(q, cache, Dv, table, torch.tensor([p]), 1.0, H, sink, device).view(H, Dv).cpu()
    if where == "past_edge":
        assert got[:, 1:].abs().max() < 1.0, "a key after the query's position leaked"
    else:
        assert abs(float(got[0, 5]) - 5.0) < 1e-3          # sink negligible: the key's value
        assert abs(float(got[1, 5]) - 2.5) < 1e-2          # sink as large as the key: half of it
    n = p + 1
    qf = q.double().view(1, H, D).expand(n, H, D).clone()
    k = keys.double()[:n, None, :].expand(n, H, D)
    close(got, O.sink_softmax_attention(qf, k, k[..., :Dv], 1.0, sink.double())[-1], torch.float32, scale=5.0)


@pytest.mark.parametrize("device", DEVICES)
def test_sink_extremes(device):
    """A huge sink silences the head; a very negative one leaves an ordinary
    softmax; the first token of a sequence sees itself and the sink only."""
    D, Dv, H = 8, 8, 3
    g = torch.Generator().manual_seed(2)
    keys = torch.randn(40, D, generator=g)
    q = torch.randn(2, H * D, generator=g)
    cache, table = paged(keys, 8, device, torch.float32)
    sink = torch.tensor([80.0, -80.0, 0.0])
    pos = torch.tensor([0, 39])
    got = run_general(q, cache, Dv, table, pos, 0.5, H, sink, device).view(2, H, Dv).cpu()
    plain = run_general(q, cache, Dv, table, pos, 0.5, H, None, device).view(2, H, Dv).cpu()
    assert got[:, 0].abs().max() < 1e-6
    assert (got[:, 1] - plain[:, 1]).abs().max() < 1e-5
    s0 = float(q[0].view(H, D)[2] @ keys[0]) * 0.5
    w = math.exp(s0) / (math.exp(s0) + 1.0)
    assert (got[0, 2] - w * keys[0, :Dv]).abs().max() < 1e-5


@pytest.mark.gpu
@pytest.mark.parametrize("row,Dv,bs", [(80, 64, 16), (128, 96, 16), (40, 24, 8), (72, 64, 32)])
def test_tiled_prefill_with_sink_over_latent_rows(row, Dv, bs):
    """MFMA prompt kernel: three sequences per launch (a fresh prompt, a
    portion continuing a long context, a two-token portion), values read from
    the key rows, sink in the denominator; a dominating key at a tile border."""
    dev, dtype = "cuda:0", torch.bfloat16
    assert ops.tiled_prefill_supported(dtype, row, Dv, True)
    g = torch.Generator().manual_seed(row)
    H, scale = 5, 0.3
    lens, news = [130, 333, 70], [130, 97, 2]
    nblk = sum((L + bs - 1) // bs for L in lens) + 1
    cache = torch.zeros(nblk, 1, bs, row, dtype=dtype)
    tables, keys, at = [], [], 1
    for L in lens:
        k = torch.randn(L, row, generator=g)
        k[64] *= 3.0  # one loud key at a 64-key border
        nb = (L + bs - 1) // bs
        ids = list(range(at, at + nb))
        at += nb
        for j in range(L):
            cache[ids[j // bs], 0, j % bs] = k[j].to(dtype)
        tables.append(ids)
        keys.append(k.to(dtype).double())
    mb = max(len(t) for t in tables)
    bt = torch.zeros(len(lens), mb, dtype=torch.int32)
    for i, t in enumerate(tables):
        bt[i, : len(t)] = torch.tensor(t)
    qsl = [0]
    for n in news:
        qsl.append(qsl[-1] + n)
    q = torch.randn(qsl[-1], H * row, generator=g).to(dtype)
    sink = torch.tensor([0.0, 2.0, -3.0, 5.0, 1.0])
    ts, tq = [], []
    for s, n in enumerate(news):
        for qb in range(0, n, 64):
            ts.append(s)
            tq.append(qb)
    cache = cache.to(dev)
    got = ops.paged_attention_prefill_tiles(
        q.to(dev), cache, cache[..., :Dv], bt.to(dev), i32(qsl, dev), i32(lens, dev), i32(ts, dev),
        i32(tq, dev), scale, H, sink=sink.to(dev),
    ).cpu()
    for s, (L, n) in enumerate(zip(lens, news)):
        for r in (0, 1, n // 2, n - 1):
            p = L - n + r
            qf = q[qsl[s] + r].double().view(1, H, row).expand(p + 1, H, row).clone()
            k = keys[s][: p + 1, None, :].expand(p + 1, H, row)
            want = O.sink_softmax_attention(qf, k, k[..., :Dv], scale, sink.double())[-1]
            close(got[qsl[s] + r].view(H, Dv), want, dtype, scale=1.0)


# -- routed experts -----------------------------------------------------------------

class _Meta:
    def __init__(self, num_prefill_tokens):
        self.num_prefill_tokens = num_prefill_tokens


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("E,top", [(5, 2), (1, 1), (4, 4), (7, 1)])
def test_scored_experts(device, dtype, E, top):
    """Sigmoid scores, unnormalised, scaling the expert INPUT: both dispatch
    paths (capacity-padded for steps with prompt rows, dense for single
    tokens) against the per-token loop."""
    skip_cpu_bf16(device, dtype)
    g = torch.Generator().manual_seed(E * 10 + top)
    T, H, ff = 9, 16, 12
    W = {"router": torch.randn(E, H, generator=g).to(torch.bfloat16)}
    for e in range(E):
        W[f"e{e}.gate"] = (torch.randn(ff, H, generator=g) * H ** -0.5).to(torch.bfloat16)
        W[f"e{e}.up"] = (torch.randn(ff, H, generator=g) * H ** -0.5).to(torch.bfloat16)
        W[f"e{e}.down"] = (torch.randn(H, ff, generator=g) * ff ** -0.5).to(torch.bfloat16)
    blk = ScoredExpertsMLP(H, ff, E, top, device=device, dtype=dtype)
    blk.load(lambda name: W[name].to(device=device, dtype=dtype), "")
    h = torch.randn(T, H, generator=g).to(dtype)
    want = O.moe_ff(h.double(), {k: v.double() for k, v in W.items()}, "", {"router": {"experts": E, "top": top}})
    for meta in (_Meta(T), _Meta(0), None):
        got = blk(h.to(device), meta)
        close(got, want, dtype)
    # scaling the input is not scaling the output: the experts are not linear
    s = torch.sigmoid(h.double() @ W["router"].double().T)
    if E == 1:
        x = h.double()
        gt, up = x @ W["e0.gate"].double().T, x @ W["e0.up"].double().T
        out_scaled = s * ((gt * torch.sigmoid(gt) * up) @ W["e0.down"].double().T)
        assert (out_scaled - want).abs().max() > 1e-3


@pytest.mark.gpu
@pytest.mark.parametrize("nsplit", [1, 3, 8])
@pytest.mark.parametrize("row,Dv,H,bs", [(80, 64, 6, 16), (576, 512, 16, 16), (136, 128, 3, 8), (40, 24, 70, 16), (320, 256, 5, 32)])
def test_latent_rows_kernel(row, Dv, H, bs, nsplit):
    """MFMA multi-query kernel, (token, head) row tiles: in one launch a
    fresh prompt, a portion continuing a long context, a two-token portion
    and two single tokens (one of them a sequence's first); values are the
    leading entries of the key rows; sink in the denominator; a loud key at a
    64-key border; head counts that do not divide the 64-row tile.  With
    nsplit > 1 the visible keys of a tile are cut into slices merged by a
    second kernel (slices of a one-key context are empty but for the first)."""
    dev, dtype = "cuda:0", torch.bfloat16
    assert ops.latent_rows_supported(dtype, row, Dv, True)
    g = torch.Generator().manual_seed(row + H)
    scale = 1.0 / math.sqrt(row)
    lens, news = [70, 333, 50, 129, 1], [70, 97, 2, 1, 1]
    nblk = sum((L + bs - 1) // bs for L in lens) + 1
    cache = torch.zeros(nblk, 1, bs, row, dtype=dtype)
    tables, keys, at = [], [], 1
    for L in lens:
        k = torch.randn(L, row, generator=g)
        if L > 64:
            k[64] *= 2.0
        nb = (L + bs - 1) // bs
        ids = list(range(at, at + nb))[::-1]
        at += nb
        for j in range(L):
            cache[ids[j // bs], 0, j % bs] = k[j].to(dtype)
        tables.append(ids)
        keys.append(k.to(dtype).double())
    mb = max(len(t) for t in tables)
    bt = torch.zeros(len(lens), mb, dtype=torch.int32)
    for i, t in enumerate(tables):
        bt[i, : len(t)] = torch.tensor(t)
    starts = [0]
    for n in news:
        starts.append(starts[-1] + n)
    R = starts[-1] + 3  # three rows of no segment at the end
    q = torch.randn(R, H * row, generator=g).to(dtype)
    sink = torch.randn(H, generator=g) * 2
    out = torch.full((R, H * Dv), 9.0, dtype=dtype, device=dev)
    ops.latent_attention_rows(
        q.to(dev), cache.to(dev), Dv, bt.to(dev), i32(starts[:-1], dev), i32(news, dev), i32(lens, dev),
        max(news), scale, H, sink=sink.to(dev), out=out, nsplit=nsplit,
    )
    got = out.cpu()
    assert float((got[starts[-1]:].float() - 9.0).abs().max()) == 0.0, "rows of no segment are left alone"
    for s, (L, n) in enumerate(zip(lens, news)):
        for r in sorted({0, 1 % n, n // 2, n - 1}):
            p = L - n + r
            qf = q[starts[s] + r].double().view(1, H, row).expand(p + 1, H, row).clone()
            k = keys[s][: p + 1, None, :].expand(p + 1, H, row)
            want = O.sink_softmax_attention(qf, k, k[..., :Dv], scale, sink.double())[-1]
            close(got[starts[s] + r].view(H, Dv), want, dtype, scale=1.0)
