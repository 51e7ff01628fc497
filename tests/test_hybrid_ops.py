"""The hybrid-model mechanisms one by one (ops layer: HIP kernels on the GPU,
the torch execution path on the CPU) against the float64 oracle functions.

Where random data would hide a fault the inputs are built so that it shows:
one key far back (or at a page / 64-key tile border, or just past the causal
edge) gets a score that dominates the softmax, stale state is left in reused
slots, the temperature is probed on both sides of each step of its floor.
"""

import math

import pytest
import torch

from llm_instance_gateway_amd import ops

from tikarax_oracle import (
    F64, o_attention, o_group_norm, o_mingru, o_query_temperature, o_xielu, o_softplus,
)

DEVICES = ["cpu", pytest.param("cuda:0", marks=pytest.mark.gpu)]
DTYPES = [torch.float32, torch.bfloat16]


def close(got, want, dtype, scale=None):
    s = scale if scale is not None else max(1.0, want.abs().max().item())
    e = (got.double().cpu() - want).abs().max().item() / s
    assert e < (2e-5 if dtype == torch.float32 else 1.5e-2), e


def rnd(*shape, seed=0, dtype=torch.float32, s=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * s).to(dtype)


# -- norms ---------------------------------------------------------------------

@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,groups", [(48, 3), (64, 1), (40, 4), (1536, 2), (6, 6)])
def test_group_norms(device, dtype, H, groups):
    eps, R, V = 1e-5, 5, 11
    table = rnd(V, H, seed=1, dtype=dtype, s=3.0)
    w = (1 + rnd(H, seed=2, s=0.3)).to(dtype)
    w2 = (1 + rnd(H, seed=3, s=0.3)).to(dtype)
    toks = torch.tensor([3, 0, 10, 3, 7])
    res = ops.embed_group_norm(toks.to(device), table.to(device), w.to(device), eps, groups)
    assert res.dtype == torch.float32
    want = o_group_norm(table.to(F64)[toks], w.to(F64), groups, eps)
    close(res, want, torch.float32)

    x = rnd(R, H, seed=4, s=5.0)
    h = ops.group_norm(x.to(device), w.to(device), eps, groups)
    assert h.dtype == dtype
    close(h, o_group_norm(x.to(F64), w.to(F64), groups, eps), dtype)

    y = rnd(R, H, seed=5, dtype=dtype, s=0.01)  # small y: eps matters inside the root
    xr = x.clone().to(device)
    h2 = ops.post_add_pre_norm(xr, y.to(device), w.to(device), w2.to(device), eps, groups)
    want_x = x.to(F64) + o_group_norm(y.to(F64), w.to(F64), groups, eps)
    close(xr, want_x, torch.float32)
    close(h2, o_group_norm(want_x, w2.to(F64), groups, eps), dtype)
    xr2 = x.clone().to(device)
    assert ops.post_add_pre_norm(xr2, y.to(device), w.to(device), None, eps, groups) is None
    close(xr2, want_x, torch.float32)


# -- activation ------------------------------------------------------------------

@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("p,q", [(0.0, 0.0), (-2.5, 1.75), (3.0, -4.0)])
def test_xielu(device, dtype, p, q):
    special = torch.tensor([-30.0, -3.0, -1.0, -1e-3, 0.0, 1e-3, 0.5, 4.0])
    z = torch.cat([special, rnd(120, seed=7, s=2.0)]).to(dtype).view(8, 16)
    got = ops.xielu(z.to(device), o_softplus(p), 0.5 + o_softplus(q))
    close(got, o_xielu(z.to(F64), p, q), dtype)


@pytest.mark.parametrize("device", DEVICES)
def test_sigmoid_gate_mul_strided(device):
    full = rnd(6, 50, seed=8).to(device)
    x = rnd(6, 20, seed=9).to(device)
    want = x.double().cpu() * torch.sigmoid(full[:, 30:].double().cpu())
    ops.sigmoid_gate_mul(x, full[:, 30:])
    close(x, want, torch.float32)


# -- minGRU ------------------------------------------------------------------------

def _segs(device, start, length, slot, fresh):
    t = lambda v: torch.tensor(v, dtype=torch.int32, device=device)
    return t(start), t(length), t(slot), t(fresh)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("W", [1, 40, 130])
def test_mingru_segments_state_and_slot_reuse(device, dtype, W):
    lens = [1, 70 if W == 130 else 700, 9, 2]   # 700: the chunked three-pass scan on the GPU
    R = sum(lens) + 3                          # trailing rows belong to no segment
    zxg = rnd(R, 3 * W, seed=10, dtype=dtype, s=1.5)
    state = torch.full((6, W), 123.0)          # stale garbage in every slot
    carried = rnd(W, seed=11)
    state[4] = carried                         # segment 2 continues a sequence
    starts = [0, 1, 1 + lens[1], 1 + lens[1] + 9]
    slots, fresh = [5, 0, 4, 2], [1, 1, 0, 1]
    st_dev = state.clone().to(device)
    out = ops.mingru_scan(zxg.to(device), st_dev, *_segs(device, starts, lens, slots, fresh), max(lens))
    z64 = zxg.to(F64)
    for s0, n, slot, fr in zip(starts, lens, slots, fresh):
        init = torch.zeros(W, dtype=F64) if fr else carried.to(F64)
        S, last = o_mingru(z64[s0 : s0 + n, :W], z64[s0 : s0 + n, W : 2 * W], init)
        g = z64[s0 : s0 + n, 2 * W :]
        close(out[s0 : s0 + n], S * g * torch.sigmoid(g), dtype)
        close(st_dev[slot], last, torch.float32)
    assert torch.equal(st_dev[1].cpu(), state[1]) and torch.equal(st_dev[3].cpu(), state[3])


@pytest.mark.parametrize("device", DEVICES)
def test_mingru_prefill_equals_stepwise(device):
    W, T = 24, 50
    zxg = rnd(T, 3 * W, seed=12, s=2.0).to(device)
    st_a = torch.zeros(2, W, device=device)
    whole = ops.mingru_scan(zxg, st_a, *_segs(device, [0], [T], [1], [1]), T)
    st_b = torch.full((2, W), -7.0, device=device)
    rows = []
    for t, n in [(0, 1), (1, 1), (2, 2), (4, 13), (17, 1), (18, 32)]:
        rows.append(ops.mingru_scan(zxg[t : t + n].contiguous(), st_b, *_segs(device, [0], [n], [0], [int(t == 0)]), n))
    assert (torch.cat(rows) - whole).abs().max().item() < 1e-5
    assert (st_b[0] - st_a[1]).abs().max().item() < 1e-5


# -- attention -------------------------------------------------------------------------

def paged(device, dtype, k, v, G, bs, n_blocks, seed):
    """Scatter one sequence's K/V [L, G*D] into caches through a shuffled
    block table; returns (k_cache, v_cache, block_table row)."""
    L = k.shape[0]
    D, Dv = k.shape[1] // G, v.shape[1] // G
    g = torch.Generator().manual_seed(seed)
    perm = torch.randperm(n_blocks, generator=g)[: (L + bs - 1) // bs]
    kc = torch.full((n_blocks + 1, G, bs, D), 9.0, dtype=dtype, device=device)
    vc = torch.full((n_blocks + 1, G, bs, Dv), -9.0, dtype=dtype, device=device)
    pos = torch.arange(L)
    slots = (perm[pos // bs] * bs + pos % bs).to(torch.int64).to(device)
    fused = torch.cat([k, v], dim=1).to(dtype).to(device)  # K and V as column blocks of one buffer
    ops.kv_scatter(fused[:, : G * D], fused[:, G * D :], kc, vc, slots)
    return kc, vc, perm.to(torch.int32)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,D,Dv", [(4, 2, 8, 12), (3, 1, 24, 8), (2, 2, 80, 136), (1, 1, 5, 3)])
def test_attention_random_prompt_and_decode_rows(device, dtype, H, G, D, Dv):
    L, bs = 150, 16
    k, v = rnd(L, G * D, seed=20, s=0.7), rnd(L, G * Dv, seed=21)
    k, v = k.to(dtype).float(), v.to(dtype).float()
    kc, vc, bt = paged(device, dtype, k, v, G, bs, 14, seed=3)
    # rows: a portion of 40 (positions 90..129), then decode rows of the same
    # sequence state at the last position, plus one padding row
    pos = list(range(90, 130)) + [149]
    q = rnd(len(pos), H * D, seed=22).to(dtype)
    gate = rnd(len(pos), H * Dv, seed=23).to(dtype)
    fused = torch.cat([q, gate], dim=1).to(device)
    tables = torch.zeros(2, 12, dtype=torch.int32)
    tables[1, : bt.numel()] = bt
    tok_seq = torch.tensor([1] * len(pos) + [-1], dtype=torch.int32, device=device)
    positions = torch.tensor(pos + [0], dtype=torch.int64, device=device)
    fused = torch.cat([fused, torch.zeros(1, fused.shape[1], dtype=dtype, device=device)])
    scale, coef, every = 0.37, 0.8, 16
    out = ops.paged_attention_general(
        fused[:, : H * D], kc, vc, tables.to(device), tok_seq, positions, scale, H,
        gate=fused[:, H * D :], temp_coef=coef, temp_every=every,
    )
    assert out.shape == (len(pos) + 1, H * Dv) and out[-1].abs().max().item() == 0
    for i, p in enumerate(pos):
        want = o_attention(q[i : i + 1].to(F64), k[: p + 1].to(F64), v[: p + 1].to(F64), H, G, scale,
                           coef, every, gate=gate[i : i + 1].to(F64), start=p)
        close(out[i : i + 1], want, dtype)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("bs", [16, 8])
def test_attention_one_key_stands_out(device, bs):
    """For every probed key position j (far back, page and 64-key tile
    borders, the query's own position) the key gets a dominating score: the
    output must be that key's value row.  A dominating key one past the
    causal edge must leave no trace."""
    D, Dv, L = 16, 6, 900
    k = rnd(L, D, seed=30, s=0.05)
    v = rnd(L, Dv, seed=31)
    q = rnd(1, D, seed=32)
    q = q / q.norm()
    qpos = [0, 1, 15, 16, 17, 63, 64, 65, 127, 128, 500, 897]
    for p in qpos:                          # each query's future neighbour dominates if it leaks
        k[p + 1] = 60.0 * q[0]
    targets = {}
    rows_q, rows_p = [], []
    for p in qpos:
        for j in {0, p, max(p - 1, 0), max(p - 15, 0), max(p - 16, 0), max(p - 64, 0), max(p - 65, 0), p // 2}:
            rows_q.append((p, j))
    # one K copy per probed (p, j): the standout key is written per row via a separate sequence
    outs = []
    for p, j in rows_q:
        kk = k.clone()
        if j <= p and j not in [x + 1 for x in qpos if x + 1 <= p]:
            kk[j] = 40.0 * q[0]
        else:
            continue
        kc, vc, bt = paged(device, torch.float32, kk, v, 1, bs, (L + bs - 1) // bs + 3, seed=p + j)
        tables = bt.view(1, -1).contiguous().to(device)
        out = ops.paged_attention_general(
            q.to(device), kc, vc, tables, torch.zeros(1, dtype=torch.int32, device=device),
            torch.tensor([p], dtype=torch.int64, device=device), 1.0, 1,
        )
        visible_leak = [x + 1 for x in qpos if x + 1 <= p and x + 1 != j]
        if not visible_leak:                # no other dominating key inside the causal range
            assert (out.cpu() - v[j]).abs().max().item() < 1e-3, (p, j)
        want = o_attention(q.to(F64), kk[: p + 1].to(F64), v[: p + 1].to(F64), 1, 1, 1.0, start=p)
        close(out, want, torch.float32)
        outs.append(out)
    assert len(outs) > 40


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_attention_portion_rows_ignore_what_lies_past_them(device, dtype):
    """A 40-row prompt portion at positions 100..139 of a sequence whose pages
    still hold a dominating key at position 140 (left by an earlier, longer
    user of the page): every row must return the value of the one standout
    key far back (position 5), untouched by what lies past the portion."""
    D, Dv, L = 24, 10, 160
    k = rnd(L, D, seed=40, s=0.02)
    v = rnd(L, Dv, seed=41)
    q = rnd(1, D, seed=42)
    q = (q / q.norm()).to(dtype).float()
    k[5] = 30.0 * q[0]
    k[140] = 60.0 * q[0]
    kc, vc, bt = paged(device, dtype, k, v, 1, 16, 12, seed=9)
    pos = list(range(100, 140))
    R = len(pos)
    out = ops.paged_attention_general(
        q.repeat(R, 1).to(dtype).to(device), kc, vc, bt.view(1, -1).contiguous().to(device),
        torch.zeros(R, dtype=torch.int32, device=device),
        torch.tensor(pos, dtype=torch.int64, device=device), 1.0, 1,
    )
    v5 = v[5].to(dtype).double()
    assert (out.double().cpu() - v5).abs().max().item() < (1e-3 if dtype == torch.float32 else 3e-2)


@pytest.mark.parametrize("device", DEVICES)
def test_query_temperature_on_both_sides_of_each_step(device):
    """tau(p) = 1 + c ln(floor((p+1)/e) + 1) changes between p = m*e - 2 and
    m*e - 1; two keys with different scores make the output depend on it."""
    D, Dv, e, c = 4, 2, 6, 0.9
    L = 40
    k = torch.zeros(L, D)
    k[:, 0] = torch.arange(L) % 2 * 1.0      # alternating scores 0 / 1
    v = torch.zeros(L, Dv)
    v[:, 0] = torch.arange(L) % 2 * 1.0
    v[:, 1] = 1.0
    q = torch.zeros(1, D)
    q[0, 0] = 2.0
    kc, vc, bt = paged(device, torch.float32, k, v, 1, 8, 7, seed=1)
    pos = [0, 4, 5, 6, 10, 11, 12, 17, 18, 35]
    R = len(pos)
    out = ops.paged_attention_general(
        q.repeat(R, 1).to(device), kc, vc, bt.view(1, -1).to(device),
        torch.zeros(R, dtype=torch.int32, device=device),
        torch.tensor(pos, dtype=torch.int64, device=device), 1.0, 1, temp_coef=c, temp_every=e,
    )
    for i, p in enumerate(pos):
        want = o_attention(q.to(F64), k[: p + 1].to(F64), v[: p + 1].to(F64), 1, 1, 1.0, c, e, start=p)
        close(out[i : i + 1], want, torch.float32)
    assert abs(o_query_temperature(4, c, e) - 1.0) < 1e-12
    assert abs(o_query_temperature(5, c, e) - (1 + c * math.log(2))) < 1e-12
    # the step is visible in the outputs: p = 4 and p = 5 differ by more than rounding
    assert (out[1] - out[2]).abs().max().item() > 1e-2


@pytest.mark.gpu
@pytest.mark.parametrize("H,G,D,Dv", [(4, 2, 8, 16), (6, 1, 48, 32), (2, 2, 80, 128), (3, 1, 24, 8), (2, 1, 128, 40), (1, 1, 64, 64)])
@pytest.mark.parametrize("bs", [16, 8])
def test_tiled_prefill_kernel(H, G, D, Dv, bs):
    """MFMA prefill tiles for padded head sizes: three sequences in one launch
    — a 100-row portion ending at position 149 (two query tiles, the second
    partial, keys crossing 32-key tiles and pages), a fresh 5-token prompt, and
    a fresh prompt of exactly one tile — with temperature and gate, from
    strided q / gate views."""
    device, dtype = "cuda:0", torch.bfloat16
    assert ops.tiled_prefill_supported(dtype, D, Dv, True)
    ctxs, ns = [150, 5, 64], [100, 5, 64]
    nblk = sum((c + bs - 1) // bs for c in ctxs) + 2
    g = torch.Generator().manual_seed(H * 100 + D)
    perm = torch.randperm(nblk, generator=g).tolist()
    kc = torch.full((nblk, G, bs, D), 7.0, dtype=dtype, device=device)
    vc = torch.full((nblk, G, bs, Dv), -7.0, dtype=dtype, device=device)
    maxb = max((c + bs - 1) // bs for c in ctxs)
    tables = torch.zeros(len(ctxs), maxb, dtype=torch.int32)
    ks, vs, at = [], [], 0
    for s, c in enumerate(ctxs):
        nb = (c + bs - 1) // bs
        blocks = perm[at : at + nb]
        at += nb
        tables[s, :nb] = torch.tensor(blocks, dtype=torch.int32)
        k = rnd(c, G * D, seed=50 + s, s=0.6).to(dtype)
        v = rnd(c, G * Dv, seed=60 + s).to(dtype)
        pos = torch.arange(c)
        slots = (torch.tensor(blocks)[pos // bs] * bs + pos % bs).to(torch.int64).to(device)
        fused = torch.cat([k, v], dim=1).to(device)
        ops.kv_scatter(fused[:, : G * D], fused[:, G * D :], kc, vc, slots)
        ks.append(k.to(F64))
        vs.append(v.to(F64))
    Tp = sum(ns)
    q = rnd(Tp, H * D, seed=70).to(dtype)
    gate = rnd(Tp, H * Dv, seed=71).to(dtype)
    fused = torch.cat([q, torch.zeros(Tp, 8, dtype=dtype), gate], dim=1).to(device)
    qsl = [0]
    for n in ns:
        qsl.append(qsl[-1] + n)
    ts, tq = [], []
    for s, n in enumerate(ns):
        for q0 in range(0, n, 64):
            ts.append(s)
            tq.append(q0)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=device)
    scale, coef, every = 0.9 / math.sqrt(D), 0.7, 16
    out = ops.paged_attention_prefill_tiles(
        fused[:, : H * D], kc, vc, tables.to(device), i32(qsl), i32(ctxs), i32(ts), i32(tq),
        scale, H, gate=fused[:, H * D + 8 :], temp_coef=coef, temp_every=every,
    )
    for s, (c, n) in enumerate(zip(ctxs, ns)):
        rows = slice(qsl[s], qsl[s + 1])
        want = o_attention(q[rows].to(F64), ks[s], vs[s], H, G, scale, coef, every,
                           gate=gate[rows].to(F64), start=c - n)
        close(out[rows], want, dtype)
