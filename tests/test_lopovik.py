"""Lopovik through the engine (scheduler, block/state pools, model runner,
kernels) against the slow float64 oracle in lopovik_oracle.py.

Every test builds its own small configuration and random bf16 checkpoint in
a temp folder, so the config reader and the safetensors loader are on the
path too.  The CPU parametrisation runs the engine's torch execution path;
the `gpu` one runs the HIP kernels (fp32 storage for sharp comparisons, bf16
for the serving precision).
"""

import json
import math
import struct

import pytest
import torch

from llm_instance_gateway_amd.engine import EngineConfig, LLMEngine, SamplingParams
from llm_instance_gateway_amd.models.config import get_model_config

import lopovik_oracle as O

DEVICES = ["cpu", pytest.param("cuda:0", marks=pytest.mark.gpu)]
DTYPES = [torch.float32, torch.bfloat16]


def lat(heads, dim, rot_dim, vdim, q_rank, kv_rank, mlp=None, base=500.0, dims=None, scale=None):
    return {
        "type": "latent_attention",
        "mixer": {
            "heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank,
            "kv_rank": kv_rank, "rot": {"base": base, "dims": rot_dim if dims is None else dims},
            "scale": scale if scale is not None else 1.2 / math.sqrt(dim + rot_dim),
        },
        "mlp": mlp,
    }


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


# sizes unlike one another; a looped span of two layers run three times, a
# layer without feed-forward inside it, two experts per token
CFG_A = {
    "architecture": "Lopovik", "vocab": 61, "width": 48, "norm": {"eps": 1e-5},
    "layers": [
        lat(3, 8, 8, 12, 24, 16, dense(40)),
        lat(2, 16, 4, 8, 20, 24, moe(5, 2, 24)),
        lat(4, 6, 6, 10, 16, 12, None, dims=4),
        lat(3, 8, 8, 12, 24, 16, moe(3, 1, 16), base=20.0),
    ],
    "loop": {"start": 1, "stop": 3, "times": 3},
}
# degenerate values: one head, one expert, sizes that are no multiple of
# anything, no loop at all
CFG_B = {
    "architecture": "Lopovik", "vocab": 31, "width": 18, "norm": {"eps": 1e-3},
    "layers": [lat(1, 5, 2, 3, 7, 6, moe(1, 1, 5)), lat(2, 3, 4, 5, 9, 10, dense(7)), lat(1, 4, 2, 4, 4, 4, None)],
}
# a loop over ALL layers, run once: the re-mix happens before layer 0
CFG_L = {
    "architecture": "Lopovik", "vocab": 40, "width": 24, "norm": {"eps": 1e-5},
    "layers": [lat(2, 8, 4, 8, 12, 12, dense(16)), lat(2, 8, 4, 8, 12, 12, moe(4, 3, 8))],
    "loop": {"start": 0, "stop": 2, "times": 1},
}
# no routed layer anywhere: on the GPU the engine pads such batches to whole
# GEMM row multiples, so rows of no sequence travel through every kernel
CFG_D = {
    "architecture": "Lopovik", "vocab": 33, "width": 32, "norm": {"eps": 1e-5},
    "layers": [lat(2, 8, 8, 8, 16, 24, dense(24)), lat(3, 4, 4, 6, 8, 12, None), lat(2, 8, 8, 8, 16, 24, dense(40))],
    "loop": {"start": 1, "stop": 3, "times": 2},
}
# cache rows of three of the MFMA kernel's size classes (80, 128, 136 entries)
CFG_C = {
    "architecture": "Lopovik", "vocab": 40, "width": 64, "norm": {"eps": 1e-5},
    "layers": [lat(4, 32, 16, 32, 48, 64, dense(96)), lat(2, 64, 32, 64, 40, 96, moe(4, 2, 32)),
               lat(3, 16, 8, 16, 24, 128, None)],
    "loop": {"start": 0, "stop": 2, "times": 2},
}


def make_checkpoint(cfg, seed):
    g = torch.Generator().manual_seed(seed)
    H, V = cfg["width"], cfg["vocab"]

    def r(*shape, s=1.0):
        return (torch.randn(*shape, generator=g) * s).to(torch.bfloat16)

    W = {"embed": r(V, H), "final.norm": r(H, s=0.2)}
    if cfg.get("loop"):
        W["loop.in"] = r(H, 2 * H, s=(2 * H) ** -0.5 * 1.4)
    for i, layer in enumerate(cfg["layers"]):
        p = "l%d." % i
        m = layer["mixer"]
        Hh, D, R, Dv, Rq, Rk = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["q_rank"], m["kv_rank"]
        W[p + "norm1"], W[p + "shift"] = r(H, s=0.2), torch.rand(H, generator=g).to(torch.bfloat16)
        W[p + "mix.dq"], W[p + "mix.dq.norm"] = r(Rq, H, s=H ** -0.5), (1 + 0.2 * torch.randn(Rq, generator=g)).to(torch.bfloat16)
        W[p + "mix.uq"] = r(Hh * (D + R), Rq, s=Rq ** -0.5 * 2)
        W[p + "mix.dkv"], W[p + "mix.dkv.norm"] = r(Rk + R, H, s=H ** -0.5), (1 + 0.2 * torch.randn(Rk, generator=g)).to(torch.bfloat16)
        W[p + "mix.uk"] = r(Hh * D, Rk, s=Rk ** -0.5 * 2)
        W[p + "mix.uv"] = r(Hh * Dv, Rk, s=Rk ** -0.5)
        W[p + "mix.sink"] = r(Hh, s=1.5)
        W[p + "mix.g"] = r(Hh * Dv, H, s=H ** -0.5)
        W[p + "mix.o"] = r(H, Hh * Dv, s=(Hh * Dv) ** -0.5)
        mlp = layer["mlp"]
        if mlp is not None:
            W[p + "norm2"] = r(H, s=0.2)
            if mlp["kind"] == "dense":
                W[p + "mlp.up"], W[p + "mlp.down"] = r(mlp["ff"], H, s=H ** -0.5), r(H, mlp["ff"], s=mlp["ff"] ** -0.5)
            else:
                ff = mlp["expert"]["ff"]
                W[p + "mlp.router"] = r(mlp["router"]["experts"], H, s=2.0 * H ** -0.5)
                for e in range(mlp["router"]["experts"]):
                    W[f"{p}mlp.e{e}.gate"] = r(ff, H, s=H ** -0.5)
                    W[f"{p}mlp.e{e}.up"] = r(ff, H, s=H ** -0.5)
                    W[f"{p}mlp.e{e}.down"] = r(H, ff, s=ff ** -0.5)
    return W


def write_model(folder, cfg, W):
    folder.mkdir(parents=True, exist_ok=True)
    (folder / "config.json").write_text(json.dumps(cfg))
    header, blobs, at = {}, [], 0
    for name, t in W.items():
        raw = t.contiguous().view(torch.uint8).numpy().tobytes() if t.numel() else b""
        header[name] = {"dtype": "BF16", "shape": list(t.shape), "data_offsets": [at, at + len(raw)]}
        blobs.append(raw)
        at += len(raw)
    hj = json.dumps(header).encode()
    with open(folder / "model.safetensors", "wb") as f:
        f.write(struct.pack("<Q", len(hj)) + hj + b"".join(blobs))
    return str(folder)


def make_engine(path, device, dtype=torch.float32, blocks=64, block_size=16, seqs=4, budget=4096, **kw):
    mc = get_model_config(path)
    cfg = EngineConfig(
        model=mc, block_size=block_size, num_kv_blocks=blocks, max_num_seqs=seqs,
        num_state_slots=seqs, max_num_batched_tokens=budget,
        max_model_len=blocks * block_size, watermark_blocks=0, enforce_eager=True, **kw,
    )
    return LLMEngine(cfg, device=device, dtype=dtype)


def rel_err(got, want):
    """Per-row RMS of the mean-free difference over the RMS of the oracle's logits."""
    d = got.double().cpu() - want
    d = d - d.mean(-1, keepdim=True)
    return (d.pow(2).mean(-1).sqrt() / want.pow(2).mean().sqrt()).max().item()


def row_errs(got, want):
    d = got.double().cpu() - want
    d = d - d.mean(-1, keepdim=True)
    return d.pow(2).mean(-1).sqrt() / want.pow(2).mean().sqrt()


def tol(dtype):
    return 2e-4 if dtype == torch.float32 else 6e-2


def assert_logits(got, want, dtype):
    """fp32: every row within rounding.  bf16: a rounded router score can
    pick another expert for a token now and then (random routers have close
    calls), which moves that row and, through the token shift, the next; so
    nine rows in ten must be within the bf16 bound and the median well inside."""
    e = row_errs(got, want)
    if dtype == torch.float32:
        assert e.max().item() < tol(dtype), e.max().item()
    else:
        assert (e < tol(dtype)).double().mean().item() >= 0.9 and e.median().item() < 2e-2, e


def tokens_for(cfg, n, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, cfg["vocab"], (n,), generator=g).tolist()


def replay_all(eng, rid, toks, cuts):
    """Feed toks in portions `cuts`, wanting every position; returns [T, V]."""
    rows, at = [], 0
    for i, n in enumerate(cuts):
        last = i == len(cuts) - 1
        res = eng.replay_step([(rid, toks[at : at + n], list(range(n)))], end=[rid] if last else [])
        rows.append(res[rid].float().cpu())
        at += n
    assert at == len(toks)
    return torch.cat(rows)


def _model(tmp_path_factory, cfg, seed, name):
    W = make_checkpoint(cfg, seed)
    return write_model(tmp_path_factory.mktemp("lpv") / name, cfg, W), W


@pytest.fixture(scope="module")
def model_a(tmp_path_factory):
    return _model(tmp_path_factory, CFG_A, 11, "a")


@pytest.fixture(scope="module")
def model_b(tmp_path_factory):
    return _model(tmp_path_factory, CFG_B, 12, "b")


@pytest.fixture(scope="module")
def model_c(tmp_path_factory):
    return _model(tmp_path_factory, CFG_C, 13, "c")


@pytest.fixture(scope="module")
def oracle_a(model_a):
    toks = tokens_for(CFG_A, 90, 5)
    res = []
    return toks, O.forward(CFG_A, model_a[1], toks, residuals=res), res


def test_config_reader_and_run_order(model_a):
    mc = get_model_config(model_a[0])
    assert mc.architecture == "lopovik" and mc.layer_loop == (1, 3, 3)
    assert mc.layer_run_order() == [0, 1, 2, 1, 2, 1, 2, 3]
    assert [r["layer"] for r in O.layer_runs(CFG_A)] == mc.layer_run_order()
    # one cache row and one shift row per layer RUN
    assert mc.kv_elems_per_token() == (16 + 8) + 3 * ((24 + 4) + (12 + 6)) + (16 + 8)
    assert mc.state_elems_per_seq() == 8 * 48 and mc.has_recurrent_state and mc.is_moe


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_whole_prompt_and_every_layer_run(model_a, oracle_a, device, dtype):
    if device == "cpu" and dtype == torch.bfloat16:
        pytest.skip("bf16 is the GPU serving precision")
    toks, want, want_res = oracle_a
    eng = make_engine(model_a[0], device, dtype)
    captured = eng.runner.model.capture_residuals = []
    got = replay_all(eng, "w", toks, [len(toks)])
    assert_logits(got, want, dtype)
    assert len(captured) == 8  # the looped layers count each time
    for i, (x, xo) in enumerate(zip(captured, want_res)):
        assert x.dtype == torch.float32, "the residual stream stays fp32"
        e = (x[: len(toks)].double().cpu() - xo).abs().max(-1).values / xo.abs().max().item()
        if dtype == torch.float32:
            assert e.max().item() < 1e-4, f"layer run {i}: {e.max().item()}"
        else:
            assert (e < 4e-2).double().mean().item() >= 0.9, f"layer run {i}: {e}"


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("which", ["b", "l", "d"])
def test_degenerate_sizes_and_loops(model_b, tmp_path, device, which):
    if which == "b":
        cfg, (path, W) = CFG_B, model_b
    else:
        cfg = CFG_L if which == "l" else CFG_D
        W = make_checkpoint(cfg, 14)
        path = write_model(tmp_path / which, cfg, W)
    toks = tokens_for(cfg, 40, 6)
    want = O.forward(cfg, W, toks)
    eng = make_engine(path, device, block_size=8)
    assert get_model_config(path).is_moe == (which != "d")
    assert rel_err(replay_all(eng, "d", toks, [17, 1, 1, 2, 19]), want) < 2e-4
    if which == "d":  # bf16 with padded batches, two requests side by side
        eng = make_engine(path, device, torch.bfloat16 if device != "cpu" else torch.float32)
        t2 = tokens_for(cfg, 21, 7)
        r1 = eng.replay_step([("x", toks[:30], list(range(30))), ("y", t2[:20], list(range(20)))])
        r2 = eng.replay_step([("x", toks[30:], list(range(10))), ("y", t2[20:], [0])], end=["x", "y"])
        got_x = torch.cat([r1["x"], r2["x"]]).float().cpu()
        got_y = torch.cat([r1["y"], r2["y"]]).float().cpu()
        assert rel_err(got_x, want) < 6e-2 and rel_err(got_y, O.forward(cfg, W, t2)) < 6e-2


@pytest.mark.parametrize("device", DEVICES)
def test_first_token_alone(model_a, oracle_a, device):
    toks, want, _ = oracle_a
    eng = make_engine(model_a[0], device)
    assert rel_err(replay_all(eng, "f", toks[:1], [1]), want[:1]) < 2e-4


@pytest.mark.parametrize("device", DEVICES)
def test_prefill_then_token_by_token(model_a, oracle_a, device):
    toks, want, _ = oracle_a
    eng = make_engine(model_a[0], device)
    got = replay_all(eng, "p", toks, [30] + [1] * 60)  # long decode crosses pages and tiles
    assert rel_err(got, want) < 2e-4
    eng2 = make_engine(model_a[0], device)
    got2 = replay_all(eng2, "q", toks[:40], [1] * 40)  # decoded from the very first token
    assert rel_err(got2, want[:40]) < 2e-4


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("cuts", [[2] * 45, [3, 13, 16, 17, 2, 31, 8], [15, 1, 16, 1, 32, 25], [64, 2, 24]])
def test_portions(model_a, oracle_a, device, cuts):
    toks, want, _ = oracle_a
    assert sum(cuts) == len(toks)
    eng = make_engine(model_a[0], device)
    assert rel_err(replay_all(eng, "c", toks, cuts), want) < 2e-4


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_mixed_batch_equals_each_alone_and_pools_are_reused(model_a, device, dtype):
    """Unequal requests share steps (portions beside single tokens), with a
    pool so small that pages and state slots of finished requests are handed
    to later ones; every logit row matches the request run alone."""
    if device == "cpu" and dtype == torch.bfloat16:
        pytest.skip("bf16 is the GPU serving precision")
    lens = {"a": 37, "b": 5, "c": 50, "d": 1, "e": 23, "f": 33}
    toks = {k: tokens_for(CFG_A, n, 100 + i) for i, (k, n) in enumerate(lens.items())}
    want = {k: O.forward(CFG_A, model_a[1], t) for k, t in toks.items()}
    plan = [
        [("a", 20), ("b", 3)],
        [("a", 1), ("b", 2), ("c", 30), ("d", 1)],           # b, d end: slots free
        [("a", 16), ("e", 7)],                                # c sits this step out; e reuses a freed slot + pages
        [("c", 20), ("e", 1), ("f", 2)],                      # a ended; c comes back and ends
        [("e", 15), ("f", 30)],
        [("f", 1)],
    ]
    eng = make_engine(model_a[0], device, dtype, blocks=9, block_size=16, seqs=4)
    at = {k: 0 for k in toks}
    got = {k: [] for k in toks}
    for step in plan:
        entries, end = [], []
        for rid, n in step:
            entries.append((rid, toks[rid][at[rid] : at[rid] + n], list(range(n))))
            at[rid] += n
            if at[rid] == lens[rid]:
                end.append(rid)
        res = eng.replay_step(entries, end)
        for rid, _ in step:
            got[rid].append(res[rid].float().cpu())
    assert all(at[k] == lens[k] for k in lens)
    bm = eng.scheduler.block_manager
    assert bm.num_free_blocks == 9 and bm.num_free_state_slots == 4
    for k in toks:
        assert_logits(torch.cat(got[k]), want[k], dtype)


@pytest.mark.parametrize("device", DEVICES)
def test_far_key_and_stale_pages(model_a, device):
    """A long prompt whose early tokens matter at the end, run after another
    request has dirtied every page and slot of the pool."""
    toks = tokens_for(CFG_A, 300, 31)
    want = O.forward(CFG_A, model_a[1], toks)
    eng = make_engine(model_a[0], device, blocks=19, block_size=16, seqs=1)
    junk = tokens_for(CFG_A, 304, 32)
    eng.replay_step([("junk", junk, [])], end=["junk"])
    got = replay_all(eng, "x", toks, [250, 1, 1, 30, 2] + [1] * 16)
    assert rel_err(got, want) < 2e-4


@pytest.mark.parametrize("device", DEVICES)
def test_greedy_generation_through_scheduler(model_a, device):
    """add_request + generate_all: chunked prefill under a tiny token budget,
    continuous batching of three requests, greedy sampling."""
    W = model_a[1]
    prompts = [tokens_for(CFG_A, n, 200 + n) for n in (19, 7, 26)]
    eng = make_engine(model_a[0], device, budget=8, blocks=32)
    seqs = [eng.add_request(p, SamplingParams(max_new_tokens=6)) for p in prompts]
    done = eng.generate_all(max_steps=200)
    assert len(done) == 3
    for seq, prompt in zip(seqs, prompts):
        toks = list(prompt)
        for step in range(6):
            logits = O.forward(CFG_A, W, toks)[-1]
            top2 = torch.topk(logits, 2).values
            if float(top2[0] - top2[1]) > 1e-3:  # an unambiguous argmax must match
                assert seq.output_token_ids[step] == int(torch.argmax(logits)), (step, seq.output_token_ids)
            toks.append(seq.output_token_ids[step])
    bm = eng.scheduler.block_manager
    assert bm.num_free_blocks == 32 and bm.num_free_state_slots == 4


@pytest.mark.parametrize("device", DEVICES)
def test_preempted_sequence_recomputes_its_state(model_a, device):
    prompt = tokens_for(CFG_A, 21, 77)
    ref = make_engine(model_a[0], device)
    s0 = ref.add_request(prompt, SamplingParams(max_new_tokens=8))
    ref.generate_all(max_steps=50)
    eng = make_engine(model_a[0], device)
    s1 = eng.add_request(prompt, SamplingParams(max_new_tokens=8))
    for _ in range(4):
        eng.step()
    sch = eng.scheduler
    sch.running.remove(s1)
    sch.block_manager.free(s1)
    s1.preempt()
    sch.waiting.appendleft(s1)
    assert s1.state_slot == -1
    eng.generate_all(max_steps=50)
    assert s1.output_token_ids == s0.output_token_ids


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_cache_rows_of_the_mfma_kernel(model_c, device, dtype):
    if device == "cpu" and dtype == torch.bfloat16:
        pytest.skip("bf16 is the GPU serving precision")
    ta, tb = tokens_for(CFG_C, 150, 41), tokens_for(CFG_C, 70, 42)
    wa, wb = O.forward(CFG_C, model_c[1], ta), O.forward(CFG_C, model_c[1], tb)
    eng = make_engine(model_c[0], device, dtype)
    if device != "cpu" and dtype == torch.bfloat16:
        assert all(l.mixer.mfma_rows(dtype, True) for l in eng.runner.model.layers)
    got_a, got_b = [], []
    # a: 100-token portion (two 64-row tiles, the second partial), then single
    # tokens; b joins with portions beside a's single tokens
    plan = [[("a", 100)], [("a", 1), ("b", 65)], [("a", 30), ("b", 1)], [("a", 1), ("b", 4)], [("a", 18)]]
    at = {"a": 0, "b": 0}
    toks = {"a": ta, "b": tb}
    for step in plan:
        entries = []
        for rid, n in step:
            entries.append((rid, toks[rid][at[rid] : at[rid] + n], list(range(n))))
            at[rid] += n
        res = eng.replay_step(entries, [r for r, _ in step if at[r] == len(toks[r])])
        for rid, _ in step:
            (got_a if rid == "a" else got_b).append(res[rid].float().cpu())
    assert_logits(torch.cat(got_a), wa, dtype)
    assert_logits(torch.cat(got_b), wb, dtype)


def assert_greedy_follows_oracle(cfg, W, prompt, outputs, margin):
    """Teacher-forced on the engine's own outputs: every chosen token's
    oracle logit is within `margin` (in units of the logits' spread) of the
    oracle's best."""
    toks = list(prompt)
    for step, tok in enumerate(outputs):
        logits = O.forward(cfg, W, toks)[-1]
        gap = float(logits.max() - logits[tok]) / float(logits.std())
        assert gap <= margin, (step, tok, gap)
        toks.append(tok)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("which", ["a", "c"])
def test_decode_graphs_replay_like_eager(model_a, model_c, dtype, which):
    """Decode-only steps replay captured hipGraphs (static per-sequence
    tables, state slots filled per step, dense expert dispatch).  Many
    replays with eager prefill steps of later requests in between; every
    generated token is checked."""
    path, W = model_a if which == "a" else model_c
    cfg = CFG_A if which == "a" else CFG_C
    mc = get_model_config(path)
    ec = EngineConfig(
        model=mc, num_kv_blocks=64, max_num_seqs=4, num_state_slots=4,
        max_num_batched_tokens=32, max_model_len=512, watermark_blocks=0, enforce_eager=False,
    )
    eng = LLMEngine(ec, device="cuda:0", dtype=dtype)
    prompts = [tokens_for(cfg, n, 300 + n) for n in (9, 40, 17)]
    seqs = [eng.add_request(prompts[0], SamplingParams(max_new_tokens=14))]
    for _ in range(5):
        eng.step()                      # prefill, then graph replays at batch 1
    seqs.append(eng.add_request(prompts[1], SamplingParams(max_new_tokens=9)))
    for _ in range(4):
        eng.step()                      # chunked eager prefill beside the decode
    seqs.append(eng.add_request(prompts[2], SamplingParams(max_new_tokens=11)))
    eng.generate_all(max_steps=100)
    assert eng.runner.graph_runner is not None and eng.runner.graph_runner.graphs
    margin = 1e-3 if dtype == torch.float32 else 0.15
    for seq, prompt in zip(seqs, prompts):
        assert seq.is_finished()
        assert_greedy_follows_oracle(cfg, W, prompt, seq.output_token_ids, margin)


def test_served_through_the_pool_and_front_door(tmp_path):
    """A model folder as the pool's base model: worker process, router, HTTP
    front door, greedy completion from prompt token ids."""
    from starlette.testclient import TestClient

    from llm_instance_gateway_amd.api.types import InferenceModel
    from llm_instance_gateway_amd.serving import EnginePool, build_app

    cfg = dict(CFG_A, vocab=300)
    W = make_checkpoint(cfg, 21)
    path = write_model(tmp_path / "served", cfg, W)
    pool = EnginePool(
        path, devices=["cpu"],
        engine_kwargs=dict(num_kv_blocks=64, max_num_seqs=4, max_num_batched_tokens=64, max_model_len=256),
    )
    pool.start()
    try:
        pool.datastore.store_model(InferenceModel(model_name="latent"))
        client = TestClient(build_app(pool))
        prompt = tokens_for(cfg, 23, 8)
        r = client.post("/v1/completions", json={"model": "latent", "prompt": prompt, "max_tokens": 5})
        assert r.status_code == 200, r.text
        out = r.json()["choices"][0]["token_ids"]
        assert len(out) == 5
        assert_greedy_follows_oracle(cfg, W, prompt, out, margin=0.2)  # workers run bf16
    finally:
        pool.stop()
