"""Tikarax through the engine (scheduler, block/state pools, model runner,
kernels) against the slow float64 oracle in tikarax_oracle.py.

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

from tikarax_oracle import o_forward

DEVICES = ["cpu", pytest.param("cuda:0", marks=pytest.mark.gpu)]


def attn(heads, kv_heads, dim, vdim, ff=None, coef=0.3, every=5, scale=None):
    return {
        "type": "attention",
        "mixer": {
            "heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
            "q_temp": {"coef": coef, "every": every},
            "scale": scale if scale is not None else 1.3 / math.sqrt(dim),
        },
        "mlp": None if ff is None else {"ff": ff, "kind": "dense"},
    }


def gru(width, ff=None):
    return {"type": "mingru", "mixer": {"width": width},
            "mlp": None if ff is None else {"ff": ff, "kind": "dense"}}


# sizes chosen to differ from one another: key size != value size, a layer
# without feed-forward, kv_heads in {1, 2, heads}, three norm groups
CFG_A = {
    "architecture": "Tikarax", "vocab": 50, "width": 48,
    "norm": {"eps": 1e-5, "groups": 3},
    "layers": [attn(4, 2, 8, 12, ff=40), gru(24, ff=56), attn(2, 1, 16, 8), gru(40), attn(3, 3, 8, 8, ff=24, every=1)],
}
# degenerate values: one group, one head, coef 0, width-1 recurrent layer
CFG_B = {
    "architecture": "Tikarax", "vocab": 31, "width": 16,
    "norm": {"eps": 1e-3, "groups": 1},
    "layers": [gru(1, ff=8), attn(1, 1, 4, 4, ff=8, coef=0.0, every=7), gru(33)],
}


def make_checkpoint(cfg, seed):
    g = torch.Generator().manual_seed(seed)
    H, V = cfg["width"], cfg["vocab"]

    def r(*shape, s=1.0):
        return (torch.randn(*shape, generator=g) * s).to(torch.bfloat16)

    def nw():
        return (1.0 + 0.2 * torch.randn(H, generator=g)).to(torch.bfloat16)

    W = {"embed": r(V, H), "embed.norm": nw(), "final.norm": nw(), "head": r(V, H, s=H ** -0.5)}
    for i, layer in enumerate(cfg["layers"]):
        p = "l%d." % i
        W[p + "norm1"], W[p + "norm1b"] = nw(), nw()
        m = layer["mixer"]
        if layer["type"] == "attention":
            nq, nk, nv = m["heads"] * m["dim"], m["kv_heads"] * m["dim"], m["kv_heads"] * m["vdim"]
            ng = m["heads"] * m["vdim"]
            W[p + "mix.q"], W[p + "mix.q.b"] = r(nq, H, s=H ** -0.5), r(nq, s=0.3)
            W[p + "mix.k"], W[p + "mix.k.b"] = r(nk, H, s=H ** -0.5), r(nk, s=0.3)
            W[p + "mix.v"], W[p + "mix.v.b"] = r(nv, H, s=H ** -0.5), r(nv, s=0.3)
            W[p + "mix.g"] = r(ng, H, s=H ** -0.5)
            W[p + "mix.o"] = r(H, ng, s=ng ** -0.5)
        else:
            w = m["width"]
            W[p + "mix.z"], W[p + "mix.z.b"] = r(w, H, s=H ** -0.5), r(w, s=0.5)
            W[p + "mix.x"], W[p + "mix.x.b"] = r(w, H, s=H ** -0.5), r(w, s=0.5)
            W[p + "mix.g"] = r(w, H, s=H ** -0.5)
            W[p + "mix.o"] = r(H, w, s=w ** -0.5)
        if layer["mlp"] is not None:
            ff = layer["mlp"]["ff"]
            W[p + "norm2"], W[p + "norm2b"] = nw(), nw()
            W[p + "mlp.up"] = r(ff, H, s=H ** -0.5)
            W[p + "mlp.down"] = r(H, ff, s=ff ** -0.5)
            W[p + "mlp.act"] = r(2, s=0.7)
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


def tol(dtype):
    return 2e-4 if dtype == torch.float32 else 6e-2


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


@pytest.fixture(scope="module")
def model_a(tmp_path_factory):
    W = make_checkpoint(CFG_A, 11)
    return write_model(tmp_path_factory.mktemp("tkx") / "a", CFG_A, W), W


@pytest.fixture(scope="module")
def model_b(tmp_path_factory):
    W = make_checkpoint(CFG_B, 12)
    return write_model(tmp_path_factory.mktemp("tkx") / "b", CFG_B, W), W


@pytest.fixture(scope="module")
def oracle_a(model_a):
    toks = tokens_for(CFG_A, 90, 5)
    res = []
    return toks, o_forward(CFG_A, model_a[1], toks, residuals=res), res


DTYPES = [torch.float32, torch.bfloat16]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_whole_prompt_and_every_layer(model_a, oracle_a, device, dtype):
    if device == "cpu" and dtype == torch.bfloat16:
        pytest.skip("bf16 is the GPU serving precision")
    toks, want, want_res = oracle_a
    eng = make_engine(model_a[0], device, dtype)
    captured = eng.runner.model.capture_residuals = []
    got = replay_all(eng, "w", toks, [len(toks)])
    assert rel_err(got, want) < tol(dtype)
    assert len(captured) == len(CFG_A["layers"])
    for i, (x, xo) in enumerate(zip(captured, want_res)):
        assert x.dtype == torch.float32, "the residual stream stays fp32"
        x = x[: len(toks)]  # rows past the tokens are GEMM-bucketing padding
        e = (x.double().cpu() - xo).abs().max().item() / xo.abs().max().item()
        assert e < (1e-4 if dtype == torch.float32 else 4e-2), f"layer {i}: {e}"


@pytest.mark.parametrize("device", DEVICES)
def test_degenerate_sizes(model_b, device):
    toks = tokens_for(CFG_B, 40, 6)
    want = o_forward(CFG_B, model_b[1], toks)
    eng = make_engine(model_b[0], device, block_size=8)
    assert rel_err(replay_all(eng, "d", toks, [17, 1, 1, 2, 19]), want) < 2e-4


@pytest.mark.parametrize("device", DEVICES)
def test_first_token_alone(model_a, oracle_a, device):
    toks, want, _ = oracle_a
    eng = make_engine(model_a[0], device)
    got = replay_all(eng, "f", toks[:1], [1])
    assert rel_err(got, want[:1]) < 2e-4


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
    """Four unequal requests share steps (portions beside single tokens),
    with a pool so small that pages and state slots of finished requests are
    handed to later ones; every logit row matches the request run alone."""
    if device == "cpu" and dtype == torch.bfloat16:
        pytest.skip("bf16 is the GPU serving precision")
    lens = {"a": 37, "b": 5, "c": 50, "d": 1, "e": 23, "f": 33}
    toks = {k: tokens_for(CFG_A, n, 100 + i) for i, (k, n) in enumerate(lens.items())}
    want = {k: o_forward(CFG_A, make_checkpoint(CFG_A, 11), t) for k, t in toks.items()}
    # steps: (id, n tokens); requests end when their tokens run out
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
        assert rel_err(torch.cat(got[k]), want[k]) < tol(dtype), k


@pytest.mark.parametrize("device", DEVICES)
def test_pool_exhaustion_is_an_error(model_a, device):
    eng = make_engine(model_a[0], device, blocks=2, block_size=16, seqs=2)
    t = tokens_for(CFG_A, 40, 3)
    with pytest.raises(RuntimeError):
        eng.replay_step([("x", t, [0])])
    eng = make_engine(model_a[0], device, blocks=8, block_size=16, seqs=2)
    eng.replay_step([("x", t[:3], []), ("y", t[:3], [])])
    with pytest.raises(RuntimeError):
        eng.replay_step([("z", t[:3], [])])  # no state slot left


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
            logits = o_forward(CFG_A, W, toks)[-1]
            top2 = torch.topk(logits, 2).values
            choice = int(torch.argmax(logits))
            if float(top2[0] - top2[1]) > 1e-3:  # an unambiguous argmax must match
                assert seq.output_token_ids[step] == choice, (step, seq.output_token_ids)
            toks.append(seq.output_token_ids[step])
    bm = eng.scheduler.block_manager
    assert bm.num_free_blocks == 32 and bm.num_free_state_slots == 4


@pytest.mark.parametrize("device", DEVICES)
def test_preempted_sequence_recomputes_its_state(model_a, device):
    """Preemption drops pages AND the state slot; the re-prefill starts the
    recurrence from zero again and generation continues identically."""
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


# key size == value size in {64, 128}: with bf16 storage on the GPU these
# layers take the tiled MFMA prefill / paged decode kernels (temperature
# folded into q, gate applied afterwards); fp32 storage takes the general one
CFG_C = {
    "architecture": "Tikarax", "vocab": 40, "width": 64,
    "norm": {"eps": 1e-5, "groups": 2},
    "layers": [attn(2, 1, 64, 64, ff=48, every=9), gru(32), attn(4, 2, 128, 128, coef=0.6, every=16)],
}


@pytest.fixture(scope="module")
def model_c(tmp_path_factory):
    W = make_checkpoint(CFG_C, 13)
    return write_model(tmp_path_factory.mktemp("tkx") / "c", CFG_C, W), W


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_head_sizes_of_the_tiled_kernels(model_c, device, dtype):
    if device == "cpu" and dtype == torch.bfloat16:
        pytest.skip("bf16 is the GPU serving precision")
    from llm_instance_gateway_amd import ops

    ta, tb = tokens_for(CFG_C, 150, 41), tokens_for(CFG_C, 70, 42)
    wa, wb = o_forward(CFG_C, model_c[1], ta), o_forward(CFG_C, model_c[1], tb)
    eng = make_engine(model_c[0], device, dtype)
    if device != "cpu" and dtype == torch.bfloat16 and ops.native_available():
        assert eng.runner.model.needs_prefill_tiles
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
    assert rel_err(torch.cat(got_a), wa) < tol(dtype)
    assert rel_err(torch.cat(got_b), wb) < tol(dtype)


def assert_greedy_follows_oracle(cfg, W, prompt, outputs, margin):
    """Teacher-forced on the engine's own outputs: every chosen token's
    oracle logit is within `margin` (in units of the logits' spread) of the
    oracle's best."""
    toks = list(prompt)
    for step, tok in enumerate(outputs):
        logits = o_forward(cfg, W, toks)[-1]
        gap = float(logits.max() - logits[tok]) / float(logits.std())
        assert gap <= margin, (step, tok, gap)
        toks.append(tok)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("which", ["a", "c"])
def test_decode_graphs_replay_like_eager(model_a, model_c, dtype, which):
    """Decode-only steps replay captured hipGraphs (static per-sequence
    tables, state slots filled per step).  Many replays with eager prefill
    steps of later requests in between; every generated token is checked."""
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
        pool.datastore.store_model(InferenceModel(model_name="hybrid"))
        client = TestClient(build_app(pool))
        prompt = tokens_for(cfg, 23, 8)
        r = client.post("/v1/completions", json={"model": "hybrid", "prompt": prompt, "max_tokens": 5})
        assert r.status_code == 200, r.text
        out = r.json()["choices"][0]["token_ids"]
        assert len(out) == 5
        assert_greedy_follows_oracle(cfg, W, prompt, out, margin=0.2)  # workers run bf16
    finally:
        pool.stop()
