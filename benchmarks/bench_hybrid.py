#!/usr/bin/env python3
"""Tikarax beside Llama at equal size: prefill and decode throughput through
the engine, and the new kernels beside their Llama counterparts against the
HBM roofline.

    python bench.py --hybrid                  # both parts, JSON lines
    python benchmarks/bench_hybrid.py --part engine|kernels [--sizes s,m]

Engine part: for each size a Tikarax stack (alternating minGRU / gated
attention layers, xIELU feed-forward) and a Llama stack with the same width,
depth, heads and a feed-forward of the same parameter count run the same
workload through LLMEngine.step(): N prompts of L tokens prefilled in
budget-sized steps, then K decode steps (hipGraph replay) at batch N.
Random weights, synthetic tokens.

Kernel part: each elementwise / scan / scatter kernel of the new design and
the like kernel of the Llama path, timed with events at the layer shapes of
the sizes above; bytes moved / time against 8 TB/s.
"""

from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))

from llm_instance_gateway_amd import ops
from llm_instance_gateway_amd.engine import EngineConfig, LLMEngine, SamplingParams
from llm_instance_gateway_amd.models.config import ModelConfig
from llm_instance_gateway_amd.models.tikarax import make_config

HBM_BYTES_PER_S = 8.0e12

# name: width, layers, heads, kv_heads, head size, ff (two-matrix), vocab
SIZES = {
    "s": dict(width=2048, layers=8, heads=16, kv_heads=4, dim=128, ff=8192, vocab=32000),
    "m": dict(width=4096, layers=8, heads=32, kv_heads=8, dim=128, ff=14336, vocab=32000),
}


def tikarax_config(name: str, z: dict) -> ModelConfig:
    layers = []
    for i in range(z["layers"]):
        mlp = {"ff": z["ff"], "kind": "dense"}
        if i % 2 == 0:
            layers.append({"type": "mingru", "mixer": {"width": z["width"]}, "mlp": mlp})
        else:
            layers.append({
                "type": "attention",
                "mixer": {"heads": z["heads"], "kv_heads": z["kv_heads"], "dim": z["dim"],
                          "vdim": z["dim"], "scale": 1.0 / math.sqrt(z["dim"]),
                          "q_temp": {"coef": 0.25, "every": 128}},
                "mlp": mlp,
            })
    return make_config(f"tikarax-{name}", z["vocab"], z["width"], layers, groups=4)


def llama_config(name: str, z: dict) -> ModelConfig:
    # three-matrix SwiGLU with the parameter count of the two-matrix ff
    inter = (2 * z["ff"] // 3 + 255) // 256 * 256
    return ModelConfig(
        name=f"llama-{name}", vocab_size=z["vocab"], hidden_size=z["width"],
        num_layers=z["layers"], num_heads=z["heads"], num_kv_heads=z["kv_heads"],
        intermediate_size=inter, head_dim=z["dim"], max_position_embeddings=8192,
    )


def engine_run(mc: ModelConfig, n_seqs: int, prompt_len: int, decode_steps: int) -> dict:
    cfg = EngineConfig(
        model=mc, num_kv_blocks=n_seqs * ((prompt_len + decode_steps) // 16 + 4),
        max_num_seqs=n_seqs, num_state_slots=n_seqs, max_num_batched_tokens=8192,
        max_model_len=4096, gpu_memory_utilization=0.9,
    )
    torch.manual_seed(0)
    eng = LLMEngine(cfg, device="cuda:0")
    g = torch.Generator().manual_seed(1)

    def fill(new_tokens: int):
        for _ in range(n_seqs):
            p = torch.randint(1, mc.vocab_size - 1, (prompt_len,), generator=g).tolist()
            eng.add_request(p, SamplingParams(max_new_tokens=new_tokens))

    def prefill_phase() -> float:
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        while eng.scheduler.num_waiting or any(s.in_prefill for s in eng.scheduler.running):
            eng.step()
        torch.cuda.synchronize()
        return time.perf_counter() - t0

    # warm-up pass: GEMM algorithm picks, graph capture
    fill(4)
    prefill_phase()
    eng.generate_all()
    # timed: median of three rounds (a round = all prompts prefilled, then
    # every sequence decoded to its end)
    t_pre, t_dec, n_steps = [], [], []
    for _ in range(3):
        fill(decode_steps + 1)
        t_pre.append(prefill_phase())
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        steps = 0
        while eng.has_work():
            eng.step()
            steps += 1
        torch.cuda.synchronize()
        t_dec.append((time.perf_counter() - t0) / max(steps, 1))
        n_steps.append(steps)
        eng.collect_finished()
    del eng
    torch.cuda.empty_cache()
    t_prefill = sorted(t_pre)[1]
    t_step = sorted(t_dec)[1]
    return {
        "prefill_tok_per_s": round(n_seqs * prompt_len / t_prefill, 1),
        "decode_tok_per_s": round(n_seqs / t_step, 1),
        "decode_ms_per_step": round(t_step * 1e3, 3),
        "prefill_s_rounds": [round(t, 4) for t in t_pre],
    }


def part_engine(sizes) -> None:
    for name in sizes:
        z = SIZES[name]
        for n_seqs, plen in ((16, 1024), (64, 512)):
            row = {"bench": "engine", "size": name, **z, "seqs": n_seqs, "prompt_len": plen, "decode_steps": 64}
            row["tikarax"] = engine_run(tikarax_config(name, z), n_seqs, plen, 64)
            row["llama"] = engine_run(llama_config(name, z), n_seqs, plen, 64)
            for k in ("prefill_tok_per_s", "decode_tok_per_s"):
                row["ratio_" + k] = round(row["tikarax"][k] / row["llama"][k], 3)
            print(json.dumps(row), flush=True)


def timeit(fn, iters: int = 30) -> float:
    for _ in range(5):
        fn()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(iters):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / iters * 1e-3


def part_kernels(sizes) -> None:
    dev, bf = "cuda:0", torch.bfloat16
    for name in sizes:
        z = SIZES[name]
        H, FF, W = z["width"], z["ff"], z["width"]
        hq, hkv, D = z["heads"], z["kv_heads"], z["dim"]
        for T in (8192, 256):  # a prefill step's rows / a decode batch
            rows = []

            def add(kernel, like, t, nbytes):
                rows.append({"kernel": kernel, "like": like, "us": round(t * 1e6, 2),
                             "GB_per_s": round(nbytes / t / 1e9, 1),
                             "of_roofline": round(nbytes / t / HBM_BYTES_PER_S, 3)})

            x32 = torch.randn(T, H, device=dev)
            y = torch.randn(T, H, device=dev, dtype=bf)
            res16 = torch.randn(T, H, device=dev, dtype=bf)
            w = torch.ones(H, device=dev, dtype=bf)
            # fused post-norm + add + pre-norm: reads y (2B) + residual (4B), writes residual (4B) + out (2B)
            add("post_add_pre_norm(groups=2, fp32 residual)", "",
                timeit(lambda: ops.post_add_pre_norm(x32, y, w, w, 1e-5, 2)), T * H * 12)
            add("fused_add_rms_norm(bf16 residual)", "post_add_pre_norm",
                timeit(lambda: ops.fused_add_rms_norm(y, res16, w, 1e-5)), T * H * 8)
            up = torch.randn(T, FF, device=dev, dtype=bf)
            add("xielu", "", timeit(lambda: ops.xielu(up, 0.7, 1.2)), T * FF * 4)
            inter = (2 * FF // 3 + 255) // 256 * 256
            gu = torch.randn(T, 2 * inter, device=dev, dtype=bf)
            add("silu_and_mul", "xielu", timeit(lambda: ops.silu_and_mul(gu)), T * inter * 6)
            # minGRU scan: one sequence per 1024 rows (prefill) or per row (decode)
            zxg = torch.randn(T, 3 * W, device=dev, dtype=bf)
            seg = 1024 if T >= 1024 else 1
            S = T // seg
            i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=dev)
            st = torch.zeros(S + 1, W, device=dev)
            segs = (i32([i * seg for i in range(S)]), i32([seg] * S), i32(list(range(S))), i32([0] * S))
            add(f"mingru_scan(segments of {seg})", "",
                timeit(lambda: ops.mingru_scan(zxg, st, *segs, seg)), T * W * 8 + 2 * S * W * 4)
            # K/V scatter from the fused projection vs the contiguous-row scatter
            bs, nblk = 16, T // 16 + 1
            kc = torch.zeros(nblk, hkv, bs, D, device=dev, dtype=bf)
            vc = torch.zeros_like(kc)
            proj = torch.randn(T, (hq + 2 * hkv + hq) * D, device=dev, dtype=bf)
            kview, vview = proj[:, hq * D:(hq + hkv) * D], proj[:, (hq + hkv) * D:(hq + 2 * hkv) * D]
            slots = torch.randperm(T, device=dev).to(torch.int64)
            add("kv_scatter(strided views)", "", timeit(lambda: ops.kv_scatter(kview, vview, kc, vc, slots)),
                T * hkv * D * 2 * 2 * 2)
            kk, vv = kview.contiguous(), vview.contiguous()
            add("reshape_and_cache", "kv_scatter", timeit(lambda: ops.reshape_and_cache(kk, vv, kc, vc, slots)),
                T * hkv * D * 2 * 2 * 2)
            pos = torch.arange(T, device=dev, dtype=torch.int64)
            qv = proj[:, : hq * D]
            add("temperature_scale_rows", "rotary_embedding",
                timeit(lambda: ops.temperature_scale_rows(qv, pos, 0.25, 128.0)), T * hq * D * 4)
            qc, kc2 = qv.contiguous(), kk.clone()
            csc = ops.build_cos_sin_cache(D, T, 10000.0, dev).float()
            add("rotary_embedding", "temperature_scale_rows",
                timeit(lambda: ops.rotary_embedding(pos, qc, kc2, csc, D)), T * (hq + hkv) * D * 4)
            o = torch.randn(T, hq * D, device=dev, dtype=bf)
            gv = proj[:, (hq + 2 * hkv) * D:]
            add("sigmoid_gate_mul", "", timeit(lambda: ops.sigmoid_gate_mul(o, gv)), T * hq * D * 6)
            emb = torch.randn(z["vocab"], H, device=dev, dtype=bf)
            ids = torch.randint(0, z["vocab"], (T,), device=dev)
            add("embed_group_norm", "", timeit(lambda: ops.embed_group_norm(ids, emb, w, 1e-5, 2)), T * H * 6)
            if T >= 1024:
                # prompt attention: 8 fresh prompts of 1024 tokens, causal;
                # flops = 2 (QK^T, PV) * 2 * sum over rows of keys seen * D * heads
                L, S = 1024, T // 1024
                nb_seq = L // bs
                kcache = torch.randn(S * nb_seq + 1, hkv, bs, D, device=dev, dtype=bf)
                vcache = torch.randn_like(kcache)
                tables = torch.arange(S * nb_seq, dtype=torch.int32, device=dev).view(S, nb_seq)
                qsl = i32([i * L for i in range(S + 1)])
                ctxl = i32([L] * S)
                tseq = i32([s_ for s_ in range(S) for _ in range(L // 64)])
                tqs = i32([q0 for _ in range(S) for q0 in range(0, L, 64)])
                tok_seq = i32([s_ for s_ in range(S) for _ in range(L)])
                posq = torch.arange(L, device=dev, dtype=torch.int64).repeat(S)
                flops = 4.0 * S * (L * (L + 1) / 2) * D * hq
                sc = 1.0 / math.sqrt(D)

                def addf(kernel, t):
                    rows.append({"kernel": kernel, "like": "attention prefill", "us": round(t * 1e6, 1),
                                 "TFLOP_per_s": round(flops / t / 1e12, 1)})

                addf("paged_attention_prefill_tiles (temperature+gate fused)", timeit(
                    lambda: ops.paged_attention_prefill_tiles(qv, kcache, vcache, tables, qsl, ctxl, tseq, tqs, sc, hq,
                                                              gate=gv, temp_coef=0.25, temp_every=128.0), 10))
                qh = qv.contiguous().view(T, hq, D)
                addf("paged_attention_prefill (64/128 kernel of the Llama path)", timeit(
                    lambda: ops.paged_attention_prefill(qh, kcache, vcache, tables, qsl, ctxl, sc,
                                                        tile_seq=tseq, tile_qstart=tqs), 10))
                addf("paged_attention_general (any-shape kernel)", timeit(
                    lambda: ops.paged_attention_general(qv, kcache, vcache, tables, tok_seq, posq, sc, hq, gate=gv,
                                                        temp_coef=0.25, temp_every=128.0), 3))
            else:
                # decode attention: T sequences with 1024 cached tokens each;
                # bytes = K and V of every sequence once
                L = 1024
                nb_seq = L // bs
                kcache = torch.randn(T * nb_seq + 1, hkv, bs, D, device=dev, dtype=bf)
                vcache = torch.randn_like(kcache)
                tables = torch.arange(T * nb_seq, dtype=torch.int32, device=dev).view(T, nb_seq)
                ctxl = i32([L] * T)
                posd = torch.full((T,), L - 1, device=dev, dtype=torch.int64)
                tok_seq = i32(list(range(T)))
                kvbytes = T * L * hkv * D * 2 * 2
                sc = 1.0 / math.sqrt(D)
                qh = qv.contiguous().view(T, hq, D)
                add("paged_attention_general (decode rows, gate+temperature fused)", "",
                    timeit(lambda: ops.paged_attention_general(qv, kcache, vcache, tables, tok_seq, posd, sc, hq,
                                                               gate=gv, temp_coef=0.25, temp_every=128.0), 10), kvbytes)
                add("paged_attention_decode (64/128 kernel of the Llama path)", "paged_attention_general",
                    timeit(lambda: ops.paged_attention_decode(qh, kcache, vcache, tables, ctxl, sc, max_ctx=L), 10), kvbytes)
            print(json.dumps({"bench": "kernels", "size": name, "rows": T, "kernels": rows}), flush=True)


def main(argv=None) -> None:
    ap = argparse.ArgumentParser(description=__doc__.splitlines()[0])
    ap.add_argument("--part", default="engine,kernels")
    ap.add_argument("--sizes", default="s,m")
    args = ap.parse_args(argv)
    assert torch.cuda.is_available(), "this benchmark needs the GPU"
    sizes = [s for s in args.sizes.split(",") if s]
    if "kernels" in args.part:
        part_kernels(sizes)
    if "engine" in args.part:
        part_engine(sizes)


if __name__ == "__main__":
    main()
