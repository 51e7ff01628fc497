#!/usr/bin/env python3
"""Lopovik beside Llama and Mixtral at equal size: prefill and decode
throughput through the engine, and the design's kernels beside their
counterparts against the roofline.

    python bench.py --latent                  # both parts, JSON lines
    python benchmarks/bench_latent.py --part engine|kernels|profile [--sizes s,m]

Engine part, per size: a Lopovik stack with squared-ReLU feed-forwards beside
a Llama stack of the same width, depth, head count and feed-forward
parameter count; and a Lopovik stack whose every second layer routes to
gated-SiLU experts beside a Mixtral stack with the same experts.  Same
workload through LLMEngine.step(): N prompts of L tokens prefilled in
budget-sized steps, then K decode steps (hipGraph replay) at batch N.
Random weights, synthetic tokens.

Kernel part: each kernel of the design and the like kernel of the Llama
path, timed with events at the layer shapes of the sizes above; bytes that
must move / time against 8 TB/s, attention in TFLOP/s (prompt) and cache
bytes / time (decode).
"""

from __future__ import annotations

import argparse
import json
import math
import os
import sys

import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))

from bench_hybrid import HBM_BYTES_PER_S, engine_run, llama_config, timeit

from llm_instance_gateway_amd import ops
from llm_instance_gateway_amd.models.config import ModelConfig
from llm_instance_gateway_amd.models.lopovik import make_config

# width, layers, heads, per-head sizes, latent ranks, feed-forward, experts
SIZES = {
    "s": dict(width=2048, layers=8, heads=16, dim=128, rot_dim=64, vdim=128, q_rank=768,
              kv_rank=512, ff=8192, experts=8, top=2, expert_ff=2048, vocab=32000),
    "m": dict(width=4096, layers=8, heads=32, dim=128, rot_dim=64, vdim=128, q_rank=1536,
              kv_rank=512, ff=14336, experts=8, top=2, expert_ff=3584, vocab=32000),
}


def lopovik_config(name: str, z: dict, routed: bool) -> ModelConfig:
    mixer = {
        "heads": z["heads"], "dim": z["dim"], "rot_dim": z["rot_dim"], "vdim": z["vdim"],
        "q_rank": z["q_rank"], "kv_rank": z["kv_rank"],
        "rot": {"base": 10000.0, "dims": z["rot_dim"]},
        "scale": 1.0 / math.sqrt(z["dim"] + z["rot_dim"]),
    }
    layers = []
    for i in range(z["layers"]):
        if routed and i % 2 == 1:
            mlp = {"kind": "moe", "expert": {"ff": z["expert_ff"]},
                   "router": {"experts": z["experts"], "top": z["top"]}}
        else:
            mlp = {"kind": "dense", "ff": z["ff"]}
        layers.append({"type": "latent_attention", "mixer": dict(mixer), "mlp": mlp})
    return make_config(f"lopovik-{name}{'-routed' if routed else ''}", z["vocab"], z["width"], layers)


def mixtral_config(name: str, z: dict) -> ModelConfig:
    return ModelConfig(
        name=f"mixtral-{name}", vocab_size=z["vocab"], hidden_size=z["width"],
        num_layers=z["layers"], num_heads=z["heads"], num_kv_heads=z["heads"] // 4,
        intermediate_size=z["expert_ff"], head_dim=128, max_position_embeddings=8192,
        num_experts=z["experts"], num_experts_per_tok=z["top"],
    )


def part_engine(sizes) -> None:
    for name in sizes:
        z = SIZES[name]
        zl = dict(z, kv_heads=z["heads"] // 4)
        for n_seqs, plen in ((16, 1024),):
            row = {"bench": "engine", "size": name, **z, "seqs": n_seqs, "prompt_len": plen, "decode_steps": 64}
            row["lopovik_dense"] = engine_run(lopovik_config(name, z, False), n_seqs, plen, 64)
            row["llama"] = engine_run(llama_config(name, zl), n_seqs, plen, 64)
            row["lopovik_routed"] = engine_run(lopovik_config(name, z, True), n_seqs, plen, 64)
            row["mixtral"] = engine_run(mixtral_config(name, z), n_seqs, plen, 64)
            for k in ("prefill_tok_per_s", "decode_tok_per_s"):
                row["dense_vs_llama_" + k] = round(row["lopovik_dense"][k] / row["llama"][k], 3)
                row["routed_vs_mixtral_" + k] = round(row["lopovik_routed"][k] / row["mixtral"][k], 3)
            print(json.dumps(row), flush=True)


def part_kernels(sizes) -> None:
    dev, bf = "cuda:0", torch.bfloat16
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=dev)
    for name in sizes:
        z = SIZES[name]
        H, FF = z["width"], z["ff"]
        hq, D, Rr, Dv, Rq, Rk = z["heads"], z["dim"], z["rot_dim"], z["vdim"], z["q_rank"], z["kv_rank"]
        row = Rk + Rr
        hkv = hq // 4
        for T in (8192, 256):  # a prefill step's rows / a decode batch
            rows = []

            def add(kernel, like, t, nbytes):
                rows.append({"kernel": kernel, "like": like, "us": round(t * 1e6, 2),
                             "GB_per_s": round(nbytes / t / 1e9, 1),
                             "of_roofline": round(nbytes / t / HBM_BYTES_PER_S, 3)})

            x32 = torch.randn(T, H, device=dev)
            y = torch.randn(T, H, device=dev, dtype=bf)
            y2 = torch.randn(T, H, device=dev, dtype=bf)
            res16 = torch.randn(T, H, device=dev, dtype=bf)
            w = torch.zeros(H, device=dev, dtype=bf)
            seg = 1024 if T >= 1024 else 1
            S = T // seg
            state = torch.zeros(S + 1, H, device=dev)
            tok_seq = i32([s_ for s_ in range(S) for _ in range(seg)])
            segs = (i32([i * seg for i in range(S)]), i32([seg] * S), i32(list(range(S))), i32([0] * S))
            # both norms + shift: reads the residual (4B), writes two activations (2B + 2B)
            add("offset_norm_shift (two norms, token shift, state)", "",
                timeit(lambda: ops.offset_norm_shift(x32, w, w, w, state, tok_seq, *segs, 1e-5)), T * H * 8)
            add("residual_add (both branches)", "", timeit(lambda: ops.residual_add(x32, y, y2)), T * H * 12)
            # the add folded into the next layer's norms: + two addends in, the new residual out
            add("offset_norm_shift with both branch outputs added on the way in", "",
                timeit(lambda: ops.offset_norm_shift(x32, w, w, w, state, tok_seq, *segs, 1e-5, y, y2)), T * H * 16)
            add("fused_add_rms_norm (bf16 residual)", "offset_norm_shift + residual_add",
                timeit(lambda: ops.fused_add_rms_norm(y, res16, torch.ones_like(w), 1e-5)), T * H * 8)
            up = torch.randn(T, FF, device=dev, dtype=bf)
            add("relu_squared", "", timeit(lambda: ops.relu_squared(up)), T * FF * 4)
            inter = (2 * FF // 3 + 255) // 256 * 256
            gu = torch.randn(T, 2 * inter, device=dev, dtype=bf)
            add("silu_mul (light library)", "", timeit(lambda: ops.silu_mul(gu)), T * inter * 6)
            add("silu_and_mul", "relu_squared, silu_mul", timeit(lambda: ops.silu_and_mul(gu)), T * inter * 6)
            # latent prep: reads the three projection parts, writes the query latent and the cache row
            bs, nblk = 16, T // 16 + 1
            proj = torch.randn(T, Rq + row + hq * Dv, device=dev, dtype=bf)
            cache = torch.zeros(nblk, 1, bs, row, device=dev, dtype=bf)
            slots = torch.randperm(T, device=dev).to(torch.int64)
            pos = torch.arange(T, device=dev, dtype=torch.int64) % 1024
            inv = ops.rotary_inv_freq(10000.0, Rr, dev)
            wq, wk = torch.ones(Rq, device=dev, dtype=bf), torch.ones(Rk, device=dev, dtype=bf)
            add("latent_kv_prep (two norms, rotation, cache write)", "",
                timeit(lambda: ops.latent_kv_prep(proj, Rq, Rk, Rr, wq, wk, 1e-5, inv, pos, slots, cache)),
                T * (2 * Rq + 2 * row) * 2)
            kc = torch.zeros(nblk, hkv, bs, 128, device=dev, dtype=bf)
            vc = torch.zeros_like(kc)
            kk = torch.randn(T, hkv * 128, device=dev, dtype=bf)
            vv = torch.randn(T, hkv * 128, device=dev, dtype=bf)
            add("reshape_and_cache", "latent_kv_prep",
                timeit(lambda: ops.reshape_and_cache(kk, vv, kc, vc, slots)), T * hkv * 128 * 2 * 2 * 2)
            q = torch.randn(T, hq * (D + Rr), device=dev, dtype=bf)
            qa = torch.zeros(T, hq, row, device=dev, dtype=bf)
            add("rotate_pack_queries", "", timeit(lambda: ops.rotate_pack_queries(q, hq, D, Rr, inv, pos, qa, Rk)),
                T * hq * Rr * 4)
            qc, kc2 = torch.randn(T, hq * 128, device=dev, dtype=bf), kk.clone()
            csc = ops.build_cos_sin_cache(128, 1024, 10000.0, dev).float()
            add("rotary_embedding", "rotate_pack_queries",
                timeit(lambda: ops.rotary_embedding(pos, qc, kc2, csc, 128)), T * (hq + hkv) * 128 * 4)
            L = 1024
            nb_seq = L // bs
            sink = torch.zeros(hq, device=dev)
            sc = 1.0 / math.sqrt(D + Rr)
            qlat = torch.randn(T, hq * row, device=dev, dtype=bf)
            if T >= 1024:
                # prompt attention: fresh prompts of 1024 tokens; useful flops count
                # 2 * (key size + value size) per (query row, visible key) pair
                S = T // L
                lcache = torch.randn(S * nb_seq + 1, 1, bs, row, device=dev, dtype=bf)
                tables = torch.arange(S * nb_seq, dtype=torch.int32, device=dev).view(S, nb_seq)
                pairs = S * (L * (L + 1) / 2) * hq
                t = timeit(lambda: ops.latent_attention_rows(
                    qlat, lcache, Rk, tables, i32([i * L for i in range(S)]), i32([L] * S), i32([L] * S), L, sc, hq,
                    sink=sink), 5)
                rows.append({"kernel": f"latent_attention_rows (keys {row}, values {Rk}, {hq} heads share them)",
                             "like": "", "us": round(t * 1e6, 1),
                             "TFLOP_per_s": round(2 * (row + Rk) * pairs / t / 1e12, 1)})
                kcache = torch.randn(S * nb_seq + 1, hkv, bs, 128, device=dev, dtype=bf)
                vcache = torch.randn_like(kcache)
                qh = torch.randn(T, hq, 128, device=dev, dtype=bf)
                tseq = i32([s_ for s_ in range(S) for _ in range(L // 64)])
                tqs = i32([q0 for _ in range(S) for q0 in range(0, L, 64)])
                t = timeit(lambda: ops.paged_attention_prefill(
                    qh, kcache, vcache, tables, i32([i * L for i in range(S + 1)]), i32([L] * S), sc,
                    tile_seq=tseq, tile_qstart=tqs), 5)
                rows.append({"kernel": "paged_attention_prefill (head size 128, Llama path)",
                             "like": "latent_attention_rows", "us": round(t * 1e6, 1),
                             "TFLOP_per_s": round(2 * (128 + 128) * pairs / t / 1e12, 1)})
            else:
                # decode: T sequences with 1024 cached tokens; bytes = every sequence's cache once
                lcache = torch.randn(T * nb_seq + 1, 1, bs, row, device=dev, dtype=bf)
                tables = torch.arange(T * nb_seq, dtype=torch.int32, device=dev).view(T, nb_seq)
                add(f"latent_attention_rows (decode, cache row {row})", "",
                    timeit(lambda: ops.latent_attention_rows(
                        qlat, lcache, Rk, tables, i32(list(range(T))), i32([1] * T), i32([L] * T), 1, sc, hq,
                        sink=sink), 10), T * L * row * 2)
                kcache = torch.randn(T * nb_seq + 1, hkv, bs, 128, device=dev, dtype=bf)
                vcache = torch.randn_like(kcache)
                qh = torch.randn(T, hq, 128, device=dev, dtype=bf)
                add("paged_attention_decode (head size 128, Llama path)", "latent_attention_rows",
                    timeit(lambda: ops.paged_attention_decode(qh, kcache, vcache, tables, i32([L] * T), sc, max_ctx=L), 10),
                    T * L * hkv * 128 * 2 * 2)
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
    if "profile" in args.part:
        # one model only (routed variant): the run to put under a profiler
        for name in sizes:
            print(json.dumps({"bench": "profile", "size": name,
                              "lopovik_routed": engine_run(lopovik_config(name, SIZES[name], True), 16, 1024, 64)}),
                  flush=True)


if __name__ == "__main__":
    main()
