"""Lopovik: a decoder-only stack of parallel layers over latent attention.

config.json lists the layers; every layer adds both of its branches to the
residual at once,

    x <- x + mixer(shift(norm1(x))) + ff(norm2(x))

with RMS norms whose stored weights are offsets from one.  `shift` blends the
mixer's input with the previous token's, h + (h_prev - h) * mu, so every
layer keeps one fp32 row per live sequence beside its paged cache.  The mixer
is latent attention (low-rank key/value latent, shared rotated key part,
softmax sink, sigmoid output gate); the feed-forward is a squared-ReLU
two-matrix block or sigmoid-routed experts whose scores scale the expert
input; a layer may have none.

A span of layers can be looped: it runs `times` times in a row with the same
weights, and before the first layer of every pass the residual is re-mixed
with the embedding output, x <- W_in [x ; x0].  Each run of a layer owns a
cache and a shift state, so the engine sees one cache entry per layer RUN.

The output head is the embedding table (tied) after a final offset norm.
The residual stream is fp32 in every mode.

Execution on the engine's flat batch, per layer run: one kernel for both
norms and the shift, the mixer (fused input GEMM, latent prep kernel, query
GEMMs, rotation, paged attention, value GEMM, gate, output GEMM), the
feed-forward.  Both branch outputs join the residual inside the NEXT layer's
norm kernel (a kernel of its own only before a pass of the loop and before
the final norm).
"""

from __future__ import annotations

import os
from typing import List, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from .. import ops
from .config import LayerSpec, ModelConfig
from .hybrid_blocks import LatentAttention, ReluSquaredMLP, ScoredExpertsMLP, _param

MIXERS = ("latent_attention",)
FF_KINDS = ("dense", "moe")


def config_from_json(raw: dict, path: str = "") -> ModelConfig:
    specs: List[LayerSpec] = []
    for i, entry in enumerate(raw["layers"]):
        t = entry["type"]
        if t not in MIXERS:
            raise ValueError(f"layer {i}: unknown mixer type {t!r}")
        mlp = entry.get("mlp")
        if mlp is not None and mlp.get("kind") not in FF_KINDS:
            raise ValueError(f"layer {i}: unknown feed-forward kind {mlp.get('kind')!r}")
        specs.append(
            LayerSpec(type=t, mixer=dict(entry["mixer"]), mlp=None if mlp is None else dict(mlp), shift=True)
        )
    loop = raw.get("loop")
    layer_loop = None
    if loop:
        a, b, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
        if not (0 <= a < b <= len(specs)) or times < 1:
            raise ValueError(f"loop {loop!r} does not fit {len(specs)} layers")
        layer_loop = (a, b, times)
    return ModelConfig(
        name=os.path.basename(os.path.normpath(path)) or "lopovik",
        architecture="lopovik",
        vocab_size=int(raw["vocab"]),
        hidden_size=int(raw["width"]),
        num_layers=len(specs),
        rms_norm_eps=float(raw["norm"]["eps"]),
        layer_specs=specs,
        layer_loop=layer_loop,
        tie_word_embeddings=True,
        weights_path=path,
        # rotation angles are computed from the position itself: no table
        # bounds the context
        max_position_embeddings=1 << 30,
    )


def make_config(
    name: str, vocab: int, width: int, layers: List[dict], eps: float = 1e-5,
    loop: Optional[dict] = None,
) -> ModelConfig:
    """A random-init config from the same fields config.json carries."""
    raw = {"vocab": vocab, "width": width, "layers": layers, "norm": {"eps": eps}}
    if loop:
        raw["loop"] = loop
    cfg = config_from_json(raw)
    cfg.name = name
    return cfg


class ParallelLayer(nn.Module):
    def __init__(self, spec: LayerSpec, hidden: int, eps: float, device, dtype) -> None:
        super().__init__()
        m = spec.mixer
        self.mixer = LatentAttention(
            hidden, m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["q_rank"], m["kv_rank"],
            m["scale"], m["rot"]["base"], m["rot"]["dims"], eps, sink=True, out_gate=True,
            device=device, dtype=dtype,
        )
        # norm weights are stored as offsets from one
        self.norm1 = _param((hidden,), device, dtype, None)
        self.shift = _param((hidden,), device, dtype, 0.5)
        self.mlp = None
        self.norm2 = None
        if spec.mlp is not None:
            self.norm2 = _param((hidden,), device, dtype, None)
            if spec.mlp["kind"] == "dense":
                self.mlp = ReluSquaredMLP(hidden, spec.mlp["ff"], device=device, dtype=dtype)
            else:
                self.mlp = ScoredExpertsMLP(
                    hidden, spec.mlp["expert"]["ff"], spec.mlp["router"]["experts"],
                    spec.mlp["router"]["top"], device=device, dtype=dtype,
                )


class LopovikForCausalLM(nn.Module):
    # the runner builds per-token sequence tables and per-sequence segments
    needs_seq_tables = True
    # no adapter hooks in the mixers: base model only
    supports_lora = False
    # single-token steps have static shapes and no host round trip
    supports_decode_graphs = True

    def __init__(self, cfg: ModelConfig, device="cpu", dtype=torch.bfloat16, tp=None) -> None:
        super().__init__()
        if tp is not None and tp.world_size > 1:
            raise NotImplementedError("Lopovik runs on one GPU per engine (no tensor parallelism)")
        assert cfg.layer_specs, "Lopovik needs per-layer specs"
        self.cfg = cfg
        self.device_ = torch.device(device)
        self.dtype_ = dtype
        H, V = cfg.hidden_size, cfg.vocab_size
        self.embed = _param((V, H), device, dtype, 1.0)
        self.final_norm = _param((H,), device, dtype, None)
        self.layers = nn.ModuleList(
            [ParallelLayer(s, H, cfg.rms_norm_eps, device, dtype) for s in cfg.layer_specs]
        )
        self.run_order = cfg.layer_run_order()
        # runs that open a pass of the loop re-mix the residual with the
        # embedding output first
        self.pass_starts = set()
        self.loop_in = None
        if cfg.layer_loop is not None:
            a, b, times = cfg.layer_loop
            self.pass_starts = {a + k * (b - a) for k in range(times)}
            self.loop_in = _param((H, 2 * H), device, dtype, 1.0 / (2 * H) ** 0.5)
        # attention addresses the batch per segment: no per-head query tiles
        self.needs_prefill_tiles = False
        # test/debug hook: when a list, forward() appends the fp32 residual
        # stream after every layer run
        self.capture_residuals: Optional[list] = None

    def decode_attention_shape(self):
        return None  # no layer uses the split paged-decode kernel

    def cache_specs(self) -> List[list]:
        """One entry per layer RUN: the latent cache and the shift state."""
        H = self.cfg.hidden_size
        return [
            [self.layers[i].mixer.cache_spec(), {"kind": "state", "width": H}]
            for i in self.run_order
        ]

    def load_weights(self, tensors) -> None:
        used = set()

        def get(name: str) -> torch.Tensor:
            if name not in tensors:
                raise KeyError(f"checkpoint has no tensor {name!r}")
            used.add(name)
            return tensors[name].to(device=self.device_, dtype=self.dtype_)

        with torch.no_grad():
            self.embed.copy_(get("embed"))
            self.final_norm.copy_(get("final.norm"))
            if self.loop_in is not None:
                self.loop_in.copy_(get("loop.in"))
            for i, layer in enumerate(self.layers):
                p = f"l{i}."
                layer.norm1.copy_(get(p + "norm1"))
                layer.shift.copy_(get(p + "shift"))
                layer.mixer.load(get, p + "mix.")
                if layer.mlp is not None:
                    layer.norm2.copy_(get(p + "norm2"))
                    layer.mlp.load(get, p + "mlp.")
        extra = sorted(set(tensors) - used)
        if extra:
            raise ValueError(f"checkpoint tensors the model does not know: {extra[:8]}")

    def forward(self, input_ids, positions, kv_caches, meta) -> torch.Tensor:
        eps = self.cfg.rms_norm_eps
        x0 = self.embed.index_select(0, input_ids).float()  # the embedding output, fp32
        x = x0
        # branch outputs of the layer before, not yet in the residual: the
        # next layer's norm kernel adds them on its way in
        pending = None
        for run, li in enumerate(self.run_order):
            layer = self.layers[li]
            if run in self.pass_starts:
                if pending is not None:
                    x = ops.residual_add(x.clone() if x is x0 else x, *pending)
                    pending = None
                x = F.linear(torch.cat([x, x0], dim=-1).to(self.dtype_), self.loop_in).float()
            lat_cache, shift_state = kv_caches[run]
            h_mix, h_ff, x = ops.offset_norm_shift(
                x, layer.norm1, layer.norm2, layer.shift, shift_state, meta.tok_seq,
                meta.seg_start, meta.seg_len, meta.seg_slot, meta.seg_fresh, eps,
                *(pending or ()),
            )
            y = layer.mixer(h_mix, positions, (lat_cache,), meta)
            f = layer.mlp(h_ff, meta) if layer.mlp is not None else None
            pending = (y, f)
            if self.capture_residuals is not None:
                x = ops.residual_add(x.clone() if x is x0 else x, y, f)
                pending = None
                self.capture_residuals.append(x.clone())
        if pending is not None:
            x = ops.residual_add(x.clone() if x is x0 else x, *pending)
        return ops.offset_rms_norm(x, self.final_norm, eps)

    def compute_logits(self, hidden: torch.Tensor, indices: torch.Tensor) -> torch.Tensor:
        return (hidden[indices] @ self.embed.t()).float()
