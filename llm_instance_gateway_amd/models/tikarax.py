"""Tikarax: a hybrid decoder-only stack.

config.json lists the layers; each has a sequence mixer — gated attention
with a logarithmic query temperature and no rotation, or a minGRU
recurrence — and an optional xIELU feed-forward.  Every sub-layer is
sandwiched between two grouped RMS norms:

    x <- x + norm_b(mixer(norm_a(x)));   x <- x + norm_d(ff(norm_c(x)))

The embedding is normalised once, the residual stream x is fp32 throughout
(whatever the activation dtype), and a final norm precedes the output head.

Execution on the engine's flat batch: per layer one fused-input GEMM, the
mixer kernel, one output GEMM, then ONE norm kernel that applies the
sub-layer's output norm, adds into the residual and produces the next
sub-layer's normalised input (ops.post_add_pre_norm).
"""

from __future__ import annotations

import os
from typing import List, Optional

import torch
import torch.nn as nn

from .. import ops
from .config import LayerSpec, ModelConfig
from .hybrid_blocks import GatedAttention, MinGRU, XieluMLP, _param


def config_from_json(raw: dict, path: str = "") -> ModelConfig:
    specs: List[LayerSpec] = []
    for i, entry in enumerate(raw["layers"]):
        t = entry["type"]
        if t not in ("attention", "mingru"):
            raise ValueError(f"layer {i}: unknown mixer type {t!r}")
        mlp = entry.get("mlp")
        if mlp is not None and mlp.get("kind", "dense") != "dense":
            raise ValueError(f"layer {i}: unknown feed-forward kind {mlp.get('kind')!r}")
        specs.append(LayerSpec(type=t, mixer=dict(entry["mixer"]), mlp=None if mlp is None else dict(mlp)))
    return ModelConfig(
        name=os.path.basename(os.path.normpath(path)) or "tikarax",
        architecture="tikarax",
        vocab_size=int(raw["vocab"]),
        hidden_size=int(raw["width"]),
        num_layers=len(specs),
        rms_norm_eps=float(raw["norm"]["eps"]),
        norm_groups=int(raw["norm"].get("groups", 1)),
        layer_specs=specs,
        weights_path=path,
        # no positional table bounds the context: positions only enter
        # through the query temperature
        max_position_embeddings=1 << 30,
    )


def make_config(
    name: str, vocab: int, width: int, layers: List[dict], eps: float = 1e-5, groups: int = 1
) -> ModelConfig:
    """A random-init config from the same fields config.json carries."""
    cfg = config_from_json(
        {"vocab": vocab, "width": width, "layers": layers, "norm": {"eps": eps, "groups": groups}}
    )
    cfg.name = name
    return cfg


class HybridLayer(nn.Module):
    def __init__(self, spec: LayerSpec, hidden: int, device, dtype) -> None:
        super().__init__()
        m = spec.mixer
        if spec.type == "attention":
            qt = m.get("q_temp") or {}
            self.mixer = GatedAttention(
                hidden, m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["scale"],
                temp_coef=qt.get("coef", 0.0), temp_every=qt.get("every", 1.0),
                out_gate=True, device=device, dtype=dtype,
            )
        else:
            self.mixer = MinGRU(hidden, m["width"], device=device, dtype=dtype)
        self.norm1 = _param((hidden,), device, dtype, None)
        self.norm1b = _param((hidden,), device, dtype, None)
        self.mlp: Optional[XieluMLP] = None
        if spec.mlp is not None:
            self.mlp = XieluMLP(hidden, spec.mlp["ff"], device=device, dtype=dtype)
            self.norm2 = _param((hidden,), device, dtype, None)
            self.norm2b = _param((hidden,), device, dtype, None)
        with torch.no_grad():
            for n in ("norm1", "norm1b", "norm2", "norm2b"):
                if hasattr(self, n):
                    getattr(self, n).fill_(1.0)


class TikaraxForCausalLM(nn.Module):
    # the runner builds per-token sequence tables and per-sequence segments
    needs_seq_tables = True
    # no adapter hooks in the mixers: base model only
    supports_lora = False
    # decode-only steps replay hipGraphs (one-token segments, static tables)
    supports_decode_graphs = True

    def __init__(self, cfg: ModelConfig, device="cpu", dtype=torch.bfloat16, tp=None) -> None:
        super().__init__()
        if tp is not None and tp.world_size > 1:
            raise NotImplementedError("Tikarax runs on one GPU per engine (no tensor parallelism)")
        assert cfg.layer_specs, "Tikarax needs per-layer specs"
        self.cfg = cfg
        self.device_ = torch.device(device)
        self.dtype_ = dtype
        H, V = cfg.hidden_size, cfg.vocab_size
        assert H % cfg.norm_groups == 0
        self.embed = _param((V, H), device, dtype, 1.0)
        self.embed_norm = _param((H,), device, dtype, None)
        self.final_norm = _param((H,), device, dtype, None)
        self.head = _param((V, H), device, dtype, 1.0 / (H ** 0.5))
        with torch.no_grad():
            self.embed_norm.fill_(1.0)
            self.final_norm.fill_(1.0)
        self.layers = nn.ModuleList(
            [HybridLayer(s, H, device, dtype) for s in cfg.layer_specs]
        )
        # attention layers whose prompt rows run an MFMA prefill kernel need
        # the runner's 64-row query tiles
        on_gpu = self.device_.type == "cuda"
        self.needs_prefill_tiles = any(
            s.type == "attention"
            and (
                ops.mfma_attention_supported(
                    dtype, s.mixer["dim"], s.mixer["vdim"], on_gpu,
                    s.mixer["heads"] // s.mixer["kv_heads"],
                )
                or ops.tiled_prefill_supported(dtype, s.mixer["dim"], s.mixer["vdim"], on_gpu)
            )
            for s in cfg.layer_specs
        )
        # test/debug hook: when a list, forward() appends the fp32 residual
        # stream after every layer
        self.capture_residuals: Optional[list] = None

    def decode_attention_shape(self):
        """(q heads, kv heads, head size) for sizing the split-decode scratch:
        the largest among layers on the MFMA path, None if there is none."""
        best = None
        for layer in self.layers:
            m = layer.mixer
            if isinstance(m, GatedAttention) and ops.mfma_attention_supported(
                self.dtype_, m.dim, m.vdim, self.device_.type == "cuda", m.heads // m.kv_heads
            ):
                cand = (m.heads, m.kv_heads, m.dim)
                if best is None or cand[0] * cand[2] > best[0] * best[2]:
                    best = cand
        return best

    def cache_specs(self) -> List[dict]:
        return [layer.mixer.cache_spec() for layer in self.layers]

    def load_weights(self, tensors) -> None:
        used = set()

        def get(name: str) -> torch.Tensor:
            if name not in tensors:
                raise KeyError(f"checkpoint has no tensor {name!r}")
            used.add(name)
            return tensors[name].to(device=self.device_, dtype=self.dtype_)

        with torch.no_grad():
            self.embed.copy_(get("embed"))
            self.embed_norm.copy_(get("embed.norm"))
            self.final_norm.copy_(get("final.norm"))
            self.head.copy_(get("head"))
            for i, layer in enumerate(self.layers):
                p = f"l{i}."
                layer.norm1.copy_(get(p + "norm1"))
                layer.norm1b.copy_(get(p + "norm1b"))
                layer.mixer.load(get, p + "mix.")
                if layer.mlp is not None:
                    layer.norm2.copy_(get(p + "norm2"))
                    layer.norm2b.copy_(get(p + "norm2b"))
                    layer.mlp.load(get, p + "mlp.")
        extra = sorted(set(tensors) - used)
        if extra:
            raise ValueError(f"checkpoint tensors the model does not know: {extra[:8]}")

    def forward(self, input_ids, positions, kv_caches, meta) -> torch.Tensor:
        eps, groups = self.cfg.rms_norm_eps, self.cfg.norm_groups
        x = ops.embed_group_norm(input_ids, self.embed, self.embed_norm, eps, groups)
        h = ops.group_norm(x, self.layers[0].norm1, eps, groups)
        n = len(self.layers)
        for i, layer in enumerate(self.layers):
            nxt = self.layers[i + 1].norm1 if i + 1 < n else self.final_norm
            y = layer.mixer(h, positions, kv_caches[i], meta)
            if layer.mlp is not None:
                h = ops.post_add_pre_norm(x, y, layer.norm1b, layer.norm2, eps, groups)
                y = layer.mlp(h)
                h = ops.post_add_pre_norm(x, y, layer.norm2b, nxt, eps, groups)
            else:
                h = ops.post_add_pre_norm(x, y, layer.norm1b, nxt, eps, groups)
            if self.capture_residuals is not None:
                self.capture_residuals.append(x.clone())
        return h  # final-normed hidden states

    def compute_logits(self, hidden: torch.Tensor, indices: torch.Tensor) -> torch.Tensor:
        return (hidden[indices] @ self.head.t()).float()
