"""Slow float64 implementation of the Lopovik design, one function per
mechanism, written from the design's equations.  It imports nothing from the
package: the tests compare the engine against it.

Weights are a dict name -> float64 tensor; `cfg` is the parsed config.json
(a dict).  Sequences are processed whole, one at a time, with explicit
loops where the loop is the definition.
"""

from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

F64 = torch.float64


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def offset_norm(x, w, eps):
    """RMS norm whose stored weight is an offset from one."""
    return rms(x, eps) * (1.0 + w)


def plain_norm(x, w, eps):
    return rms(x, eps) * w


def token_shift(h: torch.Tensor, mu: torch.Tensor) -> torch.Tensor:
    """h_t <- h_t + (h_{t-1} - h_t) * mu with h_{-1} = 0; h is [T, W]."""
    prev = torch.zeros_like(h)
    prev[1:] = h[:-1]
    return h + (prev - h) * mu


def rotate_interleaved(v: torch.Tensor, pos: torch.Tensor, base: float, dims: int) -> torch.Tensor:
    """Rotate pairs (2i, 2i+1), i < dims/2, of the last axis by pos * base^(-2i/dims);
    v is [T, ..., n] with n >= dims, pos [T]."""
    out = v.clone()
    half = dims // 2
    for i in range(half):
        f = base ** (-2.0 * i / dims)
        a = pos.to(F64) * f
        shape = [-1] + [1] * (v.dim() - 2)
        c, s = torch.cos(a).view(shape), torch.sin(a).view(shape)
        u, w = v[..., 2 * i], v[..., 2 * i + 1]
        out[..., 2 * i] = u * c - w * s
        out[..., 2 * i + 1] = w * c + u * s
    return out


def sink_softmax_attention(q, k, v, scale: float, sink: torch.Tensor) -> torch.Tensor:
    """Causal attention of one sequence with a per-head sink in the softmax
    denominator.  q, k [T, H, D]; v [T, H, Dv]; sink [H].  Returns [T, H, Dv]."""
    T, H, _ = q.shape
    out = torch.zeros(T, H, v.shape[-1], dtype=F64)
    for h in range(H):
        for i in range(T):
            s = (k[: i + 1, h] @ q[i, h]) * scale
            m = max(float(s.max()), float(sink[h]))
            e = torch.exp(s - m)
            den = e.sum() + math.exp(float(sink[h]) - m)
            out[i, h] = (e / den) @ v[: i + 1, h]
    return out


def latent_attention(h, W: Dict[str, torch.Tensor], p: str, m: dict, eps: float) -> torch.Tensor:
    """The latent-attention mixer of one sequence; h [T, width] is its
    (shifted) input, `p` the tensor prefix ('l3.mix.'), `m` the mixer's config."""
    T = h.shape[0]
    H, D, R, Dv, Rk = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    pos = torch.arange(T)
    cq = plain_norm(h @ W[p + "dq"].T, W[p + "dq.norm"], eps)
    q = (cq @ W[p + "uq"].T).view(T, H, D + R)
    dkv = h @ W[p + "dkv"].T
    c = plain_norm(dkv[:, :Rk], W[p + "dkv.norm"], eps)
    base, dims = m["rot"]["base"], m["rot"]["dims"]
    k_rot = rotate_interleaved(dkv[:, Rk:], pos, base, dims)  # [T, R], shared by the heads
    q_rot = rotate_interleaved(q[..., D:], pos, base, dims)
    k_un = (c @ W[p + "uk"].T).view(T, H, D)
    val = (c @ W[p + "uv"].T).view(T, H, Dv)
    qf = torch.cat([q[..., :D], q_rot], dim=-1)
    kf = torch.cat([k_un, k_rot[:, None, :].expand(T, H, R)], dim=-1)
    o = sink_softmax_attention(qf, kf, val, m["scale"], W[p + "sink"])
    o = o.reshape(T, H * Dv) * torch.sigmoid(h @ W[p + "g"].T)
    return o @ W[p + "o"].T


def dense_ff(h, W, p: str) -> torch.Tensor:
    """down(relu(up h)^2)."""
    return torch.relu(h @ W[p + "up"].T).pow(2) @ W[p + "down"].T


def moe_ff(h, W, p: str, mlp: dict) -> torch.Tensor:
    """Sigmoid-scored experts; the chosen scores scale each expert's INPUT and
    are not renormalised."""
    E, top = mlp["router"]["experts"], mlp["router"]["top"]
    s = torch.sigmoid(h @ W[p + "router"].T)  # [T, E]
    out = torch.zeros(h.shape[0], W[p + "e0.down"].shape[0], dtype=F64)
    for t in range(h.shape[0]):
        chosen = torch.topk(s[t], top).indices.tolist()
        for e in chosen:
            x = s[t, e] * h[t]
            g = x @ W[f"{p}e{e}.gate"].T
            u = x @ W[f"{p}e{e}.up"].T
            out[t] += (g * torch.sigmoid(g) * u) @ W[f"{p}e{e}.down"].T
    return out


def layer_runs(cfg: dict) -> List[dict]:
    """The order in which layers run: [{'layer': i, 'enter': bool}], 'enter'
    marking the first layer of a pass of the loop."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [{"layer": i, "enter": False} for i in range(n)]
    a, b, times = loop["start"], loop["stop"], loop["times"]
    runs = [{"layer": i, "enter": False} for i in range(a)]
    for _ in range(times):
        for i in range(a, b):
            runs.append({"layer": i, "enter": i == a})
    runs += [{"layer": i, "enter": False} for i in range(b, n)]
    return runs


def forward(cfg: dict, W: Dict[str, torch.Tensor], tokens: List[int], residuals: Optional[list] = None):
    """Logits [T, vocab] of one whole sequence (float64)."""
    W = {k: v.to(F64) for k, v in W.items()}
    eps = cfg["norm"]["eps"]
    x = W["embed"][torch.tensor(tokens)]
    x0 = x.clone()
    for run in layer_runs(cfg):
        i = run["layer"]
        spec = cfg["layers"][i]
        p = f"l{i}."
        if run["enter"]:
            x = torch.cat([x, x0], dim=-1) @ W["loop.in"].T
        h = token_shift(offset_norm(x, W[p + "norm1"], eps), W[p + "shift"])
        assert spec["type"] == "latent_attention"
        y = latent_attention(h, W, p + "mix.", spec["mixer"], eps)
        mlp = spec.get("mlp")
        if mlp is not None:
            h2 = offset_norm(x, W[p + "norm2"], eps)
            if mlp["kind"] == "dense":
                y = y + dense_ff(h2, W, p + "mlp.")
            else:
                y = y + moe_ff(h2, W, p + "mlp.", mlp)
        x = x + y
        if residuals is not None:
            residuals.append(x.clone())
    return offset_norm(x, W["final.norm"], eps) @ W["embed"].T
