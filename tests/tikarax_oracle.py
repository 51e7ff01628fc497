"""Slow float64 oracle for the Tikarax design, one function per mechanism.

Written from the equations alone and kept free of any import from the
package: the tests compare the engine (kernels, caches, scheduler) against
these loops.  Everything takes and returns float64 torch tensors; weights
come as a dict in checkpoint naming.

Notation: a row vector a of length n split into g consecutive parts a_1..a_g;
rms(a_i) = sqrt(mean(a_i^2) + eps).
"""

import math

import torch

F64 = torch.float64


def o_group_norm(a, w, groups, eps):
    """a [T, n] -> concat_i(a_i / rms(a_i)) * w."""
    T, n = a.shape
    part = n // groups
    out = torch.empty_like(a)
    for t in range(T):
        for i in range(groups):
            seg = a[t, i * part : (i + 1) * part]
            out[t, i * part : (i + 1) * part] = seg / math.sqrt(float((seg * seg).mean()) + eps)
    return out * w


def o_softplus(x):
    return math.log1p(math.exp(-abs(x))) + max(x, 0.0)


def o_xielu(a, p, q):
    """a > 0: sp(p) a^2 + a/2;  a <= 0: (1/2 + sp(q)) (e^a - 1 - a) + a/2."""
    cp, cn = o_softplus(p), 0.5 + o_softplus(q)
    out = torch.empty_like(a)
    flat, oflat = a.reshape(-1), out.reshape(-1)
    for i in range(flat.numel()):
        v = float(flat[i])
        oflat[i] = cp * v * v + v / 2 if v > 0 else cn * (math.expm1(v) - v) + v / 2
    return out


def o_query_temperature(pos, coef, every):
    return 1.0 + coef * math.log(math.floor((pos + 1) / every) + 1.0)


def o_attention(q, k, v, heads, kv_heads, scale, coef=0.0, every=1.0, gate=None, start=0):
    """Causal softmax attention for one sequence.  q [T, heads*dk] are the
    queries of positions start..start+T-1; k [L, kv_heads*dk], v [L,
    kv_heads*dv] hold positions 0..L-1 with L = start+T.  Query head a reads
    key/value head a // (heads / kv_heads)."""
    T = q.shape[0]
    L = k.shape[0]
    dk = q.shape[1] // heads
    dv = v.shape[1] // kv_heads
    rep = heads // kv_heads
    out = torch.zeros(T, heads * dv, dtype=F64)
    for t in range(T):
        p = start + t
        tau = o_query_temperature(p, coef, every) if coef != 0.0 else 1.0
        for a in range(heads):
            b = a // rep
            qa = q[t, a * dk : (a + 1) * dk] * tau
            s = torch.empty(p + 1, dtype=F64)
            for j in range(p + 1):
                s[j] = float(qa @ k[j, b * dk : (b + 1) * dk]) * scale
            wgt = torch.exp(s - s.max())
            wgt = wgt / wgt.sum()
            out[t, a * dv : (a + 1) * dv] = wgt @ v[: p + 1, b * dv : (b + 1) * dv]
    if gate is not None:
        out = out * torch.sigmoid(gate)
    return out


def o_mingru(zpre, u, state):
    """S_t = (1 - z_t) S_{t-1} + z_t c_t with z = sigmoid(zpre) and
    c = u + 1/2 (u >= 0) or sigmoid(u) (u < 0).  Returns (all S_t, last S)."""
    T, W = zpre.shape
    S = state.clone()
    out = torch.empty(T, W, dtype=F64)
    for t in range(T):
        z = torch.sigmoid(zpre[t])
        c = torch.where(u[t] >= 0, u[t] + 0.5, torch.sigmoid(u[t]))
        S = (1 - z) * S + z * c
        out[t] = S
    return out, S


def o_forward(cfg, W, tokens, residuals=None):
    """Whole-sequence forward from position 0; returns logits [T, vocab].
    cfg is the config.json dict, W the checkpoint tensors (any float dtype)."""
    eps, groups = cfg["norm"]["eps"], cfg["norm"]["groups"]

    def g(name):
        return W[name].to(F64)

    x = o_group_norm(g("embed")[torch.tensor(tokens)], g("embed.norm"), groups, eps)
    for i, layer in enumerate(cfg["layers"]):
        pre = "l%d." % i
        m = layer["mixer"]
        h = o_group_norm(x, g(pre + "norm1"), groups, eps)
        if layer["type"] == "attention":
            q = h @ g(pre + "mix.q").T + g(pre + "mix.q.b")
            k = h @ g(pre + "mix.k").T + g(pre + "mix.k.b")
            v = h @ g(pre + "mix.v").T + g(pre + "mix.v.b")
            qt = m.get("q_temp") or {"coef": 0.0, "every": 1.0}
            o = o_attention(
                q, k, v, m["heads"], m["kv_heads"], m["scale"], qt["coef"], qt["every"],
                gate=h @ g(pre + "mix.g").T,
            )
            y = o @ g(pre + "mix.o").T
        else:
            zpre = h @ g(pre + "mix.z").T + g(pre + "mix.z.b")
            u = h @ g(pre + "mix.x").T + g(pre + "mix.x.b")
            S, _ = o_mingru(zpre, u, torch.zeros(m["width"], dtype=F64))
            gg = h @ g(pre + "mix.g").T
            y = (S * gg * torch.sigmoid(gg)) @ g(pre + "mix.o").T
        x = x + o_group_norm(y, g(pre + "norm1b"), groups, eps)
        if layer["mlp"] is not None:
            h = o_group_norm(x, g(pre + "norm2"), groups, eps)
            act = g(pre + "mlp.act")
            y = o_xielu(h @ g(pre + "mlp.up").T, float(act[0]), float(act[1])) @ g(pre + "mlp.down").T
            x = x + o_group_norm(y, g(pre + "norm2b"), groups, eps)
        if residuals is not None:
            residuals.append(x.clone())
    return o_group_norm(x, g("final.norm"), groups, eps) @ g("head").T
