"""A plain, slow float64 statement of the Retuvik decoder, one function per mechanism, written
from the design's equations and sharing no code with the package. ``P`` maps checkpoint tensor
names to float64 tensors, ``cfg`` is the checkpoint's config.json as a dict.

Notation: n tokens, width W; wkv heads of size D (keys and values alike); attention with H query
heads over G key / value heads (query head a reads key / value head a // (H / G)), key size D,
value size E.
"""
import math

import torch


def unit_rms(x, eps):
    """x divided by its root mean square over the last axis, eps inside the root."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def group_norm(x, w, groups, eps):
    """The last axis in ``groups`` equal consecutive parts, each divided by its own root mean
    square; the whole times w."""
    n = x.shape[-1]
    parts = x.reshape(*x.shape[:-1], groups, n // groups)
    return unit_rms(parts, eps).reshape(x.shape) * w


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return math.log1p(math.exp(z))


def xielu(z, p, q):
    """softplus(p) z^2 + z / 2 above zero; (1/2 + softplus(q)) (e^z - 1 - z) + z / 2 at and below."""
    a, b = softplus(p), 0.5 + softplus(q)
    return torch.where(z > 0, a * z * z + 0.5 * z, b * (torch.expm1(torch.clamp(z, max=0.0)) - z) + 0.5 * z)


def shifted(h, mu):
    """h_t + (h_(t-1) - h_t) * mu with h_(-1) = 0."""
    before = torch.cat([torch.zeros_like(h[:1]), h[:-1]])
    return h + (before - h) * mu


def wkv_recurrence(r, k, v, w, u):
    """r, k, v, w [n, heads, D], u [heads, D]. Per head a D x D state S (rows: key channel,
    columns: value channel) that starts at zero:
        o_t[j] = sum_i r_t[i] (S[i, j] + u[i] k_t[i] v_t[j]);   S <- w_t[i] S[i, j] + k_t[i] v_t[j]."""
    n, A, D = r.shape
    out = torch.zeros(n, A, D, dtype=r.dtype)
    for a in range(A):
        S = torch.zeros(D, D, dtype=r.dtype)
        for t in range(n):
            kv = torch.outer(k[t, a], v[t, a])
            out[t, a] = (S + u[a][:, None] * kv).T @ r[t, a]
            S = w[t, a][:, None] * S + kv
    return out


def wkv_mixer(h, P, p, m, eps):
    """Time mixing with a decay that depends on the token: five shifted copies of h feed r, k, v,
    the gate and the decay's low-rank path."""
    n = h.shape[0]
    A, D = m["heads"], m["dim"]
    mix = {s: shifted(h, P[p + "mu." + s]) for s in "rkvgw"}
    r = (mix["r"] @ P[p + "r"].T).reshape(n, A, D)
    k = (mix["k"] @ P[p + "k"].T).reshape(n, A, D)
    v = (mix["v"] @ P[p + "v"].T).reshape(n, A, D)
    gate = silu(mix["g"] @ P[p + "g"].T)
    lw = torch.tanh(mix["w"] @ P[p + "w1"].T) @ P[p + "w2"].T + P[p + "w0"]
    w = torch.exp(-torch.exp(lw)).reshape(n, A, D)
    o = wkv_recurrence(r, k, v, w, P[p + "u"])
    o = unit_rms(o, eps).reshape(n, A * D) * P[p + "norm"] * gate
    return o @ P[p + "o"].T


def head_slopes(H):
    return torch.tensor([2.0 ** (-8.0 * (a + 1) / H) for a in range(H)], dtype=torch.float64)


def attention_mixer(h, P, p, m, eps):
    """Windowed attention without rotation: normed queries and keys (one weight per channel shared
    by the heads), a query factor that grows with the logarithm of the position, unit-RMS values, a
    penalty slope_a (i - j) on the scores, softmax over the last ``mask.size`` positions, and a
    sigmoid gate on the concatenated heads."""
    n = h.shape[0]
    H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = unit_rms((h @ P[p + "q"].T).reshape(n, H, D), eps) * P[p + "q.norm"]
    k = unit_rms((h @ P[p + "k"].T).reshape(n, G, D), eps) * P[p + "k.norm"]
    v = unit_rms((h @ P[p + "v"].T).reshape(n, G, E), eps)
    pos = torch.arange(n)
    qt = m.get("q_temp")
    if qt is not None:
        q = q * (1.0 + qt["coef"] * torch.log(torch.floor((pos + 1) / qt["every"]).double() + 1.0))[:, None, None]
    dist = (pos[:, None] - pos[None, :]).double()
    seen = dist >= 0
    if m.get("mask") is not None:
        seen = seen & (dist < m["mask"]["size"])
    slopes = head_slopes(H)
    out = torch.zeros(n, H, E, dtype=h.dtype)
    for a in range(H):
        g = a // (H // G)
        s = (q[:, a] @ k[:, g].T) * m["scale"] - slopes[a] * dist
        s = s.masked_fill(~seen, float("-inf"))
        out[:, a] = torch.softmax(s, dim=-1) @ v[:, g]
    out = out.reshape(n, H * E) * torch.sigmoid(h @ P[p + "g"].T)
    return out @ P[p + "o"].T


def dense_ff(h, P, p):
    z = h @ P[p + "up"].T + P[p + "up.b"]
    a = P[p + "act"].tolist()
    return xielu(z, a[0], a[1]) @ P[p + "down"].T + P[p + "down.b"]


def route(h, P, p, top):
    """Router logits, the ``top`` largest per token, softmax over those alone."""
    z = h @ P[p + "router"].T + P[p + "router.b"]
    val, idx = torch.topk(z, top, dim=-1)
    return idx, torch.softmax(val, dim=-1)


def moe_ff(h, P, p, mlp):
    idx, wt = route(h, P, p, mlp["router"]["top"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, c in zip(idx[t].tolist(), wt[t]):
            q = f"{p}e{e}."
            out[t] += c * ((silu(h[t] @ P[q + "gate"].T) * (h[t] @ P[q + "up"].T)) @ P[q + "down"].T)
    return out


def layer_runs(cfg):
    """(checkpoint layer, pass number if the run opens a pass of the loop else None) in run order."""
    n = len(cfg["layers"])
    lp = cfg.get("loop")
    if lp is None:
        return [(i, None) for i in range(n)]
    runs = [(i, None) for i in range(lp["start"])]
    for t in range(lp["times"]):
        runs += [(i, t if i == lp["start"] else None) for i in range(lp["start"], lp["stop"])]
    return runs + [(i, None) for i in range(lp["stop"], n)]


def forward(cfg, P, tokens, keep=None):
    """Logits [n, vocab] of one sequence from position 0; ``keep`` receives the residual stream
    after every layer run."""
    eps, groups = cfg["norm"]["eps"], cfg["norm"]["groups"]
    e0 = P["embed"][torch.as_tensor(tokens)] * cfg["embedding"]["scale"]
    x = e0.clone()
    for i, opens in layer_runs(cfg):
        L, p = cfg["layers"][i], f"l{i}."
        if opens is not None:
            if opens > 0:
                x = x + e0
            x = x + P["loop.step"][opens]
        h = group_norm(x, P[p + "norm1"], groups, eps)
        if L["type"] == "wkv":
            x = x + wkv_mixer(h, P, p + "mix.", L["mixer"], eps)
        elif L["type"] == "attention":
            x = x + attention_mixer(h, P, p + "mix.", L["mixer"], eps)
        else:
            raise ValueError(L["type"])
        if L.get("mlp") is not None:
            h = group_norm(x, P[p + "norm2"], groups, eps)
            x = x + (dense_ff(h, P, p + "mlp.") if L["mlp"]["kind"] == "dense" else moe_ff(h, P, p + "mlp.", L["mlp"]))
        if keep is not None:
            keep.append(x.clone())
    return group_norm(x, P["final.norm"], groups, eps) @ P["head"].T
