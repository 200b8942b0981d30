"""A plain, slow float64 statement of the Ledinex decoder, one function per mechanism, written
from the design's equations and sharing no code with the package. ``P`` maps checkpoint tensor
names to float64 tensors, ``cfg`` is the checkpoint's config.json as a dict.

Notation: n tokens, width W; attention with H query heads over G key / value heads (query head a
reads key / value head a // (H / G)), key size D, value size E; recurrences keep a D x E state per
head (rows: key channel, columns: value channel) that starts at zero.
"""
import math

import torch


def unit_rms(x, eps):
    """x divided by its root mean square over the last axis, eps inside the root."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def unit_length(x):
    return x / torch.sqrt((x * x).sum(-1, keepdim=True) + 1e-6)


def one_plus_norm(x, w, eps):
    return unit_rms(x, eps) * (1.0 + w)


def silu(z):
    return z * torch.sigmoid(z)


def input_conv(h, w):
    """h [n, C] plus its causal convolution over time, w [C, taps], the last tap on the current
    token, zeros ahead of the sequence."""
    return h + causal_conv(h, w)


def causal_conv(h, w):
    taps = w.shape[1]
    out = torch.zeros_like(h)
    for j in range(taps):
        back = taps - 1 - j
        out[back:] += h[:h.shape[0] - back] * w[:, j]
    return out


# ---- rotary tables ----------------------------------------------------------------------------------

def rotary_frequencies(rot):
    """(frequencies [dims / 2], magnitude) of a rotary spec: plain base^(-2i / dims); a scaling
    with only ``factor`` divides them all; one with ``original`` / ``fast`` / ``slow`` blends
    divided and plain frequencies along a ramp and enlarges cos and sin."""
    dims, base = int(rot["dims"]), float(rot["base"])
    f = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    sc = rot.get("scaling")
    mag = 1.0
    if sc is not None and "original" in sc:
        factor = float(sc["factor"])

        def turn_dim(turns):
            return dims * math.log(float(sc["original"]) / (2 * math.pi * turns)) / (2 * math.log(base))
        lo = max(math.floor(turn_dim(float(sc["fast"]))), 0)
        hi = min(math.ceil(turn_dim(float(sc["slow"]))), dims - 1)
        out = []
        for i, fi in enumerate(f):
            ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
            out.append(fi / factor * ramp + fi * (1.0 - ramp))
        f = out
        mag = 0.1 * math.log(factor) + 1.0
    elif sc is not None:
        f = [fi / float(sc["factor"]) for fi in f]
    return torch.tensor(f, dtype=torch.float64), mag


def turn_halves(x, pos, freq, mag=1.0):
    """x [n, heads, D]: entry i pairs with entry i + len(freq) on the leading 2 len(freq) entries;
    pair i of the token at position p turns by p * freq[i]. cos and sin are multiplied by mag."""
    r = freq.numel()
    ang = pos.to(torch.float64)[:, None, None] * freq
    c, s = torch.cos(ang) * mag, torch.sin(ang) * mag
    u, v = x[..., :r], x[..., r:2 * r]
    out = x.clone()
    out[..., :r] = u * c - v * s
    out[..., r:2 * r] = v * c + u * s
    return out


# ---- attention --------------------------------------------------------------------------------------

def softmax_attention(h, P, p, m, eps, kind):
    """The left half of a parallel mixer. ``kind`` "parallel": separate values that are turned by
    their position over all E entries and turned back at the reading position, soft-capped scores,
    every earlier key visible. "parallel_2": biased projections, the values are the keys as
    projected, a sliding window."""
    n = h.shape[0]
    H, G, D, E = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    pos = torch.arange(n)
    q, k = h @ P[p + "q"].T, h @ P[p + "k"].T
    if kind == "parallel_2":
        q, k = q + P[p + "q.b"], k + P[p + "k.b"]
        v = k.reshape(n, G, D)
    else:
        v = (h @ P[p + "v"].T).reshape(n, G, E)
    q = (unit_rms(q, eps) * P[p + "q.norm"]).reshape(n, H, D)
    k = (unit_rms(k, eps) * P[p + "k.norm"]).reshape(n, G, D)
    freq, mag = rotary_frequencies(m["rot"])
    q, k = turn_halves(q, pos, freq, mag), turn_halves(k, pos, freq, mag)
    if kind == "parallel":
        vfreq = torch.tensor([float(m["rot"]["base"]) ** (-2.0 * i / E) for i in range(E // 2)], dtype=torch.float64)
        v = turn_halves(v, pos, vfreq)
    cap = m.get("softcap")
    window = m["mask"]["size"] if m.get("mask") is not None else None
    out = torch.zeros(n, H, E, dtype=torch.float64)
    for a in range(H):
        g = a // (H // G)
        s = (q[:, a] @ k[:, g].T) * float(m["scale"])
        if cap is not None:
            s = cap * torch.tanh(s / cap)
        dist = pos[:, None] - pos[None, :]
        seen = dist >= 0
        if window is not None:
            seen = seen & (dist < window)
        s = s.masked_fill(~seen, float("-inf"))
        out[:, a] = torch.softmax(s, -1) @ v[:, g]
    if kind == "parallel":
        out = turn_halves(out, -pos, vfreq)
    return out.reshape(n, H * E) @ P[p + "o"].T


# ---- recurrences ------------------------------------------------------------------------------------

def decayed_sum(q, k, v, decay):
    """S_t = decay S_(t-1) + k_t v_t^T; o_t = S_t^T q_t. q, k [n, D], v [n, E], one head."""
    S = torch.zeros(k.shape[1], v.shape[1], dtype=torch.float64)
    out = []
    for t in range(q.shape[0]):
        S = decay * S + torch.outer(k[t], v[t])
        out.append(S.T @ q[t])
    return torch.stack(out)


def lightning_mixer(h, P, p, m, eps):
    n = h.shape[0]
    A, D = int(m["heads"]), int(m["dim"])
    E = int(m.get("vdim", D))
    q = silu(h @ P[p + "q"].T).reshape(n, A, D)
    k = silu(h @ P[p + "k"].T).reshape(n, A, D)
    v = silu(h @ P[p + "v"].T).reshape(n, A, E)
    o = torch.stack([decayed_sum(q[:, a], k[:, a], v[:, a], float(m["decay"][a])) for a in range(A)], 1)
    o = unit_rms(o.reshape(n, A * E), eps) * P[p + "norm"]
    return (o * torch.sigmoid(h @ P[p + "g"].T)) @ P[p + "o"].T


def removing_sum(r, k, v, w, a):
    """One head; r, k, w, a [n, D], v [n, E]. With u the unit-length key:
    S_t = diag(w_t) S_(t-1) - (a_t * u_t) (u_t^T S_(t-1)) + k_t v_t^T; o_t = S_t^T r_t."""
    S = torch.zeros(k.shape[1], v.shape[1], dtype=torch.float64)
    out = []
    for t in range(r.shape[0]):
        u = unit_length(k[t])
        S = w[t][:, None] * S - torch.outer(a[t] * u, u @ S) + torch.outer(k[t], v[t])
        out.append(S.T @ r[t])
    return torch.stack(out)


def removal_mixer(h, P, p, m, eps):
    n = h.shape[0]
    A, D = int(m["heads"]), int(m["dim"])
    r, k, v = ((h @ P[p + x].T).reshape(n, A, D) for x in "rkv")
    w = torch.exp(-math.exp(-0.5) * torch.sigmoid(torch.tanh(h @ P[p + "w1"].T) @ P[p + "w2"].T + P[p + "w0"]))
    a = torch.sigmoid(h @ P[p + "a"].T + P[p + "a.b"])
    w, a = w.reshape(n, A, D), a.reshape(n, A, D)
    o = torch.stack([removing_sum(r[:, i], k[:, i], v[:, i], w[:, i], a[:, i]) for i in range(A)], 1)
    o = unit_rms(o, eps).reshape(n, A * D) * P[p + "norm"]
    return (o * torch.sigmoid(h @ P[p + "g"].T)) @ P[p + "o"].T


def corrected_sum(q, k, v, beta, g):
    """One head; q, k [n, D], v [n, E], beta, g [n]: S <- g_t S; u = beta_t (v_t - S^T k_t);
    S <- S + k_t u^T; o_t = S^T q_t."""
    S = torch.zeros(k.shape[1], v.shape[1], dtype=torch.float64)
    out = []
    for t in range(q.shape[0]):
        S = g[t] * S
        u = beta[t] * (v[t] - S.T @ k[t])
        S = S + torch.outer(k[t], u)
        out.append(S.T @ q[t])
    return torch.stack(out)


def delta_mixer(h, P, p, m, eps):
    n = h.shape[0]
    A, G, D, E = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q = silu(causal_conv(h @ P[p + "q"].T, P[p + "q.conv"])).reshape(n, G, D)
    k = silu(causal_conv(h @ P[p + "k"].T, P[p + "k.conv"])).reshape(n, G, D)
    v = silu(causal_conv(h @ P[p + "v"].T, P[p + "v.conv"])).reshape(n, A, E)
    q, k = unit_length(q) * D ** -0.5, unit_length(k)
    beta = torch.sigmoid(h @ P[p + "b"].T)
    g = torch.exp(-torch.exp(P[p + "A_log"]) * torch.nn.functional.softplus(h @ P[p + "a"].T + P[p + "dt_bias"]))
    o = torch.stack([corrected_sum(q[:, i // (A // G)], k[:, i // (A // G)], v[:, i], beta[:, i], g[:, i])
                     for i in range(A)], 1)
    o = unit_rms(o, eps) * P[p + "norm"]
    return (o.reshape(n, A * E) * silu(h @ P[p + "g"].T)) @ P[p + "o"].T


# ---- feed-forward -----------------------------------------------------------------------------------

def squared_relu_ff(h, up, down):
    return torch.relu(h @ up.T) ** 2 @ down.T


def moe_ff(h, P, p, mlp):
    E, top = int(mlp["router"]["experts"]), int(mlp["router"]["top"])
    s = torch.softmax(h @ P[p + "router"].T, -1)
    val, idx = torch.topk(s, top, dim=-1)
    wt = val / (val.sum(-1, keepdim=True) + 1e-20)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for j in range(top):
            e = int(idx[t, j])
            out[t] += wt[t, j] * squared_relu_ff(h[t:t + 1], P[p + f"e{e}.up"], P[p + f"e{e}.down"])[0]
    if mlp.get("shared") is not None:
        out = out + squared_relu_ff(h, P[p + "shared.up"], P[p + "shared.down"])
    return out


# ---- the model --------------------------------------------------------------------------------------

def mixer(h, P, p, layer, eps):
    kind, m = layer["type"], layer["mixer"]
    if kind == "delta":
        return delta_mixer(h, P, p, m, eps)
    left = softmax_attention(h, P, p + "left.", m["left"], eps, kind)
    if kind == "parallel":
        right = lightning_mixer(h, P, p + "right.", m["right"], eps)
    elif kind == "parallel_2":
        right = removal_mixer(h, P, p + "right.", m["right"], eps)
    else:
        raise ValueError(kind)
    return float(m["left_scale"]) * left + float(m["right_scale"]) * right


def forward(cfg, P, tokens, keep=None):
    """Logits [n, vocab] of one sequence from position 0; ``keep`` receives the residual stream
    after every layer."""
    eps = float(cfg["norm"]["eps"])
    x = P["embed"][torch.as_tensor(tokens, dtype=torch.long)] * float(cfg["embedding"]["scale"])
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        x = x + one_plus_norm(mixer(input_conv(x, P[p + "canon1"]), P, p + "mix.", layer, eps), P[p + "norm1"], eps)
        if layer.get("mlp") is not None:
            x = x + one_plus_norm(moe_ff(input_conv(x, P[p + "canon2"]), P, p + "mlp.", layer["mlp"]), P[p + "norm2"], eps)
        if keep is not None:
            keep.append(x.clone())
    return one_plus_norm(x, P["final.norm"], eps) @ P["embed"].T * float(cfg["logit_scale"])
