"""Retuvik through the engine (model registry, grouped cache with matrix states, state slots,
Engine.step, generation) against the plain float64 statement in ``oracle_retuvik.py``, on small
random checkpoints of several shapes. Every case runs on the CPU (PyTorch statements of the ops)
and, marked ``gpu``, on the HIP kernels in fp32 and bf16.
"""
import json
import math
import os

import pytest
import torch
from safetensors.torch import save_file

import oracle_retuvik as O
from theroundtaible_amd.engine import Engine, EngineConfig, SamplingParams, Turn
from theroundtaible_amd.engine.kv_cache import KVCacheOOM
from theroundtaible_amd.models.config import GroupedAttentionSpec, WKVSpec, config_from_dir, get_config
from theroundtaible_amd.models.weights import layout_for

GPU = pytest.mark.gpu
RUNS = [("cpu", "fp32"), pytest.param(("cuda:0", "fp32"), marks=GPU), pytest.param(("cuda:0", "bf16"), marks=GPU)]

DENSE = {"kind": "dense", "ff": 56}


def moe(experts=5, top=2, ff=24):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def wkv(heads, dim, mlp=DENSE, rank=6):
    return {"type": "wkv", "mixer": {"heads": heads, "dim": dim, "decay_rank": rank}, "mlp": mlp}


def att(heads, kv, dim, vdim=None, window=11, temp=(0.4, 8), scale=None, mlp=DENSE):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": dim if vdim is None else vdim,
         "scale": 1.3 * dim ** -0.5 if scale is None else scale}
    if window:
        m["mask"] = {"size": window}
    if temp:
        m["q_temp"] = {"coef": temp[0], "every": temp[1]}
    return {"type": "attention", "mixer": m, "mlp": mlp}


def make_config(width=40, vocab=97, layers=None, loop=(1, 3, 2), embed_scale=1.7, eps=1e-5, groups=2):
    if layers is None:
        layers = [wkv(2, 12), att(6, 2, 12, mlp=moe()), wkv(3, 8, mlp=moe(4, 3)), att(4, 4, 10, vdim=14, window=5, mlp=None)]
    cfg = {"architecture": "Retuvik", "embedding": {"scale": embed_scale}, "layers": layers,
           "norm": {"eps": eps, "groups": groups}, "vocab": vocab, "width": width}
    if loop is not None:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg


def make_checkpoint(path, cfg, seed=0, edit=None):
    """Random weights for ``cfg`` (a config.json dict) written as a checkpoint directory; returns
    the float64 tensors. ``edit(P)`` may change tensors before they are written."""
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    mc = config_from_dir(path)
    g = torch.Generator().manual_seed(seed)
    P = {}
    for name, (shape, _, _) in layout_for(mc).items():
        if name.endswith(("norm1", "norm2", "final.norm", "mix.norm", "q.norm", "k.norm")):
            w = 0.6 + torch.rand(shape, generator=g)
        elif ".mu." in name:
            w = torch.rand(shape, generator=g)
        elif name.endswith("w0"):                   # decays exp(-exp(.)) spread between ~0.3 and ~0.99
            w = -4.0 + 4.2 * torch.rand(shape, generator=g)
        elif name.endswith(("mix.u", "mlp.act", "loop.step")):
            w = torch.randn(shape, generator=g) * 0.5
        elif name.endswith("router.b"):
            w = torch.randn(shape, generator=g) * 2.0
        elif name.endswith(".b"):
            w = torch.randn(shape, generator=g) * 0.5
        elif name == "embed":
            w = torch.randn(shape, generator=g)
        elif name.endswith("router"):               # clear choices: no top-k call is close
            w = torch.randn(shape, generator=g) * 2.0 / math.sqrt(shape[-1])
        else:
            w = torch.randn(shape, generator=g) / math.sqrt(shape[-1])
        P[name] = w.to(torch.bfloat16).float()      # values both number formats hold exactly
    if edit is not None:
        edit(P)
    save_file({k: v.contiguous() for k, v in P.items()}, os.path.join(path, "model.safetensors"))
    return {k: v.double() for k, v in P.items()}


def engine_for(path, run, tokens=512, block_size=16, slots=4, graphs=False):
    device, dtype = run
    if device != "cpu":
        from theroundtaible_amd.ops import hybrid
        hybrid.native()     # the GPU cases fail loudly when the extension is missing
    return Engine(EngineConfig(model=str(path), weights=str(path), dtype=dtype, device=device, block_size=block_size,
                               num_blocks=(tokens + block_size - 1) // block_size + (1 if graphs else 0),
                               use_graphs=graphs, state_slots=slots, max_batch=slots))


def close(got, want, run, what=""):
    tol = dict(rtol=0, atol=0.35) if run[1] == "bf16" else dict(rtol=0, atol=2e-3)
    torch.testing.assert_close(got.double().cpu(), want, msg=lambda m: f"{what}: {m}", **tol)


def toks(n, vocab, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def forward(cfg, P, t, keep=None):
    return O.forward(cfg, P, t, keep)


# ---- each mechanism alone (package ops on the CPU against the oracle's functions) ---------------

def _one_span(T, start=0):
    """Metadata of one span of T rows at positions start .. of a sequence in slot 0."""
    return (torch.zeros(T, dtype=torch.int32), torch.arange(start, start + T), torch.tensor([start], dtype=torch.int32),
            torch.zeros(1, dtype=torch.int32))


def _cu(n):
    return torch.tensor([0, n], dtype=torch.int32)


def test_norm_in_groups_and_shift_mixes():
    from theroundtaible_amd.ops import hybrid as Hy
    g = torch.Generator().manual_seed(3)
    T, W = 9, 24
    x = torch.randn(T, W, generator=g, dtype=torch.float64) * torch.linspace(0.2, 5.0, W, dtype=torch.float64)
    y = torch.randn(T, W, generator=g, dtype=torch.float64)
    w = 0.5 + torch.rand(W, generator=g, dtype=torch.float64)
    for groups in (1, 2, 3):
        xa = x.float().clone()
        got = Hy.add_norm(xa, y.float(), w.float(), 1e-5, torch.float32, groups)
        torch.testing.assert_close(got.double(), O.group_norm(x + y, w, groups, 1e-5), rtol=1e-5, atol=1e-5)
        torch.testing.assert_close(xa.double(), x + y, rtol=1e-6, atol=1e-6)
    assert float((O.group_norm(x, w, 1, 1e-5) - O.group_norm(x, w, 3, 1e-5)).abs().max()) > 0.1   # the groups show
    # several mixes of one normed row, whole and cut in two with the state between
    mu = torch.rand(5, W, generator=g, dtype=torch.float64)
    h = O.group_norm(x, w, 3, 1e-5)
    want = torch.stack([O.shifted(h, mu[i]) for i in range(5)])
    state = torch.zeros(1, W)
    got, _ = Hy.shift_norm(x.float(), None, w.float(), 1e-5, mu.float(), state, *_one_span(T), torch.float32, groups=3)
    torch.testing.assert_close(got.double(), want, rtol=1e-5, atol=1e-5)
    a, xa = Hy.shift_norm(x[:4].float(), None, w.float(), 1e-5, mu.float(), state, *_one_span(4), torch.float32, groups=3)
    Hy.shift_state_update(xa, w.float(), 1e-5, state, _cu(4), torch.zeros(1, dtype=torch.int32), 3)
    b, _ = Hy.shift_norm(x[4:].float(), None, w.float(), 1e-5, mu.float(), state, *_one_span(T - 4, 4), torch.float32, groups=3)
    torch.testing.assert_close(torch.cat([a, b], 1).double(), want, rtol=1e-5, atol=1e-5)


def _wkv_inputs(T, H, D, seed, decay_low=-3.0):
    g = torch.Generator().manual_seed(seed)
    r, k, v, gate = (torch.randn(T, H, D, generator=g, dtype=torch.float64) for _ in range(4))
    lw = torch.randn(T, H * D, generator=g, dtype=torch.float64)
    w0 = decay_low + 3.0 * torch.rand(H * D, generator=g, dtype=torch.float64)
    u = torch.randn(H, D, generator=g, dtype=torch.float64)
    nw = 0.5 + torch.rand(H * D, generator=g, dtype=torch.float64)
    return r, k, v, gate, lw, w0, u, nw


def _wkv_oracle(r, k, v, gate, lw, w0, u, nw, eps):
    T, H, D = r.shape
    o = O.wkv_recurrence(r, k, v, torch.exp(-torch.exp(lw + w0)).reshape(T, H, D), u)
    return O.unit_rms(o, eps).reshape(T, H * D) * nw * O.silu(gate.reshape(T, H * D))


def test_wkv_scan_whole_and_cut():
    from theroundtaible_amd.ops import hybrid as Hy
    T, H, D = 13, 3, 5
    r, k, v, gate, lw, w0, u, nw = _wkv_inputs(T, H, D, 4)
    want = _wkv_oracle(r, k, v, gate, lw, w0, u, nw, 1e-5)
    rkvg = torch.stack([t.reshape(T, H * D) for t in (r, k, v, gate)]).float()
    one = torch.zeros(1, dtype=torch.int32)
    st = torch.full((1, H * D * D), 9.0)            # a used slot: its content must not be read at position 0
    got = Hy.wkv_scan(rkvg, lw.float(), w0.float(), u.float(), nw.float(), 1e-5, st, _cu(T), one, one, torch.float32)
    torch.testing.assert_close(got.double(), want, rtol=1e-4, atol=1e-5)
    st = torch.full((1, H * D * D), 9.0)
    a = Hy.wkv_scan(rkvg[:, :6].contiguous(), lw[:6].float(), w0.float(), u.float(), nw.float(), 1e-5, st, _cu(6), one, one,
                    torch.float32)
    b = Hy.wkv_scan(rkvg[:, 6:].contiguous(), lw[6:].float(), w0.float(), u.float(), nw.float(), 1e-5, st, _cu(T - 6),
                    one + 6, one, torch.float32)
    torch.testing.assert_close(torch.cat([a, b]).double(), want, rtol=1e-4, atol=1e-5)
    # the bonus is for the current token only: with u = 0 the first token's output is zero
    dec = torch.exp(-torch.exp(lw + w0)).reshape(T, H, D)
    assert float(O.wkv_recurrence(r, k, v, dec, u * 0)[0].abs().max()) == 0.0
    assert float(O.wkv_recurrence(r, k, v, dec, u)[0].abs().max()) > 0.1


@pytest.mark.parametrize("run", RUNS)
def test_wkv_keeps_a_far_token(run):
    """Decays close to 1 in one head: the last token's r picks the key of token 0, hundreds of
    tokens (and several scan chunks) back, so its output is that token's value; a second head
    forgets fast and shows only the last tokens. A state that is lost, restarted or decayed with
    the wrong channel's factor changes the result by far more than the tolerance."""
    from theroundtaible_amd.ops import hybrid as Hy
    dev, dt = run[0], torch.bfloat16 if run[1] == "bf16" else torch.float32
    T, H, D = 331, 2, 16
    r, k, v, gate, lw, w0, u, nw = _wkv_inputs(T, H, D, 6)
    w0[:D] = -9.0                                   # head 0 keeps: decay exp(-exp(-9 + small)) per token
    lw[:, :D] *= 0.1
    k[1:, 0] *= 0.02                                # later keys of head 0 are small
    k[0, 0] = 3.0 * torch.nn.functional.normalize(k[0, 0], dim=0)
    r[-1, 0] = 4.0 * k[0, 0]
    want = _wkv_oracle(r, k, v, gate, lw, w0, u, nw, 1e-5)
    o = O.wkv_recurrence(r, k, v, torch.exp(-torch.exp(lw + w0)).reshape(T, H, D), u)[-1, 0]
    assert float(torch.nn.functional.cosine_similarity(o, v[0, 0], dim=0)) > 0.98     # the case shows token 0
    rkvg = torch.stack([t.reshape(T, H * D) for t in (r, k, v, gate)]).to(dt).to(dev)
    one = torch.zeros(1, dtype=torch.int32, device=dev)
    args = (w0.float().to(dev), u.float().to(dev), nw.float().to(dev), 1e-5)
    tol = dict(rtol=0.05, atol=0.08) if run[1] == "bf16" else dict(rtol=1e-3, atol=1e-4)
    forms = [None] + ([Hy.wkv_chunks(_cu(T), dev, min_rows=0)] if dev != "cpu" else [])
    for chunks in forms:
        st = torch.zeros(1, H * D * D, device=dev)
        got = Hy.wkv_scan(rkvg, lw.to(dt).to(dev), *args, st, _cu(T).to(dev), one, one, dt, chunks=chunks)
        torch.testing.assert_close(got.double().cpu()[-1], want[-1], **tol)
        if run[1] == "fp32":
            torch.testing.assert_close(got.double().cpu(), want, **tol)
        # the same in two spans: 200 rows, then the rest one row at a time from the kept state
        st2 = torch.zeros(1, H * D * D, device=dev)
        c2 = Hy.wkv_chunks(_cu(200), dev, min_rows=0) if chunks is not None else None
        Hy.wkv_scan(rkvg[:, :200].contiguous(), lw[:200].to(dt).to(dev), *args, st2, _cu(200).to(dev), one, one, dt, chunks=c2)
        for t in range(200, T):
            last = Hy.wkv_scan(rkvg[:, t:t + 1].contiguous(), lw[t:t + 1].to(dt).to(dev), *args, st2, _cu(1).to(dev),
                               one + t, one, dt)
        torch.testing.assert_close(last.double().cpu()[0], want[-1], **tol)
        if run[1] == "fp32":
            torch.testing.assert_close(st2.cpu(), st.cpu(), rtol=1e-3, atol=1e-4)


def _attention_case(n, H, G, D, E, BS, seed, dt, dev):
    g = torch.Generator().manual_seed(seed)
    k = O.unit_rms(torch.randn(n, G, D, generator=g, dtype=torch.float64), 0.0)
    v = torch.randn(n, G, E, generator=g, dtype=torch.float64)
    nb = (n + BS - 1) // BS
    order = torch.randperm(nb, generator=g)          # pages in any order
    kc, vc = torch.zeros(nb, G, BS, D, dtype=dt), torch.zeros(nb, G, BS, E, dtype=dt)
    for t in range(n):
        kc[order[t // BS], :, t % BS] = k[t].to(dt)
        vc[order[t // BS], :, t % BS] = v[t].to(dt)
    return k, v, kc.to(dev), vc.to(dev), order.to(torch.int32)[None].to(dev)


def _windowed(q, k, v, scale, slopes, window, i):
    """The oracle's statement for one query row at position i: q [H, D] over keys 0 .. i."""
    H, G = q.shape[0], k.shape[1]
    out = []
    for a in range(H):
        j = torch.arange(i + 1)
        s = (k[:i + 1, a // (H // G)] @ q[a]) * scale - slopes[a] * (i - j).double()
        if window:
            s = s.masked_fill(i - j >= window, float("-inf"))
        out.append(torch.softmax(s, 0) @ v[:i + 1, a // (H // G)])
    return torch.stack(out)


@pytest.mark.parametrize("run", RUNS)
@pytest.mark.parametrize("form", ["prompt", "decode"])
def test_window_edges_and_distance_penalty(run, form):
    """Attention alone on made-up queries and keys. One key's score stands far above the others:
    when it is the oldest key inside the window the output is its value, when it is one position
    older it has no weight at all; both at page borders and tile borders, in a prompt's portion
    that starts inside a page and in single decoded rows with split keys. The distance penalty
    (steep for the first head, nearly flat for the last) is part of every comparison."""
    from theroundtaible_amd.ops import hybrid as Hy
    dev, dt = run[0], torch.bfloat16 if run[1] == "bf16" else torch.float32
    H, G, D, E, BS, n, window = 4, 2, 16, 12, 8, 331, 72
    k, v, kc, vc, bt = _attention_case(n, H, G, D, E, BS, 5, dt, dev)
    slopes = O.head_slopes(H)
    rows = list(range(n - 10, n))
    # per row: the outstanding key is the oldest visible one (even rows) or the one just outside (odd rows)
    targets = [r - window + 1 if i % 2 == 0 else r - window for i, r in enumerate(rows)]
    boost = 30.0 + slopes[0] * window / 1.0        # beats the penalty of the steepest head
    q = torch.stack([torch.stack([k[j, a // 2] * float(boost) for a in range(H)]) for j in targets])
    sl = slopes.float().to(dev)
    if form == "prompt":
        out = Hy.gqa_attention(q.to(dt).to(dev), kc, vc, bt, torch.tensor([0, len(rows)], dtype=torch.int32, device=dev),
                               torch.tensor([rows[0]], dtype=torch.int32, device=dev), 1.0, None, 0.0, window=window, slopes=sl)
    else:
        B = len(rows)
        tiles = torch.stack([torch.arange(B), torch.arange(B)], 1).to(torch.int32).to(dev)
        out = Hy.gqa_attention(q.to(dt).to(dev), kc, vc, bt.expand(B, -1).contiguous(),
                               torch.arange(B + 1, dtype=torch.int32, device=dev),
                               torch.tensor(rows, dtype=torch.int32, device=dev), 1.0, None, 0.0, tiles=tiles,
                               num_splits=3 if dev != "cpu" else 1, window=window, slopes=sl)
    out = out.double().cpu().reshape(len(rows), H, E)
    for i, (r, j) in enumerate(zip(rows, targets)):
        want = _windowed(q[i], k, v, 1.0, slopes, window, r)
        tol = 0.06 if run[1] == "bf16" else 1e-4
        assert float((out[i] - want).abs().max()) < tol, f"row at {r}, key {j}"
        hit = float((want - v[j].repeat_interleave(2, 0)).abs().max())
        assert (hit < 0.05) if i % 2 == 0 else (hit > 0.3), (i, hit)      # inside: that key's value; outside: not


def test_attention_parts_alone():
    """Query / key weights, the query factor at positions on both sides of a step, unit-RMS values
    through the cache, the penalty per head, the window and the output gate against the oracle's
    mixer (identity output projection)."""
    from theroundtaible_amd.ops import hybrid as Hy
    g = torch.Generator().manual_seed(7)
    T, W, H, G, D, E = 21, 18, 4, 2, 6, 5
    m = {"heads": H, "kv_heads": G, "dim": D, "vdim": E, "scale": 0.6, "mask": {"size": 7}, "q_temp": {"coef": 0.8, "every": 4}}
    h = torch.randn(T, W, generator=g, dtype=torch.float64)
    P = {n: torch.randn(s, W, generator=g, dtype=torch.float64) / 3 for n, s in
         (("q", H * D), ("k", G * D), ("v", G * E), ("g", H * E))}
    P["q.norm"], P["k.norm"] = (0.5 + torch.rand(D, generator=g, dtype=torch.float64) for _ in range(2))
    P["o"] = torch.eye(H * E, dtype=torch.float64)
    want = O.attention_mixer(h, P, "", m, 1e-5)
    spec = GroupedAttentionSpec(H, G, D, E, 0.6, window=7, slope_base=8.0, qk_weight=True, q_temp=(0.8, 4), value_norm=True,
                                out_gate=True)
    proj = torch.cat([h @ P[n].T for n in "qkvg"], 1).float()
    kc, vc = torch.zeros(6, G, 4, D), torch.zeros(6, G, 4, E)
    bt = torch.tensor([[5, 0, 3, 1, 4, 2]], dtype=torch.int32)
    slots = torch.tensor([bt[0, t // 4] * 4 + t % 4 for t in range(T)])
    q = Hy.qk_prep(proj, spec, 0, H * D, (H + G) * D, None, 1e-5, torch.arange(T), kc, vc, slots, torch.float32,
                   q_weight=P["q.norm"].float(), k_weight=P["k.norm"].float())
    got = Hy.gqa_attention(q, kc, vc, bt, _cu(T), torch.zeros(1, dtype=torch.int32), 0.6, None, 0.0, window=7,
                           slopes=O.head_slopes(H).float(), gate=proj, gate_off=(H + G) * D + G * E)
    torch.testing.assert_close(got.double(), want, rtol=1e-4, atol=1e-5)
    # each part shows: dropping it moves the oracle's result far beyond that tolerance
    for drop in ("mask", "q_temp"):
        other = O.attention_mixer(h, P, "", {k: v for k, v in m.items() if k != drop}, 1e-5)
        assert float((other - want).abs().max()) > 0.02, drop


def test_feed_forward_parts_alone():
    from theroundtaible_amd.ops import hybrid as Hy
    g = torch.Generator().manual_seed(8)
    z = torch.tensor([[-4.0, -0.5, 0.0, 1e-3, 0.7, 3.0]], dtype=torch.float64)
    b = torch.tensor([0.1, -0.2, 0.0, 0.0, 0.3, -1.0], dtype=torch.float64)
    p, q = 0.3, -0.7
    got = Hy.xielu(z.float(), b.float(), O.softplus(p), 0.5 + O.softplus(q), torch.float32)
    torch.testing.assert_close(got.double(), O.xielu(z + b, p, q), rtol=1e-5, atol=1e-6)
    # routing: the chosen experts, largest first, and the softmax over the chosen alone
    T, W, E, Fe, top = 7, 10, 6, 4, 3
    h = torch.randn(T, W, generator=g, dtype=torch.float64)
    P = {"router": torch.randn(E, W, generator=g, dtype=torch.float64), "router.b": torch.randn(E, generator=g, dtype=torch.float64)}
    for e in range(E):
        P[f"e{e}.gate"], P[f"e{e}.up"] = (torch.randn(Fe, W, generator=g, dtype=torch.float64) / 3 for _ in range(2))
        P[f"e{e}.down"] = torch.randn(W, Fe, generator=g, dtype=torch.float64) / 2
    idx, wt = Hy.topk_softmax((h @ P["router"].T + P["router.b"]).float(), top)
    widx, wwt = O.route(h, P, "", top)
    assert idx.tolist() == widx.tolist()
    torch.testing.assert_close(wt.double(), wwt, rtol=1e-5, atol=1e-6)
    w_gu = torch.stack([torch.cat([P[f"e{e}.gate"], P[f"e{e}.up"]]) for e in range(E)]).float()
    w_d = torch.stack([P[f"e{e}.down"] for e in range(E)]).float()
    got = Hy.moe_experts(h.float(), idx, wt, w_gu, w_d, torch.float32)
    want = O.moe_ff(h, P, "", {"router": {"top": top}})
    torch.testing.assert_close(got.double(), want, rtol=1e-4, atol=1e-5)


def test_config_reader_and_registry(tmp_path):
    cfg = make_config()
    make_checkpoint(tmp_path / "m", cfg)
    mc = get_config(str(tmp_path / "m"))
    assert mc.arch == "retuvik" and mc.n_layers == 6 and mc.hidden == 40 and mc.embed_scale == 1.7 and mc.norm_groups == 2
    assert [ls.source for ls in mc.layers] == [0, 1, 2, 1, 2, 3]
    assert [ls.opens_pass for ls in mc.layers] == [None, 0, None, 1, None, None] and mc.loop_passes == 2
    assert [ls.ff_kind if ls.ff else None for ls in mc.layers] == ["dense", "moe", "moe", "moe", "moe", None]
    a = mc.layers[1].mixer
    assert (a.heads, a.kv_heads, a.dim, a.vdim, a.window, a.q_temp, a.slope_base) == (6, 2, 12, 12, 11, (0.4, 8), 8.0)
    assert a.rot is None and a.sink == 0.0 and a.qk_weight and a.value_norm and a.out_gate
    w = mc.layers[2].mixer
    assert isinstance(w, WKVSpec) and (w.heads, w.dim, w.state_size) == (3, 8, 192)
    assert (mc.layers[2].moe.experts, mc.layers[2].moe.top, mc.layers[2].ff) == (4, 3, 24)
    assert mc.kv_bytes_per_token(2) == 2 * (2 * (2 * 24) + 4 * 24)
    assert mc.n_params() == sum(math.prod(s) for s, _, _ in layout_for(mc).values())
    # keys the file does not have switch their mechanism off
    plain = make_config(layers=[att(2, 1, 8, window=0, temp=None)], loop=None)
    json.dump(plain, open(tmp_path / "m" / "config.json", "w"))
    b = get_config(str(tmp_path / "m")).layers[0].mixer
    assert b.window == 0 and b.q_temp is None and get_config(str(tmp_path / "m")).loop_passes == 0
    for bad in (dict(cfg, loop={"start": 2, "stop": 5, "times": 2}),
                dict(cfg, layers=[dict(cfg["layers"][0], type="conv")]),
                dict(cfg, norm={"eps": 1e-5, "groups": 3})):
        os.makedirs(tmp_path / "bad", exist_ok=True)
        json.dump(bad, open(tmp_path / "bad" / "config.json", "w"))
        with pytest.raises(ValueError):
            get_config(str(tmp_path / "bad"))
    tiny = get_config("tiny-retuvik")
    assert [ls.source for ls in tiny.layers] == [0, 1, 2, 1, 2, 3]


def test_decay_rank_comes_from_the_checkpoint(tmp_path):
    """The width of the decay's low-rank path is a tensor shape: a checkpoint whose config does
    not name it loads, with whatever rank its tensors have."""
    cfg = make_config(layers=[wkv(2, 8, rank=5)], loop=None)
    P = make_checkpoint(tmp_path / "m", cfg, seed=2)
    del cfg["layers"][0]["mixer"]["decay_rank"]
    json.dump(cfg, open(tmp_path / "m" / "config.json", "w"))
    e = engine_for(tmp_path / "m", ("cpu", "fp32"))
    t = toks(12, cfg["vocab"], 2)
    close(e.step([("a", t, list(range(12)))]), forward(cfg, P, t), ("cpu", "fp32"))


# ---- whole prompts, and the residual stream layer by layer ---------------------------------------

@pytest.mark.parametrize("run", RUNS)
def test_whole_prompt_and_layers(tmp_path, run):
    cfg = make_config()
    P = make_checkpoint(tmp_path / "m", cfg, seed=1)
    e = engine_for(tmp_path / "m", run)
    t = toks(45, cfg["vocab"], 1)
    layers = []
    want = forward(cfg, P, t, layers)
    got = e.step([("a", t, list(range(len(t))))])
    close(got, want, run, "logits")
    s = e.kv.seq("b")
    tok, pos, meta = e._varlen_meta([e.reserve(s, t)])
    keep = []
    with torch.no_grad():
        e.model.forward(tok, pos, e.kv, meta, keep_layers=keep)
    assert len(keep) == len(layers) == 6
    for i, (a, b) in enumerate(zip(keep, layers)):
        tol = 0.3 if run[1] == "bf16" else 1e-3
        assert float((a.double().cpu() - b).abs().max()) < tol, f"residual stream after layer run {i}"
    e.model.fuse_adds = False
    close(e.step([("c", t, list(range(len(t))))]), want, run, "separate adds")


SHAPES = {
    # one norm group; one query head per key/value head, one key/value head for all; no loop; top = 1 and top = all
    "groups": (1, [att(3, 3, 8, mlp=moe(3, 1)), wkv(1, 24), att(5, 1, 6, vdim=9, mlp=moe(3, 3))], None),
    # heads wider than a wave's 64 lanes: attention keys / values, and wkv states of 72 x 72 and 132 x 132
    "wide": (3, [att(2, 1, 72, vdim=132, mlp=None), wkv(2, 72, mlp=None), wkv(1, 132)], None),
    # more query heads per key/value head than one attention workgroup's pairs
    "many-heads": (2, [att(40, 1, 4, mlp={"kind": "dense", "ff": 24})], None),
    # a loop over everything, three times, that starts with attention; no window, no query factor
    "all-looped": (4, [att(2, 2, 8, window=0, temp=None, mlp=None), wkv(2, 6, mlp=moe(4, 2, 12))], (0, 2, 3)),
    # a loop of one pass over the last layer; a window of one token (a row sees itself only); constants that are 1
    "ones": (1, [wkv(1, 4, mlp=None), att(1, 1, 4, window=1, temp=(1.0, 1), scale=1.0, mlp={"kind": "dense", "ff": 16})], (1, 2, 1)),
    # an empty loop; the query factor stepping every position
    "empty-loop": (2, [wkv(2, 4), att(2, 1, 4, temp=(0.3, 1))], (1, 1, 4)),
}


@pytest.mark.parametrize("run", RUNS)
@pytest.mark.parametrize("shape", list(SHAPES))
def test_other_sizes(tmp_path, run, shape):
    """Sizes and constants that the usual test model makes equal or 1."""
    groups, layers, loop = SHAPES[shape]
    cfg = make_config(width=24, vocab=61, layers=layers, loop=loop, embed_scale=1.0 if shape == "ones" else 1.9,
                      groups=groups)
    P = make_checkpoint(tmp_path / "m", cfg, seed=2)
    e = engine_for(tmp_path / "m", run, block_size=8)
    t = toks(70, cfg["vocab"], 2)
    want = forward(cfg, P, t)
    got = torch.cat([e.step([("a", t[:37], list(range(37)))]), e.step([("a", t[37:39], [0, 1])])] +
                    [e.step([("a", t[i:i + 1], [0])]) for i in range(39, 70)])
    close(got, want, run, shape)


@pytest.mark.parametrize("run", RUNS)
def test_wider_layers(tmp_path, run):
    """Rows wide enough for several waves per norm workgroup, wkv heads that fill a wave, 64-wide
    attention heads with a window that crosses many key tiles and pages, eight experts: a prompt in
    portions (the first long enough for seven scan chunks), then decoded tokens."""
    layers = [wkv(8, 64, mlp={"kind": "dense", "ff": 1024}, rank=32), att(8, 2, 64, window=200, temp=(0.2, 128), mlp=moe(8, 2, 256))]
    cfg = make_config(width=512, vocab=331, layers=layers, loop=(0, 2, 2), groups=2)
    P = make_checkpoint(tmp_path / "m", cfg, seed=21)
    e = engine_for(tmp_path / "m", run, tokens=1024, block_size=32)
    t = toks(720, cfg["vocab"], 21)
    want = forward(cfg, P, t)
    got = [e.step([("a", t[:450], [0, 199, 200, 201, 449])]), e.step([("a", t[450:452], [0, 1])]),
           e.step([("a", t[452:700], [0, 247])])] + [e.step([("a", t[i:i + 1], [0])]) for i in range(700, 720)]
    rows = [0, 199, 200, 201, 449, 450, 451, 452, 699] + list(range(700, 720))
    close(torch.cat(got), want[rows], run, "wider layers")


# ---- portions, decoding, batches ------------------------------------------------------------------

@pytest.mark.parametrize("run", RUNS)
def test_prefill_against_token_by_token(tmp_path, run):
    cfg = make_config()
    P = make_checkpoint(tmp_path / "m", cfg, seed=3)
    e = engine_for(tmp_path / "m", run)
    t = toks(40, cfg["vocab"], 3)
    want = forward(cfg, P, t)
    one = torch.cat([e.step([("a", [x], [0])]) for x in t])          # from the first token on
    close(one, want, run, "token by token")
    whole = e.step([("b", t, list(range(40)))])
    close(whole, want, run, "whole")
    tol = 0.35 if run[1] == "bf16" else 1e-3
    assert float((one - whole).abs().max()) < tol


@pytest.mark.parametrize("run", RUNS)
@pytest.mark.parametrize("cuts", [[2, 2, 3, 1, 30, 2, 17, 1, 1, 5], [16, 16, 16, 16], [1, 63], [33, 31], [131, 2, 70]])
def test_portions(tmp_path, run, cuts):
    """Portions of several sizes, down to two tokens and one, cut inside and at page borders
    (pages of 16) and inside windows (11 and 5): the shift state and the wkv state carry over every
    cut. The long portions take the chunked wkv scan on the GPU."""
    cfg = make_config()
    P = make_checkpoint(tmp_path / "m", cfg, seed=4)
    e = engine_for(tmp_path / "m", run)
    t = toks(sum(cuts), cfg["vocab"], 4)
    want = forward(cfg, P, t)
    out, at = [], 0
    for n in cuts:
        out.append(e.step([("a", t[at:at + n], list(range(n)))]))
        at += n
    close(torch.cat(out), want, run, f"portions {cuts}")


@pytest.mark.parametrize("run", RUNS)
def test_mixed_batch_equals_each_alone_and_slots_are_reused(tmp_path, run):
    """Unequal requests in one batch (portions beside single tokens, requests paused for a step),
    a pool of four state slots and few pages, so both are freed and used again: a request that
    takes a used slot starts from a zero wkv state and a zero shift row."""
    cfg = make_config()
    P = make_checkpoint(tmp_path / "m", cfg, seed=5)
    e = engine_for(tmp_path / "m", run, tokens=160, slots=4)
    V = cfg["vocab"]
    reqs = {k: toks(n, V, 10 + i) for i, (k, n) in enumerate([("a", 50), ("b", 7), ("c", 33), ("d", 1), ("e", 41), ("f", 20)])}
    want = {k: forward(cfg, P, v) for k, v in reqs.items()}
    got = {k: [] for k in reqs}
    at = {k: 0 for k in reqs}
    plan = [[("a", 20), ("b", 7)], [("a", 1), ("c", 30), ("d", 1)], [("a", 2), ("c", 1)], [("c", 2), ("a", 27), ("e", 3)],
            [("e", 38), ("f", 5)], [("f", 1)], [("f", 14)]]
    for step in plan:
        entries, end = [], []
        for k, n in step:
            entries.append((k, reqs[k][at[k]:at[k] + n], list(range(n))))
            at[k] += n
            if at[k] == len(reqs[k]):
                end.append(k)
        out = e.step(entries, end=end)
        o = 0
        for k, n in step:
            got[k].append(out[o:o + n])
            o += n
    for k in reqs:
        close(torch.cat(got[k]), want[k], run, f"request {k}")
    assert e.kv.alloc.num_free == e.kv.num_blocks and len(e.kv.state.free) == 4
    with pytest.raises(KVCacheOOM):       # a fifth live request has no slot
        for i in range(5):
            e.step([(f"x{i}", [1, 2], [])])


@pytest.mark.parametrize("run", RUNS)
def test_long_decoding_past_windows_and_page_borders(tmp_path, run):
    """150 tokens, all but five decoded one by one through pages of 8: every window (11 and 5)
    slides over decoded tokens many times, the query factor steps every 8 positions."""
    cfg = make_config()
    P = make_checkpoint(tmp_path / "m", cfg, seed=7)
    e = engine_for(tmp_path / "m", run, block_size=8)
    t = toks(150, cfg["vocab"], 7)
    want = forward(cfg, P, t)
    got = torch.cat([e.step([("a", t[:5], list(range(5)))])] + [e.step([("a", [x], [0])]) for x in t[5:]])
    close(got, want, run, "long decode")


# ---- the engine's own generation path and scheduler -----------------------------------------------

def _greedy_oracle(P, cfg, prompt, n):
    seq = list(prompt)
    for _ in range(n):
        seq.append(int(forward(cfg, P, seq)[-1].argmax()))
    return seq[len(prompt):]


@pytest.mark.parametrize("run,graphs", [(("cpu", "fp32"), False), pytest.param(("cuda:0", "fp32"), False, marks=GPU),
                                        pytest.param(("cuda:0", "fp32"), True, marks=GPU)])
def test_greedy_generation_through_run_turns(tmp_path, run, graphs):
    """Greedy decoding through Engine.run_turns (tokenizer, prefix reuse, batched decode loop — the
    captured graph on the GPU) gives the oracle's tokens, for two requests of unequal length."""
    cfg = make_config(vocab=300, embed_scale=1.5)
    P = make_checkpoint(tmp_path / "m", cfg, seed=8)
    e = engine_for(tmp_path / "m", run, tokens=2048, graphs=graphs)
    sp = SamplingParams(temperature=0.0, max_new_tokens=12, ignore_eos=True, stop_on_consensus=False)
    prompts = ["De ridders aan de ronde tafel overleggen over het cachebeleid.", "Kort."]
    outs = e.run_turns([Turn("A", prompts[0], sp), Turn("B", prompts[1], sp)])
    for o, p in zip(outs, prompts):
        assert o.error is None, o.error
        ids = e.encode_prompt(p)
        assert o.ids == _greedy_oracle(P, cfg, ids, 12)
    from theroundtaible_amd.prompt import Prompt
    p2 = Prompt().add(prompts[0]).add(outs[0].text, outs[0].ids, e.tokenizer.family)
    o2 = e.run_turns([Turn("A", p2, sp)])[0]
    ids2 = e.encode_prompt(prompts[0]) + outs[0].ids
    assert o2.ids == _greedy_oracle(P, cfg, ids2, 12)


@GPU
def test_decode_steps_on_the_skinny_gemm_and_expert_rows(tmp_path):
    """Sizes the framework's skinny decode GEMM takes (K a multiple of 32, N of 16): decode steps
    run their plain linears on it and their experts row by row; the logits match the oracle and
    the same steps on the library GEMMs."""
    from theroundtaible_amd import ops
    if not ops.native_available():
        pytest.skip("main extension not built")
    cfg = make_config(width=64, vocab=80, loop=(0, 2, 2),
                      layers=[wkv(4, 16, mlp={"kind": "dense", "ff": 96}, rank=16), att(4, 2, 16, mlp=moe(6, 2, 32))])
    P = make_checkpoint(tmp_path / "m", cfg, seed=11)
    t = toks(60, cfg["vocab"], 11)
    want = forward(cfg, P, t)
    outs = []
    for skinny in (True, False):
        e = engine_for(tmp_path / "m", ("cuda:0", "bf16"))
        e.model.use_skinny = skinny
        got = torch.cat([e.step([("a", t[:20], list(range(20)))])] + [e.step([("a", [x], [0])]) for x in t[20:]])
        close(got, want, ("cuda:0", "bf16"), f"skinny={skinny}")
        outs.append(got)
        if skinny:
            assert sorted(len(d) for d in e.model._dec.values()) == [2, 4]
    assert float((outs[0] - outs[1]).abs().max()) < 0.25


def test_serving_entry_points_match_run_turns():
    """The continuous-batching entry points (prefill + first token, then decode in chunks while the
    state follows) give the tokens of a single run_turns call; random-init preset weights."""
    def eng():
        return Engine(EngineConfig(model="tiny-retuvik", weights="random:3", dtype="fp32", device="cpu",
                                   num_blocks=64, use_graphs=False, state_slots=4))
    sp = SamplingParams(temperature=0.0, max_new_tokens=10, ignore_eos=True, stop_on_consensus=False)
    turns = [Turn("A", "Eerste ridder spreekt over de cache.", sp), Turn("B", "Tweede.", sp)]
    want = [o.ids for o in eng().run_turns(turns)]
    e = eng()
    started = e.start_turns(turns)
    seqs = [s for s, _, _ in started]
    got = [[f] for _, f, _ in started]
    for steps in (4, 5):
        new = e.continue_decode(seqs, turns, [g[-1] for g in got], steps)
        for g, n in zip(got, new):
            g.extend(n)
    assert got == want
    assert all(s.state_len == s.length for s in seqs)


def test_cache_of_runs_without_pages():
    """The cache manager alone: a run whose mixer has no attention has no pages and no shift row
    unless asked; its matrix state is a row per slot and is copied by a fork."""
    from theroundtaible_amd.engine.kv_cache import GroupedKVCache
    kv = GroupedKVCache([None, (1, 4, 10)], width=5, rec_widths=[2 * 3 * 3, 0], num_blocks=8, block_size=4, device="cpu",
                        dtype=torch.float32, n_slots=2, shift_layers=[True, False])
    assert kv.k_layer(0) is None and kv.v_layer(1).shape == (8, 1, 4, 10)
    assert kv.rec[0].shape == (2, 18) and kv.rec[1] is None and kv.shift[0].shape == (2, 5) and kv.shift[1] is None
    a = kv.seq("a")
    kv.ensure_capacity(a, 6)
    a.tokens.extend(range(6))
    kv.slot_of(a)
    a.state_len = 6
    kv.rec[0][a.slot].fill_(2.0)
    b = kv.fork("a", "b", copy=True)
    assert b.slot == 1 and float(kv.rec[0][b.slot].mean()) == 2.0
    kv.free_seq("a")
    kv.free_seq("b")
    assert kv.alloc.num_free == 8 and sorted(kv.state.free) == [0, 1]
