"""Ledinex through the engine (model registry, grouped cache with convolution and matrix states,
state slots, Engine.step, generation) against the plain float64 statement in
``oracle_ledinex.py``, on small random checkpoints of several shapes. Every case runs on the CPU
(PyTorch statements of the ops) and, marked ``gpu``, on the HIP kernels in fp32 and bf16.
"""
import json
import math
import os

import pytest
import torch
from safetensors.torch import save_file

import oracle_ledinex as O
from theroundtaible_amd.engine import Engine, EngineConfig, SamplingParams, Turn
from theroundtaible_amd.engine.kv_cache import KVCacheOOM
from theroundtaible_amd.models.config import (DecaySumSpec, DeltaSpec, GroupedAttentionSpec, ParallelSpec, RemovalSpec,
                                              RotarySpec, config_from_dir, get_config)
from theroundtaible_amd.models.weights import layout_for
from theroundtaible_amd.ops import hybrid as Hy

GPU = pytest.mark.gpu
RUNS = [("cpu", "fp32"), pytest.param(("cuda:0", "fp32"), marks=GPU), pytest.param(("cuda:0", "bf16"), marks=GPU)]


def moe(experts=5, top=2, ff=24, shared=40):
    m = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if shared:
        m["shared"] = {"ff": shared}
    return m


def left(heads, kv, dim, vdim=None, rot_dims=None, base=10000.0, scaling=None, window=0, softcap=None, scale=None):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": dim if vdim is None else vdim,
         "scale": 1.4 * dim ** -0.5 if scale is None else scale,
         "rot": {"base": base, "dims": dim if rot_dims is None else rot_dims}}
    if scaling is not None:
        m["rot"]["scaling"] = scaling
    if window:
        m["mask"] = {"size": window}
    if softcap:
        m["softcap"] = softcap
    return m


YARN = {"factor": 6.0, "original": 64, "fast": 16.0, "slow": 1.0}


def par(heads=4, kv=2, dim=12, vdim=10, rheads=3, rdim=8, rvdim=6, decay=None, softcap=9.0, ls=0.7, rs=1.2, mlp="moe",
        **kw):
    decay = decay or [0.55 + 0.44 * i / max(1, rheads - 1) for i in range(rheads)]
    kw.setdefault("scaling", {"factor": 3.0})
    return {"type": "parallel", "mlp": moe() if mlp == "moe" else mlp,
            "mixer": {"left": left(heads, kv, dim, vdim, softcap=softcap, **kw), "left_scale": ls, "right_scale": rs,
                      "right": {"heads": rheads, "dim": rdim, "vdim": rvdim, "decay": decay[:rheads]}}}


def par2(heads=6, kv=2, dim=12, rheads=2, rdim=10, window=11, ls=0.9, rs=0.6, mlp="moe", **kw):
    kw.setdefault("scaling", YARN)
    kw.setdefault("rot_dims", 8)
    return {"type": "parallel_2", "mlp": moe(4, 3, 16, 24) if mlp == "moe" else mlp,
            "mixer": {"left": left(heads, kv, dim, window=window, **kw), "left_scale": ls, "right_scale": rs,
                      "right": {"heads": rheads, "dim": rdim}}}


def delta(heads=4, kv=2, dim=6, vdim=10, conv=4, mlp="moe"):
    return {"type": "delta", "mlp": moe(6, 1, 20, 0) if mlp == "moe" else mlp,
            "mixer": {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "conv": conv}}


def make_config(width=40, vocab=97, layers=None, taps=3, embed_scale=1.7, logit_scale=0.6, eps=1e-5):
    if layers is None:
        layers = [par2(), delta(), par(), delta(2, 1, 8, 4, conv=2, mlp=None), par2(3, 3, 8, 2, 6, window=5, rot_dims=8)]
    return {"architecture": "Ledinex", "canon": {"taps": taps}, "embedding": {"scale": embed_scale}, "layers": layers,
            "logit_scale": logit_scale, "norm": {"eps": eps}, "vocab": vocab, "width": width}


def settle(cfg, run):
    """bf16 runs choose every expert: rounding would otherwise flip a close router call now and
    then, and behind an output norm one flipped expert changes a whole row. The routing weights
    still count; the choice itself is covered by the fp32 runs and the router's own test."""
    if run[1] != "bf16":
        return cfg
    cfg = json.loads(json.dumps(cfg))
    for layer in cfg["layers"]:
        if layer["mlp"] is not None:
            layer["mlp"]["router"]["top"] = layer["mlp"]["router"]["experts"]
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
        shape = tuple(5 if n < 0 else n for n in shape)        # the decay path's rank is the checkpoint's
        if name.endswith(("norm1", "norm2", "final.norm")):     # stored around zero
            w = 0.4 * torch.randn(shape, generator=g)
        elif name.endswith(("mix.norm", "q.norm", "k.norm", "right.norm")):
            w = 0.6 + torch.rand(shape, generator=g)
        elif name.endswith(("canon1", "canon2")):
            w = 0.4 * torch.randn(shape, generator=g)
        elif name.endswith(".conv"):
            w = 0.4 * torch.randn(shape, generator=g)
            w[:, -1] += 1.0
        elif name.endswith("A_log"):                # decays that keep most of the state: a wiped state is rank one,
            w = -2.0 + 0.5 * torch.randn(shape, generator=g)    # and its read-out can cancel to rounding noise
        elif name.endswith(("w0", "a.b", "q.b", "k.b", "dt_bias")):
            w = torch.randn(shape, generator=g) * 0.8
        elif name == "embed":
            w = torch.randn(shape, generator=g)
        elif name.endswith("router"):               # clear choices: no top-k call is close
            w = torch.randn(shape, generator=g) * 2.5 / math.sqrt(shape[-1])
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
        Hy.native()     # the GPU cases fail loudly when the extension is missing
    return Engine(EngineConfig(model=str(path), weights=str(path), dtype=dtype, device=device, block_size=block_size,
                               num_blocks=(tokens + block_size - 1) // block_size + (1 if graphs else 0),
                               use_graphs=graphs, state_slots=slots, max_batch=slots))


def close(got, want, run, what=""):
    """fp32 runs: every logit within 2e-3 of the oracle. bf16 runs: these few-channel models are
    badly conditioned here and there (a per-head norm of a read-out that nearly cancels turns
    rounding into a visible error, and the state carries it on), so rows are judged together: the
    median row error stays under 2 % of the logits' range and at most one row in five is off by
    more than 10 % of it. A wrong kernel misses every row by about the whole range."""
    got = got.double().cpu()
    if run[1] != "bf16":
        torch.testing.assert_close(got, want, msg=lambda m: f"{what}: {m}", rtol=0, atol=2e-3)
        return
    err, span = (got - want).abs().max(-1).values, float(want.abs().max())
    assert torch.isfinite(got).all(), what
    assert float(err.median()) < 0.02 * span and float((err > 0.1 * span).double().mean()) <= 0.2, \
        f"{what}: median row error {float(err.median()):.3f}, worst {float(err.max()):.3f}, range {span:.1f}"


def toks(n, vocab, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def dev_of(run):
    return torch.device(run[0])


def dt_of(run):
    return torch.bfloat16 if run[1] == "bf16" else torch.float32


def spans(cuts, slot=1):
    """Row metadata of ONE sequence fed in portions: yields (rows, row_seq, positions, start_pos, cu_q, slots)."""
    at = 0
    for n in cuts:
        yield (slice(at, at + n), torch.zeros(n, dtype=torch.int32), torch.arange(at, at + n),
               torch.tensor([at], dtype=torch.int32), torch.tensor([0, n], dtype=torch.int32),
               torch.tensor([slot], dtype=torch.int32))
        at += n


# ---- each mechanism alone (package ops against the oracle's functions) ----------------------------

@pytest.mark.parametrize("run", RUNS)
@pytest.mark.parametrize("taps,cuts", [(3, [7, 1, 1, 2, 9]), (5, [2, 2, 1, 30]), (1, [4, 3]), (2, [1, 1, 1, 5])])
def test_input_convolution_with_the_normed_add(run, taps, cuts):
    """x + norm(y + y2) and the convolution over it, the sequence cut into portions (shorter than
    the taps too): rows ahead of a portion come from the state, zeros ahead of the sequence."""
    dev, dt = dev_of(run), dt_of(run)
    g = torch.Generator().manual_seed(taps)
    n, W = sum(cuts), 24
    x, y, y2 = (torch.randn(n, W, generator=g).to(dt).float() for _ in range(3))
    nw, cw = 0.3 * torch.randn(W, generator=g), 0.5 * torch.randn(W, taps, generator=g)
    xs = x.double() + O.one_plus_norm((y + y2).double(), nw.double(), 1e-5)
    want = O.input_conv(xs, cw.double())
    state = torch.full((3, 2, max(taps - 1, 1), W), 7.0, device=dev)        # a used slot: never read at position 0
    got, res = [], []
    for rows, rs, pos, sp, cu, sl in spans(cuts):
        one = rows.stop - rows.start == 1 and rows.start > 0
        h, r = Hy.canon_add(x[rows].to(dev), y[rows].to(dt).to(dev), y2[rows].to(dt).to(dev), (1 + nw).to(dev), 1e-5,
                            cw.to(dev), state, 1, rs.to(dev), pos.to(dev), sp.to(dev), sl.to(dev), dt, shift_state=one)
        if not one:
            Hy.conv_state_update(r, 0, W, state, 1, cu.to(dev), sp.to(dev), sl.to(dev))
        got.append(h)
        res.append(r)
    tol = 0.06 if run[1] == "bf16" else 1e-4
    assert float((torch.cat(res).double().cpu() - xs).abs().max()) < 1e-4
    assert float((torch.cat(got).double().cpu() - want).abs().max()) < tol
    assert float((state[:, 0] - 7.0).abs().max()) == 0      # the other sublayer's rows are untouched


def test_rotary_tables():
    for rot in ({"base": 5000.0, "dims": 16}, {"base": 5000.0, "dims": 16, "scaling": {"factor": 4.0}},
                {"base": 300.0, "dims": 24, "scaling": YARN},
                {"base": 300.0, "dims": 8, "scaling": {"factor": 2.0, "original": 16, "fast": 2.0, "slow": 2.0}}):
        cfg = make_config(layers=[par2(2, 1, rot["dims"], rot_dims=rot["dims"], base=rot["base"], scaling=rot.get("scaling"))])
        with_dir = config_like(cfg)
        spec = with_dir.layers[0].mixer.left.rot
        freq, mag = Hy.rotary_halves_table(spec, "cpu")
        want, wmag = O.rotary_frequencies(rot)
        assert float((freq.double() - want).abs().max() / want.abs().max()) < 1e-6 and abs(mag - wmag) < 1e-12


def config_like(cfg):
    from theroundtaible_amd.models.config import parse_ledinex
    return parse_ledinex(cfg, "t")


def _attention_case(run, spec, n, BS, seed, bias, edit=None):
    """qkv_prep_wide + gqa_attention (+ turn_back) of one sequence through a paged cache whose
    pages are scattered, against the oracle's attention on the same projections."""
    dev, dt = dev_of(run), dt_of(run)
    g = torch.Generator().manual_seed(seed)
    H, G, D, E = spec.heads, spec.kv_heads, spec.dim, spec.vdim
    nq, nk, nv = H * D, G * D, 0 if spec.value_from_key else G * E
    proj = torch.randn(n, 3 + nq + nk + nv, generator=g)
    qb, kb = (0.5 * torch.randn(nq, generator=g), 0.5 * torch.randn(nk, generator=g)) if bias else (None, None)
    qw, kw = 0.6 + torch.rand(nq, generator=g), 0.6 + torch.rand(nk, generator=g)
    if edit is not None:
        edit(proj, 3, 3 + nq)
    proj = proj.to(dt).float()
    return proj, qb, kb, qw, kw, dev, dt


def _run_attention(run, spec, rotd, proj, qb, kb, qw, kw, cuts, BS, ls=0.8):
    dev, dt = dev_of(run), dt_of(run)
    n = proj.shape[0]
    H, G, D, E = spec.heads, spec.kv_heads, spec.dim, spec.vdim
    nq, nk = H * D, G * D
    freq, mag = Hy.rotary_halves_table(spec.rot, dev)
    vfreq = Hy.rotary_halves_table(spec.value_rot, dev)[0]
    nb = (n + BS - 1) // BS
    perm = torch.randperm(nb + 3, generator=torch.Generator().manual_seed(5))[:nb].to(torch.int32)
    kc = torch.zeros(nb + 3, G, BS, D, dtype=dt, device=dev)
    vc = torch.zeros(nb + 3, G, BS, E, dtype=dt, device=dev)
    bt = perm[None].to(dev)
    out = torch.zeros(n, H * E + 5, dtype=dt, device=dev)
    for rows, rs, pos, sp, cu, sl in spans(cuts):
        T = rows.stop - rows.start
        slot_map = (perm[pos // BS].long() * BS + pos % BS).to(dev)
        p = proj[rows].to(dt).to(dev)
        q = Hy.qkv_prep_wide(p, spec, 3, 3 + nq, 3 + nq + nk, None if qb is None else qb.to(dev),
                             None if kb is None else kb.to(dev), qw.to(dev), kw.to(dev), freq, mag, vfreq, 1e-5, pos.to(dev),
                             kc, vc, slot_map, dt)
        one = T == 1 and rows.start > 0
        splits = 3 if one and dev.type == "cuda" else 1
        buf = torch.zeros(T, H * E + 5, dtype=dt, device=dev)
        o = Hy.gqa_attention(q, kc, vc, bt, cu.to(dev), sp.to(dev), spec.scale, None, 0.0, num_splits=splits, out_dtype=dt,
                             window=spec.window, softcap=spec.softcap, out_scale=1.0 if vfreq is not None else ls,
                             out_buf=None if vfreq is not None else buf, out_off=0 if vfreq is not None else 5)
        if vfreq is not None:
            Hy.turn_back(o, H, pos.to(dev), vfreq, ls, buf, 5)
        out[rows] = buf
    return out[:, 5:].double().cpu()


def _oracle_attention(spec_dict, kind, proj, qb, kb, qw, kw):
    """The oracle's attention with identity projections: h = the projected columns themselves."""
    H, G, D, E = (int(spec_dict[k]) for k in ("heads", "kv_heads", "dim", "vdim"))
    nq, nk = H * D, G * D
    nv = 0 if kind == "parallel_2" else G * E
    width = nq + nk + nv
    h = proj[:, 3:3 + width].double()
    eye = torch.eye(width, dtype=torch.float64)
    P = {"q": eye[:nq], "k": eye[nq:nq + nk], "q.norm": qw.double(), "k.norm": kw.double(),
         "o": torch.eye(H * E, dtype=torch.float64)}
    if kind == "parallel_2":
        P["q.b"], P["k.b"] = qb.double(), kb.double()
    else:
        P["v"] = eye[nq + nk:]
    return O.softmax_attention(h, P, "", spec_dict, 1e-5, kind)


@pytest.mark.parametrize("run", RUNS)
@pytest.mark.parametrize("cuts", [[37], [5, 1, 1, 2, 20, 1, 7]])
def test_attention_halves_soft_cap_turned_values(run, cuts):
    """Whole-row norms, partial rotation in halves with divided frequencies, soft cap, values turned
    and turned back, unequal key and value sizes; prompts, portions and decoded rows (split keys)."""
    d = left(4, 2, 12, 10, rot_dims=8, scaling={"factor": 3.0}, softcap=2.5, scale=0.9)
    spec = config_like(make_config(layers=[par(mlp=None) | {"mixer": {**par()["mixer"], "left": d}}])).layers[0].mixer.left
    proj, qb, kb, qw, kw, dev, dt = _attention_case(run, spec, sum(cuts), 8, 1, False)
    got = _run_attention(run, spec, 8, proj, None, None, qw, kw, cuts, 8)
    want = 0.8 * _oracle_attention(d, "parallel", proj, None, None, qw, kw)
    assert float((got - want).abs().max()) < (0.08 if run[1] == "bf16" else 2e-4)


@pytest.mark.parametrize("run", RUNS)
@pytest.mark.parametrize("window", [1, 6, 16, 17])
def test_window_edges_with_a_key_that_stands_out(run, window):
    """Biased projections, blended frequencies, values = keys, a sliding window. One key of every
    stretch is made to stand out for the queries, so a window that is one token too wide or too
    narrow changes the result by far more than the tolerance: the rows just inside and just
    outside every edge are compared, in a prompt, in portions cut at the edge, and decoded."""
    n, BS = 60, 8
    d = left(2, 1, 8, rot_dims=4, scaling=YARN, window=window, scale=1.0)
    spec = config_like(make_config(layers=[par2(mlp=None) | {"mixer": {**par2()["mixer"], "left": d}}])).layers[0].mixer.left

    def edit(proj, q0, k0):
        proj[:, k0 + 5] = 0.05
        proj[:, q0 + 5] = 6.0
        proj[:, q0 + 8 + 5] = 6.0
        for j in (3, 20, 41):       # these keys dominate every query that still sees them
            proj[j, k0 + 5] = 9.0
    proj, qb, kb, qw, kw, dev, dt = _attention_case(run, spec, n, BS, 2, True, edit)
    qb[:], kb[:] = 0.0, 0.1
    want = 0.8 * _oracle_attention(d, "parallel_2", proj, qb, kb, qw, kw)
    inside, outside = want[20 + window - 1], want[min(20 + window, n - 1)]
    if window > 1:
        assert float((inside - outside).abs().max()) > 0.5      # the edge shows in the oracle itself
    for cuts in ([n], [20 + window - 1, 1, 1, n - 21 - window], [4, 16] + [1] * 40):
        got = _run_attention(run, spec, 4, proj, qb, kb, qw, kw, cuts, BS)
        assert float((got - want).abs().max()) < (0.1 if run[1] == "bf16" else 3e-4), cuts


@pytest.mark.parametrize("run", RUNS)
def test_a_far_key_among_hundreds(run):
    """Causal attention over 700 keys on scattered pages: one early key carries almost all the
    weight of the late queries, so losing it (a page, a tile, a split) shows."""
    n = 700
    d = left(2, 2, 8, 6, rot_dims=8, scaling={"factor": 2.0}, softcap=50.0, scale=1.0)
    spec = config_like(make_config(layers=[par(mlp=None) | {"mixer": {**par()["mixer"], "left": d}}])).layers[0].mixer.left

    def edit(proj, q0, k0):
        proj[:, k0:k0 + 16] *= 0.05
        proj[2, k0:k0 + 16] = 4.0
    proj, _, _, qw, kw, dev, dt = _attention_case(run, spec, n, 16, 3, False, edit)
    qw[:], kw[:] = 1.0, 1.0
    want = 0.8 * _oracle_attention(d, "parallel", proj, None, None, qw, kw)
    got = _run_attention(run, spec, 8, proj, None, None, qw, kw, [650] + [1] * 50, 16)
    assert float((got - want).abs().max()) < (0.1 if run[1] == "bf16" else 3e-4)


def _scan(run, q, k, v, w, a, b, decay, cuts, A, D, E):
    dev = dev_of(run)
    state = torch.full((3, A * D * E), 3.0, device=dev)
    out = []
    f = lambda t, r: None if t is None else t[r].contiguous().to(dev)
    for rows, rs, pos, sp, cu, sl in spans(cuts, slot=2):
        out.append(Hy.state_scan(f(q, rows), f(k, rows), f(v, rows), f(w, rows), f(a, rows), f(b, rows),
                                 None if decay is None else decay.to(dev), state, cu.to(dev), sp.to(dev), sl.to(dev), A, D, E))
    return torch.cat(out).double().cpu()


@pytest.mark.parametrize("run", RUNS[:2])
@pytest.mark.parametrize("A,D,E", [(3, 8, 6), (2, 48, 20), (1, 72, 132), (2, 130, 8)])
@pytest.mark.parametrize("cuts", [[90], [3, 1, 1, 2, 40, 1, 17, 25]])
def test_the_three_recurrences(run, A, D, E, cuts):
    """Constant decay, generalized delta rule and gated delta rule on the one scan, whole and in
    portions (the state carries over), against the oracle's token loops. Sizes beside and beyond a
    wave, key and value sizes that differ."""
    n = sum(cuts)
    g = torch.Generator().manual_seed(D)
    q, k = torch.randn(n, A, D, generator=g) / D ** 0.5, torch.randn(n, A, D, generator=g)
    v = torch.randn(n, A, E, generator=g)
    flat = lambda t: t.reshape(n, -1).contiguous()
    # constant decay per head
    decay = torch.tensor([0.5, 0.93, 0.999][:A])
    want = torch.stack([O.decayed_sum(q[:, i].double(), k[:, i].double(), v[:, i].double(), float(decay[i])) for i in range(A)], 1)
    got = _scan(run, flat(q), flat(k), flat(v), None, None, None, decay, cuts, A, D, E)
    assert float((got - want.reshape(n, -1)).abs().max()) < 2e-3 * float(want.abs().max())
    # generalized delta rule (square state)
    w, a = torch.rand(n, A, D, generator=g) * 0.6 + 0.39, torch.rand(n, A, D, generator=g)
    vv = torch.randn(n, A, D, generator=g)
    u = O.unit_length(k.double()).float()
    want = torch.stack([O.removing_sum(q[:, i].double(), k[:, i].double(), vv[:, i].double(), w[:, i].double(), a[:, i].double())
                        for i in range(A)], 1)
    got = _scan(run, flat(q), flat(k), flat(vv), flat(w), flat(a * u), flat(u), None, cuts, A, D, D)
    assert float((got - want.reshape(n, -1)).abs().max()) < 2e-3 * float(want.abs().max())
    # gated delta rule
    beta, gd = torch.rand(n, A, generator=g), torch.rand(n, A, generator=g) * 0.3 + 0.7
    ku = O.unit_length(k.double()).float()
    want = torch.stack([O.corrected_sum(q[:, i].double(), ku[:, i].double(), v[:, i].double(), beta[:, i].double(), gd[:, i].double())
                        for i in range(A)], 1)
    bk = beta[:, :, None] * ku
    got = _scan(run, flat(q), flat(bk), flat(v), flat(gd[:, :, None].expand(n, A, D)), flat(gd[:, :, None] * bk), flat(ku),
                None, cuts, A, D, E)
    assert float((got - want.reshape(n, -1)).abs().max()) < 2e-3 * float(want.abs().max())


@pytest.mark.parametrize("run", RUNS[:2])
def test_a_far_token_in_the_state(run):
    """A slowly decaying state keeps one early token that the last query asks for, over 600 tokens
    and many portions; a fast one has lost it."""
    n, D, E = 600, 16, 8
    g = torch.Generator().manual_seed(1)
    k = 0.02 * torch.randn(n, 2, D, generator=g)
    q = 0.02 * torch.randn(n, 2, D, generator=g)
    v = torch.randn(n, 2, E, generator=g)
    k[4, :, 3], q[-1, :, 3] = 5.0, 5.0
    decay = torch.tensor([0.999, 0.9])
    flat = lambda t: t.reshape(n, -1).contiguous()
    got = _scan(run, flat(q), flat(k), flat(v), None, None, None, decay, [100, 1, 1, 298] + [1] * 200, 2, D, E)
    want = torch.stack([O.decayed_sum(q[:, i].double(), k[:, i].double(), v[:, i].double(), float(decay[i])) for i in range(2)], 1)
    assert float(want[-1, 0].abs().max()) > 5.0 and float(want[-1, 1].abs().max()) < 1.0
    assert float((got - want.reshape(n, -1)).abs().max()) < 2e-3


@pytest.mark.parametrize("run", RUNS)
@pytest.mark.parametrize("conv", [1, 2, 4])
def test_delta_rule_inputs_across_cuts(run, conv):
    """Short convolutions (state across portions), silu, unit vectors, step size and decay; then the
    scan and the gated per-head norm: the whole gated delta mixer against the oracle."""
    dev, dt = dev_of(run), dt_of(run)
    spec = DeltaSpec(4, 2, 6, 10, conv)
    A, G, D, E, C = 4, 2, 6, 10, spec.conv_channels
    cuts = [5, 1, 2, 1, 1, 14]
    n = sum(cuts)
    g = torch.Generator().manual_seed(conv)
    proj = torch.randn(n, 2 + C + A * E + 2 * A, generator=g).to(dt).float()
    cw = 0.4 * torch.randn(C, conv, generator=g)
    cw[:, -1] += 1.0
    A_log, dtb, nw = torch.randn(A, generator=g) * 0.5, torch.randn(A, generator=g), 0.6 + torch.rand(E, generator=g)
    gq, gk = G * D, 2 * G * D
    eye = torch.eye(proj.shape[1] - 2, dtype=torch.float64)
    P = {"q": eye[:gq], "k": eye[gq:gk], "v": eye[gk:C], "g": eye[C:C + A * E], "b": eye[C + A * E:C + A * E + A],
         "a": eye[C + A * E + A:], "q.conv": cw[:gq].double(), "k.conv": cw[gq:gk].double(), "v.conv": cw[gk:].double(),
         "A_log": A_log.double(), "dt_bias": dtb.double(), "norm": nw.double(), "o": torch.eye(A * E, dtype=torch.float64)}
    want = O.delta_mixer(proj[:, 2:].double(), P, "", {"heads": A, "kv_heads": G, "dim": D, "vdim": E, "conv": conv}, 1e-5)
    sconv = torch.full((3, max(conv - 1, 1), C), 5.0, device=dev)
    rec = torch.full((3, A * D * E), 5.0, device=dev)
    out = []
    for rows, rs, pos, sp, cu, sl in spans(cuts):
        one = rows.stop - rows.start == 1 and rows.start > 0
        p = proj[rows].to(dt).to(dev)
        five, v = Hy.delta_prep(p, spec, 2, 2 + C + A * E, 2 + C + A * E + A, cw.to(dev), sconv, (-torch.exp(A_log)).to(dev),
                                dtb.to(dev), rs.to(dev), pos.to(dev), sp.to(dev), sl.to(dev), shift_state=one)
        if not one:
            Hy.conv_state_update(p, 2, C, sconv, 0, cu.to(dev), sp.to(dev), sl.to(dev))
        o = Hy.state_scan(five[0], five[1], v, five[2], five[3], five[4], None, rec, cu.to(dev), sp.to(dev), sl.to(dev), A, D, E)
        buf = torch.zeros(p.shape[0], A * E, dtype=dt, device=dev)
        out.append(Hy.head_norm_gate(o, nw.to(dev), E, p, 2 + C, "silu", 1e-5, 1.0, buf, 0))
    got = torch.cat(out).double().cpu()
    assert float((got - want).abs().max()) < (0.08 if run[1] == "bf16" else 3e-4)


@pytest.mark.parametrize("run", RUNS)
def test_generalized_delta_inputs_and_whole_row_norm(run):
    dev, dt = dev_of(run), dt_of(run)
    A, D, n = 3, 10, 9
    g = torch.Generator().manual_seed(4)
    N = A * D
    proj = torch.randn(n, 1 + 5 * N, generator=g).to(dt).float()
    lw = torch.randn(n, N, generator=g).to(dt).float()
    w0, ab, nw = torch.randn(N, generator=g), torch.randn(N, generator=g), 0.6 + torch.rand(N, generator=g)
    s = Hy.removal_prep(proj.to(dt).to(dev), 1, 1 + N, 1 + 2 * N, 1 + 3 * N, lw.to(dt).to(dev), w0.to(dev), ab.to(dev), A, D).double().cpu()
    k = proj[:, 1 + N:1 + 2 * N].double().reshape(n, A, D)
    u = O.unit_length(k).reshape(n, N)
    want_w = torch.exp(-math.exp(-0.5) * torch.sigmoid(lw.double() + w0.double()))
    want_a = torch.sigmoid(proj[:, 1 + 3 * N:1 + 4 * N].double() + ab.double()) * u
    for got, want in ((s[0], proj[:, 1:1 + N].double()), (s[3], want_w), (s[4], want_a), (s[5], u)):
        assert float((got - want).abs().max()) < 1e-5
    o = torch.randn(n, N, generator=g)
    for span, weight in ((N, nw), (D, nw), (D, nw[:D])):
        buf = torch.zeros(n, N + 3, dtype=dt, device=dev)
        Hy.head_norm_gate(o.to(dev), weight.to(dev), span, proj.to(dt).to(dev), 1 + 4 * N, "sigmoid", 1e-5, 0.7, buf, 3)
        nrm = O.unit_rms(o.double().reshape(n, N // span, span), 1e-5)
        nrm = (nrm * weight.double()).reshape(n, N) if weight.numel() == span else nrm.reshape(n, N) * weight.double()
        want = nrm * torch.sigmoid(proj[:, 1 + 4 * N:].double()) * 0.7
        assert float((buf[:, 3:].double().cpu() - want).abs().max()) < (0.05 if run[1] == "bf16" else 1e-5)


@pytest.mark.parametrize("run", RUNS)
@pytest.mark.parametrize("rows", [5, 40])
def test_experts_router_and_shared_expert(run, rows):
    """Squared-ReLU experts chosen by the router (softmax over all, the chosen renormalised): the
    row-by-row kernels (few rows) and the expert-by-expert form, against the oracle."""
    dev, dt = dev_of(run), dt_of(run)
    g = torch.Generator().manual_seed(rows)
    W, F, E, top = 24, 10, 5, 2
    h = torch.randn(rows, W, generator=g).to(dt).float()
    P = {"router": torch.randn(E, W, generator=g).double()}
    for e in range(E):
        P[f"e{e}.up"] = (torch.randn(F, W, generator=g) / W ** 0.5).to(dt).double()
        P[f"e{e}.down"] = (torch.randn(W, F, generator=g) / F ** 0.5).to(dt).double()
    want = O.moe_ff(h.double(), P, "", {"router": {"experts": E, "top": top}})
    hd = h.to(dt).to(dev)
    idx, wt = Hy.route_topk(hd, P["router"].float().to(dev), top)          # one launch on the GPU
    idx2, wt2 = Hy.topk_softmax(torch.nn.functional.linear(hd.float(), P["router"].float().to(dev)), top)
    assert torch.equal(idx.cpu(), idx2.cpu()) and float((wt - wt2).abs().max()) < 1e-5
    up = torch.stack([P[f"e{e}.up"] for e in range(E)]).to(dt).to(dev)
    down = torch.stack([P[f"e{e}.down"] for e in range(E)]).to(dt).to(dev)
    for by_row in (None, False):
        got = Hy.moe_experts(hd, idx, wt, up, down, dt, by_row=by_row, act="relu2")
        assert float((got.double().cpu() - want).abs().max()) < (0.15 if run[1] == "bf16" else 1e-4)


# ---- the model through the engine -----------------------------------------------------------------

def test_config_reader_and_registry(tmp_path):
    cfg = make_config()
    make_checkpoint(tmp_path / "m", cfg)
    mc = get_config(str(tmp_path / "m"))
    assert mc.arch == "ledinex" and mc.n_layers == 5 and mc.canon_taps == 3 and mc.logit_scale == 0.6
    m0, m1, m2 = (mc.layers[i].mixer for i in range(3))
    assert isinstance(m0, ParallelSpec) and isinstance(m0.right, RemovalSpec) and m0.left.window == 11 and m0.left.bias
    assert m0.left.value_from_key and m0.left.rot.scaling[0] == "yarn" and m0.left.rot.halves and m0.left.value_rot is None
    assert isinstance(m1, DeltaSpec) and m1.conv == 4 and mc.layers[1].moe.shared_ff == 0 and mc.layers[1].moe.top == 1
    assert isinstance(m2.right, DecaySumSpec) and m2.left.softcap == 9.0 and m2.left.value_rot == RotarySpec(10000.0, 10, None, True)
    assert m2.left.rot.scaling == ("linear", 3.0) and (m2.left_scale, m2.right_scale) == (0.7, 1.2)
    assert mc.layers[3].ff == 0 and mc.layers[0].moe.act == "relu2" and mc.layers[0].moe.shared_ff == 24
    e = engine_for(tmp_path / "m", ("cpu", "fp32"))
    assert type(e.model).__name__ == "LedinexModel" and e.kv.conv[0].shape == (5, 2, 2, 40)
    assert e.kv.k_layer(1) is None and e.kv.sconv[1].shape == (5, 3, 2 * 2 * 6 + 4 * 10) and e.kv.sconv[0] is None
    assert e.kv.rec[2].shape == (5, 3 * 8 * 6)
    bad = make_config(layers=[dict(par(), type="wkv")])
    with pytest.raises(ValueError):
        config_like(bad)
    assert get_config("tiny-ledinex").arch == "ledinex"


@pytest.mark.parametrize("run", RUNS)
def test_whole_prompt_and_layers(tmp_path, run):
    cfg = settle(make_config(), run)
    P = make_checkpoint(tmp_path / "m", cfg, seed=1)
    e = engine_for(tmp_path / "m", run)
    t = toks(45, cfg["vocab"], 1)
    layers = []
    want = O.forward(cfg, P, t, layers)
    got = e.step([("a", t, list(range(len(t))))])
    close(got, want, run, "logits")
    s = e.kv.seq("b")
    tok, pos, meta = e._varlen_meta([e.reserve(s, t)])
    keep = []
    with torch.no_grad():
        e.model.forward(tok, pos, e.kv, meta, keep_layers=keep)
    assert len(keep) == len(layers) == 5
    for i, (a, b) in enumerate(zip(keep, layers)):
        err = (a.double().cpu() - b).abs().max(-1).values
        assert float(err.median() if run[1] == "bf16" else err.max()) < (0.2 if run[1] == "bf16" else 1e-3), \
            f"residual stream after layer {i}"


SHAPES = {
    # one query head per key/value head; one key/value head for all; one expert of one, all experts; five taps
    "groups": (5, [par(3, 3, 8, 8, 1, 6, 10, rot_dims=4, mlp=moe(3, 1, 12, 8)), par2(5, 1, 6, 1, 12, rot_dims=6, mlp=moe(3, 3, 8, 0))]),
    # heads wider than a wave's 64 lanes; states of 72 x 132 and 130 x 130
    "wide": (2, [par(2, 1, 72, 132, 1, 72, 132, rot_dims=40, mlp=None), par2(1, 1, 68, 1, 130, rot_dims=68, window=3, mlp=None),
                 delta(2, 1, 80, 70, conv=3, mlp=None)]),
    # more query heads per key/value head than one attention workgroup's pairs
    "many-heads": (3, [par(40, 1, 4, 4, 2, 4, 4, rot_dims=2)]),
    # no convolution beyond the current token, a window of one token, constants that are 1, no scaling of frequencies
    "ones": (1, [par2(1, 1, 4, 1, 4, window=1, rot_dims=4, scaling=None, ls=1.0, rs=1.0, scale=1.0, mlp=None),
                 par(1, 1, 4, 4, 1, 4, 4, decay=[1.0], softcap=None, scaling=None, ls=1.0, rs=1.0, mlp=moe(1, 1, 8, 0)),
                 delta(1, 1, 4, 4, conv=1)]),
    # only delta layers; value heads over fewer key heads
    "delta-only": (4, [delta(6, 2, 4, 6, conv=5), delta(2, 2, 10, 4, conv=2, mlp=None)]),
    # a ramp of blended frequencies that collapses to one step
    "steep": (3, [par2(2, 2, 8, 2, 4, rot_dims=8, scaling={"factor": 2.0, "original": 16, "fast": 2.0, "slow": 2.0})]),
}


@pytest.mark.parametrize("run", RUNS)
@pytest.mark.parametrize("shape", list(SHAPES))
def test_other_sizes(tmp_path, run, shape):
    """Sizes and constants that the usual test model makes equal or 1."""
    taps, layers = SHAPES[shape]
    one = shape == "ones"
    cfg = settle(make_config(width=24, vocab=61, layers=layers, taps=taps, embed_scale=1.0 if one else 1.9,
                             logit_scale=1.0 if one else 0.4), run)
    P = make_checkpoint(tmp_path / "m", cfg, seed=2)
    e = engine_for(tmp_path / "m", run, block_size=8)
    t = toks(70, cfg["vocab"], 2)
    want = O.forward(cfg, P, t)
    got = torch.cat([e.step([("a", t[:37], list(range(37)))]), e.step([("a", t[37:39], [0, 1])])] +
                    [e.step([("a", t[i:i + 1], [0])]) for i in range(39, 70)])
    close(got, want, run, shape)


@pytest.mark.parametrize("run", RUNS)
def test_wider_layers(tmp_path, run):
    """Rows wide enough for several waves per workgroup, 64-wide attention and recurrence heads, a
    window that crosses many key tiles and pages, eight experts: a prompt in portions (the first
    spans many scan chunks), then decoded tokens."""
    layers = [par2(8, 2, 64, 4, 64, window=200, rot_dims=32, mlp=moe(8, 2, 128, 256)),
              delta(8, 4, 64, 64, mlp=moe(8, 2, 128, 256)), par(8, 2, 64, 64, 4, 64, 64, rot_dims=64, mlp=moe(8, 2, 128, 256))]
    cfg = settle(make_config(width=512, vocab=331, layers=layers), run)
    P = make_checkpoint(tmp_path / "m", cfg, seed=21)
    e = engine_for(tmp_path / "m", run, tokens=1024, block_size=32)
    t = toks(520, cfg["vocab"], 21)
    want = O.forward(cfg, P, t)
    got = [e.step([("a", t[:300], [0, 199, 200, 201, 299])]), e.step([("a", t[300:302], [0, 1])]),
           e.step([("a", t[302:500], [0, 197])])] + [e.step([("a", t[i:i + 1], [0])]) for i in range(500, 520)]
    rows = [0, 199, 200, 201, 299, 300, 301, 302, 499] + list(range(500, 520))
    close(torch.cat(got), want[rows], run, "wider layers")


# ---- portions, decoding, batches ------------------------------------------------------------------

@pytest.mark.parametrize("run", RUNS)
def test_prefill_against_token_by_token(tmp_path, run):
    cfg = settle(make_config(), run)
    P = make_checkpoint(tmp_path / "m", cfg, seed=3)
    e = engine_for(tmp_path / "m", run)
    t = toks(40, cfg["vocab"], 3)
    want = O.forward(cfg, P, t)
    one = torch.cat([e.step([("a", [x], [0])]) for x in t])          # from the first token on
    close(one, want, run, "token by token")
    whole = e.step([("b", t, list(range(40)))])
    close(whole, want, run, "whole")
    if run[1] != "bf16":
        assert float((one - whole).abs().max()) < 1e-3


@pytest.mark.parametrize("run", RUNS)
@pytest.mark.parametrize("cuts", [[2, 2, 3, 1, 30, 2, 17, 1, 1, 5], [16, 16, 16, 16], [1, 63], [33, 31], [131, 2, 70]])
def test_portions(tmp_path, run, cuts):
    """Portions of several sizes, down to two tokens and one, cut inside and at page borders (pages
    of 16), inside windows (11 and 5) and inside the convolutions' reach: the convolution states
    and the matrix states carry over every cut."""
    cfg = settle(make_config(), run)
    P = make_checkpoint(tmp_path / "m", cfg, seed=4)
    e = engine_for(tmp_path / "m", run)
    t = toks(sum(cuts), cfg["vocab"], 4)
    want = O.forward(cfg, P, t)
    out, at = [], 0
    for n in cuts:
        out.append(e.step([("a", t[at:at + n], list(range(n)))]))
        at += n
    close(torch.cat(out), want, run, f"portions {cuts}")


@pytest.mark.parametrize("run", RUNS)
def test_mixed_batch_equals_each_alone_and_slots_are_reused(tmp_path, run):
    """Unequal requests in one batch (portions beside single tokens, requests paused for a step),
    a pool of four state slots and few pages, so both are freed and used again: a request that
    takes a used slot starts from zero matrix states and zero convolution rows."""
    cfg = settle(make_config(), run)
    P = make_checkpoint(tmp_path / "m", cfg, seed=5)
    e = engine_for(tmp_path / "m", run, tokens=160, slots=4)
    V = cfg["vocab"]
    reqs = {k: toks(n, V, 10 + i) for i, (k, n) in enumerate([("a", 50), ("b", 7), ("c", 33), ("d", 1), ("e", 41), ("f", 20)])}
    want = {k: O.forward(cfg, P, v) for k, v in reqs.items()}
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
    if run[1] == "bf16":        # judged together: a request of one row has no median to speak of
        close(torch.cat([torch.cat(got[k]) for k in reqs]), torch.cat([want[k] for k in reqs]), run, "all requests")
    else:
        for k in reqs:
            close(torch.cat(got[k]), want[k], run, f"request {k}")
    assert e.kv.alloc.num_free == e.kv.num_blocks and len(e.kv.state.free) == 4
    with pytest.raises(KVCacheOOM):       # a fifth live request has no slot
        for i in range(5):
            e.step([(f"x{i}", [1, 2], [])])


@pytest.mark.parametrize("run", RUNS)
def test_long_decoding_past_windows_and_page_borders(tmp_path, run):
    """150 tokens, all but five decoded one by one through pages of 8: every window (11 and 5)
    slides over decoded tokens many times."""
    cfg = settle(make_config(), run)
    P = make_checkpoint(tmp_path / "m", cfg, seed=7)
    e = engine_for(tmp_path / "m", run, block_size=8)
    t = toks(150, cfg["vocab"], 7)
    want = O.forward(cfg, P, t)
    got = torch.cat([e.step([("a", t[:5], list(range(5)))])] + [e.step([("a", [x], [0])]) for x in t[5:]])
    close(got, want, run, "long decode")


# ---- the engine's own generation path and scheduler -----------------------------------------------

def _greedy_oracle(P, cfg, prompt, n):
    seq = list(prompt)
    for _ in range(n):
        seq.append(int(O.forward(cfg, P, seq)[-1].argmax()))
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
    layers = [par2(4, 2, 16, 2, 16, rot_dims=8, mlp=moe(6, 2, 32, 64)), delta(4, 2, 16, 16, mlp=moe(6, 2, 32, 64)),
              par(4, 2, 16, 16, 2, 16, 16, rot_dims=16, mlp=moe(6, 2, 32, 64))]
    cfg = settle(make_config(width=64, vocab=80, layers=layers), ("cuda:0", "bf16"))
    P = make_checkpoint(tmp_path / "m", cfg, seed=11)
    t = toks(60, cfg["vocab"], 11)
    want = O.forward(cfg, P, t)
    outs = []
    for skinny in (True, False):
        e = engine_for(tmp_path / "m", ("cuda:0", "bf16"))
        e.model.use_skinny = skinny
        got = torch.cat([e.step([("a", t[:20], list(range(20)))])] + [e.step([("a", [x], [0])]) for x in t[20:]])
        close(got, want, ("cuda:0", "bf16"), f"skinny={skinny}")
        outs.append(got)
        if skinny:
            assert all("w_out" in d and "mlp.shared.down" in d for d in e.model._dec.values())
    assert float((outs[0] - outs[1]).abs().max(-1).values.median()) < 0.25


def test_serving_entry_points_match_run_turns():
    """The continuous-batching entry points (prefill + first token, then decode in chunks while the
    state follows) give the tokens of a single run_turns call; random-init preset weights."""
    def eng():
        return Engine(EngineConfig(model="tiny-ledinex", weights="random:3", dtype="fp32", device="cpu",
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


def test_trace_runner_replays_steps(tmp_path):
    """The trace runner's own entry point on the CPU: steps in, logit files out, pages and slots
    given back at the end of a request."""
    import io
    import sys
    import numpy as np
    from theroundtaible_amd import trace_run
    cfg = make_config(vocab=50)
    P = make_checkpoint(tmp_path / "m", cfg, seed=9)
    t = toks(30, 50, 9)
    want = O.forward(cfg, P, t)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": t[:20], "want": [0, 19]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": t[20:22], "want": []}], "end": []},
             {"step": 2, "entries": [{"id": "a", "tokens": t[22:], "want": [7]}, {"id": "b", "tokens": t[:3], "want": [2]}],
              "end": ["a", "b"]}]
    old_in, old_out = sys.stdin, sys.stdout
    sys.stdin, sys.stdout = io.StringIO("\n".join(json.dumps(s) for s in steps) + "\n"), io.StringIO()
    try:
        rc = trace_run.main(["--model", str(tmp_path / "m"), "--dtype", "float32", "--out", str(tmp_path / "o"),
                             "--max-tokens", "128", "--device", "cpu"])
        said = sys.stdout.getvalue()
    finally:
        sys.stdin, sys.stdout = old_in, old_out
    assert rc == 0 and [l for l in said.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    assert not os.path.exists(tmp_path / "o" / "1.f32")
    a = np.fromfile(tmp_path / "o" / "0.f32", dtype="<f4").reshape(2, 50)
    b = np.fromfile(tmp_path / "o" / "2.f32", dtype="<f4").reshape(2, 50)
    got = torch.tensor(np.concatenate([a, b])).double()
    assert float((got - want[[0, 19, 29, 2]]).abs().max()) < 2e-3
