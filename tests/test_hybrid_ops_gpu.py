"""Every HIP kernel of ``csrc/hybrid/`` against its PyTorch statement (``ops/hybrid.py`` ``ref_*``,
run on fp32 CPU copies of the same inputs), at sizes that are not multiples of the kernels' tile
shapes, in fp32 and bf16."""
import pytest
import torch

from theroundtaible_amd.models.config import GroupedAttentionSpec
from theroundtaible_amd.ops import hybrid as Hy

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]


def tol(dt):
    return dict(rtol=2e-2, atol=2e-2) if dt == torch.bfloat16 else dict(rtol=1e-4, atol=1e-5)


def spans(lens, starts):
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    row_seq = torch.repeat_interleave(torch.arange(len(lens), dtype=torch.int32), torch.tensor(lens))
    pos = torch.cat([torch.arange(s, s + n) for s, n in zip(starts, lens)])
    return cu, row_seq, pos, torch.tensor(starts, dtype=torch.int32)


def gpu(*ts):
    return [t.to(DEV) if t is not None else None for t in ts]


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("W", [20, 200, 1100])
def test_shift_norm_and_state(dt, W):
    Hy.native()
    g = torch.Generator().manual_seed(W)
    lens, starts = [5, 1, 1, 9], [0, 0, 7, 3]
    cu, row_seq, pos, sp = spans(lens, starts)
    T = sum(lens)
    slots = torch.tensor([2, 0, 3, 1], dtype=torch.int32)
    x, y = torch.randn(T, W, generator=g), torch.randn(T, W, generator=g).to(dt)
    w, mu, state = torch.rand(W, generator=g) + 0.5, torch.rand(W, generator=g), torch.randn(5, W, generator=g)
    for yy in (y, None):
        st_c, st_g = state.clone(), state.clone().to(DEV)
        want, xs = Hy.ref_shift_norm(x.clone(), yy, w, 1e-5, mu, st_c, row_seq, pos, sp, slots, torch.float32)
        Hy.ref_shift_state_update(xs, w, 1e-5, st_c, cu, slots)
        got, xg = Hy.shift_norm(*gpu(x, yy, w), 1e-5, *gpu(mu, st_g, row_seq, pos, sp, slots), dt)
        Hy.shift_state_update(xg, w.to(DEV), 1e-5, st_g, cu.to(DEV), slots.to(DEV))
        torch.testing.assert_close(got.float().cpu(), want, **tol(dt))
        torch.testing.assert_close(xg.cpu(), xs, rtol=1e-6, atol=1e-6)
        torch.testing.assert_close(st_g.cpu(), st_c, rtol=1e-5, atol=1e-5)
    # one row per sequence, the state stored by the same launch
    B = 4
    cu, row_seq, pos, sp = spans([1] * B, [0, 4, 9, 1])
    st_c, st_g = state.clone(), state.clone().to(DEV)
    want, _ = Hy.ref_shift_norm(x[:B].clone(), None, w, 1e-5, mu, st_c, row_seq, pos, sp, slots, torch.float32, True)
    got, _ = Hy.shift_norm(*gpu(x[:B], None, w), 1e-5, *gpu(mu, st_g, row_seq, pos, sp, slots), dt, shift_state=True)
    torch.testing.assert_close(got.float().cpu(), want, **tol(dt))
    torch.testing.assert_close(st_g.cpu(), st_c, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("shape", [(4, 2, 12, 20, 6, False), (3, 3, 72, 72, 0, True), (5, 1, 130, 200, 130, False),
                                   (2, 1, 1, 1, 0, False)])
def test_qk_prep(dt, shape):
    H, G, Dk, Dv, rot, vk = shape
    g = torch.Generator().manual_seed(Dk)
    T, BS, nb = 11, 4, 6
    spec = GroupedAttentionSpec(H, G, Dk, Dv, 1.0, value_from_key=vk)
    N = 3 + H * Dk + G * Dk + (0 if vk else G * Dv)
    proj = torch.randn(T, N, generator=g).to(dt)
    inv = (torch.rand(rot // 2, generator=g) if rot else None)
    pos = torch.tensor([0, 1, 2, 3, 40, 41, 900, 901, 5000, 70000, 7])
    slots = torch.randperm(nb * BS, generator=g)[:T]
    kc, vc = torch.zeros(nb, G, BS, Dk, dtype=dt), torch.zeros(nb, G, BS, Dv, dtype=dt)
    want = Hy.ref_qk_prep(proj, spec, 3, 3 + H * Dk, 3 + (H + G) * Dk, inv, 1e-5, pos, kc, vc, slots, torch.float32)
    kg, vg = torch.zeros_like(kc).to(DEV), torch.zeros_like(vc).to(DEV)
    got = Hy.qk_prep(proj.to(DEV), spec, 3, 3 + H * Dk, 3 + (H + G) * Dk, inv.to(DEV) if rot else None, 1e-5, pos.to(DEV),
                     kg, vg, slots.to(DEV), dt)
    # (angles of far positions in fp32: the two sides round p * f alike, the sine differs by ulps)
    t = dict(rtol=2e-2, atol=2e-2) if dt == torch.bfloat16 else dict(rtol=1e-3, atol=1e-4)
    torch.testing.assert_close(got.float().cpu(), want, **t)
    torch.testing.assert_close(kg.float().cpu(), kc.float(), **t)
    torch.testing.assert_close(vg.float().cpu(), vc.float(), rtol=0, atol=0)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("shape", [(6, 2, 12, 12, 16), (4, 4, 40, 20, 64), (5, 1, 72, 132, 8), (40, 1, 8, 8, 16),
                                   (8, 2, 128, 128, 32), (2, 1, 256, 256, 16)])
def test_gqa_attention_varlen_and_split(dt, shape):
    H, G, Dk, Dv, BS = shape
    g = torch.Generator().manual_seed(H * Dk)
    lens, starts = [37, 1, 2, 70], [0, 130, 63, 5]
    cu, _, _, sp = spans(lens, starts)
    T = sum(lens)
    ctx = [s + n for s, n in zip(starts, lens)]
    nblk = [(c + BS - 1) // BS for c in ctx]
    nb = sum(nblk) + 2
    perm = torch.randperm(nb, generator=g).tolist()
    bt = torch.zeros(len(lens), max(nblk), dtype=torch.int32)
    for s, n in enumerate(nblk):
        bt[s, :n] = torch.tensor([perm.pop() for _ in range(n)])
    kc = (torch.randn(nb, G, BS, Dk, generator=g) * 0.5).to(dt)
    vc = torch.randn(nb, G, BS, Dv, generator=g).to(dt)
    q = torch.randn(T, H, Dk, generator=g).to(dt)
    temp = torch.rand(H, generator=g) + 0.5
    for sink, tp in ((1.0, temp), (0.0, None)):
        want = Hy.ref_gqa_attention(q.float(), kc.float(), vc.float(), bt, cu, sp, 0.3, tp, sink, torch.float32)
        got = Hy.gqa_attention(*gpu(q, kc, vc, bt, cu, sp), 0.3, tp.to(DEV) if tp is not None else None, sink)
        torch.testing.assert_close(got.float().cpu(), want, **tol(dt))
    # one row per sequence with split keys (2, 7, 32 ranges)
    B = len(lens)
    last = torch.tensor([c - 1 for c in ctx], dtype=torch.int32)
    rows = torch.tensor([int(cu[s + 1]) - 1 for s in range(B)])
    cu1 = torch.arange(B + 1, dtype=torch.int32)
    want = Hy.ref_gqa_attention(q[rows].float(), kc.float(), vc.float(), bt, cu1, last, 0.3, temp, 1.0, torch.float32)
    tiles = torch.stack([torch.arange(B), torch.arange(B)], 1).to(torch.int32)
    for splits in (2, 7, 32):
        got = Hy.gqa_attention(*gpu(q[rows].contiguous(), kc, vc, bt, cu1, last), 0.3, temp.to(DEV), 1.0, tiles=tiles.to(DEV),
                               num_splits=splits)
        torch.testing.assert_close(got.float().cpu(), want, **tol(dt))


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("width", [7, 232, 300])
def test_mingru_scan(dt, width):
    g = torch.Generator().manual_seed(width)
    lens, starts = [33, 1, 1, 130], [0, 0, 12, 3]
    cu, _, _, sp = spans(lens, starts)
    T = sum(lens)
    slots = torch.tensor([1, 3, 0, 2], dtype=torch.int32)
    proj = torch.randn(T, 5 + 3 * width, generator=g).to(dt)
    bz, bx, state = torch.randn(width, generator=g), torch.randn(width, generator=g), torch.randn(4, width, generator=g)
    st_c, st_g = state.clone(), state.clone().to(DEV)
    want = Hy.ref_mingru_scan(proj, 5, 5 + 2 * width, 5 + width, width, bz, bx, st_c, cu, sp, slots, torch.float32)
    got = Hy.mingru_scan(proj.to(DEV), 5, 5 + 2 * width, 5 + width, width, *gpu(bz, bx, st_g, cu, sp, slots), dt)
    torch.testing.assert_close(got.float().cpu(), want, **tol(dt))
    torch.testing.assert_close(st_g.cpu(), st_c, rtol=1e-4, atol=1e-5)
    # the chunked scan (spans of 130 rows = two chunks and a short one, beside single rows)
    ch = Hy.scan_chunks(cu, DEV)
    assert ch is not None and ch[0].shape[0] == 6 and ch[1].tolist() == [0, 1, 2, 3, 6]
    st_g = state.clone().to(DEV)
    got = Hy.mingru_scan(proj.to(DEV), 5, 5 + 2 * width, 5 + width, width, *gpu(bz, bx, st_g, cu, sp, slots), dt, chunks=ch)
    torch.testing.assert_close(got.float().cpu(), want, **tol(dt))
    torch.testing.assert_close(st_g.cpu(), st_c, rtol=1e-4, atol=1e-5)
    assert Hy.scan_chunks(torch.tensor([0, 64, 65]), DEV) is None


@pytest.mark.parametrize("dt", DTYPES)
def test_normed_adds_and_activation(dt):
    g = torch.Generator().manual_seed(0)
    T, W, F = 13, 200, 77
    x = torch.randn(T, W, generator=g)
    a, b = torch.randn(T, W, generator=g).to(dt), (3 * torch.randn(T, W, generator=g)).to(dt)
    wa, wb = torch.rand(W, generator=g), torch.rand(W, generator=g)
    xg = x.clone().to(DEV)
    Hy.dual_norm_add_(xg, *gpu(a, wa, b, wb), 1e-5)
    torch.testing.assert_close(xg.cpu(), Hy.ref_dual_norm_add_(x.clone(), a, wa, b, wb, 1e-5), rtol=1e-5, atol=1e-5)
    for y in (a, None):
        xc, xg = x.clone(), x.clone().to(DEV)
        want = Hy.ref_add_norm(xc, y, wa, 1e-5, torch.float32)
        got = Hy.add_norm(xg, y.to(DEV) if y is not None else None, wa.to(DEV), 1e-5, dt)
        torch.testing.assert_close(got.float().cpu(), want, **tol(dt))
        torch.testing.assert_close(xg.cpu(), xc, rtol=1e-6, atol=1e-6)
    gu = (2 * torch.randn(T, 2 * F, generator=g)).to(dt)
    torch.testing.assert_close(Hy.limited_glu(gu.to(DEV), 1.5, dt).float().cpu(), Hy.ref_limited_glu(gu, 1.5, torch.float32),
                               **tol(dt))


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("W,groups", [(24, 3), (200, 2), (1100, 5)])
def test_grouped_norm_and_several_mixes(dt, W, groups):
    """The norm over equal parts of a row, and several token-shift mixes of one row in a launch."""
    g = torch.Generator().manual_seed(W)
    lens, starts = [5, 1, 1, 9], [0, 0, 7, 3]
    cu, row_seq, pos, sp = spans(lens, starts)
    T = sum(lens)
    slots = torch.tensor([2, 0, 3, 1], dtype=torch.int32)
    x = torch.randn(T, W, generator=g) * torch.linspace(0.1, 4.0, W)
    y = torch.randn(T, W, generator=g).to(dt)
    w, mu, state = torch.rand(W, generator=g) + 0.5, torch.rand(5, W, generator=g), torch.randn(5, W, generator=g)
    for yy in (y, None):
        st_c, st_g = state.clone(), state.clone().to(DEV)
        want, xs = Hy.ref_shift_norm(x.clone(), yy, w, 1e-5, mu, st_c, row_seq, pos, sp, slots, torch.float32, groups=groups)
        Hy.ref_shift_state_update(xs, w, 1e-5, st_c, cu, slots, groups)
        got, xg = Hy.shift_norm(*gpu(x, yy, w), 1e-5, *gpu(mu, st_g, row_seq, pos, sp, slots), dt, groups=groups)
        Hy.shift_state_update(xg, w.to(DEV), 1e-5, st_g, cu.to(DEV), slots.to(DEV), groups)
        assert got.shape == (5, T, W)
        torch.testing.assert_close(got.float().cpu(), want, **tol(dt))
        torch.testing.assert_close(xg.cpu(), xs, rtol=1e-6, atol=1e-6)
        torch.testing.assert_close(st_g.cpu(), st_c, rtol=1e-5, atol=1e-5)
        xc, xg = x.clone(), x.clone().to(DEV)
        want = Hy.ref_add_norm(xc, yy, w, 1e-5, torch.float32, groups)
        got = Hy.add_norm(xg, yy.to(DEV) if yy is not None else None, w.to(DEV), 1e-5, dt, groups)
        torch.testing.assert_close(got.float().cpu(), want, **tol(dt))
        torch.testing.assert_close(xg.cpu(), xc, rtol=1e-6, atol=1e-6)
    B = 4
    cu, row_seq, pos, sp = spans([1] * B, [0, 4, 9, 1])
    st_c, st_g = state.clone(), state.clone().to(DEV)
    want, _ = Hy.ref_shift_norm(x[:B].clone(), None, w, 1e-5, mu, st_c, row_seq, pos, sp, slots, torch.float32, True, groups)
    got, _ = Hy.shift_norm(*gpu(x[:B], None, w), 1e-5, *gpu(mu, st_g, row_seq, pos, sp, slots), dt, shift_state=True,
                           groups=groups)
    torch.testing.assert_close(got.float().cpu(), want, **tol(dt))
    torch.testing.assert_close(st_g.cpu(), st_c, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("shape", [(4, 2, 12, 20), (3, 3, 72, 72), (5, 1, 130, 200)])
def test_qk_prep_weights_factor_and_value_norm(dt, shape):
    H, G, Dk, Dv = shape
    g = torch.Generator().manual_seed(Dk)
    T, BS, nb = 11, 4, 6
    spec = GroupedAttentionSpec(H, G, Dk, Dv, 1.0, qk_weight=True, q_temp=(0.7, 3), value_norm=True)
    N = 3 + H * Dk + G * Dk + G * Dv
    proj = torch.randn(T, N, generator=g).to(dt)
    qw, kw = torch.rand(Dk, generator=g) + 0.5, torch.rand(Dk, generator=g) + 0.5
    pos = torch.tensor([0, 1, 2, 3, 40, 41, 900, 901, 5000, 70000, 7])
    slots = torch.randperm(nb * BS, generator=g)[:T]
    kc, vc = torch.zeros(nb, G, BS, Dk, dtype=dt), torch.zeros(nb, G, BS, Dv, dtype=dt)
    want = Hy.ref_qk_prep(proj, spec, 3, 3 + H * Dk, 3 + (H + G) * Dk, None, 1e-5, pos, kc, vc, slots, torch.float32, qw, kw)
    kg, vg = torch.zeros_like(kc).to(DEV), torch.zeros_like(vc).to(DEV)
    got = Hy.qk_prep(proj.to(DEV), spec, 3, 3 + H * Dk, 3 + (H + G) * Dk, None, 1e-5, pos.to(DEV), kg, vg, slots.to(DEV), dt,
                     q_weight=qw.to(DEV), k_weight=kw.to(DEV))
    t = dict(rtol=2e-2, atol=2e-2) if dt == torch.bfloat16 else dict(rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(got.float().cpu(), want, **t)
    torch.testing.assert_close(kg.float().cpu(), kc.float(), **t)
    torch.testing.assert_close(vg.float().cpu(), vc.float(), **t)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("shape", [(6, 2, 12, 12, 16, 9), (4, 4, 40, 20, 64, 64), (5, 1, 72, 132, 8, 1), (40, 1, 8, 8, 16, 100),
                                   (2, 1, 256, 256, 16, 33)])
def test_gqa_attention_window_penalty_and_gate(dt, shape):
    H, G, Dk, Dv, BS, window = shape
    g = torch.Generator().manual_seed(H * Dk)
    lens, starts = [37, 1, 2, 70], [0, 130, 63, 5]
    cu, _, _, sp = spans(lens, starts)
    T = sum(lens)
    ctx = [s + n for s, n in zip(starts, lens)]
    nblk = [(c + BS - 1) // BS for c in ctx]
    nb = sum(nblk) + 2
    perm = torch.randperm(nb, generator=g).tolist()
    bt = torch.zeros(len(lens), max(nblk), dtype=torch.int32)
    for s, n in enumerate(nblk):
        bt[s, :n] = torch.tensor([perm.pop() for _ in range(n)])
    kc = (torch.randn(nb, G, BS, Dk, generator=g) * 0.5).to(dt)
    vc = torch.randn(nb, G, BS, Dv, generator=g).to(dt)
    q = torch.randn(T, H, Dk, generator=g).to(dt)
    slopes = torch.tensor([2.0 ** (-8.0 * (a + 1) / H) for a in range(H)])
    gate = torch.randn(T, 5 + H * Dv, generator=g).to(dt)
    want = Hy.ref_gqa_attention(q.float(), kc.float(), vc.float(), bt, cu, sp, 0.3, None, 0.0, torch.float32, window, slopes,
                                gate.float(), 5)
    got = Hy.gqa_attention(*gpu(q, kc, vc, bt, cu, sp), 0.3, None, 0.0, window=window, slopes=slopes.to(DEV),
                           gate=gate.to(DEV), gate_off=5)
    torch.testing.assert_close(got.float().cpu(), want, **tol(dt))
    B = len(lens)
    last = torch.tensor([c - 1 for c in ctx], dtype=torch.int32)
    rows = torch.tensor([int(cu[s + 1]) - 1 for s in range(B)])
    cu1 = torch.arange(B + 1, dtype=torch.int32)
    g1 = gate[rows].contiguous()
    want = Hy.ref_gqa_attention(q[rows].float(), kc.float(), vc.float(), bt, cu1, last, 0.3, None, 0.0, torch.float32, window,
                                slopes, g1.float(), 5)
    tiles = torch.stack([torch.arange(B), torch.arange(B)], 1).to(torch.int32)
    for splits in (2, 7):
        got = Hy.gqa_attention(*gpu(q[rows].contiguous(), kc, vc, bt, cu1, last), 0.3, None, 0.0, tiles=tiles.to(DEV),
                               num_splits=splits, window=window, slopes=slopes.to(DEV), gate=g1.to(DEV), gate_off=5)
        torch.testing.assert_close(got.float().cpu(), want, **tol(dt))


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("H,D", [(3, 5), (2, 48), (2, 64), (1, 100), (1, 130)])
def test_wkv_scan(dt, H, D):
    """One launch over whole spans and the three chunked launches, states of several sizes (a
    wave, part of one, two and three waves of value columns), spans beside single rows."""
    g = torch.Generator().manual_seed(D)
    lens, starts = [33, 1, 1, 150], [0, 0, 12, 3]
    cu, _, _, sp = spans(lens, starts)
    T = sum(lens)
    slots = torch.tensor([1, 3, 0, 2], dtype=torch.int32)
    rkvg = (torch.randn(4, T, H * D, generator=g) * 0.7).to(dt)
    lw = torch.randn(T, H * D, generator=g).to(dt)
    w0 = -3.0 + 3.0 * torch.rand(H * D, generator=g)
    u, nw = torch.randn(H, D, generator=g), torch.rand(H * D, generator=g) + 0.5
    state = torch.randn(4, H * D * D, generator=g)
    st_c = state.clone()
    want = Hy.ref_wkv_scan(rkvg, lw, w0, u, nw, 1e-5, st_c, cu, sp, slots, torch.float32)
    t = dict(rtol=3e-2, atol=3e-2) if dt == torch.bfloat16 else dict(rtol=1e-3, atol=1e-4)
    for chunks in (None, Hy.wkv_chunks(cu, DEV)):
        st_g = state.clone().to(DEV)
        got = Hy.wkv_scan(*gpu(rkvg, lw, w0, u, nw), 1e-5, *gpu(st_g, cu, sp, slots), dt, chunks=chunks)
        torch.testing.assert_close(got.float().cpu(), want, **t)
        torch.testing.assert_close(st_g.cpu(), st_c, rtol=1e-3, atol=1e-4)
    assert Hy.wkv_chunks(cu, DEV)[1].tolist() == [0, 2, 3, 4, 9] and Hy.wkv_chunks(torch.tensor([0, 64, 66]), DEV) is None


@pytest.mark.parametrize("dt", DTYPES)
def test_feed_forward_kernels(dt):
    g = torch.Generator().manual_seed(1)
    T, W, F, E, top = 7, 72, 40, 11, 3
    a = (2 * torch.randn(T, F, generator=g)).to(dt)
    bias = torch.randn(F, generator=g)
    for b in (bias, None):
        got = Hy.xielu(a.to(DEV), b.to(DEV) if b is not None else None, 0.8, 1.3, dt)
        torch.testing.assert_close(got.float().cpu(), Hy.ref_xielu(a, b, 0.8, 1.3, torch.float32), **tol(dt))
    gu = (2 * torch.randn(T, 2 * F, generator=g)).to(dt)
    torch.testing.assert_close(Hy.silu_glu(gu.to(DEV), dt).float().cpu(), Hy.ref_silu_glu(gu, torch.float32), **tol(dt))
    for n_exp, k in ((E, top), (1, 1), (70, 70), (300, 5)):
        logits = torch.randn(T, n_exp, generator=g)
        idx, wt = Hy.topk_softmax(logits.to(DEV), k)
        val, widx = torch.topk(logits, k, dim=-1)
        assert idx.cpu().tolist() == widx.tolist()
        torch.testing.assert_close(wt.cpu(), torch.softmax(val, -1), rtol=1e-5, atol=1e-6)
    # the experts row by row (two launches) against expert by expert (library GEMMs) and the statement
    h = torch.randn(T, W, generator=g).to(dt)
    w_gu = (torch.randn(E, 2 * F, W, generator=g) / W ** 0.5).to(dt)
    w_d = (torch.randn(E, W, F, generator=g) / F ** 0.5).to(dt)
    idx, wt = Hy.topk_softmax(torch.randn(T, E, generator=g).to(DEV), top)
    want = Hy.moe_experts(h.float(), idx.cpu(), wt.cpu(), w_gu.float(), w_d.float(), torch.float32)
    for by_row in (True, False):
        got = Hy.moe_experts(*gpu(h, idx, wt, w_gu, w_d), dt, by_row=by_row)
        torch.testing.assert_close(got.float().cpu(), want, **tol(dt))
    # rows whose length is no multiple of the 16-byte loads
    h2, w2, d2 = h[:, :W - 3].contiguous(), w_gu[:, :, :W - 3].contiguous(), w_d[:, :W - 3, :F - 1].contiguous()
    w2 = torch.cat([w2[:, :F - 1], w2[:, F:2 * F - 1]], 1).contiguous()
    want = Hy.moe_experts(h2.float(), idx.cpu(), wt.cpu(), w2.float(), d2.float(), torch.float32)
    got = Hy.moe_experts(*gpu(h2, idx, wt, w2, d2), dt, by_row=True)
    torch.testing.assert_close(got.float().cpu(), want, **tol(dt))


@pytest.mark.parametrize("shape", [(4, 2, 64, 11), (8, 1, 64, 150), (7, 7, 128, 40), (3, 1, 128, 33)])
def test_any_size_attention_on_the_matrix_core_cache_layout(shape):
    """The any-size kernel reading a cache in the layout of the framework's matrix-core attention
    kernels (keys chunk-major per block, values transposed), with window and penalty, against the
    statement on a cache of plain rows filled from the same projections."""
    H, G, D, window = shape
    dt, BS = torch.bfloat16, 32
    g = torch.Generator().manual_seed(H * D + window)
    lens, starts = [70, 1, 2, 133], [0, 130, 63, 5]
    cu, _, pos, sp = spans(lens, starts)
    ctx = [s + n for s, n in zip(starts, lens)]
    nblk = [(c + BS - 1) // BS for c in ctx]
    nb = sum(nblk) + 2
    perm = torch.randperm(nb, generator=g).tolist()
    bt = torch.zeros(len(lens), max(nblk), dtype=torch.int32)
    for s, n in enumerate(nblk):
        bt[s, :n] = torch.tensor([perm.pop() for _ in range(n)])
    spec = GroupedAttentionSpec(H, G, D, D, 1.0, value_norm=True)
    slopes = torch.tensor([2.0 ** (-8.0 * (a + 1) / H) for a in range(H)])
    caches = {}
    for layout in (False, True):
        kc = torch.zeros(nb, G, BS, D, dtype=dt, device=DEV)
        vc = torch.zeros((nb, G, D, BS) if layout else (nb, G, BS, D), dtype=dt, device=DEV)
        gq = torch.Generator().manual_seed(7)
        qs = []
        for s in range(len(lens)):
            n = ctx[s]
            proj = (torch.randn(n, (H + 2 * G) * D, generator=gq) * 0.7).to(dt).to(DEV)
            slots = torch.tensor([int(bt[s, t // BS]) * BS + t % BS for t in range(n)], device=DEV)
            q = Hy.qk_prep(proj, spec, 0, H * D, (H + G) * D, None, 1e-5, torch.arange(n, device=DEV), kc, vc, slots, dt,
                           matrix_layout=layout)
            qs.append(q[starts[s]:])
        caches[layout] = (torch.cat(qs), kc, vc)
    q, kc, vc = caches[False]
    want = Hy.ref_gqa_attention(q.float().cpu(), kc.float().cpu(), vc.float().cpu(), bt, cu, sp, 0.3, None, 0.0, torch.float32,
                                window, slopes)
    qm, kcm, vcm = caches[True]
    got = Hy.gqa_attention(qm, kcm, vcm, *gpu(bt, cu, sp), 0.3, None, 0.0, window=window, slopes=slopes.to(DEV),
                           matrix_layout=True)
    torch.testing.assert_close(got.float().cpu(), want, **tol(dt))
    B = len(lens)
    last = torch.tensor([c - 1 for c in ctx], dtype=torch.int32)
    rows = torch.tensor([int(cu[s + 1]) - 1 for s in range(B)])
    cu1 = torch.arange(B + 1, dtype=torch.int32)
    tiles = torch.stack([torch.arange(B), torch.arange(B)], 1).to(torch.int32)
    got = Hy.gqa_attention(qm[rows.to(DEV)].contiguous(), kcm, vcm, *gpu(bt, cu1, last), 0.3, None, 0.0, tiles=tiles.to(DEV),
                           num_splits=3, window=window, slopes=slopes.to(DEV), matrix_layout=True)
    torch.testing.assert_close(got.float().cpu(), want[rows], **tol(dt))
