"""Ops of decoders that mix grouped attention with recurrent layers: token shift fused with the
RMS norm ahead of a mixer (one or several mixes of the same row; the norm over the whole row or over
equal parts of it), query / key preparation (rotary pairs, per-head unit RMS, optional weights, a
query factor that grows with the position, unit-RMS values) with the paged cache write,
grouped-query attention with an optional softmax sink, per-head temperature, sliding window,
distance penalty and output gate, the minGRU scan, the wkv scan (linear attention with a per-token
decay), the two-branch normed residual add, residual add + RMS norm, the clamped gated, xIELU and
silu-gated feed-forward activations, and a routed mixture of experts.

GPU tensors go to the HIP kernels of ``theroundtaible_amd._C_hybrid`` (``csrc/hybrid/``, built
in-tree by ``csrc/build.py``; :func:`ensure_built` compiles it on first use in a fresh checkout);
CPU tensors run the PyTorch statements at the end of this file. There is no silent fallback on a
GPU.

Every kernel computes in fp32 and reads / writes bf16 or fp32 tensors as given; the residual
stream and every running state are always fp32.
"""
from __future__ import annotations

import os
import sys
from typing import Optional, Tuple

import torch

_NATIVE = None
_NATIVE_ERR: Optional[BaseException] = None

MAX_HEAD_DIM = 256       # widest query / key / value head the kernels hold in registers
PAIRS_PER_TILE = 32      # (query row, head) pairs one attention workgroup takes


def native():
    global _NATIVE, _NATIVE_ERR
    if _NATIVE is None and _NATIVE_ERR is None:
        try:
            from .. import _C_hybrid  # type: ignore
            _NATIVE = _C_hybrid
        except BaseException as e:  # noqa: BLE001
            _NATIVE_ERR = e
    if _NATIVE is None:
        raise RuntimeError(f"theroundtaible_amd._C_hybrid (HIP kernels) is not built/importable: {_NATIVE_ERR}. "
                           f"Run `python csrc/build.py hybrid` (or __graft_entry__.build()).")
    return _NATIVE


def ensure_built(verbose: bool = False) -> None:
    """Compile the extension if it is missing or older than its sources (a fresh checkout's first
    GPU run); only this family's kernels are compiled."""
    global _NATIVE_ERR
    root = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    sys.path.insert(0, os.path.join(root, "csrc"))
    try:
        import build as csrc_build
        csrc_build.build_hybrid(verbose=verbose)
    finally:
        sys.path.pop(0)
    _NATIVE_ERR = None


def _gpu(t: torch.Tensor) -> bool:
    return t.is_cuda


# ---- token shift + norm ---------------------------------------------------------------------------

def shift_norm(x, y, w, eps, mu, state, row_seq, positions, start_pos, slots, out_dtype,
               shift_state: bool = False, groups: int = 1) -> Tuple[torch.Tensor, torch.Tensor]:
    """``x`` [T, W] fp32 residual, ``y`` an optional pending branch output still to be added.
    With ``xs = x + y`` and ``h_r = xs_r / rms(xs_r) * w``: returns ``(h_r + (p_r - h_r) * mu, xs)``
    where ``p_r`` is the previous token's ``h``: row r - 1 inside a span, ``state[slot]`` for the
    first row of a span that continues a sequence, zeros at position 0. ``xs`` is a new tensor
    when ``y`` is given (other rows of the launch still read the old ``x``), else ``x`` itself.
    ``shift_state`` (only with ONE row per sequence, a decode step): the same launch also stores
    ``h_r`` as the sequence's new state, so no :func:`shift_state_update` follows.
    ``mu`` [n, W] gives n mixes of the same row at once, returned as [n, T, W]. ``groups`` > 1:
    the norm divides each of that many equal consecutive parts of a row by its own RMS."""
    if _gpu(x):
        out = torch.empty((mu.shape[0],) + tuple(x.shape) if mu.dim() == 2 else x.shape, dtype=out_dtype, device=x.device)
        xs = torch.empty_like(x) if y is not None else x
        native().shift_norm(out, xs, x, y, w, float(eps), mu, state, row_seq, positions, start_pos, slots,
                            bool(shift_state), int(groups))
        return out, xs
    return ref_shift_norm(x, y, w, eps, mu, state, row_seq, positions, start_pos, slots, out_dtype, shift_state, groups)


def shift_state_update(x, w, eps, state, cu_q, slots, groups: int = 1) -> None:
    """Store the normed last row of every span as its sequence's state. Runs AFTER
    :func:`shift_norm` of the same layer (it overwrites what that one reads)."""
    if _gpu(x):
        native().shift_state_update(x, w, float(eps), state, cu_q, slots, int(groups))
        return
    ref_shift_state_update(x, w, eps, state, cu_q, slots, groups)


# ---- queries, keys, values ------------------------------------------------------------------------

def rotary_table(rot, device) -> Optional[torch.Tensor]:
    """fp32 frequencies [dims / 2] of a :class:`RotarySpec` (None: no rotation)."""
    if rot is None or rot.dims == 0:
        return None
    from .reference import rope_inv_freq
    inv, _ = rope_inv_freq(rot.dims, rot.base, rot.scaling)
    return inv.to(torch.float32).to(device).contiguous()


def qk_prep(proj, spec, q_off: int, k_off: int, v_off: int, inv_freq, eps, positions, k_cache, v_cache,
            slot_mapping, out_dtype, matrix_layout: bool = False, q_scale=None, q_weight=None,
            k_weight=None) -> torch.Tensor:
    """``proj`` [T, N]: columns ``q_off ..`` hold the projected queries (heads x dim), ``k_off ..``
    the keys (kv_heads x dim), ``v_off ..`` the values (kv_heads x vdim; ignored when the values
    are the keys). Rotates the leading ``2 * len(inv_freq)`` entries of every query / key head
    (entry 2i with 2i + 1, angle = position * inv_freq[i], fp32), divides each head by its root
    mean square, writes keys and values to the paged cache at ``slot_mapping`` and returns the
    queries [T, heads, dim]. ``matrix_layout`` (GPU): the cache of the framework's matrix-core
    attention kernels — keys chunk-major per block, values transposed ``[nb, G, vdim, BS]``;
    ``q_scale`` [heads] fp32 multiplies each query head (a per-head temperature moved into q).
    ``q_weight`` / ``k_weight`` [dim] fp32 multiply the normed queries / keys channel by channel.
    ``spec.q_temp`` = (coef, every): queries of position p times 1 + coef ln(floor((p + 1) / every) + 1);
    ``spec.value_norm``: every value head is divided by its root mean square before it is cached."""
    if _gpu(proj):
        T = proj.shape[0]
        q = torch.empty(T, spec.heads, spec.dim, dtype=out_dtype, device=proj.device)
        qt = spec.q_temp or (0.0, 0)
        native().qk_prep(q, proj, int(q_off), int(k_off), int(v_off), bool(spec.value_from_key), inv_freq, float(eps),
                         positions, k_cache, v_cache, slot_mapping, 1 if matrix_layout else 0, q_scale, q_weight, k_weight,
                         bool(spec.value_norm), float(qt[0]), int(qt[1]))
        return q
    if matrix_layout:
        raise ValueError("qk_prep: the matrix-core cache layout exists on the GPU only")
    if q_scale is not None:
        raise ValueError("qk_prep: q_scale is a GPU-path option (the CPU statement keeps the temperature in the scores)")
    return ref_qk_prep(proj, spec, q_off, k_off, v_off, inv_freq, eps, positions, k_cache, v_cache, slot_mapping,
                       out_dtype, q_weight, k_weight)


def rows_per_tile(group: int) -> int:
    """Query rows one varlen attention workgroup takes (its (row, head) pairs share a key tile)."""
    return max(1, PAIRS_PER_TILE // max(1, group))


def tile_map(cu_q: torch.Tensor, start_pos: torch.Tensor, rows: int) -> torch.Tensor:
    """[n_tiles, 2] int32 (sequence, first row) of the varlen attention launch, heaviest first."""
    items = []
    cq, sp = cu_q.tolist(), start_pos.tolist()
    for s in range(len(sp)):
        for r in range(cq[s], cq[s + 1], rows):
            items.append((sp[s] + min(r + rows, cq[s + 1]) - cq[s], s, r))
    items.sort(key=lambda x: -x[0])
    return torch.tensor([(s, r) for _, s, r in items], dtype=torch.int32).reshape(-1, 2)


class SplitWorkspace:
    """Split-key scratch of the one-row-per-sequence (decode) attention launch: per (row, head,
    split) a partial output, running maximum and sum; static, so captured graphs can hold it."""

    def __init__(self, max_rows: int, heads: int, vdim: int, max_splits: int, device):
        self.max_rows, self.max_splits = max_rows, max_splits
        self.part_o = torch.empty(max_rows * heads * max_splits * vdim, dtype=torch.float32, device=device)
        self.part_ml = torch.empty(max_rows * heads * max_splits * 2, dtype=torch.float32, device=device)


def gqa_attention(q, k_cache, v_cache, block_tables, cu_q, start_pos, scale: float, temp=None, sink: float = 0.0,
                  tiles=None, num_splits: int = 1, workspace: Optional[SplitWorkspace] = None,
                  out_dtype=None, window: int = 0, slopes=None, gate=None, gate_off: int = 0,
                  matrix_layout: bool = False, softcap: float = 0.0, out_scale: float = 1.0, out_buf=None,
                  out_off: int = 0) -> torch.Tensor:
    """Causal attention of the rows ``q`` [T, H, Dk] (span s = rows ``cu_q[s] .. cu_q[s + 1]`` at
    positions ``start_pos[s] ..`` of sequence s) over the paged keys ``k_cache`` [nb, G, BS, Dk]
    and values ``v_cache`` [nb, G, BS, Dv]: score = q . k * scale (* ``temp[h]``), weights
    exp(s_j) / (``sink`` + sum exp(s_j)). Returns [T, H * Dv]. ``tiles``: :func:`tile_map` on the
    device; ``num_splits`` > 1 (one row per span: a decode step) cuts every row's keys into that
    many ranges merged by a second launch. ``window`` > 0: row i sees only keys j with
    i - j < window. ``slopes`` [H] fp32: head h takes slopes[h] * (i - j) off its scores. ``gate``
    [T, N]: the result is multiplied by sigmoid of its columns ``gate_off .. gate_off + H * Dv``.
    ``matrix_layout`` (GPU): the cache is in the layout of the framework's matrix-core attention
    kernels (see :func:`qk_prep`), e.g. decode rows of a layer whose prompts run on those kernels.
    ``softcap`` > 0: scaled scores become softcap * tanh(score / softcap). ``out_scale`` multiplies
    the result. ``out_buf`` [T, N]: the result goes to its columns ``out_off ..`` (a wider
    activation buffer that another branch fills beside it) and ``out_buf`` is returned."""
    out_dtype = out_dtype or q.dtype
    if _gpu(q):
        T, H, _ = q.shape
        G, Dv = k_cache.shape[1], v_cache.shape[2 if matrix_layout else 3]
        out = out_buf if out_buf is not None else torch.empty(T, H * Dv, dtype=out_dtype, device=q.device)
        rows = 1 if num_splits > 1 else rows_per_tile(H // G)
        if tiles is None:
            tiles = tile_map(cu_q.cpu(), start_pos.cpu(), rows).to(q.device)
        if num_splits > 1 and workspace is None:
            workspace = SplitWorkspace(T, H, Dv, num_splits, q.device)
        native().gqa_attention(out, q, k_cache, v_cache, block_tables, cu_q, start_pos, tiles, temp, float(scale),
                               float(sink), rows, int(num_splits),
                               workspace.part_o if num_splits > 1 else None,
                               workspace.part_ml if num_splits > 1 else None, int(window), slopes, gate, int(gate_off),
                               1 if matrix_layout else 0, float(softcap), float(out_scale), int(out_off))
        return out
    if matrix_layout:
        raise ValueError("gqa_attention: the matrix-core cache layout exists on the GPU only")
    o = ref_gqa_attention(q, k_cache, v_cache, block_tables, cu_q, start_pos, scale, temp, sink,
                          torch.float32 if out_scale != 1.0 else out_dtype, window, slopes, gate, gate_off, softcap)
    if out_scale != 1.0:
        o = (o * out_scale).to(out_dtype)
    if out_buf is not None:
        out_buf[:, out_off:out_off + o.shape[1]] = o
        return out_buf
    return o


# ---- minGRU ---------------------------------------------------------------------------------------

SCAN_CHUNK = 64          # rows per chunk of the chunked scan (csrc/hybrid/hybrid_ops.hip kScanChunk)


def scan_chunks(cu_q: torch.Tensor, device=None):
    """Work lists of the chunked scan from the host copy of ``cu_q``: (chunks [n, 2] int32 =
    (sequence, first row), a sequence's chunks consecutive and in order; seq_chunk0 [S + 1] int32),
    or None when no span is longer than one chunk (the one-launch scan is used then)."""
    cq = cu_q.tolist()
    if max((b - a for a, b in zip(cq, cq[1:])), default=0) <= SCAN_CHUNK:
        return None
    chunks, first = [], [0]
    for s in range(len(cq) - 1):
        chunks += [(s, r) for r in range(cq[s], cq[s + 1], SCAN_CHUNK)]
        first.append(len(chunks))
    return (torch.tensor(chunks, dtype=torch.int32).reshape(-1, 2).to(device, non_blocking=True),
            torch.tensor(first, dtype=torch.int32).to(device, non_blocking=True))


def mingru_scan(proj, z_off: int, x_off: int, g_off: int, width: int, bz, bx, state, cu_q, start_pos, slots,
                out_dtype, chunks=None) -> torch.Tensor:
    """``proj`` [T, N] holds the three projections of the recurrence at the given column offsets.
    z = sigmoid(p_z + bz); u = p_x + bx; c = u + 1/2 where u >= 0, sigmoid(u) below;
    S_t = (1 - z_t) S_(t-1) + z_t c_t per channel, from ``state[slot]`` (zeros at position 0);
    returns S_t * silu(p_g) [T, width] and leaves every span's last S in ``state``. fp32 inside.
    ``chunks`` (GPU): :func:`scan_chunks` of this batch — spans are then scanned in chunks of
    ``SCAN_CHUNK`` rows in parallel (chunk aggregates, a carry pass, the outputs) instead of row by
    row; the results differ from the one-launch scan by rounding only."""
    if _gpu(proj):
        out = torch.empty(proj.shape[0], width, dtype=out_dtype, device=proj.device)
        if chunks is not None:
            ws = torch.empty(3 * chunks[0].shape[0] * width, dtype=torch.float32, device=proj.device)
            native().mingru_scan(out, proj, int(z_off), int(x_off), int(g_off), bz, bx, state, cu_q, start_pos, slots,
                                 chunks[0], chunks[1], ws)
        else:
            native().mingru_scan(out, proj, int(z_off), int(x_off), int(g_off), bz, bx, state, cu_q, start_pos, slots)
        return out
    return ref_mingru_scan(proj, z_off, x_off, g_off, width, bz, bx, state, cu_q, start_pos, slots, out_dtype)


# ---- residual / norms / activation ----------------------------------------------------------------

def dual_norm_add_(x, a, wa, b, wb, eps) -> torch.Tensor:
    """x += (a / rms(a) * wa + b / rms(b) * wb) / 2, in place on the fp32 residual."""
    if _gpu(x):
        native().dual_norm_add(x, a.contiguous(), wa, b.contiguous(), wb, float(eps))
        return x
    return ref_dual_norm_add_(x, a, wa, b, wb, eps)


def add_norm(x, y, w, eps, out_dtype, groups: int = 1) -> torch.Tensor:
    """x += y (in place, fp32; ``y`` may be None), returns x / rms(x) * w; with ``groups`` > 1 each
    of that many equal consecutive parts of a row is divided by its own RMS."""
    if _gpu(x):
        out = torch.empty(x.shape, dtype=out_dtype, device=x.device)
        native().add_norm(out, x, y, w, float(eps), int(groups))
        return out
    return ref_add_norm(x, y, w, eps, out_dtype, groups)


def limited_glu(gu, limit: float, out_dtype) -> torch.Tensor:
    """``gu`` [T, 2F] = (gate | up): g = min(gate, limit), u = clamp(up, -limit, limit);
    returns g * sigmoid(1.702 g) * (u + 1)."""
    if _gpu(gu):
        out = torch.empty(gu.shape[0], gu.shape[1] // 2, dtype=out_dtype, device=gu.device)
        native().limited_glu(out, gu, float(limit))
        return out
    return ref_limited_glu(gu, limit, out_dtype)


# ---- wkv ------------------------------------------------------------------------------------------

WKV_CHUNK = 32           # rows per chunk of the chunked wkv scan (csrc/hybrid/hybrid_wkv.hip kWkvChunk)


def wkv_chunks(cu_q: torch.Tensor, device=None, min_rows: int = 2 * WKV_CHUNK):
    """Work lists of the chunked wkv scan, as :func:`scan_chunks`: None when no span has more than
    ``min_rows`` rows (the one-launch scan is used then)."""
    cq = cu_q.tolist()
    if max((b - a for a, b in zip(cq, cq[1:])), default=0) <= min_rows:
        return None
    chunks, first = [], [0]
    for s in range(len(cq) - 1):
        chunks += [(s, r) for r in range(cq[s], cq[s + 1], WKV_CHUNK)]
        first.append(len(chunks))
    return (torch.tensor(chunks, dtype=torch.int32).reshape(-1, 2).to(device, non_blocking=True),
            torch.tensor(first, dtype=torch.int32).to(device, non_blocking=True))


def wkv_scan(rkvg, lw, w0, u, norm_w, eps, state, cu_q, start_pos, slots, out_dtype, chunks=None) -> torch.Tensor:
    """``rkvg`` [4, T, H * D]: the projected r, k, v and output gate; ``lw`` [T, H * D] the decay's
    low-rank path; ``w0`` [H * D], ``u`` [H, D], ``norm_w`` [H * D] fp32. Per sequence and head,
    with the D x D state S from ``state[slot]`` [H * D * D] (zeros at position 0), in fp32:
        decay = exp(-exp(lw + w0));  o_t[j] = sum_i r_t[i] (S[i, j] + u[i] k_t[i] v_t[j]);
        S[i, j] <- decay_t[i] S[i, j] + k_t[i] v_t[j]
    and returns o_t / rms(o_t per head) * norm_w * silu(gate_t) [T, H * D]; every span's last S is
    left in ``state``. ``chunks`` (GPU): :func:`wkv_chunks` of this batch — spans are then scanned
    in chunks in parallel (chunk end states and decay products, a carry pass, the outputs from each
    chunk's true start state); the results differ from the one-launch scan by rounding only."""
    if _gpu(rkvg):
        out = torch.empty(rkvg.shape[1], rkvg.shape[2], dtype=out_dtype, device=rkvg.device)
        if chunks is not None:
            H, D = u.shape
            ws = torch.empty(chunks[0].shape[0] * H * (D * D + D), dtype=torch.float32, device=rkvg.device)
            native().wkv_scan(out, rkvg, lw, w0, u, norm_w, float(eps), state, cu_q, start_pos, slots, chunks[0], chunks[1], ws)
        else:
            native().wkv_scan(out, rkvg, lw, w0, u, norm_w, float(eps), state, cu_q, start_pos, slots)
        return out
    return ref_wkv_scan(rkvg, lw, w0, u, norm_w, eps, state, cu_q, start_pos, slots, out_dtype)


# ---- feed-forward -----------------------------------------------------------------------------------

def xielu(a, bias, alpha_pos: float, alpha_neg: float, out_dtype) -> torch.Tensor:
    """z = a + bias; alpha_pos z^2 + z / 2 for z > 0, alpha_neg (e^z - 1 - z) + z / 2 otherwise."""
    if _gpu(a):
        out = torch.empty(a.shape, dtype=out_dtype, device=a.device)
        native().xielu(out, a, bias, float(alpha_pos), float(alpha_neg))
        return out
    return ref_xielu(a, bias, alpha_pos, alpha_neg, out_dtype)


def silu_glu(gu, out_dtype) -> torch.Tensor:
    """``gu`` [T, 2F] = (gate | up): silu(gate) * up."""
    if _gpu(gu):
        out = torch.empty(gu.shape[0], gu.shape[1] // 2, dtype=out_dtype, device=gu.device)
        native().silu_glu(out, gu)
        return out
    return ref_silu_glu(gu, out_dtype)


def topk_softmax(logits, top: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """Per row of fp32 ``logits`` [T, E]: the indices [T, top] int32 of the ``top`` largest (largest
    first) and the softmax over those alone [T, top] fp32."""
    if _gpu(logits) and logits.shape[1] <= 512 and top <= 64:
        idx = torch.empty(logits.shape[0], top, dtype=torch.int32, device=logits.device)
        wt = torch.empty(logits.shape[0], top, dtype=torch.float32, device=logits.device)
        native().topk_softmax(idx, wt, logits.contiguous())
        return idx, wt
    val, idx = torch.topk(logits, top, dim=-1)
    return idx.to(torch.int32), torch.softmax(val, dim=-1)


def route_topk(h, router_w, top: int, bias=None) -> Tuple[torch.Tensor, torch.Tensor]:
    """Router and choice: fp32 logits ``router_w`` [E, W] . ``h`` [T, W] (+ ``bias``), then as
    :func:`topk_softmax`. One launch on the GPU (the row in LDS, a wave per expert in turn)."""
    E, W = router_w.shape
    if _gpu(h) and E <= 512 and top <= 64 and (W + 4 + 5 * E) * 4 <= 48 * 1024:
        idx = torch.empty(h.shape[0], top, dtype=torch.int32, device=h.device)
        wt = torch.empty(h.shape[0], top, dtype=torch.float32, device=h.device)
        native().route_topk(idx, wt, h.contiguous(), router_w, bias)
        return idx, wt
    return topk_softmax(torch.nn.functional.linear(h.float(), router_w, bias), top)


MOE_ROWS = 16            # steps of up to this many rows run the experts row by row (moe_rows)


def relu2(a, out_dtype) -> torch.Tensor:
    """relu(a)^2, entry by entry."""
    if _gpu(a):
        out = torch.empty(a.shape, dtype=out_dtype, device=a.device)
        native().relu2(out, a.contiguous())
        return out
    return ref_relu2(a, out_dtype)


def moe_experts(h, idx, wt, w_gu, w_down, out_dtype, by_row: Optional[bool] = None, act: str = "silu_glu") -> torch.Tensor:
    """Mixture of experts: ``h`` [T, W]; row t runs experts ``idx[t]`` [top] and adds their
    outputs W_down[e] (silu(W_gate[e] h) * (W_up[e] h)) with the weights ``wt[t]``. ``w_gu``
    [E, 2F, W] = every expert's gate rows, then up rows; ``w_down`` [E, W, F]. ``act`` "relu2":
    the experts are W_down[e] relu(W_up[e] h)^2 and ``w_gu`` is [E, F, W]. Two forms: row by row
    (GPU steps of a few rows: two launches, no host round trip, so a captured decode step can hold
    them) and expert by expert (the rows of each expert gathered for library GEMMs, one host read of
    the expert counts; a row's experts are added in fp32 in the order of its choices whatever else is
    in the batch)."""
    T, top = idx.shape
    if by_row is None:
        by_row = _gpu(h) and T <= MOE_ROWS
    if by_row and _gpu(h):
        out = torch.empty(h.shape, dtype=out_dtype, device=h.device)
        hid = torch.empty(T * top * w_down.shape[2], dtype=torch.float32, device=h.device)
        native().moe_rows(out, hid, h.contiguous(), w_gu, w_down, idx, wt, 1 if act == "relu2" else 0)
        return out
    E, W = w_gu.shape[0], h.shape[1]
    flat = idx.reshape(-1).long()
    order = torch.argsort(flat, stable=True)            # (row, choice) pairs, expert by expert
    counts = torch.bincount(flat, minlength=E).tolist()
    hs = h.index_select(0, order // top)                # every expert's input rows, gathered once
    ys = torch.empty(T * top, W, dtype=h.dtype, device=h.device)
    at = 0
    for e, n in enumerate(counts):
        if n:
            a = torch.nn.functional.linear(hs[at:at + n], w_gu[e])
            a = relu2(a, h.dtype) if act == "relu2" else silu_glu(a, h.dtype)
            torch.mm(a, w_down[e].t(), out=ys[at:at + n])
            at += n
    back = torch.empty_like(order)
    back[order] = torch.arange(T * top, device=h.device)
    y = ys.index_select(0, back).view(T, top, W).float()
    # a row's experts are added in the order of its choices, in fp32, whatever else is in the batch
    return torch.bmm(wt.view(T, 1, top), y).view(T, W).to(out_dtype)


# ---- the PyTorch statements (CPU tensors; what the kernels are tested against) ---------------------

def _rms(x, eps, groups: int = 1):
    if groups > 1:
        return _rms(x.reshape(*x.shape[:-1], groups, x.shape[-1] // groups), eps).reshape(x.shape)
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def ref_shift_norm(x, y, w, eps, mu, state, row_seq, positions, start_pos, slots, out_dtype, shift_state=False,
                   groups=1):
    xs = x + y.float() if y is not None else x
    h = _rms(xs, eps, groups) * w
    prev = torch.zeros_like(h)
    prev[1:] = h[:-1]
    rs = row_seq.long()
    first = positions == start_pos.long()[rs]
    prev = torch.where(first[:, None], state[slots.long()[rs]], prev)
    prev = torch.where((positions == 0)[:, None], torch.zeros_like(prev), prev)
    out = h + (prev - h) * (mu[:, None, :] if mu.dim() == 2 else mu)
    if shift_state:
        state[slots.long()[rs]] = h
    return out.to(out_dtype), xs


def ref_shift_state_update(x, w, eps, state, cu_q, slots, groups=1):
    last = cu_q.long()[1:] - 1
    state[slots.long()] = _rms(x[last], eps, groups) * w


def _rotate_pairs(t, positions, inv_freq):
    """t [T, n, D] fp32: entry 2i pairs with 2i + 1 on the leading 2 * len(inv_freq) entries."""
    d = 2 * inv_freq.numel()
    ang = positions.to(torch.float32)[:, None] * inv_freq[None]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    u, v = t[..., 0:d:2], t[..., 1:d:2]
    out = t.clone()
    out[..., 0:d:2] = u * c - v * s
    out[..., 1:d:2] = v * c + u * s
    return out


def ref_qk_prep(proj, spec, q_off, k_off, v_off, inv_freq, eps, positions, k_cache, v_cache, slot_mapping, out_dtype,
                q_weight=None, k_weight=None):
    T = proj.shape[0]
    H, G, Dk, Dv = spec.heads, spec.kv_heads, spec.dim, spec.vdim
    q = proj[:, q_off:q_off + H * Dk].float().reshape(T, H, Dk)
    k = proj[:, k_off:k_off + G * Dk].float().reshape(T, G, Dk)
    v = proj[:, k_off:k_off + G * Dk] if spec.value_from_key else proj[:, v_off:v_off + G * Dv]
    if inv_freq is not None:
        q, k = _rotate_pairs(q, positions, inv_freq), _rotate_pairs(k, positions, inv_freq)
    q, k = _rms(q, eps), _rms(k, eps)
    if q_weight is not None:
        q = q * q_weight
    if k_weight is not None:
        k = k * k_weight
    if spec.q_temp is not None:
        coef, every = spec.q_temp
        steps = torch.div(positions.long() + 1, every, rounding_mode="floor").to(torch.float32)
        q = q * (1.0 + coef * torch.log(steps + 1.0))[:, None, None]
    v = v.reshape(T, G, Dv)
    if spec.value_norm:
        v = _rms(v.float(), eps)
    BS = k_cache.shape[2]
    blk, off = slot_mapping // BS, slot_mapping % BS
    k_cache[blk, :, off] = k.to(k_cache.dtype)
    v_cache[blk, :, off] = v.to(v_cache.dtype)
    return q.to(out_dtype)


def ref_gqa_attention(q, k_cache, v_cache, block_tables, cu_q, start_pos, scale, temp, sink, out_dtype,
                      window=0, slopes=None, gate=None, gate_off=0, softcap=0.0):
    T, H, Dk = q.shape
    G, BS, Dv = k_cache.shape[1], k_cache.shape[2], v_cache.shape[3]
    out = torch.empty(T, H, Dv, dtype=torch.float32, device=q.device)
    cq, sp = cu_q.tolist(), start_pos.tolist()
    hs = torch.full((H,), float(scale), dtype=torch.float32, device=q.device)
    if temp is not None:
        hs = hs * temp.float()
    for s in range(len(sp)):
        r0, r1 = cq[s], cq[s + 1]
        if r1 == r0:
            continue
        ctx = sp[s] + r1 - r0
        blocks = block_tables[s, :(ctx + BS - 1) // BS].long()
        K = k_cache[blocks].permute(1, 0, 2, 3).reshape(G, -1, Dk)[:, :ctx].float()
        V = v_cache[blocks].permute(1, 0, 2, 3).reshape(G, -1, Dv)[:, :ctx].float()
        qs = q[r0:r1].float().permute(1, 0, 2)                                       # [H, n, Dk]
        sc = torch.einsum("hnd,hkd->hnk", qs, K.repeat_interleave(H // G, 0)) * hs[:, None, None]
        if softcap > 0:
            sc = softcap * torch.tanh(sc / softcap)
        qpos = torch.arange(sp[s], ctx, device=q.device)
        dist = qpos[:, None] - torch.arange(ctx, device=q.device)[None, :]
        mask = dist >= 0
        if window > 0:
            mask = mask & (dist < window)
        if slopes is not None:
            sc = sc - slopes.float()[:, None, None] * dist.to(torch.float32)[None]
        sc = sc.masked_fill(~mask[None], float("-inf"))
        m = sc.max(-1, keepdim=True).values
        e = torch.exp(sc - m)
        den = e.sum(-1, keepdim=True) + sink * torch.exp(-m)
        out[r0:r1] = torch.einsum("hnk,hkd->hnd", e / den, V.repeat_interleave(H // G, 0)).permute(1, 0, 2)
    out = out.reshape(T, H * Dv)
    if gate is not None:
        out = out * torch.sigmoid(gate[:, gate_off:gate_off + H * Dv].float())
    return out.to(out_dtype)


def ref_mingru_scan(proj, z_off, x_off, g_off, width, bz, bx, state, cu_q, start_pos, slots, out_dtype):
    z = torch.sigmoid(proj[:, z_off:z_off + width].float() + bz)
    u = proj[:, x_off:x_off + width].float() + bx
    c = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
    g = torch.nn.functional.silu(proj[:, g_off:g_off + width].float())
    out = torch.empty(proj.shape[0], width, dtype=torch.float32, device=proj.device)
    cq, sp, sl = cu_q.tolist(), start_pos.tolist(), slots.tolist()
    for s in range(len(sp)):
        if cq[s + 1] == cq[s]:
            continue
        S = state[sl[s]].clone() if sp[s] > 0 else torch.zeros(width, dtype=torch.float32, device=proj.device)
        for r in range(cq[s], cq[s + 1]):
            S = (1 - z[r]) * S + z[r] * c[r]
            out[r] = S
        state[sl[s]] = S
    return (out * g).to(out_dtype)


def ref_dual_norm_add_(x, a, wa, b, wb, eps):
    x.add_(0.5 * (_rms(a.float(), eps) * wa + _rms(b.float(), eps) * wb))
    return x


def ref_add_norm(x, y, w, eps, out_dtype, groups=1):
    if y is not None:
        x.add_(y.float())
    return (_rms(x, eps, groups) * w).to(out_dtype)


def ref_wkv_scan(rkvg, lw, w0, u, norm_w, eps, state, cu_q, start_pos, slots, out_dtype):
    T, HD = rkvg.shape[1], rkvg.shape[2]
    H, D = u.shape
    r, k, v, g = (rkvg[i].float().reshape(T, H, D) for i in range(4))
    dec = torch.exp(-torch.exp(lw.float() + w0)).reshape(T, H, D)
    o = torch.empty(T, H, D, dtype=torch.float32, device=rkvg.device)
    cq, sp, sl = cu_q.tolist(), start_pos.tolist(), slots.tolist()
    for s in range(len(sp)):
        if cq[s + 1] == cq[s]:
            continue
        S = (state[sl[s]].reshape(H, D, D).clone() if sp[s] > 0
             else torch.zeros(H, D, D, dtype=torch.float32, device=rkvg.device))
        for t in range(cq[s], cq[s + 1]):
            kv = k[t][:, :, None] * v[t][:, None, :]
            o[t] = torch.einsum("hi,hij->hj", r[t], S + u[:, :, None] * kv)
            S = dec[t][:, :, None] * S + kv
        state[sl[s]] = S.reshape(-1)
    return (_rms(o, eps).reshape(T, HD) * norm_w * torch.nn.functional.silu(g.reshape(T, HD))).to(out_dtype)


def ref_xielu(a, bias, alpha_pos, alpha_neg, out_dtype):
    z = a.float() + (bias if bias is not None else 0.0)
    neg = alpha_neg * (torch.expm1(torch.clamp(z, max=0.0)) - z) + 0.5 * z
    return torch.where(z > 0, alpha_pos * z * z + 0.5 * z, neg).to(out_dtype)


def ref_relu2(a, out_dtype):
    return (torch.relu(a.float()) ** 2).to(out_dtype)


def ref_silu_glu(gu, out_dtype):
    F = gu.shape[1] // 2
    return (torch.nn.functional.silu(gu[:, :F].float()) * gu[:, F:].float()).to(out_dtype)


def ref_limited_glu(gu, limit, out_dtype):
    F = gu.shape[1] // 2
    g = torch.clamp(gu[:, :F].float(), max=limit)
    u = torch.clamp(gu[:, F:].float(), -limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1)).to(out_dtype)


# ---- input convolutions, whole-projection norms, matrix-state recurrences ---------------------------
#
# Layers whose sublayers read the residual stream through a causal convolution and add their
# RMS-normed output back; attention whose queries / keys are normed over the whole projection and
# rotated in halves; recurrences with a D x E fp32 state per head.

MAX_CONV_TAPS = 16


def canon_add(x, y, y2, norm_w, eps, conv_w, state, sub: int, row_seq, positions, start_pos, slots, out_dtype,
              shift_state: bool = False) -> Tuple[Optional[torch.Tensor], torch.Tensor]:
    """``x`` [T, W] fp32 residual; ``y`` an optional sublayer output still to be added (``y2``: a
    second part of it, y + y2 is what is normed). With ``xs = x + (y + y2) / rms(y + y2) * norm_w``
    (``xs = x`` when ``y`` is None) returns ``(h, xs)``, ``h_t = xs_t + sum_k conv_w[:, taps - 1 - k]
    * xs_(t - k)``: a causal convolution over time per channel, tap k reading k tokens back — from
    this batch inside a span, from ``state[slot, sub]`` [taps - 1, W] (oldest first) ahead of a span
    that continues a sequence, zeros ahead of position 0. ``xs`` is a new tensor when ``y`` is given
    (other rows of the launch still read the old ``x``). ``conv_w`` None: only the add (``h`` is
    None). ``shift_state`` (ONE row per sequence: a decode step): the launch also shifts ``xs`` into
    the state, so no :func:`conv_state_update` follows."""
    if _gpu(x):
        h = torch.empty(x.shape, dtype=out_dtype, device=x.device) if conv_w is not None else None
        xs = torch.empty_like(x) if y is not None else x
        native().canon_add(h, xs, x, y, y2, norm_w, float(eps), conv_w, state, int(sub), row_seq, positions, start_pos,
                           slots, bool(shift_state))
        return h, xs
    return ref_canon_add(x, y, y2, norm_w, eps, conv_w, state, sub, row_seq, positions, start_pos, slots, out_dtype,
                         shift_state)


def conv_state_update(x, col_off: int, channels: int, state, sub: int, cu_q, start_pos, slots) -> None:
    """Shift every span's last rows of ``x[:, col_off : col_off + channels]`` into its sequence's
    convolution state ``state[slot, sub]`` [keep, channels] (oldest first; a span shorter than the
    state keeps the newest old rows). Runs AFTER the launch that reads the state."""
    if _gpu(x):
        native().conv_state_update(x, int(col_off), int(channels), state, int(sub), cu_q, start_pos, slots)
        return
    ref_conv_state_update(x, col_off, channels, state, sub, cu_q, start_pos, slots)


def rotary_halves_table(rot, device) -> Tuple[Optional[torch.Tensor], float]:
    """(fp32 frequencies [dims / 2], cos / sin magnitude) of a :class:`RotarySpec`."""
    if rot is None or rot.dims == 0:
        return None, 1.0
    from .reference import rope_inv_freq
    inv, mag = rope_inv_freq(rot.dims, rot.base, rot.scaling)
    return inv.to(torch.float32).to(device).contiguous(), float(mag)


def qkv_prep_wide(proj, spec, q_off: int, k_off: int, v_off: int, q_bias, k_bias, q_w, k_w, freq, mag: float, vfreq,
                  eps, positions, k_cache, v_cache, slot_mapping, out_dtype) -> torch.Tensor:
    """``proj`` [T, N]: columns ``q_off ..`` hold the projected queries (heads x dim), ``k_off ..``
    the keys (kv_heads x dim), ``v_off ..`` the values (kv_heads x vdim; ignored when the values are
    the keys). Adds the biases (fp32 [heads * dim] / [kv_heads * dim], or None); divides the WHOLE
    query row and the whole key row by its root mean square and multiplies by ``q_w`` / ``k_w``
    per channel; turns the leading ``2 len(freq)`` entries of every head, entry i with entry
    i + len(freq), by position * freq[i] with cos and sin times ``mag``; writes the keys to the
    paged cache and returns the queries [T, heads, dim]. Values: the biased keys as projected
    (``spec.value_from_key``) or the value columns, turned over all vdim entries in halves by
    position * vfreq[m] when ``vfreq`` is given."""
    if _gpu(proj):
        q = torch.empty(proj.shape[0], spec.heads, spec.dim, dtype=out_dtype, device=proj.device)
        native().qkv_prep_wide(q, proj, int(q_off), int(k_off), int(v_off), bool(spec.value_from_key), q_bias, k_bias,
                               q_w, k_w, freq, float(mag), vfreq, float(eps), positions, k_cache, v_cache, slot_mapping)
        return q
    return ref_qkv_prep_wide(proj, spec, q_off, k_off, v_off, q_bias, k_bias, q_w, k_w, freq, mag, vfreq, eps, positions,
                             k_cache, v_cache, slot_mapping, out_dtype)


def turn_back(o, heads: int, positions, vfreq, scale: float, out_buf, out_off: int) -> torch.Tensor:
    """``o`` [T, heads * E]: every head turned in halves by MINUS position * vfreq[m], times
    ``scale``, into columns ``out_off ..`` of ``out_buf`` [T, N]."""
    if _gpu(o):
        native().turn_back(out_buf, int(out_off), o, int(heads), positions, vfreq, float(scale))
        return out_buf
    T, E = o.shape[0], o.shape[1] // heads
    t = _rotate_halves(o.float().reshape(T, heads, E), -positions.to(torch.float32), vfreq, 1.0)
    out_buf[:, out_off:out_off + heads * E] = (t.reshape(T, heads * E) * scale).to(out_buf.dtype)
    return out_buf


def silu_cols(proj, off: int, n: int) -> torch.Tensor:
    """fp32 silu of the columns ``off .. off + n`` of ``proj`` [T, N]."""
    if _gpu(proj):
        out = torch.empty(proj.shape[0], n, dtype=torch.float32, device=proj.device)
        native().silu_cols(out, proj, int(off))
        return out
    return torch.nn.functional.silu(proj[:, off:off + n].float())


def removal_prep(proj, r_off: int, k_off: int, v_off: int, a_off: int, lw, w0, a_bias, heads: int, dim: int):
    """Inputs of a generalized delta rule from ``proj`` [T, N] (columns of r, k, v and the removal
    rate, each heads x dim) and the decay's low-rank path ``lw`` [T, heads * dim], all math fp32:
    w = exp(-e^(-1/2) sigmoid(lw + w0)); a = sigmoid(p_a + a_bias); u = k / sqrt(sum_head(k^2) + 1e-6).
    Returns fp32 [6, T, heads * dim] = (r, k, v, w, a * u, u): the (q, k, v, w, a, b) of
    :func:`state_scan`."""
    if _gpu(proj):
        out = torch.empty(6, proj.shape[0], heads * dim, dtype=torch.float32, device=proj.device)
        native().removal_prep(out, proj, int(r_off), int(k_off), int(v_off), int(a_off), lw, w0, a_bias, int(heads))
        return out
    return ref_removal_prep(proj, r_off, k_off, v_off, a_off, lw, w0, a_bias, heads, dim)


def delta_prep(proj, spec, q_off: int, b_off: int, a_off: int, conv_w, state, neg_rate, dt_bias, row_seq, positions,
               start_pos, slots, shift_state: bool = False):
    """Inputs of a gated delta rule from ``proj`` [T, N]: columns ``q_off ..`` hold q (kv_heads x
    dim), k (kv_heads x dim), v (heads x vdim) one after the other, ``b_off ..`` / ``a_off ..`` one
    number per head. q, k, v pass a causal convolution per channel (``conv_w`` [channels, taps]
    fp32, the last tap on the current token; rows ahead of a span from ``state[slot]``
    [taps - 1, channels], zeros ahead of position 0) and silu; q and k become unit vectors per head
    (q also times dim^(-1/2)); beta = sigmoid(p_b); g = exp(neg_rate[head] * softplus(p_a + dt_bias))
    with ``neg_rate`` = -exp(A_log). Returns fp32 ``(five [5, T, heads * dim], v [T, heads * vdim])``
    with five = (q, beta k, g, g beta k, k) per value head (g repeated over dim): the (q, k, w, a, b)
    of :func:`state_scan`, which then computes S <- g S; S <- S + k (beta (v - S^T k))^T; o = S^T q.
    ``shift_state`` (ONE row per sequence): the launch also shifts the projected q, k, v row into
    ``state``."""
    if _gpu(proj):
        T = proj.shape[0]
        five = torch.empty(5, T, spec.heads * spec.dim, dtype=torch.float32, device=proj.device)
        v = torch.empty(T, spec.heads * spec.vdim, dtype=torch.float32, device=proj.device)
        native().delta_prep(five, v, proj, int(q_off), int(b_off), int(a_off), conv_w, state, neg_rate, dt_bias,
                            int(spec.heads), int(spec.kv_heads), int(spec.dim), int(spec.vdim), row_seq, positions,
                            start_pos, slots, bool(shift_state))
        return five, v
    return ref_delta_prep(proj, spec, q_off, b_off, a_off, conv_w, state, neg_rate, dt_bias, row_seq, positions,
                          start_pos, slots, shift_state)


def state_scan(q, k, v, w, a, b, decay, state, cu_q, start_pos, slots, heads: int, dim: int, vdim: int) -> torch.Tensor:
    """Matrix-state recurrence, fp32 throughout. Per sequence and head, with the dim x vdim state S
    from ``state[slot]`` (zeros at position 0), for every token in order:
        s = b_t^T S;   S <- diag(w_t) S - a_t s^T + k_t v_t^T;   o_t = S^T q_t
    ``q, k, w, a, b`` [T, heads * dim] and ``v`` [T, heads * vdim] are fp32 rows (any row stride).
    ``w`` None: every head decays by its constant ``decay[head]``; ``a`` / ``b`` None: nothing is
    removed. Returns o [T, heads * vdim] fp32 and leaves every span's last S in ``state``
    (``[n_slots, heads * vdim * dim]``, each head stored column by column)."""
    if _gpu(q):
        out = torch.empty(q.shape[0], heads * vdim, dtype=torch.float32, device=q.device)
        native().state_scan(out, q, k, v, w, a, b, decay, state, cu_q, start_pos, slots, int(heads), int(dim), int(vdim))
        return out
    return ref_state_scan(q, k, v, w, a, b, decay, state, cu_q, start_pos, slots, heads, dim, vdim)


def head_norm_gate(o, norm_w, span: int, gate, gate_off: int, gate_act: str, eps, scale: float, out_buf,
                   out_off: int) -> torch.Tensor:
    """``o`` [T, C] fp32: every ``span`` consecutive entries (a head; ``span`` = C: the whole row)
    divided by their root mean square, times ``norm_w`` (fp32 [C], or [span] shared by the heads),
    times sigmoid or silu (``gate_act``) of the columns ``gate_off ..`` of ``gate`` [T, N], times
    ``scale``, into columns ``out_off ..`` of ``out_buf``."""
    if _gpu(o):
        native().head_norm_gate(out_buf, int(out_off), o, norm_w, int(span), gate, int(gate_off),
                                1 if gate_act == "silu" else 0, float(eps), float(scale))
        return out_buf
    T, C = o.shape
    n = _rms(o.reshape(T, C // span, span), eps)
    n = (n * norm_w).reshape(T, C) if norm_w.numel() == span else n.reshape(T, C) * norm_w
    g = gate[:, gate_off:gate_off + C].float()
    g = torch.nn.functional.silu(g) if gate_act == "silu" else torch.sigmoid(g)
    out_buf[:, out_off:out_off + C] = (n * g * scale).to(out_buf.dtype)
    return out_buf


def _rotate_halves(t, positions, freq, mag):
    """t [T, n, D] fp32: entry i pairs with i + len(freq) on the leading 2 * len(freq) entries."""
    r = freq.numel()
    ang = positions.to(torch.float32)[:, None] * freq[None]
    c, s = (torch.cos(ang) * mag)[:, None, :], (torch.sin(ang) * mag)[:, None, :]
    u, v = t[..., :r], t[..., r:2 * r]
    out = t.clone()
    out[..., :r] = u * c - v * s
    out[..., r:2 * r] = v * c + u * s
    return out


def _conv_rows(xs, conv_w, st, row_seq, positions, start_pos, slots):
    """sum_k conv_w[:, taps - 1 - k] * xs_(t - k) per row, rows ahead of a span from ``st``
    [n_slots, keep, C] (oldest first), zeros ahead of position 0."""
    taps = conv_w.shape[1]
    rs = row_seq.long()
    local = positions.long() - start_pos.long()[rs]
    acc = torch.zeros_like(xs)
    T = xs.shape[0]
    for k in range(taps):
        src = torch.zeros_like(xs)
        if k == 0:
            src = xs
        else:
            src[k:] = xs[:T - k]
            from_state = (local < k) & (positions.long() >= k)
            idx = (taps - 1 - k + local).clamp(0, max(taps - 2, 0))
            src = torch.where(from_state[:, None], st[slots.long()[rs], idx], src)
            src = torch.where(((local < k) & ~from_state)[:, None], torch.zeros_like(src), src)
        acc = acc + conv_w[:, taps - 1 - k] * src
    return acc


def _shift_rows_into(st, xs, row_seq, positions, slots):
    """One row per sequence: drop the oldest state row, append this one."""
    sl = slots.long()[row_seq.long()]
    keep = st.shape[1]
    old = st[sl].clone()
    for i in range(keep - 1):
        ok = (positions.long() - (keep - 1 - i)) >= 0
        st[sl, i] = torch.where(ok[:, None], old[:, i + 1], torch.zeros_like(old[:, i + 1]))
    st[sl, keep - 1] = xs


def ref_canon_add(x, y, y2, norm_w, eps, conv_w, state, sub, row_seq, positions, start_pos, slots, out_dtype,
                  shift_state=False):
    xs = x
    if y is not None:
        yy = y.float() + (y2.float() if y2 is not None else 0.0)
        xs = x + _rms(yy, eps) * norm_w
    if conv_w is None:
        return None, xs
    taps = conv_w.shape[1]
    st = state[:, sub]
    h = xs + (_conv_rows(xs, conv_w, st, row_seq, positions, start_pos, slots) if taps > 0 else 0.0)
    if shift_state and taps > 1:
        _shift_rows_into(st, xs, row_seq, positions, slots)
    return h.to(out_dtype), xs


def ref_conv_state_update(x, col_off, channels, state, sub, cu_q, start_pos, slots):
    st = state[:, sub] if state.dim() == 4 else state
    keep = st.shape[1]
    cq, sp, sl = cu_q.tolist(), start_pos.tolist(), slots.tolist()
    for s in range(len(sp)):
        n = cq[s + 1] - cq[s]
        if n <= 0:
            continue
        old = st[sl[s]].clone()
        for i in range(keep):
            idx = n - keep + i
            if idx >= 0:
                st[sl[s], i] = x[cq[s] + idx, col_off:col_off + channels].float()
            elif sp[s] + idx >= 0:
                st[sl[s], i] = old[keep + idx]
            else:
                st[sl[s], i] = 0.0


def ref_qkv_prep_wide(proj, spec, q_off, k_off, v_off, q_bias, k_bias, q_w, k_w, freq, mag, vfreq, eps, positions,
                      k_cache, v_cache, slot_mapping, out_dtype):
    T = proj.shape[0]
    H, G, Dk, Dv = spec.heads, spec.kv_heads, spec.dim, spec.vdim
    q = proj[:, q_off:q_off + H * Dk].float()
    k = proj[:, k_off:k_off + G * Dk].float()
    if q_bias is not None:
        q = q + q_bias
    if k_bias is not None:
        k = k + k_bias
    v = k.reshape(T, G, Dk) if spec.value_from_key else proj[:, v_off:v_off + G * Dv].float().reshape(T, G, Dv)
    q = (_rms(q, eps) * q_w).reshape(T, H, Dk)
    k = (_rms(k, eps) * k_w).reshape(T, G, Dk)
    if freq is not None:
        q, k = _rotate_halves(q, positions, freq, mag), _rotate_halves(k, positions, freq, mag)
    if vfreq is not None:
        v = _rotate_halves(v, positions, vfreq, 1.0)
    BS = k_cache.shape[2]
    blk, off = slot_mapping // BS, slot_mapping % BS
    k_cache[blk, :, off] = k.to(k_cache.dtype)
    v_cache[blk, :, off] = v.to(v_cache.dtype)
    return q.to(out_dtype)


def ref_removal_prep(proj, r_off, k_off, v_off, a_off, lw, w0, a_bias, heads, dim):
    import math
    T, n = proj.shape[0], heads * dim
    r, k, v = (proj[:, o:o + n].float() for o in (r_off, k_off, v_off))
    w = torch.exp(-math.exp(-0.5) * torch.sigmoid(lw.float() + w0))
    a = torch.sigmoid(proj[:, a_off:a_off + n].float() + a_bias)
    kh = k.reshape(T, heads, dim)
    u = (kh / torch.sqrt((kh * kh).sum(-1, keepdim=True) + 1e-6)).reshape(T, n)
    return torch.stack([r, k, v, w, a * u, u])


def ref_delta_prep(proj, spec, q_off, b_off, a_off, conv_w, state, neg_rate, dt_bias, row_seq, positions, start_pos,
                   slots, shift_state=False):
    T = proj.shape[0]
    A, G, D, E = spec.heads, spec.kv_heads, spec.dim, spec.vdim
    C = 2 * G * D + A * E
    raw = proj[:, q_off:q_off + C].float()
    z = torch.nn.functional.silu(_conv_rows(raw, conv_w, state, row_seq, positions, start_pos, slots))
    if shift_state and conv_w.shape[1] > 1:
        _shift_rows_into(state, raw, row_seq, positions, slots)
    q = z[:, :G * D].reshape(T, G, D)
    k = z[:, G * D:2 * G * D].reshape(T, G, D)
    v = z[:, 2 * G * D:]
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    q, k = q.repeat_interleave(A // G, 1), k.repeat_interleave(A // G, 1)           # [T, A, D]
    beta = torch.sigmoid(proj[:, b_off:b_off + A].float())[:, :, None]
    g = torch.exp(neg_rate * torch.nn.functional.softplus(proj[:, a_off:a_off + A].float() + dt_bias))[:, :, None]
    five = torch.stack([q, beta * k, g.expand(T, A, D), g * beta * k, k]).reshape(5, T, A * D)
    return five.contiguous(), v.contiguous()


def ref_state_scan(q, k, v, w, a, b, decay, state, cu_q, start_pos, slots, heads, dim, vdim):
    T = q.shape[0]
    A, D, E = heads, dim, vdim
    q, k, v = q.float().reshape(T, A, D), k.float().reshape(T, A, D), v.float().reshape(T, A, E)
    w = w.float().reshape(T, A, D) if w is not None else None
    a = a.float().reshape(T, A, D) if a is not None else None
    b = b.float().reshape(T, A, D) if b is not None else None
    out = torch.empty(T, A, E, dtype=torch.float32, device=q.device)
    cq, sp, sl = cu_q.tolist(), start_pos.tolist(), slots.tolist()
    for s in range(len(sp)):
        if cq[s + 1] == cq[s]:
            continue
        # the stored state keeps each head column by column: [A, E, D]
        S = (state[sl[s]].reshape(A, E, D).transpose(1, 2).clone() if sp[s] > 0
             else torch.zeros(A, D, E, dtype=torch.float32, device=q.device))
        for t in range(cq[s], cq[s + 1]):
            kv = k[t][:, :, None] * v[t][:, None, :]
            dec = w[t][:, :, None] if w is not None else decay[:, None, None]
            if a is not None:
                sv = torch.einsum("hi,hij->hj", b[t], S)
                S = dec * S - a[t][:, :, None] * sv[:, None, :] + kv
            else:
                S = dec * S + kv
            out[t] = torch.einsum("hi,hij->hj", q[t], S)
        state[sl[s]] = S.transpose(1, 2).reshape(-1)
    return out.reshape(T, A * E)
