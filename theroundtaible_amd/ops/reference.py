"""Plain-PyTorch reference semantics of every hand-written kernel (the numerics oracle).

These run on CPU (unit tests, the GPT-2 CPU plumbing config) and are what the HIP
kernels in ``csrc/`` are tested against. Layouts are the engine's:

* ``k_cache``: allocated ``[num_blocks, n_kv_heads, block_size, head_dim]``, but each
  ``[block, head]`` block is CHUNK-MAJOR in memory: ``[head_dim/32][block_size][32]`` (round 6,
  csrc/common.h ``kc_elem``: a decode-attention K load instruction then reads whole 128-B lines).
  Index it through :func:`k_blocks` / :func:`k_rows` / :func:`write_k`, never as ``[blk, h, off, :]``.
* ``v_cache``: ``[num_blocks, n_kv_heads, head_dim, block_size]`` (V stored transposed per
  block, so the P.V MFMA B-operand is a contiguous load; see csrc/attention_decode.hip)
* ``slot = block_id * block_size + offset``
* ``cos_sin``: ``[max_pos, head_dim]`` fp32 = ``[cos(pos*f_i) | sin(pos*f_i)]`` over
  ``i < head_dim/2`` (Llama rotate-half convention).
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import torch

MASK64 = (1 << 64) - 1


def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    xf = x.float()
    y = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    return (y * w.float()).to(x.dtype)


def fused_add_rms_norm(x: torch.Tensor, residual: torch.Tensor, w: torch.Tensor,
                       eps: float) -> Tuple[torch.Tensor, torch.Tensor]:
    r = (x.float() + residual.float()).to(x.dtype)
    return rms_norm(r, w, eps), r


def layer_norm(x: torch.Tensor, w: torch.Tensor, b: torch.Tensor, eps: float) -> torch.Tensor:
    return torch.nn.functional.layer_norm(x.float(), (x.shape[-1],), w.float(), b.float(), eps).to(x.dtype)


def fused_add_layer_norm(x, residual, w, b, eps):
    r = (x.float() + residual.float()).to(x.dtype)
    return layer_norm(r, w, b, eps), r


def rope_inv_freq(head_dim: int, theta: float, scaling: Optional[tuple] = None) -> Tuple[torch.Tensor, float]:
    """RoPE inverse frequencies (fp64) and the cos / sin magnitude, for the checkpoint's
    ``rope_scaling`` (``models/config.py`` ``ModelConfig.rope_scaling``):

    * ``("linear", factor)``: positions / factor;
    * ``("llama3", factor, low_freq_factor, high_freq_factor, original_max_pos)`` (Llama 3.1 / 3.2):
      wavelengths past ``original / low`` divided by ``factor``, shorter than ``original / high``
      kept, the band between interpolated smoothly;
    * ``("yarn", factor, original_max_pos, beta_fast, beta_slow, attention_factor)`` (YaRN,
      Qwen2.5 long context): per-dimension blend of interpolated / extrapolated frequencies over
      the correction range, cos and sin scaled by ``attention_factor`` (the parser's default:
      0.1 ln(factor) + 1).
    The kernels read the resulting table; nothing else changes."""
    inv = 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=torch.float64) / head_dim))
    mag = 1.0
    if not scaling:
        return inv, mag
    kind = scaling[0]
    if kind == "linear":
        return inv / float(scaling[1]), mag
    if kind == "llama3":
        factor, low_ff, high_ff, orig = (float(v) for v in scaling[1:5])
        wavelen = 2 * math.pi / inv
        low_wl, high_wl = orig / low_ff, orig / high_ff
        out = torch.where(wavelen > low_wl, inv / factor, inv)
        smooth = (orig / wavelen - low_ff) / (high_ff - low_ff)
        mid = (wavelen >= high_wl) & (wavelen <= low_wl)
        return torch.where(mid, (1 - smooth) * out / factor + smooth * out, out), mag
    if kind == "yarn":
        factor, orig, beta_fast, beta_slow, att = (float(v) for v in scaling[1:6])

        def corr_dim(rot):
            return (head_dim * math.log(orig / (rot * 2 * math.pi))) / (2 * math.log(theta))
        low = max(math.floor(corr_dim(beta_fast)), 0)
        high = min(math.ceil(corr_dim(beta_slow)), head_dim - 1)
        if low == high:
            high += 0.001
        ramp = ((torch.arange(head_dim // 2, dtype=torch.float64) - low) / (high - low)).clamp(0, 1)
        extra = 1 - ramp                     # 1: keep the original frequency, 0: interpolate
        out = (inv / factor) * (1 - extra) + inv * extra
        return out, att
    raise ValueError(f"unsupported rope_scaling {scaling!r}")


def rope_cos_sin(max_pos: int, head_dim: int, theta: float, device=None,
                 scaling: Optional[tuple] = None) -> torch.Tensor:
    inv, mag = rope_inv_freq(head_dim, theta, scaling)
    t = torch.arange(max_pos, dtype=torch.float64)
    f = torch.outer(t, inv)
    return torch.cat([f.cos() * mag, f.sin() * mag], dim=-1).float().to(device)


def _rotate(x: torch.Tensor, cs: torch.Tensor) -> torch.Tensor:
    # x [T, H, D] float; cs [T, D]
    d2 = x.shape[-1] // 2
    cos, sin = cs[:, None, :d2], cs[:, None, d2:]
    x1, x2 = x[..., :d2], x[..., d2:]
    return torch.cat([x1 * cos - x2 * sin, x2 * cos + x1 * sin], dim=-1)


def rope_and_cache(qkv: torch.Tensor, positions: torch.Tensor, cos_sin: Optional[torch.Tensor],
                   k_cache: torch.Tensor, v_cache: torch.Tensor, slot_mapping: torch.Tensor,
                   n_heads: int, n_kv_heads: int, head_dim: int) -> torch.Tensor:
    """Split fused qkv, rotate q/k (if cos_sin given), scatter k/v into the paged cache, return q."""
    T = qkv.shape[0]
    q = qkv[:, :n_heads * head_dim].reshape(T, n_heads, head_dim).float()
    k = qkv[:, n_heads * head_dim:(n_heads + n_kv_heads) * head_dim].reshape(T, n_kv_heads, head_dim).float()
    v = qkv[:, (n_heads + n_kv_heads) * head_dim:].reshape(T, n_kv_heads, head_dim)
    if cos_sin is not None:
        cs = cos_sin[positions.long()]
        q = _rotate(q, cs)
        k = _rotate(k, cs)
    bs = k_cache.shape[2]
    slots = slot_mapping.long()
    blk, off = slots // bs, slots % bs
    write_k(k_cache, blk, off, k)
    v_cache[blk, :, :, off] = v.to(v_cache.dtype)
    return q.to(qkv.dtype)


def k_blocks(k_cache: torch.Tensor) -> torch.Tensor:
    """The chunk-major view of a K cache: ``[num_blocks, n_kv_heads, head_dim/32, block_size, 32]``."""
    nb, hkv, bs, d = k_cache.shape
    return k_cache.view(nb, hkv, d // 32, bs, 32)


def k_rows(k_cache: torch.Tensor, blocks: torch.Tensor) -> torch.Tensor:
    """Key rows of ``blocks`` in order: ``[len(blocks) * block_size, n_kv_heads, head_dim]``."""
    kb = k_blocks(k_cache)[blocks]                       # [n, Hkv, D/32, BS, 32]
    n, hkv, c, bs, w = kb.shape
    return kb.permute(0, 3, 1, 2, 4).reshape(n * bs, hkv, c * w)


def write_k(k_cache: torch.Tensor, blk: torch.Tensor, off: torch.Tensor, k: torch.Tensor) -> None:
    """Store key rows ``k`` ``[T, n_kv_heads, head_dim]`` at (block, offset) pairs."""
    T, hkv, d = k.shape
    k_blocks(k_cache)[blk, :, :, off, :] = k.reshape(T, hkv, d // 32, 32).to(k_cache.dtype)


def set_k_row(k_cache: torch.Tensor, blk: int, head: int, off: int, row: torch.Tensor) -> None:
    """Store one key row ``[head_dim]`` of one KV head (tests)."""
    k_blocks(k_cache)[blk, head, :, off, :] = row.reshape(-1, 32).to(k_cache.dtype)


def _gather_kv(k_cache, v_cache, block_table, n):
    bs = k_cache.shape[2]
    nblk = (n + bs - 1) // bs
    blocks = block_table[:nblk].long()
    k = k_rows(k_cache, blocks)[:n]
    v = v_cache[blocks].permute(0, 3, 1, 2).reshape(nblk * bs, v_cache.shape[1], -1)[:n]
    return k.float(), v.float()


def _sink_softmax(s: torch.Tensor, sink: float) -> torch.Tensor:
    """Softmax over the last axis with ``sink`` added to the denominator as exp(0) * sink."""
    if not sink:
        return torch.softmax(s, dim=-1)
    m = s.max(-1, keepdim=True).values.clamp_min(0.0)
    e = torch.exp(s - m)
    return e / (e.sum(-1, keepdim=True) + sink * torch.exp(-m))


def paged_attention_decode(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                           block_tables: torch.Tensor, ctx_lens: torch.Tensor, scale: float,
                           sink: float = 0.0) -> torch.Tensor:
    B, Hq, D = q.shape
    Hkv = k_cache.shape[1]
    G = Hq // Hkv
    out = torch.empty_like(q)
    for b in range(B):
        n = int(ctx_lens[b])
        k, v = _gather_kv(k_cache, v_cache, block_tables[b], n)     # [n, Hkv, D]
        qb = q[b].float().reshape(Hkv, G, D)
        s = torch.einsum("hgd,nhd->hgn", qb, k) * scale
        p = _sink_softmax(s, sink)
        o = torch.einsum("hgn,nhd->hgd", p, v)
        out[b] = o.reshape(Hq, D).to(q.dtype)
    return out


def prefill_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                      block_tables: torch.Tensor, cu_q: torch.Tensor, start_pos: torch.Tensor,
                      scale: float, sink: float = 0.0) -> torch.Tensor:
    """Varlen causal attention: sequence s has queries cu_q[s]:cu_q[s+1] at absolute positions
    start_pos[s] + i, attending to cached keys [0, start_pos[s] + i]."""
    T, Hq, D = q.shape
    Hkv = k_cache.shape[1]
    G = Hq // Hkv
    out = torch.empty_like(q)
    for s in range(cu_q.shape[0] - 1):
        a, b = int(cu_q[s]), int(cu_q[s + 1])
        if b == a:
            continue
        st = int(start_pos[s])
        n = st + (b - a)
        k, v = _gather_kv(k_cache, v_cache, block_tables[s], n)
        qs = q[a:b].float().reshape(b - a, Hkv, G, D)
        sc = torch.einsum("thgd,nhd->thgn", qs, k) * scale
        qpos = torch.arange(st, n)[:, None]
        kpos = torch.arange(n)[None, :]
        mask = (kpos <= qpos)[:, None, None, :]
        sc = sc.masked_fill(~mask, float("-inf"))
        p = _sink_softmax(sc, sink)
        o = torch.einsum("thgn,nhd->thgd", p, v)
        out[a:b] = o.reshape(b - a, Hq, D).to(q.dtype)
    return out


def rope_row_perm(n_rows: int, rope_heads: int, head_dim: int) -> torch.Tensor:
    """Source row of every output row in the pair-interleaved q/k order of the ROPE epilogue:
    row h*D + 2i <- h*D + i, row h*D + 2i + 1 <- h*D + i + D/2 (rows past the q/k heads: identity)."""
    idx = torch.arange(n_rows)
    r = rope_heads * head_dim
    if r:
        h, p = idx[:r] // head_dim, idx[:r] % head_dim
        idx[:r] = h * head_dim + p // 2 + (p % 2) * (head_dim // 2)
    return idx


def rope_bias(b: torch.Tensor, rope_heads: int, head_dim: int) -> torch.Tensor:
    """A q/k/v bias (natural order) as the ROPE epilogue adds it: fp32, in the pair-interleaved
    column order of the shuffled weight (:func:`rope_row_perm`)."""
    return b.float()[rope_row_perm(b.numel(), rope_heads, head_dim).to(b.device)].contiguous()


def fold_gamma(W, gamma=None, rope_heads: int = 0, head_dim: int = 0):
    """W * gamma[None, :] rounded to W's dtype (the RMSNorm weight folded into the next linear),
    rows optionally permuted for the ROPE epilogue (``rope_heads`` leading heads)."""
    out = W.clone() if gamma is None else (W.float() * gamma.float()[None, :]).to(W.dtype)
    if rope_heads:
        out = out[rope_row_perm(W.shape[0], rope_heads, head_dim)].contiguous()
    return out


def skinny_gemm(x, Wf, pro=0, epi=0, res=None, eps=1e-5, x2=None, xout=None):
    """Semantics of csrc/gemm_skinny.hip on the (gamma-folded, row-major) weight ``Wf``:
    y = rsqrt(mean(x^2) + eps)[:, None] * (x @ Wf^T) for the NORM prologue; NORM_ADD (pro=2)
    first forms x = bf16(x + x2) and stores it to ``xout``."""
    if pro == 2:
        x = (x.float() + x2.float()).to(x.dtype)
        if xout is not None:
            xout.copy_(x)
    M, K = x.shape
    xf = x.float()
    y = xf @ Wf.float().t()
    if pro in (1, 2):
        y = y * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    if epi == 2:
        n = Wf.shape[0] // 2
        return (torch.nn.functional.silu(y[:, :n]) * y[:, n:]).to(x.dtype)
    if epi == 1:
        res.copy_((y + res.float()).to(res.dtype))
        return None
    if epi == 3:
        return y  # fp32 pre-rope projection (see skinny_gemm_rope)
    return y.to(x.dtype)


def skinny_gemm_rope(x, Wp, pro, positions, cos_sin, k_cache, v_cache, slots, n_heads, n_kv_heads, head_dim,
                     eps=1e-5, x2=None, xout=None, bias=None):
    """ROPE-epilogue semantics: fp32 projection on the pair-permuted weight (+ the fp32 bias in
    the same column order, :func:`rope_bias`), columns restored to natural order, then RoPE +
    paged K/V scatter with no bf16 rounding in between."""
    y = skinny_gemm(x, Wp, pro, 3, None, eps, x2, xout)
    if bias is not None:
        y = y + bias.float()[None, :]
    perm = rope_row_perm(Wp.shape[0], n_heads + n_kv_heads, head_dim)
    qkv = torch.empty_like(y)
    qkv[:, perm] = y
    q = rope_and_cache(qkv, positions, cos_sin, k_cache, v_cache, slots, n_heads, n_kv_heads, head_dim)
    return q.to(x.dtype)


def silu_and_mul(x: torch.Tensor) -> torch.Tensor:
    d = x.shape[-1] // 2
    xf = x.float()
    return (torch.nn.functional.silu(xf[..., :d]) * xf[..., d:]).to(x.dtype)


def gelu_tanh(x: torch.Tensor) -> torch.Tensor:
    return torch.nn.functional.gelu(x.float(), approximate="tanh").to(x.dtype)


# ---- sampling -----------------------------------------------------------------------------
# Counter-based RNG shared bit-for-bit with csrc/sampling.hip: u = mix(seed, offset, idx).

def _mix64(z: int) -> int:
    z = (z + 0x9E3779B97F4A7C15) & MASK64
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & MASK64
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & MASK64
    return z ^ (z >> 31)


def uniform_tensor(seed: int, offset: int, n: int) -> torch.Tensor:
    """u in (0,1) for token indices 0..n-1 (vectorized with int64 wraparound arithmetic)."""
    key = _mix64((seed & MASK64) ^ _mix64(offset & MASK64))
    idx = torch.arange(n, dtype=torch.int64)
    z = _mix_t(idx + _to_signed(key))
    # top 24 bits -> (0,1)
    hi = (z >> 40) & 0xFFFFFF
    return (hi.double() + 0.5) / float(1 << 24)


def _to_signed(x: int) -> int:
    return x - (1 << 64) if x >= (1 << 63) else x


def _mix_t(z: torch.Tensor) -> torch.Tensor:
    def mul(a, c):
        return a * _to_signed(c)  # int64 multiply wraps mod 2^64

    def srl(a, s):  # logical right shift on int64
        return (a >> s) & ((1 << (64 - s)) - 1)

    z = z + _to_signed(0x9E3779B97F4A7C15)
    z = mul(z ^ srl(z, 30), 0xBF58476D1CE4E5B9)
    z = mul(z ^ srl(z, 27), 0x94D049BB133111EB)
    return z ^ srl(z, 31)


def sample(logits: torch.Tensor, temperature: torch.Tensor, top_p: torch.Tensor, top_k: torch.Tensor,
           seeds: torch.Tensor, offsets: torch.Tensor) -> torch.Tensor:
    """Greedy when temperature <= 0; else Gumbel-max over the top-k ∩ top-p set.

    Row b's noise is a pure function of (seeds[b], offsets[b], token index); the engine
    passes each knight's token position as its offset, so a knight's sample stream is
    independent of batching, graph replay and round mode."""
    B, V = logits.shape
    out = torch.empty(B, dtype=torch.int64)
    for b in range(B):
        l = logits[b].float()
        t = float(temperature[b])
        if t <= 0:
            out[b] = int(torch.argmax(l))
            continue
        z = (l - l.max()) / t
        allowed = torch.ones(V, dtype=torch.bool)
        k = int(top_k[b])
        if 0 < k < V:
            kth = torch.topk(z, k).values[-1]
            allowed &= z >= kth
        p = float(top_p[b])
        if p < 1.0:
            w = torch.where(allowed, torch.exp(z.double()), torch.zeros((), dtype=torch.float64))
            srt, _ = torch.sort(w, descending=True)
            cs = torch.cumsum(srt, 0)
            cut = int(torch.searchsorted(cs, p * cs[-1]).clamp(max=V - 1))
            thr = srt[cut]
            allowed &= w >= thr
        u = uniform_tensor(int(seeds[b]), int(offsets[b]), V)
        g = -torch.log(-torch.log(u))
        score = torch.where(allowed, z.double() + g, torch.full((), float("-inf"), dtype=torch.float64))
        out[b] = int(torch.argmax(score))
    return out


def decode_prep(slots, offsets, res, ids, positions, block_tables, embed, block_size):
    """Semantics of csrc/decode_step.hip::decode_prep (in place). A position past the block
    table (only after a turn's last step; that slot is never written) maps into block 0."""
    pos = positions.long()
    bi = pos // block_size
    inside = bi < block_tables.shape[1]
    blk = block_tables.long().gather(1, torch.where(inside, bi, 0).unsqueeze(1)).squeeze(1)
    blk = torch.where(inside, blk, 0)
    slots[:len(pos)] = blk * block_size + pos % block_size
    offsets[:len(pos)] = pos + 1
    tok = ids.long().clamp(0, embed.shape[0] - 1)
    res.copy_(embed[tok].to(res.dtype))


def decode_advance(out, ids, positions, ctx_lens, step, nxt, prep=None):
    """Semantics of csrc/decode_step.hip::decode_advance (in place); with prep operands
    (slots, offsets, res, block_tables, embed, block_size) it then runs decode_prep."""
    st = int(step.item())
    if st < out.shape[0]:
        out[st] = nxt
    ids.copy_(nxt)
    positions.add_(1)
    ctx_lens.add_(1)
    step.add_(1)
    if prep is not None:
        slots, offsets, res, bt, embed, bs = prep
        decode_prep(slots, offsets, res, ids, positions, bt, embed, bs)


PAGING_GUARD_CODES = {1: "ctx_len outside [1, max_blocks*block_size]", 2: "block-table entry outside the KV pool",
                      4: "K/V write slot does not match block_tables[pos // block_size]",
                      8: "ctx_len != position + 1"}


def paging_guard(block_tables, ctx_lens, positions, slots, err, num_blocks, block_size):
    """Semantics of csrc/decode_step.hip::paging_guard (err[0] |= violation bits, in place)."""
    code = 0
    maxb = block_tables.shape[1]
    for b in range(ctx_lens.numel()):
        ctx = int(ctx_lens[b])
        if ctx < 1 or ctx > maxb * block_size:
            code |= 1
        nt = min((max(ctx, 0) + block_size - 1) // block_size, maxb)
        row = block_tables[b, :nt]
        if nt and (int(row.min()) < 0 or int(row.max()) >= num_blocks):
            code |= 2
        if positions is not None:
            pos = int(positions[b])
            if pos + 1 != ctx:
                code |= 8
            if slots is not None and pos >= 0 and pos // block_size < maxb:
                want = int(block_tables[b, pos // block_size]) * block_size + pos % block_size
                if int(slots[b]) != want:
                    code |= 4
    err[0] = int(err[0]) | code


# ---- latent attention / input convolution / PolyNorm family (csrc/latent/*.hip) -----------------
# Row metadata shared by these ops: ``row_seq`` [T] int32 = sequence index of every row,
# ``positions`` [T] = absolute position of every row, ``start_pos`` [S] = position of each
# sequence's first row in this batch (rows of a sequence are consecutive, ``cu_q`` [S + 1]).

def scalar_rms_norm(x: torch.Tensor, g: torch.Tensor, eps: float, out_dtype=None) -> torch.Tensor:
    """RMS norm whose learned weight is ONE number; fp32 math."""
    xf = x.float()
    y = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps) * g.float()
    return y.to(out_dtype or x.dtype)


def scalar_norm_add_(res: torch.Tensor, y: torch.Tensor, g: torch.Tensor, eps: float) -> torch.Tensor:
    """res (fp32, in place) += scalar_rms_norm(y, g)."""
    res.add_(scalar_rms_norm(y, g, eps, torch.float32))
    return res


def canon_norm(x, g, eps, w, state, row_seq, positions, start_pos, slots, out_dtype):
    """h + causal depthwise conv(h) with h = scalar_rms_norm(x, g): ``w`` [W, taps] (last tap =
    the current token); inputs ahead of a sequence's first row come from ``state``
    [n_slots, taps - 1, W] (oldest first), inputs ahead of position 0 are zero."""
    h = scalar_rms_norm(x, g, eps, torch.float32)
    taps = w.shape[1]
    wf = w.float()
    out = h * (1.0 + wf[:, taps - 1])
    rs, pos = row_seq.long(), positions.long()
    local = pos - start_pos.long()[rs]
    rows = torch.arange(x.shape[0], device=x.device)
    for k in range(1, taps):
        in_batch = local >= k
        src = torch.where(in_batch.unsqueeze(1), h[(rows - k).clamp(min=0)],
                          state[slots.long()[rs], (taps - 1 - k + local).clamp(0, max(taps - 2, 0))])
        src = torch.where((pos >= k).unsqueeze(1), src, torch.zeros_like(src))
        out = out + wf[:, taps - 1 - k] * src
    return out.to(out_dtype)


def canon_state_update(x, g, eps, state, cu_q, start_pos, slots):
    """Shift each sequence's convolution state by its rows of this batch: afterwards it holds the
    last ``taps - 1`` normed inputs up to the sequence's newest row."""
    keep = state.shape[1]
    h = scalar_rms_norm(x, g, eps, torch.float32)
    cq, sp, sl = cu_q.tolist(), start_pos.tolist(), slots.tolist()
    for s in range(len(sl)):
        n = cq[s + 1] - cq[s]
        if n <= 0:
            continue
        old = state[sl[s]].clone()
        for i in range(keep):
            idx = n - keep + i              # row of this batch (>= 0) or of the old state (< 0)
            if idx >= 0:
                state[sl[s], i] = h[cq[s] + idx]
            elif sp[s] + idx >= 0:
                state[sl[s], i] = old[keep + idx]
            else:
                state[sl[s], i] = 0


def rotate_interleaved(v: torch.Tensor, positions: torch.Tensor, base: float, dims: int) -> torch.Tensor:
    """Rotary embedding on the pairs (2i, 2i + 1), i < dims / 2, of the last axis; ``v`` [T, ..., D],
    angle = position * base^(-2i / dims) in fp32."""
    if dims == 0:
        return v.float()
    i = torch.arange(dims // 2, dtype=torch.float32, device=v.device)
    f = torch.exp2(i * (-2.0 * math.log2(base) / dims))
    a = positions.float().view(-1, *([1] * (v.dim() - 1))) * f
    c, s = torch.cos(a), torch.sin(a)
    vf = v.float()
    u, w = vf[..., 0:dims:2], vf[..., 1:dims:2]
    out = vf.clone()
    out[..., 0:dims:2] = u * c - w * s
    out[..., 1:dims:2] = w * c + u * s
    return out


def latent_prep(proj, q_rank, kv_rank, rot_dim, wq, wkv, eps, positions, rot_base, rot_dims, cache_rows,
                slot_mapping, out_dtype):
    """From the fused input projection ``proj`` [T, >= q_rank + kv_rank + rot_dim]: the normed
    query latent (returned) and the cache row (normed latent | rotated shared key part), written
    at ``slot_mapping`` into ``cache_rows`` [num_blocks, block_size, kv_rank + rot_dim]."""
    cq = rms_norm(proj[:, :q_rank].float(), wq.float(), eps).to(out_dtype)
    c = rms_norm(proj[:, q_rank:q_rank + kv_rank].float(), wkv.float(), eps)
    kr = rotate_interleaved(proj[:, q_rank + kv_rank:q_rank + kv_rank + rot_dim], positions, rot_base, rot_dims)
    flat = cache_rows.view(-1, cache_rows.shape[-1])
    flat[slot_mapping.long()] = torch.cat([c, kr], -1).to(cache_rows.dtype)
    return cq


def latent_attention(q_lat, q, rot_off, cache_rows, block_tables, cu_q, start_pos, sink, scale, rot_base,
                     rot_dims, out_dtype):
    """Causal attention over the cached rows with the query folded into the latent space.

    ``q_lat`` [H, T, C] (the unrotated query of each head times its key up-projection), ``q``
    [T, H, Dq] whose entries ``rot_off:`` are the un-rotated rotary part (rotated here, by the
    row's position). Key t = cached row, value t = its first C entries. The softmax denominator
    also holds exp(sink_h). Returns [H, T, C]."""
    H, T, C = q_lat.shape
    out = torch.zeros(H, T, C, dtype=torch.float32, device=q.device)
    cq, sp = cu_q.tolist(), start_pos.tolist()
    BS = cache_rows.shape[1]
    for s in range(len(sp)):
        r0, r1 = cq[s], cq[s + 1]
        if r1 <= r0:
            continue
        n = sp[s] + (r1 - r0)
        nb = (n + BS - 1) // BS
        K = cache_rows[block_tables[s, :nb].long()].reshape(nb * BS, -1)[:n].float()
        pos = torch.arange(sp[s], n, device=q.device)
        qr = rotate_interleaved(q[r0:r1, :, rot_off:], pos, rot_base, rot_dims)          # [n_q, H, R]
        Q = torch.cat([q_lat[:, r0:r1].float(), qr.transpose(0, 1)], -1)                 # [H, n_q, C + R]
        sc = torch.einsum("hqd,kd->hqk", Q, K) * scale
        mask = torch.arange(n, device=q.device).view(1, 1, n) > pos.view(1, -1, 1)
        sc = sc.masked_fill(mask, float("-inf"))
        sk = sink.float().view(H, 1, 1)
        m = torch.maximum(sc.max(-1, keepdim=True).values, sk)
        e = torch.exp(sc - m)
        den = e.sum(-1, keepdim=True) + torch.exp(sk - m)
        out[:, r0:r1] = torch.einsum("hqk,kc->hqc", e / den, K[:, :C])
    return out.to(out_dtype)


def gate_mul(o, proj, g_off, out_dtype):
    """``o`` [H, T, Dv] head-major -> [T, H * Dv], times sigmoid of ``proj[:, g_off : g_off + H * Dv]``."""
    H, T, Dv = o.shape
    gate = torch.sigmoid(proj[:, g_off:g_off + H * Dv].float())
    return (o.float().permute(1, 0, 2).reshape(T, H * Dv) * gate).to(out_dtype)


def poly_norm(z, coef, eps, out_dtype):
    """a N(z) + b N(z^2) + c N(z^3) + e, N = divide a row by its root mean square; fp32 math."""
    zf = z.float()
    cf = coef.float()

    def n(u):
        return u * torch.rsqrt(u.pow(2).mean(-1, keepdim=True) + eps)
    return (cf[0] * n(zf) + cf[1] * n(zf * zf) + cf[2] * n(zf * zf * zf) + cf[3]).to(out_dtype)


def logit_softcap(logits, scale, cap):
    y = logits.float() * scale
    return cap * torch.tanh(y / cap) if cap > 0 else y
