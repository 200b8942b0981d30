"""Ledinex decoder: every sublayer reads the fp32 residual stream through a causal input
convolution (x + conv(x), a few taps per channel) and adds its RMS-normed output back (weights
stored around zero); the mixer is a parallel pair — softmax attention beside a matrix-state
recurrence, summed with two constants — or a gated delta rule; the feed-forward is a routed mixture
of squared-ReLU experts plus a shared expert. The logits read the embedding table.

  "parallel"    attention over all earlier keys with soft-capped scores, queries / keys normed
                over the whole projection and turned in halves (frequencies divided by a factor),
                values turned by their position and the output turned back; beside a linear
                attention with one constant decay per head.
  "parallel_2"  sliding-window attention with biased projections whose values are its unnormed
                keys, blended (YaRN) frequencies; beside a generalized delta rule with a per-token,
                per-channel decay and removal rate.
  "delta"       gated delta rule: short convolutions + silu on q, k, v, unit-length q and k, one
                decay and one step size per head and token.

Per layer (the same code for prompts, portions of prompts, single decoded tokens and any mix of
them in one batch; only the attention launch differs):

    h, x   = canon_add(x, pending)              C1 (HIP): pending sublayer output normed and added,
                                                then x + conv(x) against the kept last inputs
    proj   = h @ W_in^T                         one GEMM for every projection that reads h
    parallel*:
      q    = qkv_prep_wide(proj)                C2 (HIP): biases, whole-row norms, rotation in
                                                halves, turned values; keys / values -> paged cache
      cat[:, :left]  = gqa_attention(q)         H3 (HIP): window / soft cap, scaled result
                       (turn_back(.))           C3 (HIP): output turned back ("parallel")
      s    = removal_prep(proj) | silu_cols     C4 (HIP): decays, rates, unit keys in fp32
      o    = state_scan(s)                      C5 (HIP): the recurrence, state in registers
      cat[:, left:]  = head_norm_gate(o)        C6 (HIP): per-head / whole-row norm, weight, gate
      pending = cat @ [Wo_left | Wo_right]^T    one GEMM for both halves
    delta:
      s    = delta_prep(proj)                   C7 (HIP): short convolutions, silu, unit vectors,
                                                step size and decay per head
      o    = state_scan(s); pending = head_norm_gate(o) @ Wo^T
    h, x   = canon_add(x, pending)              C1, second convolution state
    idx, wt = route_topk(h, Wrouter)            H11 (HIP): fp32 router logits and the choice, one launch
    pending = moe_experts(h, idx, wt) (+) relu2(h @ Wsu^T) @ Wsd^T      H12 / H10, C8 (HIP)

The residual stream, every norm, positions and angles, scores and softmax, the router, the
convolution states, decays / rates / unit vectors and the whole recurrence are fp32 whatever the
model dtype; GEMM operands, the activations between them and the key / value cache take the model
dtype.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch
import torch.nn.functional as F

from ..ops import hybrid as Hy
from ..parallel.tp import TPInfo
from .config import DecaySumSpec, DeltaSpec, ModelConfig, ParallelSpec, RemovalSpec, attention_of
from .goganex import GoganexModel
from .llama import AttnMeta


class LedinexModel(GoganexModel):
    """Shares the row bookkeeping, attention tile maps, split-key workspaces and decode GEMMs of
    :class:`GoganexModel`; the layers, the cache shapes and the forward are its own."""
    matrix_attention = False       # the matrix-core attention kernels know no window or soft cap
    _DEC_LINEARS = ("w_in", "w_out", "mlp.shared.up", "mlp.shared.down")

    def __init__(self, cfg: ModelConfig, weights: Dict[str, torch.Tensor], device, dtype=torch.bfloat16,
                 tp: Optional[TPInfo] = None):
        self.cfg = cfg
        self.w = weights
        self.tp = tp or TPInfo()
        if self.tp.size > 1:
            raise ValueError(f"{cfg.name}: tensor parallelism is not supported for this architecture")
        self.device = torch.device(device)
        self.dtype = dtype
        if dtype == torch.float32:      # true fp32 products: no reduced-precision matrix mode
            torch.backends.cuda.matmul.allow_tf32 = False
            torch.backends.cudnn.allow_tf32 = False
        self.n_heads, self.n_kv_heads, self.head_dim = cfg.n_heads, cfg.n_kv_heads, cfg.head_dim
        f32 = torch.float32
        self.layers: Dict[int, Dict[str, torch.Tensor]] = {}
        for i, ls in enumerate(cfg.layers):
            p = f"l{i}."
            lw = {k[len(p):]: v for k, v in weights.items() if k.startswith(p)}
            m = ls.mixer
            off: Dict[str, int] = {}

            def stack(names):
                at, parts = 0, []
                for n in names:
                    off[n] = at
                    parts.append(lw.pop("mix." + n))
                    at += parts[-1].shape[0]
                return torch.cat(parts).contiguous()
            if isinstance(m, DeltaSpec):
                lw["w_in"] = stack(["q", "k", "v", "g", "b", "a"])
                lw["w_out"] = lw.pop("mix.o")
                lw["conv_w"] = torch.cat([lw.pop(f"mix.{n}.conv") for n in "qkv"]).to(f32).contiguous()
                lw["neg_rate"] = -torch.exp(lw.pop("mix.A_log").to(f32)).contiguous()
                fp = ("mix.dt_bias", "mix.norm")
            else:
                a, r = m.left, m.right
                names = ["left.q", "left.k"] + ([] if a.value_from_key else ["left.v"])
                if isinstance(r, DecaySumSpec):
                    names += ["right.q", "right.k", "right.v", "right.g"]
                    lw["decay"] = torch.tensor(r.decay, dtype=f32, device=self.device)
                else:
                    names += ["right.r", "right.k", "right.v", "right.a", "right.g", "right.w1"]
                lw["w_in"] = stack(names)
                lw["w_out"] = torch.cat([lw.pop("mix.left.o"), lw.pop("mix.right.o")], 1).contiguous()
                lw["freq"], lw["mag"] = Hy.rotary_halves_table(a.rot, self.device)
                lw["vfreq"] = Hy.rotary_halves_table(a.value_rot, self.device)[0]
                fp = ("mix.left.q.b", "mix.left.k.b", "mix.left.q.norm", "mix.left.k.norm", "mix.right.norm",
                      "mix.right.w0", "mix.right.a.b")
            lw["off"] = off
            if ls.ff:
                E = ls.moe.experts
                lw["w_up"] = torch.stack([lw.pop(f"mlp.e{e}.up") for e in range(E)]).contiguous()        # [E, F, W]
                lw["w_down"] = torch.stack([lw.pop(f"mlp.e{e}.down") for e in range(E)]).contiguous()    # [E, W, F]
                fp += ("mlp.router",)
            for n in ("canon1", "canon2") + fp:
                if n in lw:
                    lw[n] = lw[n].to(f32).contiguous()
            for n in ("norm1", "norm2"):        # stored around zero: the multiplier is 1 + w
                if n in lw:
                    lw[n] = (1.0 + lw[n].to(f32)).contiguous()
            self.layers[i] = lw
        self.final_norm = (1.0 + weights["final.norm"].to(f32)).contiguous()
        self._dec = None
        self._split_ws = None
        self._static = {}
        self._ws = {}

    # ---- cache ------------------------------------------------------------------------------------
    def cache_shapes(self):
        return [(a.kv_heads, a.dim, a.vdim) if a is not None else None for a in map(attention_of, self.cfg.layers)]

    def make_cache(self, num_blocks: int, block_size: int, device, dtype, n_slots: int):
        from ..engine.kv_cache import GroupedKVCache
        rec, short = [], []
        for ls in self.cfg.layers:
            m = ls.mixer
            r = m.right if isinstance(m, ParallelSpec) else m
            rec.append(r.state_size)
            short.append((m.conv_channels, m.conv) if isinstance(m, DeltaSpec) else None)
        return GroupedKVCache(self.cache_shapes(), self.cfg.hidden, rec, num_blocks, block_size, device, dtype,
                              n_slots=n_slots, shift_layers=[False] * len(rec), canon_taps=self.cfg.canon_taps,
                              short_conv=short)

    def cache_bytes_per_block(self, block_size: int, dtype_bytes: int) -> int:
        return max(1, sum(sh[0] * (sh[1] + sh[2]) for sh in self.cache_shapes() if sh is not None)) * block_size * dtype_bytes

    # ---- forward ----------------------------------------------------------------------------------
    def _window_splits(self, a, rows: int) -> int:
        """Key ranges per decoded row: as many as fill the chip, but no more than the tiles a
        window can touch."""
        splits = self.decode_splits(rows, a.kv_heads)
        if splits > 1 and a.window > 0:
            kt = max(1, Hy.native().gqa_key_tile(a.dim, a.vdim))
            splits = max(1, min(splits, (a.window + kt - 1) // kt + 1))
        return splits

    def _parallel(self, proj, m: ParallelSpec, lw, l, positions, kv, meta, b, decode):
        """Both halves of a parallel mixer into one activation buffer [T, left | right]."""
        adt, T, eps = self.dtype, proj.shape[0], self.cfg.norm_eps
        a, r, off = m.left, m.right, lw["off"]
        nl, nr = a.heads * a.vdim, r.heads * r.vdim
        cat = torch.empty(T, nl + nr, dtype=adt, device=proj.device)
        q = Hy.qkv_prep_wide(proj, a, off["left.q"], off["left.k"], off.get("left.v", 0), lw.get("mix.left.q.b"),
                             lw.get("mix.left.k.b"), lw["mix.left.q.norm"], lw["mix.left.k.norm"], lw["freq"], lw["mag"],
                             lw["vfreq"], eps, positions, kv.k_layer(l), kv.v_layer(l), meta.slot_mapping, adt)
        splits = self._window_splits(a, T) if decode else 1
        turned = lw["vfreq"] is not None
        o = Hy.gqa_attention(q, kv.k_layer(l), kv.v_layer(l), meta.block_tables, b.cu_q, b.start_pos, a.scale, None, 0.0,
                             tiles=self._tiles(meta, Hy.rows_per_tile(a.group), b) if proj.is_cuda else None,
                             num_splits=splits, workspace=self._workspace(T, a, splits), out_dtype=adt, window=a.window,
                             softcap=a.softcap, out_scale=1.0 if turned else m.left_scale,
                             out_buf=None if turned else cat, out_off=0)
        if turned:
            Hy.turn_back(o, a.heads, positions, lw["vfreq"], m.left_scale, cat, 0)
        n = r.heads * r.dim
        if isinstance(r, DecaySumSpec):
            s = Hy.silu_cols(proj, off["right.q"], 2 * n + nr)
            o = Hy.state_scan(s[:, :n], s[:, n:2 * n], s[:, 2 * n:], None, None, None, lw["decay"], kv.rec[l], b.cu_q,
                              b.start_pos, b.slots, r.heads, r.dim, r.vdim)
            span = nr                                       # the heads are normed together
        else:
            assert isinstance(r, RemovalSpec)
            low = F.linear(torch.tanh(proj[:, off["right.w1"]:]), lw["mix.right.w2"])
            s = Hy.removal_prep(proj, off["right.r"], off["right.k"], off["right.v"], off["right.a"], low,
                                lw["mix.right.w0"], lw["mix.right.a.b"], r.heads, r.dim)
            o = Hy.state_scan(s[0], s[1], s[2], s[3], s[4], s[5], None, kv.rec[l], b.cu_q, b.start_pos, b.slots,
                              r.heads, r.dim, r.dim)
            span = r.dim
        Hy.head_norm_gate(o, lw["mix.right.norm"], span, proj, off["right.g"], "sigmoid", eps, m.right_scale, cat, nl)
        return cat

    def _delta(self, proj, m: DeltaSpec, lw, l, positions, kv, b, decode):
        adt, T = self.dtype, proj.shape[0]
        off = lw["off"]
        five, v = Hy.delta_prep(proj, m, off["q"], off["b"], off["a"], lw["conv_w"], kv.sconv[l], lw["neg_rate"],
                                lw["mix.dt_bias"], b.row_seq, positions, b.start_pos, b.slots, shift_state=decode)
        if not decode:
            Hy.conv_state_update(proj, off["q"], m.conv_channels, kv.sconv[l], 0, b.cu_q, b.start_pos, b.slots)
        o = Hy.state_scan(five[0], five[1], v, five[2], five[3], five[4], None, kv.rec[l], b.cu_q, b.start_pos, b.slots,
                          m.heads, m.dim, m.vdim)
        out = torch.empty(T, m.heads * m.vdim, dtype=adt, device=proj.device)
        return Hy.head_norm_gate(o, lw["mix.norm"], m.vdim, proj, off["g"], "silu", self.cfg.norm_eps, 1.0, out, 0)

    def forward(self, ids: torch.Tensor, positions: torch.Tensor, kv, meta: AttnMeta,
                hidden: Optional[torch.Tensor] = None, keep_layers: Optional[list] = None) -> torch.Tensor:
        """Logits [rows, vocab] fp32: every row of a decode step, ``meta.last_rows`` of a varlen
        step (all rows when it is None). ``keep_layers``: a list that receives the residual stream
        after every layer (debugging / tests)."""
        cfg, adt = self.cfg, self.dtype
        eps = cfg.norm_eps
        T = ids.shape[0]
        b = self._rows(positions, meta)
        decode = meta.kind == "decode"
        skinny = decode and T <= 32 and ids.is_cuda and self.use_skinny and bool(self.decode_weights())
        x = F.embedding(ids, self.w["embed"]).float()
        if cfg.embed_scale != 1.0:
            x = x * cfg.embed_scale
        pend = pend2 = None         # a sublayer output (in up to two parts) whose normed add is still to come
        pend_w = None
        for l, ls in enumerate(cfg.layers):
            lw, m = self.layers[l], ls.mixer
            conv = kv.conv[l]
            h, x = Hy.canon_add(x, pend, pend2, pend_w, eps, lw["canon1"], conv, 0, b.row_seq, positions, b.start_pos,
                                b.slots, adt, shift_state=decode)
            if not decode:
                Hy.conv_state_update(x, 0, cfg.hidden, conv, 0, b.cu_q, b.start_pos, b.slots)
            proj = self._linear(h, l, "w_in", skinny)
            if isinstance(m, DeltaSpec):
                o = self._delta(proj, m, lw, l, positions, kv, b, decode)
            else:
                o = self._parallel(proj, m, lw, l, positions, kv, meta, b, decode)
            pend, pend2, pend_w = self._linear(o, l, "w_out", skinny), None, lw["norm1"]
            if ls.ff:
                h, x = Hy.canon_add(x, pend, None, pend_w, eps, lw["canon2"], conv, 1, b.row_seq, positions, b.start_pos,
                                    b.slots, adt, shift_state=decode)
                if not decode:
                    Hy.conv_state_update(x, 0, cfg.hidden, conv, 1, b.cu_q, b.start_pos, b.slots)
                idx, wt = Hy.route_topk(h, lw["mlp.router"], ls.moe.top)
                pend = Hy.moe_experts(h, idx, wt, lw["w_up"], lw["w_down"], adt, act="relu2")
                if ls.moe.shared_ff:
                    pend2 = self._linear(Hy.relu2(self._linear(h, l, "mlp.shared.up", skinny), adt), l, "mlp.shared.down",
                                         skinny)
                pend_w = lw["norm2"]
            if keep_layers is not None:
                _, x = Hy.canon_add(x, pend, pend2, pend_w, eps, None, conv, 0, b.row_seq, positions, b.start_pos, b.slots,
                                    adt)
                pend = pend2 = None
                keep_layers.append(x.clone())
        if not decode and meta.last_rows is not None:
            x = x.index_select(0, meta.last_rows)
            pend = pend.index_select(0, meta.last_rows) if pend is not None else None
            pend2 = pend2.index_select(0, meta.last_rows) if pend2 is not None else None
        _, x = Hy.canon_add(x, pend, pend2, pend_w, eps, None, None, 0, b.row_seq, positions, b.start_pos, b.slots, adt)
        xn = Hy.add_norm(x, None, self.final_norm, eps, adt)
        logits = F.linear(xn, self.w["embed"]).float()
        return logits * cfg.logit_scale if cfg.logit_scale != 1.0 else logits
