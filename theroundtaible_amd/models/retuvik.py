"""Retuvik decoder: pre-norm layers over an fp32 residual stream whose norms work on equal parts
of a row; the mixer is either wkv time mixing (five token-shifted copies of the input feed r, k,
v, an output gate and a low-rank decay path; a heads x dim x dim fp32 state per sequence) or
windowed grouped-query attention without rotation (weighted unit-RMS queries and keys, a query
factor that grows with the logarithm of the position, unit-RMS values, a per-head penalty on the
distance, a sigmoid output gate); the feed-forward is dense with the xIELU activation and biases,
or a routed mixture of silu-gated experts. A span of layers may run several times in a row with
the same weights, every run with a cache and state of its own; every pass of that span starts by
adding a learned step vector, and every pass but the first the embedding output again.

Per layer run (the same code for prompts, portions of prompts, single decoded tokens and any mix
of them in one batch; only the attention launch differs):

    wkv:        mix, x = shift_norm(x, pending)     H1 (HIP): pending residual add + grouped RMS norm
                                                    + the five token-shift mixes of the row
                rkvg   = mix[0..3] @ [Wr; Wk; Wv; Wg]^T           one batched GEMM
                lw     = tanh(mix[4] @ W1^T) @ W2^T              the decay's low-rank path
                o      = wkv_scan(rkvg, lw)         H8 (HIP): decay, recurrence, per-head unit RMS,
                                                    weight, silu gate; long spans in parallel chunks
    attention:  h      = add_norm(x, pending)       H6 (HIP)
                proj   = h @ [Wq; Wk; Wv; Wg]^T     one GEMM for every projection that reads h
                q      = qk_prep(proj)              H2 (HIP): norms, weights, query factor, unit-RMS
                                                    values; keys and values -> the paged cache
                o      = gqa_attention(q)           H3 (HIP): window, distance penalty, output gate
    pending = o @ Wo^T
    h       = add_norm(x, pending)                  H6 (HIP)
    dense:      pending = xielu(h @ Wup^T + b) @ Wdown^T + b     H9 (HIP) between two GEMMs
    experts:    idx, wt = topk_softmax(h @ Wrouter^T + b)        fp32 GEMM, H11 (HIP)
                pending = moe_experts(h, idx, wt)   a few rows: H12 (HIP), two launches; more rows:
                                                    each expert's rows through library GEMMs, H10

The residual stream, every norm, positions, scores and softmax, the router, the token-shift state,
the decay and the whole recurrence are fp32 whatever the model dtype; GEMM operands, the
activations between them and the key / value cache take the model dtype.
"""
from __future__ import annotations

import math
from typing import Dict, Optional

import torch
import torch.nn.functional as F

from ..ops import hybrid as Hy
from ..parallel.tp import TPInfo
from .config import GroupedAttentionSpec, ModelConfig, WKVSpec
from .goganex import GoganexModel
from .llama import AttnMeta


def _softplus(v: float) -> float:
    return v if v > 30.0 else math.log1p(math.exp(v))


class RetuvikModel(GoganexModel):
    """Shares the row bookkeeping, attention tile maps, split-key workspaces and decode GEMMs of
    :class:`GoganexModel`; the layers, the cache shapes and the forward are its own."""
    matrix_attention = False       # the matrix-core attention kernels know no window or distance penalty
    _DEC_LINEARS = ("w_in", "mix.o", "mix.w1", "mlp.up", "mlp.down")

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
        for ls in cfg.layers:
            i = ls.source
            if i in self.layers:
                continue
            p = f"l{i}."
            lw = {k[len(p):]: v for k, v in weights.items() if k.startswith(p)}
            m = ls.mixer
            if isinstance(m, WKVSpec):
                lw["mu"] = torch.stack([lw.pop("mix.mu." + n) for n in "rkvgw"]).to(f32).contiguous()
                lw["w_rkvg"] = torch.stack([lw.pop("mix." + n) for n in "rkvg"]).contiguous()     # [4, H * D, W]
                fp = ("mix.w0", "mix.u", "mix.norm")
            else:
                lw["w_in"] = torch.cat([lw.pop("mix.q"), lw.pop("mix.k"), lw.pop("mix.v"), lw.pop("mix.g")]).contiguous()
                lw["slopes"] = torch.tensor([2.0 ** (-m.slope_base * (a + 1) / m.heads) for a in range(m.heads)],
                                            dtype=f32, device=self.device) if m.slope_base > 0 else None
                fp = ("mix.q.norm", "mix.k.norm")
            if ls.ff and ls.ff_kind == "moe":
                E = ls.moe.experts
                lw["w_gu"] = torch.stack([torch.cat([lw.pop(f"mlp.e{e}.gate"), lw.pop(f"mlp.e{e}.up")])
                                          for e in range(E)]).contiguous()                           # [E, 2F, W]
                lw["w_down"] = torch.stack([lw.pop(f"mlp.e{e}.down") for e in range(E)]).contiguous()  # [E, W, F]
                fp += ("mlp.router", "mlp.router.b")
            elif ls.ff:
                a = lw.pop("mlp.act").to(torch.float64).tolist()
                lw["act"] = (_softplus(a[0]), 0.5 + _softplus(a[1]))
                fp += ("mlp.up.b",)
            for n in ("norm1", "norm2") + fp:
                if n in lw:
                    lw[n] = lw[n].to(f32).contiguous()
            self.layers[i] = lw
        self.final_norm = weights["final.norm"].to(f32).contiguous()
        self.loop_step = weights["loop.step"].to(f32).contiguous() if cfg.loop_passes else None
        self._dec = None
        self._split_ws = None
        self._static = {}
        self._ws = {}

    # ---- cache ------------------------------------------------------------------------------------
    def cache_shapes(self):
        return [(m.kv_heads, m.dim, m.vdim) if isinstance(m, GroupedAttentionSpec) else None
                for m in (ls.mixer for ls in self.cfg.layers)]

    def make_cache(self, num_blocks: int, block_size: int, device, dtype, n_slots: int):
        from ..engine.kv_cache import GroupedKVCache
        wkv = [isinstance(ls.mixer, WKVSpec) for ls in self.cfg.layers]
        rec = [ls.mixer.state_size if on else 0 for ls, on in zip(self.cfg.layers, wkv)]
        return GroupedKVCache(self.cache_shapes(), self.cfg.hidden, rec, num_blocks, block_size, device, dtype,
                              n_slots=n_slots, shift_layers=wkv)

    def cache_bytes_per_block(self, block_size: int, dtype_bytes: int) -> int:
        return max(1, sum(sh[0] * (sh[1] + sh[2]) for sh in self.cache_shapes() if sh is not None)) * block_size * dtype_bytes

    # ---- forward ----------------------------------------------------------------------------------
    def _wkv_chunks(self, meta: AttnMeta, b):
        """Work lists of the chunked wkv scan for this batch (None: no long span)."""
        cache = meta.latent_tiles if meta.latent_tiles is not None else {}
        meta.latent_tiles = cache
        if "wkv" not in cache:
            cu = meta.host_rows[0] if meta.host_rows is not None else b.cu_q.cpu()
            cache["wkv"] = Hy.wkv_chunks(cu, b.cu_q.device)
        return cache["wkv"]

    def _window_splits(self, a: GroupedAttentionSpec, rows: int) -> int:
        """Key ranges per decoded row: as many as fill the chip, but no more than the tiles a
        window can touch."""
        splits = self.decode_splits(rows, a.kv_heads)
        if splits > 1 and a.window > 0:
            kt = max(1, Hy.native().gqa_key_tile(a.dim, a.vdim))
            splits = max(1, min(splits, (a.window + kt - 1) // kt + 1))
        return splits

    def _attention(self, h, a, lw, l, src, positions, kv, meta, b, decode, skinny):
        adt, T = self.dtype, h.shape[0]
        proj = self._linear(h, src, "w_in", skinny)
        k_off = a.heads * a.dim
        v_off = k_off + a.kv_heads * a.dim
        g_off = v_off + a.kv_heads * a.vdim
        q = Hy.qk_prep(proj, a, 0, k_off, v_off, None, self.cfg.norm_eps, positions, kv.k_layer(l), kv.v_layer(l),
                       meta.slot_mapping, adt, q_weight=lw["mix.q.norm"] if a.qk_weight else None,
                       k_weight=lw["mix.k.norm"] if a.qk_weight else None)
        splits = self._window_splits(a, T) if decode else 1
        return Hy.gqa_attention(q, kv.k_layer(l), kv.v_layer(l), meta.block_tables, b.cu_q, b.start_pos, a.scale, None,
                                a.sink, tiles=self._tiles(meta, Hy.rows_per_tile(a.group), b) if proj.is_cuda else None,
                                num_splits=splits, workspace=self._workspace(T, a, splits), out_dtype=adt,
                                window=a.window, slopes=lw["slopes"], gate=proj if a.out_gate else None, gate_off=g_off)

    def _wkv(self, mix, m, lw, l, src, kv, meta, b, decode, skinny):
        adt = self.dtype
        rkvg = torch.bmm(mix[:4], lw["w_rkvg"].transpose(1, 2))                      # [4, T, H * D]
        low = F.linear(torch.tanh(self._linear(mix[4], src, "mix.w1", skinny)), lw["mix.w2"])
        chunks = self._wkv_chunks(meta, b) if mix.is_cuda and not decode else None
        return Hy.wkv_scan(rkvg, low, lw["mix.w0"], lw["mix.u"], lw["mix.norm"], self.cfg.norm_eps, kv.rec[l], b.cu_q,
                           b.start_pos, b.slots, adt, chunks=chunks)

    def forward(self, ids: torch.Tensor, positions: torch.Tensor, kv, meta: AttnMeta,
                hidden: Optional[torch.Tensor] = None, keep_layers: Optional[list] = None) -> torch.Tensor:
        """Logits [rows, vocab] fp32: every row of a decode step, ``meta.last_rows`` of a varlen
        step (all rows when it is None). ``keep_layers``: a list that receives the residual stream
        after every layer run (debugging / tests)."""
        cfg, adt = self.cfg, self.dtype
        eps, groups = cfg.norm_eps, cfg.norm_groups
        T = ids.shape[0]
        b = self._rows(positions, meta)
        decode = meta.kind == "decode"
        skinny = decode and T <= 32 and ids.is_cuda and self.use_skinny and bool(self.decode_weights())
        e0 = F.embedding(ids, self.w["embed"]).float()
        if cfg.embed_scale != 1.0:
            e0 = e0 * cfg.embed_scale
        x = e0.clone() if cfg.loop_passes > 1 else e0     # norm launches add into x in place
        pend: Optional[torch.Tensor] = None     # a branch output whose residual add is still to come
        for l, ls in enumerate(cfg.layers):
            src, lw, m = ls.source, self.layers[ls.source], ls.mixer
            if ls.opens_pass is not None:       # a pass of the looped span starts: embedding again, step vector
                x = x + self.loop_step[ls.opens_pass]
                if ls.opens_pass > 0:
                    x += e0
                if pend is not None:
                    x, pend = x.add_(pend.float()), None
            elif pend is not None and not self.fuse_adds:
                x, pend = x + pend.float(), None
            if isinstance(m, WKVSpec):
                mix, x = Hy.shift_norm(x, pend, lw["norm1"], eps, lw["mu"], kv.shift[l], b.row_seq, positions, b.start_pos,
                                       b.slots, adt, shift_state=decode, groups=groups)
                if not decode:
                    Hy.shift_state_update(x, lw["norm1"], eps, kv.shift[l], b.cu_q, b.slots, groups)
                o = self._wkv(mix, m, lw, l, src, kv, meta, b, decode, skinny)
            else:
                h = Hy.add_norm(x, pend, lw["norm1"], eps, adt, groups)
                o = self._attention(h, m, lw, l, src, positions, kv, meta, b, decode, skinny)
            pend = self._linear(o, src, "mix.o", skinny)
            if ls.ff:
                if not self.fuse_adds:
                    x, pend = x + pend.float(), None
                h = Hy.add_norm(x, pend, lw["norm2"], eps, adt, groups)
                if ls.ff_kind == "moe":
                    logits = F.linear(h.float(), lw["mlp.router"], lw["mlp.router.b"])
                    idx, wt = Hy.topk_softmax(logits, ls.moe.top)
                    pend = Hy.moe_experts(h, idx, wt, lw["w_gu"], lw["w_down"], adt)
                else:
                    act = Hy.xielu(self._linear(h, src, "mlp.up", skinny), lw["mlp.up.b"], lw["act"][0], lw["act"][1], adt)
                    if skinny and "mlp.down" in self._dec[src]:
                        pend = self._linear(act, src, "mlp.down", True).add_(lw["mlp.down.b"])
                    else:
                        pend = F.linear(act, lw["mlp.down"], lw["mlp.down.b"])
            if keep_layers is not None:
                if pend is not None:
                    x, pend = x + pend.float(), None
                keep_layers.append(x.clone())
        if not decode and meta.last_rows is not None:
            x = x.index_select(0, meta.last_rows)
            pend = pend.index_select(0, meta.last_rows) if pend is not None else None
        xn = Hy.add_norm(x, pend, self.final_norm, eps, adt, groups)
        return F.linear(xn, self.w["head"]).float()
