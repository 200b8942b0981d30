"""Weight materialization: seeded random init (benchmarks: no network, no checkpoints) or safetensors.

``random:<seed>`` generates every tensor directly on the target device with a
generator seeded by (seed, tensor name, tp rank) — an 8B model materializes in well
under a second on MI355X. ``random-full:<seed>`` builds the *unsharded* tensors on CPU
first and then shards them, so TP=1 and TP=N see identical math (TP equivalence
tests). ``random-dev:<seed>`` does the same with the full tensors generated on the target
device, one tensor at a time (GPU TP checks at 8B / 70B shapes, where CPU generation of the
unsharded model would take minutes and tens of GB of host memory per rank).
A path loads HF-named safetensors (Llama/Mistral/Qwen2/GPT-2 naming) and shards it.
"""
from __future__ import annotations

import hashlib
import os
from typing import Callable, Dict, Optional, Tuple

import torch

from ..parallel.tp import TPInfo, shard_cols, shard_rows
from .config import ModelConfig

# (shape, init-kind, parallel-kind); kinds: "normal", "ones", "zeros"; parallel: None|"row"|"col"|"qkv"|"gateup"|"vocab"


def _seed_for(base: int, name: str, rank: int) -> int:
    h = hashlib.sha256(f"{base}:{name}:{rank}".encode()).digest()
    return int.from_bytes(h[:8], "little") & ((1 << 63) - 1)


def llama_layout(cfg: ModelConfig) -> Dict[str, Tuple[Tuple[int, ...], str, Optional[str]]]:
    H, D = cfg.hidden, cfg.head_dim
    lay: Dict[str, Tuple[Tuple[int, ...], str, Optional[str]]] = {
        "embed": ((cfg.vocab, H), "normal", None),
        "final_norm": ((H,), "ones", None),
        "lm_head": ((cfg.vocab, H), "normal", "vocab"),
    }
    for i in range(cfg.n_layers):
        p = f"layers.{i}."
        lay[p + "attn_norm"] = ((H,), "ones", None)
        lay[p + "wqkv"] = (((cfg.n_heads + 2 * cfg.n_kv_heads) * D, H), "normal", "qkv")
        if cfg.qkv_bias:
            lay[p + "bqkv"] = (((cfg.n_heads + 2 * cfg.n_kv_heads) * D,), "normal", "qkv")
        lay[p + "wo"] = ((H, cfg.n_heads * D), "normal", "col")
        lay[p + "ffn_norm"] = ((H,), "ones", None)
        lay[p + "w_gate_up"] = ((2 * cfg.ffn, H), "normal", "gateup")
        lay[p + "w_down"] = ((H, cfg.ffn), "normal", "col")
    return lay


def gpt2_layout(cfg: ModelConfig) -> Dict[str, Tuple[Tuple[int, ...], str, Optional[str]]]:
    H, F = cfg.hidden, cfg.ffn
    lay: Dict[str, Tuple[Tuple[int, ...], str, Optional[str]]] = {
        "wte": ((cfg.vocab, H), "normal", None),
        "wpe": ((cfg.max_pos, H), "normal", None),
        "ln_f.w": ((H,), "ones", None), "ln_f.b": ((H,), "zeros", None),
    }
    for i in range(cfg.n_layers):
        p = f"layers.{i}."
        lay[p + "ln1.w"] = ((H,), "ones", None)
        lay[p + "ln1.b"] = ((H,), "zeros", None)
        lay[p + "w_qkv"] = ((3 * H, H), "normal", "qkv")
        lay[p + "b_qkv"] = ((3 * H,), "zeros", "qkv")
        lay[p + "w_o"] = ((H, H), "normal", "col")
        lay[p + "b_o"] = ((H,), "zeros", None)
        lay[p + "ln2.w"] = ((H,), "ones", None)
        lay[p + "ln2.b"] = ((H,), "zeros", None)
        lay[p + "w_fc"] = ((F, H), "normal", "row")
        lay[p + "b_fc"] = ((F,), "zeros", "row")
        lay[p + "w_proj"] = ((H, F), "normal", "col")
        lay[p + "b_proj"] = ((H,), "zeros", None)
    return lay


def mupulorn_layout(cfg: ModelConfig) -> Dict[str, Tuple[Tuple[int, ...], str, Optional[str]]]:
    """Checkpoint names and shapes of a Mupulorn model (linear weights [out, in]); layers that run
    another layer's weights have no tensors. Not tensor-parallel: every kind is None."""
    W = cfg.hidden
    lay: Dict[str, Tuple[Tuple[int, ...], str, Optional[str]]] = {
        "embed": ((cfg.vocab, W), "normal", None),
        "final.norm": ((), "ones", None),
        "head": ((cfg.vocab, W), "normal", None),
    }
    for i, ls in enumerate(cfg.layers):
        if ls.source != i:
            continue
        p, m = f"l{i}.", ls.mixer
        for n in ("norm1", "norm1b"):
            lay[p + n] = ((), "ones", None)
        lay[p + "canon1"] = ((W, cfg.canon_taps), "small", None)
        lay[p + "mix.dq"] = ((m.q_rank, W), "normal", None)
        lay[p + "mix.dq.norm"] = ((m.q_rank,), "ones", None)
        lay[p + "mix.uq"] = ((m.heads * (m.dim + m.rot_dim), m.q_rank), "normal", None)
        lay[p + "mix.dkv"] = ((m.kv_rank + m.rot_dim, W), "normal", None)
        lay[p + "mix.dkv.norm"] = ((m.kv_rank,), "ones", None)
        lay[p + "mix.uk"] = ((m.heads * m.dim, m.kv_rank), "normal", None)
        lay[p + "mix.uv"] = ((m.heads * m.vdim, m.kv_rank), "normal", None)
        lay[p + "mix.sink"] = ((m.heads,), "zeros", None)
        lay[p + "mix.g"] = ((m.heads * m.vdim, W), "normal", None)
        lay[p + "mix.o"] = ((W, m.heads * m.vdim), "normal", None)
        if ls.ff:
            for n in ("norm2", "norm2b"):
                lay[p + n] = ((), "ones", None)
            lay[p + "canon2"] = ((W, cfg.canon_taps), "small", None)
            lay[p + "mlp.up"] = ((ls.ff, W), "normal", None)
            lay[p + "mlp.down"] = ((W, ls.ff), "normal", None)
            lay[p + "mlp.act"] = ((4,), "poly", None)
    return lay


def goganex_layout(cfg: ModelConfig) -> Dict[str, Tuple[Tuple[int, ...], str, Optional[str]]]:
    """Checkpoint names and shapes of a Goganex model (linear weights [out, in]). A looped layer
    has one set of tensors, named by its place in the checkpoint's layer list. Not
    tensor-parallel: every kind is None."""
    from .config import ParallelSpec
    W = cfg.hidden
    lay: Dict[str, Tuple[Tuple[int, ...], str, Optional[str]]] = {
        "embed": ((cfg.vocab, W), "normal", None),
        "final.norm": ((W,), "ones", None),
        "head": ((cfg.vocab, W), "normal", None),
    }
    for ls in cfg.layers:
        p = f"l{ls.source}."
        if p + "norm1" in lay:
            continue
        lay[p + "norm1"] = ((W,), "ones", None)
        lay[p + "shift"] = ((W,), "half", None)
        if isinstance(ls.mixer, ParallelSpec):
            a, r = ls.mixer.left, ls.mixer.right
            lay[p + "mix.left.q"] = ((a.heads * a.dim, W), "normal", None)
            lay[p + "mix.left.k"] = ((a.kv_heads * a.dim, W), "normal", None)
            lay[p + "mix.left.o"] = ((W, a.heads * a.vdim), "normal", None)
            for n in ("z", "x", "g"):
                lay[p + f"mix.right.{n}"] = ((r.width, W), "normal", None)
            lay[p + "mix.right.z.b"] = ((r.width,), "zeros", None)
            lay[p + "mix.right.x.b"] = ((r.width,), "zeros", None)
            lay[p + "mix.right.o"] = ((W, r.width), "normal", None)
            lay[p + "mix.left.out"] = ((W,), "ones", None)
            lay[p + "mix.right.out"] = ((W,), "ones", None)
        else:
            a = ls.mixer
            lay[p + "mix.q"] = ((a.heads * a.dim, W), "normal", None)
            lay[p + "mix.k"] = ((a.kv_heads * a.dim, W), "normal", None)
            lay[p + "mix.v"] = ((a.kv_heads * a.vdim, W), "normal", None)
            lay[p + "mix.temp"] = ((a.heads,), "ones", None)
            lay[p + "mix.o"] = ((W, a.heads * a.vdim), "normal", None)
        if ls.ff:
            lay[p + "norm2"] = ((W,), "ones", None)
            lay[p + "mlp.gate"] = ((ls.ff, W), "normal", None)
            lay[p + "mlp.up"] = ((ls.ff, W), "normal", None)
            lay[p + "mlp.down"] = ((W, ls.ff), "normal", None)
    return lay


def retuvik_layout(cfg: ModelConfig) -> Dict[str, Tuple[Tuple[int, ...], str, Optional[str]]]:
    """Checkpoint names and shapes of a Retuvik model (linear weights [out, in]). A looped layer has
    one set of tensors, named by its place in the checkpoint's layer list. The rank of a wkv
    mixer's decay path is whatever ``mix.w1`` / ``mix.w2`` have (-1 in the shape) unless the spec
    names one. Not tensor-parallel: every kind is None."""
    from .config import WKVSpec
    W = cfg.hidden
    lay: Dict[str, Tuple[Tuple[int, ...], str, Optional[str]]] = {
        "embed": ((cfg.vocab, W), "normal", None),
        "final.norm": ((W,), "ones", None),
        "head": ((cfg.vocab, W), "normal", None),
    }
    if cfg.loop_passes:
        lay["loop.step"] = ((cfg.loop_passes, W), "normal", None)
    for ls in cfg.layers:
        p = f"l{ls.source}."
        if p + "norm1" in lay:
            continue
        lay[p + "norm1"] = ((W,), "ones", None)
        m = ls.mixer
        if isinstance(m, WKVSpec):
            rank = m.decay_rank or -1
            for n in "rkvgw":
                lay[p + "mix.mu." + n] = ((W,), "half", None)
            for n in "rkvg":
                lay[p + "mix." + n] = ((m.width, W), "normal", None)
            lay[p + "mix.w1"] = ((rank, W), "normal", None)
            lay[p + "mix.w2"] = ((m.width, rank), "normal", None)
            lay[p + "mix.w0"] = ((m.width,), "zeros", None)
            lay[p + "mix.u"] = ((m.heads, m.dim), "small", None)
            lay[p + "mix.norm"] = ((m.width,), "ones", None)
            lay[p + "mix.o"] = ((W, m.width), "normal", None)
        else:
            lay[p + "mix.q"] = ((m.heads * m.dim, W), "normal", None)
            lay[p + "mix.k"] = ((m.kv_heads * m.dim, W), "normal", None)
            lay[p + "mix.v"] = ((m.kv_heads * m.vdim, W), "normal", None)
            lay[p + "mix.q.norm"] = ((m.dim,), "ones", None)
            lay[p + "mix.k.norm"] = ((m.dim,), "ones", None)
            lay[p + "mix.g"] = ((m.heads * m.vdim, W), "normal", None)
            lay[p + "mix.o"] = ((W, m.heads * m.vdim), "normal", None)
        if not ls.ff:
            continue
        lay[p + "norm2"] = ((W,), "ones", None)
        if ls.ff_kind == "moe":
            for e in range(ls.moe.experts):
                lay[p + f"mlp.e{e}.gate"] = ((ls.ff, W), "normal", None)
                lay[p + f"mlp.e{e}.up"] = ((ls.ff, W), "normal", None)
                lay[p + f"mlp.e{e}.down"] = ((W, ls.ff), "normal", None)
            lay[p + "mlp.router"] = ((ls.moe.experts, W), "normal", None)
            lay[p + "mlp.router.b"] = ((ls.moe.experts,), "zeros", None)
        else:
            lay[p + "mlp.up"] = ((ls.ff, W), "normal", None)
            lay[p + "mlp.up.b"] = ((ls.ff,), "zeros", None)
            lay[p + "mlp.down"] = ((W, ls.ff), "normal", None)
            lay[p + "mlp.down.b"] = ((W,), "zeros", None)
            lay[p + "mlp.act"] = ((2,), "zeros", None)
    return lay


def ledinex_layout(cfg: ModelConfig) -> Dict[str, Tuple[Tuple[int, ...], str, Optional[str]]]:
    """Checkpoint names and shapes of a Ledinex model (linear weights [out, in]). The logits read
    the embedding table, so there is no head tensor. The rank of a generalized-delta mixer's decay
    path is whatever ``w1`` / ``w2`` have (-1 in the shape) unless the spec names one. Not
    tensor-parallel: every kind is None."""
    from .config import DecaySumSpec, DeltaSpec, RemovalSpec
    W = cfg.hidden
    lay: Dict[str, Tuple[Tuple[int, ...], str, Optional[str]]] = {
        "embed": ((cfg.vocab, W), "normal", None),
        "final.norm": ((W,), "zeros", None),
    }
    for i, ls in enumerate(cfg.layers):
        p, m = f"l{i}.", ls.mixer
        lay[p + "norm1"] = ((W,), "zeros", None)
        lay[p + "canon1"] = ((W, cfg.canon_taps), "small", None)
        if isinstance(m, DeltaSpec):
            q = p + "mix."
            for n, rows in (("q", m.kv_heads * m.dim), ("k", m.kv_heads * m.dim), ("v", m.heads * m.vdim)):
                lay[q + n] = ((rows, W), "normal", None)
                lay[q + n + ".conv"] = ((rows, m.conv), "conv", None)
            lay[q + "b"] = ((m.heads, W), "normal", None)
            lay[q + "a"] = ((m.heads, W), "normal", None)
            lay[q + "A_log"] = ((m.heads,), "zeros", None)
            lay[q + "dt_bias"] = ((m.heads,), "zeros", None)
            lay[q + "norm"] = ((m.vdim,), "ones", None)
            lay[q + "g"] = ((m.heads * m.vdim, W), "normal", None)
            lay[q + "o"] = ((W, m.heads * m.vdim), "normal", None)
        else:
            a, r = m.left, m.right
            q = p + "mix.left."
            lay[q + "q"] = ((a.heads * a.dim, W), "normal", None)
            lay[q + "k"] = ((a.kv_heads * a.dim, W), "normal", None)
            if a.bias:
                lay[q + "q.b"] = ((a.heads * a.dim,), "zeros", None)
                lay[q + "k.b"] = ((a.kv_heads * a.dim,), "zeros", None)
            if not a.value_from_key:
                lay[q + "v"] = ((a.kv_heads * a.vdim, W), "normal", None)
            lay[q + "q.norm"] = ((a.heads * a.dim,), "ones", None)
            lay[q + "k.norm"] = ((a.kv_heads * a.dim,), "ones", None)
            lay[q + "o"] = ((W, a.heads * a.vdim), "normal", None)
            q = p + "mix.right."
            if isinstance(r, DecaySumSpec):
                lay[q + "q"] = ((r.heads * r.dim, W), "normal", None)
                lay[q + "k"] = ((r.heads * r.dim, W), "normal", None)
                lay[q + "v"] = ((r.heads * r.vdim, W), "normal", None)
            elif isinstance(r, RemovalSpec):
                rank = r.decay_rank or -1
                for n in "rkv":
                    lay[q + n] = ((r.heads * r.dim, W), "normal", None)
                lay[q + "a"] = ((r.heads * r.dim, W), "normal", None)
                lay[q + "a.b"] = ((r.heads * r.dim,), "zeros", None)
                lay[q + "w1"] = ((rank, W), "normal", None)
                lay[q + "w2"] = ((r.heads * r.dim, rank), "normal", None)
                lay[q + "w0"] = ((r.heads * r.dim,), "zeros", None)
            lay[q + "g"] = ((r.heads * r.vdim, W), "normal", None)
            lay[q + "norm"] = ((r.heads * r.vdim,), "ones", None)
            lay[q + "o"] = ((W, r.heads * r.vdim), "normal", None)
        if not ls.ff:
            continue
        lay[p + "norm2"] = ((W,), "zeros", None)
        lay[p + "canon2"] = ((W, cfg.canon_taps), "small", None)
        for e in range(ls.moe.experts):
            lay[p + f"mlp.e{e}.up"] = ((ls.ff, W), "normal", None)
            lay[p + f"mlp.e{e}.down"] = ((W, ls.ff), "normal", None)
        lay[p + "mlp.router"] = ((ls.moe.experts, W), "normal", None)
        if ls.moe.shared_ff:
            lay[p + "mlp.shared.up"] = ((ls.moe.shared_ff, W), "normal", None)
            lay[p + "mlp.shared.down"] = ((W, ls.moe.shared_ff), "normal", None)
    return lay


def layout_for(cfg: ModelConfig):
    if cfg.arch == "mupulorn":
        return mupulorn_layout(cfg)
    if cfg.arch == "goganex":
        return goganex_layout(cfg)
    if cfg.arch == "retuvik":
        return retuvik_layout(cfg)
    if cfg.arch == "ledinex":
        return ledinex_layout(cfg)
    return gpt2_layout(cfg) if cfg.arch == "gpt2" else llama_layout(cfg)


def shard_tensor(name: str, w: torch.Tensor, kind: Optional[str], cfg: ModelConfig, tp: TPInfo) -> torch.Tensor:
    if tp.size == 1 or kind is None:
        return w
    if kind in ("row", "vocab"):
        if kind == "vocab" and w.shape[0] % tp.size:
            pad = tp.size - w.shape[0] % tp.size
            w = torch.cat([w, w.new_zeros((pad,) + tuple(w.shape[1:]))])
        return shard_rows(w, tp)
    if kind == "col":
        return shard_cols(w, tp)
    if kind == "gateup":
        g, u = w.chunk(2, dim=0)
        return torch.cat([shard_rows(g, tp), shard_rows(u, tp)])
    if kind == "qkv":
        D = cfg.head_dim
        q, k, v = w.split([cfg.n_heads * D, cfg.n_kv_heads * D, cfg.n_kv_heads * D], dim=0)
        h0, nh = tp.kv_head0(cfg.n_kv_heads), tp.kv_heads(cfg.n_kv_heads)
        return torch.cat([shard_rows(q, tp), k[h0 * D:(h0 + nh) * D], v[h0 * D:(h0 + nh) * D]])
    raise ValueError(kind)


def local_shape(shape, kind, cfg: ModelConfig, tp: TPInfo):
    if tp.size == 1 or kind is None:
        return shape
    s = list(shape)
    if kind in ("row", "gateup"):
        s[0] //= tp.size
    elif kind == "vocab":
        s[0] = (s[0] + tp.size - 1) // tp.size
    elif kind == "col":
        s[1] //= tp.size
    elif kind == "qkv":
        s[0] = (cfg.n_heads // tp.size + 2 * tp.kv_heads(cfg.n_kv_heads)) * cfg.head_dim
    return tuple(s)


def materialize(cfg: ModelConfig, spec: str, device, dtype=torch.bfloat16, tp: Optional[TPInfo] = None,
                std: float = 0.02) -> Dict[str, torch.Tensor]:
    tp = tp or TPInfo()
    lay = layout_for(cfg)
    out: Dict[str, torch.Tensor] = {}
    if spec.startswith(("random:", "random-full:", "random-dev:")):
        full = spec.startswith(("random-full:", "random-dev:"))
        gen_dev = torch.device(device) if spec.startswith("random-dev:") else torch.device("cpu")
        seed = int(spec.split(":", 1)[1] or 0)
        for name, (shape, init, kind) in lay.items():
            if full:
                g = torch.Generator(device=gen_dev).manual_seed(_seed_for(seed, name, 0))
                w = _init(shape, init, std, g, gen_dev, torch.float32)
                if init == "normal" and name in ("embed", "wte"):
                    w = w * 10  # unit-ish scale residual stream for the embedding
                out[name] = shard_tensor(name, w, kind, cfg, tp).to(device=device, dtype=dtype).contiguous()
                del w
            else:
                shp = local_shape(shape, kind, cfg, tp)
                dev = torch.device(device)
                g = torch.Generator(device=dev).manual_seed(_seed_for(seed, name, tp.rank))
                w = _init(shp, init, std, g, dev, dtype)
                if init == "normal" and name in ("embed", "wte"):
                    w.mul_(10)
                out[name] = w
        # GPT-2 reads its tied head from wte; a tied Llama-family model (random init) keeps an
        # independent vocab-parallel lm_head (checkpoints copy the embedding, load_safetensors)
        if cfg.tie_embeddings and cfg.arch == "gpt2" and "lm_head" in out:
            out.pop("lm_head")
        return out
    if os.path.isdir(spec) or spec.endswith(".safetensors"):
        return load_safetensors(cfg, spec, device, dtype, tp)
    raise ValueError(f"unknown weights spec '{spec}' (use random:<seed>, random-full:<seed>, or a path)")


def _init(shape, init, std, g, device, dtype):
    shape = tuple(32 if n < 0 else n for n in shape)     # a size the checkpoint alone would fix
    if init == "ones":
        return torch.ones(shape, device=device, dtype=dtype)
    if init == "zeros":
        return torch.zeros(shape, device=device, dtype=dtype)
    if init == "half":      # token-shift mixing weights
        return torch.full(shape, 0.5, device=device, dtype=dtype)
    if init == "poly":      # PolyNorm coefficients: equal thirds, no offset
        return torch.tensor([1 / 3, 1 / 3, 1 / 3, 0.0], device=device, dtype=dtype)
    if init == "conv":      # short convolution ahead of an activation: most of the weight on the current token
        w = torch.empty(shape, device=device, dtype=dtype)
        w.normal_(0.0, 0.1, generator=g)
        w[..., -1] += 1.0
        return w
    if init == "small":     # input-convolution taps
        w = torch.empty(shape, device=device, dtype=dtype)
        w.normal_(0.0, 0.1, generator=g)
        return w
    w = torch.empty(shape, device=device, dtype=dtype)
    w.normal_(0.0, std, generator=g)
    return w


# ---- safetensors (HF naming) -----------------------------------------------------------------

def _hf_llama_name_map(cfg: ModelConfig) -> Dict[str, Callable[[Dict[str, torch.Tensor]], torch.Tensor]]:
    m: Dict[str, Callable] = {
        "embed": lambda t: t["model.embed_tokens.weight"],
        "final_norm": lambda t: t["model.norm.weight"],
        "lm_head": lambda t: t.get("lm_head.weight", t["model.embed_tokens.weight"]),
    }
    for i in range(cfg.n_layers):
        p = f"model.layers.{i}."
        m[f"layers.{i}.attn_norm"] = lambda t, p=p: t[p + "input_layernorm.weight"]
        m[f"layers.{i}.ffn_norm"] = lambda t, p=p: t[p + "post_attention_layernorm.weight"]
        m[f"layers.{i}.wqkv"] = lambda t, p=p: torch.cat([t[p + "self_attn.q_proj.weight"],
                                                           t[p + "self_attn.k_proj.weight"],
                                                           t[p + "self_attn.v_proj.weight"]])
        if cfg.qkv_bias:
            m[f"layers.{i}.bqkv"] = lambda t, p=p: torch.cat([t[p + "self_attn.q_proj.bias"],
                                                               t[p + "self_attn.k_proj.bias"],
                                                               t[p + "self_attn.v_proj.bias"]])
        m[f"layers.{i}.wo"] = lambda t, p=p: t[p + "self_attn.o_proj.weight"]
        m[f"layers.{i}.w_gate_up"] = lambda t, p=p: torch.cat([t[p + "mlp.gate_proj.weight"],
                                                               t[p + "mlp.up_proj.weight"]])
        m[f"layers.{i}.w_down"] = lambda t, p=p: t[p + "mlp.down_proj.weight"]
    return m


def _hf_gpt2_name_map(cfg: ModelConfig):
    pre = "transformer."

    def g(t, n):
        return t[pre + n] if pre + n in t else t[n]

    m: Dict[str, Callable] = {"wte": lambda t: g(t, "wte.weight"), "wpe": lambda t: g(t, "wpe.weight"),
                              "ln_f.w": lambda t: g(t, "ln_f.weight"), "ln_f.b": lambda t: g(t, "ln_f.bias")}
    for i in range(cfg.n_layers):
        p = f"h.{i}."
        # HF GPT-2 uses Conv1D ([in, out]); transpose to [out, in]
        m[f"layers.{i}.ln1.w"] = lambda t, p=p: g(t, p + "ln_1.weight")
        m[f"layers.{i}.ln1.b"] = lambda t, p=p: g(t, p + "ln_1.bias")
        m[f"layers.{i}.w_qkv"] = lambda t, p=p: g(t, p + "attn.c_attn.weight").t()
        m[f"layers.{i}.b_qkv"] = lambda t, p=p: g(t, p + "attn.c_attn.bias")
        m[f"layers.{i}.w_o"] = lambda t, p=p: g(t, p + "attn.c_proj.weight").t()
        m[f"layers.{i}.b_o"] = lambda t, p=p: g(t, p + "attn.c_proj.bias")
        m[f"layers.{i}.ln2.w"] = lambda t, p=p: g(t, p + "ln_2.weight")
        m[f"layers.{i}.ln2.b"] = lambda t, p=p: g(t, p + "ln_2.bias")
        m[f"layers.{i}.w_fc"] = lambda t, p=p: g(t, p + "mlp.c_fc.weight").t()
        m[f"layers.{i}.b_fc"] = lambda t, p=p: g(t, p + "mlp.c_fc.bias")
        m[f"layers.{i}.w_proj"] = lambda t, p=p: g(t, p + "mlp.c_proj.weight").t()
        m[f"layers.{i}.b_proj"] = lambda t, p=p: g(t, p + "mlp.c_proj.bias")
    return m


def load_safetensors(cfg: ModelConfig, path: str, device, dtype, tp: TPInfo) -> Dict[str, torch.Tensor]:
    from safetensors.torch import load_file
    files = [path] if path.endswith(".safetensors") else sorted(
        os.path.join(path, f) for f in os.listdir(path) if f.endswith(".safetensors"))
    tensors: Dict[str, torch.Tensor] = {}
    for f in files:
        tensors.update(load_file(f, device="cpu"))
    lay = layout_for(cfg)
    out = {}
    if cfg.arch in ("mupulorn", "goganex", "retuvik", "ledinex"):
        # the checkpoint's own names; integer tables keep their type, everything else takes `dtype`
        if tp.size > 1:
            raise ValueError(f"{cfg.arch} checkpoints are not tensor-parallel")
        for name, (shape, _, _) in lay.items():
            if name not in tensors:
                raise KeyError(f"{path}: tensor '{name}' is missing")
            w = tensors[name]
            if len(w.shape) != len(shape) or any(b >= 0 and a != b for a, b in zip(w.shape, shape)):
                raise ValueError(f"{path}: tensor '{name}' has shape {tuple(w.shape)}, config.json gives {tuple(shape)}")
            out[name] = (w if not w.is_floating_point() else w.to(dtype)).to(device).contiguous()
        return out
    name_map = _hf_gpt2_name_map(cfg) if cfg.arch == "gpt2" else _hf_llama_name_map(cfg)
    for name, fn in name_map.items():
        if name == "lm_head" and cfg.tie_embeddings and cfg.arch == "gpt2":
            continue   # GPT-2 reads the tied head from wte; Llama-family models get a (sharded) copy
        w = fn(tensors)
        kind = lay[name][2]
        out[name] = shard_tensor(name, w.float(), kind, cfg, tp).to(device=device, dtype=dtype).contiguous()
    return out
