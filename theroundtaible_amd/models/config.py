"""Model architecture presets (SURVEY §2.4.1 shape table)."""
from __future__ import annotations

import json
import math
import os
from dataclasses import dataclass, replace
from typing import Callable, Dict, Optional, Tuple


@dataclass(frozen=True)
class LatentAttentionSpec:
    """Sizes and constants of one latent-attention mixer (low-rank queries; keys and values
    from one cached latent plus a rotated key part shared by all heads; a softmax sink per head)."""
    heads: int
    dim: int              # unrotated query / key dims per head
    rot_dim: int          # rotated query / key dims per head (the key part is shared by the heads)
    vdim: int             # value dims per head
    kv_rank: int          # width of the cached latent
    q_rank: int           # width of the query latent
    rot_base: float
    rot_dims: int         # leading entries of the rotated part that take the rotation
    scale: float

    @property
    def cache_row(self) -> int:
        """Cached numbers per token: the latent and the rotated key part."""
        return self.kv_rank + self.rot_dim


@dataclass(frozen=True)
class RotarySpec:
    """Rotary positions on the leading ``dims`` entries of a head, entry 2i paired with 2i + 1:
    angle = position * base^(-2i / dims), frequencies optionally rescaled (``scaling`` as in
    ``ModelConfig.rope_scaling``, e.g. ("llama3", factor, low, high, original))."""
    base: float
    dims: int
    scaling: Optional[tuple] = None
    halves: bool = False      # entry i pairs with i + dims / 2 instead of 2i with 2i + 1


@dataclass(frozen=True)
class GroupedAttentionSpec:
    """Causal attention with ``heads`` query heads over ``kv_heads`` key / value heads (query head
    h reads key / value head h // (heads / kv_heads)); queries and keys are divided by their root
    mean square per head (after the rotation, if any). ``sink`` is a constant added to the softmax
    denominator as exp(0) * sink: a key of score 0 without a value (0 = ordinary softmax).
    ``head_temp``: every head multiplies its scores by a learned number (tensor ``temp``).
    ``value_from_key``: there is no value projection, the values are the projected keys as they
    are before the norm.
    ``window`` > 0: position i sees only j with 0 <= i - j < window. ``slope_base`` > 0: head a
    takes slope_a * (i - j) off its scores, slope_a = 2^(-slope_base * (a + 1) / heads).
    ``qk_weight``: the query / key norms multiply by a learned weight per channel (tensors
    ``q.norm`` / ``k.norm``, shared by the heads). ``q_temp`` = (coef, every): the queries of
    position p are multiplied by 1 + coef * ln(floor((p + 1) / every) + 1). ``value_norm``: every
    value head is divided by its root mean square before it is cached. ``out_gate``: the
    concatenated heads are multiplied by sigmoid(W_g h) ahead of the output projection.
    ``softcap`` > 0: scores become softcap * tanh(score / softcap). ``wide_norm``: instead of the
    per-head unit RMS, the whole query projection (and the whole key projection) is divided by
    its root mean square over all heads at once and multiplied by a weight per channel (tensors
    ``q.norm`` / ``k.norm`` of the projection's size), BEFORE the rotation. ``bias``: the query and
    key projections add a bias (tensors ``q.b`` / ``k.b``). ``value_rot``: the value of position j
    is turned by j over all its entries before it is cached (pair m by j * base^(-2m / vdim), the
    pairs laid out as the key rotation's), and each head's output at position i is turned back by i."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot: Optional[RotarySpec] = None
    sink: float = 0.0
    head_temp: bool = False
    value_from_key: bool = False
    window: int = 0
    slope_base: float = 0.0
    qk_weight: bool = False
    q_temp: Optional[Tuple[float, int]] = None
    value_norm: bool = False
    out_gate: bool = False
    softcap: float = 0.0
    wide_norm: bool = False
    bias: bool = False
    value_rot: Optional[RotarySpec] = None

    @property
    def group(self) -> int:
        return self.heads // self.kv_heads

    @property
    def cache_row(self) -> int:
        """Cached numbers per token: keys and values of every key / value head."""
        return self.kv_heads * (self.dim + self.vdim)


@dataclass(frozen=True)
class MinGRUSpec:
    """Gated recurrence whose gates read only the current token (minGRU), ``width`` channels:
    S_t = (1 - z_t) S_(t-1) + z_t c_t, output gated by silu of a third projection."""
    width: int


@dataclass(frozen=True)
class DecaySumSpec:
    """Linear attention with one constant decay per head (lightning attention): per head a
    ``dim`` x ``vdim`` fp32 state, S_t = decay S_(t-1) + k_t v_t^T, o_t = S_t^T q_t, with
    q, k, v = silu of their projections; the concatenated heads are RMS-normed together, weighted,
    and gated by sigmoid of a fourth projection."""
    heads: int
    dim: int
    vdim: int
    decay: Tuple[float, ...]

    @property
    def state_size(self) -> int:
        return self.heads * self.dim * self.vdim


@dataclass(frozen=True)
class RemovalSpec:
    """Generalized delta rule: per head a ``dim`` x ``dim`` fp32 state with a per-token,
    per-channel decay w (a low-rank path through tanh, then exp(-e^(-1/2) sigmoid(.))) and a
    per-channel removal rate a = sigmoid(W_a h + b): with u the unit-length key,
    S_t = diag(w_t) S_(t-1) - (a_t * u_t)(u_t^T S_(t-1)) + k_t v_t^T, o_t = S_t^T r_t; each head
    is divided by its root mean square, weighted, and gated by sigmoid of a projection."""
    heads: int
    dim: int
    decay_rank: int = 0

    @property
    def vdim(self) -> int:
        return self.dim

    @property
    def state_size(self) -> int:
        return self.heads * self.dim * self.dim


@dataclass(frozen=True)
class DeltaSpec:
    """Gated delta rule: ``heads`` value heads of size ``vdim`` over ``kv_heads`` query / key heads
    of size ``dim``; q, k, v pass a causal convolution of ``conv`` taps per channel and silu, q and
    k are made unit vectors (q also times dim^(-1/2)); one decay g and one step size beta per head
    and token: S <- g S; S <- S + k (beta (v - S^T k))^T; o = S^T q. Each head is divided by its
    root mean square, weighted (one weight vector shared by the heads), gated by silu of a projection."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int

    @property
    def state_size(self) -> int:
        return self.heads * self.dim * self.vdim

    @property
    def conv_channels(self) -> int:
        return 2 * self.kv_heads * self.dim + self.heads * self.vdim


@dataclass(frozen=True)
class ParallelSpec:
    """Two mixers reading the same input: attention (``left``) beside a recurrence (``right``: a
    minGRU, whose layer adds half the sum of the two RMS-normed outputs; or a matrix-state
    recurrence, whose layer adds ``left_scale`` * left + ``right_scale`` * right)."""
    left: GroupedAttentionSpec
    right: object
    left_scale: float = 0.5
    right_scale: float = 0.5


@dataclass(frozen=True)
class WKVSpec:
    """Linear-attention time mixing with a per-token, per-channel decay (RWKV style): ``heads``
    heads whose keys and values are ``dim`` wide, a ``dim`` x ``dim`` fp32 state per head, and a
    low-rank path of width ``decay_rank`` from the shifted input to the decay's logarithm."""
    heads: int
    dim: int
    decay_rank: int

    @property
    def width(self) -> int:
        return self.heads * self.dim

    @property
    def state_size(self) -> int:
        """fp32 numbers of the recurrent state per sequence."""
        return self.heads * self.dim * self.dim


@dataclass(frozen=True)
class MoESpec:
    """Mixture of feed-forward experts: ``experts`` experts of width ``ff``, each token runs the
    ``top`` with the largest router logits, weighted by the softmax over those logits alone (which
    equals the softmax over all experts renormalised over the chosen ones). ``act`` "silu_glu":
    W_down (silu(W_gate h) * W_up h); "relu2": W_down relu(W_up h)^2. ``shared_ff`` > 0: one more
    expert of that width (tensors ``shared.*``) runs for every token with weight 1."""
    experts: int
    top: int
    ff: int
    act: str = "silu_glu"
    shared_ff: int = 0


@dataclass(frozen=True)
class LayerSpec:
    """One decoder layer of a per-layer-configured model: its mixer, its feed-forward (``ff`` 0 =
    none) and ``source``, the layer whose tensors it uses (itself unless its weights are shared).
    ``ff_limit``: the clamp of a limited gated feed-forward. ``moe``: the experts of a
    feed-forward of kind "moe" (``ff`` is then one expert's width). ``opens_pass``: this run is the
    first of pass number ``opens_pass`` of a looped span (None: it opens none)."""
    mixer_type: str
    mixer: object
    ff: int
    ff_kind: str
    source: int
    ff_limit: float = 0.0
    moe: Optional[MoESpec] = None
    opens_pass: Optional[int] = None


@dataclass(frozen=True)
class ModelConfig:
    name: str
    arch: str                 # "llama" (Llama-3 / Mistral / Qwen2) | "gpt2"
    n_layers: int
    hidden: int
    n_heads: int
    n_kv_heads: int
    head_dim: int
    ffn: int
    vocab: int
    max_pos: int
    rope_theta: float = 500000.0
    norm_eps: float = 1e-5
    tie_embeddings: bool = False
    qkv_bias: bool = False    # Qwen2 / Qwen2.5: biased q/k/v projections (added before RoPE)
    # checkpoint RoPE scaling (ops/reference.py rope_inv_freq): ("linear", f) | ("llama3", f, low,
    # high, original_max_pos) | ("yarn", f, original_max_pos, beta_fast, beta_slow, attention_factor)
    rope_scaling: Optional[tuple] = None
    # per-layer-configured architectures ("mupulorn"): the layers, the taps of the causal input
    # convolution ahead of every sublayer, and the output scaling / soft cap of the logits
    layers: Optional[Tuple[LayerSpec, ...]] = None
    canon_taps: int = 0
    logit_scale: float = 1.0
    logit_softcap: float = 0.0
    embed_scale: float = 1.0      # the embedding row is multiplied by it ("goganex")
    norm_groups: int = 1          # RMS norms of the residual stream work on this many equal parts ("retuvik")
    loop_passes: int = 0          # passes of the looped span that add the embedding / a step vector ("retuvik")

    @property
    def q_size(self) -> int:
        return self.n_heads * self.head_dim

    @property
    def kv_size(self) -> int:
        return self.n_kv_heads * self.head_dim

    @property
    def group(self) -> int:
        return self.n_heads // self.n_kv_heads

    def n_params(self) -> int:
        h, f, v, L = self.hidden, self.ffn, self.vocab, self.n_layers
        if self.arch in ("goganex", "retuvik", "ledinex"):
            from .weights import layout_for
            n = 0
            for shape, _, _ in layout_for(self).values():
                k = 1
                for d in shape:
                    k *= d if d >= 0 else 32
                n += k
            return n
        if self.layers is not None:
            n = 2 * v * h + 1
            for i, ls in enumerate(self.layers):
                if ls.source != i:
                    continue
                m = ls.mixer
                n += h * (m.q_rank + m.cache_row + m.heads * m.vdim) + m.q_rank + m.kv_rank + m.heads
                n += m.q_rank * m.heads * (m.dim + m.rot_dim) + m.kv_rank * m.heads * (m.dim + m.vdim)
                n += m.heads * m.vdim * h + 2 + self.canon_taps * h
                if ls.ff:
                    n += 2 * h * ls.ff + 6 + self.canon_taps * h
            return n
        if self.arch == "gpt2":
            per = 4 * h * h + 2 * h * f + 9 * h + f
            return L * per + v * h + self.max_pos * h + 2 * h
        per = h * (self.q_size + 2 * self.kv_size) + self.q_size * h + 3 * h * f + 2 * h
        if self.qkv_bias:
            per += self.q_size + 2 * self.kv_size
        emb = v * h * (1 if self.tie_embeddings else 2)
        return L * per + emb + h

    def kv_bytes_per_token(self, dtype_bytes: int = 2) -> int:
        if self.layers is not None:
            return sum(attention_of(ls).cache_row for ls in self.layers if attention_of(ls) is not None) * dtype_bytes
        return 2 * self.n_layers * self.n_kv_heads * self.head_dim * dtype_bytes


PRESETS: Dict[str, ModelConfig] = {
    "llama3-8b": ModelConfig("llama3-8b", "llama", 32, 4096, 32, 8, 128, 14336, 128256, 131072, 500000.0, 1e-5),
    # Llama 3.1 / 3.2: the same blocks with rope_type "llama3" scaling (3.2: tied embeddings;
    # 3.2-3B has GQA group 3)
    "llama3.1-8b": ModelConfig("llama3.1-8b", "llama", 32, 4096, 32, 8, 128, 14336, 128256, 131072, 500000.0, 1e-5,
                               False, False, ("llama3", 8.0, 1.0, 4.0, 8192)),
    "llama3.2-1b": ModelConfig("llama3.2-1b", "llama", 16, 2048, 32, 8, 64, 8192, 128256, 131072, 500000.0, 1e-5,
                               True, False, ("llama3", 32.0, 1.0, 4.0, 8192)),
    "llama3.2-3b": ModelConfig("llama3.2-3b", "llama", 28, 3072, 24, 8, 128, 8192, 128256, 131072, 500000.0, 1e-5,
                               True, False, ("llama3", 32.0, 1.0, 4.0, 8192)),
    "llama3-70b": ModelConfig("llama3-70b", "llama", 80, 8192, 64, 8, 128, 28672, 128256, 131072, 500000.0, 1e-5),
    "mistral-7b": ModelConfig("mistral-7b", "llama", 32, 4096, 32, 8, 128, 14336, 32000, 32768, 1000000.0, 1e-5),
    # Qwen2.5 (HF model_type "qwen2"): the Llama block with q/k/v biases; 7B: GQA 28 / 4 heads,
    # 0.5B: head_dim 64, tied embeddings (the family most local coding setups run)
    "qwen2.5-7b": ModelConfig("qwen2.5-7b", "llama", 28, 3584, 28, 4, 128, 18944, 152064, 32768, 1000000.0, 1e-6,
                              False, True),
    "qwen2.5-14b": ModelConfig("qwen2.5-14b", "llama", 48, 5120, 40, 8, 128, 13824, 152064, 32768, 1000000.0, 1e-6,
                               False, True),
    "qwen2.5-32b": ModelConfig("qwen2.5-32b", "llama", 64, 5120, 40, 8, 128, 27648, 152064, 32768, 1000000.0, 1e-6,
                               False, True),
    "qwen2.5-72b": ModelConfig("qwen2.5-72b", "llama", 80, 8192, 64, 8, 128, 29568, 152064, 32768, 1000000.0, 1e-6,
                               False, True),
    "qwen2.5-0.5b": ModelConfig("qwen2.5-0.5b", "llama", 24, 896, 14, 2, 64, 4864, 151936, 32768, 1000000.0, 1e-6,
                                True, True),
    # GPT-2-small: random init allows n_positions beyond 1024 (SURVEY §7.3 hard part 3).
    "gpt2-small": ModelConfig("gpt2-small", "gpt2", 12, 768, 12, 12, 64, 3072, 50257, 8192, 0.0, 1e-5, True),
    # test-sized models (CPU unit tests, GPU smoke)
    "tiny-llama": ModelConfig("tiny-llama", "llama", 2, 256, 4, 2, 64, 512, 32000, 4096, 10000.0, 1e-5),
    "tiny-llama-128": ModelConfig("tiny-llama-128", "llama", 2, 512, 4, 1, 128, 1024, 32000, 8192, 500000.0, 1e-5),
    "tiny-qwen": ModelConfig("tiny-qwen", "llama", 2, 256, 4, 2, 64, 512, 32000, 4096, 1000000.0, 1e-6, True, True),
    "tiny-qwen-128": ModelConfig("tiny-qwen-128", "llama", 2, 512, 4, 1, 128, 1024, 32000, 8192, 1000000.0, 1e-6,
                                 False, True),
    "tiny-gpt2": ModelConfig("tiny-gpt2", "gpt2", 2, 128, 2, 2, 64, 512, 32000, 2048, 0.0, 1e-5, True),
}


def parse_mupulorn(d: dict, name: str = "mupulorn") -> ModelConfig:
    """``config.json`` of a Mupulorn checkpoint -> :class:`ModelConfig`. Every size and every
    per-model constant comes from the file; a layer with ``weights_of`` runs another layer's tensors."""
    raw = d["layers"]
    specs = []
    for i, e in enumerate(raw):
        if e["type"] != "latent_attention":
            raise ValueError(f"{name}: layer {i}: unknown mixer type '{e['type']}'")
        src, seen = i, set()
        while "weights_of" in raw[src] and raw[src]["weights_of"] is not None:
            if src in seen:
                raise ValueError(f"{name}: layer {i}: weights_of forms a cycle")
            seen.add(src)
            src = int(raw[src]["weights_of"])
        mx = e["mixer"]
        rot = mx["rot"]
        m = LatentAttentionSpec(int(mx["heads"]), int(mx["dim"]), int(mx["rot_dim"]), int(mx["vdim"]),
                                int(mx["kv_rank"]), int(mx["q_rank"]), float(rot["base"]), int(rot["dims"]),
                                float(mx["scale"]))
        if m.rot_dims > m.rot_dim or m.rot_dims % 2:
            raise ValueError(f"{name}: layer {i}: rot.dims {m.rot_dims} does not fit rot_dim {m.rot_dim}")
        mlp = raw[src].get("mlp") if e.get("mlp", "absent") == "absent" else e.get("mlp")
        if mlp is not None and mlp.get("kind", "dense") != "dense":
            raise ValueError(f"{name}: layer {i}: unknown feed-forward kind '{mlp['kind']}'")
        specs.append(LayerSpec("latent_attention", m, int(mlp["ff"]) if mlp is not None else 0, "dense", src))
    top = max(specs, key=lambda s: s.mixer.heads).mixer
    return ModelConfig(name, "mupulorn", len(specs), int(d["width"]), top.heads, 1, top.dim + top.rot_dim,
                       max(s.ff for s in specs), int(d["vocab"]), int(d.get("max_pos", 1 << 17)),
                       specs[0].mixer.rot_base, float(d["norm"]["eps"]), layers=tuple(specs),
                       canon_taps=int(d["canon"]["taps"]), logit_scale=float(d["logit_scale"]),
                       logit_softcap=float(d["logit_softcap"]))


def attention_of(ls: LayerSpec):
    """The attention part of a layer's mixer (the left half of a parallel mixer; None for a
    mixer without attention)."""
    if isinstance(ls.mixer, (WKVSpec, DeltaSpec)):
        return None
    return ls.mixer.left if isinstance(ls.mixer, ParallelSpec) else ls.mixer


def _grouped_attention(mx: dict, where: str, **kind) -> GroupedAttentionSpec:
    rot = None
    if mx.get("rot") is not None:
        r = mx["rot"]
        sc = r.get("scaling")
        rot = RotarySpec(float(r["base"]), int(r["dims"]),
                         ("llama3", float(sc["factor"]), float(sc["low"]), float(sc["high"]), float(sc["original"]))
                         if sc is not None else None)
    a = GroupedAttentionSpec(int(mx["heads"]), int(mx["kv_heads"]), int(mx["dim"]), int(mx["vdim"]), float(mx["scale"]),
                             rot, **kind)
    if a.heads % a.kv_heads:
        raise ValueError(f"{where}: {a.heads} query heads do not divide over {a.kv_heads} key/value heads")
    if rot is not None and (rot.dims > a.dim or rot.dims % 2):
        raise ValueError(f"{where}: rot.dims {rot.dims} does not fit dim {a.dim}")
    if a.value_from_key and a.vdim != a.dim:
        raise ValueError(f"{where}: values are the keys, so vdim {a.vdim} must equal dim {a.dim}")
    return a


def parse_goganex(d: dict, name: str = "goganex") -> ModelConfig:
    """``config.json`` of a Goganex checkpoint -> :class:`ModelConfig`. ``layers`` of the result
    are the layer RUNS in execution order: the checkpoint layers ``loop.start .. loop.stop - 1``
    are run ``loop.times`` times in a row with the same tensors (``LayerSpec.source``), every run
    with a cache and state of its own."""
    raw = d["layers"]
    order = list(range(len(raw)))
    lp = d.get("loop")
    if lp is not None:
        a, b, n = int(lp["start"]), int(lp["stop"]), int(lp["times"])
        if not (0 <= a <= b <= len(raw)) or n < 1:
            raise ValueError(f"{name}: loop {lp} does not fit {len(raw)} layers")
        order = order[:a] + order[a:b] * n + order[b:]
    specs = []
    for i in order:
        e, where = raw[i], f"{name}: layer {i}"
        if e["type"] == "attention":
            mixer = _grouped_attention(e["mixer"], where, sink=1.0, head_temp=True)
        elif e["type"] == "parallel":
            mixer = ParallelSpec(_grouped_attention(e["mixer"]["left"], where, value_from_key=True),
                                 MinGRUSpec(int(e["mixer"]["right"]["width"])))
        else:
            raise ValueError(f"{where}: unknown mixer type '{e['type']}'")
        mlp = e.get("mlp")
        if mlp is not None and mlp.get("kind", "dense") != "dense":
            raise ValueError(f"{where}: unknown feed-forward kind '{mlp['kind']}'")
        specs.append(LayerSpec(e["type"], mixer, int(mlp["ff"]) if mlp is not None else 0, "dense", i,
                               float(mlp["limit"]) if mlp is not None else 0.0))
    top = max((attention_of(s) for s in specs), key=lambda m: m.heads)
    rots = [attention_of(s).rot for s in specs if attention_of(s).rot is not None]
    return ModelConfig(name, "goganex", len(specs), int(d["width"]), top.heads, top.kv_heads, top.dim,
                       max(s.ff for s in specs), int(d["vocab"]), int(d.get("max_pos", 1 << 17)),
                       rots[0].base if rots else 0.0, float(d["norm"]["eps"]), layers=tuple(specs),
                       embed_scale=float(d.get("embedding", {}).get("scale", 1.0)))


def goganex_config(name: str, n_layers: int, width: int, heads: int, kv_heads: int, dim: int, ff: int, vocab: int,
                   parallel_every: int = 4, gru_width: int = 0, loop: Optional[Tuple[int, int, int]] = None,
                   rot_base: float = 500000.0, limit: float = 7.0, max_pos: int = 1 << 17) -> ModelConfig:
    """A Goganex stack from a few sizes (benchmarks and presets): attention layers with every
    ``parallel_every``-th layer a parallel attention + minGRU layer (0: none)."""
    att = {"type": "attention",
           "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": 1.5 * dim ** -0.5,
                     "rot": {"base": rot_base, "dims": dim, "scaling": None}},
           "mlp": {"kind": "dense", "ff": ff, "limit": limit} if ff else None}
    par = {"type": "parallel",
           "mixer": {"left": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": dim ** -0.5},
                     "right": {"width": gru_width or width}},
           "mlp": att["mlp"]}
    layers = [par if parallel_every and (i + 1) % parallel_every == 0 else att for i in range(n_layers)]
    d = {"architecture": "Goganex", "embedding": {"scale": 1.0}, "layers": layers, "norm": {"eps": 1e-5},
         "vocab": vocab, "width": width, "max_pos": max_pos}
    if loop is not None:
        d["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return parse_goganex(d, name)



def parse_retuvik(d: dict, name: str = "retuvik") -> ModelConfig:
    """``config.json`` of a Retuvik checkpoint -> :class:`ModelConfig`. ``layers`` of the result are
    the layer RUNS in execution order: checkpoint layers ``loop.start .. loop.stop - 1`` run
    ``loop.times`` times in a row with the same tensors, every run with a cache and state of its
    own; the first run of pass t is marked ``opens_pass = t`` (the model adds the embedding output
    again from the second pass on, and row t of ``loop.step`` in every pass). A key the file does
    not have switches its mechanism off (no window, no query factor, no loop). The width of a wkv
    mixer's low-rank decay path is a tensor shape, not a config key: ``mixer.decay_rank`` is read
    only by random initialisation."""
    raw = d["layers"]
    runs = [(i, None) for i in range(len(raw))]
    lp = d.get("loop")
    passes = 0
    if lp is not None:
        a, b, passes = int(lp["start"]), int(lp["stop"]), int(lp["times"])
        if not (0 <= a <= b <= len(raw)) or passes < 1:
            raise ValueError(f"{name}: loop {lp} does not fit {len(raw)} layers")
        if a == b:
            passes = 0
        body = [[(i, t if i == a else None) for i in range(a, b)] for t in range(passes)]
        runs = runs[:a] + sum(body, []) + runs[b:]
    specs = []
    for i, opens in runs:
        e, where = raw[i], f"{name}: layer {i}"
        mx = e["mixer"]
        if e["type"] == "wkv":
            mixer = WKVSpec(int(mx["heads"]), int(mx["dim"]), int(mx.get("decay_rank", 0)))
        elif e["type"] == "attention":
            qt, mask = mx.get("q_temp"), mx.get("mask")
            mixer = _grouped_attention(mx, where, window=int(mask["size"]) if mask is not None else 0, slope_base=8.0,
                                       qk_weight=True, value_norm=True, out_gate=True,
                                       q_temp=(float(qt["coef"]), int(qt["every"])) if qt is not None else None)
            if mixer.window < 0 or (mixer.q_temp is not None and mixer.q_temp[1] < 1):
                raise ValueError(f"{where}: mask.size / q_temp.every out of range")
        else:
            raise ValueError(f"{where}: unknown mixer type '{e['type']}'")
        mlp = e.get("mlp")
        if mlp is None:
            specs.append(LayerSpec(e["type"], mixer, 0, "dense", i, opens_pass=opens))
        elif mlp.get("kind", "dense") == "dense":
            specs.append(LayerSpec(e["type"], mixer, int(mlp["ff"]), "dense", i, opens_pass=opens))
        elif mlp["kind"] == "moe":
            moe = MoESpec(int(mlp["router"]["experts"]), int(mlp["router"]["top"]), int(mlp["expert"]["ff"]))
            if not 1 <= moe.top <= moe.experts:
                raise ValueError(f"{where}: top {moe.top} of {moe.experts} experts")
            specs.append(LayerSpec(e["type"], mixer, moe.ff, "moe", i, moe=moe, opens_pass=opens))
        else:
            raise ValueError(f"{where}: unknown feed-forward kind '{mlp['kind']}'")
    width, groups = int(d["width"]), int(d["norm"].get("groups", 1))
    if groups < 1 or width % groups:
        raise ValueError(f"{name}: width {width} does not split into {groups} norm groups")
    atts = [s.mixer for s in specs if isinstance(s.mixer, GroupedAttentionSpec)]
    top = max(atts, key=lambda m: m.heads) if atts else None
    any_mixer = specs[0].mixer
    return ModelConfig(name, "retuvik", len(specs), width, top.heads if top else any_mixer.heads,
                       top.kv_heads if top else any_mixer.heads, top.dim if top else any_mixer.dim,
                       max([s.ff for s in specs] + [0]), int(d["vocab"]), int(d.get("max_pos", 1 << 17)), 0.0,
                       float(d["norm"]["eps"]), layers=tuple(specs),
                       embed_scale=float(d.get("embedding", {}).get("scale", 1.0)), norm_groups=groups,
                       loop_passes=passes)


def retuvik_config(name: str, n_layers: int, width: int, heads: int, kv_heads: int, dim: int, ff: int, vocab: int,
                   attention_every: int = 3, wkv_dim: int = 64, decay_rank: int = 64, window: int = 1024,
                   moe_every: int = 0, experts: int = 8, top: int = 2, expert_ff: int = 0,
                   loop: Optional[Tuple[int, int, int]] = None, groups: int = 2, max_pos: int = 1 << 17) -> ModelConfig:
    """A Retuvik stack from a few sizes (benchmarks and presets): wkv layers with every
    ``attention_every``-th layer a windowed attention layer (0: none); every ``moe_every``-th
    feed-forward a mixture of experts (0: all dense)."""
    wkv = {"type": "wkv", "mixer": {"heads": width // wkv_dim, "dim": wkv_dim, "decay_rank": decay_rank}}
    att = {"type": "attention",
           "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": dim ** -0.5,
                     "mask": {"size": window}, "q_temp": {"coef": 0.1, "every": 1024}}}
    dense = {"kind": "dense", "ff": ff} if ff else None
    moe = {"kind": "moe", "expert": {"ff": expert_ff or ff // top}, "router": {"experts": experts, "top": top}}
    layers = []
    for i in range(n_layers):
        e = dict(att if attention_every and (i + 1) % attention_every == 0 else wkv)
        e["mlp"] = moe if moe_every and (i + 1) % moe_every == 0 else dense
        layers.append(e)
    d = {"architecture": "Retuvik", "embedding": {"scale": 1.0}, "layers": layers, "norm": {"eps": 1e-5, "groups": groups},
         "vocab": vocab, "width": width, "max_pos": max_pos}
    if loop is not None:
        d["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return parse_retuvik(d, name)


def _ledinex_attention(mx: dict, kind: str, where: str) -> GroupedAttentionSpec:
    r = mx["rot"]
    sc = r.get("scaling")
    scaling = None
    if sc is not None and "original" in sc:       # blended frequencies and enlarged cos / sin (YaRN)
        f = float(sc["factor"])
        scaling = ("yarn", f, float(sc["original"]), float(sc["fast"]), float(sc["slow"]), 0.1 * math.log(f) + 1.0)
    elif sc is not None:
        scaling = ("linear", float(sc["factor"]))
    rot = RotarySpec(float(r["base"]), int(r["dims"]), scaling, halves=True)
    two = kind == "parallel_2"
    mask = mx.get("mask")
    vdim = int(mx["vdim"])
    a = GroupedAttentionSpec(int(mx["heads"]), int(mx["kv_heads"]), int(mx["dim"]), vdim, float(mx["scale"]), rot,
                             value_from_key=two, window=int(mask["size"]) if mask is not None else 0,
                             softcap=float(mx.get("softcap") or 0.0), wide_norm=True, bias=two,
                             value_rot=None if two else RotarySpec(rot.base, vdim, None, halves=True))
    if a.heads % a.kv_heads:
        raise ValueError(f"{where}: {a.heads} query heads do not divide over {a.kv_heads} key/value heads")
    if rot.dims > a.dim or rot.dims % 2 or (a.value_rot is not None and vdim % 2):
        raise ValueError(f"{where}: rot.dims {rot.dims} / vdim {vdim} do not fit the rotation")
    if a.value_from_key and a.vdim != a.dim:
        raise ValueError(f"{where}: values are the keys, so vdim {a.vdim} must equal dim {a.dim}")
    if a.window < 0:
        raise ValueError(f"{where}: mask.size out of range")
    return a


def parse_ledinex(d: dict, name: str = "ledinex") -> ModelConfig:
    """``config.json`` of a Ledinex checkpoint -> :class:`ModelConfig`. Every layer is a mixer of
    type "parallel" (attention with turned values and soft-capped scores beside a constant-decay
    linear attention), "parallel_2" (windowed attention whose values are its keys beside a
    generalized delta rule) or "delta" (a gated delta rule), and a mixture of squared-ReLU experts
    with a shared expert (or no feed-forward). A key the file does not have switches its mechanism
    off (no window, no soft cap, no frequency scaling, no shared expert)."""
    specs = []
    for i, e in enumerate(d["layers"]):
        where, kind, mx = f"{name}: layer {i}", e["type"], e["mixer"]
        if kind == "delta":
            mixer = DeltaSpec(int(mx["heads"]), int(mx["kv_heads"]), int(mx["dim"]), int(mx["vdim"]), int(mx["conv"]))
            if mixer.heads % mixer.kv_heads or mixer.conv < 1:
                raise ValueError(f"{where}: heads {mixer.heads} / kv_heads {mixer.kv_heads} / conv {mixer.conv}")
        elif kind in ("parallel", "parallel_2"):
            left, rx = _ledinex_attention(mx["left"], kind, where), mx["right"]
            if kind == "parallel":
                dec = rx["decay"]
                dec = [dec] * int(rx["heads"]) if isinstance(dec, (int, float)) else dec     # one number: every head's
                right = DecaySumSpec(int(rx["heads"]), int(rx["dim"]), int(rx.get("vdim") or rx["dim"]),
                                     tuple(float(v) for v in dec))
                if len(right.decay) != right.heads:
                    raise ValueError(f"{where}: {len(right.decay)} decays for {right.heads} heads")
            else:
                right = RemovalSpec(int(rx["heads"]), int(rx["dim"]), int(rx.get("decay_rank", 0)))
            mixer = ParallelSpec(left, right, float(mx["left_scale"]), float(mx["right_scale"]))
        else:
            raise ValueError(f"{where}: unknown mixer type '{kind}'")
        mlp = e.get("mlp")
        if mlp is None:
            specs.append(LayerSpec(kind, mixer, 0, "moe", i))
        elif mlp.get("kind") == "moe":
            sh = mlp.get("shared")
            moe = MoESpec(int(mlp["router"]["experts"]), int(mlp["router"]["top"]), int(mlp["expert"]["ff"]), "relu2",
                          int(sh["ff"]) if sh is not None else 0)
            if not 1 <= moe.top <= moe.experts:
                raise ValueError(f"{where}: top {moe.top} of {moe.experts} experts")
            specs.append(LayerSpec(kind, mixer, moe.ff, "moe", i, moe=moe))
        else:
            raise ValueError(f"{where}: unknown feed-forward kind '{mlp.get('kind')}'")
    atts = [attention_of(s) for s in specs if attention_of(s) is not None]
    top = max(atts, key=lambda m: m.heads) if atts else None
    any_mixer = specs[0].mixer
    taps = int(d["canon"]["taps"])
    if not 1 <= taps <= 16:
        raise ValueError(f"{name}: canon.taps {taps} out of range")
    return ModelConfig(name, "ledinex", len(specs), int(d["width"]), top.heads if top else any_mixer.heads,
                       top.kv_heads if top else any_mixer.kv_heads, top.dim if top else any_mixer.dim,
                       max([s.ff for s in specs] + [0]), int(d["vocab"]), int(d.get("max_pos", 1 << 17)), 0.0,
                       float(d["norm"]["eps"]), tie_embeddings=True, layers=tuple(specs), canon_taps=taps,
                       logit_scale=float(d.get("logit_scale", 1.0)),
                       embed_scale=float(d.get("embedding", {}).get("scale", 1.0)))


def ledinex_config(name: str, n_layers: int, width: int, heads: int, kv_heads: int, dim: int, ff: int, vocab: int,
                   pattern: Tuple[str, ...] = ("parallel_2", "delta", "parallel"), rec_heads: int = 0, rec_dim: int = 64,
                   window: int = 1024, experts: int = 8, top: int = 2, expert_ff: int = 0, shared_ff: int = 0,
                   taps: int = 4, conv: int = 4, decay_rank: int = 64, max_pos: int = 1 << 17) -> ModelConfig:
    """A Ledinex stack from a few sizes (benchmarks and presets): the mixer types of ``pattern``
    in turn; every feed-forward a mixture of ``experts`` squared-ReLU experts (``top`` per token,
    together ``ff`` wide unless ``expert_ff`` is given) plus a shared expert."""
    A = rec_heads or width // rec_dim
    eff = expert_ff or max(64, ff // (top + 1) // 64 * 64)
    mlp = {"kind": "moe", "expert": {"ff": eff}, "router": {"experts": experts, "top": top},
           "shared": {"ff": shared_ff or eff}} if ff else None
    left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": dim ** -0.5}
    kinds = {
        "parallel": {"left": dict(left, softcap=30.0, rot={"base": 500000.0, "dims": dim, "scaling": {"factor": 2.0}}),
                     "left_scale": 0.7, "right_scale": 0.7,
                     "right": {"heads": A, "dim": rec_dim, "vdim": rec_dim,
                               "decay": [math.exp(-2.0 ** (-1 - 5.0 * a / max(1, A - 1))) for a in range(A)]}},
        "parallel_2": {"left": dict(left, mask={"size": window},
                                    rot={"base": 100000.0, "dims": dim // 2,
                                         "scaling": {"factor": 4.0, "original": 4096, "fast": 32.0, "slow": 1.0}}),
                       "left_scale": 0.7, "right_scale": 0.7,
                       "right": {"heads": A, "dim": rec_dim, "decay_rank": decay_rank}},
        "delta": {"heads": A, "kv_heads": max(1, A // 2), "dim": rec_dim, "vdim": rec_dim, "conv": conv},
    }
    layers = [{"type": pattern[i % len(pattern)], "mixer": kinds[pattern[i % len(pattern)]], "mlp": mlp}
              for i in range(n_layers)]
    return parse_ledinex({"architecture": "Ledinex", "canon": {"taps": taps}, "embedding": {"scale": 1.0},
                          "layers": layers, "logit_scale": 1.0, "norm": {"eps": 1e-5}, "vocab": vocab, "width": width,
                          "max_pos": max_pos}, name)


def mupulorn_config(name: str, n_layers: int, width: int, heads: int, dim: int, rot_dim: int, vdim: int,
                    kv_rank: int, q_rank: int, ff: int, vocab: int, taps: int = 4, shared_every: int = 0,
                    rot_base: float = 10000.0, max_pos: int = 1 << 17) -> ModelConfig:
    """A uniform Mupulorn stack from a few sizes (benchmarks and presets). ``shared_every`` n > 0:
    layers n*k+1 .. n*k+n-1 run layer n*k's weights."""
    layer = {"type": "latent_attention",
             "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank,
                       "q_rank": q_rank, "rot": {"base": rot_base, "dims": rot_dim},
                       "scale": (dim + rot_dim) ** -0.5},
             "mlp": {"kind": "dense", "ff": ff} if ff else None}
    layers = []
    for i in range(n_layers):
        e = dict(layer)
        if shared_every > 0 and i % shared_every:
            e["weights_of"] = i - i % shared_every
        layers.append(e)
    return parse_mupulorn({"architecture": "Mupulorn", "canon": {"taps": taps}, "layers": layers,
                           "logit_scale": 1.0, "logit_softcap": 30.0, "norm": {"eps": 1e-5}, "vocab": vocab,
                           "width": width, "max_pos": max_pos}, name)


# config.json "architecture" -> parser (checkpoint directories name their own model class)
ARCHITECTURES: Dict[str, Callable[[dict, str], ModelConfig]] = {"Mupulorn": parse_mupulorn, "Goganex": parse_goganex,
                                                                "Retuvik": parse_retuvik, "Ledinex": parse_ledinex}

PRESETS.update({
    # Mupulorn (latent attention + input convolutions + PolyNorm feed-forward), random-init sizes:
    # a test-sized stack and three whose layers have the shapes of 1B / 3B / 8B-class models
    "tiny-mupulorn": mupulorn_config("tiny-mupulorn", 3, 128, 4, 32, 16, 32, 64, 48, 256, 32000, taps=4,
                                     shared_every=2),
    # (the two-matrix feed-forward is 1.5x as wide as the gated three-matrix one of the Llama preset
    # of the same class, so a layer holds about the same weights)
    "mupulorn-1b": mupulorn_config("mupulorn-1b", 16, 2048, 16, 128, 64, 128, 512, 768, 12288, 128256),
    "mupulorn-3b": mupulorn_config("mupulorn-3b", 28, 3072, 24, 128, 64, 128, 256, 1024, 12288, 128256),
    "mupulorn-8b": mupulorn_config("mupulorn-8b", 32, 4096, 32, 128, 64, 128, 512, 1536, 21504, 128256),
})


PRESETS.update({
    # Goganex (grouped attention with a softmax sink, token shift, parallel attention + minGRU
    # layers, clamped gated feed-forward), random-init sizes: a test-sized stack with a looped
    # middle, and stacks whose layers have the shapes of 1B / 3B / 8B-class Llama models
    "tiny-goganex": goganex_config("tiny-goganex", 3, 128, 4, 2, 32, 256, 32000, parallel_every=3, gru_width=96,
                                   loop=(1, 3, 2)),
    "goganex-1b": goganex_config("goganex-1b", 16, 2048, 32, 8, 64, 8192, 128256),
    "goganex-3b": goganex_config("goganex-3b", 28, 3072, 24, 8, 128, 8192, 128256),
    "goganex-8b": goganex_config("goganex-8b", 32, 4096, 32, 8, 128, 14336, 128256),
})

PRESETS.update({
    # Retuvik (wkv time mixing with a per-token decay, windowed attention with a distance penalty,
    # xIELU and mixture-of-experts feed-forwards, grouped RMS norms), random-init sizes: a test-sized
    # stack with a looped middle, and stacks whose layers have the shapes of 0.5B (Qwen2.5) / 1B / 3B /
    # 8B-class Llama models (every third layer attention, every fourth feed-forward a mixture of 8 experts, 2 per token)
    "tiny-retuvik": retuvik_config("tiny-retuvik", 4, 128, 4, 2, 32, 256, 32000, attention_every=2, wkv_dim=32,
                                   decay_rank=16, window=24, moe_every=2, experts=6, top=2, expert_ff=64,
                                   loop=(1, 3, 2)),
    "retuvik-0.5b": retuvik_config("retuvik-0.5b", 24, 896, 14, 2, 64, 4864, 151936, moe_every=4),   # Qwen2.5-0.5B's sizes
    "retuvik-1b": retuvik_config("retuvik-1b", 16, 2048, 32, 8, 64, 8192, 128256, moe_every=4),
    "retuvik-3b": retuvik_config("retuvik-3b", 28, 3072, 24, 8, 128, 8192, 128256, moe_every=4),
    "retuvik-8b": retuvik_config("retuvik-8b", 32, 4096, 32, 8, 128, 14336, 128256, moe_every=4),
})

PRESETS.update({
    # Ledinex (input convolutions, post-norm sublayers, attention beside a matrix-state recurrence,
    # gated delta rule layers, squared-ReLU experts with a shared expert), random-init sizes: a
    # test-sized stack and stacks whose layers have the shapes of 0.5B (Qwen2.5) / 1B / 3B-class models
    "tiny-ledinex": ledinex_config("tiny-ledinex", 3, 128, 4, 2, 32, 192, 32000, rec_heads=2, rec_dim=32, window=24,
                                   experts=6, top=2, expert_ff=48, shared_ff=80, decay_rank=8),
    "ledinex-0.5b": ledinex_config("ledinex-0.5b", 24, 896, 14, 2, 64, 4864, 151936),      # Qwen2.5-0.5B's sizes
    "ledinex-1b": ledinex_config("ledinex-1b", 16, 2048, 32, 8, 64, 8192, 128256),
    "ledinex-3b": ledinex_config("ledinex-3b", 28, 3072, 24, 8, 128, 8192, 128256, rec_dim=128),
})


def config_from_dir(path: str) -> ModelConfig:
    """The model a checkpoint directory declares in its ``config.json`` (key ``architecture``)."""
    with open(os.path.join(path, "config.json")) as f:
        d = json.load(f)
    arch = d.get("architecture")
    if arch not in ARCHITECTURES:
        raise KeyError(f"{path}/config.json: unknown architecture {arch!r} (known: {', '.join(ARCHITECTURES)})")
    return ARCHITECTURES[arch](d, os.path.basename(os.path.normpath(path)) or arch.lower())


def get_config(name: str, **overrides) -> ModelConfig:
    if name not in PRESETS and os.path.isfile(os.path.join(name, "config.json")):
        cfg = config_from_dir(name)
        return replace(cfg, **overrides) if overrides else cfg
    if name not in PRESETS:
        raise KeyError(f"unknown model preset '{name}' (known: {', '.join(PRESETS)})")
    cfg = PRESETS[name]
    if isinstance(overrides.get("rope_scaling"), list):   # from a JSON config
        overrides = dict(overrides, rope_scaling=tuple(overrides["rope_scaling"]))
    return replace(cfg, **overrides) if overrides else cfg
