"""Per-layer specifications for hybrid stacks (recurrent, windowed and
latent attention layers mixed in one model) and the config.json readers of
the Gurapel, Pokulorn, Munerax and Lokedra designs.

A homogeneous model is described by the flat ModelConfig fields; a hybrid
one additionally carries `layer_specs`, one LayerSpec per layer, each
naming its token mixer(s) and its feed-forward. The mixer specs are plain
frozen dataclasses so another design can reuse any of them with its own
constants.
"""
from __future__ import annotations

import dataclasses
from dataclasses import dataclass
from typing import Optional, Tuple

import torch

from ..engine.config import ModelConfig


@dataclass(frozen=True)
class DeltaRuleSpec:
    """Gated delta-rule linear attention (matrix-valued recurrent state
    per head, short causal convolutions on q/k/v)."""
    heads: int            # value heads (one state matrix each)
    qk_heads: int         # query/key heads, shared by heads // qk_heads
    dim: int              # per-head query/key size
    vdim: int             # per-head value size
    conv_taps: int        # short-convolution length
    qk_eps: float = 1e-6  # inside the unit-norm root


@dataclass(frozen=True)
class WindowAttnSpec:
    """Softmax attention over a sliding window of the paged cache with
    per-head qk RMS norm, tanh score capping and a logarithmic distance
    penalty instead of a rotation."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    window: int           # a query sees itself and window-1 earlier keys
    scale: float
    softcap: float        # 0 = no capping
    distance_bias: bool = True
    qk_norm: bool = True


@dataclass(frozen=True)
class RGLRUSpec:
    """Recurrent block around a real-gated linear recurrent unit: a GELU
    gate branch beside a conv + diagonal-recurrence branch."""
    width: int
    blocks: int           # block-diagonal gate matrices
    conv_taps: int
    decay_scale: float = 8.0


@dataclass(frozen=True)
class MoESpec:
    """Routed feed-forward. `routing`: "topk_softmax" (top-k of the
    logits, softmax over the chosen ones) or "sigmoid_groups" (sigmoid
    scores; experts form `groups` equal groups of neighbours, a group
    scores the sum of its two best experts, only the `keep_groups` best
    groups are eligible; weights are the chosen scores times `scale`, not
    renormalised) or "softmax_bias" (softmax over all experts; the choice
    adds a per-expert correction to the scores, the weights are the chosen
    scores without it, not renormalised). `act`: "silu_glu" (gated
    experts), "relu2" (ungated, squared relu) or "clamped_glu"
    (g = min(gate, limit), u = clamp(up, ±limit), g·sigmoid(1.702 g)·
    (u + 1)). `shared_ff` > 0 adds an always-on expert of that width and
    the same form."""
    experts: int
    top: int
    ff: int
    routing: str = "topk_softmax"
    act: str = "silu_glu"
    groups: int = 1
    keep_groups: int = 1
    scale: float = 1.0
    shared_ff: int = 0
    limit: float = 0.0            # clamp of "clamped_glu"


@dataclass(frozen=True)
class RotarySpec:
    """Rotation of the first `dims` dimensions of each q/k head, dimension
    i paired with i + dims/2, or with `interleaved` dimension 2i with
    2i + 1. With `factor` > 0 the frequencies are
    interpolated by parts (wavelengths beyond `original`/`slow` turns are
    divided by `factor`, those below `original`/`fast` turns kept, a
    linear ramp between) and cos/sin are scaled by 0.1·ln(factor) + 1."""
    dims: int
    base: float
    factor: float = 0.0          # 0 = plain rotation
    original: float = 0.0
    fast: float = 32.0
    slow: float = 1.0
    interleaved: bool = False

    def frequencies(self):
        """(per-pair angular frequencies as a float64 list, magnitude)."""
        import math
        half = self.dims // 2
        freq = [self.base ** (-2.0 * i / self.dims) for i in range(half)]
        if self.factor <= 0:
            return freq, 1.0

        def turn_dim(turns: float) -> float:
            return self.dims * math.log(
                self.original / (2 * math.pi * turns)) / (2 * math.log(self.base))
        lo = max(math.floor(turn_dim(self.fast)), 0)
        hi = min(math.ceil(turn_dim(self.slow)), self.dims - 1)
        out = []
        for i, f in enumerate(freq):
            ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
            out.append(f / self.factor * ramp + f * (1.0 - ramp))
        return out, 0.1 * math.log(self.factor) + 1.0


@dataclass(frozen=True)
class RotaryAttnSpec:
    """Softmax attention over the paged cache with short causal
    convolutions on q/k/v, per-head qk RMS norm (shared weight), partial
    rotation, and a choice of: sliding window that also keeps the first
    tokens, a per-head sink term in the softmax denominator, blending of
    the values with those of the stack's first value-mixing layer, and a
    sigmoid output gate."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    conv_taps: int = 0            # 0 = no convolution
    rot: Optional[RotarySpec] = None
    window: int = 0               # 0 = every earlier key
    keep_first: int = 0           # with a window: keys j < keep_first stay
    sink: bool = False
    mix_values: bool = False
    gate: bool = False
    qk_norm: bool = True
    # a chunked mask instead of a window: query i sees j <= i only with
    # floor(i / chunk) == floor(j / chunk) on absolute sequence positions
    chunk: int = 0
    bias: bool = False            # biases on the q/k/v and output projections
    tied_values: bool = False     # no value projection: v = k as cached
    unit_sink: bool = False       # a sink of score 0: denominator 1 + sum


@dataclass(frozen=True)
class MLSTMSpec:
    """Matrix-memory recurrence with an exponential input gate and a
    sigmoid forget gate kept in the log domain under a running maximum;
    gate pre-activations are soft-capped by cap·tanh(·/cap)."""
    heads: int
    dim: int
    vdim: int
    gate_cap: float
    denom_floor: float = 1e-6     # added to the read-out's denominator


@dataclass(frozen=True)
class SSDSpec:
    """Selective state space with a scalar decay per head and step
    (state [N, vdim] per head), B/C shared by heads of a group, short
    convolution on x/B/C, silu(z) gate and a grouped RMS norm."""
    heads: int
    vdim: int
    state: int
    groups: int
    norm_groups: int
    conv_taps: int


@dataclass(frozen=True)
class DenseFFSpec:
    """Gated feed-forward: g = min(gate, limit), u = clamp(up, ±limit),
    y = g·sigmoid(alpha·g)·(u + 1)."""
    ff: int
    limit: float
    alpha: float = 1.702


@dataclass(frozen=True)
class LatentAttnSpec:
    """Softmax attention whose keys and values are up-projections of one
    low-rank latent per token: the cache holds the RMS-normed latent
    (`kv_rank`) and one rotated key part (`rot_dim`) shared by all heads.
    Per head, `dim` unrotated plus `rot_dim` rotated query/key dimensions
    and `vdim` value dimensions. Options: a per-head sink in the softmax
    denominator, a per-head sigmoid output gate, and `kv_from` = index of
    an earlier layer whose cached latent and rotated key this layer
    reads instead of projecting its own. `q_rank` > 0: queries are an
    up-projection of an RMS-normed latent of that size."""
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    scale: float
    rot: Optional[RotarySpec] = None
    sink: bool = False
    gate: bool = False
    kv_from: Optional[int] = None
    q_rank: int = 0


@dataclass(frozen=True)
class DiagDeltaSpec:
    """Generalized delta rule: per head a [dim, dim] state with a decay per
    key channel, removal along the unit key at a per-channel rate, and a
    rank-one write: S <- diag(w) S - (a*u)(u^T S) + k v^T, u = k/|k|,
    w = exp(-decay_rate * sigmoid(low-rank(h) + w0)), a = sigmoid(W_a h +
    b). Read-out S^T r, unit RMS per head, a weight over all heads, a
    sigmoid output gate."""
    heads: int
    dim: int
    decay_rate: float = 0.6065306597126334     # exp(-1/2)
    k_eps: float = 1e-6                         # inside the unit-key root


@dataclass(frozen=True)
class HGRN2Spec:
    """Gated linear attention whose forget gate also sets what is written:
    per head S <- diag(f) S + (1 - f) v^T, o = S^T q, q = silu(W_q h),
    f = lower + (1 - lower) sigmoid(W_f h + b) per head and channel;
    o is RMS-normed over vdim with a weight shared by the heads."""
    heads: int
    dim: int
    vdim: int


@dataclass(frozen=True)
class LoopSpec:
    """A repeated block: layers [start, stop) execute `times` passes back
    to back on shared weights, each pass keeping caches and states of its
    own; from the second pass on, a pass opens with x += the embedding
    output."""
    start: int
    stop: int
    times: int


@dataclass(frozen=True)
class GeluGLUSpec:
    """Gated feed-forward down(gelu_tanh(gate)·up)."""
    ff: int


@dataclass(frozen=True)
class BigramSpec:
    """Hashed bigram embedding added to the token embedding: row
    (previous·mul_prev + token·mul_cur) mod buckets of a [buckets + 1,
    width] table; a sequence's first token takes the last row."""
    buckets: int
    mul_prev: int
    mul_cur: int


@dataclass(frozen=True)
class LayerSpec:
    # Munerax — "latent_attention": LatentAttnSpec, with `glu` (dense) or
    # `moe` as its feed-forward.
    # Gurapel — "delta": one DeltaRuleSpec; "parallel": WindowAttnSpec
    # beside RGLRUSpec, outputs normed and averaged.
    # Pokulorn — "mlstm": MLSTMSpec; "attention": RotaryAttnSpec;
    # "parallel": RotaryAttnSpec beside SSDSpec, outputs summed with the
    # weights `branch_scales`.
    # Lokedra — "general_delta": DiagDeltaSpec; "latent_attention":
    # LatentAttnSpec; "parallel": RotaryAttnSpec beside HGRN2Spec, summed
    # with `branch_scales`; feed-forward `moe` or none.
    kind: str
    delta: Optional[DeltaRuleSpec] = None
    attn: Optional[WindowAttnSpec] = None
    rglru: Optional[RGLRUSpec] = None
    moe: Optional[MoESpec] = None     # None = no feed-forward
    mlstm: Optional[MLSTMSpec] = None
    rattn: Optional[RotaryAttnSpec] = None
    ssd: Optional[SSDSpec] = None
    dense: Optional[DenseFFSpec] = None
    branch_scales: Tuple[float, float] = (1.0, 1.0)
    latent: Optional[LatentAttnSpec] = None
    glu: Optional[GeluGLUSpec] = None
    ddelta: Optional[DiagDeltaSpec] = None
    hgrn: Optional[HGRN2Spec] = None


def _moe_spec(m) -> Optional[MoESpec]:
    if m is None:
        return None
    if m.get("kind", "moe") != "moe":
        raise ValueError(f"unsupported feed-forward kind {m.get('kind')!r}")
    return MoESpec(experts=int(m["router"]["experts"]),
                   top=int(m["router"]["top"]), ff=int(m["expert"]["ff"]))


def _layer_spec(entry: dict) -> LayerSpec:
    kind = entry["type"]
    mx = entry["mixer"]
    moe = _moe_spec(entry.get("mlp"))
    if kind == "delta":
        return LayerSpec(kind, delta=DeltaRuleSpec(
            heads=int(mx["heads"]), qk_heads=int(mx["kv_heads"]),
            dim=int(mx["dim"]), vdim=int(mx["vdim"]),
            conv_taps=int(mx["conv"])), moe=moe)
    if kind == "parallel":
        lf, rt = mx["left"], mx["right"]
        return LayerSpec(
            kind,
            attn=WindowAttnSpec(
                heads=int(lf["heads"]), kv_heads=int(lf["kv_heads"]),
                dim=int(lf["dim"]), vdim=int(lf["vdim"]),
                window=int(lf["mask"]["size"]), scale=float(lf["scale"]),
                softcap=float(lf.get("softcap", 0.0))),
            rglru=RGLRUSpec(width=int(rt["width"]), blocks=int(rt["blocks"]),
                            conv_taps=int(rt["conv"])),
            moe=moe)
    raise ValueError(f"unknown layer type {kind!r}")


def is_gurapel_config(cfg: dict) -> bool:
    return cfg.get("architecture") == "Gurapel"


def gurapel_model_config(cfg: dict, name: str = "",
                         dtype: torch.dtype = torch.bfloat16) -> ModelConfig:
    """config.json of a Gurapel checkpoint → ModelConfig. Every size and
    per-model constant comes from the file; the flat llama-style fields
    are filled with the first attention/MoE layer's numbers only so that
    generic consumers (memory estimator, metrics) see sensible values."""
    specs: Tuple[LayerSpec, ...] = tuple(_layer_spec(e) for e in cfg["layers"])
    width = int(cfg["width"])
    attn = next((s.attn for s in specs if s.attn is not None), None)
    moe = next((s.moe for s in specs if s.moe is not None), None)
    return ModelConfig(
        name=name or "gurapel", arch="gurapel", layer_specs=specs,
        hidden_size=width, num_layers=len(specs),
        num_heads=attn.heads if attn else 1,
        num_kv_heads=attn.kv_heads if attn else 1,
        head_dim=attn.dim if attn else width,
        intermediate_size=moe.ff if moe else width,
        vocab_size=int(cfg["vocab"]),
        max_position=int(cfg["max_positions"]),
        rms_eps=float(cfg["norm"]["eps"]),
        embed_scale=float(cfg["embedding"]["scale"]),
        rms_norm_offset=True, learned_positions=True, residual_fp32=True,
        num_experts=moe.experts if moe else 0,
        num_experts_per_tok=moe.top if moe else 0,
        moe_intermediate_size=moe.ff if moe else 0,
        moe_routing="topk_softmax", dtype=dtype)


def layer_moe_config(cfg: ModelConfig, moe: MoESpec) -> ModelConfig:
    """A per-layer view of cfg for MoEMLP (layers may differ in expert
    count, top-k and width). For bf16 the expert width is rounded up to
    the 64-column tile of the fused grouped-GEMM kernels (which also keeps
    the vectorised activation kernel's alignment on the per-expert path);
    the loader zero-fills the extra gate/up rows and down columns, which
    contribute exactly nothing (silu(0)·0 = 0)."""
    ff = moe.ff
    if cfg.dtype == torch.bfloat16:
        ff = (ff + 63) // 64 * 64
    return dataclasses.replace(
        cfg, num_experts=moe.experts, num_experts_per_tok=moe.top,
        moe_intermediate_size=ff, moe_routing=moe.routing,
        moe_act="silu" if moe.act == "silu_glu" else moe.act,
        moe_bias=False, n_shared_experts=0,
        moe_shared_intermediate_size=moe.shared_ff, n_group=moe.groups,
        topk_group=moe.keep_groups, moe_norm_topk=False,
        routed_scaling_factor=moe.scale, moe_router_fp32=True,
        moe_act_limit=moe.limit)


# ---- Pokulorn ---------------------------------------------------------------

def _rotary_spec(r) -> Optional[RotarySpec]:
    if not r:
        return None
    sc = r.get("scaling") or {}
    return RotarySpec(
        dims=int(r["dims"]), base=float(r["base"]),
        factor=float(sc.get("factor", 0.0)),
        original=float(sc.get("original", 0.0)),
        fast=float(sc.get("fast", 32.0)), slow=float(sc.get("slow", 1.0)))


def _rotary_attn_spec(mx: dict, sink: bool, gate: bool) -> RotaryAttnSpec:
    mask = mx.get("mask") or {}
    return RotaryAttnSpec(
        heads=int(mx["heads"]), kv_heads=int(mx["kv_heads"]),
        dim=int(mx["dim"]), vdim=int(mx["vdim"]), scale=float(mx["scale"]),
        conv_taps=int(mx.get("conv", 0)), rot=_rotary_spec(mx.get("rot")),
        window=int(mask.get("size", 0)),
        keep_first=int(mask.get("keep_first", 0)),
        sink=sink, mix_values=bool(mx.get("v_mix", False)), gate=gate)


def _dense_spec(m) -> Optional[DenseFFSpec]:
    if m is None:
        return None
    if m.get("kind", "dense") != "dense":
        raise ValueError(f"unsupported feed-forward kind {m.get('kind')!r}")
    return DenseFFSpec(ff=int(m["ff"]), limit=float(m["limit"]))


def _pokulorn_layer(entry: dict) -> LayerSpec:
    kind, mx = entry["type"], entry["mixer"]
    dense = _dense_spec(entry.get("mlp"))
    if kind == "mlstm":
        return LayerSpec(kind, mlstm=MLSTMSpec(
            heads=int(mx["heads"]), dim=int(mx["dim"]), vdim=int(mx["vdim"]),
            gate_cap=float(mx["gate_cap"])), dense=dense)
    if kind == "attention":
        return LayerSpec(kind, rattn=_rotary_attn_spec(mx, sink=True,
                                                       gate=False),
                         dense=dense)
    if kind == "parallel":
        rt = mx["right"]
        return LayerSpec(
            kind, rattn=_rotary_attn_spec(mx["left"], sink=False, gate=True),
            ssd=SSDSpec(heads=int(rt["heads"]), vdim=int(rt["vdim"]),
                        state=int(rt["state"]), groups=int(rt["groups"]),
                        norm_groups=int(rt["norm_groups"]),
                        conv_taps=int(rt["conv"])),
            branch_scales=(float(mx["left_scale"]), float(mx["right_scale"])),
            dense=dense)
    raise ValueError(f"unknown layer type {kind!r}")


def is_pokulorn_config(cfg: dict) -> bool:
    return cfg.get("architecture") == "Pokulorn"


# the design has no position table, so its length limit is the engine's
POKULORN_DEFAULT_MAX_POSITION = 1 << 17


def pokulorn_model_config(cfg: dict, name: str = "",
                          dtype: torch.dtype = torch.bfloat16) -> ModelConfig:
    """config.json of a Pokulorn checkpoint → ModelConfig (every size, the
    layer order and every per-model constant come from the file)."""
    specs: Tuple[LayerSpec, ...] = tuple(
        _pokulorn_layer(e) for e in cfg["layers"])
    width = int(cfg["width"])
    attn = next((s.rattn for s in specs if s.rattn is not None), None)
    ff = next((s.dense for s in specs if s.dense is not None), None)
    return ModelConfig(
        name=name or "pokulorn", arch="pokulorn", layer_specs=specs,
        hidden_size=width, num_layers=len(specs),
        num_heads=attn.heads if attn else 1,
        num_kv_heads=attn.kv_heads if attn else 1,
        head_dim=attn.dim if attn else width,
        intermediate_size=ff.ff if ff else width,
        vocab_size=int(cfg["vocab"]),
        max_position=int(cfg.get("max_positions",
                                 POKULORN_DEFAULT_MAX_POSITION)),
        rms_eps=float(cfg["norm"]["eps"]),
        residual_fp32=True, dtype=dtype)


# ---- Munerax ------------------------------------------------------------------

def _munerax_ff(m):
    """config `mlp` entry → (GeluGLUSpec | None, MoESpec | None)."""
    if m is None:
        return None, None
    kind = m.get("kind", "dense")
    if kind == "dense":
        return GeluGLUSpec(ff=int(m["ff"])), None
    if kind != "moe":
        raise ValueError(f"unsupported feed-forward kind {kind!r}")
    r = m["router"]
    g = r.get("groups") or {}
    shared = m.get("shared") or {}
    return None, MoESpec(
        experts=int(r["experts"]), top=int(r["top"]),
        ff=int(m["expert"]["ff"]), routing="sigmoid_groups", act="relu2",
        groups=int(g.get("count", 1)), keep_groups=int(g.get("keep", 1)),
        scale=float(r.get("scale", 1.0)), shared_ff=int(shared.get("ff", 0)))


def _munerax_layer(entry: dict, index: int, layers: list) -> LayerSpec:
    kind, mx = entry["type"], entry["mixer"]
    if kind != "latent_attention":
        raise ValueError(f"unknown layer type {kind!r}")
    rot = mx["rot"]
    if int(rot["dims"]) != int(mx["rot_dim"]):
        raise ValueError("the rotated key part is rotated whole")
    src = mx.get("kv_from")
    if src is not None:
        src = int(src)
        other = layers[src]["mixer"] if 0 <= src < index else None
        if other is None or other.get("kv_from") is not None:
            raise ValueError(f"layer {index}: kv_from must name an earlier "
                             "layer with a down-projection of its own")
        for k in ("kv_rank", "rot_dim"):
            if int(other[k]) != int(mx[k]):
                raise ValueError(f"layer {index}: {k} differs from layer "
                                 f"{src}, whose cache it reads")
        if float(other["rot"]["base"]) != float(rot["base"]):
            raise ValueError(f"layer {index}: rotation differs from layer "
                             f"{src}, whose rotated keys it reads")
    glu, moe = _munerax_ff(entry.get("mlp"))
    return LayerSpec(kind, latent=LatentAttnSpec(
        heads=int(mx["heads"]), dim=int(mx["dim"]),
        rot_dim=int(mx["rot_dim"]), vdim=int(mx["vdim"]),
        kv_rank=int(mx["kv_rank"]), scale=float(mx["scale"]),
        rot=RotarySpec(dims=int(rot["dims"]), base=float(rot["base"])),
        sink=True, gate=True, kv_from=src), glu=glu, moe=moe)


def is_munerax_config(cfg: dict) -> bool:
    return cfg.get("architecture") == "Munerax"


def munerax_model_config(cfg: dict, name: str = "",
                         dtype: torch.dtype = torch.bfloat16) -> ModelConfig:
    """config.json of a Munerax checkpoint → ModelConfig (every size, the
    layer order and every per-model constant come from the file). The
    design has no position table, so its length limit is the engine's."""
    layers = cfg["layers"]
    specs: Tuple[LayerSpec, ...] = tuple(
        _munerax_layer(e, i, layers) for i, e in enumerate(layers))
    width = int(cfg["width"])
    att = specs[0].latent
    moe = next((s.moe for s in specs if s.moe is not None), None)
    glu = next((s.glu for s in specs if s.glu is not None), None)
    emb = cfg["embedding"]
    bg = emb.get("bigram")
    return ModelConfig(
        name=name or "munerax", arch="munerax", layer_specs=specs,
        hidden_size=width, num_layers=len(specs),
        num_heads=att.heads, num_kv_heads=1,
        head_dim=att.dim + att.rot_dim,
        intermediate_size=glu.ff if glu else (moe.ff if moe else width),
        vocab_size=int(cfg["vocab"]),
        max_position=int(cfg.get("max_positions",
                                 POKULORN_DEFAULT_MAX_POSITION)),
        rms_eps=float(cfg["norm"]["eps"]),
        embed_scale=float(emb.get("scale", 1.0)),
        bigram=BigramSpec(buckets=int(bg["buckets"]),
                          mul_prev=int(bg["mul_prev"]),
                          mul_cur=int(bg["mul_cur"])) if bg else None,
        tie_word_embeddings=True, residual_fp32=True,
        num_experts=moe.experts if moe else 0,
        num_experts_per_tok=moe.top if moe else 0,
        moe_intermediate_size=moe.ff if moe else 0, dtype=dtype)


# ---- Lokedra ------------------------------------------------------------------

def _lokedra_ff(m) -> Optional[MoESpec]:
    if m is None:
        return None
    if m.get("kind", "moe") != "moe":
        raise ValueError(f"unsupported feed-forward kind {m.get('kind')!r}")
    return MoESpec(
        experts=int(m["router"]["experts"]), top=int(m["router"]["top"]),
        ff=int(m["expert"]["ff"]), routing="softmax_bias",
        act="clamped_glu", limit=float(m["expert"]["limit"]))


def _lokedra_layer(entry: dict) -> LayerSpec:
    kind, mx = entry["type"], entry["mixer"]
    moe = _lokedra_ff(entry.get("mlp"))
    if kind == "general_delta":
        return LayerSpec(kind, ddelta=DiagDeltaSpec(
            heads=int(mx["heads"]), dim=int(mx["dim"])), moe=moe)
    if kind == "latent_attention":
        rot = _rotary_spec(mx["rot"])
        if rot.dims != int(mx["rot_dim"]):
            raise ValueError("the rotated key part is rotated whole")
        return LayerSpec(kind, latent=LatentAttnSpec(
            heads=int(mx["heads"]), dim=int(mx["dim"]),
            rot_dim=int(mx["rot_dim"]), vdim=int(mx["vdim"]),
            kv_rank=int(mx["kv_rank"]), scale=float(mx["scale"]),
            rot=dataclasses.replace(rot, interleaved=True),
            q_rank=int(mx["q_rank"])), moe=moe)
    if kind == "parallel":
        lf, rt = mx["left"], mx["right"]
        if int(lf.get("vdim", lf["dim"])) != int(lf["dim"]):
            raise ValueError("keys double as values: vdim must equal dim")
        mask = lf.get("mask") or {}
        return LayerSpec(
            kind,
            rattn=RotaryAttnSpec(
                heads=int(lf["heads"]), kv_heads=int(lf["kv_heads"]),
                dim=int(lf["dim"]), vdim=int(lf["dim"]),
                scale=float(lf["scale"]), conv_taps=int(lf.get("conv", 0)),
                chunk=int(mask.get("size", 0)), qk_norm=False, bias=True,
                tied_values=True, unit_sink=True),
            hgrn=HGRN2Spec(heads=int(rt["heads"]), dim=int(rt["dim"]),
                           vdim=int(rt["vdim"])),
            branch_scales=(float(mx["left_scale"]), float(mx["right_scale"])),
            moe=moe)
    raise ValueError(f"unknown layer type {kind!r}")


def is_lokedra_config(cfg: dict) -> bool:
    return cfg.get("architecture") == "Lokedra"


def lokedra_model_config(cfg: dict, name: str = "",
                         dtype: torch.dtype = torch.bfloat16) -> ModelConfig:
    """config.json of a Lokedra checkpoint → ModelConfig (every size, the
    layer order, the loop and every per-model constant come from the
    file). The design has no position table, so its length limit is the
    engine's."""
    specs: Tuple[LayerSpec, ...] = tuple(
        _lokedra_layer(e) for e in cfg["layers"])
    n = len(specs)
    lp = cfg.get("loop")
    loop = None
    if lp:
        loop = LoopSpec(start=int(lp["start"]), stop=int(lp["stop"]),
                        times=int(lp["times"]))
        if not (0 <= loop.start <= loop.stop <= n and loop.times >= 1):
            raise ValueError(f"loop {lp} does not fit {n} layers")
    width = int(cfg["width"])
    att = next((s.latent for s in specs if s.latent is not None), None)
    moe = next((s.moe for s in specs if s.moe is not None), None)
    return ModelConfig(
        name=name or "lokedra", arch="lokedra", layer_specs=specs,
        layer_loop=loop, hidden_size=width, num_layers=n,
        num_heads=att.heads if att else 1, num_kv_heads=1,
        head_dim=att.dim + att.rot_dim if att else width,
        intermediate_size=moe.ff if moe else width,
        vocab_size=int(cfg["vocab"]),
        max_position=int(cfg.get("max_positions",
                                 POKULORN_DEFAULT_MAX_POSITION)),
        rms_eps=float(cfg["norm"]["eps"]),
        embed_scale=float(cfg["embedding"].get("scale", 1.0)),
        rms_norm_offset=True, tie_word_embeddings=True, residual_fp32=True,
        num_experts=moe.experts if moe else 0,
        num_experts_per_tok=moe.top if moe else 0,
        moe_intermediate_size=moe.ff if moe else 0, dtype=dtype)
