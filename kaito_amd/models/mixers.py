"""Token mixers for hybrid stacks: gated delta rule, real-gated linear
recurrence, matrix-memory (mLSTM) recurrence, scalar-decay selective
state space, softmax attention over the paged cache in two flavours
(distance penalty without rotation; convolutions + rotation + window
with kept first tokens or a chunked mask + sink, optionally with the
keys as values), latent attention (one low-rank latent per token in the
cache, optionally borrowed from an earlier layer, optionally with
low-rank queries), the generalized delta rule with per-channel decay, and
gated linear attention with a tied write gate (HGRN2). Each is a self-contained module parameterised by its spec
(models/hybrid_config.py), so a design picks and combines them freely.

All follow the same calling convention:

    mixer(x, positions, cache, meta) -> y            x, y: [T, hidden]

`cache` is the dict of this layer's device tensors handed out by
`alloc_cache()` (paged K/V for attention; per-sequence state slots for the
recurrent mixers) and `meta` the step's AttnMetadata with the chunk layout
(cu_seqlens / state_slots / seq_starts / token_seq / block_tables). A
step may mix prompt chunks of any length with single decode tokens; the
kernels behind `ops.*` make no distinction.

Precision: projections run in the activation dtype (bf16 or f32, f32
accumulation); everything that feeds a recurrence, every norm, the
attention scores and softmax are f32 inside the kernels; states are f32.
"""
from __future__ import annotations

from typing import Dict

import torch
import torch.nn as nn
import torch.nn.functional as F

from .. import ops
from .hybrid_config import (DeltaRuleSpec, DenseFFSpec, DiagDeltaSpec,
                            GeluGLUSpec, HGRN2Spec, LatentAttnSpec,
                            MLSTMSpec, RGLRUSpec, RotaryAttnSpec, SSDSpec,
                            WindowAttnSpec)


def _p(*shape, dtype):
    return nn.Parameter(torch.empty(*shape, dtype=dtype), requires_grad=False)


class GatedDeltaMixer(nn.Module):
    """Linear attention with the gated delta rule. Per head the state is a
    [dim, vdim] matrix S; per token: S ← g·S, then the prediction error
    β(v − Sᵀk) is written along k, then the output is Sᵀq (it already sees
    the token's own write). q, k, v pass a short causal convolution + silu;
    q and k are unit-normalised; the output is RMS-normed per head and
    gated by silu of a fourth projection."""

    def __init__(self, hidden: int, spec: DeltaRuleSpec, dtype, norm_eps: float):
        super().__init__()
        assert spec.heads % spec.qk_heads == 0
        self.spec, self.dtype, self.norm_eps = spec, dtype, norm_eps
        self.n_qk = spec.qk_heads * spec.dim
        self.n_v = spec.heads * spec.vdim
        self.conv_ch = 2 * self.n_qk + self.n_v
        # fused input projection, rows [q | k | v | gate | a | b]
        self.in_proj = _p(self.conv_ch + self.n_v + 2 * spec.heads, hidden,
                          dtype=dtype)
        self.conv_weight = _p(self.conv_ch, spec.conv_taps,
                              dtype=torch.float32)
        self.a_log = _p(spec.heads, dtype=torch.float32)
        self.dt_bias = _p(spec.heads, dtype=torch.float32)
        self.out_norm = _p(spec.vdim, dtype=torch.float32)
        self.o_proj = _p(hidden, self.n_v, dtype=dtype)

    def alloc_cache(self, num_blocks, block_size, num_slots, device) -> Dict:
        s = self.spec
        return {
            "conv": torch.zeros(num_slots, max(s.conv_taps - 1, 1),
                                self.conv_ch, dtype=self.dtype, device=device),
            "ssm": torch.zeros(num_slots, s.heads, s.dim, s.vdim,
                               dtype=torch.float32, device=device),
        }

    def cache_bytes(self, block_size: int):
        s = self.spec
        esz = torch.empty(0, dtype=self.dtype).element_size()
        return 0, (max(s.conv_taps - 1, 1) * self.conv_ch * esz
                   + s.heads * s.dim * s.vdim * 4)

    def forward(self, x, positions, cache, meta):
        s = self.spec
        T = x.size(0)
        p = F.linear(x, self.in_proj)
        qkv = ops.causal_conv_update(
            p[:, :self.conv_ch], self.conv_weight, None, cache["conv"],
            meta.cu_seqlens, meta.state_slots, meta.seq_starts,
            meta.token_seq, act=1)
        q = qkv[:, :self.n_qk].unflatten(-1, (s.qk_heads, s.dim))
        k = qkv[:, self.n_qk:2 * self.n_qk].unflatten(-1, (s.qk_heads, s.dim))
        v = qkv[:, 2 * self.n_qk:].unflatten(-1, (s.heads, s.vdim))
        c = self.conv_ch
        gate = p[:, c:c + self.n_v].unflatten(-1, (s.heads, s.vdim))
        a = p[:, c + self.n_v:c + self.n_v + s.heads]
        b = p[:, c + self.n_v + s.heads:]
        o = ops.gated_delta_rule(
            q, k, v, gate, a, b, self.a_log, self.dt_bias, self.out_norm,
            cache["ssm"], meta.cu_seqlens, meta.state_slots, meta.seq_starts,
            s.qk_eps, self.norm_eps)
        return F.linear(o.reshape(T, self.n_v), self.o_proj)


class RGLRUMixer(nn.Module):
    """Recurrent block around a real-gated linear recurrent unit: a
    GELU-activated gate branch y beside a branch u = conv(linear(x)) that
    drives the diagonal recurrence S ← a·S + sqrt(1−a²)·i·u with
    a = exp(−c·r·softplus(λ)); r and i are sigmoid gates computed from u by
    block-diagonal matrices. Output projection of S·y."""

    def __init__(self, hidden: int, spec: RGLRUSpec, dtype):
        super().__init__()
        assert spec.width % spec.blocks == 0
        self.spec, self.dtype = spec, dtype
        w, nb = spec.width, spec.blocks
        self.bw = w // nb
        # fused input projection, rows [y | x], with bias
        self.in_proj = _p(2 * w, hidden, dtype=dtype)
        self.in_bias = _p(2 * w, dtype=dtype)
        self.conv_weight = _p(w, spec.conv_taps, dtype=torch.float32)
        self.conv_bias = _p(w, dtype=torch.float32)
        # per block, rows [recurrence gate | input gate], stored
        # transposed ([in, out]) for the batched product; f32: the gates
        # enter the recurrence
        self.gate_w = _p(nb, self.bw, 2 * self.bw, dtype=torch.float32)
        self.gate_b = _p(nb, 1, 2 * self.bw, dtype=torch.float32)
        # c · softplus(λ), folded once at load
        self.decay_rate = _p(w, dtype=torch.float32)
        self.o_proj = _p(hidden, w, dtype=dtype)

    def alloc_cache(self, num_blocks, block_size, num_slots, device) -> Dict:
        s = self.spec
        return {
            "conv": torch.zeros(num_slots, max(s.conv_taps - 1, 1), s.width,
                                dtype=self.dtype, device=device),
            "lru": torch.zeros(num_slots, s.width, dtype=torch.float32,
                               device=device),
        }

    def cache_bytes(self, block_size: int):
        s = self.spec
        esz = torch.empty(0, dtype=self.dtype).element_size()
        return 0, max(s.conv_taps - 1, 1) * s.width * esz + s.width * 4

    def forward(self, x, positions, cache, meta):
        s = self.spec
        T, w = x.size(0), s.width
        p = F.linear(x, self.in_proj, self.in_bias)
        u = ops.causal_conv_update(
            p[:, w:], self.conv_weight, self.conv_bias, cache["conv"],
            meta.cu_seqlens, meta.state_slots, meta.seq_starts,
            meta.token_seq, act=0)
        ub = u.float().view(T, s.blocks, self.bw).transpose(0, 1)
        gates = torch.baddbmm(self.gate_b, ub, self.gate_w)   # [B, T, 2bw]
        o = ops.rglru_scan(u, gates, p[:, :w], self.decay_rate, cache["lru"],
                           meta.cu_seqlens, meta.state_slots, meta.seq_starts,
                           meta.token_seq)
        return F.linear(o, self.o_proj)


class BiasedWindowAttention(nn.Module):
    """Grouped-query softmax attention over the last `window` positions of
    the paged cache. No rotation: position enters through the causal
    window and a per-head penalty r1·ln(1 + r2·distance) subtracted from
    the (optionally tanh-capped) scores. q and k are RMS-normed per head
    with a weight shared by the heads; key and value sizes may differ."""

    def __init__(self, hidden: int, spec: WindowAttnSpec, dtype, norm_eps: float):
        super().__init__()
        assert spec.heads % spec.kv_heads == 0
        self.spec, self.dtype, self.norm_eps = spec, dtype, norm_eps
        s = spec
        self.q_size = s.heads * s.dim
        self.k_size = s.kv_heads * s.dim
        self.v_size = s.kv_heads * s.vdim
        self.qkv_proj = _p(self.q_size + self.k_size + self.v_size, hidden,
                           dtype=dtype)
        if s.qk_norm:
            self.q_norm = _p(s.dim, dtype=torch.float32)
            self.k_norm = _p(s.dim, dtype=torch.float32)
        else:
            self.q_norm = self.k_norm = None
        if s.distance_bias:
            self.r1 = _p(s.heads, dtype=torch.float32)
            self.r2 = _p(s.heads, dtype=torch.float32)
        else:
            self.r1 = self.r2 = None
        self.o_proj = _p(hidden, s.heads * s.vdim, dtype=dtype)

    def alloc_cache(self, num_blocks, block_size, num_slots, device) -> Dict:
        s = self.spec
        return {
            "k": torch.zeros(num_blocks, s.kv_heads, block_size, s.dim,
                             dtype=self.dtype, device=device),
            "v": torch.zeros(num_blocks, s.kv_heads, block_size, s.vdim,
                             dtype=self.dtype, device=device),
        }

    def cache_bytes(self, block_size: int):
        s = self.spec
        esz = torch.empty(0, dtype=self.dtype).element_size()
        return s.kv_heads * block_size * (s.dim + s.vdim) * esz, 0

    def forward(self, x, positions, cache, meta):
        s = self.spec
        T = x.size(0)
        qkv = F.linear(x, self.qkv_proj)
        q = qkv[:, :self.q_size].unflatten(-1, (s.heads, s.dim))
        k = qkv[:, self.q_size:self.q_size + self.k_size].unflatten(
            -1, (s.kv_heads, s.dim))
        v = qkv[:, self.q_size + self.k_size:].unflatten(
            -1, (s.kv_heads, s.vdim))
        qn = ops.qk_norm_cache_write(q, k, v, self.q_norm, self.k_norm,
                                     self.norm_eps, cache["k"], cache["v"],
                                     meta.slot_mapping)
        tiles = None
        if meta.tile_seq is not None:
            tiles = (meta.tile_seq, meta.tile_qbase, meta.cu_seqlens,
                     meta.seq_starts)
        o = ops.window_attention(qn, cache["k"], cache["v"],
                                 meta.block_tables, meta.token_seq, positions,
                                 s.scale, s.softcap, self.r1, self.r2,
                                 s.window, tiles=tiles)
        return F.linear(o.reshape(T, -1), self.o_proj)


class RotaryWindowAttention(nn.Module):
    """Grouped-query softmax attention over the paged cache. q, k and v
    pass a short causal convolution (its tail is per-sequence state), q
    and k a per-head RMS norm and a rotation of their first `rot.dims`
    dimensions; the mask is causal, optionally a sliding window that
    also keeps the first `keep_first` tokens; a per-head sink may join
    the softmax denominator (learned, or fixed at score 0); the mask may
    instead be chunked (a query sees the earlier keys of its own block of
    `chunk` positions); values may be blended with those of the stack's
    first value-mixing layer before they are cached, or be the keys
    themselves as cached (no value projection, one cache tensor); the
    projections may carry biases; the heads' outputs may be gated by
    sigmoid of a fourth projection."""

    def __init__(self, hidden: int, spec: RotaryAttnSpec, dtype,
                 norm_eps: float):
        super().__init__()
        assert spec.heads % spec.kv_heads == 0
        self.spec, self.dtype, self.norm_eps = spec, dtype, norm_eps
        s = spec
        self.q_size = s.heads * s.dim
        self.k_size = s.kv_heads * s.dim
        if s.tied_values:
            assert s.vdim == s.dim and not s.mix_values
        self.v_size = 0 if s.tied_values else s.kv_heads * s.vdim
        self.o_size = s.heads * s.vdim
        self.conv_ch = self.q_size + self.k_size + self.v_size
        # fused input projection, rows [q | k | v | gate]
        self.qkv_proj = _p(self.conv_ch + (self.o_size if s.gate else 0),
                           hidden, dtype=dtype)
        self.qkv_bias = _p(self.qkv_proj.shape[0], dtype=dtype) \
            if s.bias else None
        self.o_bias = _p(hidden, dtype=dtype) if s.bias else None
        self.conv_weight = _p(self.conv_ch, s.conv_taps, dtype=torch.float32) \
            if s.conv_taps > 0 else None
        if s.qk_norm:
            self.q_norm = _p(s.dim, dtype=torch.float32)
            self.k_norm = _p(s.dim, dtype=torch.float32)
        else:
            self.q_norm = self.k_norm = None
        if s.rot is not None:
            assert s.rot.dims % 2 == 0 and s.rot.dims <= s.dim
            freq, self.rot_mag = s.rot.frequencies()
            self.register_buffer("inv_freq", torch.tensor(
                freq, dtype=torch.float64).float(), persistent=False)
        else:
            self.inv_freq, self.rot_mag = None, 1.0
        if s.unit_sink:
            assert not s.sink
            self.register_buffer("sinks", torch.zeros(
                s.heads, dtype=torch.float32), persistent=False)
        else:
            self.sinks = _p(s.heads, dtype=torch.float32) if s.sink else None
        # blend weight of the first value-mixing layer's values; the first
        # such layer of a stack never reads it
        self.v_lambda = 0.0
        self.o_proj = _p(hidden, self.o_size, dtype=dtype)

    def alloc_cache(self, num_blocks, block_size, num_slots, device) -> Dict:
        s = self.spec
        out = {
            "k": torch.zeros(num_blocks, s.kv_heads, block_size, s.dim,
                             dtype=self.dtype, device=device),
        }
        if not s.tied_values:
            out["v"] = torch.zeros(num_blocks, s.kv_heads, block_size,
                                   s.vdim, dtype=self.dtype, device=device)
        if s.conv_taps > 0:
            out["conv"] = torch.zeros(num_slots, max(s.conv_taps - 1, 1),
                                      self.conv_ch, dtype=self.dtype,
                                      device=device)
        return out

    def cache_bytes(self, block_size: int):
        s = self.spec
        esz = torch.empty(0, dtype=self.dtype).element_size()
        slot = max(s.conv_taps - 1, 1) * self.conv_ch * esz \
            if s.conv_taps > 0 else 0
        vdim = 0 if s.tied_values else s.vdim
        return s.kv_heads * block_size * (s.dim + vdim) * esz, slot

    def forward(self, x, positions, cache, meta):
        s = self.spec
        T = x.size(0)
        p = F.linear(x, self.qkv_proj, self.qkv_bias)
        qkv = p[:, :self.conv_ch]
        if s.conv_taps > 0:
            qkv = ops.causal_conv_update(
                qkv, self.conv_weight, None, cache["conv"], meta.cu_seqlens,
                meta.state_slots, meta.seq_starts, meta.token_seq, act=0)
        q = qkv[:, :self.q_size].unflatten(-1, (s.heads, s.dim))
        k = qkv[:, self.q_size:self.q_size + self.k_size].unflatten(
            -1, (s.kv_heads, s.dim))
        v = k if s.tied_values else qkv[:, self.q_size + self.k_size:] \
            .unflatten(-1, (s.kv_heads, s.vdim))
        v_cache = cache["k"] if s.tied_values else cache["v"]
        v_first, lam = None, 0.0
        if s.mix_values:
            shared = meta.layer_shared
            if "v_first" in shared:
                v_first, lam = shared["v_first"], self.v_lambda
            else:
                shared["v_first"] = v
        qn = ops.qk_norm_cache_write(
            q, k, v, self.q_norm, self.k_norm, self.norm_eps, cache["k"],
            v_cache, meta.slot_mapping, positions=positions,
            inv_freq=self.inv_freq, rot_mag=self.rot_mag, v_first=v_first,
            v_lambda=lam)
        tiles = None
        if meta.tile_seq is not None:
            tiles = (meta.tile_seq, meta.tile_qbase, meta.cu_seqlens,
                     meta.seq_starts)
        o = ops.window_attention(qn, cache["k"], v_cache,
                                 meta.block_tables, meta.token_seq, positions,
                                 s.scale, window=s.window, tiles=tiles,
                                 keep_first=s.keep_first, sinks=self.sinks,
                                 chunk=s.chunk)
        o = o.reshape(T, self.o_size)
        if s.gate:
            o = ops.sigmoid_mul(o, p[:, self.conv_ch:])
        return F.linear(o, self.o_proj, self.o_bias)


class MLSTMMixer(nn.Module):
    """Matrix memory with exponential gating (mLSTM): per head a [dim,
    vdim] memory C, a normaliser n and a running maximum m of the log
    gates. The gate pre-activations come from an f32 projection (they
    enter the recurrence); q/k/v and the output gate from the
    activation-dtype projection."""

    def __init__(self, hidden: int, spec: MLSTMSpec, dtype, norm_eps: float):
        super().__init__()
        self.spec, self.dtype, self.norm_eps = spec, dtype, norm_eps
        s = spec
        self.n_qk = s.heads * s.dim
        self.n_v = s.heads * s.vdim
        # fused input projection, rows [q | k | v | output gate]
        self.in_proj = _p(2 * self.n_qk + 2 * self.n_v, hidden, dtype=dtype)
        # rows [input gate | forget gate]
        self.gate_proj = _p(2 * s.heads, hidden, dtype=torch.float32)
        self.gate_bias = _p(2 * s.heads, dtype=torch.float32)
        self.out_norm = _p(self.n_v, dtype=torch.float32)
        self.o_proj = _p(hidden, self.n_v, dtype=dtype)

    def alloc_cache(self, num_blocks, block_size, num_slots, device) -> Dict:
        s = self.spec
        f32 = dict(dtype=torch.float32, device=device)
        return {"c": torch.zeros(num_slots, s.heads, s.dim, s.vdim, **f32),
                "n": torch.zeros(num_slots, s.heads, s.dim, **f32),
                "m": torch.zeros(num_slots, s.heads, **f32)}

    def cache_bytes(self, block_size: int):
        s = self.spec
        return 0, s.heads * (s.dim * s.vdim + s.dim + 1) * 4

    def forward(self, x, positions, cache, meta):
        s = self.spec
        p = F.linear(x, self.in_proj)
        gates = F.linear(x.float(), self.gate_proj, self.gate_bias)
        nq, nv = self.n_qk, self.n_v
        q = p[:, :nq].unflatten(-1, (s.heads, s.dim))
        k = p[:, nq:2 * nq].unflatten(-1, (s.heads, s.dim))
        v = p[:, 2 * nq:2 * nq + nv].unflatten(-1, (s.heads, s.vdim))
        g = p[:, 2 * nq + nv:].unflatten(-1, (s.heads, s.vdim))
        o = ops.mlstm_scan(
            q, k, v, g, gates[:, :s.heads], gates[:, s.heads:], self.out_norm,
            cache["c"], cache["n"], cache["m"], meta.cu_seqlens,
            meta.state_slots, meta.seq_starts, s.gate_cap, s.dim ** -0.5,
            self.norm_eps, s.denom_floor)
        return F.linear(o, self.o_proj)


class SSDMixer(nn.Module):
    """Selective state space with one scalar decay per head and step
    (state-space duality form): x, B, C pass a short convolution with
    bias and silu; per head S <- exp(-exp(A)·d)·S + d·B xᵀ with step size
    d = softplus(dt + bias), y = Sᵀ C + D·x; y·silu(z) is RMS-normed in
    equal parts and projected out. The step-size pre-activation comes
    from an f32 projection."""

    def __init__(self, hidden: int, spec: SSDSpec, dtype, norm_eps: float):
        super().__init__()
        assert spec.heads % spec.groups == 0
        self.spec, self.dtype, self.norm_eps = spec, dtype, norm_eps
        s = spec
        self.inner = s.heads * s.vdim
        assert self.inner % s.norm_groups == 0
        self.n_bc = s.groups * s.state
        self.conv_ch = self.inner + 2 * self.n_bc
        # fused input projection, rows [z | x | B | C]
        self.in_proj = _p(self.inner + self.conv_ch, hidden, dtype=dtype)
        self.dt_proj = _p(s.heads, hidden, dtype=torch.float32)
        self.conv_weight = _p(self.conv_ch, s.conv_taps, dtype=torch.float32)
        self.conv_bias = _p(self.conv_ch, dtype=torch.float32)
        self.a_log = _p(s.heads, dtype=torch.float32)
        self.dt_bias = _p(s.heads, dtype=torch.float32)
        self.d_skip = _p(s.heads, dtype=torch.float32)
        self.out_norm = _p(self.inner, dtype=torch.float32)
        self.o_proj = _p(hidden, self.inner, dtype=dtype)

    def alloc_cache(self, num_blocks, block_size, num_slots, device) -> Dict:
        s = self.spec
        return {
            "conv": torch.zeros(num_slots, max(s.conv_taps - 1, 1),
                                self.conv_ch, dtype=self.dtype, device=device),
            "ssm": torch.zeros(num_slots, s.heads, s.state, s.vdim,
                               dtype=torch.float32, device=device),
        }

    def cache_bytes(self, block_size: int):
        s = self.spec
        esz = torch.empty(0, dtype=self.dtype).element_size()
        return 0, (max(s.conv_taps - 1, 1) * self.conv_ch * esz
                   + s.heads * s.state * s.vdim * 4)

    def forward(self, x, positions, cache, meta):
        s = self.spec
        p = F.linear(x, self.in_proj)
        dt = F.linear(x.float(), self.dt_proj)
        xbc = ops.causal_conv_update(
            p[:, self.inner:], self.conv_weight, self.conv_bias,
            cache["conv"], meta.cu_seqlens, meta.state_slots,
            meta.seq_starts, meta.token_seq, act=1)
        xs = xbc[:, :self.inner].unflatten(-1, (s.heads, s.vdim))
        B = xbc[:, self.inner:self.inner + self.n_bc].unflatten(
            -1, (s.groups, s.state))
        C = xbc[:, self.inner + self.n_bc:].unflatten(-1, (s.groups, s.state))
        y = ops.ssd_scan(xs, B, C, dt, p[:, :self.inner], self.a_log,
                         self.dt_bias, self.d_skip, self.out_norm,
                         cache["ssm"], meta.cu_seqlens, meta.state_slots,
                         meta.seq_starts, s.norm_groups, self.norm_eps)
        return F.linear(y, self.o_proj)


class ClampedGLU(nn.Module):
    """Dense gated feed-forward with a clamped gate and a shifted linear
    branch: down(g·sigmoid(alpha·g)·(u + 1)), g = min(gate, limit),
    u = clamp(up, ±limit)."""

    def __init__(self, hidden: int, spec: DenseFFSpec, dtype):
        super().__init__()
        self.spec = spec
        self.gate_up = _p(2 * spec.ff, hidden, dtype=dtype)   # [gate | up]
        self.down = _p(hidden, spec.ff, dtype=dtype)

    def forward(self, x):
        a = ops.clamped_glu(F.linear(x, self.gate_up), self.spec.limit,
                            self.spec.alpha)
        return F.linear(a, self.down)


class LatentAttention(nn.Module):
    """Softmax attention over a paged cache of low-rank latents. Per token
    the cache holds c = rms(W_dkv x)[:rank]·w and one rotated key part of
    `rot_dim` dims shared by all heads; head h's key is [W_uk,h c | rotated
    part] and its value W_uv,h c. Queries carry `dim` unrotated and
    `rot_dim` rotated dims per head. Options: per-head sink in the softmax
    denominator, per-head sigmoid output gate read from the mixer input,
    queries through an RMS-normed latent of their own (spec.q_rank), the
    rotation pairing neighbours (2i, 2i + 1) and carrying interpolated
    frequencies with a magnitude. With spec.kv_from set the mixer has no down-projection and reads the
    cache of the layer it names (the caller passes that layer's cache).

    Two equivalent evaluations (key and value are linear in c):
      * latent form — the unrotated query is folded through W_uk
        (q_c = W_uk,hᵀ q), scores are q_c·c + q_rot·k_rot, the weighted sum
        runs over c and W_uv is applied to the result. One pass over the
        cache serves every head; used for single tokens and in f32.
      * expanded form — for prompt portions in bf16 the latents of the
        step's sequences are gathered, up-projected to per-head keys and
        values in a step-local paged scratch, and the MFMA attention
        kernel of the window mixers runs on it (fewer flops per score:
        dim + rot_dim instead of rank + rot_dim)."""

    def __init__(self, hidden: int, spec: LatentAttnSpec, dtype,
                 norm_eps: float):
        super().__init__()
        self.spec, self.dtype, self.norm_eps = spec, dtype, norm_eps
        s = spec
        assert s.rot is not None and s.rot.dims == s.rot_dim \
            and s.rot_dim % 2 == 0
        self.own_kv = s.kv_from is None
        self.q_size = s.heads * (s.dim + s.rot_dim)
        self.g_size = s.heads if s.gate else 0
        self.row = s.kv_rank + s.rot_dim
        # fused input projection, rows [q (or its latent) | gate | latent +
        # rotated key], zero rows up to a multiple of 8 so that output
        # rows stay 16-byte aligned for the kernels' vector moves
        self.q_rows = s.q_rank if s.q_rank > 0 else self.q_size
        self.in_rows = self.q_rows + self.g_size \
            + (self.row if self.own_kv else 0)
        if s.q_rank > 0:
            self.q_norm = _p(s.q_rank, dtype=torch.float32)
            self.w_uq = _p(self.q_size, s.q_rank, dtype=dtype)
        self.in_proj = _p((self.in_rows + 7) // 8 * 8, hidden, dtype=dtype)
        self.kv_norm = _p(s.kv_rank, dtype=torch.float32) \
            if self.own_kv else None
        self.w_uk = _p(s.heads * s.dim, s.kv_rank, dtype=dtype)
        self.w_uv = _p(s.heads * s.vdim, s.kv_rank, dtype=dtype)
        freq, self.rot_mag = s.rot.frequencies()
        self.register_buffer("inv_freq", torch.tensor(
            freq, dtype=torch.float64).float(), persistent=False)
        self.sinks = _p(s.heads, dtype=torch.float32) if s.sink else None
        self.o_proj = _p(hidden, s.heads * s.vdim, dtype=dtype)

    def alloc_cache(self, num_blocks, block_size, num_slots, device) -> Dict:
        if not self.own_kv:
            return {}
        return {"kv": torch.zeros(num_blocks, block_size, self.row,
                                  dtype=self.dtype, device=device)}

    def cache_bytes(self, block_size: int):
        if not self.own_kv:
            return 0, 0
        esz = torch.empty(0, dtype=self.dtype).element_size()
        return block_size * self.row * esz, 0

    def _expanded_ok(self, x, meta) -> bool:
        s = self.spec
        return (x.is_cuda and x.dtype == torch.bfloat16
                and meta.tile_seq is not None
                and meta.ctx_lens is not None
                and s.dim + s.rot_dim <= max(ops.WINDOW_MFMA_SIZES)
                and s.vdim <= max(ops.WINDOW_MFMA_VSIZES))

    def forward(self, x, positions, cache, meta):
        s = self.spec
        T, H, D = x.size(0), s.heads, s.dim
        p = F.linear(x, self.in_proj)
        if s.q_rank > 0:
            cq = ops.rms_norm_cast(p[:, :s.q_rank].contiguous(), self.q_norm,
                                   self.norm_eps, self.dtype)
            q = F.linear(cq, self.w_uq).unflatten(-1, (H, D + s.rot_dim))
        else:
            q = p[:, :self.q_size].unflatten(-1, (H, D + s.rot_dim))
        dkv = p[:, self.q_rows + self.g_size:self.in_rows] \
            if self.own_kv else None
        kv = cache["kv"]
        expanded = self._expanded_ok(x, meta)
        # the MFMA prompt kernel takes key sizes 64/128/256: pad in place
        pad = next(d for d in ops.WINDOW_MFMA_SIZES
                   if d >= D + s.rot_dim) if expanded else 0
        qr = ops.latent_rope_cache_write(
            q, dkv, self.kv_norm, self.norm_eps, kv, meta.slot_mapping,
            positions, self.inv_freq, D, pad_to=pad,
            interleaved=s.rot.interleaved, rot_mag=self.rot_mag)
        if expanded:
            o = self._expanded(qr, kv, meta)
        else:
            qc = torch.bmm(qr[..., :D].transpose(0, 1),
                           self.w_uk.view(H, D, s.kv_rank))     # [H, T, r]
            qf = torch.cat([qc.transpose(0, 1), qr[..., D:]], -1)
            oc = ops.latent_attention(qf, kv, meta.block_tables,
                                      meta.token_seq, positions, s.scale,
                                      s.kv_rank, self.sinks)     # [T, H, r]
            o = torch.bmm(oc.transpose(0, 1),
                          self.w_uv.view(H, s.vdim, s.kv_rank)
                          .transpose(1, 2)).transpose(0, 1)
        o = o.reshape(T, H * s.vdim)
        if s.gate:
            o = ops.sigmoid_mul(o, p[:, self.q_rows:self.q_rows + H])
        return F.linear(o, self.o_proj)

    def _expanded(self, qr, kv, meta):
        """Prompt portions (bf16): per-head keys and values of the step's
        sequences in a step-local paged scratch, then the MFMA kernel."""
        s = self.spec
        H, D, R, V = s.heads, s.dim, s.rot_dim, s.vdim
        Dp = qr.size(2)                 # queries arrive zero-padded
        Vp = next(v for v in ops.WINDOW_MFMA_VSIZES if v >= V)
        lat, tables = ops.latent_gather(kv, meta.block_tables, meta.ctx_lens)
        k_s, v_s = ops.latent_expand(
            F.linear(lat[:, :s.kv_rank], self.w_uk),
            F.linear(lat[:, :s.kv_rank], self.w_uv), lat, H, D, V, s.kv_rank,
            Dp, Vp, kv.size(1))
        o = ops.window_attention(
            qr, k_s, v_s, tables, meta.token_seq, None, s.scale,
            tiles=(meta.tile_seq, meta.tile_qbase, meta.cu_seqlens,
                   meta.seq_starts), sinks=self.sinks)
        return o[..., :V]


class GeluGLU(nn.Module):
    """Dense gated feed-forward down(gelu_tanh(gate x) · up x)."""

    def __init__(self, hidden: int, spec: GeluGLUSpec, dtype):
        super().__init__()
        self.spec = spec
        self.gate_up = _p(2 * spec.ff, hidden, dtype=dtype)   # [gate | up]
        self.down = _p(hidden, spec.ff, dtype=dtype)

    def forward(self, x):
        return F.linear(ops.gelu_glu(F.linear(x, self.gate_up)), self.down)


class DiagDeltaMixer(nn.Module):
    """Generalized delta rule. Per head the state S is a [dim, dim] f32
    matrix; per token, with the unit key u = k/|k|,
        S <- diag(w) S - (a*u)(u^T S) + k v^T,      o = S^T r,
    where the decay w = exp(-rate*sigmoid(W2 tanh(W1 x) + w0)) and the
    removal rate a = sigmoid(W_a x + b) are per head and key channel. o is
    divided by its RMS per head, weighted over all heads, gated by
    sigmoid(W_g x) and projected out. r, k, v and the gate come from one
    activation-dtype projection; the pre-activations of w and a from a
    projection whose result stays f32 (they enter the recurrence)."""

    def __init__(self, hidden: int, spec: DiagDeltaSpec, dtype,
                 norm_eps: float, decay_rank: int = 32):
        super().__init__()
        self.spec, self.dtype, self.norm_eps = spec, dtype, norm_eps
        self.hidden = hidden
        self.n = spec.heads * spec.dim
        # fused input projection, rows [r | k | v | gate]
        self.in_proj = _p(4 * self.n, hidden, dtype=dtype)
        self.a_bias = _p(self.n, dtype=torch.float32)
        self.w0 = _p(self.n, dtype=torch.float32)
        self.out_norm = _p(self.n, dtype=torch.float32)
        self.o_proj = _p(hidden, self.n, dtype=dtype)
        self.set_decay_rank(decay_rank)

    def set_decay_rank(self, rank: int):
        """(Re)create the low-rank decay path for a bottleneck of `rank`
        (a checkpoint's tensor shapes decide it)."""
        dev = self.in_proj.device
        self.decay_rank = rank
        # rows [removal rate a | decay bottleneck W1], f32 result
        self.gate_proj = nn.Parameter(torch.empty(
            self.n + rank, self.hidden, dtype=self.dtype, device=dev),
            requires_grad=False)
        self.w2 = nn.Parameter(torch.empty(
            self.n, rank, dtype=torch.float32, device=dev),
            requires_grad=False)

    def alloc_cache(self, num_blocks, block_size, num_slots, device) -> Dict:
        s = self.spec
        return {"ssm": torch.zeros(num_slots, s.heads, s.dim, s.dim,
                                   dtype=torch.float32, device=device)}

    def cache_bytes(self, block_size: int):
        s = self.spec
        return 0, s.heads * s.dim * s.dim * 4

    def forward(self, x, positions, cache, meta):
        s = self.spec
        n = self.n
        p = F.linear(x, self.in_proj)
        gp = ops.linear_f32(x, self.gate_proj)               # [T, n + rank]
        w_pre = F.linear(torch.tanh(gp[:, n:]), self.w2, self.w0)
        hd = (s.heads, s.dim)
        o = ops.diag_delta_rule(
            p[:, :n].unflatten(-1, hd), p[:, n:2 * n].unflatten(-1, hd),
            p[:, 2 * n:3 * n].unflatten(-1, hd), w_pre, gp[:, :n],
            p[:, 3 * n:].unflatten(-1, hd), self.out_norm, cache["ssm"],
            meta.cu_seqlens, meta.state_slots, meta.seq_starts,
            s.decay_rate, s.k_eps, self.norm_eps, a_bias=self.a_bias)
        return F.linear(o, self.o_proj)


class HGRN2Mixer(nn.Module):
    """Gated linear attention with one gate for forgetting and writing (a
    channel that keeps a fraction f takes in 1 - f): per head S <- diag(f) S + (1 - f) v^T, o = S^T q with
    q = silu(W_q x) and f = lower + (1 - lower) sigmoid(W_f x + b) per head
    and channel (f scales state rows, which are indexed like q).
    o is RMS-normed over vdim with a weight shared by the heads and
    projected out. The gate pre-activation stays f32."""

    def __init__(self, hidden: int, spec: HGRN2Spec, dtype, norm_eps: float):
        super().__init__()
        self.spec, self.dtype, self.norm_eps = spec, dtype, norm_eps
        s = spec
        self.n_q = s.heads * s.dim
        self.n_v = s.heads * s.vdim
        self.in_proj = _p(self.n_q + self.n_v, hidden, dtype=dtype)  # [q | v]
        self.f_proj = _p(self.n_q, hidden, dtype=dtype)
        self.f_bias = _p(self.n_q, dtype=torch.float32)
        self.lower = _p(self.n_q, dtype=torch.float32)
        self.out_norm = _p(s.vdim, dtype=torch.float32)
        self.o_proj = _p(hidden, self.n_v, dtype=dtype)

    def alloc_cache(self, num_blocks, block_size, num_slots, device) -> Dict:
        s = self.spec
        return {"ssm": torch.zeros(num_slots, s.heads, s.dim, s.vdim,
                                   dtype=torch.float32, device=device)}

    def cache_bytes(self, block_size: int):
        s = self.spec
        return 0, s.heads * s.dim * s.vdim * 4

    def forward(self, x, positions, cache, meta):
        s = self.spec
        p = F.linear(x, self.in_proj)
        f_pre = ops.linear_f32(x, self.f_proj)
        o = ops.hgrn2_scan(
            p[:, :self.n_q].unflatten(-1, (s.heads, s.dim)),
            p[:, self.n_q:].unflatten(-1, (s.heads, s.vdim)), f_pre,
            self.lower, self.out_norm, cache["ssm"], meta.cu_seqlens,
            meta.state_slots, meta.seq_starts, self.norm_eps,
            f_bias=self.f_bias)
        return F.linear(o, self.o_proj)
