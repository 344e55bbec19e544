"""kaito_amd.ops — gfx950 HIP kernels with a CPU fp32 reference fallback.

Dispatch policy (engine contract):
  * CUDA/ROCm tensors → the in-tree HIP extension. If the extension is
    missing on a GPU machine this raises loudly — there is NO silent
    eager fallback on GPU.
  * CPU tensors → torch_ref reference implementations (tests / no-GPU dev).

The extension is split into kernel groups (ops/_build.py GROUPS), one
shared library each; a group is built (if absent) and loaded the first
time one of its ops is called.
"""
from __future__ import annotations

import torch

from . import torch_ref
from ._build import GROUPS, SO_PATH, so_path

_LOADED: set = set()

# op name → kernel group that registers it
_OP_GROUP = {}
for _g, _names in {
    "core": ("rms_norm fused_add_rms_norm rotary_embedding silu_and_mul "
             "gelu_and_mul gelu layer_norm fused_add_layer_norm "
             "reshape_and_cache topk"),
    "attn": ("paged_attention paged_attention_sp prefill_attention "
             "context_attention mfma_tile_gemm paged_read_bw"),
    "mla": "mla_decode mla_cache_write",
    "moe": "moe_gate_silu moe_down_scatter",
    "quant": "w4a16_gemv w4a16_dequant w4a16_gemm lora_shrink lora_expand",
    "comm": ("allreduce_rmsnorm one_shot_ar_rmsnorm ipc_handle ipc_open "
             "ipc_close"),
    "mix": ("causal_conv_update "
            "qk_norm_cache_write window_attention window_attention_tiles "
            "post_norm_residual rms_norm_cast residual_add_norm "
            "scaled_residual_add_norm token_shift "
            "clamped_glu sigmoid_mul gelu_glu relu2"),
    "latent": ("bigram_embed latent_rope_cache_write latent_attention "
               "latent_expand"),
    "delta": "gated_delta_rule rglru_scan",
    "diag": "diag_delta_rule hgrn2_scan",
    "decay": "mlstm_scan ssd_scan",
}.items():
    for _n in _names.split():
        _OP_GROUP[_n] = _g

# groups that predate the split: load_extension() without arguments loads
# these, so `ops.load_extension(); torch.ops.kaito.<op>` keeps working
_LEGACY_GROUPS = ("core", "attn", "mla", "moe", "quant", "comm")


def extension_available(group: str = "core") -> bool:
    return so_path(group).exists()


def load_extension(*groups: str) -> None:
    """Load (and build, if absent) kernel groups; no arguments = every
    group except the lazily-loaded newer ones."""
    for g in (groups or _LEGACY_GROUPS):
        if g in _LOADED:
            continue
        if not so_path(g).exists():
            from ._build import build
            build(groups=[g])
        torch.ops.load_library(str(so_path(g)))
        _LOADED.add(g)


class _Kernels:
    """`_K.<op>` = torch.ops.kaito.<op> with its group loaded first."""

    def __getattr__(self, name: str):
        group = _OP_GROUP[name]
        if group not in _LOADED:
            if not torch.cuda.is_available():
                raise RuntimeError(
                    "kaito_amd.ops: got a CUDA tensor but torch.cuda is "
                    "unavailable")
            load_extension(group)
        fn = getattr(torch.ops.kaito, name)
        setattr(self, name, fn)
        return fn


_K = _Kernels()


def _require_ext() -> None:
    """Kept for callers that predate per-group loading (no-op: `_K`
    loads the group an op needs)."""


# ---------------------------------------------------------------- public ops

def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    if x.is_cuda:
        out = torch.empty_like(x)
        _K.rms_norm(out, x, weight, eps)
        return out
    return torch_ref.rms_norm(x, weight, eps)


def fused_add_rms_norm(x: torch.Tensor, residual: torch.Tensor,
                       weight: torch.Tensor, eps: float):
    """Returns (normed, residual). On GPU, `residual` is updated IN PLACE
    (residual += x) and returned."""
    if x.is_cuda:
        out = torch.empty_like(x)
        _K.fused_add_rms_norm(out, x, residual, weight, eps)
        return out, residual
    return torch_ref.fused_add_rms_norm(x, residual, weight, eps)


def rotary_embedding(positions: torch.Tensor, q: torch.Tensor, k: torch.Tensor,
                     head_dim: int, cos_sin_cache: torch.Tensor):
    """In-place on GPU; returns (q, k)."""
    if q.is_cuda:
        _K.rotary_embedding(positions, q, k, head_dim, cos_sin_cache)
        return q, k
    return torch_ref.rotary_embedding(positions, q, k, head_dim, cos_sin_cache)


def silu_and_mul(x: torch.Tensor) -> torch.Tensor:
    if x.is_cuda and x.dtype == torch.float32:
        # f32 verification mode: plain elementwise math, no bf16 kernel
        d = x.size(-1) // 2
        return torch.nn.functional.silu(x[..., :d]) * x[..., d:]
    if x.is_cuda:
        d = x.size(-1) // 2
        out = torch.empty(*x.shape[:-1], d, dtype=x.dtype, device=x.device)
        _K.silu_and_mul(out, x)
        return out
    return torch_ref.silu_and_mul(x)


def reshape_and_cache(k: torch.Tensor, v: torch.Tensor, k_cache: torch.Tensor,
                      v_cache: torch.Tensor, slot_mapping: torch.Tensor) -> None:
    """k/v: [T, KH, D] (rows may be strided views into a fused qkv buffer)."""
    if k.is_cuda:
        _K.reshape_and_cache(k, v, k_cache, v_cache, slot_mapping)
        return
    torch_ref.reshape_and_cache(k, v, k_cache, v_cache, slot_mapping)


# decode-attention implementation: "sp" = split-phase (r02, K-stream →
# exp pass → V-stream, no softmax chain in the memory loops), "fused" =
# the r01 single-pass online-softmax kernel. Overridable for A/B runs.
import os as _os
_PA_IMPL = _os.environ.get("KAITO_PA_IMPL", "sp")
# fused W4A16 GEMM for M>4: measured slower than dequant+hipBLASLt on
# MI355X (tools/bench_w4a16.py) — off unless explicitly enabled
W4A16_FUSED_GEMM = _os.environ.get("KAITO_W4A16_FUSED", "0") == "1"


def _sinks_arg(sinks, device):
    if sinks is None:
        return torch.empty(0, dtype=torch.float32, device=device)
    return sinks


def paged_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                    block_tables: torch.Tensor, seq_lens: torch.Tensor,
                    scale: float, window: int = 0,
                    sinks: torch.Tensor | None = None) -> torch.Tensor:
    if q.is_cuda:
        out = torch.empty_like(q)
        if _PA_IMPL == "sp" or window > 0 or sinks is not None \
                or k_cache.dtype == torch.uint8:
            # window/sink support lives in the split-phase kernel only
            _K.paged_attention_sp(
                out, q, k_cache, v_cache, block_tables, seq_lens, scale,
                window, _sinks_arg(sinks, q.device))
        else:
            _K.paged_attention(out, q, k_cache, v_cache,
                                            block_tables, seq_lens, scale)
        return out
    return torch_ref.paged_attention(q, k_cache, v_cache, block_tables,
                                     seq_lens, scale, window, sinks)


def mla_decode(q: torch.Tensor, cache: torch.Tensor,
               block_tables: torch.Tensor, seq_lens: torch.Tensor,
               scale: float, r: int) -> torch.Tensor:
    """Absorbed MLA decode over the compressed latent cache (DeepSeek).
    q: [T, H, r+rope]; cache: [NB, BS, r+rope] bf16. Returns [T, H, r]."""
    if q.is_cuda:
        out = torch.empty(q.size(0), q.size(1), r, dtype=q.dtype,
                          device=q.device)
        _K.mla_decode(out, q, cache, block_tables, seq_lens,
                                   scale)
        return out
    return torch_ref.mla_decode(q, cache, block_tables, seq_lens, scale, r)


def mla_cache_write(cache: torch.Tensor, c_kv: torch.Tensor,
                    k_pe: torch.Tensor, slots: torch.Tensor) -> None:
    """Scatter latent rows (c_kv ‖ k_pe) into the paged MLA cache;
    negative slots (graph-bucket padding) are skipped."""
    _K.mla_cache_write(cache, c_kv, k_pe, slots)


def prefill_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                      cu_seqlens: torch.Tensor, scale: float,
                      max_seqlen: int | None = None, window: int = 0,
                      sinks: torch.Tensor | None = None) -> torch.Tensor:
    if q.is_cuda:
        out = torch.empty_like(q)
        tile_seq, tile_qbase = _build_tiles(cu_seqlens)
        _K.prefill_attention(out, q, k, v, tile_seq, tile_qbase,
                                          cu_seqlens, scale, window,
                                          _sinks_arg(sinks, q.device))
        return out
    return torch_ref.prefill_attention(q, k, v, cu_seqlens, scale, window,
                                       sinks)


def context_attention(q: torch.Tensor, k_cache: torch.Tensor,
                      v_cache: torch.Tensor, cu_seqlens_q: torch.Tensor,
                      kv_lens: torch.Tensor, block_tables: torch.Tensor,
                      scale: float, window: int = 0,
                      sinks: torch.Tensor | None = None) -> torch.Tensor:
    """Suffix-query causal attention over the paged cache (chunked
    prefill / prefix-cache continuation)."""
    if q.is_cuda:
        out = torch.empty_like(q)
        tile_seq, tile_qbase = _build_tiles(cu_seqlens_q)
        _K.context_attention(out, q, k_cache, v_cache, tile_seq,
                                          tile_qbase, cu_seqlens_q, kv_lens,
                                          block_tables, scale, window,
                                          _sinks_arg(sinks, q.device))
        return out
    return torch_ref.context_attention(q, k_cache, v_cache, cu_seqlens_q,
                                       kv_lens, block_tables, scale, window,
                                       sinks)


def gelu_and_mul(x: torch.Tensor) -> torch.Tensor:
    """GeGLU: gelu_tanh(x[..., :d]) * x[..., d:] (gemma MLPs)."""
    if x.is_cuda:
        d = x.size(-1) // 2
        out = torch.empty(*x.shape[:-1], d, dtype=x.dtype, device=x.device)
        _K.gelu_and_mul(out, x)
        return out
    return torch_ref.gelu_and_mul(x)


def gelu(x: torch.Tensor) -> torch.Tensor:
    """Plain tanh-approx GELU (phi-2 ungated MLP)."""
    if x.is_cuda:
        out = torch.empty_like(x)
        _K.gelu(out, x.contiguous())
        return out
    return torch_ref.gelu_tanh(x)


def layer_norm(x: torch.Tensor, weight: torch.Tensor,
               bias: torch.Tensor | None, eps: float) -> torch.Tensor:
    if x.is_cuda:
        out = torch.empty_like(x)
        b = bias if bias is not None else \
            torch.empty(0, dtype=x.dtype, device=x.device)
        _K.layer_norm(out, x, weight, b, eps)
        return out
    return torch_ref.layer_norm(x, weight, bias, eps)


def fused_add_layer_norm(x: torch.Tensor, residual: torch.Tensor,
                         weight: torch.Tensor, bias: torch.Tensor | None,
                         eps: float):
    """Returns (normed, residual); residual += x in place on GPU."""
    if x.is_cuda:
        out = torch.empty_like(x)
        b = bias if bias is not None else \
            torch.empty(0, dtype=x.dtype, device=x.device)
        _K.fused_add_layer_norm(out, x, residual, weight, b, eps)
        return out, residual
    new_res = (x.float() + residual.float()).to(x.dtype)
    return torch_ref.layer_norm(new_res, weight, bias, eps), new_res


def mfma_tile_gemm(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    return _K.mfma_tile_gemm(a, b)


QTILE = 64  # must match prefill_attention.hip


def _build_tiles(cu_seqlens: torch.Tensor):
    """Map varlen batch → list of 64-row Q tiles: (seq_idx, q_base)."""
    cs = cu_seqlens.tolist()
    seqs, bases = [], []
    for i in range(len(cs) - 1):
        L = cs[i + 1] - cs[i]
        for q0 in range(0, L, QTILE):
            seqs.append(i)
            bases.append(q0)
    dev = cu_seqlens.device
    return (torch.tensor(seqs, dtype=torch.int32, device=dev),
            torch.tensor(bases, dtype=torch.int32, device=dev))


def moe_gate_silu(act: torch.Tensor, x: torch.Tensor,
                  w_gate_up: torch.Tensor, sorted_ids: torch.Tensor,
                  offsets: torch.Tensor, e_base: int,
                  n_local_experts: int, bias: torch.Tensor | None = None,
                  act_mode: int = 0, act_limit: float = 7.0) -> None:
    """Fused MoE stage 1 (GPU only): gather rows by sorted token ids,
    gate/up grouped GEMM per expert, activation epilogue into `act`
    (act_mode 0 = SwiGLU, 1 = clamped swiglu min(g, limit)·sigmoid(1.702
    g)·(clamp(u, ±limit) + 1); optional
    per-expert [E, 2*IE] bias; 2 = ungated squared relu with weights
    [E, IE, H])."""
    b = bias if bias is not None else         torch.empty(0, dtype=x.dtype, device=x.device)
    _K.moe_gate_silu(act, x, w_gate_up, sorted_ids, offsets, b, act_mode,
                     e_base, n_local_experts, act_limit)


def moe_down_scatter(out: torch.Tensor, act: torch.Tensor,
                     w_down: torch.Tensor, sorted_ids: torch.Tensor,
                     gates: torch.Tensor, offsets: torch.Tensor,
                     e_base: int, n_local_experts: int,
                     bias: torch.Tensor | None = None) -> None:
    """Fused MoE stage 2 (GPU only): down grouped GEMM (+ optional
    [E, H] bias) + gated f32 atomic scatter into `out`."""
    b = bias if bias is not None else         torch.empty(0, dtype=act.dtype, device=act.device)
    _K.moe_down_scatter(out, act, w_down, sorted_ids, gates,
                                     offsets, b, e_base, n_local_experts)


def w4a16_gemv(x: torch.Tensor, qweight: torch.Tensor, scales: torch.Tensor,
               zeros: torch.Tensor, group: int) -> torch.Tensor:
    """Group-quantized W4A16 linear, small M (decode): out = x @ W^T with
    W dequantized on the fly inside the kernel."""
    if x.is_cuda:
        out = torch.empty(x.size(0), qweight.size(0), dtype=x.dtype,
                          device=x.device)
        _K.w4a16_gemv(out, x, qweight, scales, zeros, group)
        return out
    return torch_ref.w4a16_gemv(x, qweight, scales, zeros, group)


def w4a16_dequant(qweight: torch.Tensor, scales: torch.Tensor,
                  zeros: torch.Tensor, group: int,
                  out: torch.Tensor = None) -> torch.Tensor:
    """Dequantize packed 4-bit weights to bf16 [N, K] (feeds hipBLASLt
    MFMA for large-M GEMMs)."""
    if qweight.is_cuda:
        if out is None:
            out = torch.empty(qweight.size(0), qweight.size(1) * 8,
                              dtype=torch.bfloat16, device=qweight.device)
        _K.w4a16_dequant(out, qweight, scales, zeros, group)
        return out
    ref = torch_ref.w4a16_unpack(qweight, scales, zeros, group)
    return ref.to(torch.bfloat16) if out is None else out.copy_(ref)


def w4a16_gemm(x: torch.Tensor, qweight: torch.Tensor, scales: torch.Tensor,
               zeros: torch.Tensor, group: int) -> torch.Tensor:
    """Fused inline-dequant MFMA GEMM (GPU): y = x @ dequant(W)^T.
    The 4-bit weights never round-trip through a full-precision scratch
    buffer. CPU falls back to the unpack reference."""
    if x.is_cuda:
        out = torch.empty(x.size(0), qweight.size(0), dtype=x.dtype,
                          device=x.device)
        _K.w4a16_gemm(out, x.contiguous(), qweight, scales,
                                   zeros, group)
        return out
    return torch_ref.w4a16_gemv(x, qweight, scales, zeros, group)


# ---- stateful sequence mixers (hybrid stacks; kernel group "mix") --------
#
# Batch layout shared by these ops: the rows of all chunks of a step are
# concatenated; chunk b owns rows cu_seqlens[b]..cu_seqlens[b+1], belongs
# to the sequence held in state slot state_slots[b] (<0: padding, skipped)
# and starts at sequence position seq_starts[b] (0: fresh sequence, the
# slot's old content is ignored). token_seq[t] is the chunk of row t.
# Activations may be bf16 or f32 (one dtype per call); states, small
# per-channel parameters and all recurrence math are f32.

def _none(t, like):
    return t if t is not None else \
        torch.empty(0, dtype=torch.float32, device=like.device)


def causal_conv_update(x, weight, bias, conv_state, cu_seqlens, state_slots,
                       seq_starts, token_seq, act: int = 0):
    """Depthwise causal short convolution with a carried tail.
    x [T, C] (row stride free); weight [C, taps] f32; conv_state
    [slots, taps-1, C] in x's dtype, advanced in place; act 0 none,
    1 silu. Returns [T, C]."""
    if x.is_cuda:
        out = torch.empty(x.shape, dtype=x.dtype, device=x.device)
        _K.causal_conv_update(out, x, weight, _none(bias, x), conv_state,
                              cu_seqlens, state_slots, seq_starts, token_seq,
                              act)
        return out
    return torch_ref.causal_conv_update(x, weight, bias, conv_state,
                                        cu_seqlens, state_slots, seq_starts,
                                        act)


def gated_delta_rule(q, k, v, gate, a, b, a_log, dt_bias, norm_w, state,
                     cu_seqlens, state_slots, seq_starts, qk_eps: float,
                     norm_eps: float):
    """Gated delta rule with fused unit-norm of q/k, decay/beta
    activations, output RMS norm and silu gate. q/k [T, G, D], v/gate
    [T, H, V], a/b [T, H] (row strides free); state [slots, H, D, V] f32
    in place. Returns [T, H*V]."""
    if v.is_cuda:
        T, H, V = v.shape
        out = torch.empty(T, H * V, dtype=v.dtype, device=v.device)
        _K.gated_delta_rule(out, q, k, v, gate, a, b, a_log, dt_bias, norm_w,
                            state, cu_seqlens, state_slots, seq_starts,
                            qk_eps, norm_eps)
        return out
    return torch_ref.gated_delta_rule(
        q, k, v, gate, a, b, a_log, dt_bias, norm_w, state, cu_seqlens,
        state_slots, seq_starts, qk_eps, norm_eps).reshape(v.size(0), -1)


def rglru_scan(u, gates, y, decay_rate, state, cu_seqlens, state_slots,
               seq_starts, token_seq=None):
    """Real-gated linear recurrence + GELU gate branch. u/y [T, W] (row
    strides free); gates [B, T, 2*W/B] f32; decay_rate [W] f32; state
    [slots, W] f32 in place. Returns [T, W]."""
    if u.is_cuda:
        out = torch.empty(u.shape, dtype=u.dtype, device=u.device)
        # with token_seq, prompt-sized steps take the segment-parallel scan
        _K.rglru_scan(out, u, gates, y, decay_rate, state, cu_seqlens,
                      state_slots, seq_starts,
                      token_seq if token_seq is not None else
                      torch.empty(0, dtype=torch.int32, device=u.device))
        return out
    return torch_ref.rglru_scan(u, gates, y, decay_rate, state, cu_seqlens,
                                state_slots, seq_starts)


def qk_norm_cache_write(q, k, v, q_w, k_w, eps: float, k_cache, v_cache,
                        slot_mapping, positions=None, inv_freq=None,
                        rot_mag: float = 1.0, v_first=None,
                        v_lambda: float = 0.0):
    """Per-head RMS norm of q [T, H, D] / k [T, G, D] (f32 weights [D] or
    None), optional rotation (inv_freq [R] f32: dim i of every head is
    paired with dim i + R, angle = position * inv_freq[i] in f32, cos and
    sin times rot_mag), optional value blend v <- (1 - v_lambda) v +
    v_lambda v_first, fused with the scatter of k and v [T, G, V] into
    the paged caches [blocks, G, block_size, D|V]. Returns q normed and
    rotated, [T, H, D]."""
    if q.is_cuda:
        qn = torch.empty(q.shape, dtype=q.dtype, device=q.device)
        rot = inv_freq is not None and inv_freq.numel() > 0
        _K.qk_norm_cache_write(
            qn, q, k, v, _none(q_w, q), _none(k_w, q), eps, k_cache, v_cache,
            slot_mapping,
            positions if rot else torch.empty(0, dtype=torch.long,
                                              device=q.device),
            inv_freq if rot else _none(None, q), rot_mag,
            v_first if v_first is not None else
            torch.empty(0, dtype=q.dtype, device=q.device), v_lambda)
        return qn
    return torch_ref.qk_norm_cache_write(q, k, v, q_w, k_w, eps, k_cache,
                                         v_cache, slot_mapping, positions,
                                         inv_freq, rot_mag, v_first, v_lambda)


WINDOW_MFMA_SIZES = (64, 128, 256)          # key sizes of the MFMA kernel
WINDOW_MFMA_VSIZES = (32, 64, 128, 256)     # value sizes


def window_attention(q, k_cache, v_cache, block_tables, token_seq, positions,
                     scale: float, softcap: float = 0.0, r1=None, r2=None,
                     window: int = 0, tiles=None, keep_first: int = 0,
                     sinks=None, chunk: int = 0):
    """Causal attention of query rows [T, H, D] over the paged cache (key
    size D, value size V may differ). A query at position i sees keys
    j <= i with i - j < window or j < keep_first (window <= 0: all), or,
    with `chunk` > 0, keys j <= i of i's own block of `chunk` absolute
    positions (block b = positions [b*chunk, (b+1)*chunk)). Options: tanh score capping, the distance penalty
    r1*ln(1 + r2*distance), and per-head `sinks` [H] f32 whose exp joins
    the softmax denominator. Returns [T, H, V].

    `tiles` = (tile_seq, tile_qbase, cu_seqlens, seq_starts) describes the
    step's chunks as 64-row query tiles (build_query_tiles); with it, bf16
    inputs of supported head sizes take the MFMA prompt kernel. Without
    it (decode steps) or for f32 / other sizes, the one-row-per-workgroup
    f32 kernel runs."""
    if q.is_cuda:
        T, H, D = q.shape
        out = torch.empty(T, H, v_cache.size(3), dtype=q.dtype,
                          device=q.device)
        if (tiles is not None and q.dtype == torch.bfloat16
                and D in WINDOW_MFMA_SIZES
                and v_cache.size(3) in WINDOW_MFMA_VSIZES):
            tile_seq, tile_qbase, cu, starts = tiles
            _K.window_attention_tiles(
                out, q, k_cache, v_cache, block_tables, tile_seq, tile_qbase,
                cu, starts, scale, softcap, _none(r1, q), _none(r2, q),
                window, keep_first, _none(sinks, q), chunk)
            return out
        _K.window_attention(out, q, k_cache, v_cache, block_tables, token_seq,
                            positions, scale, softcap, _none(r1, q),
                            _none(r2, q), window, keep_first,
                            _none(sinks, q), chunk)
        return out
    return torch_ref.window_attention(q, k_cache, v_cache, block_tables,
                                      token_seq, positions, scale, softcap,
                                      r1, r2, window, keep_first, sinks,
                                      chunk)


def build_query_tiles(chunk_lens, device):
    """Host-side tiling of a step's chunks into 64-row query tiles:
    (tile_seq, tile_qbase) int32 tensors."""
    seqs, bases = [], []
    for i, n in enumerate(chunk_lens):
        for q0 in range(0, n, QTILE):
            seqs.append(i)
            bases.append(q0)
    return (torch.tensor(seqs, dtype=torch.int32, device=device),
            torch.tensor(bases, dtype=torch.int32, device=device))


def post_norm_residual(x32, y, w, eps: float, out_dtype, y2=None, w_y=None,
                       w_y2=None):
    """x32 [T, H] f32 += rms(m) * w in place, m = y or, with y2,
    (rms(y)*w_y + rms(y2)*w_y2)/2. Returns x32 rounded to out_dtype."""
    if x32.is_cuda:
        if out_dtype == torch.float32:
            xo = x32
        else:
            xo = torch.empty(x32.shape, dtype=out_dtype, device=x32.device)
        _K.post_norm_residual(x32, xo, y, w, eps, _none(y2, y),
                              _none(w_y, y), _none(w_y2, y))
        return xo
    return torch_ref.post_norm_residual(x32, y, w, eps, out_dtype, y2, w_y,
                                        w_y2)


def rms_norm_cast(x, weight, eps: float, out_dtype):
    """RMS norm of f32 or bf16 rows with an f32 weight → out_dtype."""
    if x.is_cuda:
        out = torch.empty(x.shape, dtype=out_dtype, device=x.device)
        _K.rms_norm_cast(out, x, weight, eps)
        return out
    return torch_ref.rms_norm_cast(x, weight, eps, out_dtype)


def mlstm_scan(q, k, v, ogate, ipre, fpre, norm_w, state_c, state_n, state_m,
               cu_seqlens, state_slots, seq_starts, cap: float,
               q_scale: float, norm_eps: float, denom_floor: float = 1e-6):
    """Matrix-memory (mLSTM) recurrence with fused gate activations,
    normaliser, per-head RMS norm and sigmoid output gate. q/k [T, H, D],
    v/ogate [T, H, V] (row strides free), ipre/fpre [T, H] f32; states
    C [slots, H, D, V], n [slots, H, D], m [slots, H] f32 in place.
    Returns [T, H*V]."""
    if v.is_cuda:
        T, H, V = v.shape
        out = torch.empty(T, H * V, dtype=v.dtype, device=v.device)
        _K.mlstm_scan(out, q, k, v, ogate, ipre, fpre, norm_w, state_c,
                      state_n, state_m, cu_seqlens, state_slots, seq_starts,
                      cap, q_scale, norm_eps, denom_floor)
        return out
    return torch_ref.mlstm_scan(q, k, v, ogate, ipre, fpre, norm_w, state_c,
                                state_n, state_m, cu_seqlens, state_slots,
                                seq_starts, cap, q_scale, norm_eps,
                                denom_floor)


def ssd_scan(x, B, C, dt, z, a_log, dt_bias, d_skip, norm_w, state,
             cu_seqlens, state_slots, seq_starts, norm_groups: int,
             norm_eps: float):
    """Scalar-decay selective state space with fused step-size
    activation, skip term, silu(z) gate and grouped RMS norm. x
    [T, H, P], B/C [T, G, N], z [T, H*P] (row strides free), dt [T, H]
    f32; state [slots, H, N, P] f32 in place. Returns [T, H*P]."""
    if x.is_cuda:
        T, H, P = x.shape
        out = torch.empty(T, H * P, dtype=x.dtype, device=x.device)
        _K.ssd_scan(out, x, B, C, dt, z, a_log, dt_bias, d_skip, norm_w,
                    state, cu_seqlens, state_slots, seq_starts, norm_groups,
                    norm_eps)
        return out
    return torch_ref.ssd_scan(x, B, C, dt, z, a_log, dt_bias, d_skip, norm_w,
                              state, cu_seqlens, state_slots, seq_starts,
                              norm_groups, norm_eps)


def residual_add_norm(x32, y, w, eps: float, out_dtype, y2=None,
                      s1: float = 1.0, s2: float = 1.0):
    """Pre-norm residual step on an f32 stream [T, H]: x32 += s1*y
    (+ s2*y2) in place; returns rms(x32)*w rounded to out_dtype, the next
    sub-layer's input (None when w is None)."""
    if x32.is_cuda:
        h = torch.empty(x32.shape, dtype=out_dtype, device=x32.device) \
            if w is not None else x32
        _K.residual_add_norm(x32, h, y, _none(y2, y), _none(w, y), s1, s2,
                             eps)
        return h if w is not None else None
    return torch_ref.residual_add_norm(x32, y, w, eps, out_dtype, y2, s1, s2)


def clamped_glu(gu, limit: float, alpha: float = 1.702):
    """[gate | up] rows [T, 2F] -> g*sigmoid(alpha*g)*(u + 1) [T, F] with
    g = min(gate, limit), u = clamp(up, -limit, limit)."""
    if gu.is_cuda:
        out = torch.empty(gu.size(0), gu.size(1) // 2, dtype=gu.dtype,
                          device=gu.device)
        _K.clamped_glu(out, gu, limit, alpha)
        return out
    return torch_ref.clamped_glu(gu, limit, alpha)


def sigmoid_mul(x, gate):
    """x [T, N] * sigmoid(gate [T, Ng]) (gate's row stride free); with
    Ng < N each gate column serves N/Ng consecutive columns of x (one
    gate per head)."""
    if x.is_cuda:
        out = torch.empty(x.shape, dtype=x.dtype, device=x.device)
        _K.sigmoid_mul(out, x, gate)
        return out
    return torch_ref.sigmoid_mul(x, gate)


def gelu_glu(gu):
    """[gate | up] rows [T, 2F] -> gelu_tanh(gate) * up [T, F]."""
    if gu.is_cuda:
        out = torch.empty(gu.size(0), gu.size(1) // 2, dtype=gu.dtype,
                          device=gu.device)
        _K.gelu_glu(out, gu)
        return out
    return torch_ref.gelu_glu(gu)


def relu2(x):
    """relu(x)^2, element-wise, rows [T, N] (row stride free)."""
    if x.is_cuda:
        out = torch.empty(x.shape, dtype=x.dtype, device=x.device)
        _K.relu2(out, x)
        return out
    return torch_ref.relu2(x)


# ---- latent attention (kernel group "latent") -----------------------------

def bigram_embed(ids, embed, scale: float, table, buckets: int,
                 mul_prev: int, mul_cur: int, prev_state, cu_seqlens,
                 state_slots, seq_starts, token_seq):
    """f32 rows embed[ids]*scale (+ the hashed bigram row: (previous *
    mul_prev + token * mul_cur) mod buckets, row `buckets` for a
    sequence's first token). The token before a chunk's first row comes
    from prev_state [slots] int64, which is advanced to the chunk's last
    token. table None: token embedding only."""
    if ids.is_cuda:
        out = torch.empty(ids.size(0), embed.size(1), dtype=torch.float32,
                          device=ids.device)
        none = torch.empty(0, dtype=embed.dtype, device=ids.device)
        _K.bigram_embed(out, ids, embed, scale,
                        table if table is not None else none, buckets,
                        mul_prev, mul_cur,
                        prev_state if table is not None else
                        torch.empty(0, dtype=torch.long, device=ids.device),
                        cu_seqlens, state_slots, seq_starts, token_seq)
        return out
    return torch_ref.bigram_embed(ids, embed, scale, table, buckets,
                                  mul_prev, mul_cur, prev_state, cu_seqlens,
                                  state_slots, seq_starts)


def latent_rope_cache_write(q, dkv, norm_w, eps: float, cache, slot_mapping,
                            positions, inv_freq, dim: int, pad_to: int = 0,
                            interleaved: bool = False, rot_mag: float = 1.0):
    """Rotation of the last 2R dims of every head of q [T, H, dim + 2R]
    (R = len(inv_freq); i paired with i + R, or with `interleaved` 2i
    with 2i + 1; angle = position * inv_freq[i] in f32; cos and sin times
    rot_mag) and, with dkv [T, rank + 2R] given (row stride
    free), the latent row: RMS norm of the first rank dims with the f32
    weight norm_w, rotation of the last 2R, scatter into the paged latent
    cache [blocks, block_size, rank + 2R] at slot_mapping (negative slots
    skipped). Returns q rotated, contiguous; with pad_to, every head is
    zero-padded to that many dims."""
    if q.is_cuda:
        out = torch.empty(q.size(0), q.size(1), max(pad_to, q.size(2)),
                          dtype=q.dtype, device=q.device)
        own = dkv is not None
        _K.latent_rope_cache_write(
            out, q, dkv if own else torch.empty(0, 0, dtype=q.dtype,
                                                device=q.device),
            norm_w if own else _none(None, q), eps,
            cache if own else torch.empty(0, dtype=q.dtype, device=q.device),
            slot_mapping, positions, inv_freq, dim, interleaved, rot_mag)
        return out
    out = torch_ref.latent_rope_cache_write(q, dkv, norm_w, eps, cache,
                                            slot_mapping, positions,
                                            inv_freq, dim, interleaved,
                                            rot_mag)
    if pad_to > out.size(2):
        out = torch.nn.functional.pad(out, (0, pad_to - out.size(2)))
    return out


def latent_attention(q, cache, block_tables, token_seq, positions,
                     scale: float, rank: int, sinks=None):
    """Causal attention of latent-space queries [T, H, rank + P] over the
    paged latent cache [blocks, block_size, rank + P]: score = q . row *
    scale over rows 0..position of the row's sequence, optional per-head
    sinks in the denominator, output = weighted sum of the rows' first
    `rank` dims, [T, H, rank]. One pass over the cache serves all heads."""
    if q.is_cuda:
        out = torch.empty(q.size(0), q.size(1), rank, dtype=q.dtype,
                          device=q.device)
        _K.latent_attention(out, q, cache, block_tables, token_seq,
                            positions, scale, _none(sinks, q))
        return out
    return torch_ref.latent_attention(q, cache, block_tables, token_seq,
                                      positions, scale, rank, sinks)


def latent_gather(cache, block_tables, ctx_lens):
    """Whole pages of the step's sequences out of the paged latent cache:
    chunk b's first ceil(ctx_lens[b] / block_size) pages, in block-table
    order. Returns (rows [pages * block_size, row], scratch block tables
    [B, max pages] int32 numbering the gathered pages consecutively).
    ctx_lens is a host list, so the shapes are known without a device
    read; rows past a sequence's length are whatever the page holds and
    stay behind the causal mask."""
    bs, mb = cache.size(1), block_tables.size(1)
    counts = [-(-int(n) // bs) for n in ctx_lens]
    idx, tables, base = [], [], 0
    width = max(max(counts), 1)
    for b, n in enumerate(counts):
        idx.extend(range(b * mb, b * mb + n))
        tables.append(list(range(base, base + n)) + [0] * (width - n))
        base += n
    dev = cache.device
    pages = block_tables.reshape(-1)[
        torch.tensor(idx, dtype=torch.long, device=dev)].long()
    rows = cache[pages].reshape(-1, cache.size(2))
    return rows, torch.tensor(tables, dtype=torch.int32, device=dev)


def latent_expand(kn, vv, lat, H: int, D: int, V: int, rank: int, Dp: int,
                  Vp: int, block_size: int):
    """Step-local paged K/V scratch from gathered latent rows (GPU): kn
    [N, H*D] and vv [N, H*V] are the up-projected unrotated keys and
    values of rows lat [N, rank + P]; head h's key is [kn_h | lat's last P
    dims | zeros] of width Dp, its value [vv_h | zeros] of width Vp.
    Returns k [N / block_size, H, block_size, Dp], v [..., Vp]."""
    pages = lat.size(0) // block_size
    k_s = torch.empty(pages, H, block_size, Dp, dtype=lat.dtype,
                      device=lat.device)
    v_s = torch.empty(pages, H, block_size, Vp, dtype=lat.dtype,
                      device=lat.device)
    _K.latent_expand(k_s, v_s, kn, vv, lat, H, D, V, rank)
    return k_s, v_s


# ---- looped parallel-layer stacks (groups "mix" and "diag") -----------------

def linear_f32(x, weight, bias=None):
    """x [T, K] @ weight [N, K]^T (+ bias) with the result kept in f32.
    Inputs in the activation dtype are multiplied exactly and summed in
    f32, and the result is not rounded back to the activation dtype: what
    feeds a recurrence's gates. On the GPU this is the vendor bf16 GEMM
    with an f32 output; where the build lacks that, an f32 GEMM."""
    global _MM_F32_OUT
    if x.dtype != torch.float32 and x.is_cuda and _MM_F32_OUT:
        try:
            out = torch.mm(x, weight.t(), out_dtype=torch.float32)
            return out if bias is None else out + bias
        except (RuntimeError, TypeError):
            _MM_F32_OUT = False
    return torch.nn.functional.linear(x.float(), weight.float(), bias)


_MM_F32_OUT = True


def scaled_residual_add_norm(x32, terms, w, eps: float, out_dtype,
                             x_add=None):
    """Residual step with per-channel sub-layer scales on an f32 stream
    [T, H]: x32 += sum of v*y over `terms`, one to three pairs (y [T, H]
    in the activation dtype, v [H] f32), (+ x_add [T, H] f32), in place;
    returns rms(x32)*w rounded to out_dtype, the next layer's input (None
    when w is None)."""
    assert 1 <= len(terms) <= 3
    if x32.is_cuda:
        h = torch.empty(x32.shape, dtype=out_dtype, device=x32.device) \
            if w is not None else x32
        y0 = terms[0][0]
        ys = [t[0] for t in terms] + [_none(None, y0)] * (3 - len(terms))
        vs = [t[1] for t in terms] + [_none(None, y0)] * (3 - len(terms))
        _K.scaled_residual_add_norm(x32, h, ys[0], ys[1], ys[2], vs[0],
                                    vs[1], vs[2], _none(x_add, y0),
                                    _none(w, y0), eps)
        return h if w is not None else None
    return torch_ref.scaled_residual_add_norm(x32, terms, w, eps, out_dtype,
                                              x_add)


def token_shift(h, mu, state, cu_seqlens, state_slots, seq_starts,
                token_seq):
    """Blend of every row with the row before it: h_t + (h_{t-1} - h_t)*mu
    (mu [H] f32). A chunk's first row takes its predecessor from state
    [slots, H] (h's dtype; zeros at position 0), which is advanced to the
    chunk's last row. Returns [T, H]."""
    if h.is_cuda:
        out = torch.empty(h.shape, dtype=h.dtype, device=h.device)
        _K.token_shift(out, h, mu, state, cu_seqlens, state_slots,
                       seq_starts, token_seq)
        return out
    return torch_ref.token_shift(h, mu, state, cu_seqlens, state_slots,
                                 seq_starts)


def diag_delta_rule(r, k, v, w_pre, a_pre, gate, norm_w, state, cu_seqlens,
                    state_slots, seq_starts, decay_rate: float, k_eps: float,
                    norm_eps: float, a_bias=None):
    """Generalized delta rule with a decay per key channel: r/k/v/gate
    [T, H, D] (row strides free), w_pre/a_pre [T, H*D] f32 (decay and
    removal-rate pre-activations), norm_w [H*D] f32, state [slots, H, D, D]
    f32 in place. S <- diag(w) S - (a*u)(u^T S) + k v^T with u the unit
    key, w = exp(-decay_rate*sigmoid(w_pre)), a = sigmoid(a_pre + a_bias)
    (a_bias [H*D] f32, optional); read-out S^T r divided by its RMS per
    head, times norm_w, times sigmoid(gate). Returns [T, H*D]."""
    if r.is_cuda:
        T, H, D = r.shape
        out = torch.empty(T, H * D, dtype=r.dtype, device=r.device)
        _K.diag_delta_rule(out, r, k, v, w_pre, a_pre, _none(a_bias, r), gate,
                           norm_w, state, cu_seqlens, state_slots, seq_starts,
                           decay_rate, k_eps, norm_eps)
        return out
    if a_bias is not None:
        a_pre = a_pre + a_bias
    return torch_ref.diag_delta_rule(r, k, v, w_pre, a_pre, gate, norm_w,
                                     state, cu_seqlens, state_slots,
                                     seq_starts, decay_rate, k_eps, norm_eps)


def hgrn2_scan(q, v, f_pre, lower, norm_w, state, cu_seqlens, state_slots,
               seq_starts, norm_eps: float, f_bias=None):
    """Linear attention with a lower-bounded forget gate that also sets
    the write: q [T, H, D] (silu applied inside), v [T, H, V] (row strides
    free), f_pre [T, H*D] f32, lower [H*D] f32, norm_w [V] f32, state
    [slots, H, D, V] f32 in place. f = lower + (1 - lower) sigmoid(f_pre +
    f_bias) (f_bias [H*D] f32, optional), S <- diag(f) S + (1 - f) v^T, o = S^T silu(q), RMS-normed over V with
    norm_w. Returns [T, H*V]."""
    if q.is_cuda:
        T, H, V = v.shape
        out = torch.empty(T, H * V, dtype=q.dtype, device=q.device)
        _K.hgrn2_scan(out, q, v, f_pre, _none(f_bias, q), lower, norm_w,
                      state, cu_seqlens, state_slots, seq_starts, norm_eps)
        return out
    if f_bias is not None:
        f_pre = f_pre + f_bias
    return torch_ref.hgrn2_scan(q, v, f_pre, lower, norm_w, state,
                                cu_seqlens, state_slots, seq_starts,
                                norm_eps)
