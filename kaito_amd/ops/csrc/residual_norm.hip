// Norms for models that keep the residual stream in f32 and put the norm
// on the sub-layer OUTPUT:
//
//   post_norm_residual:  x32 += rms(m) * w           (in place, f32)
//       m = y                                          (one sub-layer), or
//       m = (rms(y) * w_y + rms(y2) * w_y2) / 2        (two side by side)
//     and x32's rounding to the activation dtype is emitted for the next
//     sub-layer in the same pass.
//   rms_norm_cast: rms(x) * w for f32 or bf16 rows → f32 or bf16.
//
// and for pre-norm models with an f32 stream:
//
//   residual_add_norm:   x32 += s1 * y (+ s2 * y2)   (in place, f32)
//                        h    = rms(x32) * w          (next sub-layer's input)
//   scaled_residual_add_norm:  x32 += v1*y1 (+ v2*y2) (+ v3*y3) (+ x_add)
//                        with per-channel f32 scales v, then h as above
//   token_shift:         hs_t = h_t + (h_{t-1} - h_t) * mu, the row before a
//                        chunk's first kept per sequence in a state slot
//
// One workgroup per row; m is staged in LDS (f32) between the passes.
// All weights are f32.
#include "mix_common.h"
#include <type_traits>

namespace kaito {

namespace {

template <typename T, typename TO>
__global__ void post_norm_residual_kernel(
    float* __restrict__ x32, TO* __restrict__ xo, const bool write_xo,
    const T* __restrict__ y, const int64_t y_s0, const float* __restrict__ w,
    const T* __restrict__ y2, const int64_t y2_s0,
    const float* __restrict__ w_y, const float* __restrict__ w_y2,
    const int H, const float eps) {
  extern __shared__ float m[];          // [H]
  __shared__ float red[16];
  const int row = blockIdx.x;
  const T* yr = y + (int64_t)row * y_s0;
  if (y2 != nullptr) {
    const T* y2r = y2 + (int64_t)row * y2_s0;
    float s1 = 0.f, s2 = 0.f;
    for (int i = threadIdx.x; i < H; i += blockDim.x) {
      const float a = act_ld(yr + i), b = act_ld(y2r + i);
      s1 += a * a;
      s2 += b * b;
    }
    s1 = block_reduce_sum(s1, red);
    __syncthreads();
    s2 = block_reduce_sum(s2, red);
    __syncthreads();
    const float i1 = 1.0f / sqrtf(s1 / (float)H + eps);
    const float i2 = 1.0f / sqrtf(s2 / (float)H + eps);
    for (int i = threadIdx.x; i < H; i += blockDim.x)
      m[i] = 0.5f * (act_ld(yr + i) * i1 * w_y[i] +
                     act_ld(y2r + i) * i2 * w_y2[i]);
  } else {
    for (int i = threadIdx.x; i < H; i += blockDim.x) m[i] = act_ld(yr + i);
  }
  // each thread re-reads only the m[] entries it wrote itself
  float ss = 0.f;
  for (int i = threadIdx.x; i < H; i += blockDim.x) ss += m[i] * m[i];
  ss = block_reduce_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)H + eps);
  float* xr = x32 + (int64_t)row * H;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    const float v = xr[i] + m[i] * inv * w[i];
    xr[i] = v;
    if (write_xo) act_st(xo + (int64_t)row * H + i, v);
  }
}

template <typename TI, typename TO>
__global__ void rms_norm_cast_kernel(
    TO* __restrict__ out, const TI* __restrict__ x,
    const float* __restrict__ w, const int H, const float eps) {
  __shared__ float red[16];
  const int row = blockIdx.x;
  const TI* xr = x + (int64_t)row * H;
  float ss = 0.f;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    const float v = act_ld(xr + i);
    ss += v * v;
  }
  ss = block_reduce_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)H + eps);
  for (int i = threadIdx.x; i < H; i += blockDim.x)
    act_st(out + (int64_t)row * H + i, act_ld(xr + i) * inv * w[i]);
}

// One workgroup per row. Each thread re-reads only the stream entries it
// wrote itself, so the row needs no LDS stage.
template <typename T, typename TO>
__global__ void residual_add_norm_kernel(
    float* __restrict__ x32, TO* __restrict__ h_out,
    const T* __restrict__ y, const int64_t y_s0,
    const T* __restrict__ y2, const int64_t y2_s0,
    const float* __restrict__ w, const float s1, const float s2, const int H,
    const float eps) {
  __shared__ float red[16];
  const int row = blockIdx.x;
  float* xr = x32 + (int64_t)row * H;
  const T* yr = y + (int64_t)row * y_s0;
  const T* y2r = y2 ? y2 + (int64_t)row * y2_s0 : nullptr;
  float ss = 0.f;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    float add = s1 * act_ld(yr + i);
    if (y2r) add += s2 * act_ld(y2r + i);
    const float v = xr[i] + add;
    xr[i] = v;
    ss += v * v;
  }
  if (w == nullptr) return;
  ss = block_reduce_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)H + eps);
  for (int i = threadIdx.x; i < H; i += blockDim.x)
    act_st(h_out + (int64_t)row * H + i, xr[i] * inv * w[i]);
}

// N = number of (y, v) terms, known at compile time so that the row loop
// has no branches and its loads are issued together
template <typename T, typename TO, int N>
__global__ void scaled_residual_add_norm_kernel(
    float* __restrict__ x32, TO* __restrict__ h_out,
    const T* __restrict__ y0, const int64_t s0, const T* __restrict__ y1,
    const int64_t s1, const T* __restrict__ y2, const int64_t s2,
    const float* __restrict__ v0, const float* __restrict__ v1,
    const float* __restrict__ v2, const float* __restrict__ x_add,
    const float* __restrict__ w, const int H, const float eps) {
  __shared__ float red[16];
  const int row = blockIdx.x;
  float* xr = x32 + (int64_t)row * H;
  const T* r0 = y0 + (int64_t)row * s0;
  const T* r1 = N > 1 ? y1 + (int64_t)row * s1 : nullptr;
  const T* r2 = N > 2 ? y2 + (int64_t)row * s2 : nullptr;
  const float* ar = x_add ? x_add + (int64_t)row * H : nullptr;
  float ss = 0.f;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    float add = v0[i] * act_ld(r0 + i);
    if constexpr (N > 1) add += v1[i] * act_ld(r1 + i);
    if constexpr (N > 2) add += v2[i] * act_ld(r2 + i);
    float v = xr[i] + add;
    if (ar) v += ar[i];
    xr[i] = v;
    ss += v * v;
  }
  if (w == nullptr) return;
  ss = block_reduce_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)H + eps);
  for (int i = threadIdx.x; i < H; i += blockDim.x)
    act_st(h_out + (int64_t)row * H + i, xr[i] * inv * w[i]);
}

// One workgroup per row. The first row of a chunk reads its predecessor
// from the sequence's slot (zeros at position 0) and then parks the chunk's
// LAST row of h there; every thread reads and writes the same elements of
// the slot, and no other workgroup touches it, so one launch suffices.
template <typename T>
__global__ void token_shift_kernel(
    T* __restrict__ out, const T* __restrict__ h, const float* __restrict__ mu,
    T* __restrict__ state, const int* __restrict__ cu,
    const int* __restrict__ slots, const int* __restrict__ starts,
    const int* __restrict__ token_seq, const int H) {
  const int t = blockIdx.x;
  const int b = token_seq[t];
  const T* hr = h + (int64_t)t * H;
  T* orow = out + (int64_t)t * H;
  const int slot = b >= 0 ? slots[b] : -1;
  if (slot < 0) {
    for (int i = threadIdx.x; i < H; i += blockDim.x) orow[i] = hr[i];
    return;
  }
  const bool first = t == cu[b];
  if (!first) {
    const T* pr = hr - H;
    for (int i = threadIdx.x; i < H; i += blockDim.x) {
      const float c = act_ld(hr + i);
      act_st(orow + i, c + (act_ld(pr + i) - c) * mu[i]);
    }
    return;
  }
  const bool carried = starts[b] > 0;
  T* sr = state + (int64_t)slot * H;
  const T* lr = h + (int64_t)(cu[b + 1] - 1) * H;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    const float c = act_ld(hr + i);
    const float p = carried ? act_ld(sr + i) : 0.0f;
    act_st(orow + i, c + (p - c) * mu[i]);
    sr[i] = lr[i];
  }
}

int row_threads(int H) { return H >= 1024 ? 256 : (H >= 256 ? 128 : 64); }

}  // namespace

void post_norm_residual(at::Tensor x32, at::Tensor x_out, at::Tensor y,
                        at::Tensor w, double eps, at::Tensor y2,
                        at::Tensor w_y, at::Tensor w_y2) {
  KAITO_CHECK_F32(x32);
  TORCH_CHECK(x32.dim() == 2 && y.dim() == 2 && y.stride(1) == 1 &&
              y.sizes() == x32.sizes() && is_act_dtype(y));
  const int T = x32.size(0), H = x32.size(1);
  KAITO_CHECK_F32(w);
  TORCH_CHECK(w.numel() == H);
  const bool pair = y2.numel() > 0;
  if (pair) {
    TORCH_CHECK(y2.dim() == 2 && y2.stride(1) == 1 &&
                y2.sizes() == x32.sizes() && y2.dtype() == y.dtype());
    KAITO_CHECK_F32(w_y); KAITO_CHECK_F32(w_y2);
    TORCH_CHECK(w_y.numel() == H && w_y2.numel() == H);
  }
  const bool write_xo = x_out.data_ptr() != x32.data_ptr();
  TORCH_CHECK(x_out.is_contiguous() && x_out.sizes() == x32.sizes() &&
              is_act_dtype(x_out));
  TORCH_CHECK((size_t)H * 4 <= 64 * 1024, "row too wide for the LDS stage");
  if (T == 0) return;
  auto stream = at::hip::getCurrentHIPStream();
  const int threads = row_threads(H);
  KAITO_DISPATCH_ACT(y, {
    using in_t = act_t;
    KAITO_DISPATCH_ACT(x_out, {
      hipLaunchKernelGGL((post_norm_residual_kernel<in_t, act_t>), dim3(T),
          dim3(threads), (size_t)H * 4, stream, x32.data_ptr<float>(),
          (act_t*)x_out.data_ptr(), write_xo, (const in_t*)y.data_ptr(),
          y.stride(0), w.data_ptr<float>(),
          pair ? (const in_t*)y2.data_ptr() : nullptr,
          pair ? y2.stride(0) : 0, pair ? w_y.data_ptr<float>() : nullptr,
          pair ? w_y2.data_ptr<float>() : nullptr, H, (float)eps);
    });
  });
}

void residual_add_norm(at::Tensor x32, at::Tensor h_out, at::Tensor y,
                       at::Tensor y2, at::Tensor w, double s1, double s2,
                       double eps) {
  KAITO_CHECK_F32(x32);
  TORCH_CHECK(x32.dim() == 2 && y.dim() == 2 && y.stride(1) == 1 &&
              y.sizes() == x32.sizes() && is_act_dtype(y));
  const int T = x32.size(0), H = x32.size(1);
  const bool pair = y2.numel() > 0;
  if (pair)
    TORCH_CHECK(y2.dim() == 2 && y2.stride(1) == 1 &&
                y2.sizes() == x32.sizes() && y2.dtype() == y.dtype());
  const bool norm = w.numel() > 0;
  if (norm) {
    KAITO_CHECK_F32(w);
    TORCH_CHECK(w.numel() == H && h_out.is_contiguous() &&
                h_out.sizes() == x32.sizes() && is_act_dtype(h_out) &&
                h_out.data_ptr() != x32.data_ptr());
  }
  if (T == 0) return;
  auto stream = at::hip::getCurrentHIPStream();
  const int threads = row_threads(H);
  KAITO_DISPATCH_ACT(y, {
    using in_t = act_t;
    if (!norm || h_out.dtype() == at::kFloat) {
      hipLaunchKernelGGL((residual_add_norm_kernel<in_t, float>), dim3(T),
          dim3(threads), 0, stream, x32.data_ptr<float>(),
          norm ? h_out.data_ptr<float>() : nullptr,
          (const in_t*)y.data_ptr(), y.stride(0),
          pair ? (const in_t*)y2.data_ptr() : nullptr,
          pair ? y2.stride(0) : 0, norm ? w.data_ptr<float>() : nullptr,
          (float)s1, (float)s2, H, (float)eps);
    } else {
      hipLaunchKernelGGL((residual_add_norm_kernel<in_t, bf16_act>), dim3(T),
          dim3(threads), 0, stream, x32.data_ptr<float>(),
          (bf16_act*)h_out.data_ptr(), (const in_t*)y.data_ptr(),
          y.stride(0), pair ? (const in_t*)y2.data_ptr() : nullptr,
          pair ? y2.stride(0) : 0, w.data_ptr<float>(), (float)s1, (float)s2,
          H, (float)eps);
    }
  });
}

void rms_norm_cast(at::Tensor out, at::Tensor x, at::Tensor w, double eps) {
  TORCH_CHECK(x.is_cuda() && x.is_contiguous() && is_act_dtype(x) &&
              out.is_contiguous() && is_act_dtype(out) &&
              out.sizes() == x.sizes() && x.dim() >= 1);
  const int H = x.size(-1);
  const int T = H > 0 ? x.numel() / H : 0;
  KAITO_CHECK_F32(w);
  TORCH_CHECK(w.numel() == H);
  if (T == 0) return;
  auto stream = at::hip::getCurrentHIPStream();
  const int threads = row_threads(H);
  KAITO_DISPATCH_ACT(x, {
    using in_t = act_t;
    KAITO_DISPATCH_ACT(out, {
      hipLaunchKernelGGL((rms_norm_cast_kernel<in_t, act_t>), dim3(T),
          dim3(threads), 0, stream, (act_t*)out.data_ptr(),
          (const in_t*)x.data_ptr(), w.data_ptr<float>(), H, (float)eps);
    });
  });
}

void scaled_residual_add_norm(at::Tensor x32, at::Tensor h_out, at::Tensor y0,
                              at::Tensor y1, at::Tensor y2, at::Tensor v0,
                              at::Tensor v1, at::Tensor v2, at::Tensor x_add,
                              at::Tensor w, double eps) {
  KAITO_CHECK_F32(x32);
  TORCH_CHECK(x32.dim() == 2);
  const int T = x32.size(0), H = x32.size(1);
  auto check_term = [&](const at::Tensor& y, const at::Tensor& v) {
    TORCH_CHECK(y.is_cuda() && y.dim() == 2 && y.stride(1) == 1 &&
                y.sizes() == x32.sizes() && y.dtype() == y0.dtype());
    KAITO_CHECK_F32(v);
    TORCH_CHECK(v.numel() == H);
  };
  TORCH_CHECK(is_act_dtype(y0));
  check_term(y0, v0);
  const bool t1 = y1.numel() > 0, t2 = y2.numel() > 0;
  if (t1) check_term(y1, v1);
  if (t2) check_term(y2, v2);
  TORCH_CHECK(t1 || !t2);
  const bool addx = x_add.numel() > 0;
  if (addx) {
    KAITO_CHECK_F32(x_add);
    TORCH_CHECK(x_add.sizes() == x32.sizes());
  }
  const bool norm = w.numel() > 0;
  if (norm) {
    KAITO_CHECK_F32(w);
    TORCH_CHECK(w.numel() == H && h_out.is_contiguous() &&
                h_out.sizes() == x32.sizes() && is_act_dtype(h_out));
  }
  if (T == 0) return;
  auto stream = at::hip::getCurrentHIPStream();
  const int threads = row_threads(H);
  KAITO_DISPATCH_ACT(y0, {
    using in_t = act_t;
    auto launch_n = [&](auto* ho, auto nterms) {
      using out_t = std::remove_pointer_t<decltype(ho)>;
      constexpr int N = decltype(nterms)::value;
      hipLaunchKernelGGL((scaled_residual_add_norm_kernel<in_t, out_t, N>),
          dim3(T), dim3(threads), 0, stream, x32.data_ptr<float>(), ho,
          (const in_t*)y0.data_ptr(), y0.stride(0),
          t1 ? (const in_t*)y1.data_ptr() : nullptr, t1 ? y1.stride(0) : 0,
          t2 ? (const in_t*)y2.data_ptr() : nullptr, t2 ? y2.stride(0) : 0,
          v0.data_ptr<float>(), t1 ? v1.data_ptr<float>() : nullptr,
          t2 ? v2.data_ptr<float>() : nullptr,
          addx ? x_add.data_ptr<float>() : nullptr,
          norm ? w.data_ptr<float>() : nullptr, H, (float)eps);
    };
    auto launch = [&](auto* ho) {
      if (t2) launch_n(ho, std::integral_constant<int, 3>{});
      else if (t1) launch_n(ho, std::integral_constant<int, 2>{});
      else launch_n(ho, std::integral_constant<int, 1>{});
    };
    if (norm && h_out.dtype() == at::kBFloat16)
      launch((bf16_act*)h_out.data_ptr());
    else
      launch(norm ? (float*)h_out.data_ptr() : (float*)nullptr);
  });
}

void token_shift(at::Tensor out, at::Tensor h, at::Tensor mu, at::Tensor state,
                 at::Tensor cu_seqlens, at::Tensor state_slots,
                 at::Tensor seq_starts, at::Tensor token_seq) {
  TORCH_CHECK(h.is_cuda() && h.dim() == 2 && h.is_contiguous() &&
              is_act_dtype(h));
  const int T = h.size(0), H = h.size(1);
  TORCH_CHECK(out.is_contiguous() && out.sizes() == h.sizes() &&
              out.dtype() == h.dtype());
  KAITO_CHECK_F32(mu);
  TORCH_CHECK(mu.numel() == H);
  TORCH_CHECK(state.is_cuda() && state.is_contiguous() && state.dim() == 2 &&
              state.size(1) == H && state.dtype() == h.dtype());
  KAITO_CHECK_I32(cu_seqlens); KAITO_CHECK_I32(state_slots);
  KAITO_CHECK_I32(seq_starts); KAITO_CHECK_I32(token_seq);
  TORCH_CHECK(cu_seqlens.numel() == state_slots.numel() + 1 &&
              seq_starts.numel() == state_slots.numel() &&
              token_seq.numel() == T);
  if (T == 0) return;
  auto stream = at::hip::getCurrentHIPStream();
  KAITO_DISPATCH_ACT(h, {
    hipLaunchKernelGGL((token_shift_kernel<act_t>), dim3(T),
        dim3(row_threads(H)), 0, stream, (act_t*)out.data_ptr(),
        (const act_t*)h.data_ptr(), mu.data_ptr<float>(),
        (act_t*)state.data_ptr(), cu_seqlens.data_ptr<int>(),
        state_slots.data_ptr<int>(), seq_starts.data_ptr<int>(),
        token_seq.data_ptr<int>(), H);
  });
}

}  // namespace kaito

TORCH_LIBRARY_FRAGMENT(kaito, m) {
  m.def("post_norm_residual(Tensor(a!) x32, Tensor(b!) x_out, Tensor y, Tensor w, float eps, Tensor y2, Tensor w_y, Tensor w_y2) -> ()");
  m.def("rms_norm_cast(Tensor(a!) out, Tensor x, Tensor w, float eps) -> ()");
  m.def("residual_add_norm(Tensor(a!) x32, Tensor(b!) h_out, Tensor y, Tensor y2, Tensor w, float s1, float s2, float eps) -> ()");
  m.def("scaled_residual_add_norm(Tensor(a!) x32, Tensor(b!) h_out, Tensor y0, Tensor y1, Tensor y2, Tensor v0, Tensor v1, Tensor v2, Tensor x_add, Tensor w, float eps) -> ()");
  m.def("token_shift(Tensor(a!) out, Tensor h, Tensor mu, Tensor(b!) state, Tensor cu_seqlens, Tensor state_slots, Tensor seq_starts, Tensor token_seq) -> ()");
}
TORCH_LIBRARY_IMPL(kaito, CUDA, m) {
  m.impl("post_norm_residual", &kaito::post_norm_residual);
  m.impl("rms_norm_cast", &kaito::rms_norm_cast);
  m.impl("residual_add_norm", &kaito::residual_add_norm);
  m.impl("scaled_residual_add_norm", &kaito::scaled_residual_add_norm);
  m.impl("token_shift", &kaito::token_shift);
}
