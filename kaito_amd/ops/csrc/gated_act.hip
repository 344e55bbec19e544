// Element-wise gates of the hybrid mixers and dense feed-forwards, for
// bf16 or f32 activations (f32 math):
//
//   clamped_glu:  [gate | up] rows [T, 2F] -> g * sigmoid(alpha g) * (u + 1)
//                 g = min(gate, limit), u = clamp(up, -limit, limit)
//   sigmoid_mul:  x * sigmoid(gate); a gate row narrower than x serves
//                 groups of adjacent columns (one gate per head)
//   gelu_glu:     [gate | up] rows [T, 2F] -> gelu_tanh(gate) * up
//   relu2:        relu(x)^2
#include "mix_common.h"

namespace kaito {

namespace {

template <typename T>
__global__ void clamped_glu_kernel(T* __restrict__ out,
                                   const T* __restrict__ gu,
                                   const int64_t gu_s0, const int F,
                                   const float limit, const float alpha) {
  const int t = blockIdx.y;
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= F) return;
  const T* row = gu + (int64_t)t * gu_s0;
  const float g = fminf(act_ld(row + i), limit);
  const float u = fminf(fmaxf(act_ld(row + F + i), -limit), limit);
  act_st(out + (int64_t)t * F + i, g * sigmoid_f(alpha * g) * (u + 1.0f));
}

// 16 bytes of gate and of up per thread (rows and F aligned to that)
template <typename T>
__global__ void clamped_glu_vec_kernel(T* __restrict__ out,
                                       const T* __restrict__ gu,
                                       const int64_t gu_s0, const int F,
                                       const float limit, const float alpha) {
  constexpr int VEC = 16 / (int)sizeof(T);
  const int t = blockIdx.y;
  const int i = (blockIdx.x * blockDim.x + threadIdx.x) * VEC;
  if (i >= F) return;
  const T* row = gu + (int64_t)t * gu_s0;
  T gv[VEC], uv[VEC], ov[VEC];
  *reinterpret_cast<float4_t*>(gv) =
      *reinterpret_cast<const float4_t*>(row + i);
  *reinterpret_cast<float4_t*>(uv) =
      *reinterpret_cast<const float4_t*>(row + F + i);
#pragma unroll
  for (int e = 0; e < VEC; e++) {
    const float g = fminf(act_ld(gv + e), limit);
    const float u = fminf(fmaxf(act_ld(uv + e), -limit), limit);
    act_st(ov + e, g * sigmoid_f(alpha * g) * (u + 1.0f));
  }
  *reinterpret_cast<float4_t*>(out + (int64_t)t * F + i) =
      *reinterpret_cast<const float4_t*>(ov);
}

template <typename T>
__global__ void sigmoid_mul_kernel(T* __restrict__ out,
                                   const T* __restrict__ x,
                                   const int64_t x_s0,
                                   const T* __restrict__ gate,
                                   const int64_t g_s0, const int N,
                                   const int rep) {
  const int t = blockIdx.y;
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= N) return;
  act_st(out + (int64_t)t * N + i,
         act_ld(x + (int64_t)t * x_s0 + i) *
             sigmoid_f(act_ld(gate + (int64_t)t * g_s0 + i / rep)));
}

// mode 0: gelu_tanh(in[i]) * in[F + i]; mode 1: relu(in[i])^2
template <typename T>
__global__ void unary_glu_kernel(T* __restrict__ out, const T* __restrict__ in,
                                 const int64_t in_s0, const int F,
                                 const int mode) {
  const int t = blockIdx.y;
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= F) return;
  const T* row = in + (int64_t)t * in_s0;
  const float a = act_ld(row + i);
  float r;
  if (mode == 0) r = gelu_tanh_f(a) * act_ld(row + F + i);
  else { const float m = fmaxf(a, 0.f); r = m * m; }
  act_st(out + (int64_t)t * F + i, r);
}

template <typename T>
__global__ void unary_glu_vec_kernel(T* __restrict__ out,
                                     const T* __restrict__ in,
                                     const int64_t in_s0, const int F,
                                     const int mode) {
  constexpr int VEC = 16 / (int)sizeof(T);
  const int t = blockIdx.y;
  const int i = (blockIdx.x * blockDim.x + threadIdx.x) * VEC;
  if (i >= F) return;
  const T* row = in + (int64_t)t * in_s0;
  T av[VEC], bv[VEC], ov[VEC];
  *reinterpret_cast<float4_t*>(av) =
      *reinterpret_cast<const float4_t*>(row + i);
  if (mode == 0)
    *reinterpret_cast<float4_t*>(bv) =
        *reinterpret_cast<const float4_t*>(row + F + i);
#pragma unroll
  for (int e = 0; e < VEC; e++) {
    const float a = act_ld(av + e);
    float r;
    if (mode == 0) r = gelu_tanh_f(a) * act_ld(bv + e);
    else { const float m = fmaxf(a, 0.f); r = m * m; }
    act_st(ov + e, r);
  }
  *reinterpret_cast<float4_t*>(out + (int64_t)t * F + i) =
      *reinterpret_cast<const float4_t*>(ov);
}

}  // namespace

void clamped_glu(at::Tensor out, at::Tensor gu, double limit, double alpha) {
  TORCH_CHECK(gu.is_cuda() && gu.dim() == 2 && gu.stride(1) == 1 &&
              is_act_dtype(gu) && gu.size(1) % 2 == 0);
  const int T = gu.size(0), F = gu.size(1) / 2;
  TORCH_CHECK(out.is_contiguous() && out.dtype() == gu.dtype() &&
              out.dim() == 2 && out.size(0) == T && out.size(1) == F);
  if (T == 0 || F == 0) return;
  TORCH_CHECK(T <= 65535 * 1024, "too many rows");
  auto stream = at::hip::getCurrentHIPStream();
  // rows beyond the grid's y limit are folded by looping on the host
  const int vec = 16 / (int)gu.element_size();
  const bool aligned = F % vec == 0 && gu.stride(0) % vec == 0 &&
      ((uintptr_t)gu.data_ptr()) % 16 == 0 &&
      ((uintptr_t)out.data_ptr()) % 16 == 0;
  for (int t0 = 0; t0 < T; t0 += 65535) {
    const int nt = std::min(65535, T - t0);
    KAITO_DISPATCH_ACT(gu, {
      if (aligned) {
        hipLaunchKernelGGL((clamped_glu_vec_kernel<act_t>),
            dim3((F / vec + 255) / 256, nt), dim3(256), 0, stream,
            (act_t*)out.data_ptr() + (int64_t)t0 * F,
            (const act_t*)gu.data_ptr() + (int64_t)t0 * gu.stride(0),
            gu.stride(0), F, (float)limit, (float)alpha);
      } else {
        hipLaunchKernelGGL((clamped_glu_kernel<act_t>),
            dim3((F + 255) / 256, nt), dim3(256), 0, stream,
            (act_t*)out.data_ptr() + (int64_t)t0 * F,
            (const act_t*)gu.data_ptr() + (int64_t)t0 * gu.stride(0),
            gu.stride(0), F, (float)limit, (float)alpha);
      }
    });
  }
}

void sigmoid_mul(at::Tensor out, at::Tensor x, at::Tensor gate) {
  TORCH_CHECK(x.is_cuda() && x.dim() == 2 && x.stride(1) == 1 &&
              is_act_dtype(x));
  TORCH_CHECK(gate.dim() == 2 && gate.stride(1) == 1 &&
              gate.size(0) == x.size(0) && gate.size(1) > 0 &&
              x.size(1) % gate.size(1) == 0 && gate.dtype() == x.dtype());
  TORCH_CHECK(out.is_contiguous() && out.dtype() == x.dtype() &&
              out.sizes() == x.sizes());
  const int T = x.size(0), N = x.size(1);
  if (T == 0 || N == 0) return;
  auto stream = at::hip::getCurrentHIPStream();
  for (int t0 = 0; t0 < T; t0 += 65535) {
    const int nt = std::min(65535, T - t0);
    KAITO_DISPATCH_ACT(x, {
      hipLaunchKernelGGL((sigmoid_mul_kernel<act_t>),
          dim3((N + 255) / 256, nt), dim3(256), 0, stream,
          (act_t*)out.data_ptr() + (int64_t)t0 * N,
          (const act_t*)x.data_ptr() + (int64_t)t0 * x.stride(0),
          x.stride(0),
          (const act_t*)gate.data_ptr() + (int64_t)t0 * gate.stride(0),
          gate.stride(0), N, N / (int)gate.size(1));
    });
  }
}

namespace {
void unary_glu(at::Tensor out, at::Tensor in, int F, int mode) {
  TORCH_CHECK(in.is_cuda() && in.dim() == 2 && in.stride(1) == 1 &&
              is_act_dtype(in));
  const int T = in.size(0);
  TORCH_CHECK(out.is_contiguous() && out.dtype() == in.dtype() &&
              out.dim() == 2 && out.size(0) == T && out.size(1) == F);
  if (T == 0 || F == 0) return;
  auto stream = at::hip::getCurrentHIPStream();
  const int vec = 16 / (int)in.element_size();
  const bool aligned = F % vec == 0 && in.stride(0) % vec == 0 &&
      ((uintptr_t)in.data_ptr()) % 16 == 0 &&
      ((uintptr_t)out.data_ptr()) % 16 == 0;
  for (int t0 = 0; t0 < T; t0 += 65535) {
    const int nt = std::min(65535, T - t0);
    KAITO_DISPATCH_ACT(in, {
      if (aligned) {
        hipLaunchKernelGGL((unary_glu_vec_kernel<act_t>),
            dim3((F / vec + 255) / 256, nt), dim3(256), 0, stream,
            (act_t*)out.data_ptr() + (int64_t)t0 * F,
            (const act_t*)in.data_ptr() + (int64_t)t0 * in.stride(0),
            in.stride(0), F, mode);
      } else {
        hipLaunchKernelGGL((unary_glu_kernel<act_t>),
            dim3((F + 255) / 256, nt), dim3(256), 0, stream,
            (act_t*)out.data_ptr() + (int64_t)t0 * F,
            (const act_t*)in.data_ptr() + (int64_t)t0 * in.stride(0),
            in.stride(0), F, mode);
      }
    });
  }
}
}  // namespace

void gelu_glu(at::Tensor out, at::Tensor gu) {
  TORCH_CHECK(gu.dim() == 2 && gu.size(1) % 2 == 0);
  unary_glu(out, gu, gu.size(1) / 2, 0);
}

void relu2(at::Tensor out, at::Tensor x) {
  TORCH_CHECK(x.dim() == 2);
  unary_glu(out, x, x.size(1), 1);
}

}  // namespace kaito

TORCH_LIBRARY_FRAGMENT(kaito, m) {
  m.def("clamped_glu(Tensor(a!) out, Tensor gu, float limit, float alpha) -> ()");
  m.def("sigmoid_mul(Tensor(a!) out, Tensor x, Tensor gate) -> ()");
  m.def("gelu_glu(Tensor(a!) out, Tensor gu) -> ()");
  m.def("relu2(Tensor(a!) out, Tensor x) -> ()");
}
TORCH_LIBRARY_IMPL(kaito, CUDA, m) {
  m.impl("clamped_glu", &kaito::clamped_glu);
  m.impl("sigmoid_mul", &kaito::sigmoid_mul);
  m.impl("gelu_glu", &kaito::gelu_glu);
  m.impl("relu2", &kaito::relu2);
}
