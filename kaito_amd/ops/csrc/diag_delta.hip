// Matrix-state recurrences with a decay per state ROW (key channel), for
// batches of chunks:
//
//   diag_delta_rule   S <- diag(w) S - (a*u)(u^T S) + k v^T,   o = S^T r
//                     u = k / sqrt(k.k + eps), w = exp(-rate*sigmoid(w_pre)),
//                     a = sigmoid(a_pre + a_bias); o / rms(o) per head, times a
//                     weight over all heads, times sigmoid(gate)
//   hgrn2_scan        S <- diag(f) S + (1 - f) v^T,            o = S^T q
//                     f = lower + (1 - lower) sigmoid(f_pre + f_bias),
//                     q = silu(q_pre);
//                     rms(o) over the value size with a shared weight
//
// Per head the state S is [D, V] f32 in a slot of its sequence. Both are
// one recurrence,  S <- diag(d) S - b (u^T S) + k v^T  (the second without
// the removal term), run by three launches:
//   1. prep (token-parallel, one wave per token and head): activations of
//      the gates, the unit key, and what lets the read-out be taken from
//      the state BEFORE the token:
//          S'^T r = S^T (r*d) - (u^T S)(r.b) + v (r.k)
//      so a token needs one reduction stage (u^T S and (r*d)^T S together).
//      Rows are written f32, zero-padded to the kernel's row count.
//   2. recurrence: a single-wave workgroup per (chunk, head, group of VB
//      state columns). Lane (column, part) keeps DP rows of its column in
//      registers; PARTS lanes share a column and meet in a DPP sum. Token
//      tiles are double-buffered through LDS: the next tile's loads (all
//      unconditional, the token index clamped) are issued before the current
//      tile is consumed and parked afterwards.
//   3. epilogue (token-parallel): head norm, weight, gate, store.
// A chunk that starts at position 0 starts from S = 0 whatever its slot
// held; slots < 0 are padding and skipped.
#include "mix_common.h"
#include <cstdlib>

namespace kaito {

namespace {


// ---- prep ---------------------------------------------------------------------
// scratch rows [T, H, DPAD]: u, rd (= r*d), d, b (= a*u), k; scalars [T, H]:
// rb = r.b, rk = r.k
template <typename T>
__global__ __launch_bounds__(64) void diag_delta_prep_kernel(
    float* __restrict__ su, float* __restrict__ srd, float* __restrict__ sd,
    float* __restrict__ sb, float* __restrict__ sk, float* __restrict__ srb,
    float* __restrict__ srk,
    const T* __restrict__ r, const int64_t r_s0, const int64_t r_s1,
    const T* __restrict__ k, const int64_t k_s0, const int64_t k_s1,
    const float* __restrict__ w_pre, const int64_t w_s0,
    const float* __restrict__ a_pre, const int64_t a_s0,
    const float* __restrict__ a_bias,                     // [H*D] or null
    const int H, const int D, const int DPAD, const float rate,
    const float k_eps) {
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const T* rr = r + (int64_t)t * r_s0 + (int64_t)h * r_s1;
  const T* kr = k + (int64_t)t * k_s0 + (int64_t)h * k_s1;
  const float* wr = w_pre + (int64_t)t * w_s0 + (int64_t)h * D;
  const float* ar = a_pre + (int64_t)t * a_s0 + (int64_t)h * D;
  const float* abr = a_bias ? a_bias + (int64_t)h * D : nullptr;
  float ss = 0.f;
  for (int i = lane; i < D; i += 64) {
    const float kv = act_ld(kr + i);
    ss += kv * kv;
  }
  ss = wave_reduce_sum(ss);
  const float inv = 1.0f / sqrtf(ss + k_eps);
  const int64_t o = ((int64_t)t * H + h) * DPAD;
  float rb = 0.f, rk = 0.f;
  for (int i = lane; i < DPAD; i += 64) {
    float u = 0.f, rd = 0.f, d = 0.f, b = 0.f, kv = 0.f;
    if (i < D) {
      kv = act_ld(kr + i);
      const float rv = act_ld(rr + i);
      u = kv * inv;
      d = expf(-rate * sigmoid_f(wr[i]));
      b = sigmoid_f(ar[i] + (abr ? abr[i] : 0.f)) * u;
      rd = rv * d;
      rb += rv * b;
      rk += rv * kv;
    }
    su[o + i] = u; srd[o + i] = rd; sd[o + i] = d; sb[o + i] = b;
    sk[o + i] = kv;
  }
  rb = wave_reduce_sum(rb);
  rk = wave_reduce_sum(rk);
  if (lane == 0) {
    srb[(int64_t)t * H + h] = rb;
    srk[(int64_t)t * H + h] = rk;
  }
}

// scratch rows: rd (= q*f), d (= f), k (= 1 - f); scalar rk = q.(1 - f)
template <typename T>
__global__ __launch_bounds__(64) void hgrn2_prep_kernel(
    float* __restrict__ srd, float* __restrict__ sd, float* __restrict__ sk,
    float* __restrict__ srk,
    const T* __restrict__ q, const int64_t q_s0, const int64_t q_s1,
    const float* __restrict__ f_pre, const int64_t f_s0,
    const float* __restrict__ f_bias,                     // [H*D] or null
    const float* __restrict__ lower, const int H, const int D,
    const int DPAD) {
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const T* qr = q + (int64_t)t * q_s0 + (int64_t)h * q_s1;
  const float* fr = f_pre + (int64_t)t * f_s0 + (int64_t)h * D;
  const float* lr = lower + (int64_t)h * D;
  const float* fbr = f_bias ? f_bias + (int64_t)h * D : nullptr;
  const int64_t o = ((int64_t)t * H + h) * DPAD;
  float rk = 0.f;
  for (int i = lane; i < DPAD; i += 64) {
    float rd = 0.f, d = 0.f, kv = 0.f;
    if (i < D) {
      const float lo = lr[i];
      d = lo + (1.0f - lo) * sigmoid_f(fr[i] + (fbr ? fbr[i] : 0.f));
      kv = 1.0f - d;
      const float qv = silu_f(act_ld(qr + i));
      rd = qv * d;
      rk += qv * kv;
    }
    srd[o + i] = rd; sd[o + i] = d; sk[o + i] = kv;
  }
  rk = wave_reduce_sum(rk);
  if (lane == 0) srk[(int64_t)t * H + h] = rk;
}

// ---- recurrence ----------------------------------------------------------------
// TT = tokens per LDS tile
template <typename T, int DP, int PARTS, bool REMOVE, int TT>
__global__ __launch_bounds__(64) void diag_recurrence_kernel(
    float* __restrict__ o,                                 // [T, H, V]
    const float* __restrict__ su, const float* __restrict__ srd,
    const float* __restrict__ sd, const float* __restrict__ sb,
    const float* __restrict__ sk,                          // [T, H, DPAD]
    const float* __restrict__ srb, const float* __restrict__ srk,  // [T, H]
    const T* __restrict__ v, const int64_t v_s0, const int64_t v_s1,
    float* __restrict__ state,                             // [slots, H, D, V]
    const int* __restrict__ cu, const int* __restrict__ slots,
    const int* __restrict__ starts, const int D, const int H, const int V) {
  constexpr int VB = 64 / PARTS;
  constexpr int DPAD = DP * PARTS;
  constexpr int NV = REMOVE ? 5 : 3;          // vectors per token
  // each part's DP-slice is followed by 4 floats of padding, so that the
  // PARTS slices read by one instruction do not share banks
  constexpr int DPS = DP + 4;
  constexpr int VROW = PARTS * DPS;
  constexpr int ROW = NV * VROW + VB + 4;     // vectors | v | rb rk - -
  constexpr int N4 = TT * DPAD / 4 / 64;      // float4 loads per lane, vector
  static_assert(TT * DPAD / 4 % 64 == 0, "tile must divide over the wave");
  constexpr int VN = (TT * VB + 63) / 64;
  __shared__ __attribute__((aligned(16))) float lds[2][TT * ROW];
  const int b = blockIdx.x, h = blockIdx.y;
  const int slot = slots[b];
  const int r0 = cu[b], r1 = cu[b + 1];
  if (slot < 0 || r1 <= r0) return;
  const int tid = threadIdx.x;
  const int part = tid % PARTS;
  const int jl = tid / PARTS;                 // column inside the group
  const int j = blockIdx.z * VB + jl;
  const bool live = j < V;
  const int d0 = part * DP;
  float S[DP];
  float* sp = state + (((int64_t)slot * H + h) * D) * V + (live ? j : 0);
  const bool carried = starts[b] > 0;
#pragma unroll
  for (int i = 0; i < DP; i++) {
    const int d = d0 + i;
    S[i] = (carried && live && d < D) ? sp[(int64_t)d * V] : 0.0f;
  }

  const float* vecs[5] = {srd, sd, sk, su, sb};
  float4_t rg[NV][N4];
  float rv[VN], rs = 0.f;
  auto fetch = [&](int t0) {
#pragma unroll
    for (int n = 0; n < NV; n++)
#pragma unroll
      for (int i = 0; i < N4; i++) {
        const int e = tid + i * 64;
        const int tt = e / (DPAD / 4), d = (e % (DPAD / 4)) * 4;
        const int t = min(t0 + tt, r1 - 1);
        rg[n][i] = *reinterpret_cast<const float4_t*>(
            vecs[n] + ((int64_t)t * H + h) * DPAD + d);
      }
#pragma unroll
    for (int i = 0; i < VN; i++) {
      const int e = tid + i * 64;
      const int tt = min(e / VB, TT - 1);
      const int c = min((int)blockIdx.z * VB + e % VB, V - 1);
      const int t = min(t0 + tt, r1 - 1);
      rv[i] = act_ld(v + (int64_t)t * v_s0 + (int64_t)h * v_s1 + c);
    }
    if (tid < 2 * TT) {
      const int t = min(t0 + tid / 2, r1 - 1);
      rs = ((tid & 1) ? srk : (REMOVE ? srb : srk))[(int64_t)t * H + h];
    }
  };
  auto park = [&](float* buf) {
#pragma unroll
    for (int n = 0; n < NV; n++)
#pragma unroll
      for (int i = 0; i < N4; i++) {
        const int e = tid + i * 64;
        const int tt = e / (DPAD / 4), d = (e % (DPAD / 4)) * 4;
        const int dd = (d / DP) * DPS + d % DP;
        *reinterpret_cast<float4_t*>(buf + tt * ROW + n * VROW + dd) =
            rg[n][i];
      }
#pragma unroll
    for (int i = 0; i < VN; i++) {
      const int e = tid + i * 64;
      if (e < TT * VB) buf[(e / VB) * ROW + NV * VROW + e % VB] = rv[i];
    }
    if (tid < 2 * TT)
      buf[(tid / 2) * ROW + NV * VROW + VB + (tid & 1)] = rs;
  };

  fetch(r0);
  park(lds[0]);
  __syncthreads();
  int cur = 0;
  for (int t0 = r0; t0 < r1; t0 += TT) {
    const int nt = min(TT, r1 - t0);
    const bool more = t0 + TT < r1;
    if (more) fetch(t0 + TT);
    const float* buf = lds[cur];
    for (int tt = 0; tt < nt; tt++) {
      const float* base = buf + tt * ROW + part * DPS;
      const float* lrd = base;
      const float* ld = base + VROW;
      const float* lk = base + 2 * VROW;
      const float rb = buf[tt * ROW + NV * VROW + VB];
      const float rk = buf[tt * ROW + NV * VROW + VB + 1];
      const float vj = buf[tt * ROW + NV * VROW + jl];
      float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
      float p0 = 0.f, p1 = 0.f, p2 = 0.f, p3 = 0.f;
#pragma unroll
      for (int i = 0; i < DP; i += 4) {
        const float4_t q4 = *reinterpret_cast<const float4_t*>(lrd + i);
        a0 += S[i] * q4[0]; a1 += S[i + 1] * q4[1];
        a2 += S[i + 2] * q4[2]; a3 += S[i + 3] * q4[3];
        if constexpr (REMOVE) {
          const float4_t u4 =
              *reinterpret_cast<const float4_t*>(base + 3 * VROW + i);
          p0 += S[i] * u4[0]; p1 += S[i + 1] * u4[1];
          p2 += S[i + 2] * u4[2]; p3 += S[i + 3] * u4[3];
        }
      }
      const float sa = group_reduce_sum<PARTS>((a0 + a1) + (a2 + a3));
      float oj = sa + vj * rk;
      float pr = 0.f;
      if constexpr (REMOVE) {
        pr = group_reduce_sum<PARTS>((p0 + p1) + (p2 + p3));
        oj -= pr * rb;
      }
#pragma unroll
      for (int i = 0; i < DP; i += 4) {
        const float4_t d4 = *reinterpret_cast<const float4_t*>(ld + i);
        const float4_t k4 = *reinterpret_cast<const float4_t*>(lk + i);
        if constexpr (REMOVE) {
          const float4_t b4 =
              *reinterpret_cast<const float4_t*>(base + 4 * VROW + i);
          S[i] = d4[0] * S[i] - b4[0] * pr + k4[0] * vj;
          S[i + 1] = d4[1] * S[i + 1] - b4[1] * pr + k4[1] * vj;
          S[i + 2] = d4[2] * S[i + 2] - b4[2] * pr + k4[2] * vj;
          S[i + 3] = d4[3] * S[i + 3] - b4[3] * pr + k4[3] * vj;
        } else {
          S[i] = d4[0] * S[i] + k4[0] * vj;
          S[i + 1] = d4[1] * S[i + 1] + k4[1] * vj;
          S[i + 2] = d4[2] * S[i + 2] + k4[2] * vj;
          S[i + 3] = d4[3] * S[i + 3] + k4[3] * vj;
        }
      }
      if (live && part == 0)
        o[((int64_t)(t0 + tt) * H + h) * V + j] = oj;
    }
    if (more) park(lds[cur ^ 1]);
    __syncthreads();
    cur ^= 1;
  }
  if (live) {
#pragma unroll
    for (int i = 0; i < DP; i++) {
      const int d = d0 + i;
      if (d < D) sp[(int64_t)d * V] = S[i];
    }
  }
}

// ---- epilogue ------------------------------------------------------------------
// one wave per (token, head): o / sqrt(mean(o^2) + eps) * w * sigmoid(gate);
// w is indexed over all heads (w_stride = V) or shared by them (0)
template <typename T>
__global__ __launch_bounds__(64) void diag_epilogue_kernel(
    T* __restrict__ out,                                   // [T, H*V]
    const float* __restrict__ o,                           // [T, H, V]
    const T* __restrict__ gate, const int64_t g_s0, const int64_t g_s1,
    const float* __restrict__ w, const int w_stride, const int H, const int V,
    const float eps) {
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const float* orow = o + ((int64_t)t * H + h) * V;
  float ss = 0.f;
  for (int i = lane; i < V; i += 64) ss += orow[i] * orow[i];
  ss = wave_reduce_sum(ss);
  const float inv = 1.0f / sqrtf(ss / (float)V + eps);
  const float* wr = w + (int64_t)h * w_stride;
  const T* gr = gate ? gate + (int64_t)t * g_s0 + (int64_t)h * g_s1 : nullptr;
  T* dst = out + ((int64_t)t * H + h) * V;
  for (int i = lane; i < V; i += 64) {
    float y = orow[i] * inv * wr[i];
    if (gr) y *= sigmoid_f(act_ld(gr + i));
    act_st(dst + i, y);
  }
}

struct ChunkArgs {
  const int* cu; const int* slots; const int* starts; int B;
};

ChunkArgs check_chunks(const at::Tensor& cu, const at::Tensor& slots,
                       const at::Tensor& starts, int T) {
  KAITO_CHECK_I32(cu); KAITO_CHECK_I32(slots); KAITO_CHECK_I32(starts);
  const int B = slots.numel();
  TORCH_CHECK(cu.numel() == B + 1 && starts.numel() == B);
  return {cu.data_ptr<int>(), slots.data_ptr<int>(), starts.data_ptr<int>(),
          B};
}

void check_heads(const at::Tensor& x, int T, int H, int D, const char* what) {
  TORCH_CHECK(x.is_cuda() && x.dim() == 3 && x.size(0) == T &&
              x.size(1) == H && x.size(2) == D && x.stride(2) == 1, what,
              ": expected [T, heads, dim] with unit inner stride");
}

// rows per lane and lanes per column for a state of D rows
inline int padded_rows(int D) {
  return D <= 32 ? 32 : (D <= 64 ? 64 : (D <= 128 ? 128 : 256));
}

template <typename T, bool REMOVE>
void launch_recurrence(hipStream_t stream, int B, int H, int D, int V,
                       float* o, const float* su, const float* srd,
                       const float* sd, const float* sb, const float* sk,
                       const float* srb, const float* srk, const T* v,
                       int64_t v_s0, int64_t v_s1, float* state,
                       const ChunkArgs& c) {
#define KAITO_DD_CASE(DP_, PARTS_, TTR_, TTP_)                                \
  if (dp == DP_ && parts == PARTS_) {                                         \
    constexpr int VB = 64 / PARTS_;                                           \
    constexpr int TT_ = REMOVE ? TTR_ : TTP_;                                 \
    hipLaunchKernelGGL(                                                       \
        (diag_recurrence_kernel<T, DP_, PARTS_, REMOVE, TT_>),                \
        dim3(B, H, (V + VB - 1) / VB), dim3(64), 0, stream, o, su, srd, sd,   \
        sb, sk, srb, srk, v, v_s0, v_s1, state, c.cu, c.slots, c.starts, D,   \
        H, V);                                                                \
    return;                                                                   \
  }
  // 32 rows per lane; a wave64 VALU instruction occupies its SIMD for four
  // cycles and the token loop is serial, so with few (chunk, head, column
  // group) triples the rows per lane are halved to double the waves.
  // Tokens per tile (with / without the removal term, which stages five
  // instead of three rows per token): as many as keep both LDS buffers of
  // a single-wave workgroup small enough for a CU to hold at least four
  // (one per SIMD); decode-sized steps take the shortest tile.
  int dp = 32, parts = padded_rows(D) / 32;
  const int64_t waves32 = (int64_t)B * H * ((V * parts + 63) / 64);
  // KAITO_DIAG_ROWS_PER_LANE=16|32 pins the choice (A/B runs, tests)
  const char* pin = getenv("KAITO_DIAG_ROWS_PER_LANE");
  const int want = pin ? atoi(pin) : (waves32 < 4096 ? 16 : 32);
  if (want == 16) { dp = 16; parts *= 2; }
  KAITO_DD_CASE(32, 1, 8, 8) KAITO_DD_CASE(32, 2, 4, 4)
  KAITO_DD_CASE(32, 4, 2, 2) KAITO_DD_CASE(32, 8, 1, 1)
  KAITO_DD_CASE(16, 2, 8, 8) KAITO_DD_CASE(16, 4, 8, 8)
  KAITO_DD_CASE(16, 8, 6, 8) KAITO_DD_CASE(16, 16, 3, 4)
  TORCH_CHECK(false, "diag recurrence: no kernel for ", D, " state rows");
#undef KAITO_DD_CASE
}

}  // namespace

void diag_delta_rule(at::Tensor out, at::Tensor r, at::Tensor k, at::Tensor v,
                     at::Tensor w_pre, at::Tensor a_pre, at::Tensor a_bias,
                     at::Tensor gate, at::Tensor norm_w, at::Tensor state, at::Tensor cu_seqlens,
                     at::Tensor state_slots, at::Tensor seq_starts,
                     double decay_rate, double k_eps, double norm_eps) {
  TORCH_CHECK(r.is_cuda() && r.dim() == 3 && is_act_dtype(r));
  const int T = r.size(0), H = r.size(1), D = r.size(2);
  TORCH_CHECK(D >= 1 && D <= 256, "state rows per head: 1..256, got ", D);
  check_heads(r, T, H, D, "r"); check_heads(k, T, H, D, "k");
  check_heads(v, T, H, D, "v"); check_heads(gate, T, H, D, "gate");
  TORCH_CHECK(k.dtype() == r.dtype() && v.dtype() == r.dtype() &&
              gate.dtype() == r.dtype());
  auto check_pre = [&](const at::Tensor& p) {
    TORCH_CHECK(p.is_cuda() && p.dtype() == at::kFloat && p.dim() == 2 &&
                p.size(0) == T && p.size(1) == H * D && p.stride(1) == 1,
                "gate pre-activations: f32 [T, heads*dim]");
  };
  check_pre(w_pre); check_pre(a_pre);
  const bool ab = a_bias.numel() > 0;
  if (ab) { KAITO_CHECK_F32(a_bias); TORCH_CHECK(a_bias.numel() == H * D); }
  KAITO_CHECK_F32(norm_w); KAITO_CHECK_F32(state);
  TORCH_CHECK(norm_w.numel() == H * D);
  TORCH_CHECK(state.dim() == 4 && state.size(1) == H && state.size(2) == D &&
              state.size(3) == D);
  TORCH_CHECK(out.is_contiguous() && out.dtype() == r.dtype() &&
              out.dim() == 2 && out.size(0) == T && out.size(1) == H * D);
  const ChunkArgs c = check_chunks(cu_seqlens, state_slots, seq_starts, T);
  if (T == 0) return;
  auto stream = at::hip::getCurrentHIPStream();
  const int DPAD = padded_rows(D);
  auto f32 = r.options().dtype(at::kFloat);
  at::Tensor vec = at::empty({5, T, H, DPAD}, f32);
  at::Tensor sca = at::empty({2, T, H}, f32);
  at::Tensor o = at::empty({T, H, D}, f32);
  float* vp = vec.data_ptr<float>();
  const int64_t vs = (int64_t)T * H * DPAD;
  float* su = vp, *srd = vp + vs, *sd = vp + 2 * vs, *sb = vp + 3 * vs,
      *sk = vp + 4 * vs;
  float* srb = sca.data_ptr<float>(), *srk = srb + (int64_t)T * H;
  KAITO_DISPATCH_ACT(r, {
    hipLaunchKernelGGL((diag_delta_prep_kernel<act_t>), dim3(T, H), dim3(64),
        0, stream, su, srd, sd, sb, sk, srb, srk,
        (const act_t*)r.data_ptr(), r.stride(0), r.stride(1),
        (const act_t*)k.data_ptr(), k.stride(0), k.stride(1),
        w_pre.data_ptr<float>(), w_pre.stride(0), a_pre.data_ptr<float>(),
        a_pre.stride(0), ab ? a_bias.data_ptr<float>() : nullptr, H, D, DPAD,
        (float)decay_rate, (float)k_eps);
    launch_recurrence<act_t, true>(stream, c.B, H, D, D,
        o.data_ptr<float>(), su, srd, sd, sb, sk, srb, srk,
        (const act_t*)v.data_ptr(), v.stride(0), v.stride(1),
        state.data_ptr<float>(), c);
    hipLaunchKernelGGL((diag_epilogue_kernel<act_t>), dim3(T, H), dim3(64),
        0, stream, (act_t*)out.data_ptr(), o.data_ptr<float>(),
        (const act_t*)gate.data_ptr(), gate.stride(0), gate.stride(1),
        norm_w.data_ptr<float>(), D, H, D, (float)norm_eps);
  });
}

void hgrn2_scan(at::Tensor out, at::Tensor q, at::Tensor v, at::Tensor f_pre,
                at::Tensor f_bias, at::Tensor lower, at::Tensor norm_w, at::Tensor state,
                at::Tensor cu_seqlens, at::Tensor state_slots,
                at::Tensor seq_starts, double norm_eps) {
  TORCH_CHECK(q.is_cuda() && q.dim() == 3 && is_act_dtype(q) &&
              v.dim() == 3);
  const int T = q.size(0), H = q.size(1), D = q.size(2), V = v.size(2);
  TORCH_CHECK(D >= 1 && D <= 256, "state rows per head: 1..256, got ", D);
  check_heads(q, T, H, D, "q"); check_heads(v, T, H, V, "v");
  TORCH_CHECK(v.dtype() == q.dtype());
  TORCH_CHECK(f_pre.is_cuda() && f_pre.dtype() == at::kFloat &&
              f_pre.dim() == 2 && f_pre.size(0) == T &&
              f_pre.size(1) == H * D && f_pre.stride(1) == 1,
              "gate pre-activations: f32 [T, heads*dim]");
  KAITO_CHECK_F32(lower); KAITO_CHECK_F32(norm_w); KAITO_CHECK_F32(state);
  TORCH_CHECK(lower.numel() == H * D && norm_w.numel() == V);
  const bool fb = f_bias.numel() > 0;
  if (fb) { KAITO_CHECK_F32(f_bias); TORCH_CHECK(f_bias.numel() == H * D); }
  TORCH_CHECK(state.dim() == 4 && state.size(1) == H && state.size(2) == D &&
              state.size(3) == V);
  TORCH_CHECK(out.is_contiguous() && out.dtype() == q.dtype() &&
              out.dim() == 2 && out.size(0) == T && out.size(1) == H * V);
  const ChunkArgs c = check_chunks(cu_seqlens, state_slots, seq_starts, T);
  if (T == 0) return;
  auto stream = at::hip::getCurrentHIPStream();
  const int DPAD = padded_rows(D);
  auto f32 = q.options().dtype(at::kFloat);
  at::Tensor vec = at::empty({3, T, H, DPAD}, f32);
  at::Tensor sca = at::empty({T, H}, f32);
  at::Tensor o = at::empty({T, H, V}, f32);
  float* vp = vec.data_ptr<float>();
  const int64_t vs = (int64_t)T * H * DPAD;
  float* srd = vp, *sd = vp + vs, *sk = vp + 2 * vs;
  float* srk = sca.data_ptr<float>();
  KAITO_DISPATCH_ACT(q, {
    hipLaunchKernelGGL((hgrn2_prep_kernel<act_t>), dim3(T, H), dim3(64), 0,
        stream, srd, sd, sk, srk, (const act_t*)q.data_ptr(), q.stride(0),
        q.stride(1), f_pre.data_ptr<float>(), f_pre.stride(0),
        fb ? f_bias.data_ptr<float>() : nullptr, lower.data_ptr<float>(), H,
        D, DPAD);
    launch_recurrence<act_t, false>(stream, c.B, H, D, V,
        o.data_ptr<float>(), nullptr, srd, sd, nullptr, sk, nullptr, srk,
        (const act_t*)v.data_ptr(), v.stride(0), v.stride(1),
        state.data_ptr<float>(), c);
    hipLaunchKernelGGL((diag_epilogue_kernel<act_t>), dim3(T, H), dim3(64),
        0, stream, (act_t*)out.data_ptr(), o.data_ptr<float>(),
        (const act_t*)nullptr, (int64_t)0, (int64_t)0,
        norm_w.data_ptr<float>(), 0, H, V, (float)norm_eps);
  });
}

}  // namespace kaito

TORCH_LIBRARY_FRAGMENT(kaito, m) {
  m.def("diag_delta_rule(Tensor(a!) out, Tensor r, Tensor k, Tensor v, Tensor w_pre, Tensor a_pre, Tensor a_bias, Tensor gate, Tensor norm_w, Tensor(b!) state, Tensor cu_seqlens, Tensor state_slots, Tensor seq_starts, float decay_rate, float k_eps, float norm_eps) -> ()");
  m.def("hgrn2_scan(Tensor(a!) out, Tensor q, Tensor v, Tensor f_pre, Tensor f_bias, Tensor lower, Tensor norm_w, Tensor(b!) state, Tensor cu_seqlens, Tensor state_slots, Tensor seq_starts, float norm_eps) -> ()");
}
TORCH_LIBRARY_IMPL(kaito, CUDA, m) {
  m.impl("diag_delta_rule", &kaito::diag_delta_rule);
  m.impl("hgrn2_scan", &kaito::hgrn2_scan);
}
