// Softmax attention over a sliding window of the paged K/V cache with a
// distance penalty, for batches of chunks (prompt portions and single
// decode tokens alike), plus the fused per-head qk RMS norm + cache write.
//
//   score(i, j) = cap * tanh(q_i . k_j * scale / cap)      (cap > 0)
//                 - r1_h * ln(1 + r2_h * (i - j))           (r1 given)
//   visible:      j <= i and (i - j < window or j < keep_first)
//                 (window <= 0: every j <= i); or, with chunk > 0,
//                 j <= i and floor(j / chunk) == floor(i / chunk) on
//                 absolute sequence positions
//   sinks:        with sink_h given, exp(sink_h) joins the softmax
//                 denominator (no key, no value): the running maximum
//                 starts at sink_h and the running sum at 1
//
// The q/k norm kernel optionally rotates the first 2R dims of every head
// (dim i paired with i + R, angle = position * inv_freq[i], all f32) and
// blends v with another layer's values before the cache write.
//
// Key size D and value size V are independent; caches are
// [blocks, G, block_size, D|V] in the activation dtype. Scores, softmax
// weights and the output accumulation are f32.
//
// Three kernels share these semantics:
//   window_attention_mfma_kernel   bf16 prompt portions, 64-row query tiles
//   window_attention_decode_kernel single rows (and f32 portions), the
//                                  heads of a kv group in one pass
//   window_attention_kernel        any sizes: one workgroup per (row, head),
//                                  one thread scores one key, the tile's
//                                  weights go through LDS, P.V is
//                                  thread-per-value-dim
// All fold key tiles with the running-max (online softmax) recurrence, so
// any window length works.
#include "mix_common.h"

namespace kaito {

namespace {

// ---- q/k norm (+ rotation) + cache scatter (+ value blend) ----------------
// grid (T, H + 2G): blockIdx.y < H → q head; < H+G → k head; else v head.
template <typename T>
KAITO_DEV void norm_rotate_row(T* __restrict__ dst, const T* __restrict__ src,
                               const float* __restrict__ w, const float eps,
                               const int D, const float* __restrict__ inv_freq,
                               const int R, const float pos,
                               const float rot_mag, const int lane) {
  float inv = 1.0f;
  if (w != nullptr) {
    float ss = 0.f;
    for (int d = lane; d < D; d += 64) { const float x = act_ld(src + d); ss += x * x; }
    ss = wave_reduce_sum(ss);
    inv = 1.0f / sqrtf(ss / (float)D + eps);
  }
  for (int d = lane; d < D; d += 64) {
    float val;
    if (d < 2 * R) {
      const int i = d < R ? d : d - R;
      const float a = act_ld(src + i) * inv * (w ? w[i] : 1.0f);
      const float b = act_ld(src + i + R) * inv * (w ? w[i + R] : 1.0f);
      const float ang = pos * inv_freq[i];
      const float c = cosf(ang) * rot_mag, sn = sinf(ang) * rot_mag;
      val = d < R ? a * c - b * sn : b * c + a * sn;
    } else {
      val = act_ld(src + d) * inv * (w ? w[d] : 1.0f);
    }
    act_st(dst + d, val);
  }
}

template <typename T>
__global__ void qk_norm_cache_write_kernel(
    T* __restrict__ q_out,                                   // [T, H, D]
    const T* __restrict__ q, const int64_t q_s0, const int64_t q_s1,
    const T* __restrict__ k, const int64_t k_s0, const int64_t k_s1,
    const T* __restrict__ v, const int64_t v_s0, const int64_t v_s1,
    const float* __restrict__ q_w, const float* __restrict__ k_w,
    const float eps, T* __restrict__ k_cache, T* __restrict__ v_cache,
    const int64_t* __restrict__ slots, const int H, const int G, const int D,
    const int V, const int BS, const int64_t* __restrict__ positions,
    const float* __restrict__ inv_freq, const int R, const float rot_mag,
    const T* __restrict__ v_first, const int64_t vf_s0, const int64_t vf_s1,
    const float v_lambda) {
  const int t = blockIdx.x, y = blockIdx.y, lane = threadIdx.x;
  const float pos = R > 0 ? (float)positions[t] : 0.0f;
  if (y < H) {
    norm_rotate_row(q_out + ((int64_t)t * H + y) * D,
                    q + (int64_t)t * q_s0 + (int64_t)y * q_s1, q_w, eps, D,
                    inv_freq, R, pos, rot_mag, lane);
    return;
  }
  const int64_t slot = slots[t];
  if (slot < 0) return;
  const int64_t blk = slot / BS;
  const int off = (int)(slot % BS);
  if (y < H + G) {
    const int g = y - H;
    norm_rotate_row(k_cache + ((blk * G + g) * BS + off) * D,
                    k + (int64_t)t * k_s0 + (int64_t)g * k_s1, k_w, eps, D,
                    inv_freq, R, pos, rot_mag, lane);
  } else {
    const int g = y - H - G;
    const T* src = v + (int64_t)t * v_s0 + (int64_t)g * v_s1;
    T* dst = v_cache + ((blk * G + g) * BS + off) * V;
    if (v_first != nullptr) {
      const T* vf = v_first + (int64_t)t * vf_s0 + (int64_t)g * vf_s1;
      for (int d = lane; d < V; d += 64)
        act_st(dst + d, (1.0f - v_lambda) * act_ld(src + d) +
                            v_lambda * act_ld(vf + d));
    } else {
      for (int d = lane; d < V; d += 64) dst[d] = src[d];
    }
  }
}

// ---- attention ------------------------------------------------------------
template <typename T>
KAITO_DEV float dot_row(const float* __restrict__ q, const T* __restrict__ k,
                        const int D);

template <>
KAITO_DEV float dot_row<float>(const float* __restrict__ q,
                               const float* __restrict__ k, const int D) {
  float acc = 0.f;
  int d = 0;
  if ((((uintptr_t)k) & 15) == 0) {
    for (; d + 4 <= D; d += 4) {
      const float4_t kv = *reinterpret_cast<const float4_t*>(k + d);
      acc += q[d] * kv[0] + q[d + 1] * kv[1] + q[d + 2] * kv[2] +
             q[d + 3] * kv[3];
    }
  }
  for (; d < D; d++) acc += q[d] * k[d];
  return acc;
}

template <>
KAITO_DEV float dot_row<bf16_act>(const float* __restrict__ q,
                                  const bf16_act* __restrict__ k,
                                  const int D) {
  float acc = 0.f;
  int d = 0;
  if ((((uintptr_t)k) & 15) == 0) {
    for (; d + 8 <= D; d += 8) {
      const short8_t kv = *reinterpret_cast<const short8_t*>(k + d);
#pragma unroll
      for (int i = 0; i < 8; i++) acc += q[d + i] * bf16_to_f32(kv[i]);
    }
  }
  for (; d < D; d++) acc += q[d] * bf16_to_f32(k[d].v);
  return acc;
}

template <typename T>
__global__ void window_attention_kernel(
    T* __restrict__ out,                                   // [T, H, V]
    const T* __restrict__ q,                               // [T, H, D]
    const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const int* __restrict__ block_tables, const int max_blocks,
    const int* __restrict__ token_seq, const int64_t* __restrict__ positions,
    const float scale, const float softcap, const float* __restrict__ r1,
    const float* __restrict__ r2, const int window, const int H, const int G,
    const int D, const int V, const int BS, const int keep_first,
    const float* __restrict__ sinks, const int chunk) {
  extern __shared__ float lds[];
  const int KT = blockDim.x;            // keys per tile
  float* q_s = lds;                     // [D]
  float* p_s = lds + D;                 // [KT]
  int* blk_s = reinterpret_cast<int*>(p_s + KT);   // [KT] cache row bases
  __shared__ float red[16];
  __shared__ float bcast[2];

  const int t = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int b = token_seq[t];
  T* orow = out + ((int64_t)t * H + h) * V;
  if (b < 0) {
    for (int j = tid; j < V; j += KT) act_st(orow + j, 0.0f);
    return;
  }
  const int g = h / (H / G);
  const int pos = (int)positions[t];
  const int lo = chunk > 0 ? (pos / chunk) * chunk
      : (window > 0 ? max(0, pos - window + 1) : 0);
  const int nfirst = min(keep_first, lo);       // kept keys before the window
  const int nkeys = nfirst + pos - lo + 1;
  const int* bt = block_tables + (int64_t)b * max_blocks;
  const float hr1 = r1 ? r1[h] : 0.0f, hr2 = r1 ? r2[h] : 0.0f;

  for (int d = tid; d < D; d += KT)
    q_s[d] = act_ld(q + ((int64_t)t * H + h) * D + d);

  // output dims owned by this thread: j = tid + i*KT
  constexpr int MAXV = 4;               // V <= 4 * blockDim
  float acc[MAXV];
#pragma unroll
  for (int i = 0; i < MAXV; i++) acc[i] = 0.f;
  float m_run = sinks ? sinks[h] : -INFINITY, l_run = sinks ? 1.0f : 0.f;

  for (int k0 = 0; k0 < nkeys; k0 += KT) {
    const int nk = min(KT, nkeys - k0);
    __syncthreads();                    // q_s ready / previous tile consumed
    float s = -INFINITY;
    if (tid < nk) {
      const int kx = k0 + tid;
      const int j = kx < nfirst ? kx : lo + (kx - nfirst);
      const int page = bt[j / BS];
      const int64_t rowi = ((int64_t)page * G + g) * BS + (j % BS);
      blk_s[tid] = (int)rowi;
      s = dot_row<T>(q_s, k_cache + rowi * D, D) * scale;
      if (softcap > 0.f) s = softcap * tanhf(s / softcap);
      if (r1) s -= hr1 * log1pf(hr2 * (float)(pos - j));
    }
    // tile max
    float mx = wave_reduce_max(s);
    if ((tid & 63) == 0) red[tid >> 6] = mx;
    __syncthreads();
    if (tid == 0) {
      float m = red[0];
      for (int w = 1; w < (KT >> 6); w++) m = fmaxf(m, red[w]);
      bcast[0] = m;
    }
    __syncthreads();
    const float m_new = fmaxf(m_run, bcast[0]);
    const float p = tid < nk ? expf(s - m_new) : 0.f;
    p_s[tid] = p;
    float ps = wave_reduce_sum(p);
    __syncthreads();                    // red[] free again; p_s visible
    if ((tid & 63) == 0) red[tid >> 6] = ps;
    __syncthreads();
    float tile_sum = 0.f;
    for (int w = 0; w < (KT >> 6); w++) tile_sum += red[w];
    const float corr = expf(m_run - m_new);     // 0 on the first tile
    l_run = l_run * corr + tile_sum;
    m_run = m_new;
#pragma unroll
    for (int i = 0; i < MAXV; i++) {
      const int j = tid + i * KT;
      if (j < V) {
        float a = acc[i] * corr;
        for (int kk = 0; kk < nk; kk++)
          a += p_s[kk] * act_ld(v_cache + (int64_t)blk_s[kk] * V + j);
        acc[i] = a;
      }
    }
  }
  const float inv = 1.0f / l_run;
#pragma unroll
  for (int i = 0; i < MAXV; i++) {
    const int j = tid + i * KT;
    if (j < V) act_st(orow + j, acc[i] * inv);
  }
}

// ---- MFMA prompt-portion kernel (bf16) -------------------------------------
// One workgroup = 64 query rows of one chunk x one head; 4 waves x 16 rows.
// Keys come 32 at a time through LDS: the K tile XOR-swizzled for
// conflict-free 16-byte fragment reads, the V tile transposed so the P.V
// B-fragments are contiguous. S = Q K^T and O += P V run on
// v_mfma_f32_16x16x32_bf16; scaling, capping, the distance penalty, the
// window/causal mask and the online softmax are f32 on the accumulator
// fragments; the f32 weights enter the P.V product as a bf16 value +
// remainder pair. Key and value sizes are separate template parameters.
constexpr int WQ_TILE = 64;
constexpr int WKV_TILE = 32;
constexpr int WPAD = 40;

template <int D, int DV>
__global__ __launch_bounds__(256, 2) void window_attention_mfma_kernel(
    short* __restrict__ out,              // [T, H, DV]
    const short* __restrict__ q,          // [T, H, D]
    const short* __restrict__ k_cache,    // [blocks, G, BS, D]
    const short* __restrict__ v_cache,    // [blocks, G, BS, DV]
    const int* __restrict__ tile_seq, const int* __restrict__ tile_qbase,
    const int* __restrict__ cu, const int* __restrict__ starts,
    const int* __restrict__ block_tables, const int max_blocks,
    const float scale, const float softcap, const float* __restrict__ r1,
    const float* __restrict__ r2, const int window, const int H, const int G,
    const int BS, const int keep_first, const float* __restrict__ sinks,
    const int chunk) {
  constexpr int KK = D / 32;
  constexpr int DT = DV / 16;
  const int tile = blockIdx.x;
  const int h = blockIdx.y;
  const int g = h / (H / G);
  const int seq = tile_seq[tile];
  const int q0 = tile_qbase[tile];
  const int tok0 = cu[seq];
  const int q_len = cu[seq + 1] - tok0;
  const int q_abs0 = starts[seq];          // position of the chunk's row 0
  const int kv_len = q_abs0 + q_len;
  const int* bt = block_tables + (int64_t)seq * max_blocks;
  const float hr1 = r1 ? r1[h] : 0.f, hr2 = r1 ? r2[h] : 0.f;
  const float inv_cap = softcap > 0.f ? 1.0f / softcap : 0.f;

  const int wave = threadIdx.x >> 6;
  const int lane = threadIdx.x & 63;
  const int hi = lane >> 4;
  const int lo = lane & 15;

  __shared__ short lds_k[WKV_TILE * D];
  __shared__ short lds_vt[DV * WPAD];
  // softmax weights as a bf16 pair (value + remainder): two MFMAs per value
  // tile keep ~16 mantissa bits of the f32 weight in the P.V product
  __shared__ short lds_p[4][16 * WPAD];
  __shared__ short lds_pl[4][16 * WPAD];

  const int qrow = q0 + wave * 16 + lo;
  const int qtok = tok0 + (qrow < q_len ? qrow : q_len - 1);
  bf16x8 qfrag[KK];
#pragma unroll
  for (int kk = 0; kk < KK; kk++)
    qfrag[kk] = *reinterpret_cast<const bf16x8*>(
        q + ((int64_t)qtok * H + h) * D + kk * 32 + hi * 8);

  float mrow[4], lrow[4];
  f32x4 ofrag[DT];
#pragma unroll
  for (int r = 0; r < 4; r++) {
    mrow[r] = sinks ? sinks[h] : -1e30f;
    lrow[r] = sinks ? 1.0f : 0.f;
  }
#pragma unroll
  for (int dt = 0; dt < DT; dt++) ofrag[dt] = f32x4{0.f, 0.f, 0.f, 0.f};

  const int kv_end = min(kv_len, q_abs0 + q0 + WQ_TILE);
  // first key any row of the tile may see: the window's start of the
  // tile's first row, or the start of that row's chunk
  const int vis0 = chunk > 0 ? ((q_abs0 + q0) / chunk) * chunk
      : (window > 0 ? q_abs0 + q0 - window + 1 : 0);
  const int kv_begin = vis0 > 0 ? (vis0 / WKV_TILE) * WKV_TILE : 0;
  // key tiles: those that hold kept first tokens, then the window's
  const int first_end =
      min((keep_first + WKV_TILE - 1) / WKV_TILE * WKV_TILE, kv_begin);
  for (int kv0 = first_end > 0 ? 0 : kv_begin; kv0 < kv_end;
       kv0 = (kv0 + WKV_TILE == first_end) ? kv_begin : kv0 + WKV_TILE) {
    for (int i = threadIdx.x; i < WKV_TILE * D / 8; i += 256) {
      const int row = (i * 8) / D;
      const int col = (i * 8) % D;
      const int kvp = min(kv0 + row, kv_len - 1);
      const int64_t src =
          (((int64_t)bt[kvp / BS] * G + g) * BS + (kvp % BS)) * D + col;
      const short8_t kd = *reinterpret_cast<const short8_t*>(k_cache + src);
      const int swz = (col * 2) ^ ((row & 7) << 4);
      *reinterpret_cast<short8_t*>(&lds_k[row * D + swz / 2]) = kd;
    }
    for (int i = threadIdx.x; i < WKV_TILE * DV / 8; i += 256) {
      const int row = (i * 8) / DV;
      const int col = (i * 8) % DV;
      const int kvp = min(kv0 + row, kv_len - 1);
      const int64_t src =
          (((int64_t)bt[kvp / BS] * G + g) * BS + (kvp % BS)) * DV + col;
      const short8_t vd = *reinterpret_cast<const short8_t*>(v_cache + src);
#pragma unroll
      for (int j = 0; j < 8; j++) lds_vt[(col + j) * WPAD + row] = vd[j];
    }
    __syncthreads();

    f32x4 sfrag[2];
#pragma unroll
    for (int kt = 0; kt < 2; kt++) {
      sfrag[kt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kk = 0; kk < KK; kk++) {
        const int krow = kt * 16 + lo;
        const int swz = ((kk * 32 + hi * 8) * 2) ^ ((krow & 7) << 4);
        const bf16x8 kf =
            *reinterpret_cast<const bf16x8*>(&lds_k[krow * D + swz / 2]);
        sfrag[kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
            qfrag[kk], kf, sfrag[kt], 0, 0, 0);
      }
    }

    float p[2][4];
#pragma unroll
    for (int kt = 0; kt < 2; kt++)
#pragma unroll
      for (int r = 0; r < 4; r++) {
        const int qr = q0 + wave * 16 + hi * 4 + r;
        const int q_abs = q_abs0 + qr;
        const int kvp = kv0 + kt * 16 + lo;
        float sv = sfrag[kt][r] * scale;
        if (softcap > 0.f)          // cap * tanh(s / cap), via exp
          sv = softcap * (1.0f - 2.0f / (__expf(2.0f * sv * inv_cap) + 1.0f));
        const int dist = q_abs - kvp;
        if (r1) sv -= hr1 * __logf(1.0f + hr2 * (float)max(dist, 0));
        if (dist < 0 || kvp >= kv_len || qr >= q_len ||
            (window > 0 && dist >= window && kvp >= keep_first) ||
            (chunk > 0 && kvp < (q_abs / chunk) * chunk)) sv = -1e30f;
        p[kt][r] = sv;
      }
#pragma unroll
    for (int r = 0; r < 4; r++) {
      float mx = fmaxf(p[0][r], p[1][r]);
#pragma unroll
      for (int off = 1; off < 16; off <<= 1)
        mx = fmaxf(mx, __shfl_xor(mx, off, 64));
      const float mnew = fmaxf(mrow[r], mx);
      const float corr = __expf(mrow[r] - mnew);
      lrow[r] *= corr;
#pragma unroll
      for (int dt = 0; dt < DT; dt++) ofrag[dt][r] *= corr;
      mrow[r] = mnew;
      float ps = 0.f;
#pragma unroll
      for (int kt = 0; kt < 2; kt++) {
        p[kt][r] = __expf(p[kt][r] - mnew);
        ps += p[kt][r];
      }
#pragma unroll
      for (int off = 1; off < 16; off <<= 1) ps += __shfl_xor(ps, off, 64);
      lrow[r] += ps;
    }
    {
      short* ph = lds_p[wave];
      short* pl = lds_pl[wave];
#pragma unroll
      for (int kt = 0; kt < 2; kt++)
#pragma unroll
        for (int r = 0; r < 4; r++) {
          const short hi16 = f32_to_bf16(p[kt][r]);
          const int at = (hi * 4 + r) * WPAD + kt * 16 + lo;
          ph[at] = hi16;
          pl[at] = f32_to_bf16(p[kt][r] - bf16_to_f32(hi16));
        }
    }
    __builtin_amdgcn_s_waitcnt(0);
    const bf16x8 pfrag = *reinterpret_cast<const bf16x8*>(
        &lds_p[wave][lo * WPAD + hi * 8]);
    const bf16x8 pfrag_lo = *reinterpret_cast<const bf16x8*>(
        &lds_pl[wave][lo * WPAD + hi * 8]);
#pragma unroll
    for (int dt = 0; dt < DT; dt++) {
      const bf16x8 vf = *reinterpret_cast<const bf16x8*>(
          &lds_vt[(dt * 16 + lo) * WPAD + hi * 8]);
      ofrag[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pfrag, vf,
                                                          ofrag[dt], 0, 0, 0);
      ofrag[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pfrag_lo, vf,
                                                          ofrag[dt], 0, 0, 0);
    }
    __syncthreads();
  }

#pragma unroll
  for (int r = 0; r < 4; r++) {
    const int qr = q0 + wave * 16 + hi * 4 + r;
    if (qr >= q_len) continue;
    const float inv = 1.f / fmaxf(lrow[r], 1e-30f);
    const int64_t obase = ((int64_t)(tok0 + qr) * H + h) * DV;
#pragma unroll
    for (int dt = 0; dt < DT; dt++)
      out[obase + dt * 16 + lo] = f32_to_bf16(ofrag[dt][r] * inv);
  }
}

// ---- decode kernel: one workgroup per (query row, kv head) -----------------
// All H/G query heads that share a kv head are served by one pass over its
// K and V rows (up to RT heads per workgroup; more heads take further
// passes on blockIdx.z). Per tile of up to KT keys:
//   scores : a wave takes 8 keys at a time, 8 lanes per key, each lane
//            16-byte chunks of the key row (contiguous 128 B per key); the
//            lane's slices of the RT query rows live in registers; 8-lane
//            DPP butterflies finish the dot products.
//   softmax: wave r mod 4 owns head r: tile max, exp, sum, running max and
//            sum with the rescale factor of the earlier tiles.
//   P.V    : LPR lanes cover one value row in 16-byte chunks, so one wave
//            load touches 64 / LPR rows and UNR of them are in flight;
//            weights are broadcast from LDS; the row groups of a wave are
//            folded by shuffles and the four waves meet in LDS at the end.
// The loops are unrolled by hand because the kernel is bound by the number
// of bytes in flight, not by arithmetic.
template <typename T, int RT, int NCH>
__global__ __launch_bounds__(256) void window_attention_decode_kernel(
    T* __restrict__ out, const T* __restrict__ q,
    const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const int* __restrict__ block_tables, const int max_blocks,
    const int* __restrict__ token_seq, const int64_t* __restrict__ positions,
    const float scale, const float softcap, const float* __restrict__ r1,
    const float* __restrict__ r2, const int window, const int H, const int G,
    const int D, const int V, const int BS, const int KT,
    const int keep_first, const float* __restrict__ sinks, const int chunk) {
  constexpr int VEC = 16 / (int)sizeof(T);
  extern __shared__ float lds[];
  float* s_s = lds;                            // [RT][KT]
  int* row_s = reinterpret_cast<int*>(s_s + RT * KT);   // [KT]
  float* m_s = reinterpret_cast<float*>(row_s + KT);    // [RT] running max
  float* l_s = m_s + RT;                       // [RT] running sum
  float* c_s = l_s + RT;                       // [RT] rescale of this tile
  float* acc_s = c_s + RT;                     // [4][RT][256]

  const int t = blockIdx.x, g = blockIdx.y;
  const int R = H / G;
  const int rbase = blockIdx.z * RT;
  const int nr = min(RT, R - rbase);
  const int h0 = g * R + rbase;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int sub = lane & 7, kl = lane >> 3;    // chunk lane, key in the wave
  const int b = token_seq[t];
  if (b < 0) {
    for (int r = 0; r < nr; r++)
      for (int j = tid; j < V; j += 256)
        act_st(out + ((int64_t)t * H + h0 + r) * V + j, 0.0f);
    return;
  }
  const int pos = (int)positions[t];
  const int lo = chunk > 0 ? (pos / chunk) * chunk
      : (window > 0 ? max(0, pos - window + 1) : 0);
  const int nfirst = min(keep_first, lo);       // kept keys before the window
  const int nkeys = nfirst + pos - lo + 1;
  const int* bt = block_tables + (int64_t)b * max_blocks;
  const int nchunks = D / VEC;

  float qreg[RT][NCH][VEC];
#pragma unroll
  for (int r = 0; r < RT; r++)
#pragma unroll
    for (int i = 0; i < NCH; i++) {
      const int ch = sub + 8 * i;
#pragma unroll
      for (int e = 0; e < VEC; e++)
        qreg[r][i][e] = (r < nr && ch < nchunks)
            ? act_ld(q + ((int64_t)t * H + h0 + r) * D + ch * VEC + e) : 0.0f;
    }
  float hr1[RT], hr2[RT];
#pragma unroll
  for (int r = 0; r < RT; r++) {
    hr1[r] = (r1 && r < nr) ? r1[h0 + r] : 0.0f;
    hr2[r] = (r1 && r < nr) ? r2[h0 + r] : 0.0f;
  }
  // P.V lane roles: LPR lanes cover one value row in 16-byte chunks, so a
  // wave load touches 64 / LPR rows at once
  const int vchunks = V / VEC;
  int lpr = 1;
  while (lpr < vchunks) lpr <<= 1;
  const int rpw = 64 / lpr;
  const int vch = lane % lpr, rsub = lane / lpr;
  const bool vlive = vch < vchunks;
  float acc[RT][VEC];
#pragma unroll
  for (int r = 0; r < RT; r++)
#pragma unroll
    for (int e = 0; e < VEC; e++) acc[r][e] = 0.0f;
  if (tid < RT) {
    const bool sk = sinks != nullptr && tid < nr;
    m_s[tid] = sk ? sinks[h0 + tid] : -INFINITY;
    l_s[tid] = sk ? 1.0f : 0.0f;
  }

  for (int k0 = 0; k0 < nkeys; k0 += KT) {
    const int nk = min(KT, nkeys - k0);
    __syncthreads();                 // previous tile's P.V done with s_s
    // ---- scores: UNR key groups per trip, all their loads issued first
    constexpr int UNR = 4;
    for (int kb = wave * 8 + kl; kb < nk; kb += 32 * UNR) {
      int rowi[UNR];
      float kv[UNR][NCH][VEC];
#pragma unroll
      for (int un = 0; un < UNR; un++) {
        const int kx = k0 + min(kb + 32 * un, nk - 1);
        const int j = kx < nfirst ? kx : lo + (kx - nfirst);
        rowi[un] = (bt[j / BS] * G + g) * BS + (j % BS);
      }
#pragma unroll
      for (int un = 0; un < UNR; un++) {
        const T* krow = k_cache + (int64_t)rowi[un] * D;
#pragma unroll
        for (int i = 0; i < NCH; i++) {
          const int ch = min(sub + 8 * i, nchunks - 1);
          if constexpr (sizeof(T) == 2) {
            const short8_t raw =
                *reinterpret_cast<const short8_t*>(krow + ch * VEC);
#pragma unroll
            for (int e = 0; e < VEC; e++) kv[un][i][e] = bf16_to_f32(raw[e]);
          } else {
            const float4_t raw =
                *reinterpret_cast<const float4_t*>(krow + ch * VEC);
#pragma unroll
            for (int e = 0; e < VEC; e++) kv[un][i][e] = raw[e];
          }
        }
      }
#pragma unroll
      for (int un = 0; un < UNR; un++) {
        const int kk = kb + 32 * un;
        const int kx = k0 + kk;
        const float dist =
            (float)(pos - (kx < nfirst ? kx : lo + (kx - nfirst)));
#pragma unroll
        for (int r = 0; r < RT; r++) {
          float dot = 0.0f;       // q slices of missing chunks are zero
#pragma unroll
          for (int i = 0; i < NCH; i++)
#pragma unroll
            for (int e = 0; e < VEC; e++) dot += qreg[r][i][e] * kv[un][i][e];
          float sv = group_reduce_sum<8>(dot) * scale;
          if (softcap > 0.f) sv = softcap * tanhf(sv / softcap);
          if (r1) sv -= hr1[r] * log1pf(hr2[r] * dist);
          if (sub == 0 && r < nr && kk < nk) s_s[r * KT + kk] = sv;
        }
        if (sub == 0 && kk < nk) row_s[kk] = rowi[un];
      }
    }
    __syncthreads();
    // ---- softmax statistics of the tile, one head per wave at a time
    for (int r = wave; r < nr; r += 4) {
      float mx = -INFINITY;
      for (int kk = lane; kk < nk; kk += 64) mx = fmaxf(mx, s_s[r * KT + kk]);
      mx = wave_reduce_max(mx);
      const float m_old = m_s[r];
      const float m_new = fmaxf(m_old, mx);
      float sum = 0.0f;
      for (int kk = lane; kk < nk; kk += 64) {
        const float p = expf(s_s[r * KT + kk] - m_new);
        s_s[r * KT + kk] = p;
        sum += p;
      }
      sum = wave_reduce_sum(sum);
      if (lane == 0) {
        const float corr = expf(m_old - m_new);      // 0 on the first tile
        c_s[r] = corr;
        l_s[r] = l_s[r] * corr + sum;
        m_s[r] = m_new;
      }
    }
    __syncthreads();
    // ---- P.V
#pragma unroll
    for (int r = 0; r < RT; r++) {
      const float corr = r < nr ? c_s[r] : 0.0f;
#pragma unroll
      for (int e = 0; e < VEC; e++) acc[r][e] *= corr;
    }
    const int rows_trip = 4 * rpw;           // rows per un-step, all waves
    for (int kb = wave * rpw + rsub; kb < nk; kb += rows_trip * UNR) {
      float vv[UNR][VEC], pw[UNR][RT];
#pragma unroll
      for (int un = 0; un < UNR; un++) {
        const int kk = min(kb + rows_trip * un, nk - 1);
        const bool ok = vlive && kb + rows_trip * un < nk;
        const T* vrow = v_cache + (int64_t)row_s[kk] * V +
                        min(vch, vchunks - 1) * VEC;
        if constexpr (sizeof(T) == 2) {
          const short8_t raw = *reinterpret_cast<const short8_t*>(vrow);
#pragma unroll
          for (int e = 0; e < VEC; e++) vv[un][e] = bf16_to_f32(raw[e]);
        } else {
          const float4_t raw = *reinterpret_cast<const float4_t*>(vrow);
#pragma unroll
          for (int e = 0; e < VEC; e++) vv[un][e] = raw[e];
        }
#pragma unroll
        for (int r = 0; r < RT; r++)
          pw[un][r] = (ok && r < nr) ? s_s[r * KT + kk] : 0.0f;
      }
#pragma unroll
      for (int un = 0; un < UNR; un++)
#pragma unroll
        for (int r = 0; r < RT; r++)
#pragma unroll
          for (int e = 0; e < VEC; e++) acc[r][e] += pw[un][r] * vv[un][e];
    }
  }
  // ---- fold: row groups inside the wave, then the four waves
#pragma unroll
  for (int r = 0; r < RT; r++)
#pragma unroll
    for (int e = 0; e < VEC; e++) {
      float a = acc[r][e];
      for (int off = lpr; off < 64; off <<= 1) a += __shfl_xor(a, off, 64);
      if (rsub == 0 && vlive)
        acc_s[(wave * RT + r) * 256 + vch * VEC + e] = a;
    }
  __syncthreads();
  for (int e = tid; e < nr * V; e += 256) {
    const int r = e / V, j = e % V;
    float a = 0.0f;
#pragma unroll
    for (int w = 0; w < 4; w++) a += acc_s[(w * RT + r) * 256 + j];
    act_st(out + ((int64_t)t * H + h0 + r) * V + j, a / l_s[r]);
  }
}

template <typename T, int RT>
void launch_decode(int nch, dim3 grid, size_t lds_bytes, hipStream_t stream,
                   at::Tensor& out, const at::Tensor& q,
                   const at::Tensor& k_cache, const at::Tensor& v_cache,
                   const at::Tensor& block_tables,
                   const at::Tensor& token_seq, const at::Tensor& positions,
                   float scale, float softcap, const float* r1,
                   const float* r2, int window, int H, int G, int D, int V,
                   int BS, int KT, int keep_first, const float* sinks,
                   int chunk) {
#define KAITO_WDEC(NCH_)                                                     \
  if (nch == NCH_) {                                                         \
    hipLaunchKernelGGL((window_attention_decode_kernel<T, RT, NCH_>), grid,  \
        dim3(256), lds_bytes, stream, (T*)out.data_ptr(),                    \
        (const T*)q.data_ptr(), (const T*)k_cache.data_ptr(),                \
        (const T*)v_cache.data_ptr(), block_tables.data_ptr<int>(),          \
        (int)block_tables.size(1), token_seq.data_ptr<int>(),                \
        positions.data_ptr<int64_t>(), scale, softcap, r1, r2, window, H, G, \
        D, V, BS, KT, keep_first, sinks, chunk);                             \
    return;                                                                  \
  }
  KAITO_WDEC(1) KAITO_WDEC(2) KAITO_WDEC(4)
#undef KAITO_WDEC
}

// Whether the decode kernel takes these sizes (16-byte chunks of the key
// and value rows, at most 32 chunks per key, value rows of at most 256).
inline bool decode_kernel_fits(int D, int V, int elem) {
  const int vec = 16 / elem;
  return D % vec == 0 && D / vec <= 32 && V % vec == 0 && V <= 256;
}

}  // namespace

void qk_norm_cache_write(at::Tensor q_out, at::Tensor q, at::Tensor k,
                         at::Tensor v, at::Tensor q_w, at::Tensor k_w,
                         double eps, at::Tensor k_cache, at::Tensor v_cache,
                         at::Tensor slot_mapping, at::Tensor positions,
                         at::Tensor inv_freq, double rot_mag,
                         at::Tensor v_first, double v_lambda) {
  TORCH_CHECK(q.is_cuda() && q.dim() == 3 && k.dim() == 3 && v.dim() == 3);
  const int T = q.size(0), H = q.size(1), D = q.size(2);
  const int G = k.size(1), V = v.size(2);
  TORCH_CHECK(k.size(0) == T && v.size(0) == T && k.size(2) == D &&
              v.size(1) == G);
  for (const at::Tensor* t : {&q, &k, &v})
    TORCH_CHECK(t->stride(2) == 1 && t->dtype() == q.dtype());
  TORCH_CHECK(is_act_dtype(q) && q_out.is_contiguous() &&
              q_out.sizes() == q.sizes() && q_out.dtype() == q.dtype());
  TORCH_CHECK(k_cache.is_contiguous() && v_cache.is_contiguous() &&
              k_cache.dim() == 4 && v_cache.dim() == 4 &&
              k_cache.dtype() == q.dtype() && v_cache.dtype() == q.dtype());
  TORCH_CHECK(k_cache.size(1) == G && k_cache.size(3) == D &&
              v_cache.size(1) == G && v_cache.size(3) == V &&
              v_cache.size(0) == k_cache.size(0) &&
              v_cache.size(2) == k_cache.size(2));
  const int BS = k_cache.size(2);
  const bool qn = q_w.numel() > 0, kn = k_w.numel() > 0;
  if (qn) { KAITO_CHECK_F32(q_w); TORCH_CHECK(q_w.numel() == D); }
  if (kn) { KAITO_CHECK_F32(k_w); TORCH_CHECK(k_w.numel() == D); }
  TORCH_CHECK(slot_mapping.is_cuda() && slot_mapping.dtype() == at::kLong &&
              slot_mapping.is_contiguous() && slot_mapping.size(0) == T);
  const int R = (int)inv_freq.numel();
  if (R > 0) {
    KAITO_CHECK_F32(inv_freq);
    TORCH_CHECK(2 * R <= D, "rotated dims exceed the head size");
    TORCH_CHECK(positions.is_cuda() && positions.dtype() == at::kLong &&
                positions.is_contiguous() && positions.size(0) == T);
  }
  const bool blend = v_first.numel() > 0;
  if (blend)
    TORCH_CHECK(v_first.dim() == 3 && v_first.sizes() == v.sizes() &&
                v_first.stride(2) == 1 && v_first.dtype() == v.dtype());
  if (T == 0) return;
  auto stream = at::hip::getCurrentHIPStream();
  KAITO_DISPATCH_ACT(q, {
    hipLaunchKernelGGL((qk_norm_cache_write_kernel<act_t>),
        dim3(T, H + 2 * G), dim3(64), 0, stream, (act_t*)q_out.data_ptr(),
        (const act_t*)q.data_ptr(), q.stride(0), q.stride(1),
        (const act_t*)k.data_ptr(), k.stride(0), k.stride(1),
        (const act_t*)v.data_ptr(), v.stride(0), v.stride(1),
        qn ? q_w.data_ptr<float>() : nullptr,
        kn ? k_w.data_ptr<float>() : nullptr, (float)eps,
        (act_t*)k_cache.data_ptr(), (act_t*)v_cache.data_ptr(),
        slot_mapping.data_ptr<int64_t>(), H, G, D, V, BS,
        R > 0 ? positions.data_ptr<int64_t>() : nullptr,
        R > 0 ? inv_freq.data_ptr<float>() : nullptr, R, (float)rot_mag,
        blend ? (const act_t*)v_first.data_ptr() : nullptr,
        blend ? v_first.stride(0) : 0, blend ? v_first.stride(1) : 0,
        (float)v_lambda);
  });
}

void window_attention(at::Tensor out, at::Tensor q, at::Tensor k_cache,
                      at::Tensor v_cache, at::Tensor block_tables,
                      at::Tensor token_seq, at::Tensor positions,
                      double scale, double softcap, at::Tensor r1,
                      at::Tensor r2, int64_t window, int64_t keep_first,
                      at::Tensor sinks, int64_t chunk) {
  TORCH_CHECK(q.is_cuda() && q.dim() == 3 && q.is_contiguous() &&
              is_act_dtype(q));
  TORCH_CHECK(keep_first >= 0 && keep_first < (1 << 30));
  TORCH_CHECK(chunk >= 0 && chunk < (1 << 30));
  // a chunked mask replaces the window: the keys a row sees are at most
  // one chunk, so tiles are sized by it
  if (chunk > 0) window = chunk;
  const int kf = (window > 0 && chunk == 0) ? (int)keep_first : 0;
  const bool has_sinks = sinks.numel() > 0;
  if (has_sinks) {
    KAITO_CHECK_F32(sinks);
    TORCH_CHECK(sinks.numel() == q.size(1));
  }
  const int T = q.size(0), H = q.size(1), D = q.size(2);
  TORCH_CHECK(k_cache.is_contiguous() && v_cache.is_contiguous() &&
              k_cache.dim() == 4 && v_cache.dim() == 4 &&
              k_cache.dtype() == q.dtype() && v_cache.dtype() == q.dtype());
  const int G = k_cache.size(1), BS = k_cache.size(2), V = v_cache.size(3);
  TORCH_CHECK(k_cache.size(3) == D && v_cache.size(1) == G &&
              v_cache.size(2) == BS && H % G == 0);
  TORCH_CHECK(out.is_contiguous() && out.dtype() == q.dtype() &&
              out.dim() == 3 && out.size(0) == T && out.size(1) == H &&
              out.size(2) == V);
  KAITO_CHECK_I32(block_tables); KAITO_CHECK_I32(token_seq);
  TORCH_CHECK(block_tables.dim() == 2 && token_seq.size(0) == T);
  TORCH_CHECK(positions.is_cuda() && positions.dtype() == at::kLong &&
              positions.is_contiguous() && positions.size(0) == T);
  const bool bias = r1.numel() > 0;
  if (bias) {
    KAITO_CHECK_F32(r1); KAITO_CHECK_F32(r2);
    TORCH_CHECK(r1.numel() == H && r2.numel() == H);
  }
  TORCH_CHECK((int64_t)k_cache.size(0) * G * BS < (1ll << 31));
  if (T == 0) return;
  auto stream0 = at::hip::getCurrentHIPStream();
  if (decode_kernel_fits(D, V, (int)q.element_size())) {
    const int R = H / G;
    // heads per workgroup: share K/V reads across the group when the step
    // has rows enough to fill the chip, else favour more workgroups
    int rt = R >= 8 ? 8 : (R > 2 ? 4 : (R == 2 ? 2 : 1));
    while (rt > 1 && (int64_t)T * G * ((R + rt - 1) / rt) < 1024) rt >>= 1;
    const int vec = 16 / (int)q.element_size();
    const int chunks = D / vec;
    const int nch = chunks <= 8 ? 1 : (chunks <= 16 ? 2 : 4);
    int KT = rt == 8 ? 512 : 1024;         // keeps the LDS stage under 64 KB
    if (window > 0 && window + kf < KT) KT = ((int)window + kf + 31) / 32 * 32;
    const size_t lds_bytes =
        ((size_t)rt * KT + KT + 3 * rt + 4 * rt * 256) * 4;
    const dim3 grid(T, G, (R + rt - 1) / rt);
    const float* p1 = bias ? r1.data_ptr<float>() : nullptr;
    const float* p2 = bias ? r2.data_ptr<float>() : nullptr;
    const float* ps = has_sinks ? sinks.data_ptr<float>() : nullptr;
    KAITO_DISPATCH_ACT(q, {
      if (rt == 8)
        launch_decode<act_t, 8>(nch, grid, lds_bytes, stream0, out, q,
            k_cache, v_cache, block_tables, token_seq, positions,
            (float)scale, (float)softcap, p1, p2, (int)window, H, G, D, V,
            BS, KT, kf, ps, (int)chunk);
      else if (rt == 4)
        launch_decode<act_t, 4>(nch, grid, lds_bytes, stream0, out, q,
            k_cache, v_cache, block_tables, token_seq, positions,
            (float)scale, (float)softcap, p1, p2, (int)window, H, G, D, V,
            BS, KT, kf, ps, (int)chunk);
      else if (rt == 2)
        launch_decode<act_t, 2>(nch, grid, lds_bytes, stream0, out, q,
            k_cache, v_cache, block_tables, token_seq, positions,
            (float)scale, (float)softcap, p1, p2, (int)window, H, G, D, V,
            BS, KT, kf, ps, (int)chunk);
      else
        launch_decode<act_t, 1>(nch, grid, lds_bytes, stream0, out, q,
            k_cache, v_cache, block_tables, token_seq, positions,
            (float)scale, (float)softcap, p1, p2, (int)window, H, G, D, V,
            BS, KT, kf, ps, (int)chunk);
    });
    return;
  }
  // other sizes: one head per workgroup, one key per thread
  // keys per tile: the window when it is short, else 256
  int threads = 256;
  if (window > 0 && window + kf <= 64) threads = 64;
  else if (window > 0 && window + kf <= 128) threads = 128;
  while (4 * threads < V) threads <<= 1;
  TORCH_CHECK(threads <= 1024, "value size too large: ", V);
  const size_t lds_bytes = ((size_t)D + 2 * threads) * 4;
  auto stream = at::hip::getCurrentHIPStream();
  KAITO_DISPATCH_ACT(q, {
    hipLaunchKernelGGL((window_attention_kernel<act_t>), dim3(T, H),
        dim3(threads), lds_bytes, stream, (act_t*)out.data_ptr(),
        (const act_t*)q.data_ptr(), (const act_t*)k_cache.data_ptr(),
        (const act_t*)v_cache.data_ptr(), block_tables.data_ptr<int>(),
        (int)block_tables.size(1), token_seq.data_ptr<int>(),
        positions.data_ptr<int64_t>(), (float)scale, (float)softcap,
        bias ? r1.data_ptr<float>() : nullptr,
        bias ? r2.data_ptr<float>() : nullptr, (int)window, H, G, D, V, BS,
        kf, has_sinks ? sinks.data_ptr<float>() : nullptr, (int)chunk);
  });
}

// Prompt-portion path: 64-row query tiles (tile_seq[i] = chunk, tile_qbase[i]
// = first row of the tile inside its chunk) on the MFMA kernel. bf16 with
// key/value sizes from {64, 128, 256}; callers fall back to
// window_attention otherwise (see window_attention_tiles_supported).
void window_attention_tiles(at::Tensor out, at::Tensor q, at::Tensor k_cache,
                            at::Tensor v_cache, at::Tensor block_tables,
                            at::Tensor tile_seq, at::Tensor tile_qbase,
                            at::Tensor cu_seqlens, at::Tensor seq_starts,
                            double scale, double softcap, at::Tensor r1,
                            at::Tensor r2, int64_t window, int64_t keep_first,
                            at::Tensor sinks, int64_t chunk) {
  TORCH_CHECK(q.is_cuda() && q.dim() == 3 && q.is_contiguous() &&
              q.dtype() == at::kBFloat16);
  TORCH_CHECK(keep_first >= 0 && keep_first < (1 << 30));
  TORCH_CHECK(chunk >= 0 && chunk < (1 << 30));
  if (chunk > 0) window = 0;          // a chunked mask replaces the window
  const int kf = window > 0 ? (int)keep_first : 0;
  const bool has_sinks = sinks.numel() > 0;
  if (has_sinks) {
    KAITO_CHECK_F32(sinks);
    TORCH_CHECK(sinks.numel() == q.size(1));
  }
  const int T = q.size(0), H = q.size(1), D = q.size(2);
  TORCH_CHECK(k_cache.is_contiguous() && v_cache.is_contiguous() &&
              k_cache.dim() == 4 && v_cache.dim() == 4 &&
              k_cache.dtype() == q.dtype() && v_cache.dtype() == q.dtype());
  const int G = k_cache.size(1), BS = k_cache.size(2), V = v_cache.size(3);
  TORCH_CHECK(k_cache.size(3) == D && v_cache.size(1) == G &&
              v_cache.size(2) == BS && H % G == 0);
  TORCH_CHECK(out.is_contiguous() && out.dtype() == q.dtype() &&
              out.dim() == 3 && out.size(0) == T && out.size(1) == H &&
              out.size(2) == V);
  KAITO_CHECK_I32(block_tables); KAITO_CHECK_I32(tile_seq);
  KAITO_CHECK_I32(tile_qbase); KAITO_CHECK_I32(cu_seqlens);
  KAITO_CHECK_I32(seq_starts);
  TORCH_CHECK(block_tables.dim() == 2 &&
              tile_qbase.size(0) == tile_seq.size(0) &&
              cu_seqlens.size(0) == seq_starts.size(0) + 1 &&
              block_tables.size(0) >= seq_starts.size(0));
  const bool bias = r1.numel() > 0;
  if (bias) {
    KAITO_CHECK_F32(r1); KAITO_CHECK_F32(r2);
    TORCH_CHECK(r1.numel() == H && r2.numel() == H);
  }
  const int ntiles = tile_seq.size(0);
  if (ntiles == 0 || T == 0) return;
  auto stream = at::hip::getCurrentHIPStream();
#define KAITO_WIN_CASE(D_, DV_)                                              \
  if (D == D_ && V == DV_) {                                                 \
    hipLaunchKernelGGL((window_attention_mfma_kernel<D_, DV_>),              \
        dim3(ntiles, H), dim3(256), 0, stream, (short*)out.data_ptr(),       \
        (const short*)q.data_ptr(), (const short*)k_cache.data_ptr(),        \
        (const short*)v_cache.data_ptr(), tile_seq.data_ptr<int>(),          \
        tile_qbase.data_ptr<int>(), cu_seqlens.data_ptr<int>(),              \
        seq_starts.data_ptr<int>(), block_tables.data_ptr<int>(),            \
        (int)block_tables.size(1), (float)scale, (float)softcap,             \
        bias ? r1.data_ptr<float>() : nullptr,                               \
        bias ? r2.data_ptr<float>() : nullptr, (int)window, H, G, BS, kf,    \
        has_sinks ? sinks.data_ptr<float>() : nullptr, (int)chunk);          \
    return;                                                                  \
  }
  KAITO_WIN_CASE(64, 64) KAITO_WIN_CASE(64, 128) KAITO_WIN_CASE(128, 64)
  KAITO_WIN_CASE(128, 128) KAITO_WIN_CASE(128, 256) KAITO_WIN_CASE(256, 128)
  KAITO_WIN_CASE(256, 256) KAITO_WIN_CASE(64, 256) KAITO_WIN_CASE(256, 64)
  KAITO_WIN_CASE(64, 32) KAITO_WIN_CASE(128, 32) KAITO_WIN_CASE(256, 32)
#undef KAITO_WIN_CASE
  TORCH_CHECK(false, "window_attention_tiles: key sizes {64, 128, 256} and "
              "value sizes {32, 64, 128, 256}, got ", D, "/", V);
}

}  // namespace kaito

TORCH_LIBRARY_FRAGMENT(kaito, m) {
  m.def("window_attention_tiles(Tensor(a!) out, Tensor q, Tensor k_cache, Tensor v_cache, Tensor block_tables, Tensor tile_seq, Tensor tile_qbase, Tensor cu_seqlens, Tensor seq_starts, float scale, float softcap, Tensor r1, Tensor r2, int window, int keep_first, Tensor sinks, int chunk) -> ()");
  m.def("qk_norm_cache_write(Tensor(a!) q_out, Tensor q, Tensor k, Tensor v, Tensor q_w, Tensor k_w, float eps, Tensor(b!) k_cache, Tensor(c!) v_cache, Tensor slot_mapping, Tensor positions, Tensor inv_freq, float rot_mag, Tensor v_first, float v_lambda) -> ()");
  m.def("window_attention(Tensor(a!) out, Tensor q, Tensor k_cache, Tensor v_cache, Tensor block_tables, Tensor token_seq, Tensor positions, float scale, float softcap, Tensor r1, Tensor r2, int window, int keep_first, Tensor sinks, int chunk) -> ()");
}
TORCH_LIBRARY_IMPL(kaito, CUDA, m) {
  m.impl("qk_norm_cache_write", &kaito::qk_norm_cache_write);
  m.impl("window_attention", &kaito::window_attention);
  m.impl("window_attention_tiles", &kaito::window_attention_tiles);
}
