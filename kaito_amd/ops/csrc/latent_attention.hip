// Latent attention over a paged cache of low-rank latents, for batches of
// chunks (prompt portions and single decode tokens alike), and the hashed
// bigram embedding. Activations are bf16 or f32; all arithmetic is f32.
//
// Cache layout: [blocks, block_size, rank + P] — per token the RMS-normed
// latent c (rank dims) followed by one rotated key part (P dims) shared by
// all heads. Keys and values of head h are linear in c (k_h = [W_uk,h c |
// rotated part], v_h = W_uv,h c), so attention can run in the latent
// space: with q_c = W_uk,h^T q_h,
//
//   score(i, j) = (q_c,i . c_j + q_rot,i . k_rot,j) * scale,   j <= i
//   out_c,i     = sum_j softmax_j(score)(+ sink) * c_j
//
// and W_uv,h is applied to out_c afterwards. One pass over the cache rows
// serves every head of the tile.
//
//   bigram_embed              token embedding * scale + hashed bigram row
//   latent_rope_cache_write   rotation of q's rotated part; RMS norm of the
//                             latent + rotation of the shared key part +
//                             scatter into the paged cache
//   latent_attention          the latent-space attention above. bf16: MFMA
//                             kernel, workgroup per (row, 16 heads, split
//                             of the keys), partials joined by a merge
//                             kernel. f32 and odd sizes: workgroup per
//                             (row, 8 heads), 32 cache rows per tile
//                             through LDS, online softmax, per-head sink
//   latent_expand             packs up-projected keys/values of gathered
//                             cache rows into a step-local paged K/V scratch
//                             [pages, H, block_size, Dp|Vp] (zero padded)
//                             for the MFMA prompt kernel of the window mixers
#include "mix_common.h"
#include <algorithm>

namespace kaito {

namespace {

// ---- embedding --------------------------------------------------------------
// grid (T). A chunk's first row takes its previous token from prev_state
// (or none at position 0); prev_state is advanced by a second launch that is
// ordered after every read.
template <typename T>
__global__ void bigram_embed_kernel(
    float* __restrict__ out,                       // [T, W]
    const int64_t* __restrict__ ids, const T* __restrict__ embed,
    const float scale, const T* __restrict__ table, const int64_t buckets,
    const int64_t mul_prev, const int64_t mul_cur,
    const int64_t* __restrict__ prev_state, const int* __restrict__ cu,
    const int* __restrict__ slots, const int* __restrict__ starts,
    const int* __restrict__ token_seq, const int W) {
  const int t = blockIdx.x;
  const int b = token_seq[t];
  float* orow = out + (int64_t)t * W;
  if (b < 0 || slots[b] < 0) {
    for (int d = threadIdx.x; d < W; d += blockDim.x) orow[d] = 0.f;
    return;
  }
  const int64_t tok = ids[t];
  const T* erow = embed + tok * W;
  if (table == nullptr) {
    for (int d = threadIdx.x; d < W; d += blockDim.x)
      orow[d] = act_ld(erow + d) * scale;
    return;
  }
  int64_t prev;
  if (t == cu[b]) prev = starts[b] == 0 ? -1 : prev_state[slots[b]];
  else prev = ids[t - 1];
  const int64_t r =
      prev < 0 ? buckets : (prev * mul_prev + tok * mul_cur) % buckets;
  const T* brow = table + r * W;
  for (int d = threadIdx.x; d < W; d += blockDim.x)
    orow[d] = act_ld(erow + d) * scale + act_ld(brow + d);
}

__global__ void bigram_state_kernel(int64_t* __restrict__ prev_state,
                                    const int64_t* __restrict__ ids,
                                    const int* __restrict__ cu,
                                    const int* __restrict__ slots,
                                    const int B) {
  const int b = blockIdx.x * blockDim.x + threadIdx.x;
  if (b >= B) return;
  if (slots[b] >= 0 && cu[b + 1] > cu[b]) prev_state[slots[b]] = ids[cu[b + 1] - 1];
}

// ---- rotation + latent norm + cache scatter ----------------------------------
// grid (T, ceil(items / 4)), 4 waves, one item of the row per wave: item
// y < H is head y of q (first `dim` dims copied, the 2R after them rotated,
// the tail up to HDo zeroed; 16-byte moves when `vec`), item H the latent
// row (only for a mixer with a down-projection of its own).
template <typename T>
__global__ __launch_bounds__(256) void latent_rope_cache_write_kernel(
    T* __restrict__ q_out,                 // [T, H, HDo >= dim + 2R], 0-padded
    const T* __restrict__ q, const int64_t q_s0,    // [T, H, dim + 2R] view
    const T* __restrict__ dkv, const int64_t dkv_s0,   // [T, rank + 2R] view
    const float* __restrict__ norm_w, const float eps,
    T* __restrict__ cache, const int64_t* __restrict__ slot_mapping,
    const int64_t* __restrict__ positions,
    const float* __restrict__ inv_freq, const int H, const int dim,
    const int R, const int rank, const int HDo, const bool vec,
    const bool interleaved, const float mag) {
  const int t = blockIdx.x, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const float pos = (float)positions[t];
  // pair i is dims (i, i + R), or (2i, 2i + 1) when interleaved
  const int pa = interleaved ? 2 : 1, pb = interleaved ? 1 : R;
  const int items = H + (dkv != nullptr ? 1 : 0);
  const int HD = dim + 2 * R;
  constexpr int VEC = 16 / (int)sizeof(T);
  {
    const int y = blockIdx.y * 4 + wave;
    if (y >= items) return;
    if (y < H) {
      const T* src = q + (int64_t)t * q_s0 + (int64_t)y * HD;
      T* dst = q_out + ((int64_t)t * H + y) * HDo;
      if (vec) {
        for (int d = lane * VEC; d < dim; d += 64 * VEC)
          *reinterpret_cast<float4_t*>(dst + d) =
              *reinterpret_cast<const float4_t*>(src + d);
        const float4_t zero = {0.f, 0.f, 0.f, 0.f};
        for (int d = HD + lane * VEC; d < HDo; d += 64 * VEC)
          *reinterpret_cast<float4_t*>(dst + d) = zero;
      } else {
        for (int d = lane; d < dim; d += 64) dst[d] = src[d];
        for (int d = HD + lane; d < HDo; d += 64) act_st(dst + d, 0.f);
      }
      for (int i = lane; i < R; i += 64) {
        const float ang = pos * inv_freq[i];
        const float c = cosf(ang) * mag, s = sinf(ang) * mag;
        const int ia = dim + i * pa, ib = ia + pb;
        const float u = act_ld(src + ia), v = act_ld(src + ib);
        act_st(dst + ia, u * c - v * s);
        act_st(dst + ib, v * c + u * s);
      }
      return;
    }
    const int64_t slot = slot_mapping[t];
    if (slot < 0) return;
    const T* src = dkv + (int64_t)t * dkv_s0;
    T* dst = cache + slot * (int64_t)(rank + 2 * R);
    float ss = 0.f;
    for (int d = lane; d < rank; d += 64) { const float x = act_ld(src + d); ss += x * x; }
    ss = wave_reduce_sum(ss);
    const float inv = 1.0f / sqrtf(ss / (float)rank + eps);
    for (int d = lane; d < rank; d += 64)
      act_st(dst + d, act_ld(src + d) * inv * norm_w[d]);
    for (int i = lane; i < R; i += 64) {
      const float ang = pos * inv_freq[i];
      const float c = cosf(ang) * mag, s = sinf(ang) * mag;
      const int ia = rank + i * pa, ib = ia + pb;
      const float u = act_ld(src + ia), v = act_ld(src + ib);
      act_st(dst + ia, u * c - v * s);
      act_st(dst + ib, v * c + u * s);
    }
  }
}

// ---- latent-space attention ---------------------------------------------------
constexpr int LA_HT = 8;      // heads per workgroup
constexpr int LA_KT = 32;     // cache rows per tile
constexpr int LA_MAXI = 32;   // rank <= 32 * LA_MAXI

template <typename T> struct lds_pad;                 // row padding, elements
template <> struct lds_pad<float> { static constexpr int v = 1; };
template <> struct lds_pad<bf16_act> { static constexpr int v = 2; };

// grid (T, ceil(H / 8)), block 256. Thread (h = tid / 32, k = tid % 32):
// in the score phase it dots query h with tile row k; in the accumulation
// phase it owns output dims k, k + 32, ... of head h. The 32 lanes of a head
// are one half of a wave, so the head's running maximum and sum live in
// registers, the same in all its lanes.
template <typename T>
__global__ __launch_bounds__(256) void latent_attention_kernel(
    T* __restrict__ out,                            // [T, H, rank]
    const T* __restrict__ q,                        // [T, H, DT]
    const T* __restrict__ cache,                    // [pages, BS, DT]
    const int* __restrict__ block_tables, const int max_blocks,
    const int* __restrict__ token_seq, const int64_t* __restrict__ positions,
    const float scale, const float* __restrict__ sinks, const int H,
    const int DT, const int rank, const int BS) {
  extern __shared__ __align__(16) unsigned char lds_raw[];
  const int RS = DT + lds_pad<T>::v;                 // padded row, elements
  float* q_s = reinterpret_cast<float*>(lds_raw);   // [HT][DT]
  float* p_s = q_s + LA_HT * DT;                    // [HT][KT]
  T* kv_s = reinterpret_cast<T*>(p_s + LA_HT * LA_KT);   // [KT][RS]

  const int t = blockIdx.x, h0 = blockIdx.y * LA_HT, tid = threadIdx.x;
  const int hl = tid >> 5, k = tid & 31, h = h0 + hl;
  const bool live = h < H;
  const int b = token_seq[t];
  T* orow = out + ((int64_t)t * H + h) * rank;
  if (b < 0) {
    if (live) for (int d = k; d < rank; d += 32) act_st(orow + d, 0.f);
    return;
  }
  const int nkeys = (int)positions[t] + 1;
  const int* bt = block_tables + (int64_t)b * max_blocks;

  for (int i = tid; i < LA_HT * DT; i += 256) {
    const int hh = h0 + i / DT;
    q_s[i] = hh < H ? act_ld(q + ((int64_t)t * H + hh) * DT + i % DT) : 0.f;
  }
  float acc[LA_MAXI];
#pragma unroll
  for (int i = 0; i < LA_MAXI; i++) acc[i] = 0.f;
  const bool sink = sinks != nullptr && live;
  float m_run = sink ? sinks[h] : -INFINITY, l_run = sink ? 1.0f : 0.f;
  const int wave = tid >> 6, lane = tid & 63;

  for (int k0 = 0; k0 < nkeys; k0 += LA_KT) {
    const int nk = min(LA_KT, nkeys - k0);
    __syncthreads();              // q_s ready / previous tile consumed
    for (int r = wave; r < nk; r += 4) {
      const int j = k0 + r;
      const T* src = cache + ((int64_t)bt[j / BS] * BS + j % BS) * DT;
      for (int d = lane; d < DT; d += 64) kv_s[r * RS + d] = src[d];
    }
    __syncthreads();
    float s = -INFINITY;
    if (k < nk) {
      const float* qh = q_s + hl * DT;
      const T* row = kv_s + k * RS;
      float a0 = 0.f, a1 = 0.f;
      int d = 0;
      for (; d + 2 <= DT; d += 2) {
        a0 += qh[d] * act_ld(row + d);
        a1 += qh[d + 1] * act_ld(row + d + 1);
      }
      if (d < DT) a0 += qh[d] * act_ld(row + d);
      s = (a0 + a1) * scale;
    }
    const float m_new = fmaxf(m_run, group_reduce_max<32>(s));
    const float p = k < nk ? expf(s - m_new) : 0.f;
    p_s[hl * LA_KT + k] = p;
    float ps = p;
#pragma unroll
    for (int off = 16; off > 0; off >>= 1) ps += __shfl_xor(ps, off, 64);
    const float corr = expf(m_run - m_new);   // 0 on a first tile without sink
    l_run = l_run * corr + ps;
    m_run = m_new;
    __syncthreads();              // p_s visible
    const float* ph = p_s + hl * LA_KT;
#pragma unroll
    for (int i = 0; i < LA_MAXI; i++) {
      const int d = k + 32 * i;
      if (d < rank) {
        float a = acc[i] * corr;
        for (int kk = 0; kk < nk; kk++)
          a += ph[kk] * act_ld(kv_s + kk * RS + d);
        acc[i] = a;
      }
    }
  }
  if (!live) return;
  const float inv = 1.0f / l_run;
#pragma unroll
  for (int i = 0; i < LA_MAXI; i++) {
    const int d = k + 32 * i;
    if (d < rank) act_st(orow + d, acc[i] * inv);
  }
}

// ---- latent-space attention on the matrix cores (bf16) -----------------------
// Workgroup = one row x 16 heads x one split of the row's keys; 4 waves.
// The 16 heads are the M side of v_mfma_f32_16x16x32_bf16. Per tile of 32
// cache rows, staged once into LDS row-major (scores) and, for the first
// `rank` dims, transposed (weighted sum), while the next tile's rows are
// already being fetched into registers:
//   scores   S[16 x 32] = Q[16 x DT] K^T: the DT/32 k-steps are dealt to the
//            4 waves (their query fragments stay in registers), partial sums
//            meet in LDS;
//   softmax  f32, thread (head, 2 keys), running maximum and sum per head in
//            registers; weights leave as a bf16 value + remainder pair;
//   sum      O[16 x rank] += P[16 x 32] C[32 x rank]: the rank/16 column
//            tiles are dealt to the 4 waves, two MFMAs per tile (value and
//            remainder), accumulators rescaled by the head's correction.
// With S > 1 splits a workgroup covers a contiguous share of the key tiles
// and leaves unnormalised (sum, maximum, denominator) partials for
// latent_merge_kernel; the sink enters in split 0.
constexpr int LM_KTP = 40;     // key stride of the transposed tile and of P

template <int MAXKS, int NT>
__global__ __launch_bounds__(256) void latent_attention_mfma_kernel(
    short* __restrict__ out,                        // [T, H, rank]
    float* __restrict__ part_acc,                   // [T, S, H, rank]
    float* __restrict__ part_ml,                    // [T, S, H, 2]
    const short* __restrict__ q,                    // [T, H, DT]
    const short* __restrict__ cache,                // [pages, BS, DT]
    const int* __restrict__ block_tables, const int max_blocks,
    const int* __restrict__ token_seq, const int64_t* __restrict__ positions,
    const float scale, const float* __restrict__ sinks, const int H,
    const int DT, const int rank, const int BS, const int S) {
  extern __shared__ __align__(16) unsigned char lds_raw[];
  const int DTp = (DT + 31) & ~31, RS = DTp + 8;
  const int rankp = (rank + 15) & ~15;
  short* kv_s = reinterpret_cast<short*>(lds_raw);          // [32][RS]
  short* vt_s = kv_s + 32 * RS;                             // [rankp][KTP]
  short* p_hi = vt_s + rankp * LM_KTP;                      // [16][KTP]
  short* p_lo = p_hi + 16 * LM_KTP;                         // [16][KTP]
  float* part_s = reinterpret_cast<float*>(p_lo + 16 * LM_KTP);  // [4][16][32]
  float* s_corr = part_s + 4 * 16 * 32;                     // [16]
  float* s_l = s_corr + 16;                                 // [16]
  float* s_m = s_l + 16;                                    // [16]

  const int t = blockIdx.x, h0 = blockIdx.y * 16, split = blockIdx.z;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int lo = lane & 15, hi = lane >> 4;
  const int sh = tid >> 4, sj = tid & 15;       // softmax role: head, key pair
  const int b = token_seq[t];
  const int nkeys = b < 0 ? 0 : (int)positions[t] + 1;
  const int nt_all = (nkeys + 31) >> 5;
  const int tile_lo = (int)((int64_t)nt_all * split / S);
  const int tile_hi = (int)((int64_t)nt_all * (split + 1) / S);
  const int* bt = block_tables + (int64_t)max(b, 0) * max_blocks;

  // zero what staging never writes: the k padding of the rows and the
  // rows of the transposed tile past the rank
  for (int i = tid; i < 32 * (RS - DT); i += 256)
    kv_s[(i / (RS - DT)) * RS + DT + i % (RS - DT)] = 0;
  for (int i = tid; i < (rankp - rank) * LM_KTP; i += 256)
    vt_s[rank * LM_KTP + i] = 0;

  // this wave's query fragments: k-steps wave, wave + 4, ...
  const int nks = DTp >> 5;
  bf16x8 qf[MAXKS];
#pragma unroll
  for (int i = 0; i < MAXKS; i++) {
    const int d = ((wave + 4 * i) << 5) + hi * 8;
    bf16x8 v = {0, 0, 0, 0, 0, 0, 0, 0};
    if (h0 + lo < H && d < DT)
      v = *reinterpret_cast<const bf16x8*>(
          q + ((int64_t)t * H + h0 + lo) * DT + d);
    qf[i] = v;
  }
  f32x4 acc[NT];
#pragma unroll
  for (int i = 0; i < NT; i++) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
  const bool sink = sinks != nullptr && split == 0 && h0 + sh < H;
  float m_run = sink ? sinks[h0 + sh] : -INFINITY;
  float l_run = sink ? 1.0f : 0.f;
  const int nchunk = DT >> 3, key = tid & 31;

  // A thread owns cache row `key` of the tile and the 16-byte chunks
  // tid/32, tid/32 + 8, ... of it. The next tile's chunks are fetched into
  // registers while the current tile is computed.
  constexpr int MAXC = 2 * MAXKS;
  union chunk_t { bf16x8 v; uint32_t w[4]; };
  chunk_t nxt[MAXC];
  auto fetch = [&](const int tile) {
    const int j = (tile << 5) + key;
    const short* src = j < nkeys
        ? cache + ((int64_t)bt[j / BS] * BS + j % BS) * DT : nullptr;
#pragma unroll
    for (int i = 0; i < MAXC; i++) {
      const int dc = (tid >> 5) + 8 * i;
      bf16x8 v = {0, 0, 0, 0, 0, 0, 0, 0};     // rows past the end are zero
      if (src != nullptr && dc < nchunk)
        v = *reinterpret_cast<const bf16x8*>(src + dc * 8);
      nxt[i].v = v;
    }
  };
  if (tile_lo < tile_hi) fetch(tile_lo);
  const bool odd = key & 1;

  for (int tile = tile_lo; tile < tile_hi; tile++) {
    const int k0 = tile << 5;
    const int nk = min(32, nkeys - k0);
    __syncthreads();            // previous tile consumed
#pragma unroll
    for (int i = 0; i < MAXC; i++) {
      const int dc = (tid >> 5) + 8 * i;
      if (dc < nchunk) {
        *reinterpret_cast<bf16x8*>(kv_s + key * RS + dc * 8) = nxt[i].v;
        if (dc * 8 < rank) {
          // transposed copy: neighbouring lanes hold neighbouring keys, so
          // a pair trades halves and each lane stores two keys at once
#pragma unroll
          for (int jj = 0; jj < 4; jj++) {
            const uint32_t own = nxt[i].w[jj];
            const uint32_t oth = (uint32_t)__shfl_xor((int)own, 1, 64);
            const uint32_t two = odd ? ((oth >> 16) | (own & 0xffff0000u))
                                     : ((own & 0xffffu) | (oth << 16));
            *reinterpret_cast<uint32_t*>(
                vt_s + (dc * 8 + 2 * jj + (odd ? 1 : 0)) * LM_KTP +
                (key & ~1)) = two;
          }
        }
      }
    }
    if (tile + 1 < tile_hi) fetch(tile + 1);
    __syncthreads();
    // scores: partial over this wave's k-steps
    f32x4 sc[2] = {f32x4{0.f, 0.f, 0.f, 0.f}, f32x4{0.f, 0.f, 0.f, 0.f}};
#pragma unroll
    for (int i = 0; i < MAXKS; i++) {
      const int ks = wave + 4 * i;
      if (ks < nks) {
#pragma unroll
        for (int nt = 0; nt < 2; nt++) {
          const bf16x8 kb = *reinterpret_cast<const bf16x8*>(
              kv_s + (nt * 16 + lo) * RS + (ks << 5) + hi * 8);
          sc[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qf[i], kb, sc[nt],
                                                           0, 0, 0);
        }
      }
    }
#pragma unroll
    for (int nt = 0; nt < 2; nt++)
#pragma unroll
      for (int r = 0; r < 4; r++)
        part_s[(wave * 16 + hi * 4 + r) * 32 + nt * 16 + lo] = sc[nt][r];
    __syncthreads();
    // softmax: head sh, keys sj and sj + 16
    {
      float s0 = 0.f, s1 = 0.f;
#pragma unroll
      for (int w = 0; w < 4; w++) {
        s0 += part_s[(w * 16 + sh) * 32 + sj];
        s1 += part_s[(w * 16 + sh) * 32 + sj + 16];
      }
      s0 = sj < nk ? s0 * scale : -INFINITY;
      s1 = sj + 16 < nk ? s1 * scale : -INFINITY;
      const float m_new =
          fmaxf(m_run, group_reduce_max<16>(fmaxf(s0, s1)));
      const float p0 = sj < nk ? expf(s0 - m_new) : 0.f;
      const float p1 = sj + 16 < nk ? expf(s1 - m_new) : 0.f;
      const float ps = group_reduce_sum<16>(p0 + p1);
      const float corr = expf(m_run - m_new);
      l_run = l_run * corr + ps;
      m_run = m_new;
      const short h0b = f32_to_bf16(p0), h1b = f32_to_bf16(p1);
      p_hi[sh * LM_KTP + sj] = h0b;
      p_hi[sh * LM_KTP + sj + 16] = h1b;
      p_lo[sh * LM_KTP + sj] = f32_to_bf16(p0 - bf16_to_f32(h0b));
      p_lo[sh * LM_KTP + sj + 16] = f32_to_bf16(p1 - bf16_to_f32(h1b));
      if (sj == 0) s_corr[sh] = corr;
    }
    __syncthreads();
    // weighted sum over this wave's column tiles
    {
      const bf16x8 ah = *reinterpret_cast<const bf16x8*>(
          p_hi + lo * LM_KTP + hi * 8);
      const bf16x8 al = *reinterpret_cast<const bf16x8*>(
          p_lo + lo * LM_KTP + hi * 8);
      float cr[4];
#pragma unroll
      for (int r = 0; r < 4; r++) cr[r] = s_corr[hi * 4 + r];
#pragma unroll
      for (int i = 0; i < NT; i++) {
        const int n = wave + 4 * i;
        if (n * 16 < rankp) {
          const bf16x8 vb = *reinterpret_cast<const bf16x8*>(
              vt_s + (n * 16 + lo) * LM_KTP + hi * 8);
          f32x4 a = acc[i];
#pragma unroll
          for (int r = 0; r < 4; r++) a[r] *= cr[r];
          a = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ah, vb, a, 0, 0, 0);
          a = __builtin_amdgcn_mfma_f32_16x16x32_bf16(al, vb, a, 0, 0, 0);
          acc[i] = a;
        }
      }
    }
  }
  if (b < 0 && split == 0) { m_run = 0.f; l_run = 1.0f; }   // padding row: zeros
  __syncthreads();
  if (sj == 0) { s_l[sh] = l_run; s_m[sh] = m_run; }
  __syncthreads();
  if (S > 1 && sj == 0 && h0 + sh < H) {
    float* ml = part_ml + (((int64_t)t * S + split) * H + h0 + sh) * 2;
    ml[0] = m_run;
    ml[1] = l_run;
  }
#pragma unroll
  for (int i = 0; i < NT; i++) {
    const int d = (wave + 4 * i) * 16 + lo;
    if (d >= rank) continue;
#pragma unroll
    for (int r = 0; r < 4; r++) {
      const int hh = hi * 4 + r;
      if (h0 + hh >= H) continue;
      if (S > 1) {
        part_acc[(((int64_t)t * S + split) * H + h0 + hh) * rank + d] =
            acc[i][r];
      } else {
        out[((int64_t)t * H + h0 + hh) * rank + d] =
            f32_to_bf16(acc[i][r] / s_l[hh]);
      }
    }
  }
}

// grid (T, H), block 128: joins the S <= 16 partials of a (row, head); a
// thread owns 4 adjacent output dims (rank is a multiple of 8).
__global__ void latent_merge_kernel(short* __restrict__ out,
                                    const float* __restrict__ part_acc,
                                    const float* __restrict__ part_ml,
                                    const int H, const int rank,
                                    const int S) {
  const int t = blockIdx.x, h = blockIdx.y;
  const float* ml = part_ml + ((int64_t)t * S * H + h) * 2;
  const int64_t ml_step = (int64_t)H * 2, acc_step = (int64_t)H * rank;
  float w[16];
  float M = -INFINITY;
#pragma unroll
  for (int s = 0; s < 16; s++)
    if (s < S) M = fmaxf(M, ml[s * ml_step]);
  float L = 0.f;
#pragma unroll
  for (int s = 0; s < 16; s++) {
    w[s] = s < S ? expf(ml[s * ml_step] - M) : 0.f;
    if (s < S) L += ml[s * ml_step + 1] * w[s];
  }
  const float inv = 1.0f / L;
  const float* acc = part_acc + ((int64_t)t * S * H + h) * rank;
  for (int d = threadIdx.x * 4; d < rank; d += blockDim.x * 4) {
    float4_t a = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < 16; s++)
      if (s < S)
        a += w[s] * *reinterpret_cast<const float4_t*>(acc + s * acc_step + d);
    short4_t o;
#pragma unroll
    for (int e = 0; e < 4; e++) o[e] = f32_to_bf16(a[e] * inv);
    *reinterpret_cast<short4_t*>(out + ((int64_t)t * H + h) * rank + d) = o;
  }
}

// ---- expansion into a step-local K/V scratch -------------------------------
// grid (N rows, H), one wave. Row n of the gathered cache rows lands in
// scratch page n / BS, slot n % BS.
template <typename T>
__global__ void latent_expand_kernel(
    T* __restrict__ k_s, T* __restrict__ v_s,       // [pages, H, BS, Dp|Vp]
    const T* __restrict__ kn,                       // [N, H*D]
    const T* __restrict__ vv,                       // [N, H*V]
    const T* __restrict__ lat,                      // [N, rank + P]
    const int H, const int D, const int V, const int P, const int rank,
    const int Dp, const int Vp, const int BS) {
  const int n = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int64_t row = ((int64_t)(n / BS) * H + h) * BS + n % BS;
  T* kd = k_s + row * Dp;
  T* vd = v_s + row * Vp;
  const T* ks = kn + ((int64_t)n * H + h) * D;
  const T* vs = vv + ((int64_t)n * H + h) * V;
  const T* ls = lat + (int64_t)n * (rank + P) + rank;
  for (int d = lane; d < Dp; d += 64) {
    if (d < D) kd[d] = ks[d];
    else if (d < D + P) kd[d] = ls[d - D];
    else act_st(kd + d, 0.f);
  }
  for (int d = lane; d < Vp; d += 64) {
    if (d < V) vd[d] = vs[d];
    else act_st(vd + d, 0.f);
  }
}

}  // namespace

void bigram_embed(at::Tensor out, at::Tensor ids, at::Tensor embed,
                  double scale, at::Tensor table, int64_t buckets,
                  int64_t mul_prev, int64_t mul_cur, at::Tensor prev_state,
                  at::Tensor cu_seqlens, at::Tensor state_slots,
                  at::Tensor seq_starts, at::Tensor token_seq) {
  TORCH_CHECK(ids.is_cuda() && ids.dtype() == at::kLong && ids.is_contiguous());
  TORCH_CHECK(embed.dim() == 2 && embed.is_contiguous() && is_act_dtype(embed));
  const int T = ids.size(0), W = embed.size(1);
  KAITO_CHECK_F32(out);
  TORCH_CHECK(out.dim() == 2 && out.size(0) == T && out.size(1) == W);
  KAITO_CHECK_I32(cu_seqlens); KAITO_CHECK_I32(state_slots);
  KAITO_CHECK_I32(seq_starts); KAITO_CHECK_I32(token_seq);
  const int B = state_slots.size(0);
  TORCH_CHECK(cu_seqlens.size(0) == B + 1 && seq_starts.size(0) == B &&
              token_seq.size(0) == T);
  const bool bg = table.numel() > 0;
  if (bg) {
    TORCH_CHECK(table.dim() == 2 && table.is_contiguous() &&
                table.dtype() == embed.dtype() && table.size(1) == W &&
                table.size(0) == buckets + 1 && buckets > 0);
    TORCH_CHECK(prev_state.is_cuda() && prev_state.dtype() == at::kLong &&
                prev_state.is_contiguous());
  }
  if (T == 0) return;
  auto stream = at::hip::getCurrentHIPStream();
  KAITO_DISPATCH_ACT(embed, {
    hipLaunchKernelGGL((bigram_embed_kernel<act_t>), dim3(T),
        dim3(W >= 1024 ? 256 : 128), 0, stream, out.data_ptr<float>(),
        ids.data_ptr<int64_t>(), (const act_t*)embed.data_ptr(), (float)scale,
        bg ? (const act_t*)table.data_ptr() : nullptr, buckets, mul_prev,
        mul_cur, bg ? prev_state.data_ptr<int64_t>() : nullptr,
        cu_seqlens.data_ptr<int>(), state_slots.data_ptr<int>(),
        seq_starts.data_ptr<int>(), token_seq.data_ptr<int>(), W);
  });
  if (bg)
    hipLaunchKernelGGL(bigram_state_kernel, dim3((B + 127) / 128), dim3(128),
        0, stream, prev_state.data_ptr<int64_t>(), ids.data_ptr<int64_t>(),
        cu_seqlens.data_ptr<int>(), state_slots.data_ptr<int>(), B);
}

void latent_rope_cache_write(at::Tensor q_out, at::Tensor q, at::Tensor dkv,
                             at::Tensor norm_w, double eps, at::Tensor cache,
                             at::Tensor slot_mapping, at::Tensor positions,
                             at::Tensor inv_freq, int64_t dim,
                             bool interleaved, double rot_mag) {
  TORCH_CHECK(q.is_cuda() && q.dim() == 3 && is_act_dtype(q) &&
              q.stride(2) == 1);
  const int T = q.size(0), H = q.size(1), HD = q.size(2);
  TORCH_CHECK(q.stride(1) == HD, "heads of q must be adjacent");
  KAITO_CHECK_F32(inv_freq);
  const int R = inv_freq.numel();
  TORCH_CHECK(R > 0 && dim >= 0 && dim + 2 * R == HD,
              "head size must be dim + 2 * len(inv_freq)");
  TORCH_CHECK(q_out.is_contiguous() && q_out.dtype() == q.dtype() &&
              q_out.dim() == 3 && q_out.size(0) == T && q_out.size(1) == H &&
              q_out.size(2) >= HD);
  TORCH_CHECK(positions.is_cuda() && positions.dtype() == at::kLong &&
              positions.is_contiguous() && positions.size(0) == T);
  const bool own = dkv.numel() > 0;
  int rank = 0;
  if (own) {
    TORCH_CHECK(dkv.dim() == 2 && dkv.size(0) == T && dkv.stride(1) == 1 &&
                dkv.dtype() == q.dtype());
    rank = dkv.size(1) - 2 * R;
    TORCH_CHECK(rank > 0);
    KAITO_CHECK_F32(norm_w);
    TORCH_CHECK(norm_w.numel() == rank);
    TORCH_CHECK(cache.is_contiguous() && cache.dtype() == q.dtype() &&
                cache.dim() == 3 && cache.size(2) == rank + 2 * R);
    TORCH_CHECK(slot_mapping.is_cuda() && slot_mapping.dtype() == at::kLong &&
                slot_mapping.is_contiguous() && slot_mapping.size(0) == T);
  }
  if (T == 0) return;
  auto stream = at::hip::getCurrentHIPStream();
  const int items = H + (own ? 1 : 0);
  TORCH_CHECK(items <= 4 * 65535);
  // 16-byte moves for the copied and the zeroed parts of a head
  const int ve = 16 / (int)q.element_size();
  const int HDo = q_out.size(2);
  const bool vec = dim % ve == 0 && HD % ve == 0 && HDo % ve == 0 &&
      q.stride(0) % ve == 0 && ((uintptr_t)q.data_ptr()) % 16 == 0 &&
      ((uintptr_t)q_out.data_ptr()) % 16 == 0;
  KAITO_DISPATCH_ACT(q, {
    hipLaunchKernelGGL((latent_rope_cache_write_kernel<act_t>),
        dim3(T, (items + 3) / 4), dim3(256), 0, stream,
        (act_t*)q_out.data_ptr(), (const act_t*)q.data_ptr(), q.stride(0),
        own ? (const act_t*)dkv.data_ptr() : nullptr,
        own ? dkv.stride(0) : 0, own ? norm_w.data_ptr<float>() : nullptr,
        (float)eps, own ? (act_t*)cache.data_ptr() : nullptr,
        own ? slot_mapping.data_ptr<int64_t>() : nullptr,
        positions.data_ptr<int64_t>(), inv_freq.data_ptr<float>(), H,
        (int)dim, R, rank, HDo, vec, interleaved, (float)rot_mag);
  });
}

void latent_attention(at::Tensor out, at::Tensor q, at::Tensor cache,
                      at::Tensor block_tables, at::Tensor token_seq,
                      at::Tensor positions, double scale, at::Tensor sinks) {
  TORCH_CHECK(q.is_cuda() && q.dim() == 3 && q.is_contiguous() &&
              is_act_dtype(q));
  const int T = q.size(0), H = q.size(1), DT = q.size(2);
  TORCH_CHECK(cache.is_contiguous() && cache.dtype() == q.dtype() &&
              cache.dim() == 3 && cache.size(2) == DT);
  const int BS = cache.size(1);
  TORCH_CHECK(out.is_contiguous() && out.dtype() == q.dtype() &&
              out.dim() == 3 && out.size(0) == T && out.size(1) == H);
  const int rank = out.size(2);
  TORCH_CHECK(rank > 0 && rank <= DT && rank <= 32 * LA_MAXI,
              "latent rank up to ", 32 * LA_MAXI);
  KAITO_CHECK_I32(block_tables); KAITO_CHECK_I32(token_seq);
  TORCH_CHECK(block_tables.dim() == 2 && token_seq.size(0) == T);
  TORCH_CHECK(positions.is_cuda() && positions.dtype() == at::kLong &&
              positions.is_contiguous() && positions.size(0) == T);
  const bool sk = sinks.numel() > 0;
  if (sk) { KAITO_CHECK_F32(sinks); TORCH_CHECK(sinks.numel() == H); }
  TORCH_CHECK((int64_t)cache.size(0) * BS < (1ll << 31));
  if (T == 0) return;
  auto stream = at::hip::getCurrentHIPStream();
  // bf16 with 16-byte chunks per row: the MFMA kernel
  if (q.dtype() == at::kBFloat16 && DT % 8 == 0 && rank % 8 == 0 &&
      DT <= 640 && rank <= 512) {
    const int tiles_h = (H + 15) / 16;
    // enough workgroups for the chip when rows x head tiles are few
    // (one workgroup per CU: a tile pair of 32 rows takes most of its LDS)
    int S = (256 + T * tiles_h - 1) / std::max(1, T * tiles_h);
    S = std::max(1, std::min(S, 16));
    const int DTp = (DT + 31) & ~31, rankp = (rank + 15) & ~15;
    const size_t lds = (size_t)(32 * (DTp + 8) + rankp * LM_KTP +
                                2 * 16 * LM_KTP) * 2 +
        (size_t)(4 * 16 * 32 + 48) * 4;
    at::Tensor pacc, pml;
    if (S > 1) {
      pacc = at::empty({T, S, H, rank}, q.options().dtype(at::kFloat));
      pml = at::empty({T, S, H, 2}, q.options().dtype(at::kFloat));
    }
    const bool small = DT <= 256 && rank <= 128;
    auto launch = [&](auto kern) {
      static bool raised = false;
      if (!raised) {
        HIP_CHECK_KAITO(hipFuncSetAttribute(
            reinterpret_cast<const void*>(kern),
            hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
        raised = true;
      }
      hipLaunchKernelGGL(kern, dim3(T, tiles_h, S), dim3(256), lds, stream,
          (short*)out.data_ptr(), S > 1 ? pacc.data_ptr<float>() : nullptr,
          S > 1 ? pml.data_ptr<float>() : nullptr,
          (const short*)q.data_ptr(), (const short*)cache.data_ptr(),
          block_tables.data_ptr<int>(), (int)block_tables.size(1),
          token_seq.data_ptr<int>(), positions.data_ptr<int64_t>(),
          (float)scale, sk ? sinks.data_ptr<float>() : nullptr, H, DT, rank,
          BS, S);
    };
    if (small) launch(&latent_attention_mfma_kernel<2, 2>);
    else launch(&latent_attention_mfma_kernel<5, 8>);
    if (S > 1)
      hipLaunchKernelGGL(latent_merge_kernel, dim3(T, H), dim3(128), 0, stream,
          (short*)out.data_ptr(), pacc.data_ptr<float>(),
          pml.data_ptr<float>(), H, rank, S);
    return;
  }
  const int pad = q.dtype() == at::kFloat ? 1 : 2;
  const size_t lds = (size_t)(LA_HT * DT + LA_HT * LA_KT) * 4 +
      (size_t)LA_KT * (DT + pad) * q.element_size();
  TORCH_CHECK(lds <= 160 * 1024, "latent row too wide for this kernel: ", DT);
  TORCH_CHECK(H <= 65535 * LA_HT);
  KAITO_DISPATCH_ACT(q, {
    // raised once per element type, to the most a workgroup may take
    static bool raised = false;
    if (lds > 48 * 1024 && !raised) {
      HIP_CHECK_KAITO(hipFuncSetAttribute(
          reinterpret_cast<const void*>(&latent_attention_kernel<act_t>),
          hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
      raised = true;
    }
    hipLaunchKernelGGL((latent_attention_kernel<act_t>),
        dim3(T, (H + LA_HT - 1) / LA_HT), dim3(256), lds, stream,
        (act_t*)out.data_ptr(), (const act_t*)q.data_ptr(),
        (const act_t*)cache.data_ptr(), block_tables.data_ptr<int>(),
        (int)block_tables.size(1), token_seq.data_ptr<int>(),
        positions.data_ptr<int64_t>(), (float)scale,
        sk ? sinks.data_ptr<float>() : nullptr, H, DT, rank, BS);
  });
}

void latent_expand(at::Tensor k_s, at::Tensor v_s, at::Tensor kn,
                   at::Tensor vv, at::Tensor lat, int64_t H, int64_t D,
                   int64_t V, int64_t rank) {
  TORCH_CHECK(lat.is_cuda() && lat.dim() == 2 && lat.is_contiguous() &&
              is_act_dtype(lat));
  const int N = lat.size(0), P = lat.size(1) - rank;
  TORCH_CHECK(P >= 0 && rank > 0);
  TORCH_CHECK(kn.is_contiguous() && kn.dtype() == lat.dtype() &&
              kn.dim() == 2 && kn.size(0) == N && kn.size(1) == H * D);
  TORCH_CHECK(vv.is_contiguous() && vv.dtype() == lat.dtype() &&
              vv.dim() == 2 && vv.size(0) == N && vv.size(1) == H * V);
  TORCH_CHECK(k_s.is_contiguous() && v_s.is_contiguous() &&
              k_s.dtype() == lat.dtype() && v_s.dtype() == lat.dtype() &&
              k_s.dim() == 4 && v_s.dim() == 4);
  const int BS = k_s.size(2), Dp = k_s.size(3), Vp = v_s.size(3);
  TORCH_CHECK(k_s.size(1) == H && v_s.size(1) == H && v_s.size(2) == BS &&
              v_s.size(0) == k_s.size(0) && Dp >= D + P && Vp >= V);
  TORCH_CHECK((int64_t)k_s.size(0) * BS >= N, "scratch has too few pages");
  if (N == 0) return;
  TORCH_CHECK(H <= 65535);
  auto stream = at::hip::getCurrentHIPStream();
  KAITO_DISPATCH_ACT(lat, {
    hipLaunchKernelGGL((latent_expand_kernel<act_t>), dim3(N, (int)H),
        dim3(64), 0, stream, (act_t*)k_s.data_ptr(), (act_t*)v_s.data_ptr(),
        (const act_t*)kn.data_ptr(), (const act_t*)vv.data_ptr(),
        (const act_t*)lat.data_ptr(), (int)H, (int)D, (int)V, P, (int)rank,
        Dp, Vp, BS);
  });
}

}  // namespace kaito

TORCH_LIBRARY_FRAGMENT(kaito, m) {
  m.def("bigram_embed(Tensor(a!) out, Tensor ids, Tensor embed, float scale, Tensor table, int buckets, int mul_prev, int mul_cur, Tensor(b!) prev_state, Tensor cu_seqlens, Tensor state_slots, Tensor seq_starts, Tensor token_seq) -> ()");
  m.def("latent_rope_cache_write(Tensor(a!) q_out, Tensor q, Tensor dkv, Tensor norm_w, float eps, Tensor(b!) cache, Tensor slot_mapping, Tensor positions, Tensor inv_freq, int dim, bool interleaved, float rot_mag) -> ()");
  m.def("latent_attention(Tensor(a!) out, Tensor q, Tensor cache, Tensor block_tables, Tensor token_seq, Tensor positions, float scale, Tensor sinks) -> ()");
  m.def("latent_expand(Tensor(a!) k_s, Tensor(b!) v_s, Tensor kn, Tensor vv, Tensor lat, int H, int D, int V, int rank) -> ()");
}
TORCH_LIBRARY_IMPL(kaito, CUDA, m) {
  m.impl("bigram_embed", &kaito::bigram_embed);
  m.impl("latent_rope_cache_write", &kaito::latent_rope_cache_write);
  m.impl("latent_attention", &kaito::latent_attention);
  m.impl("latent_expand", &kaito::latent_expand);
}
