// Paged latent attention (gfx950): position-free, absorbed form.
//
//   ctx[t, a, :] = sum_j softmax_j(scale * q~[t, a, :] . c_j) * c_j,  j <= pos(t)
//
// where c_j (width R) are the cached latents of row t's sequence, read
// through its block table. Keys AND values are the same latent row, so a
// key tile staged in LDS serves the score product and the weighted sum.
// All heads of a row — and all rows of a sequence — read the same stream:
// a workgroup takes a tile of up to 16 (row, head) pairs of ONE sequence
// (host-built list: 16 rows x 1 head for long portions, rows x heads for
// decode rows) and walks that sequence's latents once for all of them.
//
// Pool layout: [nblocks, P, BS, R]. Plane 0 holds a page's latents row by
// row ([BS][R]); bf16 pools carry a second plane with the same page
// transposed ([R][BS]) so that BOTH matrix products of the MFMA path find
// their reduction axis contiguous: scores reduce over R (plane 0), the
// weighted sum reduces over keys (plane 1).
//
// Two paths. The MFMA path (bf16 pool with both planes, BS = 16, R % 32
// == 0) rounds the scaled q~ and the softmax weights to bf16 and runs both
// products on v_mfma_f32_16x16x32_bf16 with fp32 accumulation; softmax
// statistics stay fp32. Per 64-key tile: wave w multiplies the tile's 16
// pairs with keys 16w..16w+15 (B operand straight from plane 0, 16 B per
// lane), scores meet in LDS for the online softmax, then wave w owns the
// output channels of n-tiles w, w+4, ... and multiplies P (A operand, LDS)
// with plane 1. The exact path: fp32 scores, fp32 online softmax, fp32
// weighted sums on the vector ALUs, for pools of bf16 or fp32 latents and
// any R. Per key tile: (1) 256 lanes stage KT latent rows as fp32 in LDS
// (row stride R+1: conflict-free for the per-key dots), (2) lane (pair e,
// key slot kk) computes the pair's scores against keys kk, kk+16, ..., the
// 16 lanes of a pair reduce max/sum with shuffles and update the running
// (m, l), (3) wave w accumulates pairs w, w+4, w+8, w+12: lane i owns
// channels i, i+64, ... of each.
#include "common.h"

namespace {

constexpr int G = 16;         // (row, head) pairs per workgroup
constexpr int THREADS = 256;

template <typename T> DEVICE_INLINE float ldf(const T* p);
template <> DEVICE_INLINE float ldf<float>(const float* p) { return *p; }
template <> DEVICE_INLINE float ldf<unsigned short>(const unsigned short* p) {
  return bf2f(*p);
}

// tiles: int32 [ntiles, 6] = row0, nrows, head0, nheads, seq, (unused)
template <typename TC, int NJ, int KT>
__global__ __launch_bounds__(THREADS) void latent_attn_exact_kernel(
    float* __restrict__ ctx, const float* __restrict__ q_lat,
    const TC* __restrict__ cache, const int* __restrict__ block_tables,
    const int* __restrict__ tiles, const int* __restrict__ pos32, float scale,
    int T, int H, int R, int BS, int nseq, int maxb, int nblocks,
    long page_stride, long q_rs, long q_hs, long o_rs, long o_hs) {
  extern __shared__ float sm[];
  const int RS = R + 1;
  float* qs = sm;                    // [G][R]
  float* ks = qs + G * R;            // [KT][RS]
  float* ps = ks + KT * RS;          // [G][KT]
  float* als = ps + G * KT;          // [G] rescale of the running sum
  float* lsum = als + G;             // [G] final denominators
  __shared__ int e_pos[G];
  __shared__ long e_off[G];          // pair's offset into q_lat
  __shared__ long e_out[G];          // pair's offset into ctx

  const int* tl = tiles + (long)blockIdx.x * 6;
  const int row0 = tl[0], nrows = tl[1], head0 = tl[2], nheads = tl[3];
  const int seq = tl[4];
  const int n_ent = nrows * nheads;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  // a tile that does not fit the operands is skipped, never dereferenced
  if (row0 < 0 || nrows < 1 || row0 + nrows > T || head0 < 0 || nheads < 1 ||
      head0 + nheads > H || n_ent > G || seq < 0 || seq >= nseq)
    return;

  if (tid < G) {
    int p = -1;
    long off = 0, oo = 0;
    if (tid < n_ent) {
      const int row = row0 + tid / nheads;
      const int head = head0 + tid % nheads;
      p = min(max(pos32[row], 0), maxb * BS - 1);
      off = (long)row * q_rs + (long)head * q_hs;
      oo = (long)row * o_rs + (long)head * o_hs;
    }
    e_pos[tid] = p;
    e_off[tid] = off;
    e_out[tid] = oo;
  }
  __syncthreads();
  int jmax = -1;
#pragma unroll
  for (int e = 0; e < G; ++e) jmax = max(jmax, e_pos[e]);
  // queries, pre-scaled
  for (int e = wave; e < G; e += 4) {
    const bool ok = e < n_ent;
    const float* qp = q_lat + e_off[e];
    for (int r = lane; r < R; r += 64) qs[e * R + r] = ok ? qp[r] * scale : 0.f;
  }

  // score-phase role: pair e_s, key slots kk, kk+16, ...
  const int e_s = tid >> 4, kk = tid & 15;
  const int my_pos = e_pos[e_s];
  float m_run = -INFINITY, l_run = 0.f;
  // sum-phase role: pairs wave + 4*i, channels lane + 64*j
  float acc[4][NJ];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < NJ; ++j) acc[i][j] = 0.f;

  const int* bt = block_tables + (long)seq * maxb;
  for (int k0 = 0; k0 <= jmax; k0 += KT) {
    __syncthreads();   // previous tile fully consumed (and qs written)
    for (int k = wave; k < KT; k += 4) {
      const int j = k0 + k;
      float* dst = ks + k * RS;
      if (j <= jmax) {
        const int blk = min(max(bt[j / BS], 0), nblocks - 1);
        const TC* src = cache + (long)blk * page_stride + (long)(j % BS) * R;
        for (int r = lane; r < R; r += 64) dst[r] = ldf(src + r);
      } else {
        for (int r = lane; r < R; r += 64) dst[r] = 0.f;
      }
    }
    __syncthreads();
    // (2) scores
    float s[KT / 16];
#pragma unroll
    for (int u = 0; u < KT / 16; ++u) s[u] = 0.f;
    {
      const float* qp = qs + e_s * R;
      for (int r = 0; r < R; ++r) {
        const float qv = qp[r];
#pragma unroll
        for (int u = 0; u < KT / 16; ++u) s[u] += qv * ks[(kk + 16 * u) * RS + r];
      }
    }
    float mx = -INFINITY;
#pragma unroll
    for (int u = 0; u < KT / 16; ++u) {
      if (k0 + kk + 16 * u > my_pos) s[u] = -INFINITY;
      mx = fmaxf(mx, s[u]);
    }
#pragma unroll
    for (int m = 8; m >= 1; m >>= 1) mx = fmaxf(mx, __shfl_xor(mx, m, WAVE_SIZE));
    const float m_new = fmaxf(m_run, mx);
    float alpha = 1.f, psum = 0.f;
    if (m_new == -INFINITY) {        // nothing visible yet (padding pair)
#pragma unroll
      for (int u = 0; u < KT / 16; ++u) ps[e_s * KT + kk + 16 * u] = 0.f;
    } else {
      alpha = expf(m_run - m_new);   // exp(-inf) = 0 on the first tile
#pragma unroll
      for (int u = 0; u < KT / 16; ++u) {
        const float p = expf(s[u] - m_new);
        ps[e_s * KT + kk + 16 * u] = p;
        psum += p;
      }
    }
    psum = group16_reduce_sum(psum);
    l_run = l_run * alpha + psum;
    m_run = m_new;
    if (kk == 0) als[e_s] = alpha;
    __syncthreads();
    // (3) weighted sums
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float a = als[wave + 4 * i];
#pragma unroll
      for (int j = 0; j < NJ; ++j) acc[i][j] *= a;
    }
    for (int k = 0; k < KT; ++k) {
      float kv[NJ];
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        const int r = lane + 64 * j;
        kv[j] = r < R ? ks[k * RS + r] : 0.f;
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float p = ps[(wave + 4 * i) * KT + k];
#pragma unroll
        for (int j = 0; j < NJ; ++j) acc[i][j] += p * kv[j];
      }
    }
  }
  if (kk == 0) lsum[e_s] = l_run;
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int e = wave + 4 * i;
    if (e >= n_ent) continue;
    const float inv = 1.0f / lsum[e];
    float* op = ctx + e_out[e];
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      const int r = lane + 64 * j;
      if (r < R) op[r] = acc[i][j] * inv;
    }
  }
}

template <typename TC, int NJ, int KT>
void launch_exact(float* ctx, const float* q_lat, const void* cache,
                  const int* bt, const int* tiles, const int* pos32, int ntiles,
                  float scale, int T, int H, int R, int BS, int nseq, int maxb,
                  int nblocks, long page_stride, long q_rs, long q_hs,
                  long o_rs, long o_hs, hipStream_t s) {
  const size_t smem =
      (size_t)(G * R + KT * (R + 1) + G * KT + 2 * G) * sizeof(float);
  auto kern = latent_attn_exact_kernel<TC, NJ, KT>;
  if (smem > 48 * 1024)
    (void)hipFuncSetAttribute((const void*)kern,
                              hipFuncAttributeMaxDynamicSharedMemorySize,
                              (int)smem);
  kern<<<ntiles, THREADS, smem, s>>>(ctx, q_lat, (const TC*)cache, bt, tiles,
                                     pos32, scale, T, H, R, BS, nseq, maxb,
                                     nblocks, page_stride, q_rs, q_hs, o_rs,
                                     o_hs);
}


// ---- MFMA path ---------------------------------------------------------------

typedef __attribute__((ext_vector_type(8))) short la_s16x8;

DEVICE_INLINE f32x4 la_mfma(u16x8 a, u16x8 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(
      __builtin_bit_cast(la_s16x8, a), __builtin_bit_cast(la_s16x8, b), c, 0, 0, 0);
}

constexpr int MKT = 64;            // keys per tile (16 per wave)
constexpr int MSS = MKT + 4;       // fp32 score row stride
constexpr int MPS = MKT + 8;       // bf16 weight row stride (16 B aligned)

template <typename T> DEVICE_INLINE void stf(T* p, float v);
template <> DEVICE_INLINE void stf<float>(float* p, float v) { *p = v; }
template <> DEVICE_INLINE void stf<unsigned short>(unsigned short* p, float v) {
  *p = f2bf(v);
}

// NT: 16-channel n-tiles per wave (wave w owns n-tiles w, w+4, ...).
// TQ / TO: q~ and ctx element types (fp32 or bf16), addressed through row
// and head strides so the batched projections around the kernel need no
// transposing copies. gridDim.y > 1 splits every tile's key range evenly
// over that many workgroups (few tiles, long contexts: decode); each then
// leaves an unnormalised partial (acc, m, l) for latent_attn_merge_kernel.
template <int NT, typename TQ, typename TO>
__global__ __launch_bounds__(THREADS) void latent_attn_mfma_kernel(
    TO* __restrict__ ctx, const TQ* __restrict__ q_lat,
    const unsigned short* __restrict__ pool,
    const int* __restrict__ block_tables, const int* __restrict__ tiles,
    const int* __restrict__ pos32, float scale, int T, int H, int R, int nseq,
    int maxb, int nblocks, long page_stride, long q_rs, long q_hs, long o_rs,
    long o_hs, float* __restrict__ ws_acc, float* __restrict__ ws_ml) {
  constexpr int BS = 16;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  const int QS = R + 8;                               // bf16 row stride
  unsigned short* Ql = reinterpret_cast<unsigned short*>(smem_raw);  // [G][QS]
  unsigned short* Pl = Ql + G * QS;                   // [G][MPS]
  float* Ss = reinterpret_cast<float*>(Pl + G * MPS); // [G][MSS]
  float* als = Ss + G * MSS;                          // [G]
  float* lsum = als + G;                              // [G]
  __shared__ int e_pos[G];
  __shared__ long e_off[G];
  __shared__ long e_out[G];

  const int* tl = tiles + (long)blockIdx.x * 6;
  const int row0 = tl[0], nrows = tl[1], head0 = tl[2], nheads = tl[3];
  const int seq = tl[4];
  const int n_ent = nrows * nheads;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int lc = lane & 15, lg = lane >> 4;
  if (row0 < 0 || nrows < 1 || row0 + nrows > T || head0 < 0 || nheads < 1 ||
      head0 + nheads > H || n_ent > G || seq < 0 || seq >= nseq)
    return;

  if (tid < G) {
    int p = -1;
    long off = 0, oo = 0;
    if (tid < n_ent) {
      const int row = row0 + tid / nheads;
      const int head = head0 + tid % nheads;
      p = min(max(pos32[row], 0), maxb * BS - 1);
      off = (long)row * q_rs + (long)head * q_hs;
      oo = (long)row * o_rs + (long)head * o_hs;
    }
    e_pos[tid] = p;
    e_off[tid] = off;
    e_out[tid] = oo;
  }
  __syncthreads();
  int jmax = -1;
#pragma unroll
  for (int e = 0; e < G; ++e) jmax = max(jmax, e_pos[e]);
  for (int e = wave; e < G; e += 4) {
    const bool ok = e < n_ent;
    const TQ* qp = q_lat + e_off[e];
    for (int r = lane; r < R; r += 64)
      Ql[e * QS + r] = f2bf(ok ? ldf(qp + r) * scale : 0.f);
  }

  const int e_s = tid >> 4, kk = tid & 15;    // softmax role
  const int my_pos = e_pos[e_s];
  float m_run = -INFINITY, l_run = 0.f;
  f32x4 acc[NT];
#pragma unroll
  for (int i = 0; i < NT; ++i) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};

  const int* bt = block_tables + (long)seq * maxb;
  const int last_page = jmax >> 4;
  const int nsplit = gridDim.y, split = blockIdx.y;
  const int per = ((jmax + MKT) / MKT + nsplit - 1) / nsplit;   // key tiles
  const int kbeg = split * per * MKT;
  const int kend = min(jmax + 1, kbeg + per * MKT);
  for (int k0 = kbeg; k0 < kend; k0 += MKT) {
    __syncthreads();   // Ql staged / previous tile's Pl and als consumed
    {
      // scores: this wave's 16 keys; keys past jmax re-read key jmax (their
      // weights are masked to zero below)
      const int key = min(k0 + wave * 16 + lc, jmax);
      const int blk = min(max(bt[key >> 4], 0), nblocks - 1);
      const unsigned short* rowp =
          pool + (long)blk * page_stride + (long)(key & 15) * R;
      const unsigned short* qrow = Ql + lc * QS;
      f32x4 sacc{0.f, 0.f, 0.f, 0.f};
      // several key loads in flight per wave: the products are short
#pragma unroll 4
      for (int r = 0; r < R; r += 32) {
        const u16x8 a = *reinterpret_cast<const u16x8*>(qrow + r + lg * 8);
        const u16x8 b = *reinterpret_cast<const u16x8*>(rowp + r + lg * 8);
        sacc = la_mfma(a, b, sacc);
      }
#pragma unroll
      for (int r = 0; r < 4; ++r)
        Ss[(lg * 4 + r) * MSS + wave * 16 + lc] = sacc[r];
    }
    __syncthreads();
    {
      float sv[4];
      float mx = -INFINITY;
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        sv[u] = Ss[e_s * MSS + kk + 16 * u];
        if (k0 + kk + 16 * u > my_pos) sv[u] = -INFINITY;
        mx = fmaxf(mx, sv[u]);
      }
#pragma unroll
      for (int m = 8; m >= 1; m >>= 1) mx = fmaxf(mx, __shfl_xor(mx, m, WAVE_SIZE));
      const float m_new = fmaxf(m_run, mx);
      float alpha = 1.f, psum = 0.f;
      if (m_new == -INFINITY) {
#pragma unroll
        for (int u = 0; u < 4; ++u) Pl[e_s * MPS + kk + 16 * u] = 0;
      } else {
        alpha = __expf(m_run - m_new);
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const float p = __expf(sv[u] - m_new);
          Pl[e_s * MPS + kk + 16 * u] = f2bf(p);
          psum += p;
        }
      }
      psum = group16_reduce_sum(psum);
      l_run = l_run * alpha + psum;
      m_run = m_new;
      if (kk == 0) als[e_s] = alpha;
    }
    __syncthreads();
    {
      float ar[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) ar[r] = als[lg * 4 + r];
#pragma unroll
      for (int i = 0; i < NT; ++i)
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[i][r] *= ar[r];
#pragma unroll
      for (int ks = 0; ks < MKT; ks += 32) {
        const u16x8 a =
            *reinterpret_cast<const u16x8*>(Pl + lc * MPS + ks + lg * 8);
        // 8 consecutive keys of one page; groups wholly past jmax read the
        // last valid page (weights there are zero)
        const int keyb = k0 + ks + lg * 8;
        const int pg = min(keyb >> 4, last_page);
        const int blk = min(max(bt[pg], 0), nblocks - 1);
        const unsigned short* pt =
            pool + (long)blk * page_stride + (long)BS * R + (keyb & 15);
#pragma unroll
        for (int i = 0; i < NT; ++i) {
          const int ch = (wave + 4 * i) * 16 + lc;
          if ((wave + 4 * i) * 16 < R) {       // uniform over the wave
            const u16x8 b = *reinterpret_cast<const u16x8*>(pt + (long)ch * BS);
            acc[i] = la_mfma(a, b, acc[i]);
          }
        }
      }
    }
  }
  if (nsplit > 1) {
    const long slot = (long)blockIdx.x * nsplit + split;
    if (kk == 0) {
      ws_ml[(slot * G + e_s) * 2] = m_run;
      ws_ml[(slot * G + e_s) * 2 + 1] = l_run;
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int e = lg * 4 + r;
      float* wp = ws_acc + (slot * G + e) * R;
#pragma unroll
      for (int i = 0; i < NT; ++i) {
        const int ch = (wave + 4 * i) * 16 + lc;
        if (ch < R) wp[ch] = acc[i][r];
      }
    }
    return;
  }
  if (kk == 0) lsum[e_s] = l_run;
  __syncthreads();
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int e = lg * 4 + r;
    if (e >= n_ent) continue;
    const float inv = 1.0f / lsum[e];
    TO* op = ctx + e_out[e];
#pragma unroll
    for (int i = 0; i < NT; ++i) {
      const int ch = (wave + 4 * i) * 16 + lc;
      if (ch < R) stf(op + ch, acc[i][r] * inv);
    }
  }
}

// ctx = sum_s acc_s exp(m_s - M) / sum_s l_s exp(m_s - M) over a tile's
// splits; one workgroup of 128 lanes per (tile, pair)
constexpr int MERGE_THREADS = 128;

template <typename TO>
__global__ __launch_bounds__(MERGE_THREADS) void latent_attn_merge_kernel(
    TO* __restrict__ ctx, const int* __restrict__ tiles,
    const float* __restrict__ ws_acc, const float* __restrict__ ws_ml,
    int nsplit, int T, int H, int R, long o_rs, long o_hs) {
  const int* tl = tiles + (long)blockIdx.x * 6;
  const int row0 = tl[0], nrows = tl[1], head0 = tl[2], nheads = tl[3];
  const int n_ent = nrows * nheads;
  const int e = blockIdx.y;
  if (row0 < 0 || nrows < 1 || row0 + nrows > T || head0 < 0 || nheads < 1 ||
      head0 + nheads > H || n_ent > G || e >= n_ent)
    return;
  const long base = (long)blockIdx.x * nsplit;
  float M = -INFINITY;
  for (int s = 0; s < nsplit; ++s)
    M = fmaxf(M, ws_ml[((base + s) * G + e) * 2]);
  float L = 0.f;
  for (int s = 0; s < nsplit; ++s) {
    const float* ml = ws_ml + ((base + s) * G + e) * 2;
    if (ml[0] != -INFINITY) L += ml[1] * __expf(ml[0] - M);
  }
  const float inv = 1.0f / L;
  const int row = row0 + e / nheads, head = head0 + e % nheads;
  TO* op = ctx + (long)row * o_rs + (long)head * o_hs;
  for (int ch = threadIdx.x; ch < R; ch += MERGE_THREADS) {
    float v = 0.f;
    for (int s = 0; s < nsplit; ++s) {
      const float m = ws_ml[((base + s) * G + e) * 2];
      if (m != -INFINITY)
        v += ws_acc[((base + s) * G + e) * R + ch] * __expf(m - M);
    }
    stf(op + ch, v * inv);
  }
}

template <int NT, typename TQ, typename TO>
void launch_mfma(void* ctx, const void* q_lat, const void* cache,
                 const int* bt, const int* tiles, const int* pos32, int ntiles,
                 float scale, int T, int H, int R, int nseq, int maxb,
                 int nblocks, long page_stride, long q_rs, long q_hs, long o_rs,
                 long o_hs, int nsplit, float* ws_acc, float* ws_ml,
                 hipStream_t s) {
  const size_t smem = (size_t)G * (R + 8) * 2 + (size_t)G * MPS * 2 +
                      (size_t)(G * MSS + 2 * G) * sizeof(float);
  latent_attn_mfma_kernel<NT, TQ, TO><<<dim3(ntiles, nsplit), THREADS, smem, s>>>(
      (TO*)ctx, (const TQ*)q_lat, (const unsigned short*)cache, bt, tiles,
      pos32, scale, T, H, R, nseq, maxb, nblocks, page_stride, q_rs, q_hs,
      o_rs, o_hs, ws_acc, ws_ml);
  if (nsplit > 1)
    latent_attn_merge_kernel<TO><<<dim3(ntiles, G), MERGE_THREADS, 0, s>>>(
        (TO*)ctx, tiles, ws_acc, ws_ml, nsplit, T, H, R, o_rs, o_hs);
}

template <typename TQ, typename TO>
void dispatch_mfma(void* ctx, const void* q_lat, const void* cache,
                   const int* bt, const int* tiles, const int* pos32,
                   int ntiles, float scale, int T, int H, int R, int nseq,
                   int maxb, int nblocks, long page_stride, long q_rs,
                   long q_hs, long o_rs, long o_hs, int nsplit, float* ws_acc,
                   float* ws_ml, hipStream_t s) {
#define LM_ARGS ctx, q_lat, cache, bt, tiles, pos32, ntiles, scale, T, H, R, nseq, maxb, nblocks, page_stride, q_rs, q_hs, o_rs, o_hs, nsplit, ws_acc, ws_ml, s
  const int nt = (R / 16 + 3) / 4;
  if (nt <= 1) launch_mfma<1, TQ, TO>(LM_ARGS);
  else if (nt <= 2) launch_mfma<2, TQ, TO>(LM_ARGS);
  else if (nt <= 4) launch_mfma<4, TQ, TO>(LM_ARGS);
  else if (nt <= 8) launch_mfma<8, TQ, TO>(LM_ARGS);
  else launch_mfma<16, TQ, TO>(LM_ARGS);
#undef LM_ARGS
}

template <typename TC>
void dispatch_exact(float* ctx, const float* q_lat, const void* cache,
                    const int* bt, const int* tiles, const int* pos32,
                    int ntiles, float scale, int T, int H, int R, int BS,
                    int nseq, int maxb, int nblocks, long page_stride,
                    long q_rs, long q_hs, long o_rs, long o_hs,
                    hipStream_t s) {
#define LA_ARGS ctx, q_lat, cache, bt, tiles, pos32, ntiles, scale, T, H, R, BS, nseq, maxb, nblocks, page_stride, q_rs, q_hs, o_rs, o_hs, s
  if (R <= 64) launch_exact<TC, 1, 32>(LA_ARGS);
  else if (R <= 128) launch_exact<TC, 2, 32>(LA_ARGS);
  else if (R <= 256) launch_exact<TC, 4, 32>(LA_ARGS);
  else if (R <= 512) launch_exact<TC, 8, 32>(LA_ARGS);
  else launch_exact<TC, 16, 16>(LA_ARGS);
#undef LA_ARGS
}

}  // namespace

// largest latent width the exact path's LDS tiling covers
int latent_attn_max_rank() { return 1024; }

// 1 when (pool dtype, planes, page size, width) take the MFMA path
int latent_attn_uses_mfma(int cache_bf, int planes, int BS, int R) {
  return cache_bf && planes == 2 && BS == 16 && R % 32 == 0 && R <= 1024;
}

// io_bf: q~ and ctx are bf16 (MFMA path only), else fp32. nsplit > 1 needs
// ws_acc [ntiles*nsplit*16*R] and ws_ml [ntiles*nsplit*16*2] fp32.
void latent_attention_launch(void* ctx, const void* q_lat, const void* cache,
                             const int* block_tables, const int* tiles,
                             const int* pos32, int ntiles, float scale, int T,
                             int H, int R, int BS, int nseq, int maxb,
                             int nblocks, int planes, int cache_bf,
                             int force_exact, int io_bf, long q_rs, long q_hs,
                             long o_rs, long o_hs, int nsplit, float* ws_acc,
                             float* ws_ml, hipStream_t s) {
  if (ntiles == 0) return;
  const long page_stride = (long)planes * BS * R;
  if (!force_exact && latent_attn_uses_mfma(cache_bf, planes, BS, R)) {
    if (io_bf)
      dispatch_mfma<unsigned short, unsigned short>(
          ctx, q_lat, cache, block_tables, tiles, pos32, ntiles, scale, T, H, R,
          nseq, maxb, nblocks, page_stride, q_rs, q_hs, o_rs, o_hs, nsplit,
          ws_acc, ws_ml, s);
    else
      dispatch_mfma<float, float>(
          ctx, q_lat, cache, block_tables, tiles, pos32, ntiles, scale, T, H, R,
          nseq, maxb, nblocks, page_stride, q_rs, q_hs, o_rs, o_hs, nsplit,
          ws_acc, ws_ml, s);
    return;
  }
  if (cache_bf)
    dispatch_exact<unsigned short>((float*)ctx, (const float*)q_lat, cache,
                                   block_tables, tiles, pos32, ntiles, scale, T,
                                   H, R, BS, nseq, maxb, nblocks, page_stride,
                                   q_rs, q_hs, o_rs, o_hs, s);
  else
    dispatch_exact<float>((float*)ctx, (const float*)q_lat, cache, block_tables,
                          tiles, pos32, ntiles, scale, T, H, R, BS, nseq, maxb,
                          nblocks, page_stride, q_rs, q_hs, o_rs, o_hs, s);
}
