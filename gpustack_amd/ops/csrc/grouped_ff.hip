// Grouped ungated expert feed-forward for decode-sized batches (gfx950):
//
//   u[j, :] = act(x[tok_j] . Wu[e_j]^T)        grouped_up_act
//   y[j, :] = u[j] . Wd[e_j]^T                  grouped_down
//
// over the expert-sorted assignment list j (tok_j, per-expert offsets and
// counts are computed on the device by the caller, so nothing here waits
// for the host and the launch grids — experts x 64-column tiles — do not
// depend on the routing outcome: the whole expert block can be captured
// in a hipGraph). A workgroup owns 64 output columns of one expert (16 per
// wave) and walks that expert's rows 16 at a time: the rows are staged in
// LDS in 512-element K chunks, the weight panel streams from HBM straight
// into the MFMA B operand (v_mfma_f32_16x16x32_bf16, fp32 accumulate). The
// panel is re-read per 16-row tile, which is free while experts hold a few
// rows (decode) and the reason prompts take per-expert library GEMMs.
// The routing weights are applied later, in fp32, by moe_combine.
#include "common.h"

namespace {

constexpr int GF_BN = 64;
constexpr int GF_KC = 512;
constexpr int GF_THREADS = 256;
constexpr int GF_LD = GF_KC + 8;   // LDS row stride (bf16), breaks bank cycle

typedef __attribute__((ext_vector_type(8))) short gf_s16x8;

DEVICE_INLINE f32x4 gf_mfma(u16x8 a, u16x8 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(
      __builtin_bit_cast(gf_s16x8, a), __builtin_bit_cast(gf_s16x8, b), c, 0, 0, 0);
}

DEVICE_INLINE float gf_act(float z, int mode) {
  switch (mode) {
    case 0: { const float r = fmaxf(z, 0.f); return r * r; }
    case 1: return 0.5f * z * (1.0f + erff(z * 0.70710678118654752f));
    case 2: {
      const float u = 0.7978845608028654f * (z + 0.044715f * z * z * z);
      return 0.5f * z * (1.0f + tanhf(u));
    }
    default: return z / (1.0f + expf(-z));
  }
}

// 16 rows x kc columns of src into LDS; rows come from tok[] (gather) or
// are consecutive from base_row; row ids are clamped to the source
DEVICE_INLINE void gf_stage(unsigned short* lds, const unsigned short* src,
                            long stride, const int* tok, int base_row,
                            int nrows, int k0, int kc, int tid, int src_rows) {
  const int per = kc / 8;
  for (int u = tid; u < 16 * per; u += GF_THREADS) {
    const int row = u / per;
    const int kk = (u % per) * 8;
    u16x8 val = {0, 0, 0, 0, 0, 0, 0, 0};
    if (row < nrows) {
      int r = tok != nullptr ? tok[row] : base_row + row;
      r = min(max(r, 0), src_rows - 1);
      val = *reinterpret_cast<const u16x8*>(src + (long)r * stride + k0 + kk);
    }
    *reinterpret_cast<u16x8*>(lds + row * GF_LD + kk) = val;
  }
}

// out[j, N] = f(src_rows(j) [K] . w[e, N, K]^T); GATHER: rows via tok
template <bool GATHER>
__global__ __launch_bounds__(GF_THREADS) void grouped_ff_kernel(
    unsigned short* __restrict__ out, const unsigned short* __restrict__ src,
    const unsigned short* __restrict__ w, const int* __restrict__ s_tok,
    const int* __restrict__ offs, const int* __restrict__ counts, int K, int N,
    int TK, int src_rows, int act_mode) {
  const int nnt = N / GF_BN;
  const int e = blockIdx.x / nnt;
  const int nt = blockIdx.x % nnt;
  const int base = min(max(offs[e], 0), TK);
  const int cnt = min(max(counts[e], 0), TK - base);
  if (cnt == 0) return;
  const int tid = threadIdx.x;
  const int lane = tid & (WAVE_SIZE - 1), wave = tid / WAVE_SIZE;
  const int lc = lane & 15, lg = lane >> 4;
  __shared__ unsigned short Xl[16 * GF_LD];
  const unsigned short* panel =
      w + ((long)e * N + nt * GF_BN + wave * 16 + lc) * K;
  for (int m0 = 0; m0 < cnt; m0 += 16) {
    const int nrows = min(16, cnt - m0);
    f32x4 acc{0.f, 0.f, 0.f, 0.f};
    for (int k0 = 0; k0 < K; k0 += GF_KC) {
      const int kc = min(GF_KC, K - k0);
      __syncthreads();
      gf_stage(Xl, src, K, GATHER ? s_tok + base + m0 : nullptr, base + m0,
               nrows, k0, kc, tid, src_rows);
      __syncthreads();
      auto body = [&](int kk) {
        const u16x8 a =
            *reinterpret_cast<const u16x8*>(Xl + lc * GF_LD + kk + lg * 8);
        const u16x8 b =
            *reinterpret_cast<const u16x8*>(panel + k0 + kk + lg * 8);
        acc = gf_mfma(a, b, acc);
      };
      if (kc == GF_KC) {
#pragma unroll
        for (int kk = 0; kk < GF_KC; kk += 32) body(kk);
      } else {
        for (int kk = 0; kk < kc; kk += 32) body(kk);
      }
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int row = lg * 4 + r;
      if (row >= nrows) continue;
      const float v = act_mode >= 0 ? gf_act(acc[r], act_mode) : acc[r];
      out[(long)(base + m0 + row) * N + nt * GF_BN + wave * 16 + lc] = f2bf(v);
    }
  }
}

}  // namespace

// K % 32 == 0 and N % 64 == 0 are checked by the caller
void grouped_up_act_launch(void* u, const void* x, const void* w,
                           const int* s_tok, const int* offs,
                           const int* counts, int E, int K, int N, int TK,
                           int T, int act_mode, hipStream_t s) {
  if (TK == 0) return;
  grouped_ff_kernel<true><<<E * (N / GF_BN), GF_THREADS, 0, s>>>(
      (unsigned short*)u, (const unsigned short*)x, (const unsigned short*)w,
      s_tok, offs, counts, K, N, TK, T, act_mode);
}

void grouped_down_launch(void* y, const void* u, const void* w,
                         const int* offs, const int* counts, int E, int K,
                         int N, int TK, hipStream_t s) {
  if (TK == 0) return;
  grouped_ff_kernel<false><<<E * (N / GF_BN), GF_THREADS, 0, s>>>(
      (unsigned short*)y, (const unsigned short*)u, (const unsigned short*)w,
      nullptr, offs, counts, K, N, TK, TK, -1);
}
