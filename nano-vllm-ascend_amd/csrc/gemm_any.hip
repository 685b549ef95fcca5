// General-shape projections with fp32 activations: y = alpha * x . w^T for ANY M, N, K (no multiple-of-64 contract),
// weights bf16 or fp32 as stored ([N][K] row-major), fp32 accumulation, fp32 output - plain, and grouped over
// expert-sorted rows (one launch for all experts of a sparse feed-forward, SwiGLU optionally in the epilogue).
//
// These serve the model families whose residual stream, norms and recurrences are kept in 32-bit floats and whose
// widths are not the fragment-native kernels' (csrc/gemm_skinny*.hpp, gemm_tile.hip): four kernels,
//
//   gemm_any_mfma_kernel   bf16 weights: a 64 x 64 (from 512 rows: 128 x 128, with SwiGLU 128 x 64) output tile per 4-wave
//                          workgroup, x rounded to bf16 on its way into LDS, v_mfma_f32_16x16x32_bf16, the next K
//                          step's operands fetched while the current one is multiplied, edges zero-filled
//   gemm_any_skinny_kernel bf16 weights, up to 64 rows per tile (decode batches, a decode step's experts): 16 features per
//                          workgroup, the waves split K, fragments straight from memory
//   gemm_any_fma_kernel    true 32-bit: fp32 (or bf16, widened exactly) weights, x NOT rounded, plain FMA chains in k
//                          order - the float32 serving mode, and the routers of sparse feed-forwards in either mode
//   gemm_any_rows_kernel   M <= 8 rows, and the exact mode up to 64: one wave per (output feature, batch of rows)
//                          streams its weight row once, lanes split K in 16-byte pieces, butterfly reduction; both
//                          dtypes, x not rounded
//
// A row of the result is a function of its own x row and the weights only: the summation order over k does not depend
// on M, on the row's place in the batch or on the tile it falls into (each kernel has ONE fixed order), so the same
// token gives the same bits whatever it is batched with, within one kernel; between kernels (a row computed in a
// prompt's portion vs alone) results differ by rounding only.
#include "mi_common.hpp"

namespace mi {

struct GemmAnyArgs {
  const float* x;
  int64_t ldx;
  const void* w;    // [groups][N][K]
  const void* w2;   // nullptr, or the second weight of the SwiGLU epilogue: y = silu(x w^T) * (x w2^T)
  float* y;
  int64_t ldy;
  int M, N, K;
  float alpha;
  const int32_t* group_offsets;  // nullptr: one group of M rows; else rows of group g = [off[g], off[g + 1])
  const int32_t* x_rows;         // nullptr or the x row of each (sorted) row
  const int32_t* y_rows;         // nullptr or the y row of each (sorted) row
  // epilogue: v = acc + bias[n]; with w2: v = act(v) * (acc2 + bias2[n]), else v = act(v); v *= alpha;
  // gate: v *= sigmoid(gate[y row][n])
  const float* bias;
  const float* bias2;
  int act;  // MI_ACT_*
  const float* gate;
  int64_t ldgate;
  // batched form (group_offsets == nullptr, gridDim.z > 1): batch b multiplies the M rows at x + b * x_batch with
  // w[b] into y + b * y_batch (a per-head projection of head-major rows: the batch stride is a head's width)
  int64_t x_batch, y_batch, gate_batch;
  // grouped form: sorted row m's accumulators are multiplied by row_scale[row_scale_rows ? row_scale_rows[m] : m] before
  // anything else (= its x row scaled, without touching x: an expert whose routing weight goes into its INPUT)
  const float* row_scale;
  const int32_t* row_scale_rows;
  float limit;  // MI_ACT_CLAMPED_GLU
};

template <typename TW>
__device__ __forceinline__ float w_load(const TW* p);
template <>
__device__ __forceinline__ float w_load<float>(const float* p) { return *p; }
template <>
__device__ __forceinline__ float w_load<uint16_t>(const uint16_t* p) { return bf2f(*p); }

__device__ __forceinline__ bool dev_aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
__device__ __forceinline__ float silu_f(float z) { return z / (1.f + expf(-z)); }
__device__ __forceinline__ float act_f(int act, float z) {
  switch (act) {
    case MI_ACT_SILU: return silu_f(z);
    case MI_ACT_GELU_TANH: return 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
    case MI_ACT_GELU_ERF: return 0.5f * z * (1.f + erff(z * 0.7071067811865476f));
    case MI_ACT_SIGMOID: return 1.f / (1.f + expf(-z));
    default: return z;  // (MI_ACT_SOFTCAP is finish()'s: it needs the cap)
  }
}
// what every kernel does to an accumulator (pair) before it stores it
template <bool DUAL>
__device__ __forceinline__ float finish(const GemmAnyArgs& a, int64_t m, int64_t yrow, int n, float v, float v2) {
  if (a.row_scale) {
    const float rs = a.row_scale[a.row_scale_rows ? a.row_scale_rows[m] : m];
    v *= rs, v2 *= rs;
  }
  if (a.bias) v += a.bias[n];
  if (DUAL) {
    if (a.bias2) v2 += a.bias2[n];
    if (a.act == MI_ACT_CLAMPED_GLU) {  // g sigmoid(1.702 g) (u + 1) with g capped from above, u clamped to +-limit
      const float g = fminf(v, a.limit), u = fminf(fmaxf(v2, -a.limit), a.limit);
      v = g / (1.f + expf(-1.702f * g)) * (u + 1.f);
    } else {
      v = act_f(a.act, v) * v2;
    }
  } else {
    v = a.act == MI_ACT_SOFTCAP ? tanhf(v / a.alpha) : act_f(a.act, v);  // (times alpha below: alpha tanh(v / alpha))
  }
  v *= a.alpha;
  if (a.gate) v *= 1.f / (1.f + expf(-a.gate[yrow * a.ldgate + n]));
  return v;
}
// the operands of this workgroup's group (grouped form) or batch (batched form)
template <typename TW, bool DUAL>
__device__ __forceinline__ void select_group(GemmAnyArgs& a, const TW*& w, const TW*& w2, int& m_lo, int& m_hi) {
  m_lo = 0, m_hi = a.M;
  w = static_cast<const TW*>(a.w);
  w2 = static_cast<const TW*>(a.w2);
  if (a.group_offsets) {
    m_lo = a.group_offsets[blockIdx.z];
    m_hi = a.group_offsets[blockIdx.z + 1];
  } else if (blockIdx.z > 0) {
    a.x += (int64_t)blockIdx.z * a.x_batch;
    a.y += (int64_t)blockIdx.z * a.y_batch;
    if (a.gate) a.gate += (int64_t)blockIdx.z * a.gate_batch;
  }
  w += (int64_t)blockIdx.z * a.N * a.K;
  if (DUAL) w2 += (int64_t)blockIdx.z * a.N * a.K;
}

// eight consecutive operands as floats: one 16-byte (bf16) / two 16-byte (fp32) loads, or element-wise at an edge
template <typename TW>
__device__ __forceinline__ void load8(const TW* p, int n_valid, bool vec, float (&v)[8]);
template <>
__device__ __forceinline__ void load8<uint16_t>(const uint16_t* p, int n_valid, bool vec, float (&v)[8]) {
  if (vec && n_valid >= 8) {
    const u32x4 w = *reinterpret_cast<const u32x4*>(p);
    v[0] = lo_bf(w[0]), v[1] = hi_bf(w[0]), v[2] = lo_bf(w[1]), v[3] = hi_bf(w[1]);
    v[4] = lo_bf(w[2]), v[5] = hi_bf(w[2]), v[6] = lo_bf(w[3]), v[7] = hi_bf(w[3]);
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = i < n_valid ? bf2f(p[i]) : 0.f;
  }
}
template <>
__device__ __forceinline__ void load8<float>(const float* p, int n_valid, bool vec, float (&v)[8]) {
  if (vec && n_valid >= 8) {
    const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
    v[0] = a.x, v[1] = a.y, v[2] = a.z, v[3] = a.w, v[4] = b.x, v[5] = b.y, v[6] = b.z, v[7] = b.w;
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = i < n_valid ? p[i] : 0.f;
  }
}

// ---------------------------------------------------------------------------------------------------------------
// exact kernel: 64 x 64 tile, 256 threads, 4 x 4 outputs per thread, k ascending
// ---------------------------------------------------------------------------------------------------------------
template <typename TW, bool DUAL, int RT>  // RT rows per thread: a 64 x 64 tile (4) or 16 x 64 (1: few features, many rows)
__global__ __launch_bounds__(256) void gemm_any_fma_kernel(GemmAnyArgs a) {
  constexpr int BM = 16 * RT, BN = 64, BK = 32, PAD = 4;
  __shared__ float As[BK][BM + PAD];
  __shared__ float Bs[DUAL ? 2 : 1][BK][BN + PAD];
  const int tid = threadIdx.x;
  int m_lo, m_hi;
  const TW *w, *w2;
  select_group<TW, DUAL>(a, w, w2, m_lo, m_hi);
  const int m0 = m_lo + blockIdx.y * BM;
  if (m0 >= m_hi) return;
  const int n0 = blockIdx.x * BN;
  const int lr = tid >> 2, lk = (tid & 3) * 8;  // this thread stages 8 consecutive k of one row
  int64_t xrow = -1;
  if (lr < BM && m0 + lr < m_hi) xrow = a.x_rows ? a.x_rows[m0 + lr] : m0 + lr;
  const int wrow = n0 + lr < a.N ? n0 + lr : -1;
  float acc[DUAL ? 2 : 1][RT][4] = {};
  const int ty = tid >> 4, tx = tid & 15;
  for (int k0 = 0; k0 < a.K; k0 += BK) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int k = k0 + lk + i;
      if (lr < BM) As[lk + i][lr] = (xrow >= 0 && k < a.K) ? a.x[xrow * a.ldx + k] : 0.f;
      Bs[0][lk + i][lr] = (wrow >= 0 && k < a.K) ? w_load<TW>(w + (int64_t)wrow * a.K + k) : 0.f;
      if (DUAL) Bs[1][lk + i][lr] = (wrow >= 0 && k < a.K) ? w_load<TW>(w2 + (int64_t)wrow * a.K + k) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < BK; ++k) {
      float av[RT], bv[DUAL ? 2 : 1][4];
#pragma unroll
      for (int i = 0; i < RT; ++i) av[i] = As[k][ty * RT + i];
#pragma unroll
      for (int d = 0; d < (DUAL ? 2 : 1); ++d)
#pragma unroll
        for (int j = 0; j < 4; ++j) bv[d][j] = Bs[d][k][tx * 4 + j];
#pragma unroll
      for (int d = 0; d < (DUAL ? 2 : 1); ++d)
#pragma unroll
        for (int i = 0; i < RT; ++i)
#pragma unroll
          for (int j = 0; j < 4; ++j) acc[d][i][j] = fmaf(av[i], bv[d][j], acc[d][i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < RT; ++i) {
    const int m = m0 + ty * RT + i;
    if (m >= m_hi) continue;
    const int64_t yrow = a.y_rows ? a.y_rows[m] : m;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n >= a.N) continue;
      a.y[yrow * a.ldy + n] = finish<DUAL>(a, m, yrow, n, acc[0][i][j], acc[DUAL ? 1 : 0][i][j]);
    }
  }
}

// ---------------------------------------------------------------------------------------------------------------
// MFMA kernel (bf16 weights): 4 waves as 2 x 2, each FM x FN fragments of 16 x 16 - a 64 x 64 tile, or 128 x 128
// (SwiGLU: 128 x 64) for prefill-sized launches, where every LDS fragment feeds four MFMAs instead of two;
// K in steps of 64 (a weight row's piece = one 128-byte line).  LDS holds the tile's x rows and weight rows as bf16
// [64][64 + 8].
// ---------------------------------------------------------------------------------------------------------------
template <bool DUAL, int FM, int FN>  // a wave's tile: FM x FN fragments of 16 x 16; the workgroup's: 2 x 2 waves
__global__ __launch_bounds__(256) void gemm_any_mfma_kernel(GemmAnyArgs a) {
  constexpr int BM = 32 * FM, BN = 32 * FN, BK = 64, LD = BK + 8;
  constexpr int ND = DUAL ? 2 : 1;
  __shared__ __attribute__((aligned(16))) uint16_t As[BM][LD];
  __shared__ __attribute__((aligned(16))) uint16_t Bs[ND][BN][LD];
  const int tid = threadIdx.x;
  int m_lo, m_hi;
  const uint16_t *w, *w2;
  select_group<uint16_t, DUAL>(a, w, w2, m_lo, m_hi);
  const int m0 = m_lo + blockIdx.y * BM;
  if (m0 >= m_hi) return;
  const int n0 = blockIdx.x * BN;
  // staging: a thread takes 16 consecutive k of one row (a row's 64 k = one 128-byte line of weights), 64 rows per pass
  const int lr = tid >> 2, lk = (tid & 3) * 16;
  int64_t xrow[BM / 64];
  int wrow[BN / 64];
#pragma unroll
  for (int p = 0; p < BM / 64; ++p) {
    const int m = m0 + p * 64 + lr;
    xrow[p] = m < m_hi ? (a.x_rows ? a.x_rows[m] : m) : -1;
  }
#pragma unroll
  for (int p = 0; p < BN / 64; ++p) wrow[p] = n0 + p * 64 + lr < a.N ? n0 + p * 64 + lr : -1;
  const bool w_vec = (a.K % 8 == 0) && dev_aligned16(a.w) && (!DUAL || dev_aligned16(a.w2));
  const bool x_vec = (a.ldx % 4 == 0) && dev_aligned16(a.x);
  const int wave = tid >> 6, lane = tid & 63;
  const int wm = (wave >> 1) * 16 * FM, wn = (wave & 1) * 16 * FN;
  const int fr = lane & 15, fk = (lane >> 4) * 8;
  f32x4 acc[ND][FM][FN];
#pragma unroll
  for (int d = 0; d < ND; ++d)
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
      for (int j = 0; j < FN; ++j) acc[d][i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
  // the tile's operands travel memory -> registers -> LDS; the registers of K step k + 1 are loaded while step k's
  // MFMAs run, so the global-memory latency is not paid between the two barriers
  u32x4 xreg[2][BM / 64], wreg[ND][2][BN / 64];
  auto fetch = [&](int k0) {
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      const int k = k0 + lk + half * 8;
#pragma unroll
      for (int p = 0; p < BM / 64; ++p) {
        float xv[8];
        if (xrow[p] >= 0) load8<float>(a.x + xrow[p] * a.ldx + k, a.K - k, x_vec, xv);
        else {
#pragma unroll
          for (int i = 0; i < 8; ++i) xv[i] = 0.f;
        }
        xreg[half][p] = u32x4{pack_bf(xv[0], xv[1]), pack_bf(xv[2], xv[3]), pack_bf(xv[4], xv[5]), pack_bf(xv[6], xv[7])};
      }
#pragma unroll
      for (int d = 0; d < ND; ++d)
#pragma unroll
        for (int p = 0; p < BN / 64; ++p) {
          const uint16_t* wp = (d ? w2 : w) + (int64_t)wrow[p] * a.K + k;
          u32x4 v = {0u, 0u, 0u, 0u};
          if (wrow[p] >= 0 && k < a.K) {
            if (w_vec && k + 8 <= a.K) {
              v = *reinterpret_cast<const u32x4*>(wp);
            } else {
              uint16_t e[8];
#pragma unroll
              for (int i = 0; i < 8; ++i) e[i] = k + i < a.K ? wp[i] : (uint16_t)0;
              v = u32x4{(uint32_t)e[0] | ((uint32_t)e[1] << 16), (uint32_t)e[2] | ((uint32_t)e[3] << 16),
                        (uint32_t)e[4] | ((uint32_t)e[5] << 16), (uint32_t)e[6] | ((uint32_t)e[7] << 16)};
            }
          }
          wreg[d][half][p] = v;
        }
    }
  };
  fetch(0);
  for (int k0 = 0; k0 < a.K; k0 += BK) {
#pragma unroll
    for (int half = 0; half < 2; ++half) {
#pragma unroll
      for (int p = 0; p < BM / 64; ++p) *reinterpret_cast<u32x4*>(&As[p * 64 + lr][lk + half * 8]) = xreg[half][p];
#pragma unroll
      for (int d = 0; d < ND; ++d)
#pragma unroll
        for (int p = 0; p < BN / 64; ++p) *reinterpret_cast<u32x4*>(&Bs[d][p * 64 + lr][lk + half * 8]) = wreg[d][half][p];
    }
    __syncthreads();
    if (k0 + BK < a.K) fetch(k0 + BK);
    // D[n][m] = sum_k W[n][k] X[m][k]: weights on the MFMA's row axis, so a lane's four results are four consecutive
    // FEATURES of one x row
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      bf16x8 af[FM], bfr[ND][FN];
#pragma unroll
      for (int i = 0; i < FM; ++i) af[i] = as_frag(*reinterpret_cast<const u32x4*>(&As[wm + i * 16 + fr][ks * 32 + fk]));
#pragma unroll
      for (int d = 0; d < ND; ++d)
#pragma unroll
        for (int j = 0; j < FN; ++j)
          bfr[d][j] = as_frag(*reinterpret_cast<const u32x4*>(&Bs[d][wn + j * 16 + fr][ks * 32 + fk]));
#pragma unroll
      for (int d = 0; d < ND; ++d)
#pragma unroll
        for (int i = 0; i < FM; ++i)
#pragma unroll
          for (int j = 0; j < FN; ++j)
            acc[d][i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(bfr[d][j], af[i], acc[d][i][j], 0, 0, 0);
    }
    __syncthreads();
  }
  // fragment (i, j): x row = wm + i*16 + (lane & 15), features wn + j*16 + (lane >> 4) * 4 + r
#pragma unroll
  for (int i = 0; i < FM; ++i) {
    const int m = m0 + wm + i * 16 + (lane & 15);
    if (m >= m_hi) continue;
    const int64_t yrow = a.y_rows ? a.y_rows[m] : m;
#pragma unroll
    for (int j = 0; j < FN; ++j) {
      const int n = n0 + wn + j * 16 + (lane >> 4) * 4;
      float v[4];
#pragma unroll
      for (int r = 0; r < 4; ++r)
        v[r] = n + r < a.N ? finish<DUAL>(a, m, yrow, n + r, acc[0][i][j][r], acc[ND - 1][i][j][r]) : 0.f;
      float* yp = a.y + yrow * a.ldy + n;
      if (n + 4 <= a.N && (a.ldy % 4 == 0) && dev_aligned16(a.y)) {
        *reinterpret_cast<float4*>(yp) = float4{v[0], v[1], v[2], v[3]};
      } else {
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (n + r < a.N) yp[r] = v[r];
      }
    }
  }
}

// ---------------------------------------------------------------------------------------------------------------
// up to 64 rows per tile (decode batches, a decode step's experts): 16 output features per workgroup, so that even a
// 1024-feature projection spreads over 64 workgroups; the four waves take the K steps of 32 in turn (together they read
// 256 contiguous bytes of every weight row per round), operands go from memory straight into MFMA fragments - no LDS
// staging, no barrier inside the K loop - and the waves' accumulators are added in wave order through LDS at the end.
// ---------------------------------------------------------------------------------------------------------------
template <bool DUAL, int MF>  // MF fragments of 16 rows
__global__ __launch_bounds__(256) void gemm_any_skinny_kernel(GemmAnyArgs a) {
  __shared__ __attribute__((aligned(16))) float red[3][DUAL ? 2 : 1][MF][64][4];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  int m_lo, m_hi;
  const uint16_t *w, *w2;
  select_group<uint16_t, DUAL>(a, w, w2, m_lo, m_hi);
  const int m0 = m_lo + blockIdx.y * 16 * MF;
  if (m0 >= m_hi) return;
  const int n0 = blockIdx.x * 16;
  const int fr = lane & 15, kk = (lane >> 4) * 8;
  const int wrow = n0 + fr < a.N ? n0 + fr : -1;
  int64_t xrow[MF];
#pragma unroll
  for (int f = 0; f < MF; ++f) {
    const int m = m0 + f * 16 + fr;
    xrow[f] = m < m_hi ? (a.x_rows ? a.x_rows[m] : m) : -1;
  }
  const bool w_vec = (a.K % 8 == 0) && dev_aligned16(a.w) && (!DUAL || dev_aligned16(a.w2));
  const bool x_vec = (a.ldx % 4 == 0) && dev_aligned16(a.x);
  f32x4 acc[DUAL ? 2 : 1][MF];
#pragma unroll
  for (int d = 0; d < (DUAL ? 2 : 1); ++d)
#pragma unroll
    for (int f = 0; f < MF; ++f) acc[d][f] = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int k0 = wave * 32; k0 < a.K; k0 += 4 * 32) {
    const int k = k0 + kk;
    bf16x8 wf[DUAL ? 2 : 1];
#pragma unroll
    for (int d = 0; d < (DUAL ? 2 : 1); ++d) {
      const uint16_t* wp = (d ? w2 : w) + (int64_t)wrow * a.K + k;
      u32x4 v = {0u, 0u, 0u, 0u};
      if (wrow >= 0 && k < a.K) {
        if (w_vec && k + 8 <= a.K) {
          v = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(wp));
        } else {
          uint16_t e[8];
#pragma unroll
          for (int i = 0; i < 8; ++i) e[i] = k + i < a.K ? wp[i] : (uint16_t)0;
          v = u32x4{(uint32_t)e[0] | ((uint32_t)e[1] << 16), (uint32_t)e[2] | ((uint32_t)e[3] << 16),
                    (uint32_t)e[4] | ((uint32_t)e[5] << 16), (uint32_t)e[6] | ((uint32_t)e[7] << 16)};
        }
      }
      wf[d] = as_frag(v);
    }
#pragma unroll
    for (int f = 0; f < MF; ++f) {
      float xv[8];
      if (xrow[f] >= 0) load8<float>(a.x + xrow[f] * a.ldx + k, a.K - k, x_vec, xv);
      else {
#pragma unroll
        for (int i = 0; i < 8; ++i) xv[i] = 0.f;
      }
      const bf16x8 xf = as_frag(u32x4{pack_bf(xv[0], xv[1]), pack_bf(xv[2], xv[3]), pack_bf(xv[4], xv[5]), pack_bf(xv[6], xv[7])});
#pragma unroll
      for (int d = 0; d < (DUAL ? 2 : 1); ++d)
        acc[d][f] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[d], xf, acc[d][f], 0, 0, 0);
    }
  }
  if (wave > 0) {
#pragma unroll
    for (int d = 0; d < (DUAL ? 2 : 1); ++d)
#pragma unroll
      for (int f = 0; f < MF; ++f) *reinterpret_cast<f32x4*>(red[wave - 1][d][f][lane]) = acc[d][f];
  }
  __syncthreads();
  if (wave > 0) return;
#pragma unroll
  for (int ow = 0; ow < 3; ++ow)
#pragma unroll
    for (int d = 0; d < (DUAL ? 2 : 1); ++d)
#pragma unroll
      for (int f = 0; f < MF; ++f) acc[d][f] += *reinterpret_cast<const f32x4*>(red[ow][d][f][lane]);
  // a lane holds features n0 + (lane >> 4) * 4 + r of x row (lane & 15) of every fragment
#pragma unroll
  for (int f = 0; f < MF; ++f) {
    const int m = m0 + f * 16 + fr;
    if (m >= m_hi) continue;
    const int64_t yrow = a.y_rows ? a.y_rows[m] : m;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int n = n0 + (lane >> 4) * 4 + r;
      if (n >= a.N) continue;
      a.y[yrow * a.ldy + n] = finish<DUAL>(a, m, yrow, n, acc[0][f][r], acc[DUAL ? 1 : 0][f][r]);
    }
  }
}

// ---------------------------------------------------------------------------------------------------------------
// few rows: one wave per output feature and batch of MT rows (blockIdx.y); the lanes take K in pieces of 8, ascending,
// 16-byte loads where the operands allow it, then a butterfly over the lanes
// ---------------------------------------------------------------------------------------------------------------
template <typename TW, int MT, bool DUAL>
__global__ __launch_bounds__(256) void gemm_any_rows_kernel(GemmAnyArgs a) {
  const int lane = threadIdx.x & 63;
  const int n = blockIdx.x * 4 + (threadIdx.x >> 6);
  int m_lo, m_hi;
  const TW *w, *w2;
  select_group<TW, DUAL>(a, w, w2, m_lo, m_hi);
  const int m0 = m_lo + blockIdx.y * MT;
  if (n >= a.N || m0 >= m_hi) return;  // (whole waves: the reductions below see all 64 lanes)
  const bool w_vec = a.K % 8 == 0 && dev_aligned16(a.w) && (!DUAL || dev_aligned16(a.w2));
  const bool x_vec = a.ldx % 4 == 0 && dev_aligned16(a.x);
  float acc[DUAL ? 2 : 1][MT] = {};
  int64_t xr[MT];
#pragma unroll
  for (int r = 0; r < MT; ++r) xr[r] = m0 + r < m_hi ? (a.x_rows ? a.x_rows[m0 + r] : m0 + r) : -1;
  for (int k0 = lane * 8; k0 < a.K; k0 += 64 * 8) {
    float wv[DUAL ? 2 : 1][8];
    load8<TW>(w + (int64_t)n * a.K + k0, a.K - k0, w_vec, wv[0]);
    if (DUAL) load8<TW>(w2 + (int64_t)n * a.K + k0, a.K - k0, w_vec, wv[DUAL ? 1 : 0]);
#pragma unroll
    for (int r = 0; r < MT; ++r) {
      if (xr[r] < 0) continue;
      float xv[8];
      load8<float>(a.x + xr[r] * a.ldx + k0, a.K - k0, x_vec, xv);
#pragma unroll
      for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int d = 0; d < (DUAL ? 2 : 1); ++d) acc[d][r] = fmaf(xv[i], wv[d][i], acc[d][r]);
    }
  }
#pragma unroll
  for (int r = 0; r < MT; ++r) {
    const float v = wave_sum(acc[0][r]);
    const float v2 = DUAL ? wave_sum(acc[DUAL ? 1 : 0][r]) : 0.f;
    if (lane == 0 && xr[r] >= 0) {
      const int64_t yrow = a.y_rows ? a.y_rows[m0 + r] : m0 + r;
      a.y[yrow * a.ldy + n] = finish<DUAL>(a, m0 + r, yrow, n, v, v2);
    }
  }
}

template <typename TW, bool DUAL>
static int launch_any(const GemmAnyArgs& a, int groups, int rows_per_group_max, int mode, hipStream_t st) {
  // mode 0: product (MFMA for bf16 weights, the row kernel for few rows); 1: exact (FMA chains / row kernel, x unrounded)
  // few rows (per group): the weight-streaming row kernel.  Also the exact mode up to 64 rows: a router's few output
  // features would make one tile of the FMA kernel walk all of K alone
  const bool few = rows_per_group_max <= 8 || (mode == 1 && rows_per_group_max <= 64);
  if (few) {
    const int mt = rows_per_group_max <= 1 ? 1 : rows_per_group_max <= 4 ? 4 : 8;
    const dim3 grid((a.N + 3) / 4, (rows_per_group_max + mt - 1) / mt, groups);
    if (mt == 1) hipLaunchKernelGGL((gemm_any_rows_kernel<TW, 1, DUAL>), grid, dim3(256), 0, st, a);
    else if (mt == 4) hipLaunchKernelGGL((gemm_any_rows_kernel<TW, 4, DUAL>), grid, dim3(256), 0, st, a);
    else hipLaunchKernelGGL((gemm_any_rows_kernel<TW, 8, DUAL>), grid, dim3(256), 0, st, a);
    return check_launch();
  }
  const dim3 grid((a.N + 63) / 64, (rows_per_group_max + 63) / 64, groups);
  if constexpr (sizeof(TW) == 2) {
    if (mode == 0 && rows_per_group_max >= 512 && a.N >= 128) {  // prefill-sized: 128-row tiles, 128 (SwiGLU: 64) features
      if (DUAL) {
        hipLaunchKernelGGL((gemm_any_mfma_kernel<DUAL, 4, 2>), dim3((a.N + 63) / 64, (rows_per_group_max + 127) / 128, groups),
                           dim3(256), 0, st, a);
      } else {
        hipLaunchKernelGGL((gemm_any_mfma_kernel<DUAL, 4, 4>), dim3((a.N + 127) / 128, (rows_per_group_max + 127) / 128, groups),
                           dim3(256), 0, st, a);
      }
      return check_launch();
    }
    if (mode == 0 && (rows_per_group_max <= 64 || (groups > 1 && rows_per_group_max <= 8 * groups))) {
      // decode-sized: 16-feature workgroups (grouped: tiles of 32 rows, an expert's few rows fill the first)
      if (groups > 1 || rows_per_group_max <= 32) {
        const dim3 g2((a.N + 15) / 16, (rows_per_group_max + 31) / 32, groups);
        hipLaunchKernelGGL((gemm_any_skinny_kernel<DUAL, 2>), g2, dim3(256), 0, st, a);
      } else {
        const dim3 g4((a.N + 15) / 16, 1, groups);
        hipLaunchKernelGGL((gemm_any_skinny_kernel<DUAL, 4>), g4, dim3(256), 0, st, a);
      }
      return check_launch();
    }
    if (mode == 0) {
      hipLaunchKernelGGL((gemm_any_mfma_kernel<DUAL, 2, 2>), grid, dim3(256), 0, st, a);
      return check_launch();
    }
  }
  if (a.N <= 64 && rows_per_group_max >= 1024) {  // a router over a prompt: one column of tiles - short tiles, more of them
    hipLaunchKernelGGL((gemm_any_fma_kernel<TW, DUAL, 1>), dim3(1, (rows_per_group_max + 15) / 16, groups), dim3(256), 0, st, a);
    return check_launch();
  }
  hipLaunchKernelGGL((gemm_any_fma_kernel<TW, DUAL, 4>), grid, dim3(256), 0, st, a);
  return check_launch();
}

}  // namespace mi

using namespace mi;

static int gemm_any_dispatch(const GemmAnyArgs& a, int w_dtype, int groups, int rows_max, int mode, hipStream_t st) {
  if (a.M == 0 || a.N == 0 || rows_max == 0) return MI_OK;
  if (w_dtype == MI_DTYPE_BF16)
    return a.w2 ? launch_any<uint16_t, true>(a, groups, rows_max, mode, st) : launch_any<uint16_t, false>(a, groups, rows_max, mode, st);
  if (w_dtype == MI_DTYPE_F32)
    return a.w2 ? launch_any<float, true>(a, groups, rows_max, mode, st) : launch_any<float, false>(a, groups, rows_max, mode, st);
  return MI_EINVAL;
}

static bool act_ok(int act) { return act >= MI_ACT_NONE && act <= MI_ACT_SOFTCAP; }

extern "C" int mi_gemm_any(const float* x, int64_t ldx, const void* w, int w_dtype, float* y, int64_t ldy, int M, int N,
                           int K, float alpha, int exact, mi_stream stream) {
  return mi_gemm_any_act(x, ldx, w, nullptr, w_dtype, nullptr, nullptr, MI_ACT_NONE, y, ldy, M, N, K, alpha, exact, stream);
}

extern "C" int mi_gemm_any_act(const float* x, int64_t ldx, const void* w, const void* w2, int w_dtype, const float* bias,
                               const float* bias2, int act, float* y, int64_t ldy, int M, int N, int K, float alpha,
                               int exact, mi_stream stream) {
  if (!x || !w || !y || M < 0 || N < 0 || K < 1 || ldx < K || ldy < N || !act_ok(act) || (bias2 && !w2)) return MI_EINVAL;
  if (act == MI_ACT_SOFTCAP && (w2 || !(alpha > 0.f))) return MI_EINVAL;
  GemmAnyArgs a{x, ldx, w, w2, y, ldy, M, N, K, alpha, nullptr, nullptr, nullptr, bias, bias2, act, nullptr, 0, 0, 0, 0, nullptr, nullptr, 0.f};
  return gemm_any_dispatch(a, w_dtype, 1, M, exact ? 1 : 0, S(stream));
}

extern "C" int mi_gemm_any_batched(const float* x, int64_t ldx, int64_t x_batch, const void* w, int w_dtype, float* y,
                                   int64_t ldy, int64_t y_batch, const float* gate, int64_t ldgate, int64_t gate_batch,
                                   int n_batch, int M, int N, int K, int exact, mi_stream stream) {
  if (!x || !w || !y || n_batch < 1 || M < 0 || N < 0 || K < 1 || ldx < K || ldy < N) return MI_EINVAL;
  if (n_batch > 65535) return MI_EUNSUPPORTED;
  GemmAnyArgs a{x, ldx, w, nullptr, y, ldy, M, N, K, 1.0f, nullptr, nullptr, nullptr, nullptr, nullptr, MI_ACT_NONE,
                gate, ldgate, x_batch, y_batch, gate_batch, nullptr, nullptr, 0.f};
  return gemm_any_dispatch(a, w_dtype, n_batch, M, exact ? 1 : 0, S(stream));
}

extern "C" int mi_gemm_any_grouped(const float* x, int64_t ldx, const int32_t* x_rows, const void* w, const void* w2,
                                   int w_dtype, const int32_t* group_offsets, int n_groups, int rows_per_group_max,
                                   float* y, int64_t ldy, const int32_t* y_rows, int N, int K, int exact,
                                   mi_stream stream) {
  return mi_gemm_any_grouped_act(x, ldx, x_rows, w, w2, w_dtype, w2 ? MI_ACT_SILU : MI_ACT_NONE, group_offsets, n_groups,
                                 rows_per_group_max, y, ldy, y_rows, N, K, exact, stream);
}

extern "C" int mi_gemm_any_grouped_act(const float* x, int64_t ldx, const int32_t* x_rows, const void* w, const void* w2,
                                       int w_dtype, int act, const int32_t* group_offsets, int n_groups,
                                       int rows_per_group_max, float* y, int64_t ldy, const int32_t* y_rows, int N, int K,
                                       int exact, mi_stream stream) {
  if (act == MI_ACT_CLAMPED_GLU) return MI_EINVAL;  // (needs its limit: mi_gemm_any_grouped_glu)
  return mi_gemm_any_grouped_glu(x, ldx, x_rows, w, w2, w_dtype, act, 0.f, nullptr, nullptr, group_offsets, n_groups,
                                 rows_per_group_max, y, ldy, y_rows, N, K, exact, stream);
}

extern "C" int mi_gemm_any_grouped_glu(const float* x, int64_t ldx, const int32_t* x_rows, const void* w, const void* w2,
                                       int w_dtype, int act, float limit, const float* row_scale,
                                       const int32_t* row_scale_rows, const int32_t* group_offsets, int n_groups,
                                       int rows_per_group_max, float* y, int64_t ldy, const int32_t* y_rows, int N, int K,
                                       int exact, mi_stream stream) {
  if (!x || !w || !y || !group_offsets || n_groups < 1 || rows_per_group_max < 0 || N < 0 || K < 1 ||
      !(act_ok(act) || act == MI_ACT_CLAMPED_GLU) || act == MI_ACT_SOFTCAP)
    return MI_EINVAL;
  if (act == MI_ACT_CLAMPED_GLU && (!w2 || !(limit > 0.f))) return MI_EINVAL;
  if (row_scale_rows && !row_scale) return MI_EINVAL;
  if (n_groups > 65535) return MI_EUNSUPPORTED;
  GemmAnyArgs a{x, ldx, w, w2, y, ldy, rows_per_group_max, N, K, 1.0f, group_offsets, x_rows, y_rows, nullptr, nullptr,
                act, nullptr, 0, 0, 0, 0, row_scale, row_scale_rows, limit};
  return gemm_any_dispatch(a, w_dtype, n_groups, rows_per_group_max, exact ? 1 : 0, S(stream));
}
