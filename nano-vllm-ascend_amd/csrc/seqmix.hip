// Sequence mixers and row operators of the model families that keep their residual stream in 32-bit floats:
//
//   mi_embedding_f32            table rows (bf16 or fp32) -> fp32 residual rows
//   mi_layernorm_f32            LayerNorm with weight and bias; optionally ADDED to a residual in place
//                               (x <- x + LN(y): the norm sits on the sublayer's output)
//   mi_swa_prepare              sliding-window attention, K/V side: ONE root-mean-square norm over a token's whole q
//                               projection and one over its whole k projection (not per head), optional mixing of the
//                               values with an earlier layer's values of the same token, K / V rows to the paged cache
//   mi_swa_attention            paged sliding-window attention with a per-head linear distance bias
//                               s_ij = scale q_i.k_j - slope_h (i - j), keys 0 <= i - j < window, separate key and value
//                               head sizes, grouped heads, optional sigmoid output gate; prompt portions and single
//                               decoded tokens in one launch (a row's keys are addressed through its sequence's block
//                               table and total length); three kernels: matrix cores for prompt portions over a bf16
//                               cache, 16-byte-load VALU form (decode: four waves per row and head), element-wise form
//   mi_causal_conv_silu         short causal depthwise convolution over time + SiLU, carried across steps by a
//   mi_causal_conv_state        per-sequence state slot holding the last taps - 1 inputs
//   mi_channel_delta            gated delta rule with one decay per head AND key channel:
//                               S <- diag(g_t) S;  u = beta_t (v_t - S^T k_t);  S <- S + k_t u^T;  o_t = S^T q_t
//                               with unit-norm q / k, per-head RMS norm of o, sigmoid gate; the fp32 state lives in a
//                               per-sequence slot (mi_channel_delta_state_elems floats) and is carried from step to step
//   mi_route_grouped            router of a sparse feed-forward: softmax scores, additive choice correction, choice
//                               restricted to the best groups of experts, top-k; weights = un-renormalised scores
//   mi_moe_combine_f32          out[t] = sum_k w[t][k] * (identity expert ? h[t] : y[t * top_k + k])
//   mi_causal_conv              the convolution with its activation and a "beside the identity" flag (y = x + conv(x))
//   mi_gated_norm_add_f32       res += rms(y * sigmoid(gate)) * w, and the norm of the sum for the next sublayer
//   mi_linear_attention         S <- diag(a_t) S + k_t v_t^T, o_t = S^T q_t with a decay per head or a forget gate per
//                               key channel that also writes (k = 1 - f); read-out norm per head or over all heads, gate
//   (further down: the pre-norm families' residual stack, minimal gated recurrence, latent and log-biased attention,
//   plain top-k routing - each with its own header comment)
//
// Everything here is computed in fp32 (expf / logf / sqrtf of the device library, no fast-math), for both serving
// dtypes: the bf16 mode differs only in the dtype of the WEIGHTS and of the K/V cache (and in the matrix-core attention
// of prompt portions, whose two products take q and the softmax weights as bf16 hi + lo pairs: fp32 quantities to 2^-17).
// A step's rows are described by cu_q [n_seqs + 1] (row range of each sequence) and kv_lens [n_seqs] (the sequence's
// length INCLUDING this step's rows): row r of sequence s sits at position kv_lens[s] - (cu_q[s+1] - cu_q[s]) + r.
#include "mi_common.hpp"

namespace mi {

__device__ __forceinline__ float sigmoid_f(float z) { return 1.f / (1.f + expf(-z)); }
__device__ __forceinline__ float softplus_f(float z) { return z > 20.f ? z : log1pf(expf(z)); }

template <typename T>
__device__ __forceinline__ float ld_f(const T* p);
template <>
__device__ __forceinline__ float ld_f<float>(const float* p) { return *p; }
template <>
__device__ __forceinline__ float ld_f<uint16_t>(const uint16_t* p) { return bf2f(*p); }
template <typename T>
__device__ __forceinline__ void st_f(T* p, float v);
template <>
__device__ __forceinline__ void st_f<float>(float* p, float v) { *p = v; }
template <>
__device__ __forceinline__ void st_f<uint16_t>(uint16_t* p, float v) { *p = f2bf(v); }

// sum over a 256-thread workgroup; every thread gets the result.  red: 4 floats of LDS per concurrent reduction.
__device__ __forceinline__ float block_sum256(float v, float* red) {
  v = wave_sum(v);
  __syncthreads();  // (red may still be read from the previous reduction)
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  return (red[0] + red[1]) + (red[2] + red[3]);
}

// the sequence a step row belongs to (n_seqs is small: a linear walk, identical on every lane)
__device__ __forceinline__ int seq_of_row(const int32_t* cu_q, int n_seqs, int row) {
  int s = 0;
  while (s + 1 < n_seqs && row >= cu_q[s + 1]) ++s;
  return s;
}

template <typename TT>
__global__ __launch_bounds__(256) void embedding_f32_kernel(const int64_t* __restrict__ ids, const TT* __restrict__ table,
                                                            float* __restrict__ out, int width, int vocab,
                                                            float scale) {
  const int64_t id = ids[blockIdx.x];
  if (id < 0 || id >= vocab) return;
  for (int c = threadIdx.x; c < width; c += 256)
    out[(int64_t)blockIdx.x * width + c] = ld_f<TT>(table + id * width + c) * scale;
}

// one workgroup per row; mean, then the mean of squared deviations (two passes over the row, which stays in L1)
__global__ __launch_bounds__(256) void layernorm_f32_kernel(const float* __restrict__ y, int64_t ldy,
                                                            const float* __restrict__ w, const float* __restrict__ b,
                                                            float* __restrict__ out, int64_t ldo, int width, float eps,
                                                            int add) {
  __shared__ float red[4];
  const float* yr = y + (int64_t)blockIdx.x * ldy;
  float s = 0.f;
  for (int c = threadIdx.x; c < width; c += 256) s += yr[c];
  const float mean = block_sum256(s, red) / (float)width;
  float q = 0.f;
  for (int c = threadIdx.x; c < width; c += 256) {
    const float d = yr[c] - mean;
    q += d * d;
  }
  const float var = block_sum256(q, red) / (float)width;
  const float rstd = 1.f / sqrtf(var + eps);
  float* o = out + (int64_t)blockIdx.x * ldo;
  for (int c = threadIdx.x; c < width; c += 256) {
    const float v = (yr[c] - mean) * rstd * w[c] + b[c];
    o[c] = add ? o[c] + v : v;
  }
}

// ---------------------------------------------------------------------------------------------------------------
// sliding-window attention
// ---------------------------------------------------------------------------------------------------------------
// One workgroup per step row.  q (qn values at proj + q_off) is normalised in place; k is normalised and stored; v is
// mixed (written back in place, so that a later layer can take it as ITS v_first only if this layer is the first mixing
// one - the caller keeps that tensor) and stored.  Cache layout [blocks][kv heads][block][dim], slot = block * block_size
// + offset, slot < 0: not stored.
template <typename TC>
__global__ __launch_bounds__(256) void swa_prepare_kernel(float* __restrict__ proj, int64_t ld, int q_off, int k_off,
                                                          int v_off, int nq, int nk, int nv,
                                                          const float* __restrict__ qn_w, const float* __restrict__ kn_w,
                                                          float eps, const float* __restrict__ v_first, int64_t ld_vf,
                                                          const float* __restrict__ lam_p, TC* __restrict__ k_cache,
                                                          TC* __restrict__ v_cache, const int32_t* __restrict__ slots,
                                                          int G, int D, int Dv, int block_size) {
  __shared__ float red[4];
  float* row = proj + (int64_t)blockIdx.x * ld;
  float sq = 0.f, sk = 0.f;
  for (int c = threadIdx.x; c < nq; c += 256) sq += row[q_off + c] * row[q_off + c];
  for (int c = threadIdx.x; c < nk; c += 256) sk += row[k_off + c] * row[k_off + c];
  const float rq = 1.f / sqrtf(block_sum256(sq, red) / (float)nq + eps);
  const float rk = 1.f / sqrtf(block_sum256(sk, red) / (float)nk + eps);
  for (int c = threadIdx.x; c < nq; c += 256) row[q_off + c] = row[q_off + c] * rq * qn_w[c];
  const int slot = slots[blockIdx.x];
  const int64_t blk = slot >= 0 ? slot / block_size : 0;
  const int off = slot >= 0 ? slot % block_size : 0;
  for (int c = threadIdx.x; c < nk; c += 256) {
    const float v = row[k_off + c] * rk * kn_w[c];
    if (slot >= 0) st_f<TC>(k_cache + ((blk * G + c / D) * block_size + off) * D + c % D, v);
  }
  const float lam = (v_first && lam_p) ? *lam_p : 0.f;
  for (int c = threadIdx.x; c < nv; c += 256) {
    float v = row[v_off + c];
    if (v_first) {
      v = (1.f - lam) * v + lam * v_first[(int64_t)blockIdx.x * ld_vf + c];
      row[v_off + c] = v;
    }
    if (slot >= 0) st_f<TC>(v_cache + ((blk * G + c / Dv) * block_size + off) * Dv + c % Dv, v);
  }
}

// Distance bias of a score, taken off it: kind MI_BIAS_SLOPE: 2^(-8 (h + 1) / H) * dist (p1 == nullptr) or p1[h] * dist;
// MI_BIAS_LOG: p1[h] * ln(1 + p2[h] * dist); MI_BIAS_NONE: nothing.  ldv: elements between two tokens' value rows (Dv,
// or the key row's length when the values are the leading channels of the key rows of the same cache).
// sink != nullptr: a row's softmax normalises by sum_j exp(s_j) + exp(sink[h]): the extra term is a learned per-head
// logit taken as it is (the score scale does not touch it) that only soaks up weight - nothing is added to the output
// for it.
// softcap > 0: the scaled, biased score s becomes softcap * tanh(s / softcap) before the mask and the softmax.
// value_heads: the value cache has this many heads (a divisor of the key heads G; query head h reads value head
// h / (H / value_heads)) - fewer, wider value heads than key heads let every query head weigh the values of SEVERAL
// key/value heads at once (value rows holding the heads side by side), which is what mixing the heads' softmax weights
// afterwards needs.
struct AttnBias {
  int kind;
  const float* p1;
  const float* p2;
  const float* sink;
  float softcap;
  int value_heads;
};
__device__ __forceinline__ float capped(const AttnBias& bias, float s) {
  return bias.softcap > 0.f ? bias.softcap * tanhf(s / bias.softcap) : s;
}
// the denominator of a finished row: its keys' sum l (relative to the running maximum m) plus the head's sink
__device__ __forceinline__ float with_sink(const AttnBias& bias, int h, float m, float l) {
  return bias.sink ? l + expf(bias.sink[h] - m) : l;
}
struct HeadBias {
  float a, b;
  bool log;
};
__device__ __forceinline__ HeadBias head_bias(const AttnBias& bias, int h, int H) {
  HeadBias r{0.f, 0.f, bias.kind == MI_BIAS_LOG};
  if (bias.kind == MI_BIAS_SLOPE) r.a = bias.p1 ? bias.p1[h] : exp2f(-8.f * (float)(h + 1) / (float)H);
  else if (bias.kind == MI_BIAS_LOG) r.a = bias.p1[h], r.b = bias.p2[h];
  return r;
}
__device__ __forceinline__ float dist_bias(const HeadBias& hb, int dist) {
  return hb.log ? hb.a * log1pf(hb.b * (float)dist) : hb.a * (float)dist;
}

// Row of a token in a paged cache [blocks][kv heads][block_size][.]: (table[key / block_size] * G + g) * block_size +
// key % block_size, in 32-bit arithmetic (rows of a cache are far fewer than 2^32; the byte offset is formed from it with
// one 32 x 32 -> 64-bit multiply-add), the division a shift when block_size is a power of two (bs_shift >= 0).
__device__ __forceinline__ int block_shift(int block_size) {
  return (block_size & (block_size - 1)) == 0 ? __builtin_ctz((unsigned)block_size) : -1;
}
__device__ __forceinline__ uint32_t cache_row(const int32_t* table, int key, int G, int g, int block_size, int bs_shift) {
  const int blk = bs_shift >= 0 ? key >> bs_shift : key / block_size;
  const int off = bs_shift >= 0 ? key & (block_size - 1) : key - blk * block_size;
  return ((uint32_t)table[blk] * (uint32_t)G + (uint32_t)g) * (uint32_t)block_size + (uint32_t)off;
}

// The general form (any head sizes): one wave per (row, head); lanes over keys for the scores, over value channels for
// the output, element-wise loads.
template <typename TC, int VPL>  // VPL: value channels per lane (Dv <= 64 * VPL)
__global__ __launch_bounds__(256) void swa_attention_kernel(const float* __restrict__ q, int64_t ldq,
                                                            const TC* __restrict__ k_cache, const TC* __restrict__ v_cache,
                                                            const int32_t* __restrict__ block_tables, int table_cols,
                                                            const int32_t* __restrict__ cu_q,
                                                            const int32_t* __restrict__ kv_lens, int n_seqs, int n_rows,
                                                            int H, int G, int D, int Dv, int block_size, int window,
                                                            float scale, AttnBias bias, int64_t ldv,
                                                            const float* __restrict__ gate, int64_t ldg,
                                                            float* __restrict__ out, int64_t ldo) {
  extern __shared__ float smem[];  // per wave: q [D], p [64]
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int wid = blockIdx.x * 4 + wave;
  if (wid >= n_rows * H) return;
  const int row = wid / H, h = wid % H;
  float* qs = smem + wave * (D + 64);
  float* ps = qs + D;
  for (int d = lane; d < D; d += 64) qs[d] = q[(int64_t)row * ldq + h * D + d];
  const int s = seq_of_row(cu_q, n_seqs, row);
  const int pos = kv_lens[s] - (cu_q[s + 1] - cu_q[s]) + (row - cu_q[s]);
  const int lo = max(0, pos - window + 1);
  const int g = h / (H / G);
  const int Gv = bias.value_heads, gv = h / (H / Gv);
  const HeadBias hb = head_bias(bias, h, H);
  const int32_t* table = block_tables + (int64_t)s * table_cols;
  float m = -INFINITY, l = 0.f;
  float acc[VPL];
#pragma unroll
  for (int i = 0; i < VPL; ++i) acc[i] = 0.f;
  __builtin_amdgcn_wave_barrier();
  for (int j0 = lo; j0 <= pos; j0 += 64) {
    const int j = j0 + lane;
    float sc = -INFINITY;
    if (j <= pos) {
      const int64_t blk = table[j / block_size];
      const TC* kr = k_cache + ((blk * G + g) * block_size + j % block_size) * D;
      float dot = 0.f;
      for (int d = 0; d < D; ++d) dot = fmaf(qs[d], ld_f<TC>(kr + d), dot);
      sc = capped(bias, dot * scale - dist_bias(hb, pos - j));
    }
    const float m_new = fmaxf(m, wave_max(sc));
    const float p = j <= pos ? expf(sc - m_new) : 0.f;
    const float corr = expf(m - m_new);  // (first chunk: exp(-inf) = 0)
    l = l * corr + wave_sum(p);
    m = m_new;
    ps[lane] = p;
    __builtin_amdgcn_wave_barrier();
    const int n_keys = min(64, pos - j0 + 1);
#pragma unroll
    for (int i = 0; i < VPL; ++i) acc[i] *= corr;
    for (int jj = 0; jj < n_keys; ++jj) {
      const int jk = j0 + jj;
      const int64_t blk = table[jk / block_size];
      const TC* vr = v_cache + ((blk * Gv + gv) * block_size + jk % block_size) * ldv;
      const float pj = ps[jj];
#pragma unroll
      for (int i = 0; i < VPL; ++i) {
        const int d = lane + 64 * i;
        if (d < Dv) acc[i] = fmaf(pj, ld_f<TC>(vr + d), acc[i]);
      }
    }
    __builtin_amdgcn_wave_barrier();
  }
  const float inv = 1.f / with_sink(bias, h, m, l);
#pragma unroll
  for (int i = 0; i < VPL; ++i) {
    const int d = lane + 64 * i;
    if (d < Dv) {
      float o = acc[i] * inv;
      if (gate) o *= sigmoid_f(gate[(int64_t)row * ldg + h * Dv + d]);
      out[(int64_t)row * ldo + h * Dv + d] = o;
    }
  }
}

// The product form: head sizes that are whole 16-byte pieces (D and Dv multiples of 8 for a bf16 cache, of 4 for fp32).
// A wave takes RPW consecutive step rows of one head; rows of the same sequence (consecutive positions, windows that
// differ by one key each) are handled TOGETHER: every K vector a lane loads is dotted with all of their queries, every
// V vector multiplied into all of their accumulators, so a prompt's portion reads its keys and values RPW times less
// often than row by row.  Scores: lane = key, the key's row in 16-byte loads.  Output: a V row is covered by LPR lanes
// (16-byte piece each), 64 / LPR keys per pass, the key groups' partial sums added at the end.  Online softmax per row
// with the usual guard for a chunk in which a row sees nothing yet.
template <typename TC, int VEC>
__device__ __forceinline__ void ld_vec(const TC* p, float (&v)[VEC]);
template <>
__device__ __forceinline__ void ld_vec<uint16_t, 8>(const uint16_t* p, float (&v)[8]) {
  const u32x4 w = *reinterpret_cast<const u32x4*>(p);
  v[0] = lo_bf(w[0]), v[1] = hi_bf(w[0]), v[2] = lo_bf(w[1]), v[3] = hi_bf(w[1]);
  v[4] = lo_bf(w[2]), v[5] = hi_bf(w[2]), v[6] = lo_bf(w[3]), v[7] = hi_bf(w[3]);
}
template <>
__device__ __forceinline__ void ld_vec<float, 4>(const float* p, float (&v)[4]) {
  const float4 w = *reinterpret_cast<const float4*>(p);
  v[0] = w.x, v[1] = w.y, v[2] = w.z, v[3] = w.w;
}

// SPLIT = 4 (single-row steps: decode): the four waves of a workgroup share ONE (row, head), take the window's 64-key
// chunks in turn and merge their (max, sum, accumulator) triples through LDS - four times the waves in flight where a
// step has only rows x heads units of work.
template <typename TC, int VEC, int RPW, int SPLIT>
__global__ __launch_bounds__(256) void swa_attention_vec_kernel(const float* __restrict__ q, int64_t ldq,
                                                                const TC* __restrict__ k_cache,
                                                                const TC* __restrict__ v_cache,
                                                                const int32_t* __restrict__ block_tables, int table_cols,
                                                                const int32_t* __restrict__ cu_q,
                                                                const int32_t* __restrict__ kv_lens, int n_seqs,
                                                                int n_rows, int H, int G, int D, int Dv, int block_size,
                                                                int window, float scale, AttnBias bias, int64_t ldv,
                                                                int lpr_log2, const float* __restrict__ gate, int64_t ldg,
                                                                float* __restrict__ out, int64_t ldo) {
  static_assert(SPLIT == 1 || RPW == 1, "the split form is the single-row form");
  extern __shared__ float smem[];  // per wave: q [RPW][D], p [RPW][64]; SPLIT > 1: then per wave {m, l, acc [Dv]}
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int wid = SPLIT > 1 ? (int)blockIdx.x : (int)blockIdx.x * 4 + wave;
  const int cw = SPLIT > 1 ? wave : 0;
  const int n_groups = (n_rows + RPW - 1) / RPW;
  if (wid >= n_groups * H) return;  // (SPLIT > 1: the whole workgroup)
  const int rg = wid / H, h = wid % H;
  float* qs = smem + wave * RPW * (D + 64);
  float* ps = qs + RPW * D;
  const int g = h / (H / G);
  const int Gv = bias.value_heads, gv = h / (H / Gv);
  const HeadBias hb = head_bias(bias, h, H);
  const int lpr = 1 << lpr_log2, kg = lane >> lpr_log2, cg = lane & (lpr - 1), kpp = 64 >> lpr_log2;
  const int group_end = min(rg * RPW + RPW, n_rows);
  for (int first = rg * RPW; first < group_end;) {
    const int s = seq_of_row(cu_q, n_seqs, first);
    const int end = min(cu_q[s + 1], group_end), nr = end - first;
    const int pos0 = kv_lens[s] - (cu_q[s + 1] - cu_q[s]) + (first - cu_q[s]);
    const int32_t* table = block_tables + (int64_t)s * table_cols;
    __builtin_amdgcn_wave_barrier();
    for (int r = 0; r < nr; ++r)
      for (int d = lane; d < D; d += 64) qs[r * D + d] = q[(int64_t)(first + r) * ldq + h * D + d];
    __builtin_amdgcn_wave_barrier();
    const int lo = max(0, pos0 - window + 1), hi = pos0 + nr - 1;
    float m[RPW], l[RPW], acc[RPW][VEC];
#pragma unroll
    for (int r = 0; r < RPW; ++r) {
      m[r] = -INFINITY, l[r] = 0.f;
#pragma unroll
      for (int e = 0; e < VEC; ++e) acc[r][e] = 0.f;
    }
    for (int j0 = lo + 64 * cw; j0 <= hi; j0 += 64 * SPLIT) {
      const int j = j0 + lane;
      float dots[RPW];
#pragma unroll
      for (int r = 0; r < RPW; ++r) dots[r] = 0.f;
      if (j <= hi) {
        const int64_t blk = table[j / block_size];
        const TC* kr = k_cache + ((blk * G + g) * block_size + j % block_size) * D;
        for (int d0 = 0; d0 < D; d0 += VEC) {
          float kv[VEC];
          ld_vec<TC, VEC>(kr + d0, kv);
#pragma unroll
          for (int r = 0; r < RPW; ++r)
#pragma unroll
            for (int e4 = 0; e4 < VEC; e4 += 4) {  // (D is a multiple of VEC: 16-byte LDS reads, the same address in every lane)
              const float4 qv = *reinterpret_cast<const float4*>(qs + r * D + d0 + e4);
              dots[r] = fmaf(qv.x, kv[e4], dots[r]);
              dots[r] = fmaf(qv.y, kv[e4 + 1], dots[r]);
              dots[r] = fmaf(qv.z, kv[e4 + 2], dots[r]);
              dots[r] = fmaf(qv.w, kv[e4 + 3], dots[r]);
            }
        }
      }
#pragma unroll
      for (int r = 0; r < RPW; ++r) {
        const int pos = pos0 + r;
        const bool vis = r < nr && j <= pos && j > pos - window;
        const float sc = vis ? capped(bias, dots[r] * scale - dist_bias(hb, pos - j)) : -INFINITY;
        const float m_new = fmaxf(m[r], wave_max(sc));
        const float p = vis ? expf(sc - m_new) : 0.f;
        const float corr = m[r] == -INFINITY ? 0.f : expf(m[r] - m_new);
        l[r] = l[r] * corr + wave_sum(p);
        m[r] = m_new;
        ps[r * 64 + lane] = p;
#pragma unroll
        for (int e = 0; e < VEC; ++e) acc[r][e] *= corr;
      }
      __builtin_amdgcn_wave_barrier();
      const int nk = min(64, hi - j0 + 1);
      if (cg * VEC < Dv) {
        for (int jj = kg; jj < nk; jj += kpp) {
          const int jk = j0 + jj;
          const int64_t blk = table[jk / block_size];
          float vv[VEC];
          ld_vec<TC, VEC>(v_cache + ((blk * Gv + gv) * block_size + jk % block_size) * ldv + cg * VEC, vv);
#pragma unroll
          for (int r = 0; r < RPW; ++r) {
            const float pj = ps[r * 64 + jj];
#pragma unroll
            for (int e = 0; e < VEC; ++e) acc[r][e] = fmaf(pj, vv[e], acc[r][e]);
          }
        }
      }
      __builtin_amdgcn_wave_barrier();
    }
    for (int off = lpr; off < 64; off <<= 1)
#pragma unroll
      for (int r = 0; r < RPW; ++r)
#pragma unroll
        for (int e = 0; e < VEC; ++e) acc[r][e] += __shfl_xor(acc[r][e], off);
    if constexpr (SPLIT > 1) {
      float* part = smem + 4 * RPW * (D + 64);  // [SPLIT][2 + Dv]
      if (kg == 0 && cg * VEC < Dv)
#pragma unroll
        for (int e = 0; e < VEC; ++e) part[wave * (2 + Dv) + 2 + cg * VEC + e] = acc[0][e];
      if (lane == 0) part[wave * (2 + Dv)] = m[0], part[wave * (2 + Dv) + 1] = l[0];
      __syncthreads();
      if (wave != 0) return;
      float mm = -INFINITY;
      for (int w2 = 0; w2 < SPLIT; ++w2) mm = fmaxf(mm, part[w2 * (2 + Dv)]);
      float lsum = 0.f;
#pragma unroll
      for (int e = 0; e < VEC; ++e) acc[0][e] = 0.f;
      for (int w2 = 0; w2 < SPLIT; ++w2) {  // (a wave without a chunk: max -inf, weight 0)
        const float mw = part[w2 * (2 + Dv)];
        const float f = mw == -INFINITY ? 0.f : expf(mw - mm);
        lsum = fmaf(part[w2 * (2 + Dv) + 1], f, lsum);
        if (cg * VEC < Dv)
#pragma unroll
          for (int e = 0; e < VEC; ++e) acc[0][e] = fmaf(part[w2 * (2 + Dv) + 2 + cg * VEC + e], f, acc[0][e]);
      }
      l[0] = lsum;
      m[0] = mm;
    }
    if (kg == 0 && cg * VEC < Dv) {
#pragma unroll
      for (int r = 0; r < RPW; ++r) {
        if (r >= nr) continue;
        const float inv = 1.f / with_sink(bias, h, m[r], l[r]);
        const int64_t row = first + r;
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          const int d = cg * VEC + e;
          float o = acc[r][e] * inv;
          if (gate) o *= sigmoid_f(gate[row * ldg + h * Dv + d]);
          out[row * ldo + h * Dv + d] = o;
        }
      }
    }
    first = end;
  }
}

// The matrix-core form for prompt portions over a bf16 cache (D a multiple of 32, Dv of 16): a wave takes 16 consecutive
// step rows of one head.  S^T = K Q^T on v_mfma_f32_16x16x32_bf16 with the KEYS on the row axis (the A operand is a key's
// cache row as stored: 16-byte loads), 32 keys per round; O^T += V^T P^T with the contraction slots ordered as the score
// registers are (slot 8 g + e of lane group g = key 4 g + e of the first 16-key tile for e < 4, of the second for
// e >= 4), so the softmax weights go from the accumulators into the B operand without leaving their lane; the V^T
// operand gathers its eight keys' elements.  Scores and weights stay fp32 quantities: q and p enter the MFMAs as
// bf16 hi + lo pairs (two MFMAs each, products exact, fp32 accumulation: 16 mantissa bits of q and p against the 8 of a
// plain bf16 operand), scale, distance bias, mask, running maximum and sum are fp32 VALU work on the accumulators.
template <int DKM, int DVM, bool PAIR>
__global__ __launch_bounds__(256) void swa_attention_mfma_kernel(const float* __restrict__ q, int64_t ldq,
                                                                 const uint16_t* __restrict__ k_cache,
                                                                 const uint16_t* __restrict__ v_cache,
                                                                 const int32_t* __restrict__ block_tables, int table_cols,
                                                                 const int32_t* __restrict__ cu_q,
                                                                 const int32_t* __restrict__ kv_lens, int n_seqs,
                                                                 int n_rows, int H, int G, int D, int Dv, int block_size,
                                                                 int window, float scale, AttnBias bias, int64_t ldv,
                                                                 const float* __restrict__ gate, int64_t ldg,
                                                                 float* __restrict__ out, int64_t ldo) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int wid = blockIdx.x * 4 + wave;
  const int n_groups = (n_rows + 15) / 16;
  if (wid >= n_groups * H) return;
  const int rg = wid / H, h = wid % H;
  const int g = h / (H / G);
  const int Gv = bias.value_heads, gv = h / (H / Gv);
  const HeadBias hb = head_bias(bias, h, H);
  const int qi = lane & 15, kg = lane >> 4;
  const int dk = D / 32, dvt = Dv / 16;
  const int bs_shift = block_shift(block_size);
  const bool q_vec = (ldq % 4 == 0) && ((reinterpret_cast<uintptr_t>(q) & 15u) == 0) && (D % 4 == 0);
  const int group_end = min(rg * 16 + 16, n_rows);
  for (int first = rg * 16; first < group_end;) {
    const int s = seq_of_row(cu_q, n_seqs, first);
    const int end = min(cu_q[s + 1], group_end), nr = end - first;
    const int pos0 = kv_lens[s] - (cu_q[s + 1] - cu_q[s]) + (first - cu_q[s]);
    const int32_t* table = block_tables + (int64_t)s * table_cols;
    bf16x8 qh[DKM], ql[DKM];
#pragma unroll
    for (int ks = 0; ks < DKM; ++ks) {
      float xv[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      if (ks < dk && qi < nr) {
        const float* qp = q + (int64_t)(first + qi) * ldq + h * D + ks * 32 + kg * 8;
        if (q_vec) {
          const float4 a = *reinterpret_cast<const float4*>(qp), b = *reinterpret_cast<const float4*>(qp + 4);
          xv[0] = a.x, xv[1] = a.y, xv[2] = a.z, xv[3] = a.w, xv[4] = b.x, xv[5] = b.y, xv[6] = b.z, xv[7] = b.w;
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e) xv[e] = qp[e];
        }
      }
      float lo[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) lo[e] = xv[e] - rbf(xv[e]);
      qh[ks] = as_frag(u32x4{pack_bf(xv[0], xv[1]), pack_bf(xv[2], xv[3]), pack_bf(xv[4], xv[5]), pack_bf(xv[6], xv[7])});
      ql[ks] = as_frag(u32x4{pack_bf(lo[0], lo[1]), pack_bf(lo[2], lo[3]), pack_bf(lo[4], lo[5]), pack_bf(lo[6], lo[7])});
    }
    const int lo_key = max(0, pos0 - window + 1), hi_key = pos0 + nr - 1;
    const int my_pos = pos0 + qi;
    float m = -INFINITY, l = 0.f;
    f32x4 oacc[DVM];
#pragma unroll
    for (int dt = 0; dt < DVM; ++dt) oacc[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
    for (int j0 = lo_key; j0 <= hi_key; j0 += 32) {
      f32x4 sacc[2] = {f32x4{0.f, 0.f, 0.f, 0.f}, f32x4{0.f, 0.f, 0.f, 0.f}};
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        // this lane's row of the K operand; rows beyond the last key repeat it (their scores are masked below), so
        // that every load is unconditional and a round's loads are all in flight together
        const int key = min(j0 + t * 16 + qi, hi_key);
        const uint16_t* kr =
            k_cache + (int64_t)cache_row(table, key, G, g, block_size, bs_shift) * D + kg * 8;
#pragma unroll
        for (int ks = 0; ks < DKM; ++ks) {
          if (ks < dk) {
            const bf16x8 kf = as_frag(*reinterpret_cast<const u32x4*>(kr + ks * 32));
            sacc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qh[ks], sacc[t], 0, 0, 0);
            sacc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, ql[ks], sacc[t], 0, 0, 0);
          }
        }
      }
      float sc[8];
      bool vis[8];
      int dist[8];
      float mx = -INFINITY;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int key = j0 + (e >> 2) * 16 + kg * 4 + (e & 3);
        vis[e] = qi < nr && key <= my_pos && key > my_pos - window;
        sc[e] = sacc[e >> 2][e & 3] * scale;
        dist[e] = my_pos - key;
      }
      // the bias kind is the same for the whole launch: a branch every wave takes the same way, so that the logarithms
      // are not evaluated (and thrown away) where the bias is linear or absent
      if (bias.kind == MI_BIAS_LOG) {
#pragma unroll
        for (int e = 0; e < 8; ++e) sc[e] -= hb.a * log1pf(hb.b * (float)max(dist[e], 0));
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) sc[e] -= hb.a * (float)dist[e];
      }
      if (bias.softcap > 0.f) {
#pragma unroll
        for (int e = 0; e < 8; ++e) sc[e] = bias.softcap * tanhf(sc[e] / bias.softcap);
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        sc[e] = vis[e] ? sc[e] : -INFINITY;
        mx = fmaxf(mx, sc[e]);
      }
      mx = xor_max<32>(xor_max<16>(mx));
      const float m_new = fmaxf(m, mx);
      const float corr = m == -INFINITY ? 0.f : expf(m - m_new);
      float pv[8], psum = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        pv[e] = vis[e] ? expf(sc[e] - m_new) : 0.f;
        psum += pv[e];
      }
      psum = xor_sum<32>(xor_sum<16>(psum));
      l = l * corr + psum;
      m = m_new;
      float plo[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) plo[e] = pv[e] - rbf(pv[e]);
      const bf16x8 ph = as_frag(u32x4{pack_bf(pv[0], pv[1]), pack_bf(pv[2], pv[3]), pack_bf(pv[4], pv[5]), pack_bf(pv[6], pv[7])});
      const bf16x8 pl = as_frag(u32x4{pack_bf(plo[0], plo[1]), pack_bf(plo[2], plo[3]), pack_bf(plo[4], plo[5]), pack_bf(plo[6], plo[7])});
      // V^T operand: the lane's eight keys (its contraction slots) at ONE channel per 16-channel tile - or, when Dv is a
      // multiple of 32 (PAIR), at TWO neighbouring channels per 32-channel pair of tiles with one 4-byte load: the low
      // halves feed the tile of the pair's even channels, the high halves the tile of its odd channels
      const uint16_t* vrow[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int key = min(j0 + (e >> 2) * 16 + kg * 4 + (e & 3), hi_key);  // (beyond the last key: weight 0)
        vrow[e] = v_cache + (int64_t)cache_row(table, key, Gv, gv, block_size, bs_shift) * (int)ldv +
                  (PAIR ? 2 * qi : qi);
      }
      if constexpr (PAIR) {
#pragma unroll
        for (int dp = 0; dp < DVM / 2; ++dp) {
          if (2 * dp < dvt) {
            uint32_t w[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) w[e] = *reinterpret_cast<const uint32_t*>(vrow[e] + dp * 32);
            const bf16x8 v_even = as_frag(u32x4{(w[0] & 0xffffu) | (w[1] << 16), (w[2] & 0xffffu) | (w[3] << 16),
                                                (w[4] & 0xffffu) | (w[5] << 16), (w[6] & 0xffffu) | (w[7] << 16)});
            const bf16x8 v_odd = as_frag(u32x4{(w[0] >> 16) | (w[1] & 0xffff0000u), (w[2] >> 16) | (w[3] & 0xffff0000u),
                                               (w[4] >> 16) | (w[5] & 0xffff0000u), (w[6] >> 16) | (w[7] & 0xffff0000u)});
            oacc[2 * dp] *= corr;
            oacc[2 * dp + 1] *= corr;
            oacc[2 * dp] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(v_even, ph, oacc[2 * dp], 0, 0, 0);
            oacc[2 * dp] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(v_even, pl, oacc[2 * dp], 0, 0, 0);
            oacc[2 * dp + 1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(v_odd, ph, oacc[2 * dp + 1], 0, 0, 0);
            oacc[2 * dp + 1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(v_odd, pl, oacc[2 * dp + 1], 0, 0, 0);
          }
        }
      } else {
#pragma unroll
        for (int dt = 0; dt < DVM; ++dt) {
          if (dt < dvt) {
            uint32_t ve[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) ve[e] = (uint32_t)vrow[e][dt * 16];
            const bf16x8 vf = as_frag(u32x4{ve[0] | (ve[1] << 16), ve[2] | (ve[3] << 16), ve[4] | (ve[5] << 16), ve[6] | (ve[7] << 16)});
            oacc[dt] *= corr;
            oacc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, ph, oacc[dt], 0, 0, 0);
            oacc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pl, oacc[dt], 0, 0, 0);
          }
        }
      }
    }
    if (qi < nr) {
      // the lane holds channels 16 dt + 4 kg + r of its query's output (PAIR: tile 2 dp + b holds the channels
      // 32 dp + 2 (4 kg + r) + b, i.e. the lane has the eight consecutive channels 32 dp + 8 kg .. + 7)
      const float inv = 1.f / with_sink(bias, h, m, l);
      const int64_t row = first + qi;
#pragma unroll
      for (int dt = 0; dt < DVM; ++dt) {
        if (dt < dvt) {
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int d = PAIR ? (dt >> 1) * 32 + 2 * (kg * 4 + r) + (dt & 1) : dt * 16 + kg * 4 + r;
            float o = oacc[dt][r] * inv;
            if (gate) o *= sigmoid_f(gate[row * ldg + h * Dv + d]);
            out[row * ldo + h * Dv + d] = o;
          }
        }
      }
    }
    first = end;
  }
}

// The matrix-core form for DECODE steps (one row per sequence) over a bf16 cache: a workgroup takes one (row, kv head) and
// up to 16 of the query heads that read it - the heads are the 16 columns of the score tile where the prompt form has 16
// consecutive rows of one head, so every K and V element the workgroup loads serves all of the group's heads (latent
// attention: ONE cache row for every head).  Its four waves take the rounds of 32 keys in turn and merge their (max, sum,
// accumulator) triples through LDS.  Arithmetic as in the prompt form: q and the softmax weights as bf16 hi + lo pairs.
template <int DKM, int DVM, bool PAIR>
__global__ __launch_bounds__(256) void paged_attention_heads_mfma_kernel(
    const float* __restrict__ q, int64_t ldq, const uint16_t* __restrict__ k_cache, const uint16_t* __restrict__ v_cache,
    const int32_t* __restrict__ block_tables, int table_cols, const int32_t* __restrict__ kv_lens, int H, int G, int D,
    int Dv, int block_size, int window, float scale, AttnBias bias, int64_t ldv, const float* __restrict__ gate,
    int64_t ldg, float* __restrict__ out, int64_t ldo, int n_split, float* __restrict__ ws) {
  __shared__ __attribute__((aligned(16))) float part_o[3][DVM][64][4];
  __shared__ float part_ml[3][2][64];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int row = blockIdx.x, g = blockIdx.y;
  const int Gv = bias.value_heads, gv = g / (G / Gv);
  const int hpg = H / G;
  const int split = blockIdx.z % n_split;                 // this workgroup's share of the rounds of keys
  const int h0 = g * hpg + (blockIdx.z / n_split) * 16;   // first head of this workgroup's columns
  const int nh = min(16, g * hpg + hpg - h0);             // valid columns
  const int qi = lane & 15, kg = lane >> 4;
  const int dk = D / 32, dvt = Dv / 16;
  const int bs_shift = block_shift(block_size);
  const int pos = kv_lens[row] - 1;
  const int32_t* table = block_tables + (int64_t)row * table_cols;
  const HeadBias hb = head_bias(bias, qi < nh ? h0 + qi : h0, H);
  const bool q_vec = (ldq % 4 == 0) && ((reinterpret_cast<uintptr_t>(q) & 15u) == 0) && (D % 4 == 0);
  bf16x8 qh[DKM], ql[DKM];
#pragma unroll
  for (int ks = 0; ks < DKM; ++ks) {
    float xv[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if (ks < dk && qi < nh) {
      const float* qp = q + (int64_t)row * ldq + (int64_t)(h0 + qi) * D + ks * 32 + kg * 8;
      if (q_vec) {
        const float4 a = *reinterpret_cast<const float4*>(qp), b = *reinterpret_cast<const float4*>(qp + 4);
        xv[0] = a.x, xv[1] = a.y, xv[2] = a.z, xv[3] = a.w, xv[4] = b.x, xv[5] = b.y, xv[6] = b.z, xv[7] = b.w;
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) xv[e] = qp[e];
      }
    }
    float lo[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) lo[e] = xv[e] - rbf(xv[e]);
    qh[ks] = as_frag(u32x4{pack_bf(xv[0], xv[1]), pack_bf(xv[2], xv[3]), pack_bf(xv[4], xv[5]), pack_bf(xv[6], xv[7])});
    ql[ks] = as_frag(u32x4{pack_bf(lo[0], lo[1]), pack_bf(lo[2], lo[3]), pack_bf(lo[4], lo[5]), pack_bf(lo[6], lo[7])});
  }
  const int lo_key = max(0, pos - window + 1), hi_key = pos;
  float m = -INFINITY, l = 0.f;
  f32x4 oacc[DVM];
#pragma unroll
  for (int dt = 0; dt < DVM; ++dt) oacc[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int j0 = lo_key + 32 * (split * 4 + wave); j0 <= hi_key; j0 += 32 * 4 * n_split) {
    f32x4 sacc[2] = {f32x4{0.f, 0.f, 0.f, 0.f}, f32x4{0.f, 0.f, 0.f, 0.f}};
    // the round's V words are requested together with its K rows (their addresses do not depend on the scores): one
    // memory latency per round instead of two behind one another.  The V^T operand: the lane's eight keys (its
    // contraction slots) at two neighbouring channels per 32-channel pair of tiles (PAIR), else one channel per tile
    const uint16_t* vrow[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int key = min(j0 + (e >> 2) * 16 + kg * 4 + (e & 3), hi_key);  // (beyond the last key: weight 0)
      vrow[e] = v_cache + (int64_t)cache_row(table, key, Gv, gv, block_size, bs_shift) * (int)ldv +
                (PAIR ? 2 * qi : qi);
    }
    uint32_t vw[PAIR ? DVM / 2 : 1][8];
    if constexpr (PAIR) {
#pragma unroll
      for (int dp = 0; dp < DVM / 2; ++dp)
        if (2 * dp < dvt) {
#pragma unroll
          for (int e = 0; e < 8; ++e) vw[dp][e] = *reinterpret_cast<const uint32_t*>(vrow[e] + dp * 32);
        }
    }
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      // this lane's row of the K operand; rows beyond the last key repeat it (their scores are masked below), so
      // that every load is unconditional and a round's loads are all in flight together
      const int key = min(j0 + t * 16 + qi, hi_key);
      const uint16_t* kr =
          k_cache + (int64_t)cache_row(table, key, G, g, block_size, bs_shift) * D + kg * 8;
#pragma unroll
      for (int ks = 0; ks < DKM; ++ks) {
        if (ks < dk) {
          const bf16x8 kf = as_frag(*reinterpret_cast<const u32x4*>(kr + ks * 32));
          sacc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qh[ks], sacc[t], 0, 0, 0);
          sacc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, ql[ks], sacc[t], 0, 0, 0);
        }
      }
    }
    float sc[8];
    bool vis[8];
    int dist[8];
    float mx = -INFINITY;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int key = j0 + (e >> 2) * 16 + kg * 4 + (e & 3);
      vis[e] = qi < nh && key <= hi_key;
      sc[e] = sacc[e >> 2][e & 3] * scale;
      dist[e] = pos - key;
    }
    // (the bias kind is the same for the whole launch: see the prompt form)
    if (bias.kind == MI_BIAS_LOG) {
#pragma unroll
      for (int e = 0; e < 8; ++e) sc[e] -= hb.a * log1pf(hb.b * (float)max(dist[e], 0));
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) sc[e] -= hb.a * (float)dist[e];
    }
    if (bias.softcap > 0.f) {
#pragma unroll
      for (int e = 0; e < 8; ++e) sc[e] = bias.softcap * tanhf(sc[e] / bias.softcap);
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      sc[e] = vis[e] ? sc[e] : -INFINITY;
      mx = fmaxf(mx, sc[e]);
    }
    mx = xor_max<32>(xor_max<16>(mx));
    const float m_new = fmaxf(m, mx);
    const float corr = m == -INFINITY ? 0.f : expf(m - m_new);
    float pv[8], psum = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      pv[e] = vis[e] ? expf(sc[e] - m_new) : 0.f;
      psum += pv[e];
    }
    psum = xor_sum<32>(xor_sum<16>(psum));
    l = l * corr + psum;
    m = m_new;
    float plo[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) plo[e] = pv[e] - rbf(pv[e]);
    const bf16x8 ph = as_frag(u32x4{pack_bf(pv[0], pv[1]), pack_bf(pv[2], pv[3]), pack_bf(pv[4], pv[5]), pack_bf(pv[6], pv[7])});
    const bf16x8 pl = as_frag(u32x4{pack_bf(plo[0], plo[1]), pack_bf(plo[2], plo[3]), pack_bf(plo[4], plo[5]), pack_bf(plo[6], plo[7])});
    if constexpr (PAIR) {
#pragma unroll
      for (int dp = 0; dp < DVM / 2; ++dp) {
        if (2 * dp < dvt) {
          const uint32_t(&w)[8] = vw[dp];
          const bf16x8 v_even = as_frag(u32x4{(w[0] & 0xffffu) | (w[1] << 16), (w[2] & 0xffffu) | (w[3] << 16),
                                              (w[4] & 0xffffu) | (w[5] << 16), (w[6] & 0xffffu) | (w[7] << 16)});
          const bf16x8 v_odd = as_frag(u32x4{(w[0] >> 16) | (w[1] & 0xffff0000u), (w[2] >> 16) | (w[3] & 0xffff0000u),
                                             (w[4] >> 16) | (w[5] & 0xffff0000u), (w[6] >> 16) | (w[7] & 0xffff0000u)});
          oacc[2 * dp] *= corr;
          oacc[2 * dp + 1] *= corr;
          oacc[2 * dp] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(v_even, ph, oacc[2 * dp], 0, 0, 0);
          oacc[2 * dp] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(v_even, pl, oacc[2 * dp], 0, 0, 0);
          oacc[2 * dp + 1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(v_odd, ph, oacc[2 * dp + 1], 0, 0, 0);
          oacc[2 * dp + 1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(v_odd, pl, oacc[2 * dp + 1], 0, 0, 0);
        }
      }
    } else {
#pragma unroll
      for (int dt = 0; dt < DVM; ++dt) {
        if (dt < dvt) {
          uint32_t ve[8];
#pragma unroll
          for (int e = 0; e < 8; ++e) ve[e] = (uint32_t)vrow[e][dt * 16];
          const bf16x8 vf = as_frag(u32x4{ve[0] | (ve[1] << 16), ve[2] | (ve[3] << 16), ve[4] | (ve[5] << 16), ve[6] | (ve[7] << 16)});
          oacc[dt] *= corr;
          oacc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, ph, oacc[dt], 0, 0, 0);
          oacc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pl, oacc[dt], 0, 0, 0);
        }
      }
    }
  }
  // merge the four waves' partial results (same lane layout in every wave); a wave without a round has m = -inf, l = 0
  if (wave > 0) {
#pragma unroll
    for (int dt = 0; dt < DVM; ++dt)
      if (dt < dvt) *reinterpret_cast<f32x4*>(part_o[wave - 1][dt][lane]) = oacc[dt];
    part_ml[wave - 1][0][lane] = m;
    part_ml[wave - 1][1][lane] = l;
  }
  __syncthreads();
  if (wave > 0 || qi >= nh) return;
  float mm = m;
#pragma unroll
  for (int w = 0; w < 3; ++w) mm = fmaxf(mm, part_ml[w][0][lane]);
  const float f0 = m == -INFINITY ? 0.f : expf(m - mm);
  l *= f0;
#pragma unroll
  for (int dt = 0; dt < DVM; ++dt) oacc[dt] *= f0;
#pragma unroll
  for (int w = 0; w < 3; ++w) {
    const float mw = part_ml[w][0][lane];
    const float f = mw == -INFINITY ? 0.f : expf(mw - mm);
    l = fmaf(part_ml[w][1][lane], f, l);
#pragma unroll
    for (int dt = 0; dt < DVM; ++dt)
      if (dt < dvt) {
        const f32x4 o = *reinterpret_cast<const f32x4*>(part_o[w][dt][lane]);
        oacc[dt] += o * f;
      }
  }
  if (n_split > 1) {
    // several workgroups share this (row, head): leave (max, sum, unnormalised accumulator) for the merge kernel
    float* p = ws + (((int64_t)row * H + h0 + qi) * n_split + split) * (2 + Dv);
    if (kg == 0) p[0] = mm, p[1] = l;
#pragma unroll
    for (int dt = 0; dt < DVM; ++dt) {
      if (dt < dvt) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int d = PAIR ? (dt >> 1) * 32 + 2 * (kg * 4 + r) + (dt & 1) : dt * 16 + kg * 4 + r;
          p[2 + d] = oacc[dt][r];
        }
      }
    }
    return;
  }
  const float inv = 1.f / with_sink(bias, h0 + qi, mm, l);
  const int64_t obase = (int64_t)row * ldo + (int64_t)(h0 + qi) * Dv;
  const int64_t gbase = (int64_t)row * ldg + (int64_t)(h0 + qi) * Dv;
#pragma unroll
  for (int dt = 0; dt < DVM; ++dt) {
    if (dt < dvt) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int d = PAIR ? (dt >> 1) * 32 + 2 * (kg * 4 + r) + (dt & 1) : dt * 16 + kg * 4 + r;
        float o = oacc[dt][r] * inv;
        if (gate) o *= sigmoid_f(gate[gbase + d]);
        out[obase + d] = o;
      }
    }
  }
}

// the partial results of the NS workgroups that shared a (row, head) -> the output row; a wave per (row, head), the
// partials' loads unrolled (all in flight together)
template <int NS>
__global__ __launch_bounds__(256) void paged_attention_merge_kernel(const float* __restrict__ ws, int n_units, int H, int Dv,
                                                                    const float* __restrict__ gate, int64_t ldg,
                                                                    const float* __restrict__ sink,
                                                                    float* __restrict__ out, int64_t ldo) {
  const int unit = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (unit >= n_units) return;
  const int row = unit / H, h = unit % H;
  const int64_t stride = 2 + Dv;
  const float* p = ws + (int64_t)unit * NS * stride;
  float m[NS], f[NS];
  float mm = -INFINITY, l = 0.f;
#pragma unroll
  for (int i = 0; i < NS; ++i) m[i] = p[i * stride];
#pragma unroll
  for (int i = 0; i < NS; ++i) mm = fmaxf(mm, m[i]);
#pragma unroll
  for (int i = 0; i < NS; ++i) {
    f[i] = m[i] == -INFINITY ? 0.f : expf(m[i] - mm);
    l = fmaf(p[i * stride + 1], f[i], l);
  }
  if (sink) l += expf(sink[h] - mm);
  const float inv = 1.f / l;
  for (int d = lane; d < Dv; d += 64) {
    float v[NS];
#pragma unroll
    for (int i = 0; i < NS; ++i) v[i] = p[i * stride + 2 + d];
    float o = 0.f;
#pragma unroll
    for (int i = 0; i < NS; ++i) o = fmaf(v[i], f[i], o);
    o *= inv;
    if (gate) o *= sigmoid_f(gate[(int64_t)row * ldg + (int64_t)h * Dv + d]);
    out[(int64_t)row * ldo + (int64_t)h * Dv + d] = o;
  }
}

// ---------------------------------------------------------------------------------------------------------------
// short causal convolution with a carried tail
// ---------------------------------------------------------------------------------------------------------------
// y[r][c] = act(sum_j w[c][j] * in[r - (taps - 1) + j]) (+ in[r] when add_input); inputs before the step's first row
// come from the sequence's state slot (the last taps - 1 inputs, oldest first) - zeros when the sequence starts in this
// step.  silu: act = silu, else the identity.
__global__ __launch_bounds__(256) void causal_conv_kernel(const float* __restrict__ x, int64_t ldx,
                                                               const float* __restrict__ w, int taps,
                                                               const float* __restrict__ state,
                                                               const int32_t* __restrict__ cu_q,
                                                               const int32_t* __restrict__ kv_lens,
                                                               const int32_t* __restrict__ slot_ids, int n_seqs, int C,
                                                               int silu, int add_input, float* __restrict__ y,
                                                               int64_t ldy) {
  const int row = blockIdx.x;
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= C) return;
  const int s = seq_of_row(cu_q, n_seqs, row);
  const int r = row - cu_q[s];
  const int start = kv_lens[s] - (cu_q[s + 1] - cu_q[s]);
  const float* st = state + (int64_t)slot_ids[s] * (taps - 1) * C;
  float acc = 0.f;
  for (int j = 0; j < taps; ++j) {
    const int rr = r - (taps - 1) + j;  // row of this sequence's step, or before it
    float v;
    if (rr >= 0) v = x[(int64_t)(cu_q[s] + rr) * ldx + c];
    else v = start > 0 ? st[(int64_t)(taps - 1 + rr) * C + c] : 0.f;  // (a state written at position p holds inputs p-taps+1..p-1, zeros before 0)
    acc = fmaf(w[(int64_t)c * taps + j], v, acc);
  }
  if (silu) acc = acc / (1.f + expf(-acc));
  if (add_input) acc += x[(int64_t)row * ldx + c];
  y[(int64_t)row * ldy + c] = acc;
}

// the new tail: the last taps - 1 inputs of (old tail ++ this step's rows).  One thread per (sequence, channel) reads
// everything it needs before it writes, and no other thread touches its entries.
__global__ __launch_bounds__(256) void causal_conv_state_kernel(const float* __restrict__ x, int64_t ldx, int taps,
                                                                float* __restrict__ state,
                                                                const int32_t* __restrict__ cu_q,
                                                                const int32_t* __restrict__ kv_lens,
                                                                const int32_t* __restrict__ slot_ids, int C) {
  const int s = blockIdx.y;
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= C) return;
  const int n = cu_q[s + 1] - cu_q[s];
  if (n == 0) return;
  const int start = kv_lens[s] - n;
  float* st = state + (int64_t)slot_ids[s] * (taps - 1) * C;
  float tail[16];
  const int L = taps - 1;
  for (int i = 0; i < L; ++i) {
    const int rr = n - L + i;  // row of this step, or (negative) an entry of the old tail
    if (rr >= 0) tail[i] = x[(int64_t)(cu_q[s] + rr) * ldx + c];
    else tail[i] = start > 0 ? st[(int64_t)(L + rr) * C + c] : 0.f;
  }
  for (int i = 0; i < L; ++i) st[(int64_t)i * C + c] = tail[i];
}

// Both in one launch for steps in which no sequence brings more than a few rows (decode steps, short portions): a thread
// per (sequence, channel) keeps the tail in registers, walks its rows and writes the tail back - nothing else reads or
// writes its entries, so there is no order to keep between launches.  The taps are summed in causal_conv_kernel's order.
__global__ __launch_bounds__(256) void causal_conv_step_kernel(const float* __restrict__ x, int64_t ldx,
                                                               const float* __restrict__ w, int taps,
                                                               float* __restrict__ state,
                                                               const int32_t* __restrict__ cu_q,
                                                               const int32_t* __restrict__ kv_lens,
                                                               const int32_t* __restrict__ slot_ids, int C, int silu,
                                                               int add_input, float* __restrict__ y, int64_t ldy) {
  const int s = blockIdx.y;
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= C) return;
  const int r0 = cu_q[s], n = cu_q[s + 1] - r0;
  if (n == 0) return;
  const int start = kv_lens[s] - n;
  const int L = taps - 1;
  float* st = state + (int64_t)slot_ids[s] * L * C;
  float tail[16], wt[17];
#pragma unroll
  for (int i = 0; i < 16; ++i) tail[i] = (i < L && start > 0) ? st[(int64_t)i * C + c] : 0.f;
#pragma unroll
  for (int j = 0; j < 17; ++j) wt[j] = j < taps ? w[(int64_t)c * taps + j] : 0.f;
  for (int r = 0; r < n; ++r) {
    const float xr = x[(int64_t)(r0 + r) * ldx + c];
    float acc = 0.f;
#pragma unroll
    for (int j = 0; j < 16; ++j)
      if (j < L) acc = fmaf(wt[j], tail[j], acc);
    float wl = 0.f;
#pragma unroll
    for (int j = 0; j < 17; ++j)
      if (j == L) wl = wt[j];
    acc = fmaf(wl, xr, acc);
    if (silu) acc = acc / (1.f + expf(-acc));
    if (add_input) acc += xr;
    y[(int64_t)(r0 + r) * ldy + c] = acc;
#pragma unroll
    for (int i = 0; i < 15; ++i) tail[i] = i + 1 < L ? tail[i + 1] : tail[i];
#pragma unroll
    for (int i = 0; i < 16; ++i)
      if (i == L - 1) tail[i] = xr;
  }
#pragma unroll
  for (int i = 0; i < 16; ++i)
    if (i < L) st[(int64_t)i * C + c] = tail[i];
}

// ---------------------------------------------------------------------------------------------------------------
// gated delta rule, decay per head and key channel
// ---------------------------------------------------------------------------------------------------------------
// Three launches.  delta_prepare_kernel (parallel over rows): the row's unit q and k per q/k head, its decay vector and
// beta per head - everything with a transcendental in it - into a workspace [rows][2 G D + H D + H].
// channel_delta_kernel (the recurrence): the columns of S (one per value channel) never exchange anything: S^T k, the
// rank-one update and S^T q are per-column sums over the key channels.  One workgroup = 32 value columns of one
// (sequence, head); a column is held by FOUR lanes (a quad), each keeping DR of the (padded) 4 * DR key channels of it
// in registers for the whole walk over the sequence's rows of this step - lane r of the quad owns the channels
// (4 jj + r) * 4 + e, so that a quad's LDS reads of the row's k / q / decay vectors are four consecutive 16-byte pieces
// and the two sums over the key channels end in two DPP steps inside the quad.  The prepared vectors of 16 rows at a
// time are copied into LDS, loaded one batch ahead (in flight while the current batch is walked); between two batches
// the walk needs no barrier.  The state is kept in memory in THREAD order ([slot][head][column block][DR][128]: register
// ii of thread t at ii * 128 + t), read and written fully coalesced and touched by nothing else.
// delta_finish_kernel: per-head RMS norm of the raw read-out, weight, sigmoid gate.
constexpr int kDeltaCols = 32, kDeltaRows = 16, kDeltaThreads = 4 * kDeltaCols;

// workspace row: [q G*D | k G*D | decay H*D | beta H]
__global__ __launch_bounds__(256) void delta_prepare_kernel(const float* __restrict__ qkv, int64_t ld, int q_off, int k_off,
                                                            const float* __restrict__ beta_pre, int64_t ld_beta,
                                                            const float* __restrict__ decay_pre, int64_t ld_decay,
                                                            const float* __restrict__ dt_bias,
                                                            const float* __restrict__ a_log, int H, int G, int D,
                                                            float* __restrict__ ws) {
  const int64_t row = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  float* out = ws + row * (int64_t)(2 * G * D + H * D + H);
  const float q_scale = 1.f / sqrtf((float)D);
  for (int u = wave; u < 2 * G; u += 4) {  // (q | k, head): a wave each
    const bool is_k = u >= G;
    const float* src = qkv + row * ld + (is_k ? k_off + (u - G) * D : q_off + u * D);
    float sq = 0.f;
    for (int i = lane; i < D; i += 64) sq = fmaf(src[i], src[i], sq);
    const float nrm = (is_k ? 1.f : q_scale) / sqrtf(wave_sum(sq) + 1e-6f);
    for (int i = lane; i < D; i += 64) out[u * D + i] = src[i] * nrm;
  }
  for (int e = threadIdx.x; e < H * D; e += 256) {
    const float rate = expf(a_log[e / D]);
    out[2 * G * D + e] = expf(-rate * softplus_f(decay_pre[row * ld_decay + e] + dt_bias[e]));
  }
  for (int h = threadIdx.x; h < H; h += 256) out[2 * G * D + H * D + h] = sigmoid_f(beta_pre[row * ld_beta + h]);
}

template <int DR>
__global__ __launch_bounds__(kDeltaThreads) void channel_delta_kernel(const float* __restrict__ qkv, int64_t ld, int v_off,
                                                                      const float* __restrict__ ws,
                                                                      float* __restrict__ state,
                                                                      const int32_t* __restrict__ cu_q,
                                                                      const int32_t* __restrict__ kv_lens,
                                                                      const int32_t* __restrict__ slot_ids, int H, int G,
                                                                      int D, int Dv, float* __restrict__ out,
                                                                      int64_t ldo) {
  constexpr int DP = 4 * DR;  // padded key channels
  __shared__ __attribute__((aligned(16))) float qs[kDeltaRows][DP];
  __shared__ __attribute__((aligned(16))) float ks[kDeltaRows][DP];
  __shared__ __attribute__((aligned(16))) float gs[kDeltaRows][DP];
  __shared__ float vs[kDeltaRows][kDeltaCols];
  __shared__ float bs[kDeltaRows];
  const int s = blockIdx.x, h = blockIdx.y, cb = blockIdx.z;
  const int tid = threadIdx.x, r = tid & 3, col = tid >> 2;
  const int c = cb * kDeltaCols + col;
  const int r0 = cu_q[s], n = cu_q[s + 1] - r0;
  if (n == 0) return;
  const int start = kv_lens[s] - n;
  const int kvh = h / (H / G);
  const int64_t ws_ld = 2 * G * D + H * D + H;
  float* slot = state + (((int64_t)slot_ids[s] * H + h) * gridDim.z + cb) * DR * kDeltaThreads;
  float st[DR];
#pragma unroll
  for (int ii = 0; ii < DR; ++ii) st[ii] = start > 0 ? slot[ii * kDeltaThreads + tid] : 0.f;
  // staging: 8 lanes per row copy the row's prepared vectors (zeros beyond D and beyond the step's rows)
  const int pt = tid >> 3, ps = tid & 7;
  constexpr int PE = DP / 8;
  float rq[PE], rk[PE], rg[PE], rv[kDeltaCols / 8], rb;
  auto fetch = [&](int c0) {
    const bool live = c0 + pt < n;
    const int64_t row = r0 + (live ? c0 + pt : 0);
    const float* w = ws + row * ws_ld;
#pragma unroll
    for (int m = 0; m < PE; ++m) {
      const int i = ps + 8 * m;
      const bool ok = live && i < D;
      rq[m] = ok ? w[kvh * D + i] : 0.f;
      rk[m] = ok ? w[(G + kvh) * D + i] : 0.f;
      rg[m] = ok ? w[2 * G * D + h * D + i] : 0.f;
    }
#pragma unroll
    for (int m = 0; m < kDeltaCols / 8; ++m) {
      const int cc = cb * kDeltaCols + ps + 8 * m;
      rv[m] = (live && cc < Dv) ? qkv[row * ld + v_off + h * Dv + cc] : 0.f;
    }
    rb = live ? w[2 * G * D + H * D + h] : 0.f;
  };
  fetch(0);
  for (int c0 = 0; c0 < n; c0 += kDeltaRows) {
    __syncthreads();  // the previous rows' vectors have been consumed
#pragma unroll
    for (int m = 0; m < PE; ++m) qs[pt][ps + 8 * m] = rq[m], ks[pt][ps + 8 * m] = rk[m], gs[pt][ps + 8 * m] = rg[m];
#pragma unroll
    for (int m = 0; m < kDeltaCols / 8; ++m) vs[pt][ps + 8 * m] = rv[m];
    if (ps == 0) bs[pt] = rb;
    __syncthreads();
    if (c0 + kDeltaRows < n) fetch(c0 + kDeltaRows);
    const int nt = min(kDeltaRows, n - c0);
    for (int t = 0; t < nt; ++t) {
      const float4* g4 = reinterpret_cast<const float4*>(gs[t]);
      const float4* k4 = reinterpret_cast<const float4*>(ks[t]);
      const float4* q4 = reinterpret_cast<const float4*>(qs[t]);
      float d0 = 0.f, d1 = 0.f, d2 = 0.f, d3 = 0.f;  // (four chains instead of one: the wave has its SIMD to itself)
#pragma unroll
      for (int jj = 0; jj < DR / 4; ++jj) {
        const float4 gv = g4[jj * 4 + r], kv = k4[jj * 4 + r];
        st[jj * 4 + 0] *= gv.x, st[jj * 4 + 1] *= gv.y, st[jj * 4 + 2] *= gv.z, st[jj * 4 + 3] *= gv.w;
        d0 = fmaf(st[jj * 4 + 0], kv.x, d0);
        d1 = fmaf(st[jj * 4 + 1], kv.y, d1);
        d2 = fmaf(st[jj * 4 + 2], kv.z, d2);
        d3 = fmaf(st[jj * 4 + 3], kv.w, d3);
      }
      const float dot = xor_sum<2>(xor_sum<1>((d0 + d1) + (d2 + d3)));
      const float u = bs[t] * (vs[t][col] - dot);
      float o0 = 0.f, o1 = 0.f, o2 = 0.f, o3 = 0.f;
#pragma unroll
      for (int jj = 0; jj < DR / 4; ++jj) {
        const float4 kv = k4[jj * 4 + r], qv = q4[jj * 4 + r];
        st[jj * 4 + 0] = fmaf(kv.x, u, st[jj * 4 + 0]);
        st[jj * 4 + 1] = fmaf(kv.y, u, st[jj * 4 + 1]);
        st[jj * 4 + 2] = fmaf(kv.z, u, st[jj * 4 + 2]);
        st[jj * 4 + 3] = fmaf(kv.w, u, st[jj * 4 + 3]);
        o0 = fmaf(st[jj * 4 + 0], qv.x, o0);
        o1 = fmaf(st[jj * 4 + 1], qv.y, o1);
        o2 = fmaf(st[jj * 4 + 2], qv.z, o2);
        o3 = fmaf(st[jj * 4 + 3], qv.w, o3);
      }
      const float o = xor_sum<2>(xor_sum<1>((o0 + o1) + (o2 + o3)));
      if (r == 0 && c < Dv) out[(int64_t)(r0 + c0 + t) * ldo + h * Dv + c] = o;
    }
  }
#pragma unroll
  for (int ii = 0; ii < DR; ++ii) slot[ii * kDeltaThreads + tid] = st[ii];
}

// out[row][h] <- out_scale * out / rms(out over Dv) * norm_w (* act(gate) with a gate; norm_w may be nullptr: no weight;
// gate_act: MI_ACT_SIGMOID or MI_ACT_SILU): one wave per (row, head), in place
__global__ __launch_bounds__(256) void delta_finish_kernel(float* __restrict__ out, int64_t ldo,
                                                           const float* __restrict__ gate_pre, int64_t ld_gate,
                                                           const float* __restrict__ norm_w, int n_rows, int H, int Dv,
                                                           float eps, int gate_act, float out_scale) {
  const int lane = threadIdx.x & 63;
  const int wid = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (wid >= n_rows * H) return;
  const int row = wid / H, h = wid % H;
  float* o = out + (int64_t)row * ldo + h * Dv;
  float sq = 0.f;
  for (int d = lane; d < Dv; d += 64) sq = fmaf(o[d], o[d], sq);
  const float rstd = out_scale / sqrtf(wave_sum(sq) / (float)Dv + eps);
  for (int d = lane; d < Dv; d += 64) {
    float v = o[d] * rstd;
    if (norm_w) v *= norm_w[d];
    if (gate_pre) {
      const float z = gate_pre[(int64_t)row * ld_gate + h * Dv + d];
      v *= gate_act == MI_ACT_SILU ? z * sigmoid_f(z) : sigmoid_f(z);
    }
    o[d] = v;
  }
}

// ---------------------------------------------------------------------------------------------------------------
// sparse feed-forward: routing and combination
// ---------------------------------------------------------------------------------------------------------------
// One wave per token; a lane holds the outputs lane, lane + 64, ... (n <= 512: eight per lane).  Choice scores go through
// LDS for the group maxima; groups and then outputs are picked by repeated arg-max over the wave (larger value first,
// equal values: the lower index), NaN scores counting as 0.
__device__ __forceinline__ void wave_argmax(float& v, int& idx) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) {
    const float ov = __shfl_xor(v, off);
    const int oi = __shfl_xor(idx, off);
    if (ov > v || (ov == v && oi < idx)) v = ov, idx = oi;
  }
}

// score_kind: MI_ROUTE_SOFTMAX (scores = softmax over the outputs) or MI_ROUTE_SIGMOID (each output's own sigmoid);
// group_kind: a group's value is its best choice score (MI_ROUTE_GROUP_MAX) or the sum of its two best
// (MI_ROUTE_GROUP_TOP2; a group of one output: that output's score).
__global__ __launch_bounds__(256) void route_grouped_kernel(const float* __restrict__ logits, int64_t ld,
                                                            const float* __restrict__ correction, int T, int n, int top_k,
                                                            int n_groups, int keep, int score_kind, int group_kind,
                                                            int32_t* __restrict__ ids, float* __restrict__ wts) {
  __shared__ float choice_s[4][512];
  __shared__ int kept_s[4][512];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int t = blockIdx.x * 4 + wave;
  if (t >= T) return;
  const float* z = logits + (int64_t)t * ld;
  constexpr int EPL = 8;
  const int big = 1 << 30;
  float sc[EPL], ch[EPL];
  float mx = -INFINITY;
#pragma unroll
  for (int i = 0; i < EPL; ++i) {
    const int e = lane + 64 * i;
    sc[i] = e < n ? z[e] : -INFINITY;
    mx = fmaxf(mx, sc[i]);
  }
  mx = wave_max(mx);
  float sum = 0.f;
  if (score_kind == MI_ROUTE_SOFTMAX) {
#pragma unroll
    for (int i = 0; i < EPL; ++i) {
      sc[i] = lane + 64 * i < n ? expf(sc[i] - mx) : 0.f;
      sum += sc[i];
    }
    sum = wave_sum(sum);
  } else {
    sum = 1.f;
#pragma unroll
    for (int i = 0; i < EPL; ++i) sc[i] = lane + 64 * i < n ? sigmoid_f(sc[i]) : 0.f;
  }
#pragma unroll
  for (int i = 0; i < EPL; ++i) {
    const int e = lane + 64 * i;
    sc[i] = sc[i] / sum;
    if (!(sc[i] == sc[i])) sc[i] = 0.f;
    ch[i] = e < n ? sc[i] + correction[e] : -INFINITY;
    if (e < n) choice_s[wave][e] = ch[i];
  }
  __builtin_amdgcn_wave_barrier();
  const int per = n / n_groups;
  float gsc[EPL];
  unsigned g_taken = 0;
#pragma unroll
  for (int i = 0; i < EPL; ++i) {
    const int gi = lane + 64 * i;
    float gv = -INFINITY;
    if (gi < n_groups) {
      float second = -INFINITY;
      for (int e = gi * per; e < (gi + 1) * per; ++e) {
        const float c = choice_s[wave][e];
        if (c > gv) second = gv, gv = c;
        else if (c > second) second = c;
      }
      if (group_kind == MI_ROUTE_GROUP_TOP2 && per > 1) gv += second;
      kept_s[wave][gi] = 0;
    }
    gsc[i] = gv;
  }
  for (int it = 0; it < keep; ++it) {
    float bv = -INFINITY;
    int bi = big;
#pragma unroll
    for (int i = 0; i < EPL; ++i) {
      const int gi = lane + 64 * i;
      if (gi < n_groups && !(g_taken >> i & 1) && (bi == big || gsc[i] > bv)) bv = gsc[i], bi = gi;
    }
    wave_argmax(bv, bi);
    if ((bi & 63) == lane) {
      g_taken |= 1u << (bi >> 6);
      kept_s[wave][bi] = 1;
    }
  }
  __builtin_amdgcn_wave_barrier();
  unsigned taken = 0;
#pragma unroll
  for (int i = 0; i < EPL; ++i) {
    const int e = lane + 64 * i;
    if (e >= n || !kept_s[wave][e / per]) taken |= 1u << i;  // not eligible
  }
  for (int it = 0; it < top_k; ++it) {
    float bv = -INFINITY;
    int bi = big;
#pragma unroll
    for (int i = 0; i < EPL; ++i)
      if (!(taken >> i & 1) && (bi == big || ch[i] > bv)) bv = ch[i], bi = lane + 64 * i;
    wave_argmax(bv, bi);
    if ((bi & 63) == lane) {
      const int i = bi >> 6;
      taken |= 1u << i;
      ids[(int64_t)t * top_k + it] = bi;
      float w = 0.f;
#pragma unroll
      for (int i2 = 0; i2 < EPL; ++i2)
        if (i2 == i) w = sc[i2];
      wts[(int64_t)t * top_k + it] = w;
    }
  }
}

__global__ __launch_bounds__(256) void moe_combine_f32_kernel(const float* __restrict__ y, const float* __restrict__ h,
                                                              int64_t ldh, const int32_t* __restrict__ ids,
                                                              const float* __restrict__ wts, int top_k, int n_experts,
                                                              int width, float* __restrict__ out, int64_t ldo) {
  const int t = blockIdx.x;
  for (int c = threadIdx.x; c < width; c += 256) {
    float acc = 0.f;
    for (int k = 0; k < top_k; ++k) {
      const int e = ids[(int64_t)t * top_k + k];
      const float v = e >= n_experts ? h[(int64_t)t * ldh + c] : y[((int64_t)t * top_k + k) * width + c];
      acc = fmaf(wts[(int64_t)t * top_k + k], v, acc);
    }
    out[(int64_t)t * ldo + c] = acc;
  }
}

// ---------------------------------------------------------------------------------------------------------------
// pre-norm residual streams: RMS norm, residual update, depth-weighted mixing of the layers' results
// ---------------------------------------------------------------------------------------------------------------
// One workgroup per row.  res += mult * y + vec (y, vec may be nullptr; vec [width] is the same for every row);
// w != nullptr: out = res / sqrt(mean(res^2) + eps) * (w + shift) (shift 1: weights stored around zero).  res == out is
// allowed (a plain norm in place).
__global__ __launch_bounds__(256) void add_rmsnorm_f32_kernel(float* __restrict__ res, int64_t ldr,
                                                              const float* __restrict__ y, int64_t ldy, float mult,
                                                              const float* __restrict__ vec,
                                                              const float* __restrict__ w, float shift, float eps,
                                                              float* __restrict__ out, int64_t ldo, int width) {
  __shared__ float red[4];
  float* r = res + (int64_t)blockIdx.x * ldr;
  const float* yr = y ? y + (int64_t)blockIdx.x * ldy : nullptr;
  float sq = 0.f;
  for (int c = threadIdx.x; c < width; c += 256) {
    float v = r[c];
    if (yr) v = fmaf(mult, yr[c], v);
    if (vec) v += vec[c];
    if (yr || vec) r[c] = v;
    sq = fmaf(v, v, sq);
  }
  if (!w) return;
  const float rstd = 1.f / sqrtf(block_sum256(sq, red) / (float)width + eps);
  float* o = out + (int64_t)blockIdx.x * ldo;
  for (int c = threadIdx.x; c < width; c += 256) o[c] = r[c] * rstd * (w[c] + shift);  // (a thread re-reads its own writes)
}

// The results X_0 .. X_{n-1} of the embedding and of the layers so far are the slots of one buffer (slot_stride floats
// apart).  X_{n-1} += mult * y (the last sublayer's output, may be nullptr); slot n <- sum_j coef[j] X_j; norm_w != nullptr:
// h = slot n / rms * (norm_w + shift) - what the next layer's mixer reads.
__global__ __launch_bounds__(256) void depth_mix_f32_kernel(float* __restrict__ stack, int64_t slot_stride, int n,
                                                            const float* __restrict__ coef, const float* __restrict__ y,
                                                            int64_t ldy, float mult, const float* __restrict__ norm_w,
                                                            float shift, float eps, float* __restrict__ h, int64_t ldh,
                                                            int width) {
  __shared__ float red[4];
  float* base = stack + (int64_t)blockIdx.x * width;
  float* last = base + (int64_t)(n - 1) * slot_stride;
  float* dst = base + (int64_t)n * slot_stride;
  const float* yr = y ? y + (int64_t)blockIdx.x * ldy : nullptr;
  float sq = 0.f;
  for (int c = threadIdx.x; c < width; c += 256) {
    float xl = last[c];
    if (yr) {
      xl = fmaf(mult, yr[c], xl);
      last[c] = xl;
    }
    float acc = 0.f;
    for (int j = 0; j + 1 < n; ++j) acc = fmaf(coef[j], base[(int64_t)j * slot_stride + c], acc);
    acc = fmaf(coef[n - 1], xl, acc);
    dst[c] = acc;
    sq = fmaf(acc, acc, sq);
  }
  if (!norm_w) return;
  const float rstd = 1.f / sqrtf(block_sum256(sq, red) / (float)width + eps);
  float* o = h + (int64_t)blockIdx.x * ldh;
  for (int c = threadIdx.x; c < width; c += 256) o[c] = dst[c] * rstd * (norm_w[c] + shift);
}

// ---------------------------------------------------------------------------------------------------------------
// minimal gated recurrence: S_p = (1 - z_p) S_{p-1} + z_p c_p per channel, out = S_p * silu(g_p)
// ---------------------------------------------------------------------------------------------------------------
// z = sigmoid(zp), c = up + 1/2 (up >= 0) | sigmoid(up) (up < 0); zp, up, gp are columns of one projection buffer.
// The recurrence is linear in S, so a sequence's rows of this step are cut into segments of kScanSeg rows that are
// walked in parallel: (1) every segment but a sequence's last computes its (A, B) with S_end = A S_start + B;
// (2) one thread per (sequence, channel) turns them into every segment's S_start, beginning with the slot's state (zero
// when the sequence starts in this step); (3) every segment walks its rows from its S_start and writes the outputs, a
// sequence's last segment also the slot's new state.  A step whose sequences all fit one segment (decode steps, short
// portions) is launch (3) alone.
constexpr int kScanSeg = 64;

struct ScanSeg {
  int s, first, count, index, total;  // sequence, first step row, rows, segment index within the sequence, its segments
};
// segment `id` of the step (segments are numbered sequence by sequence); count = 0: beyond the last one
__device__ __forceinline__ ScanSeg scan_segment(const int32_t* cu_q, int n_seqs, int id) {
  ScanSeg r{0, 0, 0, 0, 0};
  for (int s = 0; s < n_seqs; ++s) {
    const int n = cu_q[s + 1] - cu_q[s];
    const int segs = (n + kScanSeg - 1) / kScanSeg;
    if (id < segs) {
      r.s = s, r.index = id, r.total = segs;
      r.first = cu_q[s] + id * kScanSeg;
      r.count = min(kScanSeg, n - id * kScanSeg);
      return r;
    }
    id -= segs;
  }
  return r;
}
__device__ __forceinline__ void mingru_gates(float zp, float up, float& keep, float& add) {
  const float z = sigmoid_f(zp);
  const float c = up >= 0.f ? up + 0.5f : sigmoid_f(up);
  keep = 1.f - z;
  add = z * c;
}

__global__ __launch_bounds__(256) void mingru_summary_kernel(const float* __restrict__ proj, int64_t ld, int z_off,
                                                             int x_off, const int32_t* __restrict__ cu_q, int n_seqs,
                                                             int width, float* __restrict__ summary) {
  const int c = blockIdx.x * 256 + threadIdx.x;
  const ScanSeg sg = scan_segment(cu_q, n_seqs, blockIdx.y);
  if (c >= width || sg.count == 0 || sg.index + 1 == sg.total) return;
  float A = 1.f, B = 0.f;
  // eight rows' operands are fetched before the first of them is used: the loads do not depend on the running pair
  for (int r0 = 0; r0 < sg.count; r0 += 8) {
    float zp[8], up[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float* row = proj + (int64_t)(sg.first + min(r0 + i, sg.count - 1)) * ld;
      zp[i] = row[z_off + c], up[i] = row[x_off + c];
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      if (r0 + i < sg.count) {
        float keep, add;
        mingru_gates(zp[i], up[i], keep, add);
        A *= keep;
        B = fmaf(keep, B, add);
      }
    }
  }
  summary[((int64_t)blockIdx.y * 2) * width + c] = A;
  summary[((int64_t)blockIdx.y * 2 + 1) * width + c] = B;
}

// S_start of every segment, written over the segment's A (segment 0 of a sequence: the carried state)
__global__ __launch_bounds__(256) void mingru_carry_kernel(float* __restrict__ summary, const float* __restrict__ state,
                                                           const int32_t* __restrict__ cu_q,
                                                           const int32_t* __restrict__ kv_lens,
                                                           const int32_t* __restrict__ slot_ids, int width) {
  const int s = blockIdx.y;
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= width) return;
  const int n = cu_q[s + 1] - cu_q[s];
  if (n == 0) return;
  int id0 = 0;
  for (int t = 0; t < s; ++t) id0 += (cu_q[t + 1] - cu_q[t] + kScanSeg - 1) / kScanSeg;
  const int segs = (n + kScanSeg - 1) / kScanSeg;
  float S = kv_lens[s] - n > 0 ? state[(int64_t)slot_ids[s] * width + c] : 0.f;
  for (int k = 0; k < segs; ++k) {
    float* e = summary + ((int64_t)(id0 + k) * 2) * width + c;
    const float A = e[0], B = e[width];
    e[0] = S;
    if (k + 1 < segs) S = fmaf(A, S, B);
  }
}

template <bool CARRIED>  // CARRIED: S_start from the summary buffer; else every sequence is one segment: from the slot
__global__ __launch_bounds__(256) void mingru_walk_kernel(const float* __restrict__ proj, int64_t ld, int z_off, int x_off,
                                                          int g_off, const float* __restrict__ summary,
                                                          float* __restrict__ state, const int32_t* __restrict__ cu_q,
                                                          const int32_t* __restrict__ kv_lens,
                                                          const int32_t* __restrict__ slot_ids, int n_seqs, int width,
                                                          float* __restrict__ out, int64_t ldo) {
  const int c = blockIdx.x * 256 + threadIdx.x;
  const ScanSeg sg = scan_segment(cu_q, n_seqs, blockIdx.y);
  if (c >= width || sg.count == 0) return;
  float S;
  if (CARRIED) S = summary[((int64_t)blockIdx.y * 2) * width + c];
  else S = kv_lens[sg.s] - (cu_q[sg.s + 1] - cu_q[sg.s]) > 0 ? state[(int64_t)slot_ids[sg.s] * width + c] : 0.f;
  for (int r0 = 0; r0 < sg.count; r0 += 8) {
    float zp[8], up[8], gp[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float* row = proj + (int64_t)(sg.first + min(r0 + i, sg.count - 1)) * ld;
      zp[i] = row[z_off + c], up[i] = row[x_off + c], gp[i] = row[g_off + c];
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      if (r0 + i < sg.count) {
        float keep, add;
        mingru_gates(zp[i], up[i], keep, add);
        S = fmaf(keep, S, add);
        out[(int64_t)(sg.first + r0 + i) * ldo + c] = S * (gp[i] / (1.f + expf(-gp[i])));
      }
    }
  }
  if (sg.index + 1 == sg.total) state[(int64_t)slot_ids[sg.s] * width + c] = S;
}

// ---------------------------------------------------------------------------------------------------------------
// per-row preparation of the paged attentions without a whole-projection norm
// ---------------------------------------------------------------------------------------------------------------
// Plain grouped heads: q <- q * (1 + coef * ln(floor((p + 1) / every) + 1)) in place (every < 1: no temperature), k and
// v rows to the cache.  One workgroup per row.
template <typename TC>
__global__ __launch_bounds__(256) void kv_store_temp_kernel(float* __restrict__ proj, int64_t ld, int q_off, int k_off,
                                                            int v_off, int nq, float coef, int every,
                                                            const int32_t* __restrict__ cu_q,
                                                            const int32_t* __restrict__ kv_lens, int n_seqs,
                                                            TC* __restrict__ k_cache, TC* __restrict__ v_cache,
                                                            const int32_t* __restrict__ slots, int G, int D, int Dv,
                                                            int block_size) {
  const int row = blockIdx.x;
  float* r = proj + (int64_t)row * ld;
  if (every >= 1) {
    const int s = seq_of_row(cu_q, n_seqs, row);
    const int pos = kv_lens[s] - (cu_q[s + 1] - cu_q[s]) + (row - cu_q[s]);
    const float temp = 1.f + coef * logf((float)((pos + 1) / every) + 1.f);
    for (int c = threadIdx.x; c < nq; c += 256) r[q_off + c] *= temp;
  }
  const int slot = slots[row];
  if (slot < 0) return;
  const int64_t blk = slot / block_size;
  const int off = slot % block_size;
  for (int c = threadIdx.x; c < G * D; c += 256)
    st_f<TC>(k_cache + ((blk * G + c / D) * block_size + off) * D + c % D, r[k_off + c]);
  for (int c = threadIdx.x; c < G * Dv; c += 256)
    st_f<TC>(v_cache + ((blk * G + c / Dv) * block_size + off) * Dv + c % Dv, r[v_off + c]);
}

// Latent attention: the row's compressed key/value c (C entries at c_off) is RMS-normed with a plain weight and stored as
// the leading C channels of the row's cache entry, the shared rotated key part (R entries behind it) is rotated by the
// row's position and stored behind them: a cache row is [c | r], one "kv head" that every query head reads, keys = the
// whole row, values = its first C channels.  The rotated part of every query head (R entries at q_off + h * (D + R) + D)
// is rotated and written to qx[row][h][C ..] - the head's absorbed key-space query [W_uk^T q | rot(q_r)] whose first C
// entries a batched projection fills in.  Rotation: the first `dims` entries, pairs (i, i + dims / 2), angle
// pos * inv_freq[i] formed and turned into sine and cosine in fp32 (sincosf of the device library); inv_freq [dims / 2]
// is the host's table of base^(-2 i / dims), rounded once from double.
template <typename TC>
__global__ __launch_bounds__(256) void latent_prepare_kernel(const float* __restrict__ proj, int64_t ld,
                                                             const float* __restrict__ q, int64_t ldq, int q_off,
                                                             int c_off, int H, int D, int R, int C, int dims,
                                                             const float* __restrict__ inv_freq,
                                                             const float* __restrict__ norm_w, float eps,
                                                             const int32_t* __restrict__ cu_q,
                                                             const int32_t* __restrict__ kv_lens, int n_seqs,
                                                             TC* __restrict__ cache, const int32_t* __restrict__ slots,
                                                             float* __restrict__ qx, int64_t ldqx) {
  __shared__ float red[4];
  const int row = blockIdx.x;
  const float* r = proj + (int64_t)row * ld;
  const int s = seq_of_row(cu_q, n_seqs, row);
  const int pos = kv_lens[s] - (cu_q[s + 1] - cu_q[s]) + (row - cu_q[s]);
  float sq = 0.f;
  for (int c = threadIdx.x; c < C; c += 256) sq = fmaf(r[c_off + c], r[c_off + c], sq);
  const float rstd = 1.f / sqrtf(block_sum256(sq, red) / (float)C + eps);
  const int slot = slots[row];
  TC* dst = slot >= 0 ? cache + (int64_t)slot * (C + R) : nullptr;
  if (dst)
    for (int c = threadIdx.x; c < C; c += 256) st_f<TC>(dst + c, r[c_off + c] * rstd * norm_w[c]);
  const int half = dims / 2;
  // unit u = 0: the shared key part; u = 1 + h: query head h
  for (int i = threadIdx.x; i < (H + 1) * R; i += 256) {
    const int u = i / R, e = i % R;
    const float* src = u == 0 ? r + c_off + C : q + (int64_t)row * ldq + q_off + (int64_t)(u - 1) * (D + R) + D;
    float v = src[e];
    if (e < dims) {
      const int f = e < half ? e : e - half;
      const float ang = (float)pos * inv_freq[f];
      float sn, cs;
      sincosf(ang, &sn, &cs);
      v = e < half ? src[e] * cs - src[e + half] * sn : src[e] * cs + src[e - half] * sn;
    }
    if (u == 0) {
      if (dst) st_f<TC>(dst + C + e, v);
    } else {
      qx[(int64_t)row * ldqx + (int64_t)(u - 1) * (C + R) + C + e] = v;
    }
  }
}

// ---------------------------------------------------------------------------------------------------------------
// plain top-k router: the top_k largest logits (equal values: the lower index), weights = softmax over the chosen
// ---------------------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void route_topk_kernel(const float* __restrict__ logits, int64_t ld, int T, int n,
                                                         int top_k, int32_t* __restrict__ ids, float* __restrict__ wts) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int t = blockIdx.x * 4 + wave;
  if (t >= T) return;
  const float* z = logits + (int64_t)t * ld;
  constexpr int EPL = 8;
  const int big = 1 << 30;
  float sc[EPL];
#pragma unroll
  for (int i = 0; i < EPL; ++i) {
    const int e = lane + 64 * i;
    sc[i] = e < n ? z[e] : -INFINITY;
    if (!(sc[i] == sc[i])) sc[i] = -INFINITY;
  }
  unsigned taken = 0;
#pragma unroll
  for (int i = 0; i < EPL; ++i)
    if (lane + 64 * i >= n) taken |= 1u << i;
  float top = 0.f, sum = 0.f;
  float mine[EPL];  // exp(logit - top) of the outputs this lane gave away, in pick order
  int my_slot[EPL], n_mine = 0;
  for (int it = 0; it < top_k; ++it) {
    float bv = -INFINITY;
    int bi = big;
#pragma unroll
    for (int i = 0; i < EPL; ++i)
      if (!(taken >> i & 1) && (bi == big || sc[i] > bv)) bv = sc[i], bi = lane + 64 * i;
    wave_argmax(bv, bi);
    if (it == 0) top = bv;
    const float p = expf(bv - top);
    sum += p;
    if ((bi & 63) == lane) {
      taken |= 1u << (bi >> 6);
      ids[(int64_t)t * top_k + it] = bi;
#pragma unroll
      for (int i = 0; i < EPL; ++i)
        if (i == n_mine) mine[i] = p, my_slot[i] = it;
      ++n_mine;
    }
  }
#pragma unroll
  for (int i = 0; i < EPL; ++i)
    if (i < n_mine) wts[(int64_t)t * top_k + my_slot[i]] = mine[i] / sum;
}

// out[t] = sum_k w[t][k] y[t * top_k + k] + sigmoid(shared_gate[t]) * shared[t]   (shared == nullptr: no shared part;
// wts == nullptr: every weight 1 - experts whose weight already went into their input)
__global__ __launch_bounds__(256) void moe_combine_shared_kernel(const float* __restrict__ y, const int32_t* __restrict__ ids,
                                                                 const float* __restrict__ wts, int top_k, int width,
                                                                 const float* __restrict__ shared, int64_t lds_,
                                                                 const float* __restrict__ shared_gate, int64_t ldsg,
                                                                 float* __restrict__ out, int64_t ldo) {
  const int t = blockIdx.x;
  const float sgate = shared ? sigmoid_f(shared_gate[(int64_t)t * ldsg]) : 0.f;
  for (int c = threadIdx.x; c < width; c += 256) {
    float acc = 0.f;
    for (int k = 0; k < top_k; ++k)
      acc = fmaf(wts ? wts[(int64_t)t * top_k + k] : 1.f, y[((int64_t)t * top_k + k) * width + c], acc);
    if (shared) acc = fmaf(sgate, shared[(int64_t)t * lds_ + c], acc);
    out[(int64_t)t * ldo + c] = acc;
  }
}


// ---------------------------------------------------------------------------------------------------------------
// gated sublayer output behind its own norm, added to the residual: res += rms(y * sigmoid(gate)) * w_post
// ---------------------------------------------------------------------------------------------------------------
// One workgroup per row.  v = y * sigmoid(gate_pre) (gate_pre may be nullptr: v = y); res += v / sqrt(mean(v^2) + eps) *
// w_post; w_next != nullptr: out = res / sqrt(mean(res^2) + eps) * w_next - what the next sublayer reads.  A thread keeps
// its (up to eight) gated values in registers between the two passes; wider rows recompute them.
__global__ __launch_bounds__(256) void gated_norm_add_f32_kernel(float* __restrict__ res, int64_t ldr,
                                                                 const float* __restrict__ y, int64_t ldy,
                                                                 const float* __restrict__ gate_pre, int64_t ldg,
                                                                 const float* __restrict__ w_post, float eps,
                                                                 const float* __restrict__ w_next,
                                                                 float* __restrict__ out, int64_t ldo, int width) {
  __shared__ float red[4];
  constexpr int KEEP = 8;
  float* r = res + (int64_t)blockIdx.x * ldr;
  const float* yr = y + (int64_t)blockIdx.x * ldy;
  const float* gr = gate_pre ? gate_pre + (int64_t)blockIdx.x * ldg : nullptr;
  float kept[KEEP];
  float sq = 0.f;
  int i = 0;
  for (int c = threadIdx.x; c < width; c += 256, ++i) {
    float v = yr[c];
    if (gr) v *= sigmoid_f(gr[c]);
    if (i < KEEP) kept[i] = v;
    sq = fmaf(v, v, sq);
  }
  const float rstd = 1.f / sqrtf(block_sum256(sq, red) / (float)width + eps);
  float sq2 = 0.f;
  i = 0;
  for (int c = threadIdx.x; c < width; c += 256, ++i) {
    float v;
    if (i < KEEP) v = kept[i];
    else {
      v = yr[c];
      if (gr) v *= sigmoid_f(gr[c]);
    }
    const float x = fmaf(v * rstd, w_post[c], r[c]);
    r[c] = x;
    if (i < KEEP) kept[i] = x;
    sq2 = fmaf(x, x, sq2);
  }
  if (!w_next) return;
  const float rstd2 = 1.f / sqrtf(block_sum256(sq2, red) / (float)width + eps);
  float* o = out + (int64_t)blockIdx.x * ldo;
  i = 0;
  for (int c = threadIdx.x; c < width; c += 256, ++i) o[c] = (i < KEEP ? kept[i] : r[c]) * rstd2 * w_next[c];
}

// ---------------------------------------------------------------------------------------------------------------
// linear attention with a decayed matrix state: S <- diag(a_t) S + k_t v_t^T,  o_t = S^T q_t
// ---------------------------------------------------------------------------------------------------------------
// Two kinds of decay (DECAY):
//   MI_DECAY_HEAD    a_t = decay[h] for every key channel of head h and every row; q, k, v = act(projection)
//   MI_DECAY_FORGET  a_t = f_t = lower + (1 - lower) * sigmoid(z_t + f_bias) per key channel (z at k_off), and what is
//                    written is k_t = 1 - f_t: the forget gate also decides how much of v_t enters
// The walk has channel_delta_kernel's shape with SIXTEEN lanes per value column (the rule has one pass over the state per
// row where the delta rule has two, and a prompt step's few (sequence, head) units should put two waves on every SIMD:
// measured on 8 sequences x 1024 rows x 8 heads x 128 x 128 channels, 4 / 8 / 16 lanes per column: 785 / 417 / 304 us):
// a workgroup = 32 value columns of one (sequence, head) = 512 threads; lane r of a column's sixteen keeps the key
// channels (16 jj + r) * 4 + e in registers for the whole walk over the step's rows; the rows' vectors of 16 rows at a
// time go through LDS, loaded one batch ahead as raw projections (32 lanes per row) and turned into q / k / a
// (activations, gate, lower bound) on their way into LDS - no separate preparation launch; the sum over the key channels
// ends in four DPP steps inside a 16-lane row.  The state lives in memory as [slot][head][column block][key channel / 4]
// [32 columns][4]: a thread's four channels of a column are one 16-byte piece, a wave's loads whole 256-byte runs.
constexpr int kLinLanes = 16, kLinThreads = kLinLanes * kDeltaCols, kLinStage = kLinThreads / kDeltaRows;
static_assert(kLinStage * kDeltaRows == kLinThreads && kDeltaCols % kLinStage == 0, "whole staging lanes per row");
static_assert(kLinLanes == 16, "the read-out's butterfly (1, 2, 4, 8) spans a column's lanes");

template <int DR, int DECAY>  // DR: key channels per lane (the head's channels padded to kLinLanes * DR)
__global__ __launch_bounds__(kLinThreads) void linear_attention_kernel(
    const float* __restrict__ proj, int64_t ld, int q_off, int k_off, int v_off, int q_act, int k_act, int v_act,
    const float* __restrict__ decay, const float* __restrict__ f_bias, const float* __restrict__ lower,
    float* __restrict__ state, const int32_t* __restrict__ cu_q, const int32_t* __restrict__ kv_lens,
    const int32_t* __restrict__ slot_ids, int H, int D, int Dv, float* __restrict__ out, int64_t ldo) {
  constexpr int DP = kLinLanes * DR;  // padded key channels
  constexpr bool FORGET = DECAY == MI_DECAY_FORGET;
  __shared__ __attribute__((aligned(16))) float qs[kDeltaRows][DP];
  __shared__ __attribute__((aligned(16))) float ks[kDeltaRows][DP];
  __shared__ __attribute__((aligned(16))) float gs[FORGET ? kDeltaRows : 1][DP];
  __shared__ float vs[kDeltaRows][kDeltaCols];
  const int s = blockIdx.x, h = blockIdx.y, cb = blockIdx.z;
  const int tid = threadIdx.x, r = tid & (kLinLanes - 1), col = tid / kLinLanes;
  const int c = cb * kDeltaCols + col;
  const int r0 = cu_q[s], n = cu_q[s + 1] - r0;
  if (n == 0) return;
  const int start = kv_lens[s] - n;
  float* slot = state + (((int64_t)slot_ids[s] * H + h) * gridDim.z + cb) * DP * kDeltaCols;
  float st[DR];
#pragma unroll
  for (int jj = 0; jj < DR / 4; ++jj) {
    float4 v4{0.f, 0.f, 0.f, 0.f};
    if (start > 0) v4 = *reinterpret_cast<const float4*>(slot + ((jj * kLinLanes + r) * kDeltaCols + col) * 4);
    st[jj * 4 + 0] = v4.x, st[jj * 4 + 1] = v4.y, st[jj * 4 + 2] = v4.z, st[jj * 4 + 3] = v4.w;
  }
  const float head_decay = FORGET ? 0.f : decay[h];
  // staging: kLinStage lanes per row copy the row's vectors (zeros beyond D and beyond the step's rows)
  const int pt = tid / kLinStage, ps = tid % kLinStage;
  constexpr int PE = DP / kLinStage;
  float rq[PE], rk[PE], rv[kDeltaCols / kLinStage];
  auto fetch = [&](int c0) {
    const bool live = c0 + pt < n;
    const int64_t row = r0 + (live ? c0 + pt : 0);
    const float* p = proj + row * ld;
#pragma unroll
    for (int m = 0; m < PE; ++m) {
      const int i = ps + kLinStage * m;
      const bool ok = live && i < D;
      rq[m] = ok ? p[q_off + h * D + i] : 0.f;
      rk[m] = ok ? p[k_off + h * D + i] : 0.f;
    }
#pragma unroll
    for (int m = 0; m < kDeltaCols / kLinStage; ++m) {
      const int cc = cb * kDeltaCols + ps + kLinStage * m;
      rv[m] = (live && cc < Dv) ? p[v_off + h * Dv + cc] : 0.f;
    }
  };
  auto act = [](int kind, float z) { return kind == MI_ACT_SILU ? z / (1.f + expf(-z)) : z; };
  fetch(0);
  for (int c0 = 0; c0 < n; c0 += kDeltaRows) {
    __syncthreads();  // the previous rows' vectors have been consumed
    const bool live = c0 + pt < n;
#pragma unroll
    for (int m = 0; m < PE; ++m) {
      const int i = ps + kLinStage * m;
      const bool ok = live && i < D;
      qs[pt][i] = ok ? act(q_act, rq[m]) : 0.f;
      if constexpr (FORGET) {
        const float lo = i < D ? lower[h * D + i] : 0.f, fb = i < D ? f_bias[h * D + i] : 0.f;  // (cached: every batch)
        const float f = lo + (1.f - lo) * sigmoid_f(rk[m] + fb);
        gs[pt][i] = ok ? f : 0.f;
        ks[pt][i] = ok ? 1.f - f : 0.f;
      } else {
        ks[pt][i] = ok ? act(k_act, rk[m]) : 0.f;
      }
    }
#pragma unroll
    for (int m = 0; m < kDeltaCols / kLinStage; ++m) vs[pt][ps + kLinStage * m] = act(v_act, rv[m]);
    __syncthreads();
    if (c0 + kDeltaRows < n) fetch(c0 + kDeltaRows);
    const int nt = min(kDeltaRows, n - c0);
    for (int t = 0; t < nt; ++t) {
      const float4* k4 = reinterpret_cast<const float4*>(ks[t]);
      const float4* q4 = reinterpret_cast<const float4*>(qs[t]);
      const float4* g4 = reinterpret_cast<const float4*>(gs[FORGET ? t : 0]);
      const float v = vs[t][col];
      float o0 = 0.f, o1 = 0.f, o2 = 0.f, o3 = 0.f;
#pragma unroll
      for (int jj = 0; jj < DR / 4; ++jj) {
        const float4 kv = k4[jj * kLinLanes + r], qv = q4[jj * kLinLanes + r];
        float4 gv{head_decay, head_decay, head_decay, head_decay};
        if constexpr (FORGET) gv = g4[jj * kLinLanes + r];
        st[jj * 4 + 0] = fmaf(gv.x, st[jj * 4 + 0], kv.x * v);
        st[jj * 4 + 1] = fmaf(gv.y, st[jj * 4 + 1], kv.y * v);
        st[jj * 4 + 2] = fmaf(gv.z, st[jj * 4 + 2], kv.z * v);
        st[jj * 4 + 3] = fmaf(gv.w, st[jj * 4 + 3], kv.w * v);
        o0 = fmaf(st[jj * 4 + 0], qv.x, o0);
        o1 = fmaf(st[jj * 4 + 1], qv.y, o1);
        o2 = fmaf(st[jj * 4 + 2], qv.z, o2);
        o3 = fmaf(st[jj * 4 + 3], qv.w, o3);
      }
      const float o = xor_sum<8>(xor_sum<4>(xor_sum<2>(xor_sum<1>((o0 + o1) + (o2 + o3)))));
      if (r == 0 && c < Dv) out[(int64_t)(r0 + c0 + t) * ldo + h * Dv + c] = o;
    }
  }
#pragma unroll
  for (int jj = 0; jj < DR / 4; ++jj)
    *reinterpret_cast<float4*>(slot + ((jj * kLinLanes + r) * kDeltaCols + col) * 4) =
        float4{st[jj * 4 + 0], st[jj * 4 + 1], st[jj * 4 + 2], st[jj * 4 + 3]};
}

// out[row] <- out / rms(out over the row's `width` channels) * norm_w (* sigmoid(gate)): a workgroup per row, in place -
// the read-out's norm over ALL heads of a row (delta_finish_kernel's wave per unit is for a norm per head)
__global__ __launch_bounds__(256) void row_norm_gate_kernel(float* __restrict__ out, int64_t ldo,
                                                            const float* __restrict__ gate_pre, int64_t ld_gate,
                                                            const float* __restrict__ norm_w, int width, float eps) {
  __shared__ float red[4];
  float* o = out + (int64_t)blockIdx.x * ldo;
  float sq = 0.f;
  for (int d = threadIdx.x; d < width; d += 256) sq = fmaf(o[d], o[d], sq);
  const float rstd = 1.f / sqrtf(block_sum256(sq, red) / (float)width + eps);
  for (int d = threadIdx.x; d < width; d += 256)
    o[d] = o[d] * rstd * norm_w[d] * (gate_pre ? sigmoid_f(gate_pre[(int64_t)blockIdx.x * ld_gate + d]) : 1.f);
}

// ---------------------------------------------------------------------------------------------------------------
// rotary positions on projected heads, unit norm per head, K / V rows to the pages
// ---------------------------------------------------------------------------------------------------------------
// One workgroup per step row, a wave per head in turn (H query heads at q_off, G key heads at k_off of the row).  The
// first rot_dims channels of a head are rotated by the angles pos * inv_freq[i] (fp32 product, sincosf), cos and sin
// times `amp`: channel pairs (2i, 2i + 1) (layout MI_ROT_INTERLEAVED) or (i, i + rot_dims / 2) (MI_ROT_HALVES).  Then,
// unit_norm: the head is divided by sqrt(mean(head^2) + eps); key heads are multiplied by k_mult on top.  Query heads
// are written back in place.  Key heads go to the paged cache [blocks][G][block_size][D] when k_cache != nullptr (rows
// with slot < 0 store nothing), else back in place.  v_cache != nullptr: the row's Gv value heads of Dv channels at v_off
// are copied to [blocks][Gv][block_size][Dv] as they are.
template <typename TC>
__global__ __launch_bounds__(256) void rotary_store_kernel(float* __restrict__ proj, int64_t ld, int q_off, int k_off,
                                                           int v_off, int H, int G, int D, int Gv, int Dv, int rot_dims,
                                                           int layout, const float* __restrict__ inv_freq, float amp,
                                                           int unit_norm, float eps, float k_mult,
                                                           const int32_t* __restrict__ cu_q,
                                                           const int32_t* __restrict__ kv_lens, int n_seqs,
                                                           TC* __restrict__ k_cache, TC* __restrict__ v_cache,
                                                           const int32_t* __restrict__ slots, int block_size) {
  extern __shared__ float smem[];  // per wave: one head [D]
  const int row = blockIdx.x, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int s = seq_of_row(cu_q, n_seqs, row);
  const float pos = (float)(kv_lens[s] - (cu_q[s + 1] - cu_q[s]) + (row - cu_q[s]));
  const int slot = slots ? slots[row] : -1;
  const int64_t blk = slot >= 0 ? slot / block_size : 0;
  const int off = slot >= 0 ? slot % block_size : 0;
  float* hv = smem + wave * D;
  float* base = proj + (int64_t)row * ld;
  const int half = rot_dims / 2;
  for (int head = wave; head < H + G; head += 4) {
    const bool is_k = head >= H;
    float* src = base + (is_k ? k_off + (head - H) * D : q_off + head * D);
    for (int d = lane; d < D; d += 64) hv[d] = src[d];
    __builtin_amdgcn_wave_barrier();
    for (int i = lane; i < half; i += 64) {
      float sn, cs;
      sincosf(pos * inv_freq[i], &sn, &cs);
      sn *= amp, cs *= amp;
      const int ia = layout == MI_ROT_INTERLEAVED ? 2 * i : i, ib = layout == MI_ROT_INTERLEAVED ? 2 * i + 1 : i + half;
      const float a = hv[ia], b = hv[ib];
      hv[ia] = a * cs - b * sn;
      hv[ib] = b * cs + a * sn;
    }
    __builtin_amdgcn_wave_barrier();
    float mult = is_k ? k_mult : 1.f;
    if (unit_norm) {
      float sq = 0.f;
      for (int d = lane; d < D; d += 64) sq = fmaf(hv[d], hv[d], sq);
      mult *= 1.f / sqrtf(wave_sum(sq) / (float)D + eps);
    }
    if (is_k && k_cache) {
      if (slot >= 0) {
        TC* dst = k_cache + ((blk * G + (head - H)) * block_size + off) * D;
        for (int d = lane; d < D; d += 64) st_f<TC>(dst + d, hv[d] * mult);
      }
    } else {
      for (int d = lane; d < D; d += 64) src[d] = hv[d] * mult;
    }
    __builtin_amdgcn_wave_barrier();
  }
  if (v_cache && slot >= 0) {
    const float* v = base + v_off;
    for (int c = threadIdx.x; c < Gv * Dv; c += 256) {
      const int g = c / Dv, d = c - g * Dv;
      st_f<TC>(v_cache + ((blk * Gv + g) * block_size + off) * Dv + d, v[c]);
    }
  }
}

// Mixing of the heads' softmax weights, done on the read-outs (the mixing is linear in the weights): `o` holds, for every
// query head g, that head's weights applied to the values of n_chunk key/value heads [c0, c0 + n_chunk) side by side
// ([rows][H][n_chunk * Dv]); out[row][h][:] = out_scale * sum_g talk[h][g] * o[row][g][(kv(h) - c0) * Dv + :] for the heads
// h whose own key/value head kv(h) = h / (H / G) lies in the chunk.  A thread per (row, h, d).
__global__ __launch_bounds__(256) void head_mix_kernel(const float* __restrict__ o, int64_t ldo_in,
                                                       const float* __restrict__ talk, int n_rows, int H, int G, int Dv,
                                                       int c0, int n_chunk, float out_scale, float* __restrict__ out,
                                                       int64_t ldo) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (int64_t)n_rows * H * Dv) return;
  const int d = (int)(idx % Dv), h = (int)((idx / Dv) % H);
  const int64_t row = idx / ((int64_t)Dv * H);
  const int c = h / (H / G) - c0;
  if (c < 0 || c >= n_chunk) return;
  const float* src = o + row * ldo_in + c * Dv + d;
  float acc = 0.f;
  for (int g = 0; g < H; ++g) acc = fmaf(talk[h * H + g], src[(int64_t)g * n_chunk * Dv], acc);
  out[row * ldo + h * Dv + d] = acc * out_scale;
}

}  // namespace mi

using namespace mi;

extern "C" int mi_embedding_f32(const int64_t* ids, const void* table, int table_dtype, float* out, int n, int width,
                                int vocab, float scale, mi_stream stream) {
  if (!ids || !table || !out || n < 0 || width < 1) return MI_EINVAL;
  if (n == 0) return MI_OK;
  if (table_dtype == MI_DTYPE_BF16)
    hipLaunchKernelGGL((embedding_f32_kernel<uint16_t>), dim3(n), dim3(256), 0, S(stream), ids,
                       static_cast<const uint16_t*>(table), out, width, vocab, scale);
  else if (table_dtype == MI_DTYPE_F32)
    hipLaunchKernelGGL((embedding_f32_kernel<float>), dim3(n), dim3(256), 0, S(stream), ids,
                       static_cast<const float*>(table), out, width, vocab, scale);
  else return MI_EINVAL;
  return check_launch();
}

extern "C" int mi_layernorm_f32(const float* y, int64_t ldy, const float* w, const float* b, float* out, int64_t ldo,
                                int rows, int width, float eps, int add_to_out, mi_stream stream) {
  if (!y || !w || !b || !out || rows < 0 || width < 1 || ldy < width || ldo < width) return MI_EINVAL;
  if (rows == 0) return MI_OK;
  hipLaunchKernelGGL(layernorm_f32_kernel, dim3(rows), dim3(256), 0, S(stream), y, ldy, w, b, out, ldo, width, eps,
                     add_to_out);
  return check_launch();
}

extern "C" int mi_swa_prepare(float* proj, int64_t ld, int q_off, int k_off, int v_off, const float* qn_w,
                              const float* kn_w, float eps, const float* v_first, int64_t ld_vf, const float* lam,
                              void* k_cache, void* v_cache, int cache_dtype, const int32_t* slots, int rows, int H,
                              int G, int D, int Dv, int block_size, mi_stream stream) {
  if (!proj || !qn_w || !kn_w || !k_cache || !v_cache || !slots || rows < 0) return MI_EINVAL;
  if (H < 1 || G < 1 || D < 1 || Dv < 1 || block_size < 1 || (v_first && !lam)) return MI_EINVAL;
  if (rows == 0) return MI_OK;
  if (cache_dtype == MI_DTYPE_BF16)
    hipLaunchKernelGGL((swa_prepare_kernel<uint16_t>), dim3(rows), dim3(256), 0, S(stream), proj, ld, q_off, k_off,
                       v_off, H * D, G * D, G * Dv, qn_w, kn_w, eps, v_first, ld_vf, lam,
                       static_cast<uint16_t*>(k_cache), static_cast<uint16_t*>(v_cache), slots, G, D, Dv, block_size);
  else if (cache_dtype == MI_DTYPE_F32)
    hipLaunchKernelGGL((swa_prepare_kernel<float>), dim3(rows), dim3(256), 0, S(stream), proj, ld, q_off, k_off, v_off,
                       H * D, G * D, G * Dv, qn_w, kn_w, eps, v_first, ld_vf, lam, static_cast<float*>(k_cache),
                       static_cast<float*>(v_cache), slots, G, D, Dv, block_size);
  else return MI_EINVAL;
  return check_launch();
}

template <typename TC>
static int launch_swa(const float* q, int64_t ldq, const void* kc, const void* vc, const int32_t* bt, int cols,
                      const int32_t* cu_q, const int32_t* kv_lens, int n_seqs, int rows, int H, int G, int D, int Dv,
                      int block_size, int window, float scale, AttnBias bias, int64_t ldv, const float* gate, int64_t ldg,
                      float* out, int64_t ldo, float* ws, int64_t ws_elems, hipStream_t st) {
  const TC* k = static_cast<const TC*>(kc);
  const TC* v = static_cast<const TC*>(vc);
  constexpr int VEC = 16 / sizeof(TC);
  // (v may point at a column of wider value rows: the fast forms load it in 16-byte / 4-byte pieces)
  const bool v16 = (reinterpret_cast<uintptr_t>(vc) & 15u) == 0;
  if constexpr (sizeof(TC) == 2) {
    // prompt portions over a bf16 cache: the matrix-core form
    if (v16 && rows > n_seqs && D % 32 == 0 && Dv % 16 == 0 && D <= 256 && Dv <= 256 && ldv % 2 == 0) {
      const dim3 grid_m((((rows + 15) / 16) * H + 3) / 4);
#define MI_SWA_MFMA(DKM, DVM, PAIR)                                                                                    \
  hipLaunchKernelGGL((swa_attention_mfma_kernel<DKM, DVM, PAIR>), grid_m, dim3(256), 0, st, q, ldq, k, v, bt, cols, cu_q, \
                     kv_lens, n_seqs, rows, H, G, D, Dv, block_size, window, scale, bias, ldv, gate, ldg, out, ldo)
      const bool small = D <= 128 && Dv <= 128, pair = Dv % 32 == 0;
      if (small && pair) MI_SWA_MFMA(4, 8, true);
      else if (small) MI_SWA_MFMA(4, 8, false);
      else if (pair) MI_SWA_MFMA(8, 16, true);
      else MI_SWA_MFMA(8, 16, false);
#undef MI_SWA_MFMA
      return check_launch();
    }
  }
  if constexpr (sizeof(TC) == 2) {
    // decode steps (a row per sequence) over a bf16 cache: the matrix-core form with a kv head's query heads as columns
    if (v16 && rows == n_seqs && D % 32 == 0 && Dv % 16 == 0 && D <= 256 && Dv <= 256 && ldv % 2 == 0 && G <= 65535) {
      // few (row, kv head) units: up to 16 workgroups share one, each taking every n_split-th batch of four rounds, and
      // a second launch merges their partial results (workspace: rows * H * n_split * (2 + Dv) floats)
      const int chunks = (H / G + 15) / 16;
      int n_split = 1;
      while (n_split < 16 && (int64_t)rows * G * chunks * n_split < 256 &&
             (int64_t)rows * H * (2 * n_split) * (2 + Dv) <= ws_elems)
        n_split *= 2;
      if (!ws) n_split = 1;
      const dim3 grid_h(rows, G, chunks * n_split);
#define MI_HEADS_MFMA(DKM, DVM, PAIR)                                                                                  \
  hipLaunchKernelGGL((paged_attention_heads_mfma_kernel<DKM, DVM, PAIR>), grid_h, dim3(256), 0, st, q, ldq, k, v, bt,   \
                     cols, kv_lens, H, G, D, Dv, block_size, window, scale, bias, ldv, gate, ldg, out, ldo, n_split, ws)
      const bool small = D <= 128 && Dv <= 128, pair = Dv % 32 == 0;
      if (small && pair) MI_HEADS_MFMA(4, 8, true);
      else if (small) MI_HEADS_MFMA(4, 8, false);
      else if (pair) MI_HEADS_MFMA(8, 16, true);
      else MI_HEADS_MFMA(8, 16, false);
#undef MI_HEADS_MFMA
      if (check_launch() != MI_OK) return MI_ELAUNCH;
      if (n_split == 1) return MI_OK;
#define MI_MERGE(NS)                                                                                                  \
  hipLaunchKernelGGL((paged_attention_merge_kernel<NS>), dim3((rows * H + 3) / 4), dim3(256), 0, st, ws, rows * H, H, Dv, \
                     gate, ldg, bias.sink, out, ldo)
      if (n_split == 2) MI_MERGE(2);
      else if (n_split == 4) MI_MERGE(4);
      else if (n_split == 8) MI_MERGE(8);
      else MI_MERGE(16);
#undef MI_MERGE
      return check_launch();
    }
  }
  if (v16 && D % VEC == 0 && Dv % VEC == 0 && Dv / VEC <= 64 && ldv % VEC == 0) {
    int lpr_log2 = 0;
    while ((1 << lpr_log2) * VEC < Dv) ++lpr_log2;
    // rows == n_seqs: every sequence brings one row (a decode step): a wave per row; else four rows per wave
    const int rpw = rows > n_seqs ? 4 : 1;
    const size_t lds_v = (4 * (size_t)rpw * (D + 64) + (rpw == 1 ? 4 * (size_t)(2 + Dv) : 0)) * sizeof(float);
    if (lds_v <= 48 * 1024) {
      if (rpw == 4)
        hipLaunchKernelGGL((swa_attention_vec_kernel<TC, VEC, 4, 1>), dim3((((rows + 3) / 4) * H + 3) / 4), dim3(256),
                           lds_v, st, q, ldq, k, v, bt, cols, cu_q, kv_lens, n_seqs, rows, H, G, D, Dv, block_size, window,
                           scale, bias, ldv, lpr_log2, gate, ldg, out, ldo);
      else
        hipLaunchKernelGGL((swa_attention_vec_kernel<TC, VEC, 1, 4>), dim3(rows * H), dim3(256), lds_v, st, q, ldq, k, v,
                           bt, cols, cu_q, kv_lens, n_seqs, rows, H, G, D, Dv, block_size, window, scale, bias, ldv, lpr_log2,
                           gate, ldg, out, ldo);
      return check_launch();
    }
  }
  const dim3 grid((rows * H + 3) / 4), block(256);
  const size_t lds = 4 * (size_t)(D + 64) * sizeof(float);
  if (lds > 48 * 1024) return MI_EUNSUPPORTED;
#define MI_SWA(VPL)                                                                                                  \
  hipLaunchKernelGGL((swa_attention_kernel<TC, VPL>), grid, block, lds, st, q, ldq, k, v, bt, cols, cu_q, kv_lens,     \
                     n_seqs, rows, H, G, D, Dv, block_size, window, scale, bias, ldv, gate, ldg, out, ldo)
  if (Dv <= 64) MI_SWA(1);
  else if (Dv <= 128) MI_SWA(2);
  else if (Dv <= 256) MI_SWA(4);
  else MI_SWA(8);
#undef MI_SWA
  return check_launch();
}

extern "C" int mi_swa_attention(const float* q, int64_t ldq, const void* k_cache, const void* v_cache, int cache_dtype,
                                const int32_t* block_tables, int table_cols, const int32_t* cu_q, const int32_t* kv_lens,
                                int n_seqs, int rows, int H, int G, int D, int Dv, int block_size, int window,
                                float scale, const float* gate, int64_t ldg, float* out, int64_t ldo, mi_stream stream) {
  return mi_paged_attention_f32(q, ldq, k_cache, v_cache, Dv, cache_dtype, block_tables, table_cols, cu_q, kv_lens, n_seqs,
                                rows, H, G, D, Dv, block_size, window, scale, MI_BIAS_SLOPE, nullptr, nullptr, nullptr, gate,
                                ldg, out, ldo, nullptr, 0, stream);
}

extern "C" int mi_paged_attention_f32(const float* q, int64_t ldq, const void* k_cache, const void* v_cache, int64_t ldv,
                                      int cache_dtype, const int32_t* block_tables, int table_cols, const int32_t* cu_q,
                                      const int32_t* kv_lens, int n_seqs, int rows, int H, int G, int D, int Dv,
                                      int block_size, int window, float scale, int bias_kind, const float* bias_p1,
                                      const float* bias_p2, const float* sink, const float* gate, int64_t ldg,
                                      float* out, int64_t ldo, float* workspace, int64_t workspace_elems,
                                      mi_stream stream) {
  return mi_paged_attention_ext(q, ldq, k_cache, v_cache, ldv, cache_dtype, block_tables, table_cols, cu_q, kv_lens, n_seqs,
                                rows, H, G, D, Dv, block_size, window, scale, bias_kind, bias_p1, bias_p2, sink, 0.f, G,
                                gate, ldg, out, ldo, workspace, workspace_elems, stream);
}

extern "C" int mi_paged_attention_ext(const float* q, int64_t ldq, const void* k_cache, const void* v_cache, int64_t ldv,
                                      int cache_dtype, const int32_t* block_tables, int table_cols, const int32_t* cu_q,
                                      const int32_t* kv_lens, int n_seqs, int rows, int H, int G, int D, int Dv,
                                      int block_size, int window, float scale, int bias_kind, const float* bias_p1,
                                      const float* bias_p2, const float* sink, float softcap, int value_heads,
                                      const float* gate, int64_t ldg, float* out, int64_t ldo, float* workspace,
                                      int64_t workspace_elems, mi_stream stream) {
  if (!q || !k_cache || !v_cache || !block_tables || !cu_q || !kv_lens || !out || rows < 0 || n_seqs < 1) return MI_EINVAL;
  if (H < 1 || G < 1 || H % G || D < 1 || Dv < 1 || block_size < 1 || window < 1 || table_cols < 1 || ldv < Dv) return MI_EINVAL;
  if (value_heads < 1 || G % value_heads || !(softcap >= 0.f)) return MI_EINVAL;
  if (bias_kind != MI_BIAS_SLOPE && bias_kind != MI_BIAS_LOG && bias_kind != MI_BIAS_NONE) return MI_EINVAL;
  if (bias_kind == MI_BIAS_LOG && (!bias_p1 || !bias_p2)) return MI_EINVAL;
  if (Dv > 512 || D > 4096) return MI_EUNSUPPORTED;
  if (rows == 0) return MI_OK;
  const AttnBias bias{bias_kind, bias_p1, bias_p2, sink, softcap, value_heads};
  if (cache_dtype == MI_DTYPE_BF16)
    return launch_swa<uint16_t>(q, ldq, k_cache, v_cache, block_tables, table_cols, cu_q, kv_lens, n_seqs, rows, H, G, D,
                                Dv, block_size, window, scale, bias, ldv, gate, ldg, out, ldo, workspace, workspace_elems,
                                S(stream));
  if (cache_dtype == MI_DTYPE_F32)
    return launch_swa<float>(q, ldq, k_cache, v_cache, block_tables, table_cols, cu_q, kv_lens, n_seqs, rows, H, G, D, Dv,
                             block_size, window, scale, bias, ldv, gate, ldg, out, ldo, workspace, workspace_elems,
                             S(stream));
  return MI_EINVAL;
}

extern "C" int mi_causal_conv(const float* x, int64_t ldx, const float* w, int taps, const float* state,
                              const int32_t* cu_q, const int32_t* kv_lens, const int32_t* slot_ids, int n_seqs, int rows,
                              int channels, int silu, int add_input, float* y, int64_t ldy, mi_stream stream) {
  if (!x || !w || !state || !cu_q || !kv_lens || !slot_ids || !y || rows < 0 || n_seqs < 1 || channels < 1) return MI_EINVAL;
  if (taps < 1 || taps > 17) return MI_EUNSUPPORTED;
  if (rows == 0) return MI_OK;
  hipLaunchKernelGGL(causal_conv_kernel, dim3(rows, (channels + 255) / 256), dim3(256), 0, S(stream), x, ldx, w, taps,
                     state, cu_q, kv_lens, slot_ids, n_seqs, channels, silu, add_input, y, ldy);
  return check_launch();
}

extern "C" int mi_causal_conv_advance(const float* x, int64_t ldx, const float* w, int taps, float* state,
                                      const int32_t* cu_q, const int32_t* kv_lens, const int32_t* slot_ids, int n_seqs,
                                      int rows, int max_rows_per_seq, int channels, int silu, int add_input, float* y,
                                      int64_t ldy, mi_stream stream) {
  if (!x || !w || !state || !cu_q || !kv_lens || !slot_ids || !y || rows < 0 || n_seqs < 1 || channels < 1) return MI_EINVAL;
  if (taps < 1 || taps > 17 || n_seqs > 65535) return MI_EUNSUPPORTED;
  if (rows == 0) return MI_OK;
  if (max_rows_per_seq >= 1 && max_rows_per_seq <= 8) {
    hipLaunchKernelGGL(causal_conv_step_kernel, dim3((channels + 255) / 256, n_seqs), dim3(256), 0, S(stream), x, ldx, w,
                       taps, state, cu_q, kv_lens, slot_ids, channels, silu, add_input, y, ldy);
    return check_launch();
  }
  const int rc = mi_causal_conv(x, ldx, w, taps, state, cu_q, kv_lens, slot_ids, n_seqs, rows, channels, silu, add_input, y,
                                ldy, stream);
  if (rc != MI_OK) return rc;
  return mi_causal_conv_state(x, ldx, taps, state, cu_q, kv_lens, slot_ids, n_seqs, channels, stream);
}

extern "C" int mi_causal_conv_silu(const float* x, int64_t ldx, const float* w, int taps, const float* state,
                                   const int32_t* cu_q, const int32_t* kv_lens, const int32_t* slot_ids, int n_seqs,
                                   int rows, int channels, float* y, int64_t ldy, mi_stream stream) {
  return mi_causal_conv(x, ldx, w, taps, state, cu_q, kv_lens, slot_ids, n_seqs, rows, channels, 1, 0, y, ldy, stream);
}

extern "C" int mi_causal_conv_state(const float* x, int64_t ldx, int taps, float* state, const int32_t* cu_q,
                                    const int32_t* kv_lens, const int32_t* slot_ids, int n_seqs, int channels,
                                    mi_stream stream) {
  if (!x || !state || !cu_q || !kv_lens || !slot_ids || n_seqs < 1 || channels < 1) return MI_EINVAL;
  if (taps < 1 || taps > 17) return MI_EUNSUPPORTED;
  if (taps == 1) return MI_OK;
  hipLaunchKernelGGL(causal_conv_state_kernel, dim3((channels + 255) / 256, n_seqs), dim3(256), 0, S(stream), x, ldx,
                     taps, state, cu_q, kv_lens, slot_ids, channels);
  return check_launch();
}

static int delta_dr(int D) { return D <= 64 ? 16 : D <= 128 ? 32 : D <= 256 ? 64 : 0; }

extern "C" int64_t mi_channel_delta_state_elems(int H, int D, int Dv) {
  const int dr = delta_dr(D);
  if (H < 1 || D < 1 || Dv < 1 || dr == 0) return -1;
  return (int64_t)H * ((Dv + kDeltaCols - 1) / kDeltaCols) * dr * kDeltaThreads;
}

extern "C" int64_t mi_channel_delta_workspace_elems(int n_rows, int H, int G, int D) {
  if (n_rows < 0 || H < 1 || G < 1 || D < 1) return -1;
  return (int64_t)n_rows * (2 * (int64_t)G * D + (int64_t)H * D + H);
}

extern "C" int mi_channel_delta(const float* qkv, int64_t ld, int q_off, int k_off, int v_off, const float* beta_pre,
                                int64_t ld_beta, const float* decay_pre, int64_t ld_decay, const float* dt_bias,
                                const float* a_log, const float* gate_pre, int64_t ld_gate, const float* norm_w,
                                float* state, const int32_t* cu_q, const int32_t* kv_lens, const int32_t* slot_ids,
                                int n_seqs, int n_rows, int H, int G, int D, int Dv, float eps, float* workspace,
                                float* out, int64_t ldo, mi_stream stream) {
  if (!qkv || !beta_pre || !decay_pre || !dt_bias || !a_log || !gate_pre || !norm_w || !state || !cu_q || !kv_lens ||
      !slot_ids || !out || !workspace || n_seqs < 1 || n_rows < 0)
    return MI_EINVAL;
  if (H < 1 || G < 1 || H % G || D < 1 || Dv < 1) return MI_EINVAL;
  const int dr = delta_dr(D);
  if (dr == 0 || n_seqs > 65535) return MI_EUNSUPPORTED;
  if (n_rows == 0) return MI_OK;
  hipLaunchKernelGGL(delta_prepare_kernel, dim3(n_rows), dim3(256), 0, S(stream), qkv, ld, q_off, k_off, beta_pre, ld_beta,
                     decay_pre, ld_decay, dt_bias, a_log, H, G, D, workspace);
  if (check_launch() != MI_OK) return MI_ELAUNCH;
  const dim3 grid(n_seqs, H, (Dv + kDeltaCols - 1) / kDeltaCols), block(kDeltaThreads);
#define MI_DELTA(DR)                                                                                                  \
  hipLaunchKernelGGL((channel_delta_kernel<DR>), grid, block, 0, S(stream), qkv, ld, v_off, workspace, state, cu_q,     \
                     kv_lens, slot_ids, H, G, D, Dv, out, ldo)
  if (dr == 16) MI_DELTA(16);
  else if (dr == 32) MI_DELTA(32);
  else MI_DELTA(64);
#undef MI_DELTA
  if (check_launch() != MI_OK) return MI_ELAUNCH;
  hipLaunchKernelGGL(delta_finish_kernel, dim3((n_rows * H + 3) / 4), dim3(256), 0, S(stream), out, ldo, gate_pre,
                     ld_gate, norm_w, n_rows, H, Dv, eps, MI_ACT_SIGMOID, 1.f);
  return check_launch();
}

extern "C" int mi_route_grouped(const float* logits, int64_t ld, const float* correction, int n_tokens, int n_outputs,
                                int top_k, int n_groups, int keep, int score_kind, int group_kind, int32_t* ids,
                                float* weights, mi_stream stream) {
  if (!logits || !correction || !ids || !weights || n_tokens < 0) return MI_EINVAL;
  if ((score_kind != MI_ROUTE_SOFTMAX && score_kind != MI_ROUTE_SIGMOID) ||
      (group_kind != MI_ROUTE_GROUP_MAX && group_kind != MI_ROUTE_GROUP_TOP2))
    return MI_EINVAL;
  if (n_outputs < 1 || n_outputs > 512 || n_groups < 1 || n_outputs % n_groups || keep < 1 || keep > n_groups ||
      top_k < 1 || top_k > keep * (n_outputs / n_groups))
    return MI_EUNSUPPORTED;
  if (n_tokens == 0) return MI_OK;
  hipLaunchKernelGGL(route_grouped_kernel, dim3((n_tokens + 3) / 4), dim3(256), 0, S(stream), logits, ld, correction,
                     n_tokens, n_outputs, top_k, n_groups, keep, score_kind, group_kind, ids, weights);
  return check_launch();
}

extern "C" int mi_moe_combine_f32(const float* y, const float* h, int64_t ldh, const int32_t* ids, const float* weights,
                                  int n_tokens, int top_k, int n_experts, int width, float* out, int64_t ldo,
                                  mi_stream stream) {
  if (!y || !h || !ids || !weights || !out || n_tokens < 0 || top_k < 1 || width < 1) return MI_EINVAL;
  if (n_tokens == 0) return MI_OK;
  hipLaunchKernelGGL(moe_combine_f32_kernel, dim3(n_tokens), dim3(256), 0, S(stream), y, h, ldh, ids, weights, top_k,
                     n_experts, width, out, ldo);
  return check_launch();
}

extern "C" int mi_add_rmsnorm_f32(float* res, int64_t ldr, const float* y, int64_t ldy, float mult, const float* w,
                                  float shift, float eps, float* out, int64_t ldo, int rows, int width, mi_stream stream) {
  return mi_add_vec_rmsnorm_f32(res, ldr, y, ldy, mult, nullptr, w, shift, eps, out, ldo, rows, width, stream);
}

extern "C" int mi_add_vec_rmsnorm_f32(float* res, int64_t ldr, const float* y, int64_t ldy, float mult, const float* vec,
                                      const float* w, float shift, float eps, float* out, int64_t ldo, int rows, int width,
                                      mi_stream stream) {
  if (!res || rows < 0 || width < 1 || ldr < width || (y && ldy < width) || (w && (!out || ldo < width))) return MI_EINVAL;
  if (rows == 0 || (!y && !w && !vec)) return MI_OK;
  hipLaunchKernelGGL(add_rmsnorm_f32_kernel, dim3(rows), dim3(256), 0, S(stream), res, ldr, y, ldy, mult, vec, w, shift,
                     eps, out, ldo, width);
  return check_launch();
}

extern "C" int mi_depth_mix_f32(float* stack, int64_t slot_stride, int n, const float* coef, const float* y, int64_t ldy,
                                float mult, const float* norm_w, float shift, float eps, float* h, int64_t ldh, int rows,
                                int width, mi_stream stream) {
  if (!stack || !coef || n < 1 || rows < 0 || width < 1 || slot_stride < (int64_t)rows * width) return MI_EINVAL;
  if ((y && ldy < width) || (norm_w && (!h || ldh < width))) return MI_EINVAL;
  if (rows == 0) return MI_OK;
  hipLaunchKernelGGL(depth_mix_f32_kernel, dim3(rows), dim3(256), 0, S(stream), stack, slot_stride, n, coef, y, ldy, mult,
                     norm_w, shift, eps, h, ldh, width);
  return check_launch();
}

extern "C" int64_t mi_mingru_scan_workspace_elems(int rows, int n_seqs, int width) {
  if (rows < 0 || n_seqs < 1 || width < 1) return -1;
  return 2 * (int64_t)(rows / kScanSeg + n_seqs) * width;
}

extern "C" int mi_mingru_scan(const float* proj, int64_t ld, int z_off, int x_off, int g_off, float* state,
                              const int32_t* cu_q, const int32_t* kv_lens, const int32_t* slot_ids, int n_seqs, int rows,
                              int max_rows_per_seq, int width, float* workspace, float* out, int64_t ldo,
                              mi_stream stream) {
  if (!proj || !state || !cu_q || !kv_lens || !slot_ids || !out || n_seqs < 1 || rows < 0 || width < 1) return MI_EINVAL;
  if (z_off < 0 || x_off < 0 || g_off < 0 || ld < width || ldo < width || max_rows_per_seq < 1) return MI_EINVAL;
  if (n_seqs > 65535) return MI_EUNSUPPORTED;
  if (rows == 0) return MI_OK;
  const int cb = (width + 255) / 256;
  const int max_segs = rows / kScanSeg + n_seqs;  // (sum over the sequences of ceil(rows_s / seg) is at most this)
  if (max_rows_per_seq <= kScanSeg) {
    hipLaunchKernelGGL((mingru_walk_kernel<false>), dim3(cb, n_seqs), dim3(256), 0, S(stream), proj, ld, z_off, x_off, g_off,
                       (const float*)nullptr, state, cu_q, kv_lens, slot_ids, n_seqs, width, out, ldo);
    return check_launch();
  }
  if (!workspace || max_segs > 65535) return !workspace ? MI_EINVAL : MI_EUNSUPPORTED;
  hipLaunchKernelGGL(mingru_summary_kernel, dim3(cb, max_segs), dim3(256), 0, S(stream), proj, ld, z_off, x_off, cu_q,
                     n_seqs, width, workspace);
  if (check_launch() != MI_OK) return MI_ELAUNCH;
  hipLaunchKernelGGL(mingru_carry_kernel, dim3(cb, n_seqs), dim3(256), 0, S(stream), workspace, state, cu_q, kv_lens,
                     slot_ids, width);
  if (check_launch() != MI_OK) return MI_ELAUNCH;
  hipLaunchKernelGGL((mingru_walk_kernel<true>), dim3(cb, max_segs), dim3(256), 0, S(stream), proj, ld, z_off, x_off, g_off,
                     workspace, state, cu_q, kv_lens, slot_ids, n_seqs, width, out, ldo);
  return check_launch();
}

extern "C" int mi_kv_store_temp(float* proj, int64_t ld, int q_off, int k_off, int v_off, float temp_coef, int temp_every,
                                const int32_t* cu_q, const int32_t* kv_lens, int n_seqs, void* k_cache, void* v_cache,
                                int cache_dtype, const int32_t* slots, int rows, int H, int G, int D, int Dv,
                                int block_size, mi_stream stream) {
  if (!proj || !cu_q || !kv_lens || !k_cache || !v_cache || !slots || rows < 0 || n_seqs < 1) return MI_EINVAL;
  if (H < 1 || G < 1 || D < 1 || Dv < 1 || block_size < 1) return MI_EINVAL;
  if (rows == 0) return MI_OK;
  if (cache_dtype == MI_DTYPE_BF16)
    hipLaunchKernelGGL((kv_store_temp_kernel<uint16_t>), dim3(rows), dim3(256), 0, S(stream), proj, ld, q_off, k_off, v_off,
                       H * D, temp_coef, temp_every, cu_q, kv_lens, n_seqs, static_cast<uint16_t*>(k_cache),
                       static_cast<uint16_t*>(v_cache), slots, G, D, Dv, block_size);
  else if (cache_dtype == MI_DTYPE_F32)
    hipLaunchKernelGGL((kv_store_temp_kernel<float>), dim3(rows), dim3(256), 0, S(stream), proj, ld, q_off, k_off, v_off,
                       H * D, temp_coef, temp_every, cu_q, kv_lens, n_seqs, static_cast<float*>(k_cache),
                       static_cast<float*>(v_cache), slots, G, D, Dv, block_size);
  else return MI_EINVAL;
  return check_launch();
}

extern "C" int mi_latent_prepare(const float* proj, int64_t ld, const float* q, int64_t ldq, int q_off, int c_off, int H,
                                 int D, int R, int C, int rot_dims, const float* inv_freq, const float* norm_w, float eps, const int32_t* cu_q,
                                 const int32_t* kv_lens, int n_seqs, void* cache, int cache_dtype, const int32_t* slots,
                                 float* qx, int64_t ldqx, int rows, mi_stream stream) {
  if (!proj || !q || !norm_w || !cu_q || !kv_lens || !cache || !slots || !qx || rows < 0 || n_seqs < 1) return MI_EINVAL;
  if (H < 1 || D < 0 || R < 0 || C < 1 || rot_dims < 0 || rot_dims > R || rot_dims % 2 || ldqx < (int64_t)H * (C + R))
    return MI_EINVAL;
  if (rot_dims > 0 && !inv_freq) return MI_EINVAL;
  if (rows == 0) return MI_OK;
  if (cache_dtype == MI_DTYPE_BF16)
    hipLaunchKernelGGL((latent_prepare_kernel<uint16_t>), dim3(rows), dim3(256), 0, S(stream), proj, ld, q, ldq, q_off, c_off,
                       H, D, R, C, rot_dims, inv_freq, norm_w, eps, cu_q, kv_lens, n_seqs, static_cast<uint16_t*>(cache), slots,
                       qx, ldqx);
  else if (cache_dtype == MI_DTYPE_F32)
    hipLaunchKernelGGL((latent_prepare_kernel<float>), dim3(rows), dim3(256), 0, S(stream), proj, ld, q, ldq, q_off, c_off, H,
                       D, R, C, rot_dims, inv_freq, norm_w, eps, cu_q, kv_lens, n_seqs, static_cast<float*>(cache), slots, qx,
                       ldqx);
  else return MI_EINVAL;
  return check_launch();
}

extern "C" int mi_route_topk(const float* logits, int64_t ld, int n_tokens, int n_outputs, int top_k, int32_t* ids,
                             float* weights, mi_stream stream) {
  if (!logits || !ids || !weights || n_tokens < 0 || ld < n_outputs) return MI_EINVAL;
  if (n_outputs < 1 || n_outputs > 512 || top_k < 1 || top_k > n_outputs) return MI_EUNSUPPORTED;
  if (n_tokens == 0) return MI_OK;
  hipLaunchKernelGGL(route_topk_kernel, dim3((n_tokens + 3) / 4), dim3(256), 0, S(stream), logits, ld, n_tokens, n_outputs,
                     top_k, ids, weights);
  return check_launch();
}

extern "C" int mi_moe_combine_shared(const float* y, const int32_t* ids, const float* weights, int n_tokens, int top_k,
                                     int width, const float* shared, int64_t ld_shared, const float* shared_gate,
                                     int64_t ld_gate, float* out, int64_t ldo, mi_stream stream) {
  if (!y || !ids || !out || n_tokens < 0 || top_k < 1 || width < 1 || (shared && !shared_gate)) return MI_EINVAL;
  if (n_tokens == 0) return MI_OK;
  hipLaunchKernelGGL(moe_combine_shared_kernel, dim3(n_tokens), dim3(256), 0, S(stream), y, ids, weights, top_k, width,
                     shared, ld_shared, shared_gate, ld_gate, out, ldo);
  return check_launch();
}

extern "C" int mi_gated_norm_add_f32(float* res, int64_t ldr, const float* y, int64_t ldy, const float* gate_pre,
                                     int64_t ldg, const float* w_post, float eps, const float* w_next, float* out,
                                     int64_t ldo, int rows, int width, mi_stream stream) {
  if (!res || !y || !w_post || rows < 0 || width < 1 || (w_next && !out)) return MI_EINVAL;
  if (rows == 0) return MI_OK;
  hipLaunchKernelGGL(gated_norm_add_f32_kernel, dim3(rows), dim3(256), 0, S(stream), res, ldr, y, ldy, gate_pre, ldg,
                     w_post, eps, w_next, out, ldo, width);
  return check_launch();
}

// key channels per lane of linear_attention_kernel: the head's channels padded to 64, 128 or 256 over a column's lanes
static int linear_dr(int D) { return D <= 64 ? 64 / kLinLanes : D <= 128 ? 128 / kLinLanes : D <= 256 ? 256 / kLinLanes : 0; }

extern "C" int64_t mi_linear_attention_state_elems(int H, int D, int Dv) {
  const int dr = linear_dr(D);
  if (!dr) return -1;
  return (int64_t)H * ((Dv + kDeltaCols - 1) / kDeltaCols) * dr * kLinThreads;
}

extern "C" int mi_linear_attention(const float* proj, int64_t ld, int q_off, int k_off, int v_off, int q_act, int k_act,
                                   int v_act, int decay_kind, const float* decay, const float* f_bias, const float* lower,
                                   const float* gate_pre, int64_t ld_gate, const float* norm_w, int norm_groups,
                                   float* state, const int32_t* cu_q, const int32_t* kv_lens, const int32_t* slot_ids,
                                   int n_seqs, int n_rows, int H, int D, int Dv, float eps, float* out, int64_t ldo,
                                   mi_stream stream) {
  if (!proj || !state || !cu_q || !kv_lens || !slot_ids || !out || n_rows < 0 || n_seqs < 1) return MI_EINVAL;
  if (H < 1 || D < 1 || Dv < 1 || ldo < (int64_t)H * Dv) return MI_EINVAL;
  if (decay_kind == MI_DECAY_HEAD ? !decay : decay_kind == MI_DECAY_FORGET ? (!f_bias || !lower) : true) return MI_EINVAL;
  if (norm_w && norm_groups != 1 && norm_groups != H) return MI_EINVAL;
  for (int a : {q_act, k_act, v_act})
    if (a != MI_ACT_NONE && a != MI_ACT_SILU) return MI_EUNSUPPORTED;
  const int dr = linear_dr(D);
  if (!dr || H > 65535) return MI_EUNSUPPORTED;
  if (n_rows == 0) return MI_OK;
  const dim3 grid(n_seqs, H, (Dv + kDeltaCols - 1) / kDeltaCols);
#define MI_LINATTN(DR, KIND)                                                                                          \
  hipLaunchKernelGGL((linear_attention_kernel<DR, KIND>), grid, dim3(kLinThreads), 0, S(stream), proj, ld, q_off,    \
                     k_off, v_off, q_act, k_act, v_act, decay, f_bias, lower, state, cu_q, kv_lens, slot_ids, H, D, Dv, \
                     out, ldo)
  if (decay_kind == MI_DECAY_HEAD) {
    if (dr == 64 / kLinLanes) MI_LINATTN(64 / kLinLanes, MI_DECAY_HEAD);
    else if (dr == 128 / kLinLanes) MI_LINATTN(128 / kLinLanes, MI_DECAY_HEAD);
    else MI_LINATTN(256 / kLinLanes, MI_DECAY_HEAD);
  } else {
    if (dr == 64 / kLinLanes) MI_LINATTN(64 / kLinLanes, MI_DECAY_FORGET);
    else if (dr == 128 / kLinLanes) MI_LINATTN(128 / kLinLanes, MI_DECAY_FORGET);
    else MI_LINATTN(256 / kLinLanes, MI_DECAY_FORGET);
  }
#undef MI_LINATTN
  if (check_launch() != MI_OK) return MI_ELAUNCH;
  if (!norm_w) return MI_OK;
  // the read-out's norm: over each head's value channels (norm_groups == H, weight [Dv]) or over all heads' channels
  // together (norm_groups == 1, weight [H * Dv]); then the sigmoid gate, if any
  if (norm_groups == 1 && H > 1)
    hipLaunchKernelGGL(row_norm_gate_kernel, dim3(n_rows), dim3(256), 0, S(stream), out, ldo, gate_pre, ld_gate, norm_w,
                       H * Dv, eps);
  else
    hipLaunchKernelGGL(delta_finish_kernel, dim3((n_rows * H + 3) / 4), dim3(256), 0, S(stream), out, ldo, gate_pre,
                       ld_gate, norm_w, n_rows, H, Dv, eps, MI_ACT_SIGMOID, 1.f);
  return check_launch();
}

extern "C" int mi_rotary_store(float* proj, int64_t ld, int q_off, int k_off, int v_off, int H, int G, int D, int Gv, int Dv,
                               int rot_dims, int layout, const float* inv_freq, float amp, int unit_norm, float eps,
                               float k_mult, const int32_t* cu_q, const int32_t* kv_lens, int n_seqs, void* k_cache,
                               void* v_cache, int cache_dtype, const int32_t* slots, int rows, int block_size,
                               mi_stream stream) {
  if (!proj || !cu_q || !kv_lens || rows < 0 || n_seqs < 1 || H < 0 || G < 0 || D < 1 || block_size < 1) return MI_EINVAL;
  if (rot_dims < 0 || rot_dims > D || rot_dims % 2 || (rot_dims && !inv_freq)) return MI_EINVAL;
  if (layout != MI_ROT_INTERLEAVED && layout != MI_ROT_HALVES) return MI_EINVAL;
  if ((k_cache || v_cache) && !slots) return MI_EINVAL;
  if (v_cache && (Gv < 1 || Dv < 1)) return MI_EINVAL;
  if (q_off + (int64_t)H * D > ld || k_off + (int64_t)G * D > ld || (v_cache && v_off + (int64_t)Gv * Dv > ld)) return MI_EINVAL;
  const size_t lds = 4 * (size_t)D * sizeof(float);
  if (lds > 48 * 1024) return MI_EUNSUPPORTED;
  if (rows == 0) return MI_OK;
  if (cache_dtype == MI_DTYPE_BF16)
    hipLaunchKernelGGL(rotary_store_kernel<uint16_t>, dim3(rows), dim3(256), lds, S(stream), proj, ld, q_off, k_off, v_off,
                       H, G, D, Gv, Dv, rot_dims, layout, inv_freq, amp, unit_norm, eps, k_mult, cu_q, kv_lens, n_seqs,
                       static_cast<uint16_t*>(k_cache), static_cast<uint16_t*>(v_cache), slots, block_size);
  else if (cache_dtype == MI_DTYPE_F32)
    hipLaunchKernelGGL(rotary_store_kernel<float>, dim3(rows), dim3(256), lds, S(stream), proj, ld, q_off, k_off, v_off, H,
                       G, D, Gv, Dv, rot_dims, layout, inv_freq, amp, unit_norm, eps, k_mult, cu_q, kv_lens, n_seqs,
                       static_cast<float*>(k_cache), static_cast<float*>(v_cache), slots, block_size);
  else
    return MI_EINVAL;
  return check_launch();
}

extern "C" int mi_head_mix(const float* o, int64_t ldo_in, const float* talk, int rows, int H, int G, int Dv, int c0,
                           int n_chunk, float out_scale, float* out, int64_t ldo, mi_stream stream) {
  if (!o || !talk || !out || rows < 0 || H < 1 || G < 1 || H % G || Dv < 1 || c0 < 0 || n_chunk < 1 || c0 + n_chunk > G)
    return MI_EINVAL;
  if (ldo_in < (int64_t)H * n_chunk * Dv || ldo < (int64_t)H * Dv) return MI_EINVAL;
  if (rows == 0) return MI_OK;
  const int64_t n = (int64_t)rows * H * Dv;
  hipLaunchKernelGGL(head_mix_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, S(stream), o, ldo_in, talk, rows, H,
                     G, Dv, c0, n_chunk, out_scale, out, ldo);
  return check_launch();
}

extern "C" int mi_head_norm_gate(float* out, int64_t ldo, const float* gate_pre, int64_t ld_gate, int gate_act,
                                 const float* norm_w, float out_scale, int rows, int H, int Dv, float eps,
                                 mi_stream stream) {
  if (!out || rows < 0 || H < 1 || Dv < 1 || ldo < (int64_t)H * Dv || (gate_pre && ld_gate < (int64_t)H * Dv)) return MI_EINVAL;
  if (gate_act != MI_ACT_SIGMOID && gate_act != MI_ACT_SILU) return MI_EINVAL;
  if (rows == 0) return MI_OK;
  hipLaunchKernelGGL(delta_finish_kernel, dim3((rows * H + 3) / 4), dim3(256), 0, S(stream), out, ldo, gate_pre, ld_gate,
                     norm_w, rows, H, Dv, eps, gate_act, out_scale);
  return check_launch();
}
