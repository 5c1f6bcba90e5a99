// Flex-attention forward / dq / dk-dv in float32 on the fp32 matrix cores (v_mfma_f32_32x32x2_f32:
// genuine fp32 products and fp32 accumulation, 64 cycles per 32 x 32 x 2 block), head dim 64 or 128.
// The small fp32 problems this path serves (configuration 1: 2 MB of operands, 0.27 GFLOP) are bound by
// how long the longest chain of dependent work is, not by bandwidth: a work-group owns 32 "owner" rows
// (q rows for forward and dq, kv rows for dk/dv), and its NW waves split the streamed side between them in
// units of 32 rows (wave w takes units w, w + NW, ... of the owner tile's list in the block map) and merge
// their partial results through LDS at the end.  NW = 4 (one wave per SIMD) in general; head dim 64 on a grid
// that leaves CUs idle takes NW = 8: the two waves of a SIMD hide each other's operand loads, which nothing
// prefetches (208 registers per lane at head dim 64 allow two waves; head dim 128 needs 304).  Operands go from global memory (L2-resident at these sizes) straight
// into MFMA operand registers: no LDS staging, no barriers in the main loop.
//
// MFMA operand layout (32x32x2 fp32): lane L supplies A[L % 32][L / 32] and B[L / 32][L % 32] (one float
// each) and holds C[8 (i / 4) + 4 (L / 32) + i % 4][L % 32] in accumulator element i.  A contraction over
// the head dimension takes D / 2 MFMAs; MFMA 4 g + j contracts d = 8 g + j (lanes 0-31) and d = 8 g + 4 + j
// (lanes 32-63), so that a lane's operands for four consecutive MFMAs are one 16-byte load.
#include "fa_common.hpp"
#include "launch.hpp"

namespace fa {

namespace f32m {
constexpr int BO = 32;   // owner rows per work-group
constexpr int BT = 64;   // granularity of the block map on both sides (f32_tile)
}  // namespace f32m

__device__ __forceinline__ f32x16 mfma_f32(float a, float b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
}

// The lane's D / 2 operand values of row `row` (D floats): f32x4 number g holds d = 8 g + 4 half + {0..3}.
template <int D>
__device__ __forceinline__ void load_operand_row(f32x4 (&dst)[D / 8], const float* row, int half) {
#pragma unroll
  for (int g = 0; g < D / 8; ++g) dst[g] = *reinterpret_cast<const f32x4*>(row + 8 * g + 4 * half);
}

// C[32 x 32] = A B^T over the head dimension, A's rows from `a_row` (global), B's rows in registers.
template <int D>
__device__ __forceinline__ f32x16 dot_block(const float* a_row, const f32x4 (&b)[D / 8], int half) {
  f32x4 a[D / 8];
  load_operand_row<D>(a, a_row, half);
  f32x16 c;
#pragma unroll
  for (int e = 0; e < 16; ++e) c[e] = 0.f;
#pragma unroll
  for (int g = 0; g < D / 8; ++g) {
#pragma unroll
    for (int j = 0; j < 4; ++j) c = mfma_f32(a[g][j], b[g][j], c);
  }
  return c;
}

// acc[db] (32 d x 32 columns, db < D / 32) += X^T w, X = 32 rows of D floats from `x_rows` (row stride D),
// w = the lane's 16 weights of those rows (element i: row acc_row(i, half), this lane's column).
template <int D>
__device__ __forceinline__ void accumulate_rows(f32x16 (&acc)[D / 32], const float* x_rows, const float (&w)[16], int l32, int half) {
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const float* r = x_rows + (size_t)acc_row(i, half) * D + l32;
#pragma unroll
    for (int db = 0; db < D / 32; ++db) acc[db] = mfma_f32(r[32 * db], w[i], acc[db]);
  }
}

// ------------------------------------------------------------------------------------------
// forward: lane = q column of S^T = K Q^T; O^T accumulates V^T P^T
// ------------------------------------------------------------------------------------------
template <int D, int SCORE, int NW>
__global__ __launch_bounds__(64 * NW) void fwd_f32_mfma_kernel(FwdArgs a) {
  using namespace f32m;
  constexpr int ND = D / 32;
  extern __shared__ __attribute__((aligned(16))) char smem_raw[];
  float (*sO)[BO][D + 1] = reinterpret_cast<float (*)[BO][D + 1]>(smem_raw);   // [wave][row][d]
  float (*sM)[BO] = reinterpret_cast<float (*)[BO]>(smem_raw + sizeof(float) * NW * BO * (D + 1));
  float (*sL)[BO] = sM + NW;

  const int nO = a.Sq / BO, nK = a.map.nk;
  const int wg = blockIdx.x;
  const int bh = wg / nO, ob = nO - 1 - (wg % nO);
  const int qb = ob / (BT / BO);
  const int b = bh / a.Hq, h = bh % a.Hq, hk = h / (a.Hq / a.Hkv);
  const MaskArgs mk = mask_of_batch(a.mask, b, a.Sq, a.Sk);
  const int tid = threadIdx.x, w = tid >> 6, lane = tid & 63, l32 = lane & 31, half = lane >> 5;
  const int q_idx = ob * BO + l32;

  const float* Qg = static_cast<const float*>(a.q) + ((size_t)bh * a.Sq + q_idx) * D;
  const float* Kg = static_cast<const float*>(a.k) + (size_t)(b * a.Hkv + hk) * a.Sk * D;
  const float* Vg = static_cast<const float*>(a.v) + (size_t)(b * a.Hkv + hk) * a.Sk * D;

  ScoreMod<SCORE> sm;
  sm.init(a.score, a.sm_scale, h, b);
  const bool has_doc = (mk.flags & FLEXATTN_MASK_DOC) != 0;
  const int doc_i = has_doc ? mk.doc_q[q_idx] : 0;

  f32x4 qf[D / 8];
  load_operand_row<D>(qf, Qg, half);
  f32x16 acc[ND];
#pragma unroll
  for (int db = 0; db < ND; ++db)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[db][e] = 0.f;
  float m_run = kNegInf, l_run = 0.f;  // (m: the row's maximum over this wave's keys; l: the lane's half of the sum)

  const int n_tiles = a.map.cnt[qb];
  const int* tile_idx = a.map.idx + (size_t)qb * nK;
  const uint8_t* tile_state = a.map.state + (size_t)qb * nK;

  static_assert(BT == 64, "a list entry is two units of 32 rows");
  for (int u = w; u < 2 * n_tiles; u += NW) {
    const int kb = tile_idx[u >> 1];
    const bool partial = tile_state[kb] == 1;
    {
      const int j0 = kb * BT + 32 * (u & 1);
      const f32x16 s = dot_block<D>(Kg + (size_t)(j0 + l32) * D, qf, half);
      float x[16];
      float m_blk = kNegInf;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int j = j0 + acc_row(i, half);
        float v = sm.to_log2(s[i], q_idx, j) + sm.bias2(q_idx, j);
        if (partial) {
          const int doc_j = has_doc ? mk.doc_k[j] : 0;
          if (!keep_elem(mk, q_idx, j, doc_i, doc_j)) v = kNegInf;
        }
        x[i] = v;
        m_blk = fmaxf(m_blk, v);
      }
      m_blk = half_max(m_blk);
      const float m_new = fmaxf(m_run, m_blk);
      const float m_safe = (m_new == kNegInf) ? 0.f : m_new;
      const float alpha = exp2f(m_run - m_safe);
      m_run = m_new;
      l_run *= alpha;
#pragma unroll
      for (int db = 0; db < ND; ++db)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[db][e] *= alpha;
      float p[16];
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        p[i] = exp2f(x[i] - m_safe);
        l_run += p[i];
      }
      accumulate_rows<D>(acc, Vg + (size_t)j0 * D, p, l32, half);
    }
  }

  // ---- the waves' partial results (each relative to its own maximum) into one ----
  const float l_wave = half_sum(l_run);
  if (half == 0) {
    sM[w][l32] = m_run;
    sL[w][l32] = l_wave;
  }
#pragma unroll
  for (int db = 0; db < ND; ++db)
#pragma unroll
    for (int i = 0; i < 16; ++i) sO[w][l32][32 * db + acc_row(i, half)] = acc[db][i];
  __syncthreads();
  constexpr int TPR = 2 * NW, CPT = D / TPR;   // threads per owner row, columns per thread
  const int r = tid / TPR, c0 = (tid % TPR) * CPT;
  float m_all = kNegInf;
#pragma unroll
  for (int ww = 0; ww < NW; ++ww) m_all = fmaxf(m_all, sM[ww][r]);
  const float m_safe = (m_all == kNegInf) ? 0.f : m_all;
  float f[NW], l_all = 0.f;
#pragma unroll
  for (int ww = 0; ww < NW; ++ww) {
    f[ww] = exp2f(sM[ww][r] - m_safe);   // (0 for a wave that kept nothing)
    l_all += sL[ww][r] * f[ww];
  }
  const float inv = (l_all > 0.f) ? 1.0f / l_all : 0.f;
  float* Og = static_cast<float*>(a.o) + ((size_t)bh * a.Sq + ob * BO + r) * D + c0;
#pragma unroll
  for (int c = 0; c < CPT; ++c) {
    float o = 0.f;
#pragma unroll
    for (int ww = 0; ww < NW; ++ww) o = __builtin_fmaf(sO[ww][r][c0 + c], f[ww], o);
    Og[c] = o * inv;
  }
  if (a.l != nullptr && (tid % TPR) == 0) {
    a.l[(size_t)bh * a.Sq + ob * BO + r] = l_all;
    a.m[(size_t)bh * a.Sq + ob * BO + r] = m_all * kLn2;
  }
}

// Sum of the waves' accumulators (each [ND][16] in MFMA layout: column = the lane's owner row) through
// LDS, written out as rows of D floats: 2 NW threads per row, D / (2 NW) consecutive columns each.
template <int D, int NW>
__device__ __forceinline__ void merge_and_store(const f32x16 (&acc)[D / 32], float (*stage)[f32m::BO][D + 1], float* out_rows,
                                                float mul, int tid) {
  const int w = tid >> 6, l32 = tid & 31, half = (tid >> 5) & 1;
#pragma unroll
  for (int db = 0; db < D / 32; ++db)
#pragma unroll
    for (int i = 0; i < 16; ++i) stage[w][l32][32 * db + acc_row(i, half)] = acc[db][i];
  __syncthreads();
  constexpr int TPR = 2 * NW, CPT = D / TPR;
  const int r = tid / TPR, c0 = (tid % TPR) * CPT;
#pragma unroll
  for (int c = 0; c < CPT; ++c) {
    float x = 0.f;
#pragma unroll
    for (int ww = 0; ww < NW; ++ww) x += stage[ww][r][c0 + c];
    out_rows[(size_t)r * D + c0 + c] = x * mul;
  }
}

__device__ __forceinline__ float lse2_from(float l, float m) {
  return (l > 0.f) ? __builtin_fmaf(m, kLog2e, log2f(l)) : __builtin_huge_valf();
}

// ------------------------------------------------------------------------------------------
// dq: lane = q column; S^T = K Q^T, dP^T = V dO^T, dq^T += K^T dS^T
// ------------------------------------------------------------------------------------------
template <int D, int SCORE, int NW>
__global__ __launch_bounds__(64 * NW) void bwd_dq_f32_mfma_kernel(BwdArgs a) {
  using namespace f32m;
  constexpr int ND = D / 32;
  extern __shared__ __attribute__((aligned(16))) char smem_raw[];
  float (*sA)[BO][D + 1] = reinterpret_cast<float (*)[BO][D + 1]>(smem_raw);

  const int nO = a.Sq / BO, nK = a.map.nk;
  const int wg = blockIdx.x;
  const int bh = wg / nO, ob = nO - 1 - (wg % nO);
  const int qb = ob / (BT / BO);
  const int b = bh / a.Hq, h = bh % a.Hq, hk = h / (a.Hq / a.Hkv);
  const MaskArgs mk = mask_of_batch(a.mask, b, a.Sq, a.Sk);
  const int tid = threadIdx.x, w = tid >> 6, lane = tid & 63, l32 = lane & 31, half = lane >> 5;
  const int q_idx = ob * BO + l32;
  const size_t row = (size_t)bh * a.Sq + q_idx;

  const float* Kg = static_cast<const float*>(a.k) + (size_t)(b * a.Hkv + hk) * a.Sk * D;
  const float* Vg = static_cast<const float*>(a.v) + (size_t)(b * a.Hkv + hk) * a.Sk * D;

  ScoreMod<SCORE> sm;
  sm.init(a.score, a.sm_scale, h, b);
  const bool has_doc = (mk.flags & FLEXATTN_MASK_DOC) != 0;
  const int doc_i = has_doc ? mk.doc_q[q_idx] : 0;

  f32x4 qf[D / 8], dof[D / 8];
  load_operand_row<D>(qf, static_cast<const float*>(a.q) + row * D, half);
  load_operand_row<D>(dof, static_cast<const float*>(a.dout) + row * D, half);
  const float lse2 = lse2_from(a.l[row], a.m[row]);
  const float dl = a.delta[row];
  f32x16 acc[ND];
#pragma unroll
  for (int db = 0; db < ND; ++db)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[db][e] = 0.f;

  const int n_tiles = a.map.cnt[qb];
  const int* tile_idx = a.map.idx + (size_t)qb * nK;
  const uint8_t* tile_state = a.map.state + (size_t)qb * nK;
  for (int u = w; u < 2 * n_tiles; u += NW) {
    const int kb = tile_idx[u >> 1];
    const bool partial = tile_state[kb] == 1;
    {
      const int j0 = kb * BT + 32 * (u & 1);
      const f32x16 s = dot_block<D>(Kg + (size_t)(j0 + l32) * D, qf, half);
      const f32x16 dp = dot_block<D>(Vg + (size_t)(j0 + l32) * D, dof, half);
      float ds[16];
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int j = j0 + acc_row(i, half);
        const float tv = sm.to_log2(s[i], q_idx, j);   // (the score function's value: what its derivative is taken from)
        float x = tv + sm.bias2(q_idx, j);
        if (partial) {
          const int doc_j = has_doc ? mk.doc_k[j] : 0;
          if (!keep_elem(mk, q_idx, j, doc_i, doc_j)) x = kNegInf;
        }
        const float pe = exp2f(x - lse2);
        const float gl = (x == kNegInf) ? 0.f : pe * (dp[i] - dl);   // gradient with respect to the logit (the bias's share)
        if (a.dab != nullptr) a.dab[row * (size_t)a.Sk + j] = gl;
        ds[i] = (x == kNegInf) ? 0.f : gl * sm.dfactor(tv, s[i], q_idx, j);
      }
      accumulate_rows<D>(acc, Kg + (size_t)j0 * D, ds, l32, half);
    }
  }
  merge_and_store<D, NW>(acc, sA, static_cast<float*>(a.dq) + ((size_t)bh * a.Sq + ob * BO) * D, 1.0f, tid);
}

// ------------------------------------------------------------------------------------------
// dk/dv: lane = kv column; S = Q K^T, dP = dO V^T, dv^T += dO^T P, dk^T += Q^T dS, over the q tiles of the
// kv block's list and the q heads of its kv head
// ------------------------------------------------------------------------------------------
template <int D, int SCORE, int NW>
__global__ __launch_bounds__(64 * NW) void bwd_dkv_f32_mfma_kernel(BwdArgs a) {
  using namespace f32m;
  constexpr int ND = D / 32;
  extern __shared__ __attribute__((aligned(16))) char smem_raw[];
  float (*sA)[BO][D + 1] = reinterpret_cast<float (*)[BO][D + 1]>(smem_raw);   // (dk, then dv)

  const int nO = a.Sk / BO, nQ = a.map.nq;
  const int wg = blockIdx.x;
  const int bhk = wg / nO, ob = wg % nO;
  const int kb = ob / (BT / BO);
  const int b = bhk / a.Hkv, hk = bhk % a.Hkv, group = a.Hq / a.Hkv;
  const MaskArgs mk = mask_of_batch(a.mask, b, a.Sq, a.Sk);
  const int tid = threadIdx.x, w = tid >> 6, lane = tid & 63, l32 = lane & 31, half = lane >> 5;
  const int k_idx = ob * BO + l32;
  const size_t krow = (size_t)bhk * a.Sk + k_idx;

  const bool has_doc = (mk.flags & FLEXATTN_MASK_DOC) != 0;
  const int doc_j = has_doc ? mk.doc_k[k_idx] : 0;
  f32x4 kf[D / 8], vf[D / 8];
  load_operand_row<D>(kf, static_cast<const float*>(a.k) + krow * D, half);
  load_operand_row<D>(vf, static_cast<const float*>(a.v) + krow * D, half);
  f32x16 dk_acc[ND], dv_acc[ND];
#pragma unroll
  for (int db = 0; db < ND; ++db)
#pragma unroll
    for (int e = 0; e < 16; ++e) dk_acc[db][e] = dv_acc[db][e] = 0.f;

  const int n_tiles = a.map.cnt[kb];
  const int* tile_idx = a.map.idx + (size_t)kb * nQ;
  const uint8_t* state = a.map.state;
  for (int u = w; u < 2 * group * n_tiles; u += NW) {
    const int it = u >> 1;
    const int g = it / n_tiles, qb = tile_idx[it - g * n_tiles];
    const int h = hk * group + g;
    const size_t head_row = (size_t)(b * a.Hq + h) * a.Sq;
    const float* Qg = static_cast<const float*>(a.q) + head_row * D;
    const float* dOg = static_cast<const float*>(a.dout) + head_row * D;
    ScoreMod<SCORE> sm;
    sm.init(a.score, a.sm_scale, h, b);
    const bool partial = state[(size_t)qb * a.map.nk + kb] == 1;
    {
      const int i0 = qb * BT + 32 * (u & 1);
      const f32x16 s = dot_block<D>(Qg + (size_t)(i0 + l32) * D, kf, half);
      const f32x16 dp = dot_block<D>(dOg + (size_t)(i0 + l32) * D, vf, half);
      float pv[16], ds[16];
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int i = i0 + acc_row(e, half);
        const float tv = sm.to_log2(s[e], i, k_idx);
        float x = tv + sm.bias2(i, k_idx);
        if (partial) {
          const int doc_i = has_doc ? mk.doc_q[i] : 0;
          if (!keep_elem(mk, i, k_idx, doc_i, doc_j)) x = kNegInf;
        }
        const float pe = exp2f(x - lse2_from(a.l[head_row + i], a.m[head_row + i]));
        pv[e] = pe;
        ds[e] = (x == kNegInf) ? 0.f : pe * (dp[e] - a.delta[head_row + i]) * sm.dfactor(tv, s[e], i, k_idx);
      }
      accumulate_rows<D>(dv_acc, dOg + (size_t)i0 * D, pv, l32, half);
      accumulate_rows<D>(dk_acc, Qg + (size_t)i0 * D, ds, l32, half);
    }
  }
  merge_and_store<D, NW>(dk_acc, sA, static_cast<float*>(a.dk) + ((size_t)bhk * a.Sk + ob * BO) * D, 1.0f, tid);
  __syncthreads();  // (the stage is read by other threads than wrote it: all of dk is out before dv goes in)
  merge_and_store<D, NW>(dv_acc, sA, static_cast<float*>(a.dv) + ((size_t)bhk * a.Sk + ob * BO) * D, 1.0f, tid);
}

template <typename Kern, typename Args>
static int launch_mfma(Kern kern, int grid, int waves, int lds, const Args& a, hipStream_t stream, const char* what) {
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, lds);
  if (e != hipSuccess) return set_error(FLEXATTN_ELAUNCH, "hipFuncSetAttribute(%s): %s", what, hipGetErrorString(e));
  hipLaunchKernelGGL(kern, dim3(grid), dim3(64 * waves), lds, stream, a);
  return check_launch(what);
}

#define FA_F32M_DISPATCH(KERNEL, GRID, LDS, ARGS, WHAT)                                                                            \
  switch ((ARGS).score.kind) {                                                                                                \
    case FLEXATTN_SCORE_NONE: return launch_mfma(KERNEL<DD, FLEXATTN_SCORE_NONE, NWW>, GRID, NWW, LDS, ARGS, stream, WHAT);             \
    case FLEXATTN_SCORE_ALIBI: return launch_mfma(KERNEL<DD, FLEXATTN_SCORE_ALIBI, NWW>, GRID, NWW, LDS, ARGS, stream, WHAT);           \
    case FLEXATTN_SCORE_SOFTCAP: return launch_mfma(KERNEL<DD, FLEXATTN_SCORE_SOFTCAP, NWW>, GRID, NWW, LDS, ARGS, stream, WHAT);       \
    case FLEXATTN_SCORE_ALIBI_TILE: return launch_mfma(KERNEL<DD, FLEXATTN_SCORE_ALIBI_TILE, NWW>, GRID, NWW, LDS, ARGS, stream, WHAT); \
    case FLEXATTN_SCORE_CUSTOM: return launch_mfma(KERNEL<DD, FLEXATTN_SCORE_CUSTOM, NWW>, GRID, NWW, LDS, ARGS, stream, WHAT);         \
  }                                                                                                                           \
  return set_error(FLEXATTN_EINVAL, "unknown score kind %d", (ARGS).score.kind);

// Eight waves per work-group where two fit a SIMD (head dim 64) and the grid is small enough to leave CUs idle
// (at most two work-groups per CU): the extra waves then cost nothing and hide the operand loads.
static bool wide_groups(int D, int grid) { return D == 64 && grid <= 512; }

template <int DD, int NWW>
static int fwd_f32_mfma_d(const FwdArgs& a, hipStream_t stream) {
  const int grid = a.B * a.Hq * (a.Sq / f32m::BO);
  const int lds = 4 * (NWW * f32m::BO * (DD + 1) + 2 * NWW * f32m::BO);
  FA_F32M_DISPATCH(fwd_f32_mfma_kernel, grid, lds, a, "flexattn_fwd f32")
}

template <int DD, int NWW>
static int bwd_dq_f32_mfma_d(const BwdArgs& a, hipStream_t stream) {
  const int grid = a.B * a.Hq * (a.Sq / f32m::BO);
  const int lds = 4 * NWW * f32m::BO * (DD + 1);
  FA_F32M_DISPATCH(bwd_dq_f32_mfma_kernel, grid, lds, a, "flexattn_bwd_dq f32")
}
template <int DD, int NWW>
static int bwd_dkv_f32_mfma_d(const BwdArgs& a, hipStream_t stream) {
  const int grid = a.B * a.Hkv * (a.Sk / f32m::BO);
  const int lds = 4 * NWW * f32m::BO * (DD + 1);
  FA_F32M_DISPATCH(bwd_dkv_f32_mfma_kernel, grid, lds, a, "flexattn_bwd_dkv f32")
}

int bwd_dq_f32_mfma(const BwdArgs& a, int D, hipStream_t stream) {
  if (D == 64)
    return wide_groups(D, a.B * a.Hq * (a.Sq / f32m::BO)) ? bwd_dq_f32_mfma_d<64, 8>(a, stream) : bwd_dq_f32_mfma_d<64, 4>(a, stream);
  if (D == 128) return bwd_dq_f32_mfma_d<128, 4>(a, stream);
  return set_error(FLEXATTN_ENOTSUP, "fp32 dq: head dim %d not in {64, 128}", D);
}
int bwd_dkv_f32_mfma(const BwdArgs& a, int D, hipStream_t stream) {
  if (D == 64)
    return wide_groups(D, a.B * a.Hkv * (a.Sk / f32m::BO)) ? bwd_dkv_f32_mfma_d<64, 8>(a, stream)
                                                          : bwd_dkv_f32_mfma_d<64, 4>(a, stream);
  if (D == 128) return bwd_dkv_f32_mfma_d<128, 4>(a, stream);
  return set_error(FLEXATTN_ENOTSUP, "fp32 dk/dv: head dim %d not in {64, 128}", D);
}

int fwd_f32_mfma(const FwdArgs& a, int D, hipStream_t stream) {
  if (D == 64)
    return wide_groups(D, a.B * a.Hq * (a.Sq / f32m::BO)) ? fwd_f32_mfma_d<64, 8>(a, stream) : fwd_f32_mfma_d<64, 4>(a, stream);
  if (D == 128) return fwd_f32_mfma_d<128, 4>(a, stream);
  return set_error(FLEXATTN_ENOTSUP, "fp32 forward: head dim %d not in {64, 128}", D);
}

}  // namespace fa
