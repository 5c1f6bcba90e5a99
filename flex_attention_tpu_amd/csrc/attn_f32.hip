// Flex-attention forward / dq / dk-dv in float32 with genuine fp32 FMAs (no MFMA, no reduced
// precision): the exact-arithmetic path for small fp32 problems, head dim 64 or 128.
//
// All three kernels share one shape: a work-group of 256 lanes owns 64 "owner" rows (q rows for
// forward and dq, kv rows for dk/dv), four lanes per row, each lane holding an interleaved quarter
// of the head dimension in registers.  The other side streams through LDS in 64-row tiles listed
// by the block map; every lane of a wave reads the same streamed row, so LDS reads broadcast.
#include "fa_common.hpp"
#include "launch.hpp"

namespace fa {

namespace f32_cfg {
constexpr int BQ = 64;
constexpr int BK = 64;
constexpr int CH = 8;  // streamed rows handled per softmax update
}  // namespace f32_cfg

template <int NV>
__device__ __forceinline__ float dot_slice(const f32x4 (&a)[NV], const float* row, int sub) {
  float acc = 0.f;
#pragma unroll
  for (int c = 0; c < NV; ++c) {
    const f32x4 b = *reinterpret_cast<const f32x4*>(row + (sub + 4 * c) * 4);
    acc = __builtin_fmaf(a[c][0], b[0], acc);
    acc = __builtin_fmaf(a[c][1], b[1], acc);
    acc = __builtin_fmaf(a[c][2], b[2], acc);
    acc = __builtin_fmaf(a[c][3], b[3], acc);
  }
  return acc;
}

__device__ __forceinline__ float quad_sum(float x) {
  x += __shfl_xor(x, 1);
  x += __shfl_xor(x, 2);
  return x;
}

template <int NV>
__device__ __forceinline__ void axpy_slice(f32x4 (&acc)[NV], float s, const float* row, int sub) {
#pragma unroll
  for (int c = 0; c < NV; ++c) {
    const f32x4 b = *reinterpret_cast<const f32x4*>(row + (sub + 4 * c) * 4);
    acc[c][0] = __builtin_fmaf(s, b[0], acc[c][0]);
    acc[c][1] = __builtin_fmaf(s, b[1], acc[c][1]);
    acc[c][2] = __builtin_fmaf(s, b[2], acc[c][2]);
    acc[c][3] = __builtin_fmaf(s, b[3], acc[c][3]);
  }
}

template <int NV>
__device__ __forceinline__ void load_slice(f32x4 (&dst)[NV], const float* row, int sub) {
#pragma unroll
  for (int c = 0; c < NV; ++c) dst[c] = *reinterpret_cast<const f32x4*>(row + (sub + 4 * c) * 4);
}

template <int NV>
__device__ __forceinline__ void store_slice(float* row, const f32x4 (&src)[NV], int sub, float mul) {
#pragma unroll
  for (int c = 0; c < NV; ++c) {
    f32x4 v = src[c];
    v[0] *= mul; v[1] *= mul; v[2] *= mul; v[3] *= mul;
    *reinterpret_cast<f32x4*>(row + (sub + 4 * c) * 4) = v;
  }
}

// Copies a [rows x D] fp32 tile from global to LDS with all 256 lanes.
template <int D>
__device__ __forceinline__ void copy_tile(float* dst, const float* src, int rows, int tid) {
  const int n4 = rows * D / 4;
  for (int i = tid; i < n4; i += 256)
    reinterpret_cast<f32x4*>(dst)[i] = reinterpret_cast<const f32x4*>(src)[i];
}

__device__ __forceinline__ float lse2_of(float l, float m) {
  return (l > 0.f) ? __builtin_fmaf(m, kLog2e, log2f(l)) : __builtin_huge_valf();
}

// ------------------------------------------------------------------------------------------
// forward
// ------------------------------------------------------------------------------------------
template <int D, int SCORE>
__global__ __launch_bounds__(256) void fwd_f32_kernel(FwdArgs a) {
  using namespace f32_cfg;
  constexpr int NV = D / 16;
  extern __shared__ __attribute__((aligned(16))) char smem_raw[];
  float* sK = reinterpret_cast<float*>(smem_raw);
  float* sV = sK + BK * D;

  const int nQ = a.Sq / BQ, nK = a.map.nk;
  const int wg = blockIdx.x;
  const int bh = wg / nQ, qb = nQ - 1 - (wg % nQ);
  const int b = bh / a.Hq, h = bh % a.Hq, hk = h / (a.Hq / a.Hkv);
  const MaskArgs mk = mask_of_batch(a.mask, b, a.Sq, a.Sk);
  const int tid = threadIdx.x, sub = tid & 3, r = tid >> 2;
  const int q_idx = qb * BQ + r;

  const float* Qg = static_cast<const float*>(a.q) + ((size_t)bh * a.Sq + q_idx) * D;
  const float* Kg = static_cast<const float*>(a.k) + (size_t)(b * a.Hkv + hk) * a.Sk * D;
  const float* Vg = static_cast<const float*>(a.v) + (size_t)(b * a.Hkv + hk) * a.Sk * D;

  ScoreMod<SCORE> sm;
  sm.init(a.score, a.sm_scale, h, b);
  const int doc_i = (mk.flags & FLEXATTN_MASK_DOC) ? mk.doc_q[q_idx] : 0;

  f32x4 qv[NV], acc[NV];
  load_slice<NV>(qv, Qg, sub);
#pragma unroll
  for (int c = 0; c < NV; ++c) acc[c] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m_run = kNegInf, l_run = 0.f;

  const int n_tiles = a.map.cnt[qb];
  const int* tile_idx = a.map.idx + (size_t)qb * nK;
  const uint8_t* tile_state = a.map.state + (size_t)qb * nK;

  for (int t = 0; t < n_tiles; ++t) {
    const int kb = tile_idx[t];
    const bool partial = tile_state[kb] == 1;
    __syncthreads();
    copy_tile<D>(sK, Kg + (size_t)kb * BK * D, BK, tid);
    copy_tile<D>(sV, Vg + (size_t)kb * BK * D, BK, tid);
    __syncthreads();
    for (int j0 = 0; j0 < BK; j0 += CH) {
      float tv[CH];
      float m_new = m_run;
#pragma unroll
      for (int jj = 0; jj < CH; ++jj) {
        const int j = kb * BK + j0 + jj;
        float s = quad_sum(dot_slice<NV>(qv, sK + (j0 + jj) * D, sub));
        float x = sm.to_log2(s, q_idx, j) + sm.bias2(q_idx, j);
        if (partial) {
          const int doc_j = (mk.flags & FLEXATTN_MASK_DOC) ? mk.doc_k[j] : 0;
          if (!keep_elem(mk, q_idx, j, doc_i, doc_j)) x = kNegInf;
        }
        tv[jj] = x;
        m_new = fmaxf(m_new, x);
      }
      const float m_safe = (m_new == kNegInf) ? 0.f : m_new;
      const float alpha = exp2f(m_run - m_safe);
      m_run = m_new;
      l_run *= alpha;
#pragma unroll
      for (int c = 0; c < NV; ++c) {
        acc[c][0] *= alpha; acc[c][1] *= alpha; acc[c][2] *= alpha; acc[c][3] *= alpha;
      }
#pragma unroll
      for (int jj = 0; jj < CH; ++jj) {
        const float p = exp2f(tv[jj] - m_safe);
        l_run += p;
        axpy_slice<NV>(acc, p, sV + (j0 + jj) * D, sub);
      }
    }
  }

  const float inv = (l_run > 0.f) ? 1.0f / l_run : 0.f;
  float* Og = static_cast<float*>(a.o) + ((size_t)bh * a.Sq + q_idx) * D;
  store_slice<NV>(Og, acc, sub, inv);
  if (a.l != nullptr && sub == 0) {
    a.l[(size_t)bh * a.Sq + q_idx] = l_run;
    a.m[(size_t)bh * a.Sq + q_idx] = m_run * kLn2;
  }
}

// ------------------------------------------------------------------------------------------
// dq
// ------------------------------------------------------------------------------------------
template <int D, int SCORE>
__global__ __launch_bounds__(256) void bwd_dq_f32_kernel(BwdArgs a) {
  using namespace f32_cfg;
  constexpr int NV = D / 16;
  extern __shared__ __attribute__((aligned(16))) char smem_raw[];
  float* sK = reinterpret_cast<float*>(smem_raw);
  float* sV = sK + BK * D;

  const int nQ = a.Sq / BQ, nK = a.map.nk;
  const int wg = blockIdx.x;
  const int bh = wg / nQ, qb = nQ - 1 - (wg % nQ);
  const int b = bh / a.Hq, h = bh % a.Hq, hk = h / (a.Hq / a.Hkv);
  const MaskArgs mk = mask_of_batch(a.mask, b, a.Sq, a.Sk);
  const int tid = threadIdx.x, sub = tid & 3, r = tid >> 2;
  const int q_idx = qb * BQ + r;
  const size_t row = (size_t)bh * a.Sq + q_idx;

  const float* Kg = static_cast<const float*>(a.k) + (size_t)(b * a.Hkv + hk) * a.Sk * D;
  const float* Vg = static_cast<const float*>(a.v) + (size_t)(b * a.Hkv + hk) * a.Sk * D;

  ScoreMod<SCORE> sm;
  sm.init(a.score, a.sm_scale, h, b);
  const int doc_i = (mk.flags & FLEXATTN_MASK_DOC) ? mk.doc_q[q_idx] : 0;

  f32x4 qv[NV], dov[NV], acc[NV];
  load_slice<NV>(qv, static_cast<const float*>(a.q) + row * D, sub);
  load_slice<NV>(dov, static_cast<const float*>(a.dout) + row * D, sub);
#pragma unroll
  for (int c = 0; c < NV; ++c) acc[c] = f32x4{0.f, 0.f, 0.f, 0.f};
  const float lse2 = lse2_of(a.l[row], a.m[row]);
  const float dl = a.delta[row];

  const int n_tiles = a.map.cnt[qb];
  const int* tile_idx = a.map.idx + (size_t)qb * nK;
  const uint8_t* tile_state = a.map.state + (size_t)qb * nK;

  for (int t = 0; t < n_tiles; ++t) {
    const int kb = tile_idx[t];
    const bool partial = tile_state[kb] == 1;
    __syncthreads();
    copy_tile<D>(sK, Kg + (size_t)kb * BK * D, BK, tid);
    copy_tile<D>(sV, Vg + (size_t)kb * BK * D, BK, tid);
    __syncthreads();
    for (int jj = 0; jj < BK; ++jj) {
      const int j = kb * BK + jj;
      const float s = quad_sum(dot_slice<NV>(qv, sK + jj * D, sub));
      const float dp = quad_sum(dot_slice<NV>(dov, sV + jj * D, sub));
      const float tv = sm.to_log2(s, q_idx, j);  // (the score function's value: what its derivative is taken from)
      float x = tv + sm.bias2(q_idx, j);
      if (partial) {
        const int doc_j = (mk.flags & FLEXATTN_MASK_DOC) ? mk.doc_k[j] : 0;
        if (!keep_elem(mk, q_idx, j, doc_i, doc_j)) x = kNegInf;
      }
      const float p = exp2f(x - lse2);
      const float gl = (x == kNegInf) ? 0.f : p * (dp - dl);   // gradient with respect to the logit (the bias's share)
      if (a.dab != nullptr && sub == 0) a.dab[row * (size_t)a.Sk + j] = gl;
      const float ds = (x == kNegInf) ? 0.f : gl * sm.dfactor(tv, s, q_idx, j);
      axpy_slice<NV>(acc, ds, sK + jj * D, sub);
    }
  }
  store_slice<NV>(static_cast<float*>(a.dq) + row * D, acc, sub, 1.0f);
}

// ------------------------------------------------------------------------------------------
// dk / dv
// ------------------------------------------------------------------------------------------
template <int D, int SCORE>
__global__ __launch_bounds__(256) void bwd_dkv_f32_kernel(BwdArgs a) {
  using namespace f32_cfg;
  constexpr int NV = D / 16;
  extern __shared__ __attribute__((aligned(16))) char smem_raw[];
  float* sQ = reinterpret_cast<float*>(smem_raw);
  float* sDO = sQ + BQ * D;
  float* sLse = sDO + BQ * D;
  float* sDl = sLse + BQ;

  const int nKb = a.Sk / BK, nQ = a.map.nq;
  const int wg = blockIdx.x;
  const int bhk = wg / nKb, kb = wg % nKb;
  const int b = bhk / a.Hkv, hk = bhk % a.Hkv;
  const MaskArgs mk = mask_of_batch(a.mask, b, a.Sq, a.Sk);
  const int group = a.Hq / a.Hkv;
  const int tid = threadIdx.x, sub = tid & 3, r = tid >> 2;
  const int k_idx = kb * BK + r;
  const size_t krow = (size_t)bhk * a.Sk + k_idx;

  f32x4 kv[NV], vv[NV], dk_acc[NV], dv_acc[NV];
  load_slice<NV>(kv, static_cast<const float*>(a.k) + krow * D, sub);
  load_slice<NV>(vv, static_cast<const float*>(a.v) + krow * D, sub);
#pragma unroll
  for (int c = 0; c < NV; ++c) {
    dk_acc[c] = f32x4{0.f, 0.f, 0.f, 0.f};
    dv_acc[c] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  const int doc_j = (mk.flags & FLEXATTN_MASK_DOC) ? mk.doc_k[k_idx] : 0;

  const int n_tiles = a.map.cnt[kb];
  const int* tile_idx = a.map.idx + (size_t)kb * nQ;

  for (int g = 0; g < group; ++g) {
    const int h = hk * group + g;
    const size_t qbase = (size_t)(b * a.Hq + h) * a.Sq;
    ScoreMod<SCORE> sm;
    sm.init(a.score, a.sm_scale, h, b);
    for (int t = 0; t < n_tiles; ++t) {
      const int qb = tile_idx[t];
      const bool partial = a.map.state[(size_t)qb * a.map.nk + kb] == 1;
      __syncthreads();
      copy_tile<D>(sQ, static_cast<const float*>(a.q) + (qbase + (size_t)qb * BQ) * D, BQ, tid);
      copy_tile<D>(sDO, static_cast<const float*>(a.dout) + (qbase + (size_t)qb * BQ) * D, BQ, tid);
      if (tid < BQ) {
        const size_t rr = qbase + (size_t)qb * BQ + tid;
        sLse[tid] = lse2_of(a.l[rr], a.m[rr]);
        sDl[tid] = a.delta[rr];
      }
      __syncthreads();
      // The tile's 64 terms are summed on their own and then added to the running totals: the
      // rounding error of a long sum (thousands of q rows times the group's heads) then grows with
      // the number of tiles, not of rows.
      f32x4 dk_t[NV], dv_t[NV];
#pragma unroll
      for (int c = 0; c < NV; ++c) {
        dk_t[c] = f32x4{0.f, 0.f, 0.f, 0.f};
        dv_t[c] = f32x4{0.f, 0.f, 0.f, 0.f};
      }
      for (int ii = 0; ii < BQ; ++ii) {
        const int i = qb * BQ + ii;
        const float s = quad_sum(dot_slice<NV>(kv, sQ + ii * D, sub));
        const float dp = quad_sum(dot_slice<NV>(vv, sDO + ii * D, sub));
        const float tv = sm.to_log2(s, i, k_idx);
        float x = tv + sm.bias2(i, k_idx);
        if (partial) {
          const int doc_i = (mk.flags & FLEXATTN_MASK_DOC) ? mk.doc_q[i] : 0;
          if (!keep_elem(mk, i, k_idx, doc_i, doc_j)) x = kNegInf;
        }
        const float p = exp2f(x - sLse[ii]);
        const float ds = (x == kNegInf) ? 0.f : p * (dp - sDl[ii]) * sm.dfactor(tv, s, i, k_idx);
        axpy_slice<NV>(dv_t, p, sDO + ii * D, sub);
        axpy_slice<NV>(dk_t, ds, sQ + ii * D, sub);
      }
#pragma unroll
      for (int c = 0; c < NV; ++c) {
        dk_acc[c] += dk_t[c];
        dv_acc[c] += dv_t[c];
      }
    }
  }
  store_slice<NV>(static_cast<float*>(a.dk) + krow * D, dk_acc, sub, 1.0f);
  store_slice<NV>(static_cast<float*>(a.dv) + krow * D, dv_acc, sub, 1.0f);
}

// ------------------------------------------------------------------------------------------
// launch
// ------------------------------------------------------------------------------------------
template <typename Kern, typename Args>
static int launch_with_lds(Kern kern, int grid, int lds, const Args& a, hipStream_t stream, const char* what) {
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, lds);
  if (e != hipSuccess) return set_error(FLEXATTN_ELAUNCH, "hipFuncSetAttribute(%s): %s", what, hipGetErrorString(e));
  hipLaunchKernelGGL(kern, dim3(grid), dim3(256), lds, stream, a);
  return check_launch(what);
}

#define FA_F32_DISPATCH(KERNEL, GRID, LDS, ARGS, WHAT)                                               \
  switch ((ARGS).score.kind) {                                                                        \
    case FLEXATTN_SCORE_NONE:                                                                         \
      return launch_with_lds(KERNEL<DD, FLEXATTN_SCORE_NONE>, GRID, LDS, ARGS, stream, WHAT);         \
    case FLEXATTN_SCORE_ALIBI:                                                                        \
      return launch_with_lds(KERNEL<DD, FLEXATTN_SCORE_ALIBI>, GRID, LDS, ARGS, stream, WHAT);        \
    case FLEXATTN_SCORE_SOFTCAP:                                                                      \
      return launch_with_lds(KERNEL<DD, FLEXATTN_SCORE_SOFTCAP>, GRID, LDS, ARGS, stream, WHAT);      \
    case FLEXATTN_SCORE_ALIBI_TILE:                                                                   \
      return launch_with_lds(KERNEL<DD, FLEXATTN_SCORE_ALIBI_TILE>, GRID, LDS, ARGS, stream, WHAT);   \
    case FLEXATTN_SCORE_CUSTOM:                                                                       \
      return launch_with_lds(KERNEL<DD, FLEXATTN_SCORE_CUSTOM>, GRID, LDS, ARGS, stream, WHAT);       \
  }                                                                                                   \
  return set_error(FLEXATTN_EINVAL, "unknown score kind %d", (ARGS).score.kind);

template <int DD>
static int fwd_f32_d(const FwdArgs& a, hipStream_t stream) {
  const int grid = a.B * a.Hq * (a.Sq / f32_cfg::BQ);
  const int lds = 2 * f32_cfg::BK * DD * 4;
  FA_F32_DISPATCH(fwd_f32_kernel, grid, lds, a, "flexattn_fwd f32")
}
template <int DD>
static int bwd_dq_f32_d(const BwdArgs& a, hipStream_t stream) {
  const int grid = a.B * a.Hq * (a.Sq / f32_cfg::BQ);
  const int lds = 2 * f32_cfg::BK * DD * 4;
  FA_F32_DISPATCH(bwd_dq_f32_kernel, grid, lds, a, "flexattn_bwd_dq f32")
}
template <int DD>
static int bwd_dkv_f32_d(const BwdArgs& a, hipStream_t stream) {
  const int grid = a.B * a.Hkv * (a.Sk / f32_cfg::BK);
  const int lds = 2 * f32_cfg::BQ * DD * 4 + 2 * f32_cfg::BQ * 4;
  FA_F32_DISPATCH(bwd_dkv_f32_kernel, grid, lds, a, "flexattn_bwd_dkv f32")
}

int fwd_f32(const FwdArgs& a, int D, hipStream_t stream) {
  if (D == 64) return fwd_f32_d<64>(a, stream);
  if (D == 128) return fwd_f32_d<128>(a, stream);
  return set_error(FLEXATTN_ENOTSUP, "fp32 forward: head dim %d not in {64, 128}", D);
}
int bwd_dq_f32(const BwdArgs& a, int D, hipStream_t stream) {
  if (D == 64) return bwd_dq_f32_d<64>(a, stream);
  if (D == 128) return bwd_dq_f32_d<128>(a, stream);
  return set_error(FLEXATTN_ENOTSUP, "fp32 dq: head dim %d not in {64, 128}", D);
}
int bwd_dkv_f32(const BwdArgs& a, int D, hipStream_t stream) {
  if (D == 64) return bwd_dkv_f32_d<64>(a, stream);
  if (D == 128) return bwd_dkv_f32_d<128>(a, stream);
  return set_error(FLEXATTN_ENOTSUP, "fp32 dk/dv: head dim %d not in {64, 128}", D);
}
void f32_tile(int* bq, int* bk) {
  *bq = f32_cfg::BQ;
  *bk = f32_cfg::BK;
}

}  // namespace fa
