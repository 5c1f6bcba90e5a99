// Flex-attention forward, bf16, head dim 128, gfx950.
//
// One work-group = 4 waves = one 128-row Q tile of one (batch, head); each wave owns 32 q rows.
// The kernel works on S^T = K Q^T so that one lane holds one q row's scores: softmax statistics
// stay lane-private apart from one exchange between the two 32-lane halves.  K/V tiles of 64 rows
// are double-buffered in LDS; P goes straight from the QK accumulators to the B operand of the
// PV MFMA (O^T = V^T P^T), V^T is fetched with transposing LDS reads.
#include "fa_common.hpp"
#include "launch.hpp"

namespace fa {

namespace fwd_cfg {
constexpr int BM = 128;          // q rows per work-group
constexpr int BN = 64;           // kv rows per step
constexpr int D = 128;
constexpr int KSTR = D + 8;      // LDS row stride of K (elements): 16 B pad -> conflict-free b128 row reads
constexpr int VSTR = D + 32;     // LDS row stride of V: 64 B pad -> 4 rows x 64 B of a transposing read hit distinct banks
constexpr int K_TILE = BN * KSTR;
constexpr int V_TILE = BN * VSTR;
constexpr int LDS_BYTES = 2 * (K_TILE + V_TILE) * 2;
}  // namespace fwd_cfg

template <int SCORE>
__global__ __launch_bounds__(256, 2) void fwd_bf16_d128_kernel(FwdArgs a) {
  using namespace fwd_cfg;
  extern __shared__ __attribute__((aligned(16))) char smem_raw[];
  bf16_t* sK = reinterpret_cast<bf16_t*>(smem_raw);
  bf16_t* sV = sK + 2 * K_TILE;

  const int nQ = a.Sq / BM;
  const int nK = a.map.nk;
  const int n_wg = a.B * a.Hq * nQ;
  const int wg = xcd_remap(blockIdx.x, n_wg);
  const int bh = wg / nQ;
  const int qb = nQ - 1 - (wg % nQ);  // longest rows first under causal masks
  const int b = bh / a.Hq;
  const int h = bh % a.Hq;
  const int hk = h / (a.Hq / a.Hkv);

  const int tid = threadIdx.x;
  const int w = tid >> 6;
  const int lane = tid & 63;
  const int l32 = lane & 31;
  const int hh = lane >> 5;

  const bf16_t* Qg = static_cast<const bf16_t*>(a.q) + ((size_t)bh * a.Sq + (size_t)qb * BM) * D;
  const bf16_t* Kg = static_cast<const bf16_t*>(a.k) + ((size_t)(b * a.Hkv + hk) * a.Sk) * D;
  const bf16_t* Vg = static_cast<const bf16_t*>(a.v) + ((size_t)(b * a.Hkv + hk) * a.Sk) * D;
  bf16_t* Og = static_cast<bf16_t*>(a.o) + ((size_t)bh * a.Sq + (size_t)qb * BM) * D;

  const int q_local = w * 32 + l32;
  const int q_idx = qb * BM + q_local;

  ScoreMod<SCORE> sm;
  sm.init(a.score, a.sm_scale, h);

  // Q^T as B operand: lane holds q row l32, 8 consecutive d per k-step.
  bf16x8 qreg[8];
#pragma unroll
  for (int ks = 0; ks < 8; ++ks)
    qreg[ks] = *reinterpret_cast<const bf16x8*>(Qg + (size_t)q_local * D + ks * 16 + hh * 8);

  const int n_tiles = a.map.cnt[qb];
  const int* tile_idx = a.map.idx + (size_t)qb * nK;
  const uint8_t* tile_state = a.map.state + (size_t)qb * nK;

  int doc_i = 0;
  if (a.mask.flags & FLEXATTN_MASK_DOC) doc_i = a.mask.doc_q[q_idx];

  f32x16 o_acc[4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int e = 0; e < 16; ++e) o_acc[i][e] = 0.f;
  float m_run = kNegInf;  // running max, log2 domain
  float l_run = 0.f;      // this lane's half of the running sum

  // global -> LDS copy: 64 rows x 16 chunks of 16 B; thread handles chunk tid%16 of rows tid/16 + 16*j.
  const int cp_chunk = tid & 15;
  const int cp_row = tid >> 4;
  bf16x8 kst[4], vst[4];
  auto g_load = [&](int kb) {
    const bf16_t* kp = Kg + ((size_t)kb * BN + cp_row) * D + cp_chunk * 8;
    const bf16_t* vp = Vg + ((size_t)kb * BN + cp_row) * D + cp_chunk * 8;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      kst[j] = *reinterpret_cast<const bf16x8*>(kp + (size_t)j * 16 * D);
      vst[j] = *reinterpret_cast<const bf16x8*>(vp + (size_t)j * 16 * D);
    }
  };
  auto s_store = [&](int buf) {
    bf16_t* kd = sK + buf * K_TILE + cp_row * KSTR + cp_chunk * 8;
    bf16_t* vd = sV + buf * V_TILE + cp_row * VSTR + cp_chunk * 8;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      *reinterpret_cast<bf16x8*>(kd + j * 16 * KSTR) = kst[j];
      *reinterpret_cast<bf16x8*>(vd + j * 16 * VSTR) = vst[j];
    }
  };

  if (n_tiles > 0) {
    g_load(tile_idx[0]);
    s_store(0);
  }
  __syncthreads();

  for (int t = 0; t < n_tiles; ++t) {
    const int buf = t & 1;
    const int kb = tile_idx[t];
    const bool partial = tile_state[kb] == 1;
    if (t + 1 < n_tiles) g_load(tile_idx[t + 1]);

    // ---- S^T = K Q^T : two 32(kv) x 32(q) accumulator tiles ----
    f32x16 s_acc[2];
    const bf16_t* kbase = sK + buf * K_TILE + l32 * KSTR + hh * 8;
#pragma unroll
    for (int c = 0; c < 2; ++c) {
#pragma unroll
      for (int e = 0; e < 16; ++e) s_acc[c][e] = 0.f;
#pragma unroll
      for (int ks = 0; ks < 8; ++ks) {
        bf16x8 kf = *reinterpret_cast<const bf16x8*>(kbase + c * 32 * KSTR + ks * 16);
        s_acc[c] = mfma32(kf, qreg[ks], s_acc[c]);
      }
    }

    // ---- score mod, mask, online softmax (log2 domain) ----
    const int kv0 = kb * BN;
    float m_tile = kNegInf;
#pragma unroll
    for (int c = 0; c < 2; ++c) {
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int j = kv0 + 32 * c + acc_row(e, hh);
        float tv = sm.to_log2(s_acc[c][e], q_idx, j);
        if (partial) {
          int doc_j = 0;
          if (a.mask.flags & FLEXATTN_MASK_DOC) doc_j = a.mask.doc_k[j];
          if (!keep_elem(a.mask, q_idx, j, doc_i, doc_j)) tv = kNegInf;
        }
        s_acc[c][e] = tv;
        m_tile = fmaxf(m_tile, tv);
      }
    }
    m_tile = half_max(m_tile);
    const float m_new = fmaxf(m_run, m_tile);
    const float m_safe = (m_new == kNegInf) ? 0.f : m_new;
    const float alpha = fast_exp2(m_run - m_safe);
    m_run = m_new;
    float l_tile = 0.f;
    bf16x8 p[4];
#pragma unroll
    for (int c = 0; c < 2; ++c) {
#pragma unroll
      for (int e = 0; e < 16; e += 2) {
        float p0 = fast_exp2(s_acc[c][e] - m_safe);
        float p1 = fast_exp2(s_acc[c][e + 1] - m_safe);
        l_tile += p0 + p1;
        bf16x2 pk = pack_bf16(p0, p1);
        p[2 * c + (e >> 3)][e & 7] = pk[0];
        p[2 * c + (e >> 3)][(e & 7) + 1] = pk[1];
      }
    }
    l_run = l_run * alpha + l_tile;
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
      for (int e = 0; e < 16; ++e) o_acc[db][e] *= alpha;

    // ---- O^T += V^T P^T ----
    const bf16_t* vbase = sV + buf * V_TILE + (4 * hh + ((lane & 15) >> 2)) * VSTR + 16 * ((lane & 31) >> 4) +
                          4 * (lane & 3);
#pragma unroll
    for (int tt = 0; tt < 4; ++tt) {
#pragma unroll
      for (int db = 0; db < 4; ++db) {
        const bf16_t* vp = vbase + (16 * tt) * VSTR + 32 * db;
        bf16x8 vf = join_tr(lds_read_tr16(vp), lds_read_tr16(vp + 8 * VSTR));
        o_acc[db] = mfma32(vf, p[tt], o_acc[db]);
      }
    }

    if (t + 1 < n_tiles) s_store(buf ^ 1);
    __syncthreads();
  }

  // ---- epilogue ----
  const float l_tot = half_sum(l_run);
  const float inv = (l_tot > 0.f) ? 1.0f / l_tot : 0.f;
#pragma unroll
  for (int db = 0; db < 4; ++db) {
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      bf16x2 lo = pack_bf16(o_acc[db][4 * g] * inv, o_acc[db][4 * g + 1] * inv);
      bf16x2 hi = pack_bf16(o_acc[db][4 * g + 2] * inv, o_acc[db][4 * g + 3] * inv);
      bf16x4 out = {lo[0], lo[1], hi[0], hi[1]};
      *reinterpret_cast<bf16x4*>(Og + (size_t)q_local * D + 32 * db + 8 * g + 4 * hh) = out;
    }
  }
  if (a.l != nullptr && hh == 0) {
    const size_t r = (size_t)bh * a.Sq + q_idx;
    a.l[r] = l_tot;
    a.m[r] = m_run * kLn2;  // back to natural units
  }
}

template <int SCORE>
static int launch_fwd(const FwdArgs& a, hipStream_t stream) {
  using namespace fwd_cfg;
  auto kern = fwd_bf16_d128_kernel<SCORE>;
  static hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES);
  if (attr != hipSuccess) return set_error(FLEXATTN_ELAUNCH, "hipFuncSetAttribute(fwd): %s", hipGetErrorString(attr));
  const int n_wg = a.B * a.Hq * (a.Sq / BM);
  hipLaunchKernelGGL(kern, dim3(n_wg), dim3(256), LDS_BYTES, stream, a);
  return check_launch("flexattn_fwd bf16");
}

int fwd_bf16_d128(const FwdArgs& a, hipStream_t stream) {
  switch (a.score.kind) {
    case FLEXATTN_SCORE_NONE: return launch_fwd<FLEXATTN_SCORE_NONE>(a, stream);
    case FLEXATTN_SCORE_ALIBI: return launch_fwd<FLEXATTN_SCORE_ALIBI>(a, stream);
    case FLEXATTN_SCORE_SOFTCAP: return launch_fwd<FLEXATTN_SCORE_SOFTCAP>(a, stream);
    case FLEXATTN_SCORE_ALIBI_TILE: return launch_fwd<FLEXATTN_SCORE_ALIBI_TILE>(a, stream);
  }
  return set_error(FLEXATTN_EINVAL, "unknown score kind %d", a.score.kind);
}

void fwd_bf16_d128_tile(int* bq, int* bk) {
  *bq = fwd_cfg::BM;
  *bk = fwd_cfg::BN;
}

}  // namespace fa
