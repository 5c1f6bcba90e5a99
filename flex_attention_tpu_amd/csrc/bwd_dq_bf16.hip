// Flex-attention dq backward, bf16, head dim 128, gfx950.
//
// Same decomposition as the forward: one work-group = 4 waves = one 128-row Q tile, 32 q rows per
// wave, kv tiles of 64 rows double-buffered in LDS, everything computed transposed so that a lane
// owns one q row:   S^T = K Q^T,  dP^T = V dO^T,  P = exp2(S' - lse),  dS = P (dP - delta) f'(S),
// dq^T += K^T dS^T.  K is read twice from LDS: row-wise for S^T and with transposing reads for
// the K^T operand of the dq product.
#include "fa_common.hpp"
#include "launch.hpp"

namespace fa {

namespace dq_cfg {
constexpr int BM = 128;
constexpr int BN = 64;
constexpr int D = 128;
constexpr int KSTR = D + 24;  // 304 B rows: conflict-free for both b128 row reads and transposing reads
constexpr int VSTR = D + 8;   // 272 B rows: V is only read row-wise
constexpr int K_TILE = BN * KSTR;
constexpr int V_TILE = BN * VSTR;
constexpr int LDS_BYTES = 2 * (K_TILE + V_TILE) * 2;
}  // namespace dq_cfg

template <int SCORE>
__global__ __launch_bounds__(256, 2) void bwd_dq_bf16_d128_kernel(BwdArgs a) {
  using namespace dq_cfg;
  extern __shared__ __attribute__((aligned(16))) char smem_raw[];
  bf16_t* sK = reinterpret_cast<bf16_t*>(smem_raw);
  bf16_t* sV = sK + 2 * K_TILE;

  const int nQ = a.Sq / BM;
  const int nK = a.map.nk;
  const int n_wg = a.B * a.Hq * nQ;
  const int wg = xcd_remap(blockIdx.x, n_wg);
  const int bh = wg / nQ;
  const int qb = nQ - 1 - (wg % nQ);
  const int b = bh / a.Hq;
  const int h = bh % a.Hq;
  const int hk = h / (a.Hq / a.Hkv);

  const int tid = threadIdx.x;
  const int w = tid >> 6;
  const int lane = tid & 63;
  const int l32 = lane & 31;
  const int hh = lane >> 5;

  const size_t q_off = ((size_t)bh * a.Sq + (size_t)qb * BM) * D;
  const bf16_t* Qg = static_cast<const bf16_t*>(a.q) + q_off;
  const bf16_t* dOg = static_cast<const bf16_t*>(a.dout) + q_off;
  bf16_t* dQg = static_cast<bf16_t*>(a.dq) + q_off;
  const bf16_t* Kg = static_cast<const bf16_t*>(a.k) + ((size_t)(b * a.Hkv + hk) * a.Sk) * D;
  const bf16_t* Vg = static_cast<const bf16_t*>(a.v) + ((size_t)(b * a.Hkv + hk) * a.Sk) * D;

  const int q_local = w * 32 + l32;
  const int q_idx = qb * BM + q_local;
  const size_t row = (size_t)bh * a.Sq + q_idx;

  ScoreMod<SCORE> sm;
  sm.init(a.score, a.sm_scale, h);

  bf16x8 qreg[8], doreg[8];
#pragma unroll
  for (int ks = 0; ks < 8; ++ks) {
    qreg[ks] = *reinterpret_cast<const bf16x8*>(Qg + (size_t)q_local * D + ks * 16 + hh * 8);
    doreg[ks] = *reinterpret_cast<const bf16x8*>(dOg + (size_t)q_local * D + ks * 16 + hh * 8);
  }
  const float l_i = a.l[row], m_i = a.m[row];
  const float lse2 = (l_i > 0.f) ? __builtin_fmaf(m_i, kLog2e, log2f(l_i)) : __builtin_huge_valf();
  const float delta = a.delta[row];

  const int n_tiles = a.map.cnt[qb];
  const int* tile_idx = a.map.idx + (size_t)qb * nK;
  const uint8_t* tile_state = a.map.state + (size_t)qb * nK;
  int doc_i = 0;
  if (a.mask.flags & FLEXATTN_MASK_DOC) doc_i = a.mask.doc_q[q_idx];

  f32x16 dq_acc[4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int e = 0; e < 16; ++e) dq_acc[i][e] = 0.f;

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
    const int kv0 = kb * BN;

    const bf16_t* kbase = sK + buf * K_TILE + l32 * KSTR + hh * 8;
    const bf16_t* vbase = sV + buf * V_TILE + l32 * VSTR + hh * 8;
    const bf16_t* ktbase = sK + buf * K_TILE + (4 * hh + ((lane & 15) >> 2)) * KSTR + 16 * ((lane & 31) >> 4) +
                           4 * (lane & 3);
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      f32x16 s_acc, dp_acc;
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        s_acc[e] = 0.f;
        dp_acc[e] = 0.f;
      }
#pragma unroll
      for (int ks = 0; ks < 8; ++ks) {
        bf16x8 kf = *reinterpret_cast<const bf16x8*>(kbase + c * 32 * KSTR + ks * 16);
        s_acc = mfma32(kf, qreg[ks], s_acc);
      }
#pragma unroll
      for (int ks = 0; ks < 8; ++ks) {
        bf16x8 vf = *reinterpret_cast<const bf16x8*>(vbase + c * 32 * VSTR + ks * 16);
        dp_acc = mfma32(vf, doreg[ks], dp_acc);
      }
      bf16x8 ds[2];
#pragma unroll
      for (int e = 0; e < 16; e += 2) {
        float dsv[2];
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          const int j = kv0 + 32 * c + acc_row(e + u, hh);
          float tv = sm.to_log2(s_acc[e + u], q_idx, j);
          bool keep = true;
          if (partial) {
            int doc_j = 0;
            if (a.mask.flags & FLEXATTN_MASK_DOC) doc_j = a.mask.doc_k[j];
            keep = keep_elem(a.mask, q_idx, j, doc_i, doc_j);
          }
          const float p = fast_exp2(tv - lse2);
          const float g = p * (dp_acc[e + u] - delta) * sm.dfactor(tv);
          dsv[u] = keep ? g : 0.f;
        }
        bf16x2 pk = pack_bf16(dsv[0], dsv[1]);
        ds[e >> 3][e & 7] = pk[0];
        ds[e >> 3][(e & 7) + 1] = pk[1];
      }
      // dq^T += K^T dS^T for the two 16-row kv groups of this 32-row block
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const int tt = 2 * c + u;
#pragma unroll
        for (int db = 0; db < 4; ++db) {
          const bf16_t* kp = ktbase + (16 * tt) * KSTR + 32 * db;
          bf16x8 kf = join_tr(lds_read_tr16(kp), lds_read_tr16(kp + 8 * KSTR));
          dq_acc[db] = mfma32(kf, ds[u], dq_acc[db]);
        }
      }
    }

    if (t + 1 < n_tiles) s_store(buf ^ 1);
    __syncthreads();
  }

#pragma unroll
  for (int db = 0; db < 4; ++db) {
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      bf16x2 lo = pack_bf16(dq_acc[db][4 * g], dq_acc[db][4 * g + 1]);
      bf16x2 hi = pack_bf16(dq_acc[db][4 * g + 2], dq_acc[db][4 * g + 3]);
      bf16x4 out = {lo[0], lo[1], hi[0], hi[1]};
      *reinterpret_cast<bf16x4*>(dQg + (size_t)q_local * D + 32 * db + 8 * g + 4 * hh) = out;
    }
  }
}

template <int SCORE>
static int launch_dq(const BwdArgs& a, hipStream_t stream) {
  using namespace dq_cfg;
  auto kern = bwd_dq_bf16_d128_kernel<SCORE>;
  static hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES);
  if (attr != hipSuccess) return set_error(FLEXATTN_ELAUNCH, "hipFuncSetAttribute(dq): %s", hipGetErrorString(attr));
  const int n_wg = a.B * a.Hq * (a.Sq / BM);
  hipLaunchKernelGGL(kern, dim3(n_wg), dim3(256), LDS_BYTES, stream, a);
  return check_launch("flexattn_bwd_dq bf16");
}

int bwd_dq_bf16_d128(const BwdArgs& a, hipStream_t stream) {
  switch (a.score.kind) {
    case FLEXATTN_SCORE_NONE: return launch_dq<FLEXATTN_SCORE_NONE>(a, stream);
    case FLEXATTN_SCORE_ALIBI: return launch_dq<FLEXATTN_SCORE_ALIBI>(a, stream);
    case FLEXATTN_SCORE_SOFTCAP: return launch_dq<FLEXATTN_SCORE_SOFTCAP>(a, stream);
    case FLEXATTN_SCORE_ALIBI_TILE: return launch_dq<FLEXATTN_SCORE_ALIBI_TILE>(a, stream);
  }
  return set_error(FLEXATTN_EINVAL, "unknown score kind %d", a.score.kind);
}

void bwd_dq_bf16_d128_tile(int* bq, int* bk) {
  *bq = dq_cfg::BM;
  *bk = dq_cfg::BN;
}

}  // namespace fa
