// Flex-attention dk/dv backward, bf16, head dim 128, gfx950.
//
// One work-group = 4 waves = one 128-row KV tile of one (batch, kv head); each wave owns 32 kv
// rows, whose K and V stay in registers as MFMA B operands.  Q / dO tiles of 64 rows (with their
// lse and delta) stream through double-buffered LDS, for every query head of the KV group and
// every q tile the transposed block map lists.  Per tile:
//   S = Q K^T,  dP = dO V^T   (lane owns a kv column, accumulator rows are q),
//   P = exp2(S' - lse_q),  dS = P (dP - delta_q) f'(S),
//   dv^T += dO^T P,  dk^T += Q^T dS   (dO^T, Q^T via transposing LDS reads).
// Each dk/dv tile has exactly one writer, so the result is deterministic and needs no atomics.
#include "fa_common.hpp"
#include "launch.hpp"

namespace fa {

namespace dkv_cfg {
constexpr int BNK = 128;  // kv rows per work-group
constexpr int BQ = 64;    // q rows per step
constexpr int D = 128;
constexpr int QSTR = D + 24;  // 304 B rows: conflict-free for b128 row reads and transposing reads
constexpr int Q_TILE = BQ * QSTR;
constexpr int LDS_BYTES = 2 * (2 * Q_TILE * 2 + 2 * BQ * 4);
}  // namespace dkv_cfg

template <int SCORE>
__global__ __launch_bounds__(256, 1) void bwd_dkv_bf16_d128_kernel(BwdArgs a) {
  using namespace dkv_cfg;
  extern __shared__ __attribute__((aligned(16))) char smem_raw[];
  bf16_t* sQ = reinterpret_cast<bf16_t*>(smem_raw);
  bf16_t* sDO = sQ + 2 * Q_TILE;
  float* sLse = reinterpret_cast<float*>(sDO + 2 * Q_TILE);
  float* sDl = sLse + 2 * BQ;

  const int nKb = a.Sk / BNK;
  const int nQ = a.map.nq;
  const int n_wg = a.B * a.Hkv * nKb;
  const int wg = xcd_remap(blockIdx.x, n_wg);
  const int bhk = wg / nKb;
  const int kb = wg % nKb;  // low kv tiles have the most q tiles under causal masks: they go first
  const int b = bhk / a.Hkv;
  const int hk = bhk % a.Hkv;
  const int group = a.Hq / a.Hkv;

  const int tid = threadIdx.x;
  const int w = tid >> 6;
  const int lane = tid & 63;
  const int l32 = lane & 31;
  const int hh = lane >> 5;

  const int kv_local = w * 32 + l32;
  const int k_idx = kb * BNK + kv_local;
  const size_t kv_off = ((size_t)bhk * a.Sk + (size_t)kb * BNK) * D;
  const bf16_t* Kg = static_cast<const bf16_t*>(a.k) + kv_off;
  const bf16_t* Vg = static_cast<const bf16_t*>(a.v) + kv_off;

  bf16x8 kreg[8], vreg[8];
#pragma unroll
  for (int ks = 0; ks < 8; ++ks) {
    kreg[ks] = *reinterpret_cast<const bf16x8*>(Kg + (size_t)kv_local * D + ks * 16 + hh * 8);
    vreg[ks] = *reinterpret_cast<const bf16x8*>(Vg + (size_t)kv_local * D + ks * 16 + hh * 8);
  }
  int doc_j = 0;
  if (a.mask.flags & FLEXATTN_MASK_DOC) doc_j = a.mask.doc_k[k_idx];

  f32x16 dk_acc[4], dv_acc[4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      dk_acc[i][e] = 0.f;
      dv_acc[i][e] = 0.f;
    }

  const int n_tiles = a.map.cnt[kb];
  const int* tile_idx = a.map.idx + (size_t)kb * nQ;
  const int n_iter = n_tiles * group;

  const int cp_chunk = tid & 15;
  const int cp_row = tid >> 4;
  bf16x8 qst[4], dost[4];
  float lse_st = 0.f, dl_st = 0.f;
  auto g_load = [&](int it) {
    const int g = it / n_tiles;
    const int qb = tile_idx[it - g * n_tiles];
    const size_t rbase = ((size_t)(b * a.Hq + hk * group + g) * a.Sq + (size_t)qb * BQ);
    const bf16_t* qp = static_cast<const bf16_t*>(a.q) + (rbase + cp_row) * D + cp_chunk * 8;
    const bf16_t* dp = static_cast<const bf16_t*>(a.dout) + (rbase + cp_row) * D + cp_chunk * 8;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      qst[j] = *reinterpret_cast<const bf16x8*>(qp + (size_t)j * 16 * D);
      dost[j] = *reinterpret_cast<const bf16x8*>(dp + (size_t)j * 16 * D);
    }
    if (tid < BQ) {
      const float l_i = a.l[rbase + tid], m_i = a.m[rbase + tid];
      lse_st = (l_i > 0.f) ? __builtin_fmaf(m_i, kLog2e, log2f(l_i)) : __builtin_huge_valf();
      dl_st = a.delta[rbase + tid];
    }
  };
  auto s_store = [&](int buf) {
    bf16_t* qd = sQ + buf * Q_TILE + cp_row * QSTR + cp_chunk * 8;
    bf16_t* dd = sDO + buf * Q_TILE + cp_row * QSTR + cp_chunk * 8;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      *reinterpret_cast<bf16x8*>(qd + j * 16 * QSTR) = qst[j];
      *reinterpret_cast<bf16x8*>(dd + j * 16 * QSTR) = dost[j];
    }
    if (tid < BQ) {
      sLse[buf * BQ + tid] = lse_st;
      sDl[buf * BQ + tid] = dl_st;
    }
  };

  if (n_iter > 0) {
    g_load(0);
    s_store(0);
  }
  __syncthreads();

  ScoreMod<SCORE> sm;
  for (int it = 0; it < n_iter; ++it) {
    const int buf = it & 1;
    const int g = it / n_tiles;
    const int qb = tile_idx[it - g * n_tiles];
    const bool partial = a.map.state[(size_t)qb * a.map.nk + kb] == 1;
    sm.init(a.score, a.sm_scale, hk * group + g);
    if (it + 1 < n_iter) g_load(it + 1);
    const int q0 = qb * BQ;

    const bf16_t* qbase = sQ + buf * Q_TILE + l32 * QSTR + hh * 8;
    const bf16_t* dobase = sDO + buf * Q_TILE + l32 * QSTR + hh * 8;
    const int tr_off = (4 * hh + ((lane & 15) >> 2)) * QSTR + 16 * ((lane & 31) >> 4) + 4 * (lane & 3);
    const bf16_t* qtbase = sQ + buf * Q_TILE + tr_off;
    const bf16_t* dotbase = sDO + buf * Q_TILE + tr_off;

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
        bf16x8 qf = *reinterpret_cast<const bf16x8*>(qbase + c * 32 * QSTR + ks * 16);
        s_acc = mfma32(qf, kreg[ks], s_acc);
      }
#pragma unroll
      for (int ks = 0; ks < 8; ++ks) {
        bf16x8 df = *reinterpret_cast<const bf16x8*>(dobase + c * 32 * QSTR + ks * 16);
        dp_acc = mfma32(df, vreg[ks], dp_acc);
      }
      bf16x8 pb[2], dsb[2];
#pragma unroll
      for (int g4 = 0; g4 < 4; ++g4) {
        const f32x4 lse4 = *reinterpret_cast<const f32x4*>(sLse + buf * BQ + 32 * c + 8 * g4 + 4 * hh);
        const f32x4 dl4 = *reinterpret_cast<const f32x4*>(sDl + buf * BQ + 32 * c + 8 * g4 + 4 * hh);
        float pv[4], dsv[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int e = 4 * g4 + u;
          const int i = q0 + 32 * c + 8 * g4 + 4 * hh + u;
          float tv = sm.to_log2(s_acc[e], i, k_idx);
          bool keep = true;
          if (partial) {
            int doc_i = 0;
            if (a.mask.flags & FLEXATTN_MASK_DOC) doc_i = a.mask.doc_q[i];
            keep = keep_elem(a.mask, i, k_idx, doc_i, doc_j);
          }
          const float p = fast_exp2(tv - lse4[u]);
          const float gd = p * (dp_acc[e] - dl4[u]) * sm.dfactor(tv);
          pv[u] = keep ? p : 0.f;
          dsv[u] = keep ? gd : 0.f;
        }
        bf16x2 p01 = pack_bf16(pv[0], pv[1]), p23 = pack_bf16(pv[2], pv[3]);
        bf16x2 d01 = pack_bf16(dsv[0], dsv[1]), d23 = pack_bf16(dsv[2], dsv[3]);
        const int o = 4 * (g4 & 1);
        pb[g4 >> 1][o] = p01[0]; pb[g4 >> 1][o + 1] = p01[1]; pb[g4 >> 1][o + 2] = p23[0]; pb[g4 >> 1][o + 3] = p23[1];
        dsb[g4 >> 1][o] = d01[0]; dsb[g4 >> 1][o + 1] = d01[1]; dsb[g4 >> 1][o + 2] = d23[0]; dsb[g4 >> 1][o + 3] = d23[1];
      }
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const int tt = 2 * c + u;  // 16-row q group inside the 64-row tile
#pragma unroll
        for (int db = 0; db < 4; ++db) {
          const bf16_t* dp = dotbase + (16 * tt) * QSTR + 32 * db;
          bf16x8 dof = join_tr(lds_read_tr16(dp), lds_read_tr16(dp + 8 * QSTR));
          dv_acc[db] = mfma32(dof, pb[u], dv_acc[db]);
        }
#pragma unroll
        for (int db = 0; db < 4; ++db) {
          const bf16_t* qp = qtbase + (16 * tt) * QSTR + 32 * db;
          bf16x8 qf = join_tr(lds_read_tr16(qp), lds_read_tr16(qp + 8 * QSTR));
          dk_acc[db] = mfma32(qf, dsb[u], dk_acc[db]);
        }
      }
    }

    if (it + 1 < n_iter) s_store(buf ^ 1);
    __syncthreads();
  }

  bf16_t* dKg = static_cast<bf16_t*>(a.dk) + kv_off;
  bf16_t* dVg = static_cast<bf16_t*>(a.dv) + kv_off;
#pragma unroll
  for (int db = 0; db < 4; ++db) {
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      bf16x2 lo = pack_bf16(dk_acc[db][4 * g], dk_acc[db][4 * g + 1]);
      bf16x2 hi = pack_bf16(dk_acc[db][4 * g + 2], dk_acc[db][4 * g + 3]);
      bf16x4 out = {lo[0], lo[1], hi[0], hi[1]};
      *reinterpret_cast<bf16x4*>(dKg + (size_t)kv_local * D + 32 * db + 8 * g + 4 * hh) = out;
      lo = pack_bf16(dv_acc[db][4 * g], dv_acc[db][4 * g + 1]);
      hi = pack_bf16(dv_acc[db][4 * g + 2], dv_acc[db][4 * g + 3]);
      bf16x4 out2 = {lo[0], lo[1], hi[0], hi[1]};
      *reinterpret_cast<bf16x4*>(dVg + (size_t)kv_local * D + 32 * db + 8 * g + 4 * hh) = out2;
    }
  }
}

template <int SCORE>
static int launch_dkv(const BwdArgs& a, hipStream_t stream) {
  using namespace dkv_cfg;
  auto kern = bwd_dkv_bf16_d128_kernel<SCORE>;
  static hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES);
  if (attr != hipSuccess) return set_error(FLEXATTN_ELAUNCH, "hipFuncSetAttribute(dkv): %s", hipGetErrorString(attr));
  const int n_wg = a.B * a.Hkv * (a.Sk / BNK);
  hipLaunchKernelGGL(kern, dim3(n_wg), dim3(256), LDS_BYTES, stream, a);
  return check_launch("flexattn_bwd_dkv bf16");
}

int bwd_dkv_bf16_d128(const BwdArgs& a, hipStream_t stream) {
  switch (a.score.kind) {
    case FLEXATTN_SCORE_NONE: return launch_dkv<FLEXATTN_SCORE_NONE>(a, stream);
    case FLEXATTN_SCORE_ALIBI: return launch_dkv<FLEXATTN_SCORE_ALIBI>(a, stream);
    case FLEXATTN_SCORE_SOFTCAP: return launch_dkv<FLEXATTN_SCORE_SOFTCAP>(a, stream);
    case FLEXATTN_SCORE_ALIBI_TILE: return launch_dkv<FLEXATTN_SCORE_ALIBI_TILE>(a, stream);
  }
  return set_error(FLEXATTN_EINVAL, "unknown score kind %d", a.score.kind);
}

void bwd_dkv_bf16_d128_tile(int* bq, int* bk) {
  *bq = dkv_cfg::BQ;
  *bk = dkv_cfg::BNK;
}

}  // namespace fa
