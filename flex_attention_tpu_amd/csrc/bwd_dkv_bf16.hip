// Flex-attention dk/dv backward, bf16, head dim 128, gfx950.
//
// One work-group = 4 waves = one 128-row KV tile of one (batch, kv head); each wave owns 32 kv
// rows, whose K and V stay in registers as MFMA B operands.  Q / dO tiles of 128 rows stream
// through double-buffered LDS (LDS-direct loads, swizzled unpadded tiles) together with their
// lse and delta, for every query head of the KV group and every q tile the transposed block map
// lists.  Per tile:
//   S = Q K^T,  dP = dO V^T   (lane owns a kv column, accumulator rows are q),
//   P = exp2(S' - lse_q),  dS = P (dP - delta_q) f'(S),
//   dv^T += dO^T P,  dk^T += Q^T dS   (dO^T, Q^T via transposing LDS reads).
// Each dk/dv tile has exactly one writer, so the result is deterministic and needs no atomics.
#include "fa_common.hpp"
#include "launch.hpp"
#include "tile_io.hpp"

#include <type_traits>

namespace fa {

namespace dkv_cfg {
constexpr int BNK = 128;  // kv rows per work-group
constexpr int BQ = 128;   // q rows per step (two 64-row LDS tiles)
constexpr int D = 128;
constexpr int LDS_BYTES = 8 * kTileElems * 2 + 4 * BQ * 4;  // (Q, dO) x 2 buffers x 2 tiles, lse x2, delta x2
}  // namespace dkv_cfg

template <int SCORE>
__global__ __launch_bounds__(256, 1) void bwd_dkv_bf16_d128_kernel(BwdArgs a) {
  using namespace dkv_cfg;
  extern __shared__ __attribute__((aligned(1024))) char smem_raw[];
  bf16_t* sQ = reinterpret_cast<bf16_t*>(smem_raw);
  bf16_t* sDO = sQ + 4 * kTileElems;
  float* sLse = reinterpret_cast<float*>(sDO + 4 * kTileElems);
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
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  const int l32 = lane & 31;
  const int hh = lane >> 5;

  const int kv_local = w * 32 + l32;
  const int k_idx = kb * BNK + kv_local;
  const size_t kv_off = ((size_t)bhk * a.Sk + (size_t)kb * BNK) * D;
  const bf16_t* Kg = static_cast<const bf16_t*>(a.k) + kv_off;
  const bf16_t* Vg = static_cast<const bf16_t*>(a.v) + kv_off;
  const bf16_t* Qall = static_cast<const bf16_t*>(a.q);
  const bf16_t* dOall = static_cast<const bf16_t*>(a.dout);

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

  // Iteration `it` covers q tile tile_idx[it % n_tiles] of query head hk*group + it / n_tiles.
  // Its q block index is fetched two iterations ahead, its state one iteration ahead.
  auto q_block_of = [&](int it) { return tile_idx[it % n_tiles]; };
  int qb_cur = 0, qb_nxt = 0, st_cur = 0;
  if (n_iter > 0) qb_cur = q_block_of(0);
  if (n_iter > 1) qb_nxt = q_block_of(1);
  if (n_iter > 0) st_cur = a.map.state[(size_t)qb_cur * a.map.nk + kb];

  TileLoader<4> loader;
  loader.init(w, lane);
  float lse_st = 0.f, dl_st = 0.f;
  auto issue_tile = [&](int it, int qb, int buf) {
    const int g = it / n_tiles;
    const size_t rbase = ((size_t)(b * a.Hq + hk * group + g) * a.Sq + (size_t)qb * BQ);
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      loader.load(Qall + (rbase + half * kTileRows) * D, sQ + (2 * buf + half) * kTileElems);
      loader.load(dOall + (rbase + half * kTileRows) * D, sDO + (2 * buf + half) * kTileElems);
    }
    if (tid < BQ) {
      const float l_i = a.l[rbase + tid], m_i = a.m[rbase + tid];
      lse_st = (l_i > 0.f) ? __builtin_fmaf(m_i, kLog2e, log2f(l_i)) : __builtin_huge_valf();
      dl_st = a.delta[rbase + tid];
    }
  };
  auto store_rows = [&](int buf) {
    if (tid < BQ) {
      sLse[buf * BQ + tid] = lse_st;
      sDl[buf * BQ + tid] = dl_st;
    }
  };
  if (n_iter > 0) {
    issue_tile(0, __builtin_amdgcn_readfirstlane(qb_cur), 0);
    store_rows(0);
  }
  wait_vmem_all();
  __syncthreads();

  // lane-constant byte offsets of the operand reads inside a tile (see tile_io.hpp)
  const int r_sw = swz(l32);
  const int t_row = 4 * hh + ((lane & 15) >> 2);
  const int t_chunk = 2 * ((lane & 31) >> 4) + ((lane & 3) >> 1);
  const int t_half = 4 * (lane & 1);
  unsigned r_off[8], t_off[4][2];
#pragma unroll
  for (int ks = 0; ks < 8; ++ks) r_off[ks] = (unsigned)(l32 * kTileD + (((2 * ks + hh) ^ r_sw) << 3)) * 2u;
#pragma unroll
  for (int db = 0; db < 4; ++db) {
    t_off[db][0] = (unsigned)(tile_off(t_row, 4 * db + t_chunk) + t_half) * 2u;
    t_off[db][1] = (unsigned)(tile_off(t_row + 8, 4 * db + t_chunk) + t_half) * 2u;
  }

  ScoreMod<SCORE> sm;
  for (int it = 0; it < n_iter; ++it) {
    const int buf = it & 1;
    const int qb = __builtin_amdgcn_readfirstlane(qb_cur);
    const bool partial = __builtin_amdgcn_readfirstlane(st_cur) == 1;
    sm.init(a.score, a.sm_scale, hk * group + it / n_tiles);
    const int qb_n2 = (it + 2 < n_iter) ? q_block_of(it + 2) : 0;
    int st_nxt = 0;
    if (it + 1 < n_iter) {
      const int qbn = __builtin_amdgcn_readfirstlane(qb_nxt);
      st_nxt = a.map.state[(size_t)qbn * a.map.nk + kb];
      issue_tile(it + 1, qbn, buf ^ 1);
    }
    const int q0 = qb * BQ;
#pragma unroll
    for (int cc = 0; cc < 4; ++cc) {
      const int c = cc & 1;  // 32-row block inside the 64-row LDS tile cc >> 1
      const char* qt = reinterpret_cast<const char*>(sQ + (2 * buf + (cc >> 1)) * kTileElems);
      const char* dot = reinterpret_cast<const char*>(sDO + (2 * buf + (cc >> 1)) * kTileElems);
      f32x16 s_acc, dp_acc;
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        s_acc[e] = 0.f;
        dp_acc[e] = 0.f;
      }
      {
        bf16x8 qf[8];
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) qf[ks] = *reinterpret_cast<const bf16x8*>(qt + r_off[ks] + c * 32 * kTileD * 2);
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) s_acc = mfma32(qf[ks], kreg[ks], s_acc);
      }
      {
        bf16x8 df[8];
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) df[ks] = *reinterpret_cast<const bf16x8*>(dot + r_off[ks] + c * 32 * kTileD * 2);
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) dp_acc = mfma32(df[ks], vreg[ks], dp_acc);
      }
      // transposed fragments of this 32-row q block for the dv / dk products
      s16x4 dolo[2][4], dohi[2][4], qlo[2][4], qhi[2][4];
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int db = 0; db < 4; ++db) {
          const int off = (32 * c + 16 * u) * kTileD * 2;
          dolo[u][db] = lds_read_tr16(reinterpret_cast<const bf16_t*>(dot + t_off[db][0] + off));
          dohi[u][db] = lds_read_tr16(reinterpret_cast<const bf16_t*>(dot + t_off[db][1] + off));
          qlo[u][db] = lds_read_tr16(reinterpret_cast<const bf16_t*>(qt + t_off[db][0] + off));
          qhi[u][db] = lds_read_tr16(reinterpret_cast<const bf16_t*>(qt + t_off[db][1] + off));
        }

      bf16x8 pb[2], dsb[2];
      auto elementwise = [&](auto masked) {
        constexpr bool MASKED = decltype(masked)::value;
        const bool has_doc = MASKED && (a.mask.flags & FLEXATTN_MASK_DOC) != 0;
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4) {
          const int r0 = 32 * cc + 8 * g4 + 4 * hh;  // the lane's q rows come in runs of 4
          const f32x4 lse4 = *reinterpret_cast<const f32x4*>(sLse + buf * BQ + r0);
          const f32x4 dl4 = *reinterpret_cast<const f32x4*>(sDl + buf * BQ + r0);
          int di[4] = {0, 0, 0, 0};
          if (MASKED && has_doc) {
            const auto d4 = *reinterpret_cast<const int __attribute__((ext_vector_type(4)))*>(a.mask.doc_q + q0 + r0);
            di[0] = d4[0]; di[1] = d4[1]; di[2] = d4[2]; di[3] = d4[3];
          }
          float pv[4], dsv[4];
#pragma unroll
          for (int u = 0; u < 4; ++u) {
            const int e = 4 * g4 + u;
            const int i = q0 + r0 + u;
            const float tv = sm.to_log2(s_acc[e], i, k_idx);
            float pe = fast_exp2(tv - lse4[u]);
            float gd = pe * (dp_acc[e] - dl4[u]) * sm.dfactor(tv);
            if (MASKED) {
              const bool keep = keep_elem(a.mask, i, k_idx, di[u], doc_j);
              pe = keep ? pe : 0.f;
              gd = keep ? gd : 0.f;
            }
            pv[u] = pe;
            dsv[u] = gd;
          }
          const bf16x2 p01 = pack_bf16(pv[0], pv[1]), p23 = pack_bf16(pv[2], pv[3]);
          const bf16x2 d01 = pack_bf16(dsv[0], dsv[1]), d23 = pack_bf16(dsv[2], dsv[3]);
          const int o = 4 * (g4 & 1);
          pb[g4 >> 1][o] = p01[0]; pb[g4 >> 1][o + 1] = p01[1]; pb[g4 >> 1][o + 2] = p23[0]; pb[g4 >> 1][o + 3] = p23[1];
          dsb[g4 >> 1][o] = d01[0]; dsb[g4 >> 1][o + 1] = d01[1]; dsb[g4 >> 1][o + 2] = d23[0]; dsb[g4 >> 1][o + 3] = d23[1];
        }
      };
      if (partial) {
        elementwise(std::true_type{});
      } else {
        elementwise(std::false_type{});
      }

#pragma unroll
      for (int u = 0; u < 2; ++u) {
#pragma unroll
        for (int db = 0; db < 4; ++db) {
          dv_acc[db] = mfma32(join_tr(dolo[u][db], dohi[u][db]), pb[u], dv_acc[db]);
          dk_acc[db] = mfma32(join_tr(qlo[u][db], qhi[u][db]), dsb[u], dk_acc[db]);
        }
      }
    }

    qb_cur = qb_nxt; qb_nxt = qb_n2;
    st_cur = st_nxt;
    if (it + 1 < n_iter) store_rows(buf ^ 1);
    wait_vmem_all();
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
