// Flex-attention dq backward, bf16, head dim 128, gfx950.
//
// Same decomposition as the forward: one work-group = 4 waves = one 128-row Q tile, 32 q rows per
// wave, kv tiles of 64 rows double-buffered in LDS by LDS-direct loads (swizzled, unpadded tiles),
// everything computed transposed so that a lane owns one q row:
//   S^T = K Q^T,  dP^T = V dO^T,  P = exp2(S' - lse),  dS = P (dP - delta) f'(S),  dq^T += K^T dS^T.
// K is read twice from LDS: row-wise for S^T and with transposing reads for the K^T operand of
// the dq product.  Q and dO stay in registers as MFMA B operands.
#include "fa_common.hpp"
#include "launch.hpp"
#include "tile_io.hpp"

#include <type_traits>

namespace fa {

namespace dq_cfg {
constexpr int BM = 128;
constexpr int BN = 64;
constexpr int D = 128;
constexpr int LDS_BYTES = 4 * kTileElems * 2;  // K x2, V x2
}  // namespace dq_cfg

template <int SCORE>
__global__ __launch_bounds__(256, 2) void bwd_dq_bf16_d128_kernel(BwdArgs a) {
  using namespace dq_cfg;
  extern __shared__ __attribute__((aligned(1024))) char smem_raw[];
  bf16_t* sK = reinterpret_cast<bf16_t*>(smem_raw);
  bf16_t* sV = sK + 2 * kTileElems;

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
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
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

  // Tile indices and states are fetched ahead of use (index three tiles, state two tiles ahead) so
  // that no iteration waits on a load it has just issued.
  int kb_cur = 0, kb_nxt = 0, kb_n2 = 0, st_cur = 0, st_nxt = 0;
  if (n_tiles > 0) kb_cur = tile_idx[0];
  if (n_tiles > 1) kb_nxt = tile_idx[1];
  if (n_tiles > 2) kb_n2 = tile_idx[2];
  if (n_tiles > 0) st_cur = tile_state[kb_cur];
  if (n_tiles > 1) st_nxt = tile_state[kb_nxt];
  TileLoader<4> loader;
  loader.init(w, lane);
  if (n_tiles > 0) {
    const int kb0 = __builtin_amdgcn_readfirstlane(kb_cur);
    loader.load(Kg + (size_t)kb0 * BN * D, sK);
    loader.load(Vg + (size_t)kb0 * BN * D, sV);
  }
  wait_vmem_all();
  __syncthreads();

  // lane-constant byte offsets of the operand reads inside a tile (see tile_io.hpp)
  const int k_sw = swz(l32);
  const int t_row = 4 * hh + ((lane & 15) >> 2);
  const int t_chunk = 2 * ((lane & 31) >> 4) + ((lane & 3) >> 1);
  const int t_half = 4 * (lane & 1);
  unsigned r_off[8], t_off[4][2];
#pragma unroll
  for (int ks = 0; ks < 8; ++ks) r_off[ks] = (unsigned)(l32 * kTileD + (((2 * ks + hh) ^ k_sw) << 3)) * 2u;
#pragma unroll
  for (int db = 0; db < 4; ++db) {
    t_off[db][0] = (unsigned)(tile_off(t_row, 4 * db + t_chunk) + t_half) * 2u;
    t_off[db][1] = (unsigned)(tile_off(t_row + 8, 4 * db + t_chunk) + t_half) * 2u;
  }

  for (int t = 0; t < n_tiles; ++t) {
    const int buf = t & 1;
    const int kb = __builtin_amdgcn_readfirstlane(kb_cur);
    const bool partial = __builtin_amdgcn_readfirstlane(st_cur) == 1;
    const int kb_n3 = (t + 3 < n_tiles) ? tile_idx[t + 3] : 0;
    const int st_n2 = (t + 2 < n_tiles) ? tile_state[kb_n2] : 0;
    if (t + 1 < n_tiles) {
      const int kbn = __builtin_amdgcn_readfirstlane(kb_nxt);
      loader.load(Kg + (size_t)kbn * BN * D, sK + (buf ^ 1) * kTileElems);
      loader.load(Vg + (size_t)kbn * BN * D, sV + (buf ^ 1) * kTileElems);
    }
    const int kv0 = kb * BN;
    const char* kt = reinterpret_cast<const char*>(sK + buf * kTileElems);
    const char* vt = reinterpret_cast<const char*>(sV + buf * kTileElems);

#pragma unroll
    for (int c = 0; c < 2; ++c) {
      // ---- S^T and dP^T for kv rows [32c, 32c+32) ----
      f32x16 s_acc, dp_acc;
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        s_acc[e] = 0.f;
        dp_acc[e] = 0.f;
      }
      {
        bf16x8 kf[8];
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) kf[ks] = *reinterpret_cast<const bf16x8*>(kt + r_off[ks] + c * 32 * kTileD * 2);
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) s_acc = mfma32(kf[ks], qreg[ks], s_acc);
      }
      {
        bf16x8 vf[8];
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) vf[ks] = *reinterpret_cast<const bf16x8*>(vt + r_off[ks] + c * 32 * kTileD * 2);
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) dp_acc = mfma32(vf[ks], doreg[ks], dp_acc);
      }
      // K^T fragments for the dq product
      s16x4 klo[2][4], khi[2][4];
      auto read_kt = [&](int u) {
#pragma unroll
        for (int db = 0; db < 4; ++db) {
          const int off = (32 * c + 16 * u) * kTileD * 2;
          klo[u][db] = lds_read_tr16(reinterpret_cast<const bf16_t*>(kt + t_off[db][0] + off));
          khi[u][db] = lds_read_tr16(reinterpret_cast<const bf16_t*>(kt + t_off[db][1] + off));
        }
      };

      // ---- P, dS -> bf16 ----
      bf16x8 ds[2];
      auto elementwise = [&](auto masked) {
        constexpr bool MASKED = decltype(masked)::value;
        const bool has_doc = MASKED && (a.mask.flags & FLEXATTN_MASK_DOC) != 0;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const int j0 = kv0 + 32 * c + 8 * g + 4 * hh;
          int dj[4] = {0, 0, 0, 0};
          if (MASKED && has_doc) {
            const auto d4 = *reinterpret_cast<const int __attribute__((ext_vector_type(4)))*>(a.mask.doc_k + j0);
            dj[0] = d4[0]; dj[1] = d4[1]; dj[2] = d4[2]; dj[3] = d4[3];
          }
          float dsv[4];
#pragma unroll
          for (int u = 0; u < 4; ++u) {
            const int e = 4 * g + u;
            const float tv = sm.to_log2(s_acc[e], q_idx, j0 + u);
            const float pe = fast_exp2(tv - lse2);
            float gd = pe * (dp_acc[e] - delta) * sm.dfactor(tv);
            if (MASKED) gd = keep_elem(a.mask, q_idx, j0 + u, doc_i, dj[u]) ? gd : 0.f;
            dsv[u] = gd;
          }
          const bf16x2 d01 = pack_bf16(dsv[0], dsv[1]), d23 = pack_bf16(dsv[2], dsv[3]);
          const int o = 4 * (g & 1);
          ds[g >> 1][o] = d01[0]; ds[g >> 1][o + 1] = d01[1]; ds[g >> 1][o + 2] = d23[0]; ds[g >> 1][o + 3] = d23[1];
        }
      };
      if (partial) {
        elementwise(std::true_type{});
      } else {
        elementwise(std::false_type{});
      }

      // ---- dq^T += K^T dS^T for the two 16-row kv groups of this block ----
      read_kt(0);
      read_kt(1);
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int db = 0; db < 4; ++db) dq_acc[db] = mfma32(join_tr(klo[u][db], khi[u][db]), ds[u], dq_acc[db]);
    }

    kb_cur = kb_nxt; kb_nxt = kb_n2; kb_n2 = kb_n3;
    st_cur = st_nxt; st_nxt = st_n2;
    wait_vmem_all();
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
