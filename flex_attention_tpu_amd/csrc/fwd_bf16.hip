// Flex-attention forward, bf16, head dim 128, gfx950.
//
// One work-group = 4 waves = one 128-row Q tile of one (batch, head); each wave owns 32 q rows.
// The kernel works on S^T = K Q^T so that one lane holds one q row's scores: softmax statistics
// stay lane-private apart from one exchange between the two 32-lane halves.  K/V tiles of 64 rows
// are double-buffered in LDS by LDS-direct loads issued one tile ahead; P goes straight from the
// QK accumulators to the B operand of the PV MFMA (O^T = V^T P^T); V^T is fetched with
// transposing LDS reads.
#include "fa_common.hpp"
#include "launch.hpp"
#include "tile_io.hpp"

namespace fa {

namespace fwd_cfg {
constexpr int BM = 128;  // q rows per work-group
constexpr int BN = 64;   // kv rows per step
constexpr int D = 128;
constexpr int LDS_BYTES = 4 * kTileElems * 2;  // K x2, V x2
}  // namespace fwd_cfg

template <int SCORE>
__global__ __launch_bounds__(256, 2) void fwd_bf16_d128_kernel(FwdArgs a) {
  using namespace fwd_cfg;
  extern __shared__ __attribute__((aligned(1024))) char smem_raw[];
  bf16_t* sK = reinterpret_cast<bf16_t*>(smem_raw);
  bf16_t* sV = sK + 2 * kTileElems;

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
  float m_run = kNegInf;  // running max: raw dot-product units (plain score) or log2-domain logits
  float l_run = 0.f;      // this lane's half of the running sum

  // Tile indices and states are fetched ahead of use (index three tiles, state two tiles ahead) so
  // that no iteration waits on a load it has just issued.
  int kb_cur = 0, kb_nxt = 0, kb_n2 = 0, st_cur = 0, st_nxt = 0;
  if (n_tiles > 0) kb_cur = tile_idx[0];
  if (n_tiles > 1) kb_nxt = tile_idx[1];
  if (n_tiles > 2) kb_n2 = tile_idx[2];
  if (n_tiles > 0) st_cur = tile_state[kb_cur];
  if (n_tiles > 1) st_nxt = tile_state[kb_nxt];
  TileLoader<4> loader;
  loader.init(__builtin_amdgcn_readfirstlane(w), lane);
  if (n_tiles > 0) {
    const int kb0 = __builtin_amdgcn_readfirstlane(kb_cur);
    loader.load(Kg + (size_t)kb0 * BN * D, sK);
    loader.load(Vg + (size_t)kb0 * BN * D, sV);
  }
  wait_vmem_all();
  __syncthreads();

  // lane-constant pieces of the LDS addresses
  const int k_sw = swz(l32);                               // row reads: rows l32 (+32c)
  const int v_row = 4 * hh + ((lane & 15) >> 2);           // transposing reads: row inside a 16-row group
  const int v_chunk = 2 * ((lane & 31) >> 4) + ((lane & 3) >> 1);
  const int v_half = 4 * (lane & 1);
  // Byte offsets inside a tile of this lane's operand reads; the row block (32c for K rows, 16tt
  // for V^T groups) is an immediate and the buffer a per-step base.
  unsigned k_off[8], v_off[4][2];
#pragma unroll
  for (int ks = 0; ks < 8; ++ks) k_off[ks] = (unsigned)(l32 * kTileD + (((2 * ks + hh) ^ k_sw) << 3)) * 2u;
#pragma unroll
  for (int db = 0; db < 4; ++db) {
    v_off[db][0] = (unsigned)(tile_off(v_row, 4 * db + v_chunk) + v_half) * 2u;
    v_off[db][1] = (unsigned)(tile_off(v_row + 8, 4 * db + v_chunk) + v_half) * 2u;
  }
#define FA_INTERLEAVE(N_MFMA, READS)                                   \
  _Pragma("unroll") for (int i_ = 0; i_ < (N_MFMA); ++i_) {            \
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                 \
    __builtin_amdgcn_sched_group_barrier(0x100, (READS), 0);           \
  }

  for (int t = 0; t < n_tiles; ++t) {
    const int buf = t & 1;
    const int kb = __builtin_amdgcn_readfirstlane(kb_cur);
    const bool partial = __builtin_amdgcn_readfirstlane(st_cur) == 1;
    const int kb_n3 = (t + 3 < n_tiles) ? tile_idx[t + 3] : 0;
    const int st_n2 = (t + 2 < n_tiles) ? tile_state[kb_n2] : 0;
    // The next tile's LDS-direct loads are issued two at a time between the MFMA stages below.
    const bool prefetch = t + 1 < n_tiles;
    const int kbn = __builtin_amdgcn_readfirstlane(kb_nxt);
    const bf16_t* k_next = Kg + (size_t)kbn * BN * D;
    const bf16_t* v_next = Vg + (size_t)kbn * BN * D;

    // ---- S^T = K Q^T : two 32(kv) x 32(q) accumulator tiles ----
    // LDS operand reads run one stage (4 MFMAs) ahead of the MFMAs that consume them, so the LDS
    // pipe and the matrix pipe overlap inside the wave; sched_barrier fences the stages.  The
    // first half of V^T is fetched before the softmax, whose VALU work hides that latency.
    f32x16 s_acc[2];
    const char* kt = reinterpret_cast<const char*>(sK + buf * kTileElems);
    const char* vt = reinterpret_cast<const char*>(sV + buf * kTileElems);
    bf16x8 kf[4][4];             // [2c + ks/4][ks%4]
    s16x4 vlo[4][4], vhi[4][4];  // [tt][db]
    auto read_k = [&](int g) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        kf[g][i] = *reinterpret_cast<const bf16x8*>(kt + k_off[4 * (g & 1) + i] + (g >> 1) * 32 * kTileD * 2);
    };
    auto read_v = [&](int tt) {
#pragma unroll
      for (int db = 0; db < 4; ++db) {
        vlo[tt][db] = lds_read_tr16(reinterpret_cast<const bf16_t*>(vt + v_off[db][0] + tt * 16 * kTileD * 2));
        vhi[tt][db] = lds_read_tr16(reinterpret_cast<const bf16_t*>(vt + v_off[db][1] + tt * 16 * kTileD * 2));
      }
    };
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
      for (int e = 0; e < 16; ++e) s_acc[c][e] = 0.f;
    read_k(0);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      if (g < 3) {
        read_k(g + 1);
      } else {
        read_v(0);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) s_acc[g >> 1] = mfma32(kf[g][i], qreg[4 * (g & 1) + i], s_acc[g >> 1]);
      if (g < 3) {
        FA_INTERLEAVE(4, 1)
      } else {
        FA_INTERLEAVE(4, 2)
      }
      __builtin_amdgcn_sched_barrier(0);
      if (prefetch) {
        loader.load_block(k_next, sK + (buf ^ 1) * kTileElems, g);
        loader.load_block(v_next, sV + (buf ^ 1) * kTileElems, g);
      }
    }
    read_v(1);

    // ---- score mod, mask, online softmax ----
    // For the plain score the running maximum is kept on the raw dot products and the scale is
    // folded into the exponent (one FMA per element); score mods go through the log2-domain logit.
    const int kv0 = kb * BN;
    constexpr bool kPlain = (SCORE == FLEXATTN_SCORE_NONE);
    float m_tile = kNegInf;
    if (!partial) {
#pragma unroll
      for (int c = 0; c < 2; ++c) {
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          if (!kPlain) s_acc[c][e] = sm.to_log2(s_acc[c][e], q_idx, kv0 + 32 * c + acc_row(e, hh));
          m_tile = fmaxf(m_tile, s_acc[c][e]);
        }
      }
    } else {
      // the lane's kv indices come in runs of 4: kv0 + 32c + 8g + 4hh + {0..3}
      const bool has_doc = (a.mask.flags & FLEXATTN_MASK_DOC) != 0;
#pragma unroll
      for (int c = 0; c < 2; ++c) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const int j0 = kv0 + 32 * c + 8 * g + 4 * hh;
          int dj[4] = {0, 0, 0, 0};
          if (has_doc) {
            const auto d4 = *reinterpret_cast<const int __attribute__((ext_vector_type(4)))*>(a.mask.doc_k + j0);
            dj[0] = d4[0]; dj[1] = d4[1]; dj[2] = d4[2]; dj[3] = d4[3];
          }
#pragma unroll
          for (int u = 0; u < 4; ++u) {
            const int e = 4 * g + u;
            float tv = kPlain ? s_acc[c][e] : sm.to_log2(s_acc[c][e], q_idx, j0 + u);
            tv = keep_elem(a.mask, q_idx, j0 + u, doc_i, dj[u]) ? tv : kNegInf;
            s_acc[c][e] = tv;
            m_tile = fmaxf(m_tile, tv);
          }
        }
      }
    }
    m_tile = half_max(m_tile);
    const float m_new = fmaxf(m_run, m_tile);
    const float m_safe = (m_new == kNegInf) ? 0.f : m_new;
    const float e_scale = kPlain ? sm.c2 : 1.0f;  // exponent = e_scale * (s - m)
    // Rescale the accumulators only when some row's maximum moved (wave-uniform test).
    if (__builtin_amdgcn_ballot_w64(m_new != m_run) != 0) {
      const float alpha = fast_exp2((m_run - m_safe) * e_scale);
      l_run *= alpha;
#pragma unroll
      for (int db = 0; db < 4; ++db)
#pragma unroll
        for (int e = 0; e < 16; ++e) o_acc[db][e] *= alpha;
      m_run = m_new;
    }
    const float neg_m = -m_safe * e_scale;
    float l_tile = 0.f;
    const bf16x2 ones2 = {(bf16_t)1.0f, (bf16_t)1.0f};
    bf16x8 p[4];
#pragma unroll
    for (int c = 0; c < 2; ++c) {
#pragma unroll
      for (int e = 0; e < 16; e += 2) {
        float p0, p1;
        if (kPlain) {
          p0 = fast_exp2(__builtin_fmaf(s_acc[c][e], e_scale, neg_m));
          p1 = fast_exp2(__builtin_fmaf(s_acc[c][e + 1], e_scale, neg_m));
        } else {
          p0 = fast_exp2(s_acc[c][e] + neg_m);
          p1 = fast_exp2(s_acc[c][e + 1] + neg_m);
        }
        bf16x2 pk = pack_bf16(p0, p1);
        l_tile = __builtin_amdgcn_fdot2_f32_bf16(pk, ones2, l_tile, false);  // sums what P V will use
        p[2 * c + (e >> 3)][e & 7] = pk[0];
        p[2 * c + (e >> 3)][(e & 7) + 1] = pk[1];
      }
    }
    l_run += l_tile;

    // ---- O^T += V^T P^T ----
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int tt = 0; tt < 4; ++tt) {
      if (tt < 2) read_v(tt + 2);
#pragma unroll
      for (int db = 0; db < 4; ++db) o_acc[db] = mfma32(join_tr(vlo[tt][db], vhi[tt][db]), p[tt], o_acc[db]);
      if (tt < 2) { FA_INTERLEAVE(4, 2) }
      __builtin_amdgcn_sched_barrier(0);
    }

    kb_cur = kb_nxt; kb_nxt = kb_n2; kb_n2 = kb_n3;
    st_cur = st_nxt; st_nxt = st_n2;
    wait_vmem_all();
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
    a.m[r] = (SCORE == FLEXATTN_SCORE_NONE) ? m_run * a.sm_scale : m_run * kLn2;  // natural units
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
