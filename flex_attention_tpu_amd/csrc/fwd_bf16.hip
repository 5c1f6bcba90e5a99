// Flex-attention forward, bf16, head dim 128 (generated streams and compiled loop) and 256 (compiled loop), gfx950.
//
// One work-group = 4 waves = one 128-row Q tile of one (batch, head); each wave owns 32 q rows.
// The kernel works on S^T = K Q^T so that one lane holds one q row's scores: softmax statistics
// stay lane-private apart from one exchange between the two 32-lane halves.  K/V tiles of 64 rows
// are double-buffered in LDS by LDS-direct loads issued one tile ahead; P goes straight from the
// QK accumulators to the B operand of the PV MFMA (O^T = V^T P^T); V^T is fetched with
// transposing LDS reads.
#include <cstdlib>

#include "fa_common.hpp"
#include "launch.hpp"
#include "tile_io.hpp"

// registers of the generated run loop (gen_fwd_tile.py): v[66:199], a[192:255], s[60:100]
#define FA_FWD_RUN_VGPRS "v66", "v67", "v68", "v69", "v70", "v71", "v72", "v73", "v74", "v75", "v76", "v77", "v78", "v79", "v80", \
  "v81", "v82", "v83", "v84", "v85", "v86", "v87", "v88", "v89", "v90", "v91", "v92", "v93", "v94", "v95", \
  "v96", "v97", "v98", "v99", "v100", "v101", "v102", "v103", "v104", "v105", "v106", "v107", "v108", "v109", \
  "v110", "v111", "v112", "v113", "v114", "v115", "v116", "v117", "v118", "v119", "v120", "v121", "v122", \
  "v123", "v124", "v125", "v126", "v127", "v128", "v129", "v130", "v131", "v132", "v133", "v134", "v135", \
  "v136", "v137", "v138", "v139", "v140", "v141", "v142", "v143", "v144", "v145", "v146", "v147", "v148", \
  "v149", "v150", "v151", "v152", "v153", "v154", "v155", "v156", "v157", "v158", "v159", "v160", "v161", \
  "v162", "v163", "v164", "v165", "v166", "v167", "v168", "v169", "v170", "v171", "v172", "v173", "v174", \
  "v175", "v176", "v177", "v178", "v179", "v180", "v181", "v182", "v183", "v184", "v185", "v186", "v187", \
  "v188", "v189", "v190", "v191", "v192", "v193", "v194", "v195", "v196", "v197", "v198", "v199", "a192", \
  "a193", "a194", "a195", "a196", "a197", "a198", "a199", "a200", "a201", "a202", "a203", "a204", "a205", \
  "a206", "a207", "a208", "a209", "a210", "a211", "a212", "a213", "a214", "a215", "a216", "a217", "a218", \
  "a219", "a220", "a221", "a222", "a223", "a224", "a225", "a226", "a227", "a228", "a229", "a230", "a231", \
  "a232", "a233", "a234", "a235", "a236", "a237", "a238", "a239", "a240", "a241", "a242", "a243", "a244", \
  "a245", "a246", "a247", "a248", "a249", "a250", "a251", "a252", "a253", "a254", "a255"
#define FA_FWD_RUN_SGPRS "s60", "s61", "s62", "s63", "s64", "s65", "s66", "s67", "s68", "s69", "s70", "s71", \
  "s72", "s73", "s74", "s75", "s76", "s77", "s78", "s79", "s80", "s81", "s82", "s83", "s84", "s85", "s86", \
  "s87", "s88", "s89", "s90", "s91", "s92", "s93", "s94", "s95", "s96", "s97", "s98", "s99", "s100"

#include "fwd_tile.inc"

namespace fa {

namespace fwd_cfg {
constexpr int BM = 128;  // q rows per work-group
constexpr int BN = 64;   // kv rows per step
constexpr int D = 128;
constexpr int LDS_BYTES = 4 * kTileElems * 2;  // K x2, V x2, per 128 columns of the head dimension
// plain-score kernel: 256 q rows per work item, steps of two kv tiles: (K, K, V, V) x 2 buffers, per-wave
// tables, wave counters, merged kv list, the two state rows
constexpr int MAX_LIST = 4096;       // kv tiles of a row that the merged list and the state rows in LDS hold (262144 tokens)
constexpr int PREFETCH_LIST = 1024;  // of which an item's prefetch carries this many in registers; the rest is read when the item starts
constexpr int PLAIN_LDS_BYTES = 8 * kTileElems * 2 + 4 * 16 * 4 + 16 + MAX_LIST * 4 + 2 * MAX_LIST + kDocStageBytes + kMaxSortedItems * 4;
}  // namespace fwd_cfg


// Register-resident state of the generated streams: every asm statement names it with the same
// physical-register constraints, so it stays put and the compiler keeps those registers free.
struct FwdPinned {
  f32x16 o[8];    // a[0:127]: O^T accumulators of q block 0 (4) and 1 (4)
  bf16x8 q[16];   // a[128:191]: Q^T fragments of q block 0 (8) and 1 (8)
};
#define FA_FWD_PINNED(st)                                                                                       \
  "+{a[0:15]}"(st.o[0]), "+{a[16:31]}"(st.o[1]), "+{a[32:47]}"(st.o[2]), "+{a[48:63]}"(st.o[3]),                \
      "+{a[64:79]}"(st.o[4]), "+{a[80:95]}"(st.o[5]), "+{a[96:111]}"(st.o[6]), "+{a[112:127]}"(st.o[7]),        \
      "+{a[128:131]}"(st.q[0]), "+{a[132:135]}"(st.q[1]), "+{a[136:139]}"(st.q[2]), "+{a[140:143]}"(st.q[3]),   \
      "+{a[144:147]}"(st.q[4]), "+{a[148:151]}"(st.q[5]), "+{a[152:155]}"(st.q[6]), "+{a[156:159]}"(st.q[7]),   \
      "+{a[160:163]}"(st.q[8]), "+{a[164:167]}"(st.q[9]), "+{a[168:171]}"(st.q[10]), "+{a[172:175]}"(st.q[11]), \
      "+{a[176:179]}"(st.q[12]), "+{a[180:183]}"(st.q[13]), "+{a[184:187]}"(st.q[14]), "+{a[188:191]}"(st.q[15])

// Head dimension 128 NP: a row of K or V is NP panels of 128 columns, each panel of a 64-row tile one LDS tile
// (tile_io.hpp) at [buffer][panel]; the contraction of S runs over the panels, O^T has four accumulators per panel.
template <int SCORE, int NP>
__global__ __launch_bounds__(256, NP == 1 ? 2 : 1) void fwd_bf16_kernel(FwdArgs a) {
  using namespace fwd_cfg;
  constexpr int D = 128 * NP;
  extern __shared__ __attribute__((aligned(1024))) char smem_raw[];
  bf16_t* sK = reinterpret_cast<bf16_t*>(smem_raw);
  bf16_t* sV = sK + 2 * NP * kTileElems;

  const int nQ = a.Sq / BM;
  const int nK = a.map.nk;
  const int n_wg = a.B * a.Hq * nQ;
  const int wg = xcd_remap(blockIdx.x, n_wg);
  const int bh = wg / nQ;
  const int qb = nQ - 1 - (wg % nQ);  // longest rows first under causal masks
  const int b = bh / a.Hq;
  const MaskArgs mk = mask_of_batch(a.mask, b, a.Sq, a.Sk);
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
  sm.init(a.score, a.sm_scale, h, b);

  // Q^T as B operand: lane holds q row l32, 8 consecutive d per k-step.
  bf16x8 qreg[8 * NP];
#pragma unroll
  for (int ks = 0; ks < 8 * NP; ++ks)
    qreg[ks] = *reinterpret_cast<const bf16x8*>(Qg + (size_t)q_local * D + ks * 16 + hh * 8);

  const int n_tiles = a.map.cnt[qb];
  const int* tile_idx = a.map.idx + (size_t)qb * nK;
  const uint8_t* tile_state = a.map.state + (size_t)qb * nK;

  int doc_i = 0;
  if (mk.flags & FLEXATTN_MASK_DOC) doc_i = mk.doc_q[q_idx];

  f32x16 o_acc[4 * NP];
#pragma unroll
  for (int i = 0; i < 4 * NP; ++i)
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
  TileLoader<4, D> loader;
  loader.init(__builtin_amdgcn_readfirstlane(w), lane);
  if (n_tiles > 0) {
    const int kb0 = __builtin_amdgcn_readfirstlane(kb_cur);
#pragma unroll
    for (int pn = 0; pn < NP; ++pn) {
      loader.load(Kg + (size_t)kb0 * BN * D + 128 * pn, sK + pn * kTileElems);
      loader.load(Vg + (size_t)kb0 * BN * D + 128 * pn, sV + pn * kTileElems);
    }
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
    const char* kt = reinterpret_cast<const char*>(sK + buf * NP * kTileElems);
    const char* vt = reinterpret_cast<const char*>(sV + buf * NP * kTileElems);
    constexpr int NG = 4 * NP;        // stages of four MFMAs of S: g = (2 NP) c + 2 panel + half of the panel's k-steps
    constexpr int kPanel = kTileElems * 2;   // bytes
    bf16x8 kf[NG][4];
    s16x4 vlo[4][4 * NP], vhi[4][4 * NP];  // [tt][db]
    // Plain scores fetch the first half of V^T ahead of the softmax, which hides the latency; a score function's
    // own arithmetic, or the wider rows, need those registers in the softmax (the compiler spilled otherwise)
    constexpr bool kEarlyV = NP == 1 && (SCORE == FLEXATTN_SCORE_NONE || SCORE == kScoreBiasOnly);
    auto read_k = [&](int g) {
      const int c = g / (2 * NP), pn = (g % (2 * NP)) >> 1;
#pragma unroll
      for (int i = 0; i < 4; ++i)
        kf[g][i] = *reinterpret_cast<const bf16x8*>(kt + pn * kPanel + k_off[4 * (g & 1) + i] + c * 32 * kTileD * 2);
    };
    auto read_v = [&](int tt) {
#pragma unroll
      for (int db = 0; db < 4 * NP; ++db) {
        vlo[tt][db] = lds_read_tr16(reinterpret_cast<const bf16_t*>(vt + (db >> 2) * kPanel + v_off[db & 3][0] + tt * 16 * kTileD * 2));
        vhi[tt][db] = lds_read_tr16(reinterpret_cast<const bf16_t*>(vt + (db >> 2) * kPanel + v_off[db & 3][1] + tt * 16 * kTileD * 2));
      }
    };
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
      for (int e = 0; e < 16; ++e) s_acc[c][e] = 0.f;
    read_k(0);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int g = 0; g < NG; ++g) {
      if (g < NG - 1) {
        read_k(g + 1);
      } else if (kEarlyV) {
        read_v(0);
      }
      const int c = g / (2 * NP), pn = (g % (2 * NP)) >> 1;
#pragma unroll
      for (int i = 0; i < 4; ++i) s_acc[c] = mfma32(kf[g][i], qreg[8 * pn + 4 * (g & 1) + i], s_acc[c]);
      if (g < NG - 1) {
        FA_INTERLEAVE(4, 1)
      } else {
        FA_INTERLEAVE(4, 2 * NP)
      }
      __builtin_amdgcn_sched_barrier(0);
      if (prefetch) {   // (stage g copies block g % 4 of panel g / 4 of the next K and V tiles)
        loader.load_block(k_next + 128 * (g >> 2), sK + ((buf ^ 1) * NP + (g >> 2)) * kTileElems, g & 3);
        loader.load_block(v_next + 128 * (g >> 2), sV + ((buf ^ 1) * NP + (g >> 2)) * kTileElems, g & 3);
      }
    }
    if (kEarlyV) read_v(1);

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
          if (!kPlain) {
            const int j = kv0 + 32 * c + acc_row(e, hh);
            s_acc[c][e] = sm.to_log2(s_acc[c][e], q_idx, j) + sm.bias2(q_idx, j);
          }
          m_tile = fmaxf(m_tile, s_acc[c][e]);
        }
      }
    } else {
      // the lane's kv indices come in runs of 4: kv0 + 32c + 8g + 4hh + {0..3}
      const bool has_doc = (mk.flags & FLEXATTN_MASK_DOC) != 0;
#pragma unroll
      for (int c = 0; c < 2; ++c) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const int j0 = kv0 + 32 * c + 8 * g + 4 * hh;
          int dj[4] = {0, 0, 0, 0};
          if (has_doc) {
            const auto d4 = *reinterpret_cast<const int __attribute__((ext_vector_type(4)))*>(mk.doc_k + j0);
            dj[0] = d4[0]; dj[1] = d4[1]; dj[2] = d4[2]; dj[3] = d4[3];
          }
#pragma unroll
          for (int u = 0; u < 4; ++u) {
            const int e = 4 * g + u;
            float tv = kPlain ? s_acc[c][e] : sm.to_log2(s_acc[c][e], q_idx, j0 + u) + sm.bias2(q_idx, j0 + u);
            tv = keep_elem(mk, q_idx, j0 + u, doc_i, dj[u]) ? tv : kNegInf;
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
      for (int db = 0; db < 4 * NP; ++db)
#pragma unroll
        for (int e = 0; e < 16; ++e) o_acc[db][e] *= alpha;
      m_run = m_new;
    }
    const float neg_m = -m_safe * e_scale;
    float l_tile = 0.f;
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
        l_tile += p0 + p1;  // (the fp32 values: l is the softmax denominator the backward divides by)
        p[2 * c + (e >> 3)][e & 7] = pk[0];
        p[2 * c + (e >> 3)][(e & 7) + 1] = pk[1];
      }
    }
    l_run += l_tile;

    // ---- O^T += V^T P^T ----
    __builtin_amdgcn_sched_barrier(0);
    if (!kEarlyV) {
      read_v(0);
      read_v(1);
    }
#pragma unroll
    for (int tt = 0; tt < 4; ++tt) {
      if (tt < 2) read_v(tt + 2);
#pragma unroll
      for (int db = 0; db < 4 * NP; ++db) o_acc[db] = mfma32(join_tr(vlo[tt][db], vhi[tt][db]), p[tt], o_acc[db]);
      if (tt < 2) { FA_INTERLEAVE(4 * NP, 2) }
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
  for (int db = 0; db < 4 * NP; ++db) {
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

template <int SCORE, int NP = 1>
static int launch_fwd(const FwdArgs& a, hipStream_t stream) {
  using namespace fwd_cfg;
  auto kern = fwd_bf16_kernel<SCORE, NP>;
  static hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, NP * LDS_BYTES);
  if (attr != hipSuccess) return set_error(FLEXATTN_ELAUNCH, "hipFuncSetAttribute(fwd): %s", hipGetErrorString(attr));
  const int n_wg = a.B * a.Hq * (a.Sq / BM);
  hipLaunchKernelGGL(kern, dim3(n_wg), dim3(256), NP * LDS_BYTES, stream, a);
  return check_launch("flexattn_fwd bf16");
}

#ifndef FLEXATTN_CUSTOM_ONLY
// ------------------------------------------------------------------------------------------------
// Plain score: the main loop runs inside generated asm statements (gen_fwd_tile.py).  A work item is
// a pair of 128-row q tiles of one head (q block x = tile 2 qb2 + x; wave w owns rows 32 w .. of
// each); its kv tiles are the union of the two tiles' non-empty entries of the block map's state
// rows, merged into one list in LDS.  A step is two list entries (128 kv rows); one statement
// executes a run of consecutive full steps, or one partial step with the lane's keep bits.
// Work-groups are persistent (one per CU) when persistent_ok() finds a balanced schedule.  The
// kernel has no static shared memory: the dynamic buffer starts at LDS address 0.
// ------------------------------------------------------------------------------------------------
// ALIBI: the score gets slopes[h] (j - i) added; the streams then build the accumulator input of every
// S chain, slope' (j - i) - M, with one fp32 MFMA per chain (see gen_fwd_tile.py).
// DOCS: the mask compares document ids; those of a partial step's kv tiles are staged through LDS
// (stage_doc_ids).  (A template parameter: the staging code costs the other masks registers.)
// SOFTCAP: s' = cap tanh(s / cap) is bounded by the cap, so the reference maximum is the constant cap and the
// streams track no maximum at all: Q goes in multiplied by 2 log2(e) sm_scale / cap, an S chain gives u with
// e^(2 s / cap) = 2^u, and p = 2^(-2 cap' r), r = 1 / (2^u + 1), cap' = cap log2(e).  The residuals are returned
// relative to that bound, m = cap and l = sum exp(s' - cap): m + log l is the row's logsumexp as always, which
// is all the backward kernels take from them.  (Caps up to 50 / log2(e): beyond, p could leave the range of the
// accumulation; the compiled kernel takes those.)
// KIND: 0 plain, 1 ALIBI, 2 SOFTCAP.
template <int KIND, bool DOCS>
__global__ __launch_bounds__(256, 1) void fwd_bf16_d128_plain_kernel(FwdArgs a) {
  using namespace fwd_cfg;
  constexpr bool ALIBI = KIND == 1;
  constexpr bool SOFTCAP = KIND == 2;
  extern __shared__ __attribute__((aligned(1024))) char smem_raw[];
  bf16_t* sT = reinterpret_cast<bf16_t*>(smem_raw);  // buffer b: K tile 0, K tile 1, V tile 0, V tile 1
  unsigned* sTbl = reinterpret_cast<unsigned*>(sT + 8 * kTileElems);
  int* sCnt = reinterpret_cast<int*>(sTbl + 4 * 16);
  int* sList = sCnt + 4;
  unsigned char* sStA = reinterpret_cast<unsigned char*>(sList + MAX_LIST);
  unsigned char* sStB = sStA + MAX_LIST;

  const int nQ = a.Sq / BM;
  const int nQ2 = (nQ + 1) >> 1;
  const int nK = a.map.nk;
  const int n_wg = a.B * a.Hq * nQ2;
  const int tid = threadIdx.x;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  const int l32 = lane & 31;
  const int hh = lane >> 5;
  const int q_local = w * 32 + l32;

  TileLoader<4> loader;
  loader.init(w, lane);
  const int r_sw = swz(l32);
  const int t_row = 4 * hh + ((lane & 15) >> 2);
  const int t_chunk = 2 * ((lane & 31) >> 4) + ((lane & 3) >> 1);
  const int t_half = 4 * (lane & 1);
  const unsigned base0 = (unsigned)(size_t)sT;
  // Byte addresses of the lane's operand fragments in LDS step buffer 0 (K half-tile 0); the run
  // loop flips them between the two buffers together with `buf`, across items too.
  unsigned ra[8], ta[8];
#pragma unroll
  for (int ks = 0; ks < 8; ++ks) ra[ks] = base0 + (unsigned)(l32 * kTileD + (((2 * ks + hh) ^ r_sw) << 3)) * 2u;
#pragma unroll
  for (int i = 0; i < 8; ++i)
    ta[i] = base0 + (unsigned)(tile_off(t_row + 8 * (i & 1), 4 * (i >> 1) + t_chunk) + t_half) * 2u;
  int buf = 0;

  bool resident = false;  // the item's first step was already copied into buffer `buf` by the previous item's last step

  // (opaque(): addresses derived from its result are computed where they are used instead of once
  // before the item loop, where they would have to be kept through every run)
  auto opaque = [](int x) {
    asm volatile("" : "+v"(x));
    return x;
  };
  // Everything an item needs from global memory before its first step, fetched while the previous
  // item runs (plain loads whose values are not touched until that item's last run).
  constexpr int kListRegs = PREFETCH_LIST / 256;
  static_assert(kListRegs <= 4, "the packed state words hold four tiles per lane");
  struct ItemRegs {
    RowBlock q[2];      // the wave's 32 Q rows of each q tile (full-row layout, see rows_load)
    int doc[2];
    int klo[2], khi[2]; // (DOCS) first and last kv position that carries the row's document id, where known
    unsigned sa, sb;    // byte j: state of kv tile tid + 256 j in the state row of q tile 0 / 1
    unsigned head;      // states of kv tile `lane` in both rows: where the merged list starts
  };
  const int n_items = n_wg / (int)gridDim.x;
  const PersistentPlan plan = persistent_plan((int)blockIdx.x, n_wg, nQ2);
  const int group = a.Hq / a.Hkv;
  const float inv_group = 1.0f / (float)group;
  // under document masks a persistent work-group takes its items from the longest-first schedule (sorted_items)
  const bool sorted = DOCS && gridDim.x != (unsigned)n_wg;
  int* sItems = reinterpret_cast<int*>(sStB + MAX_LIST) + 4 * 128;
  if (DOCS && sorted)
    sorted_items([&](int t) { return a.map.cnt[2 * t] + (2 * t + 1 < nQ ? a.map.cnt[2 * t + 1] : 0); }, nQ2, n_wg / nQ2,
                 group, (int)blockIdx.x, n_items, tid, reinterpret_cast<int*>(smem_raw), sItems);
  auto geometry = [&](int item, int& bh, int& qb2) {
    if (DOCS && sorted) {
      const int v = sItems[item];
      bh = v >> 16;
      qb2 = v & 0xffff;
      return;
    }
    persistent_item(plan, (int)blockIdx.x, item, (int)gridDim.x, n_wg, nQ2, bh, qb2);
    if (gridDim.x == (unsigned)n_wg) qb2 = nQ2 - 1 - qb2;  // one item each: longest first
  };
  // (batch, kv head) pair of a (batch, q head) pair: bh / group, exact for the small numbers involved
  auto kv_pair = [&](int bh) { return group == 1 ? bh : (int)(((float)bh + 0.5f) * inv_group); };
  // (DOCS) document arrays given per batch entry: the rows of the entry of a (batch, q head) pair
  auto doc_rows = [&](int bh, int S) { return (DOCS && a.mask.doc_batched) ? (size_t)(bh / a.Hq) * (size_t)S : (size_t)0; };
  auto fetch = [&](int item, ItemRegs& r) {
    int bh, qb2;
    geometry(item, bh, qb2);
    const size_t dq_rows = doc_rows(bh, a.Sq);
    const int tid_here = opaque(tid);
    const int lane_here = tid_here & 63;
    const int row_here = (tid_here >> 6) * 32 + (lane_here & 31);
    const int w_here = tid_here >> 6;
    r.sa = r.sb = r.head = 0u;
#pragma unroll
    for (int x = 0; x < 2; ++x) {
      const int qb = min(2 * qb2 + x, nQ - 1);  // (a missing second tile repeats the first; nothing of it is stored)
      rows_load(r.q[x], static_cast<const bf16_t*>(a.q) + ((size_t)bh * a.Sq + (size_t)qb * BM + w_here * 32) * D, lane_here);
      r.doc[x] = (a.mask.flags & FLEXATTN_MASK_DOC) ? a.mask.doc_q[dq_rows + qb * BM + row_here] : 0;
      if constexpr (DOCS) {
        const bool ranged = a.mask.doc_q_range != nullptr;
        r.klo[x] = ranged ? a.mask.doc_q_range[2 * (dq_rows + qb * BM + row_here)] : 0;
        r.khi[x] = ranged ? a.mask.doc_q_range[2 * (dq_rows + qb * BM + row_here) + 1] : 0;
      }
      const uint8_t* row = a.map.state + (size_t)qb * nK;
      const bool valid = 2 * qb2 + x < nQ;
      unsigned packed = 0u;
#pragma unroll
      for (int j = 0; j < kListRegs; ++j) {
        const int t = tid_here + 256 * j;
        const unsigned v = (valid && t < nK) ? row[t] : 0u;
        packed |= v << (8 * j);
      }
      if (x == 0) r.sa = packed; else r.sb = packed;
      const unsigned hv = (valid && lane_here < nK) ? row[lane_here] : 0u;
      r.head |= hv << (8 * x);
    }
  };
  // What is left of an item's fetched values once its Q^T fragments sit in their registers.
  struct ItemHead {
    int doc[2];
    int klo[2], khi[2];
    unsigned sa, sb;
  };
  FwdPinned st;
  // Q goes in multiplied by sm_scale * log2(e): the streams' scores are then in the log2 domain
  const float cap2 = SOFTCAP ? a.score.cap * kLog2e : 0.f;
  const float c2 = SOFTCAP ? 2.0f * kLog2e * a.sm_scale / a.score.cap : a.sm_scale * kLog2e;
  auto scaled = [c2](unsigned two) {
    const float lo = __builtin_bit_cast(float, two << 16) * c2;
    const float hi = __builtin_bit_cast(float, two & 0xffff0000u) * c2;
    return __builtin_bit_cast(unsigned, pack_bf16(lo, hi));
  };
  // (`stage`: the wave's 16 KB of a free LDS step buffer)
  auto consume = [&](const ItemRegs& r, ItemHead& c, char* stage) {
    u32x4 q0[8], q1[8];
    const int lane_here = opaque(lane);
    rows_to_fragments(r.q[0], stage, lane_here, q0);
    rows_to_fragments(r.q[1], stage + 8192, lane_here, q1);
#define FA_PUT(KS, Q0, Q1)                                                                                        \
  asm volatile(FA_FWD_PUT_##KS                                                                                    \
               : "={" Q0 "}"(st.q[KS]), "={" Q1 "}"(st.q[8 + KS])                                                 \
               : "v"(scaled(q0[KS][0])), "v"(scaled(q0[KS][1])), "v"(scaled(q0[KS][2])), "v"(scaled(q0[KS][3])),  \
                 "v"(scaled(q1[KS][0])), "v"(scaled(q1[KS][1])), "v"(scaled(q1[KS][2])), "v"(scaled(q1[KS][3])));
    FA_PUT(0, "a[128:131]", "a[160:163]") FA_PUT(1, "a[132:135]", "a[164:167]") FA_PUT(2, "a[136:139]", "a[168:171]")
    FA_PUT(3, "a[140:143]", "a[172:175]") FA_PUT(4, "a[144:147]", "a[176:179]") FA_PUT(5, "a[148:151]", "a[180:183]")
    FA_PUT(6, "a[152:155]", "a[184:187]") FA_PUT(7, "a[156:159]", "a[188:191]")
#undef FA_PUT
    c.doc[0] = r.doc[0];
    c.doc[1] = r.doc[1];
    if constexpr (DOCS) {
      c.klo[0] = r.klo[0]; c.klo[1] = r.klo[1];
      c.khi[0] = r.khi[0]; c.khi[1] = r.khi[1];
    }
    c.sa = r.sa;
    c.sb = r.sb;
  };

  ItemRegs pre;
  ItemHead cur;
  fetch(0, pre);
  consume(pre, cur, reinterpret_cast<char*>(sT + 4 * kTileElems) + w * 16384);
  for (int item = 0; item < n_items; ++item) {
    int bh, qb2;
    geometry(item, bh, qb2);
    const bf16_t* Kg = static_cast<const bf16_t*>(a.k) + ((size_t)kv_pair(bh) * a.Sk) * D;
    const bf16_t* Vg = static_cast<const bf16_t*>(a.v) + ((size_t)kv_pair(bh) * a.Sk) * D;
    if (item > 0) __syncthreads();  // the previous item's list and state rows are dead from here

    // the two state rows into LDS, then the merged list of kv tiles that are non-empty for either
    // q tile, in ascending order (ballot compaction per wave, wave offsets through LDS)
    const int tid_p = opaque(tid);  // (fresh per item: see opaque())
#pragma unroll
    for (int j = 0; j < kListRegs; ++j) {
      const int t = tid_p + 256 * j;
      if (t < nK) {
        sStA[t] = (unsigned char)((cur.sa >> (8 * j)) & 0xffu);
        sStB[t] = (unsigned char)((cur.sb >> (8 * j)) & 0xffu);
      }
    }
    int n_list = 0;
    auto append = [&](bool present, int t) {   // tiles t of all 256 threads, in thread order, behind the list so far
      const unsigned long long mask = __ballot(present);
      if (lane == 0) sCnt[w] = __builtin_popcountll(mask);
      __syncthreads();
      int off = n_list;
      for (int ww = 0; ww < 4; ++ww) {
        const int cw = sCnt[ww];
        if (ww < w) off += cw;
        n_list += cw;
      }
      if (present) sList[off + __builtin_popcountll(mask & ((1ull << lane) - 1ull))] = t;
      __syncthreads();
    };
#pragma unroll
    for (int j = 0; j < kListRegs; ++j) {
      if (256 * j < nK) {
        const int t = tid_p + 256 * j;
        append(t < nK && (((cur.sa | cur.sb) >> (8 * j)) & 0xffu) != 0u, t);
      }
    }
    if (nK > PREFETCH_LIST) {
      // rows longer than the prefetched part (more than 65536 tokens): the rest of the two state rows straight
      // from global memory (an item is then thousands of steps long: the wait does not show)
      const int qa = min(2 * qb2, nQ - 1), qb_ = min(2 * qb2 + 1, nQ - 1);
      const bool valid_b = 2 * qb2 + 1 < nQ;
      const uint8_t* row_a = a.map.state + (size_t)qa * nK;
      const uint8_t* row_b = a.map.state + (size_t)qb_ * nK;
      for (int base = PREFETCH_LIST; base < nK; base += 256) {
        const int t = base + tid_p;
        unsigned sa = 0u, sb = 0u;
        if (t < nK) {
          sa = row_a[t];
          sb = valid_b ? row_b[t] : 0u;
          sStA[t] = (unsigned char)sa;
          sStB[t] = (unsigned char)sb;
        }
        append((sa | sb) != 0u, t);
      }
    }
    n_list = __builtin_amdgcn_readfirstlane(n_list);
    const int n_steps = (n_list + 1) >> 1;

    asm volatile(FA_FWD_ZERO_ACC
                 : "={a[0:15]}"(st.o[0]), "={a[16:31]}"(st.o[1]), "={a[32:47]}"(st.o[2]), "={a[48:63]}"(st.o[3]),
                   "={a[64:79]}"(st.o[4]), "={a[80:95]}"(st.o[5]), "={a[96:111]}"(st.o[6]), "={a[112:127]}"(st.o[7]));
    const int doc_i[2] = {cur.doc[0], cur.doc[1]};
    // (DOCS) with sorted kv ids the keys of a row's document are one interval: the keep bits of a partial tile
    // then have a closed form (keep_bits32_range) and no ids are read
    const bool ranged = DOCS && a.mask.doc_q_range != nullptr && keep_bits_have_range(a.mask);
    const int q_idx[2] = {(2 * qb2) * BM + q_local, (2 * qb2 + 1) * BM + q_local};
    // softmax state of the lane's two q rows (log2 domain): reference maximum M, running maximum
    // relative to it, sum of 2^(score - M)
    // (softcap: the reference is the constant cap and the streams leave M and Mt alone)
    float M[2] = {cap2, cap2}, Mt[2] = {SOFTCAP ? 0.f : kNegInf, SOFTCAP ? 0.f : kNegInf}, L[2] = {0.f, 0.f};
    // operands of the fp32 MFMA that makes the S chains' accumulator input under a position bias
    // (addv: -M of the lane's q row in lanes 0-31, which the streams keep up to date; the slope in the others)
    const float a2 = ALIBI ? a.score.slopes[bh % a.Hq] * kLog2e : 0.f;
    const float aone = hh ? (float)l32 : 1.f;
    const float mulv = hh ? 0.f : a2;
    float addv[2] = {hh ? a2 : 0.f, hh ? a2 : 0.f};

    // entry e of the list in the order the steps take it: ascending kv tiles; descending under a position
    // bias, which (slopes are positive) is largest at the last key, so that the running maximum settles early
    auto list_at = [&](int e) { return sList[ALIBI ? n_list - 1 - e : e]; };
    auto entry = [&](int e) { return list_at(e < n_list ? e : n_list - 1); };
    if (n_list > 0 && !resident) {
      // first step into the current buffer (a missing second entry repeats the first: finite data, masked out)
      const int ka = __builtin_amdgcn_readfirstlane(entry(0));
      const int kbb = __builtin_amdgcn_readfirstlane(entry(1));
      bf16_t* dst = sT + (size_t)buf * 4 * kTileElems;
      loader.load(Kg + (size_t)ka * BN * D, dst);
      loader.load(Kg + (size_t)kbb * BN * D, dst + kTileElems);
      loader.load(Vg + (size_t)ka * BN * D, dst + 2 * kTileElems);
      loader.load(Vg + (size_t)kbb * BN * D, dst + 3 * kTileElems);
      wait_vmem_all();
    }
    resident = false;
    unsigned* tbl = sTbl + w * 16;
    const unsigned tbl_addr = (unsigned)(size_t)tbl;
    const unsigned lst_addr = (unsigned)(size_t)sList;
    __syncthreads();
    // The next item's data lands while this item runs.  (The last item fetches itself again: every
    // path then redefines the fetched registers, and the compiler need not merge old values in.)
    const bool has_next = item + 1 < n_items;
    int bh_n = bh, qb2_n = qb2;
    if (has_next) geometry(item + 1, bh_n, qb2_n);
    fetch(has_next ? item + 1 : item, pre);

    int it = 0;
    int kba1 = (n_list > 0) ? __builtin_amdgcn_readfirstlane(entry(2)) : 0;
    int kbb1 = (n_list > 0) ? __builtin_amdgcn_readfirstlane(entry(3)) : 0;
    // Work-group constants of the run loop, one table per wave (order: TABLE in gen_fwd_tile.py),
    // written and read by the same wave.  The "next item" entries start out as this item's own first
    // step; the run that ends the item overwrites them when the next item's list head is known.
    if (lane == 0 && n_list > 0) {
      const int ka = entry(0), kbb = entry(1);
      tbl[0] = (unsigned)n_list;
      tbl[1] = base0 + (unsigned)w * 4096u;  // LDS address of the wave's first 1 KB block in buffer 0
      tbl[2] = __builtin_bit_cast(unsigned, SOFTCAP ? -2.0f * cap2 : c2);
      tbl[3] = (unsigned)n_steps;
      tbl[4] = (unsigned)(size_t)Kg;
      tbl[5] = (unsigned)((size_t)Kg >> 32);
      tbl[6] = (unsigned)(size_t)Vg;
      tbl[7] = (unsigned)((size_t)Vg >> 32);
      tbl[8] = (unsigned)ka;
      tbl[9] = (unsigned)kbb;
      tbl[10] = (unsigned)(size_t)Kg;
      tbl[11] = (unsigned)((size_t)Kg >> 32);
      tbl[12] = (unsigned)(size_t)Vg;
      tbl[13] = (unsigned)((size_t)Vg >> 32);
      tbl[14] = 0u;
      tbl[15] = 0u;
    }
    // a step is full when both of its entries exist and are full for both q tiles
    auto entry_full = [&](int e) {
      const int k = list_at(e);
      return sStA[k] == 2 && sStB[k] == 2;
    };
    auto step_full = [&](int sidx) { return 2 * sidx + 1 < n_list && entry_full(2 * sidx) && entry_full(2 * sidx + 1); };

    while (it < n_steps) {
      const bool partial = __builtin_amdgcn_readfirstlane(step_full(it) ? 0 : 1) == 1;
      int it_end = it + 1;
      unsigned km[4] = {0u, 0u, 0u, 0u};  // keep bits of q block x, kv tile hx of the step: km[2 x + hx]
      if (partial) {
        int* sDoc = reinterpret_cast<int*>(sStB + MAX_LIST) + w * 128;  // the wave's stage for document ids
        if constexpr (DOCS) {
          if (!ranged)
            stage_doc_ids(a.mask.doc_k + doc_rows(bh, a.Sk), __builtin_amdgcn_readfirstlane(entry(2 * it)) * BN,
                          __builtin_amdgcn_readfirstlane(entry(2 * it + 1)) * BN, lane, sDoc);
        }
#pragma unroll
        for (int hx = 0; hx < 2; ++hx) {
          const int e = 2 * it + hx;
          if (e >= n_list) continue;  // missing half: all dropped
          const int k = __builtin_amdgcn_readfirstlane(list_at(e));
#pragma unroll
          for (int x = 0; x < 2; ++x) {
            const int state = __builtin_amdgcn_readfirstlane((int)(x == 0 ? sStA[k] : sStB[k]));
            if (state == 2) {
              km[2 * x + hx] = 0xffffffffu;
            } else if (state == 1) {
              if constexpr (DOCS)
                km[2 * x + hx] = ranged ? keep_bits32_range<true>(a.mask, q_idx[x], k * BN + 4 * hh, cur.klo[x], cur.khi[x])
                                        : keep_bits32_staged<true>(a.mask, q_idx[x], k * BN + 4 * hh, doc_i[x], sDoc + 64 * hx + 4 * hh);
              else
                km[2 * x + hx] = keep_bits32<true>(a.mask, q_idx[x], k * BN + 4 * hh, doc_i[x], a.mask.doc_k);
            }
          }
        }
      } else {
        // the run of full steps ends before the next partial one: lanes look 64 steps ahead at a time
        bool found = false;
        while (!found && it_end < n_steps) {
          const int j = it_end + lane;
          const bool is_partial = j < n_steps && !step_full(j);
          const unsigned long long hits = __ballot(is_partial);
          if (hits != 0ull) {
            it_end += __builtin_ctzll(hits);
            found = true;
          } else {
            it_end = (it_end + 64 < n_steps) ? it_end + 64 : n_steps;
          }
        }
      }
      it_end = __builtin_amdgcn_readfirstlane(it_end);
      const int partial_flag = partial ? 1 : 0;
      if (it_end == n_steps && has_next) {
        // The run ends the item: its last step copies the next item's first step, if that item's
        // list starts within kv tiles 0..63 (every wave fetched those states).  The fetched values
        // are first touched here, an item's length after their loads were issued.
        int ka_n = -1, kb_n = -1;
        if constexpr (ALIBI) {
          // the next item's list is walked from its end: its last two tiles, from the packed state words
          // (lane tid of the work-group holds tiles tid + 256 j), wave maxima exchanged through LDS
          // (rows longer than the prefetched part: the end of the list is not among the fetched states; the next
          // item then loads its first step itself)
          int top1 = -1, top2 = -1;
          if (nK <= PREFETCH_LIST) {
#pragma unroll
            for (int j = 0; j < kListRegs; ++j) {
              unsigned long long m = __ballot((((pre.sa | pre.sb) >> (8 * j)) & 0xffu) != 0u && tid + 256 * j < nK);
              while (m != 0ull && top2 < w * 64 + 256 * j) {  // (tiles of a later j are larger: they replace both)
                const int t = w * 64 + 256 * j + 63 - __builtin_clzll(m);
                m &= ~(1ull << (63 - __builtin_clzll(m)));
                if (t > top1) { top2 = top1; top1 = t; } else if (t > top2) { top2 = t; }
              }
            }
          }
          if (lane == 0) sCnt[w] = (top1 & 0xffff) | (top2 << 16);
          __syncthreads();
#pragma unroll
          for (int ww = 0; ww < 4; ++ww) {
            const int v = sCnt[ww];
            const int c1 = (int)(short)(v & 0xffff), c2x = v >> 16;
            if (c1 > ka_n) { kb_n = ka_n > c2x ? ka_n : c2x; ka_n = c1; } else if (c1 > kb_n) { kb_n = c1; }
          }
          __syncthreads();
          if (kb_n < 0) kb_n = ka_n;
        } else {
          // ... if that item's list starts within kv tiles 0..63 (every wave fetched those states)
          const unsigned long long mask = __ballot(lane < nK && pre.head != 0u);
          const int cnt = __builtin_popcountll(mask);
          if (cnt >= 2 || (cnt == 1 && nK <= 64)) {
            ka_n = __builtin_ctzll(mask);
            kb_n = cnt >= 2 ? __builtin_ctzll(mask & (mask - 1ull)) : ka_n;
          }
        }
        if (ka_n >= 0) {
          const bf16_t* Kg_n = static_cast<const bf16_t*>(a.k) + ((size_t)kv_pair(bh_n) * a.Sk) * D;
          const bf16_t* Vg_n = static_cast<const bf16_t*>(a.v) + ((size_t)kv_pair(bh_n) * a.Sk) * D;
          if (lane == 0) {
            tbl[8] = (unsigned)ka_n;
            tbl[9] = (unsigned)kb_n;
            tbl[10] = (unsigned)(size_t)Kg_n;
            tbl[11] = (unsigned)((size_t)Kg_n >> 32);
            tbl[12] = (unsigned)(size_t)Vg_n;
            tbl[13] = (unsigned)((size_t)Vg_n >> 32);
          }
          resident = true;
        }
      }
      // no scalar operands (see gen_fwd_tile.py): the loop state travels in VGPRs
#define FA_FWD_CALL(RUN, OUT_MORE, CLOB_MORE, ...)                                                                         \
  asm volatile(RUN                                                                                               \
               : FA_FWD_PINNED(st), [it] "+v"(it), [kba1] "+v"(kba1), [kbb1] "+v"(kbb1), [buf] "+v"(buf),         \
                 [M0] "+v"(M[0]), [M1] "+v"(M[1]), [Mt0] "+v"(Mt[0]), [Mt1] "+v"(Mt[1]), [L0] "+v"(L[0]),         \
                 [L1] "+v"(L[1]), [r0] "+v"(ra[0]), [r1] "+v"(ra[1]), [r2] "+v"(ra[2]), [r3] "+v"(ra[3]),         \
                 [r4] "+v"(ra[4]), [r5] "+v"(ra[5]), [r6] "+v"(ra[6]), [r7] "+v"(ra[7]), [t0] "+v"(ta[0]),        \
                 [t1] "+v"(ta[1]), [t2] "+v"(ta[2]), [t3] "+v"(ta[3]), [t4] "+v"(ta[4]), [t5] "+v"(ta[5]),        \
                 [t6] "+v"(ta[6]), [t7] "+v"(ta[7]) OUT_MORE                                                     \
               : [it_end] "v"(it_end), [partial] "v"(partial_flag), [tbl] "v"(tbl_addr), [lst] "v"(lst_addr),     \
                 [g0] "v"(loader.goff[0]), [g1v] "v"(loader.goff[1]), [g2] "v"(loader.goff[2]),                  \
                 [g3] "v"(loader.goff[3]), [m0] "v"(km[0]), [m1] "v"(km[1]), [m2] "v"(km[2]), [m3] "v"(km[3]),    \
                 ##__VA_ARGS__                                                                                   \
               : "memory", "scc", "vcc", "m0", FA_FWD_RUN_SGPRS, FA_FWD_RUN_VGPRS CLOB_MORE)
#define FA_FWD_ADDV , [addv0] "+v"(addv[0]), [addv1] "+v"(addv[1])
#define FA_FWD_ALIBI_CLOBBERS , "s101", "v200", "v201"
      if constexpr (ALIBI) {
        const int ka0 = __builtin_amdgcn_readfirstlane(entry(2 * it));
        const int kb0 = __builtin_amdgcn_readfirstlane(entry(2 * it + 1));
        FA_FWD_CALL(FA_FWD_RUN_ALIBI, FA_FWD_ADDV, FA_FWD_ALIBI_CLOBBERS, [aone] "v"(aone), [mulv] "v"(mulv), [iq] "v"(q_idx[0]), [ka0] "v"(ka0),
                    [kb0] "v"(kb0));
      } else if constexpr (SOFTCAP) {
        FA_FWD_CALL(FA_FWD_RUN_SOFTCAP, , );
      } else {
        FA_FWD_CALL(FA_FWD_RUN, , );
      }
#undef FA_FWD_ADDV
#undef FA_FWD_ALIBI_CLOBBERS
#undef FA_FWD_CALL
      it = __builtin_amdgcn_readfirstlane(it);
      buf = __builtin_amdgcn_readfirstlane(buf);
    }

    // ---- item epilogue ----
    // The next item's Q^T fragments go into their registers before this item's stores are issued
    // (their loads are long done; behind the stores the wait would include the stores).
    // (Buffer `buf` may hold the next item's first step: the other one is free.)
    char* stage = reinterpret_cast<char*>(sT + (size_t)(buf ^ 1) * 4 * kTileElems) + w * 16384;
    consume(pre, cur, stage);

    // O = O^T / l as bf16 rows, staged through the same wave-private LDS (16-byte chunks XOR-swizzled
    // by row) so that every store instruction writes four complete 256-byte rows; exact (l, m) from
    // the reference-maximum bookkeeping.
    {
      const int lane_here = opaque(lane);
      const int row_here = lane_here & 31;
      const unsigned wr = (unsigned)row_here * 256u + 8u * (unsigned)(lane_here >> 5);
      float inv[2];
#pragma unroll
      for (int x = 0; x < 2; ++x) {
        const float l_tot = half_sum(L[x]);
        const float mt_row = half_max(Mt[x]);  // (the streams keep the running maximum per lane)
        inv[x] = (l_tot > 0.f) ? 1.0f / l_tot : 0.f;
        if (2 * qb2 + x < nQ && a.l != nullptr && lane_here < 32) {
          const size_t r = (size_t)bh * a.Sq + q_idx[x];
          // sums were taken against the reference maximum M: move them to the true maximum M + Mt
          a.l[r] = (l_tot > 0.f) ? l_tot * fast_exp2(-mt_row) : 0.f;
          a.m[r] = (l_tot > 0.f) ? (M[x] + mt_row) * kLn2 : kNegInf;  // natural units
        }
      }
#define FA_GET(T, SRC, REG)                                                                                        \
  {                                                                                                                \
    float xv[16];                                                                                                  \
    asm volatile(FA_FWD_GET_ACC_##T                                                                                \
                 : "=v"(xv[0]), "=v"(xv[1]), "=v"(xv[2]), "=v"(xv[3]), "=v"(xv[4]), "=v"(xv[5]), "=v"(xv[6]),      \
                   "=v"(xv[7]), "=v"(xv[8]), "=v"(xv[9]), "=v"(xv[10]), "=v"(xv[11]), "=v"(xv[12]), "=v"(xv[13]),  \
                   "=v"(xv[14]), "=v"(xv[15])                                                                      \
                 : "{" REG "}"(SRC));                                                                              \
    const float sc_ = inv[T / 4];                                                                                  \
    _Pragma("unroll") for (int g = 0; g < 4; ++g) {                                                                \
      const bf16x2 lo = pack_bf16(xv[4 * g] * sc_, xv[4 * g + 1] * sc_);                                           \
      const bf16x2 hi = pack_bf16(xv[4 * g + 2] * sc_, xv[4 * g + 3] * sc_);                                       \
      const bf16x4 out = {lo[0], lo[1], hi[0], hi[1]};                                                             \
      *reinterpret_cast<bf16x4*>(stage + (T / 4) * 8192 + wr +                                                     \
                                 (unsigned)(((4 * (T % 4) + g) ^ (row_here & 15)) << 4)) = out;                    \
    }                                                                                                              \
  }
      FA_GET(0, st.o[0], "a[0:15]") FA_GET(1, st.o[1], "a[16:31]") FA_GET(2, st.o[2], "a[32:47]")
      FA_GET(3, st.o[3], "a[48:63]") FA_GET(4, st.o[4], "a[64:79]") FA_GET(5, st.o[5], "a[80:95]")
      FA_GET(6, st.o[6], "a[96:111]") FA_GET(7, st.o[7], "a[112:127]")
#undef FA_GET
      __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
      __builtin_amdgcn_wave_barrier();
      const int chunk = lane_here & 15;
#pragma unroll
      for (int x = 0; x < 2; ++x) {
        if (2 * qb2 + x < nQ) {
          bf16_t* Og = static_cast<bf16_t*>(a.o) + ((size_t)bh * a.Sq + (size_t)(2 * qb2 + x) * BM + w * 32) * D;
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            const int r = 4 * i + (lane_here >> 4);
            const u32x4 v = *reinterpret_cast<const u32x4*>(stage + x * 8192 + (unsigned)r * 256u +
                                                            (unsigned)((chunk ^ (r & 15)) << 4));
            *reinterpret_cast<u32x4*>(Og + (size_t)r * D + chunk * 8) = v;
          }
        }
      }
    }
  }  // work items
}

template <int KIND, bool DOCS>
static int launch_fwd_plain_on(const FwdArgs& a, hipStream_t stream) {
  using namespace fwd_cfg;
  auto kern = fwd_bf16_d128_plain_kernel<KIND, DOCS>;
  static hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, PLAIN_LDS_BYTES);
  if (attr != hipSuccess) return set_error(FLEXATTN_ELAUNCH, "hipFuncSetAttribute(fwd): %s", hipGetErrorString(attr));
  const int nQ2 = (a.Sq / BM + 1) / 2;
  const int n_wg = a.B * a.Hq * nQ2;
  // (document masks take the longest-first schedule of sorted_items)
  const bool persistent = DOCS ? sorted_schedule_ok(n_wg, nQ2) : persistent_ok(n_wg, nQ2);
  const int grid = (persistent && n_wg > 256) ? 256 : n_wg;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(256), PLAIN_LDS_BYTES, stream, a);
  return check_launch("flexattn_fwd bf16");
}

template <int KIND>
static int launch_fwd_plain(const FwdArgs& a, hipStream_t stream) {
  return (a.mask.flags & FLEXATTN_MASK_DOC) ? launch_fwd_plain_on<KIND, true>(a, stream)
                                            : launch_fwd_plain_on<KIND, false>(a, stream);
}

#endif  // FLEXATTN_CUSTOM_ONLY

int fwd_bf16_d128(const FwdArgs& a, hipStream_t stream) {
#ifdef FLEXATTN_CUSTOM_ONLY
  // functor library of a compiled score function: the kernels with a compiled main loop only
  switch (a.score.kind) {
    case FLEXATTN_SCORE_NONE:
      return a.score.ab ? launch_fwd<kScoreBiasOnly>(a, stream) : launch_fwd<FLEXATTN_SCORE_NONE>(a, stream);
    case FLEXATTN_SCORE_CUSTOM: return launch_fwd<FLEXATTN_SCORE_CUSTOM>(a, stream);
  }
  return set_error(FLEXATTN_ENOTSUP, "this functor library holds the plain and the compiled score function only (kind %d asked)", a.score.kind);
#else
  // The generated-stream kernel (one wave per SIMD, 64 q rows per wave) keeps the state rows and the
  // merged kv list in LDS, hence the bound on the list length.
  // and has no additive bias.
  // Its scale is folded into bf16 Q, which must not cost the logits their accuracy (folded_scale_ok).  (A variant of
  // the stream that scales the raw product instead, one fma per score, was correct but slower than the compiled
  // kernel where it is needed: 0.76 against 0.68 ms on B=4, H=32, S=4096 at sm_scale = 1, where logits of standard
  // deviation 11 also move the reference maximum often.)
  const float fold = a.score.kind == FLEXATTN_SCORE_SOFTCAP ? 2.0f * kLog2e * a.sm_scale / a.score.cap : a.sm_scale * kLog2e;
  const bool stream_ok = !(a.flags & FLEXATTN_FLAG_COMPILED_LOOP) && a.map.nk <= fwd_cfg::MAX_LIST && a.score.ab == nullptr;
  const bool fold_ok = folded_scale_ok(fold, a.sm_scale, 128);
  switch (a.score.kind) {
    case FLEXATTN_SCORE_NONE:
      if (a.score.ab != nullptr) return launch_fwd<kScoreBiasOnly>(a, stream);
      return stream_ok && fold_ok ? launch_fwd_plain<0>(a, stream) : launch_fwd<FLEXATTN_SCORE_NONE>(a, stream);
    case FLEXATTN_SCORE_ALIBI:
      return stream_ok && fold_ok ? launch_fwd_plain<1>(a, stream) : launch_fwd<FLEXATTN_SCORE_ALIBI>(a, stream);
    case FLEXATTN_SCORE_SOFTCAP:
      return (stream_ok && fold_ok && a.score.cap * kLog2e <= 50.f) ? launch_fwd_plain<2>(a, stream)
                                                                      : launch_fwd<FLEXATTN_SCORE_SOFTCAP>(a, stream);
    case FLEXATTN_SCORE_ALIBI_TILE: return launch_fwd<FLEXATTN_SCORE_ALIBI_TILE>(a, stream);
  }
  return set_error(FLEXATTN_EINVAL, "unknown score kind %d", a.score.kind);
#endif
}

// Head dim 256: the kernels with a compiled main loop (two 128-column panels per row), every score kind.
int fwd_bf16_d256(const FwdArgs& a, hipStream_t stream) {
  switch (a.score.kind) {
    case FLEXATTN_SCORE_NONE:
      return a.score.ab ? launch_fwd<kScoreBiasOnly, 2>(a, stream) : launch_fwd<FLEXATTN_SCORE_NONE, 2>(a, stream);
#ifdef FLEXATTN_CUSTOM_ONLY
    case FLEXATTN_SCORE_CUSTOM: return launch_fwd<FLEXATTN_SCORE_CUSTOM, 2>(a, stream);
#else
    case FLEXATTN_SCORE_ALIBI: return launch_fwd<FLEXATTN_SCORE_ALIBI, 2>(a, stream);
    case FLEXATTN_SCORE_SOFTCAP: return launch_fwd<FLEXATTN_SCORE_SOFTCAP, 2>(a, stream);
    case FLEXATTN_SCORE_ALIBI_TILE: return launch_fwd<FLEXATTN_SCORE_ALIBI_TILE, 2>(a, stream);
#endif
  }
  return set_error(FLEXATTN_ENOTSUP, "score kind %d is not in this library", a.score.kind);
}

void fwd_bf16_d128_tile(int* bq, int* bk) {
  *bq = fwd_cfg::BM;
  *bk = fwd_cfg::BN;
}

}  // namespace fa
