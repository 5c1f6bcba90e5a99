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

// registers of the generated run loop (gen_dq_tile.py): v[66:183], a[128:191], s[60:100]
#define FA_DQ_RUN_VGPRS "v66", "v67", "v68", "v69", "v70", "v71", "v72", "v73", "v74", "v75", "v76", "v77", "v78", "v79", "v80", \
  "v81", "v82", "v83", "v84", "v85", "v86", "v87", "v88", "v89", "v90", "v91", "v92", "v93", "v94", "v95", \
  "v96", "v97", "v98", "v99", "v100", "v101", "v102", "v103", "v104", "v105", "v106", "v107", "v108", "v109", \
  "v110", "v111", "v112", "v113", "v114", "v115", "v116", "v117", "v118", "v119", "v120", "v121", "v122", \
  "v123", "v124", "v125", "v126", "v127", "v128", "v129", "v130", "v131", "v132", "v133", "v134", "v135", \
  "v136", "v137", "v138", "v139", "v140", "v141", "v142", "v143", "v144", "v145", "v146", "v147", "v148", \
  "v149", "v150", "v151", "v152", "v153", "v154", "v155", "v156", "v157", "v158", "v159", "v160", "v161", \
  "v162", "v163", "v164", "v165", "v166", "v167", "v168", "v169", "v170", "v171", "v172", "v173", "v174", \
  "v175", "v176", "v177", "v178", "v179", "v180", "v181", "v182", "v183", "a128", "a129", "a130", "a131", \
  "a132", "a133", "a134", "a135", "a136", "a137", "a138", "a139", "a140", "a141", "a142", "a143", "a144", \
  "a145", "a146", "a147", "a148", "a149", "a150", "a151", "a152", "a153", "a154", "a155", "a156", "a157", \
  "a158", "a159", "a160", "a161", "a162", "a163", "a164", "a165", "a166", "a167", "a168", "a169", "a170", \
  "a171", "a172", "a173", "a174", "a175", "a176", "a177", "a178", "a179", "a180", "a181", "a182", "a183", \
  "a184", "a185", "a186", "a187", "a188", "a189", "a190", "a191"
#define FA_DQ_RUN_SGPRS "s60", "s61", "s62", "s63", "s64", "s65", "s66", "s67", "s68", "s69", "s70", "s71", \
  "s72", "s73", "s74", "s75", "s76", "s77", "s78", "s79", "s80", "s81", "s82", "s83", "s84", "s85", "s86", \
  "s87", "s88", "s89", "s90", "s91", "s92", "s93", "s94", "s95", "s96", "s97", "s98", "s99", "s100"

#include "bwd_dq_tile.inc"

namespace fa {

namespace dq_cfg {
constexpr int BM = 128;
constexpr int BN = 64;
constexpr int D = 128;
constexpr int LDS_BYTES = 4 * kTileElems * 2;  // K x2, V x2, per 128 columns of the head dimension
// plain-score kernel: steps of two kv tiles, (K, K, V, V) x 2 buffers, per-wave tables, cached kv list + states
constexpr int MAX_LIST = 4096;       // kv tiles of a row whose list and states the kernel caches in LDS (262144 tokens)
constexpr int PREFETCH_LIST = 2048;  // of which an item's prefetch carries this many in registers; the rest is read when the item starts
constexpr int PLAIN_LDS_BYTES = 8 * kTileElems * 2 + 4 * 16 * 4 + MAX_LIST * 5 + kDocStageBytes + kMaxSortedItems * 4;
}  // namespace dq_cfg


// Register-resident state of the generated streams: every asm statement names it with the same
// physical-register constraints, so it stays put and the compiler keeps those registers free.
struct DqPinned {
  f32x16 dq[4];      // a[0:63]
  bf16x8 q[8], d[8];  // a[64:95], a[96:127]
};
#define FA_DQ_PINNED(st)                                                                                      \
  "+{a[0:15]}"(st.dq[0]), "+{a[16:31]}"(st.dq[1]), "+{a[32:47]}"(st.dq[2]), "+{a[48:63]}"(st.dq[3]),          \
      "+{a[64:67]}"(st.q[0]), "+{a[68:71]}"(st.q[1]), "+{a[72:75]}"(st.q[2]), "+{a[76:79]}"(st.q[3]),         \
      "+{a[80:83]}"(st.q[4]), "+{a[84:87]}"(st.q[5]), "+{a[88:91]}"(st.q[6]), "+{a[92:95]}"(st.q[7]),         \
      "+{a[96:99]}"(st.d[0]), "+{a[100:103]}"(st.d[1]), "+{a[104:107]}"(st.d[2]), "+{a[108:111]}"(st.d[3]),   \
      "+{a[112:115]}"(st.d[4]), "+{a[116:119]}"(st.d[5]), "+{a[120:123]}"(st.d[6]), "+{a[124:127]}"(st.d[7])

// Head dimension 128 NP: a row of K or V is NP panels of 128 columns, each panel of a 64-row tile one LDS tile
// (tile_io.hpp) at [buffer][panel]; the contractions of S and dP run over the panels, dq^T has four accumulators
// per panel.
template <int SCORE, int NP>
__global__ __launch_bounds__(256, NP == 1 ? 2 : 1) void bwd_dq_bf16_kernel(BwdArgs a) {
  using namespace dq_cfg;
  constexpr int D = 128 * NP;
  constexpr int kPanel = kTileElems * 2;   // bytes
  extern __shared__ __attribute__((aligned(1024))) char smem_raw[];
  bf16_t* sK = reinterpret_cast<bf16_t*>(smem_raw);
  bf16_t* sV = sK + 2 * NP * kTileElems;

  const int nQ = a.Sq / BM;
  const int nK = a.map.nk;
  const int n_wg = a.B * a.Hq * nQ;
  const int wg = xcd_remap(blockIdx.x, n_wg);
  const int bh = wg / nQ;
  const int qb = nQ - 1 - (wg % nQ);
  const int b = bh / a.Hq;
  const MaskArgs mk = mask_of_batch(a.mask, b, a.Sq, a.Sk);
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
  sm.init(a.score, a.sm_scale, h, b);

  bf16x8 qreg[8 * NP], doreg[8 * NP];
#pragma unroll
  for (int ks = 0; ks < 8 * NP; ++ks) {
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
  if (mk.flags & FLEXATTN_MASK_DOC) doc_i = mk.doc_q[q_idx];
  float* dab_row = a.dab != nullptr ? a.dab + row * (size_t)a.Sk : nullptr;  // this lane's row of the bias gradient

  f32x16 dq_acc[4 * NP];
#pragma unroll
  for (int i = 0; i < 4 * NP; ++i)
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
  TileLoader<4, D> loader;
  loader.init(w, lane);
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
#pragma unroll
      for (int pn = 0; pn < NP; ++pn) {
        loader.load(Kg + (size_t)kbn * BN * D + 128 * pn, sK + ((buf ^ 1) * NP + pn) * kTileElems);
        loader.load(Vg + (size_t)kbn * BN * D + 128 * pn, sV + ((buf ^ 1) * NP + pn) * kTileElems);
      }
    }
    const int kv0 = kb * BN;
    const char* kt = reinterpret_cast<const char*>(sK + buf * NP * kTileElems);
    const char* vt = reinterpret_cast<const char*>(sV + buf * NP * kTileElems);

#pragma clang loop unroll_count(NP == 1 ? 2 : 1)   // (wider rows: rolled, which keeps the second block's operand loads out of the first block's registers: 1.37 -> 1.25 ms on B=4, H=16, S=4096, D=256)
    for (int c = 0; c < 2; ++c) {
      // ---- S^T and dP^T for kv rows [32c, 32c+32) ----
      f32x16 s_acc, dp_acc;
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        s_acc[e] = 0.f;
        dp_acc[e] = 0.f;
      }
#pragma unroll
      for (int pn = 0; pn < NP; ++pn) {
        bf16x8 kf[8];
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) kf[ks] = *reinterpret_cast<const bf16x8*>(kt + pn * kPanel + r_off[ks] + c * 32 * kTileD * 2);
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) s_acc = mfma32(kf[ks], qreg[8 * pn + ks], s_acc);
      }
#pragma unroll
      for (int pn = 0; pn < NP; ++pn) {
        bf16x8 vf[8];
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) vf[ks] = *reinterpret_cast<const bf16x8*>(vt + pn * kPanel + r_off[ks] + c * 32 * kTileD * 2);
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) dp_acc = mfma32(vf[ks], doreg[8 * pn + ks], dp_acc);
      }
      // K^T fragments for the dq product
      s16x4 klo[2][4 * NP], khi[2][4 * NP];
      auto read_kt = [&](int u) {
#pragma unroll
        for (int db = 0; db < 4 * NP; ++db) {
          const int off = (32 * c + 16 * u) * kTileD * 2 + (db >> 2) * kPanel;
          klo[u][db] = lds_read_tr16(reinterpret_cast<const bf16_t*>(kt + t_off[db & 3][0] + off));
          khi[u][db] = lds_read_tr16(reinterpret_cast<const bf16_t*>(kt + t_off[db & 3][1] + off));
        }
      };

      // ---- P, dS -> bf16 ----
      bf16x8 ds[2];
      auto elementwise = [&](auto masked) {
        constexpr bool MASKED = decltype(masked)::value;
        const bool has_doc = MASKED && (mk.flags & FLEXATTN_MASK_DOC) != 0;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const int j0 = kv0 + 32 * c + 8 * g + 4 * hh;
          int dj[4] = {0, 0, 0, 0};
          if (MASKED && has_doc) {
            const auto d4 = *reinterpret_cast<const int __attribute__((ext_vector_type(4)))*>(mk.doc_k + j0);
            dj[0] = d4[0]; dj[1] = d4[1]; dj[2] = d4[2]; dj[3] = d4[3];
          }
          float dsv[4];
          f32x4 gb;   // the gradient with respect to the logits themselves: what an additive bias receives
#pragma unroll
          for (int u = 0; u < 4; ++u) {
            const int e = 4 * g + u;
            const float tv = sm.to_log2(s_acc[e], q_idx, j0 + u);
            const float pe = fast_exp2(tv + sm.bias2(q_idx, j0 + u) - lse2);
            float gl = pe * (dp_acc[e] - delta);
            float gd = gl * sm.dfactor(tv, s_acc[e], q_idx, j0 + u);
            if (MASKED) {   // (selected, not multiplied: a score function may return anything at a dropped element)
              const bool keep = keep_elem(mk, q_idx, j0 + u, doc_i, dj[u]);
              gl = keep ? gl : 0.f;
              gd = keep ? gd : 0.f;
            }
            gb[u] = gl;
            dsv[u] = gd;
          }
          if (dab_row != nullptr) *reinterpret_cast<f32x4*>(dab_row + j0) = gb;
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
        for (int db = 0; db < 4 * NP; ++db) dq_acc[db] = mfma32(join_tr(klo[u][db], khi[u][db]), ds[u], dq_acc[db]);
    }

    kb_cur = kb_nxt; kb_nxt = kb_n2; kb_n2 = kb_n3;
    st_cur = st_nxt; st_nxt = st_n2;
    wait_vmem_all();
    __syncthreads();
  }

#pragma unroll
  for (int db = 0; db < 4 * NP; ++db) {
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      bf16x2 lo = pack_bf16(dq_acc[db][4 * g], dq_acc[db][4 * g + 1]);
      bf16x2 hi = pack_bf16(dq_acc[db][4 * g + 2], dq_acc[db][4 * g + 3]);
      bf16x4 out = {lo[0], lo[1], hi[0], hi[1]};
      *reinterpret_cast<bf16x4*>(dQg + (size_t)q_local * D + 32 * db + 8 * g + 4 * hh) = out;
    }
  }
}

template <int SCORE, int NP = 1>
static int launch_dq(const BwdArgs& a, hipStream_t stream) {
  using namespace dq_cfg;
  auto kern = bwd_dq_bf16_kernel<SCORE, NP>;
  static hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, NP * LDS_BYTES);
  if (attr != hipSuccess) return set_error(FLEXATTN_ELAUNCH, "hipFuncSetAttribute(dq): %s", hipGetErrorString(attr));
  const int n_wg = a.B * a.Hq * (a.Sq / BM);
  hipLaunchKernelGGL(kern, dim3(n_wg), dim3(256), NP * LDS_BYTES, stream, a);
  return check_launch("flexattn_bwd_dq bf16");
}

#ifndef FLEXATTN_CUSTOM_ONLY
// ------------------------------------------------------------------------------------------------
// Plain score: the main loop runs inside generated asm statements (gen_dq_tile.py).  A step is two
// entries of the q tile's kv list (128 kv rows); one statement executes a run of consecutive full
// steps, or one partial step with the lane's keep bits.  Work-groups are persistent (one per CU)
// when persistent_ok() finds a balanced schedule.  The kernel has no static shared memory: the
// dynamic buffer starts at LDS address 0 (the run loop toggles buffers by address bits).
// ------------------------------------------------------------------------------------------------
// ALIBI: the score gets slopes[h] (j - i) added; the streams then build the accumulator input of every
// S chain, slope' (j - i) - lse, with one fp32 MFMA per 32-key block (see gen_dq_tile.py).
// DOCS: the mask compares document ids; a persistent work-group then takes its items from the longest-first
// schedule (sorted_items).  (A template parameter: the code costs the other masks registers.)
// SOFTCAP: s' = cap tanh(s / cap).  Q goes in multiplied by 2 log2(e) sm_scale / cap, so that an S chain gives u
// with e^(2 s / cap) = 2^u; the stream turns it into r = 1 / (2^u + 1) (tanh = 1 - 2 r), the exponent
// cap' - lse - 2 cap' r (cap' = cap log2 e) and the derivative's r (1 - r); the factor 4 sm_scale that is left
// goes onto dq in the epilogue.
// EXACT: plain scores with Q unscaled in its registers; the stream turns the raw product into the exponent with one
// fma per element (c2 <q, k> - lse).  For scales too large to fold into bf16 Q (folded_scale_ok).
// KIND: 0 plain, 1 ALIBI, 2 SOFTCAP, 3 EXACT.
template <int KIND, bool DOCS>
__global__ __launch_bounds__(256, 1) void bwd_dq_bf16_d128_plain_kernel(BwdArgs a) {
  using namespace dq_cfg;
  constexpr bool ALIBI = KIND == 1;
  constexpr bool SOFTCAP = KIND == 2;
  constexpr bool EXACT = KIND == 3;
  extern __shared__ __attribute__((aligned(1024))) char smem_raw[];
  bf16_t* sT = reinterpret_cast<bf16_t*>(smem_raw);  // buffer b: K tile 0, K tile 1, V tile 0, V tile 1
  unsigned* sTbl = reinterpret_cast<unsigned*>(sT + 8 * kTileElems);
  int* sIdx = reinterpret_cast<int*>(sTbl + 4 * 16);
  unsigned char* sSt = reinterpret_cast<unsigned char*>(sIdx + MAX_LIST);

  const int nQ = a.Sq / BM;
  const int nK = a.map.nk;
  const int n_wg = a.B * a.Hq * nQ;
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

  // Everything an item needs from global memory before its first step.  It is fetched while the
  // previous item runs (plain loads whose values are not touched until then), so that an item
  // starts after one memory round trip (its first kv tiles) instead of a chain of dependent ones.
  constexpr int kListRegs = PREFETCH_LIST / 256;
  struct ItemRegs {
    RowBlock q, d;       // the wave's 32 Q / dO rows (full-row layout, see rows_load)
    float l, m, delta;
    int doc;
    int klo, khi;                  // (DOCS) first and last kv position that carries the row's document id, where known
    int n_tiles, kb0, kb1;         // list length and its first two entries
    int idx[kListRegs];            // kv list entries tid + 256 j
    unsigned char st[kListRegs];   // state of kv tile tid + 256 j in the q tile's state row
  };
  const int n_items = n_wg / (int)gridDim.x;
  const PersistentPlan plan = persistent_plan((int)blockIdx.x, n_wg, nQ);
  const int group = a.Hq / a.Hkv;
  const float inv_group = 1.0f / (float)group;
  const bool sorted = DOCS && gridDim.x != (unsigned)n_wg;
  int* sItems = reinterpret_cast<int*>(sSt + MAX_LIST) + 4 * 128;
  if (DOCS && sorted)
    sorted_items([&](int t) { return a.map.cnt[t]; }, nQ, n_wg / nQ, group, (int)blockIdx.x, n_items, tid,
                 reinterpret_cast<int*>(smem_raw), sItems);
  auto geometry = [&](int item, int& bh, int& qb) {
    if (DOCS && sorted) {
      const int v = sItems[item];
      bh = v >> 16;
      qb = v & 0xffff;
      return;
    }
    persistent_item(plan, (int)blockIdx.x, item, (int)gridDim.x, n_wg, nQ, bh, qb);
    if (gridDim.x == (unsigned)n_wg) qb = nQ - 1 - qb;  // one item each: longest first
  };
  // (batch, kv head) pair of a (batch, q head) pair: bh / group, exact for the small numbers involved
  auto kv_pair = [&](int bh) { return group == 1 ? bh : (int)(((float)bh + 0.5f) * inv_group); };
  // (DOCS) document arrays given per batch entry: the rows of the entry of a (batch, q head) pair
  auto doc_rows = [&](int bh, int S) { return (DOCS && a.mask.doc_batched) ? (size_t)(bh / a.Hq) * (size_t)S : (size_t)0; };
  auto fetch = [&](int item, ItemRegs& r) {
    int bh, qb;
    geometry(item, bh, qb);
    const size_t q_off = ((size_t)bh * a.Sq + (size_t)qb * BM + w * 32) * D;
    rows_load(r.q, static_cast<const bf16_t*>(a.q) + q_off, lane);
    rows_load(r.d, static_cast<const bf16_t*>(a.dout) + q_off, lane);
    const size_t row = (size_t)bh * a.Sq + qb * BM + q_local;
    r.l = a.l[row];
    r.m = a.m[row];
    r.delta = a.delta[row];
    const size_t dq_rows = doc_rows(bh, a.Sq);
    r.doc = (a.mask.flags & FLEXATTN_MASK_DOC) ? a.mask.doc_q[dq_rows + qb * BM + q_local] : 0;
    if constexpr (DOCS) {
      const bool have = a.mask.doc_q_range != nullptr;
      r.klo = have ? a.mask.doc_q_range[2 * (dq_rows + qb * BM + q_local)] : 0;
      r.khi = have ? a.mask.doc_q_range[2 * (dq_rows + qb * BM + q_local) + 1] : 0;
    }
    r.n_tiles = a.map.cnt[qb];
    const int* tile_idx = a.map.idx + (size_t)qb * nK;
    r.kb0 = tile_idx[0];                // (nK >= 1: always readable; meaningful only if the list is not empty)
    r.kb1 = tile_idx[nK > 1 ? 1 : 0];
    const uint8_t* tile_state = a.map.state + (size_t)qb * nK;
#pragma unroll
    for (int j = 0; j < kListRegs; ++j) {
      const int t = tid + 256 * j;
      r.idx[j] = (t < nK) ? tile_idx[t] : 0;  // (slots past the list length hold no valid entry and are never used)
      r.st[j] = (t < nK) ? tile_state[t] : 0;
    }
  };

  // Byte addresses of the lane's operand fragments in LDS step buffer 0; the run loop flips them
  // between the two buffers together with `buf`, across items too.
  unsigned ra[8], ta[8];
#pragma unroll
  for (int ks = 0; ks < 8; ++ks) ra[ks] = base0 + (unsigned)(l32 * kTileD + (((2 * ks + hh) ^ r_sw) << 3)) * 2u;
#pragma unroll
  for (int i = 0; i < 8; ++i)
    ta[i] = base0 + (unsigned)(tile_off(t_row + 8 * (i & 1), 4 * (i >> 1) + t_chunk) + t_half) * 2u;
  int buf = 0;
  bool resident = false;  // the item's first step was already copied into buffer `buf` by the previous item's last step

  // What is left of an item's fetched values once its Q^T / dO^T fragments sit in their registers.
  struct ItemHead {
    float l, m, delta;
    int doc, klo, khi, n_tiles, kb0, kb1;
    int idx[kListRegs];
    unsigned char st[kListRegs];
  };
  DqPinned st;
  // Q goes in multiplied by sm_scale * log2(e): the streams' scores are then in the log2 domain
  const float cap2 = SOFTCAP ? a.score.cap * kLog2e : 0.f;
  const float c2 = SOFTCAP ? 2.0f * kLog2e * a.sm_scale / a.score.cap : a.sm_scale * kLog2e;
  const float out_scale = SOFTCAP ? 4.0f * a.sm_scale : a.sm_scale;
  const float q_mul = EXACT ? 1.0f : c2;   // (EXACT: Q stays as it is; the stream scales the fp32 product)
  auto scaled = [q_mul](unsigned two) {
    const float lo = __builtin_bit_cast(float, two << 16) * q_mul;
    const float hi = __builtin_bit_cast(float, two & 0xffff0000u) * q_mul;
    return __builtin_bit_cast(unsigned, pack_bf16(lo, hi));
  };
  // (`stage`: the wave's 16 KB of a free LDS step buffer)
  auto consume = [&](const ItemRegs& r, ItemHead& c, char* stage) {
    u32x4 qw[8], dw[8];
    rows_to_fragments(r.q, stage, lane, qw);
    rows_to_fragments(r.d, stage + 8192, lane, dw);
#define FA_PUT(KS, QR, DR)                                                                                    \
  asm volatile(FA_DQ_PUT_##KS                                                                                 \
               : "={" QR "}"(st.q[KS]), "={" DR "}"(st.d[KS])                                                 \
               : "v"(scaled(qw[KS][0])), "v"(scaled(qw[KS][1])), "v"(scaled(qw[KS][2])), "v"(scaled(qw[KS][3])), \
                 "v"(dw[KS][0]), "v"(dw[KS][1]), "v"(dw[KS][2]), "v"(dw[KS][3]));
    FA_PUT(0, "a[64:67]", "a[96:99]") FA_PUT(1, "a[68:71]", "a[100:103]") FA_PUT(2, "a[72:75]", "a[104:107]")
    FA_PUT(3, "a[76:79]", "a[108:111]") FA_PUT(4, "a[80:83]", "a[112:115]") FA_PUT(5, "a[84:87]", "a[116:119]")
    FA_PUT(6, "a[88:91]", "a[120:123]") FA_PUT(7, "a[92:95]", "a[124:127]")
#undef FA_PUT
    c.l = r.l; c.m = r.m; c.delta = r.delta; c.doc = r.doc;
    if constexpr (DOCS) { c.klo = r.klo; c.khi = r.khi; }
    c.n_tiles = __builtin_amdgcn_readfirstlane(r.n_tiles);
    c.kb0 = __builtin_amdgcn_readfirstlane(r.kb0);
    c.kb1 = __builtin_amdgcn_readfirstlane(r.kb1);
#pragma unroll
    for (int j = 0; j < kListRegs; ++j) {
      c.idx[j] = r.idx[j];
      c.st[j] = r.st[j];
    }
  };
  // (opaque(): addresses derived from its result are computed where they are used instead of once
  // before the item loop, where they would have to be kept through every run)
  auto opaque = [](int x) {
    asm volatile("" : "+v"(x));
    return x;
  };

  ItemRegs pre;
  ItemHead cur;
  fetch(0, pre);
  consume(pre, cur, reinterpret_cast<char*>(sT + 4 * kTileElems) + w * 16384);
  for (int item = 0; item < n_items; ++item) {
    int bh, qb;
    geometry(item, bh, qb);
    if (item > 0) __syncthreads();  // the previous item's LDS contents are dead from here

    bf16_t* dQg = static_cast<bf16_t*>(a.dq) + ((size_t)bh * a.Sq + (size_t)qb * BM) * D;
    const bf16_t* Kg = static_cast<const bf16_t*>(a.k) + ((size_t)kv_pair(bh) * a.Sk) * D;
    const bf16_t* Vg = static_cast<const bf16_t*>(a.v) + ((size_t)kv_pair(bh) * a.Sk) * D;
    const int q_idx = qb * BM + q_local;
    const int* tile_idx = a.map.idx + (size_t)qb * nK;

    // the q tile's kv list and its state row into LDS
    const int n_tiles = cur.n_tiles;
    const int n_steps = (n_tiles + 1) >> 1;
    const int tid_p = opaque(tid);  // (fresh per item: see opaque())
#pragma unroll
    for (int j = 0; j < kListRegs; ++j) {
      const int t = tid_p + 256 * j;
      if (t < nK) {
        sIdx[t] = cur.idx[j];
        sSt[t] = cur.st[j];
      }
    }
    if (nK > PREFETCH_LIST) {
      // rows longer than the prefetched part (more than 131072 tokens): the rest straight from global memory
      // (an item is then thousands of steps long: the wait does not show)
      const uint8_t* state_row = a.map.state + (size_t)qb * nK;
      for (int t = PREFETCH_LIST + tid_p; t < nK; t += 256) {
        sIdx[t] = tile_idx[t];
        sSt[t] = state_row[t];
      }
    }

    asm volatile(FA_DQ_ZERO_ACC
                 : "={a[0:15]}"(st.dq[0]), "={a[16:31]}"(st.dq[1]), "={a[32:47]}"(st.dq[2]), "={a[48:63]}"(st.dq[3]));
    const float lse2 = (cur.l > 0.f) ? __builtin_fmaf(cur.m, kLog2e, log2f(cur.l)) : __builtin_huge_valf();
    const float delta = cur.delta;
    // operands of the fp32 MFMA that makes the S chains' accumulator input under a position bias
    const float a2 = ALIBI ? a.score.slopes[bh % a.Hq] * kLog2e : 0.f;
    const float aone = hh ? (float)l32 : 1.f;
    const float mulv = hh ? 0.f : a2;
    const float addv = hh ? a2 : -lse2;
    const int doc_i = cur.doc;
    // (DOCS) with sorted kv ids the keys of the row's document are one interval: the keep bits of a partial tile
    // then have a closed form (keep_bits32_range) and no ids are read
    const bool ranged = DOCS && a.mask.doc_q_range != nullptr && keep_bits_have_range(a.mask);
    const int kb_first = cur.kb0;
    const int kb_second = (n_tiles > 1) ? cur.kb1 : kb_first;
    if (n_tiles > 0 && !resident) {
      // first step into the current buffer (a missing second entry repeats the first: finite data, masked out)
      bf16_t* dst = sT + (size_t)buf * 4 * kTileElems;
      loader.load(Kg + (size_t)kb_first * BN * D, dst);
      loader.load(Kg + (size_t)kb_second * BN * D, dst + kTileElems);
      loader.load(Vg + (size_t)kb_first * BN * D, dst + 2 * kTileElems);
      loader.load(Vg + (size_t)kb_second * BN * D, dst + 3 * kTileElems);
      wait_vmem_all();
    }
    unsigned* tbl = sTbl + w * 16;
    const unsigned tbl_addr = (unsigned)(size_t)tbl;
    __syncthreads();
    // The next item's data lands while this item runs.  (The last item fetches itself again: every
    // path then redefines the fetched registers, and the compiler need not merge old values in.)
    const bool has_next = item + 1 < n_items;
    int bh_n = bh, qb_n = qb;
    if (has_next) geometry(item + 1, bh_n, qb_n);
    fetch(has_next ? item + 1 : item, pre);
    const bf16_t* Kg_n = static_cast<const bf16_t*>(a.k) + ((size_t)kv_pair(bh_n) * a.Sk) * D;
    const bf16_t* Vg_n = static_cast<const bf16_t*>(a.v) + ((size_t)kv_pair(bh_n) * a.Sk) * D;

    // carried: the kv tile indices of step it + 1 (clamped into the list)
    int it = 0;
    auto entry = [&](int e) { return sIdx[e < n_tiles ? e : n_tiles - 1]; };
    int kba1 = (n_tiles > 0) ? __builtin_amdgcn_readfirstlane(entry(2)) : 0;
    int kbb1 = (n_tiles > 0) ? __builtin_amdgcn_readfirstlane(entry(3)) : 0;
    // step s is full when both of its entries exist and are full
    auto step_full = [&](int sidx) {
      return sSt[sIdx[2 * sidx]] == 2 && 2 * sidx + 1 < n_tiles && sSt[sIdx[2 * sidx + 1]] == 2;
    };

    // first partial step at or behind `from` (n_steps if none): lanes look 64 steps ahead at a time
    auto next_partial = [&](int from) {
      int pos = from;
      bool found = false;
      while (!found && pos < n_steps) {
        const int j = pos + lane;
        const bool is_partial = j < n_steps && !step_full(j);
        const unsigned long long hits = __ballot(is_partial);
        if (hits != 0ull) {
          pos += __builtin_ctzll(hits);
          found = true;
        } else {
          pos = (pos + 64 < n_steps) ? pos + 64 : n_steps;
        }
      }
      return __builtin_amdgcn_readfirstlane(pos);
    };
    while (it < n_steps) {
      // A run: at most one partial step and the full steps next to it.  Either it starts with the
      // partial step and goes on to the step before the next partial one, or it starts with full
      // steps and ends with the first partial step behind them.
      int it_part = next_partial(it);
      int it_end;
      if (it_part == it) {
        it_end = next_partial(it + 1);
      } else {
        it_end = (it_part < n_steps) ? it_part + 1 : n_steps;
      }
      unsigned km[2] = {0u, 0u};
      if (it_part < n_steps) {
        // the lane's keep bits: element e of kv block c sits at bit 16 (c & 1) + e of km[c >> 1]
        int* sDoc = reinterpret_cast<int*>(sSt + MAX_LIST) + w * 128;  // the wave's stage for document ids
        if ((a.mask.flags & FLEXATTN_MASK_DOC) && !ranged) {
          const int e1 = 2 * it_part + 1 < n_tiles ? 2 * it_part + 1 : 2 * it_part;
          stage_doc_ids(a.mask.doc_k + doc_rows(bh, a.Sk), __builtin_amdgcn_readfirstlane(sIdx[2 * it_part]) * BN,
                        __builtin_amdgcn_readfirstlane(sIdx[e1]) * BN, lane, sDoc);
        }
#pragma unroll
        for (int hx = 0; hx < 2; ++hx) {
          const int e = 2 * it_part + hx;
          if (e >= n_tiles) continue;  // missing half: all dropped
          const int kt = __builtin_amdgcn_readfirstlane(sIdx[e]);
          const int state = __builtin_amdgcn_readfirstlane((int)sSt[kt]);
          if (state == 2) {
            km[hx] = 0xffffffffu;
          } else if (DOCS && ranged) {
            km[hx] = keep_bits32_range<true>(a.mask, q_idx, kt * BN + 4 * hh, cur.klo, cur.khi);
          } else if (a.mask.flags & FLEXATTN_MASK_DOC) {
            km[hx] = keep_bits32_staged<true>(a.mask, q_idx, kt * BN + 4 * hh, doc_i, sDoc + 64 * hx + 4 * hh);
          } else {
            km[hx] = keep_bits32<true>(a.mask, q_idx, kt * BN + 4 * hh, doc_i, nullptr);
          }
        }
      } else {
        it_part = -1;
      }
      const int partial_flag = it_part;  // the step of the run that takes the masked stream (-1: none)
      // Work-group constants of the run loop, one table per wave (order: TABLE in gen_dq_tile.py),
      // written and read by the same wave.  A run that ends the item also names the next item's
      // first step (its values were fetched at the start of this item; only now are they touched).
      {
        int kb_na = kb_first, kb_nb = kb_second;
        if (it_end == n_steps && has_next) {
          const int nt = __builtin_amdgcn_readfirstlane(pre.n_tiles);
          kb_na = nt > 0 ? __builtin_amdgcn_readfirstlane(pre.kb0) : 0;
          kb_nb = nt > 1 ? __builtin_amdgcn_readfirstlane(pre.kb1) : kb_na;
        }
        if (lane == 0) {
          tbl[0] = (unsigned)n_tiles;
          tbl[1] = base0 + (unsigned)w * 4096u;  // LDS address of the wave's first 1 KB block in buffer 0
          tbl[2] = __builtin_bit_cast(unsigned, SOFTCAP ? -2.0f * cap2 : c2);
          tbl[3] = (unsigned)n_steps;
          tbl[4] = (unsigned)(size_t)tile_idx;
          tbl[5] = (unsigned)((size_t)tile_idx >> 32);
          tbl[6] = (unsigned)(size_t)Kg;
          tbl[7] = (unsigned)((size_t)Kg >> 32);
          tbl[8] = (unsigned)(size_t)Vg;
          tbl[9] = (unsigned)((size_t)Vg >> 32);
          tbl[10] = (unsigned)kb_na;
          tbl[11] = (unsigned)kb_nb;
          tbl[12] = (unsigned)(size_t)Kg_n;
          tbl[13] = (unsigned)((size_t)Kg_n >> 32);
          tbl[14] = (unsigned)(size_t)Vg_n;
          tbl[15] = (unsigned)((size_t)Vg_n >> 32);
        }
      }
      // no scalar operands (see gen_dq_tile.py): the loop state travels in VGPRs
#define FA_DQ_CALL(RUN, CLOB_MORE, ...)                                                                                   \
  asm volatile(RUN                                                                                               \
               : FA_DQ_PINNED(st), [it] "+v"(it), [kba1] "+v"(kba1), [kbb1] "+v"(kbb1), [buf] "+v"(buf),          \
                 [r0] "+v"(ra[0]), [r1] "+v"(ra[1]), [r2] "+v"(ra[2]), [r3] "+v"(ra[3]), [r4] "+v"(ra[4]),        \
                 [r5] "+v"(ra[5]), [r6] "+v"(ra[6]), [r7] "+v"(ra[7]), [t0] "+v"(ta[0]), [t1] "+v"(ta[1]),        \
                 [t2] "+v"(ta[2]), [t3] "+v"(ta[3]), [t4] "+v"(ta[4]), [t5] "+v"(ta[5]), [t6] "+v"(ta[6]),        \
                 [t7] "+v"(ta[7])                                                                                \
               : [it_end] "v"(it_end), [partial] "v"(partial_flag), [tbl] "v"(tbl_addr), [dl] "v"(delta),         \
                 [g0] "v"(loader.goff[0]), [g1v] "v"(loader.goff[1]), [g2] "v"(loader.goff[2]),                  \
                 [g3] "v"(loader.goff[3]), [m0] "v"(km[0]), [m1] "v"(km[1]), __VA_ARGS__                          \
               : "memory", "scc", "vcc", "m0", FA_DQ_RUN_SGPRS, FA_DQ_RUN_VGPRS CLOB_MORE)
      if constexpr (ALIBI) {
        const int ka0 = __builtin_amdgcn_readfirstlane(entry(2 * it));
        const int kb0 = __builtin_amdgcn_readfirstlane(entry(2 * it + 1));
#define FA_DQ_ALIBI_CLOBBERS , "s101", "v184", "v185", "v186"
        FA_DQ_CALL(FA_DQ_RUN_ALIBI, FA_DQ_ALIBI_CLOBBERS, [aone] "v"(aone), [mulv] "v"(mulv), [addv] "v"(addv), [iq] "v"(q_idx), [ka0] "v"(ka0),
                   [kb0] "v"(kb0));
      } else if constexpr (SOFTCAP) {
        const float caplse = cap2 - lse2;
        FA_DQ_CALL(FA_DQ_RUN_SOFTCAP, , [lse] "v"(caplse));
      } else if constexpr (EXACT) {
        FA_DQ_CALL(FA_DQ_RUN_EXACT, , [lse] "v"(lse2));
      } else {
        FA_DQ_CALL(FA_DQ_RUN, , [lse] "v"(lse2));
      }
#undef FA_DQ_CALL
#undef FA_DQ_ALIBI_CLOBBERS
      it = __builtin_amdgcn_readfirstlane(it);
      buf = __builtin_amdgcn_readfirstlane(buf);
    }
    // the last step of a non-empty item copied the next item's first step into buffer `buf`
    resident = n_steps > 0 && has_next && __builtin_amdgcn_readfirstlane(pre.n_tiles) > 0;

    // ---- item epilogue ----
    // The next item's Q^T / dO^T fragments go into their registers before this item's stores are
    // issued (their loads are long done; behind the stores the wait would include the stores).
    // (Buffer `buf` may hold the next item's first step: the other one is free.)
    char* stage = reinterpret_cast<char*>(sT + (size_t)(buf ^ 1) * 4 * kTileElems) + w * 16384;
    consume(pre, cur, stage);

    // dq: bf16 rows staged through the same wave-private LDS (16-byte chunks XOR-swizzled by row), so
    // that every store instruction writes four complete 256-byte rows.
    {
      const int lane_here = opaque(lane);
      const int row_here = lane_here & 31;
      const unsigned wr = (unsigned)row_here * 256u + 8u * (unsigned)(lane_here >> 5);
#define FA_GET(T, SRC, REG)                                                                                        \
  {                                                                                                                \
    float x[16];                                                                                                   \
    asm volatile(FA_DQ_GET_ACC_##T                                                                                 \
                 : "=v"(x[0]), "=v"(x[1]), "=v"(x[2]), "=v"(x[3]), "=v"(x[4]), "=v"(x[5]), "=v"(x[6]), "=v"(x[7]), \
                   "=v"(x[8]), "=v"(x[9]), "=v"(x[10]), "=v"(x[11]), "=v"(x[12]), "=v"(x[13]), "=v"(x[14]),        \
                   "=v"(x[15])                                                                                     \
                 : "{" REG "}"(SRC));                                                                              \
    _Pragma("unroll") for (int g = 0; g < 4; ++g) {                                                                \
      /* the streams leave the constant sm_scale (softcap: 4 sm_scale) out of dS: apply it once */                 \
      const bf16x2 lo = pack_bf16(x[4 * g] * out_scale, x[4 * g + 1] * out_scale);                                 \
      const bf16x2 hi = pack_bf16(x[4 * g + 2] * out_scale, x[4 * g + 3] * out_scale);                             \
      const bf16x4 out = {lo[0], lo[1], hi[0], hi[1]};                                                             \
      *reinterpret_cast<bf16x4*>(stage + wr + (unsigned)(((4 * T + g) ^ (row_here & 15)) << 4)) = out;             \
    }                                                                                                              \
  }
      FA_GET(0, st.dq[0], "a[0:15]") FA_GET(1, st.dq[1], "a[16:31]")
      FA_GET(2, st.dq[2], "a[32:47]") FA_GET(3, st.dq[3], "a[48:63]")
#undef FA_GET
      __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
      __builtin_amdgcn_wave_barrier();
      bf16_t* out_rows = dQg + (size_t)(w * 32) * D;
      const int chunk = lane_here & 15;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int r = 4 * i + (lane_here >> 4);
        const u32x4 x = *reinterpret_cast<const u32x4*>(stage + (unsigned)r * 256u + (unsigned)((chunk ^ (r & 15)) << 4));
        *reinterpret_cast<u32x4*>(out_rows + (size_t)r * D + chunk * 8) = x;
      }
    }
  }  // work items
}

template <int KIND, bool DOCS>
static int launch_dq_plain_on(const BwdArgs& a, hipStream_t stream) {
  using namespace dq_cfg;
  auto kern = bwd_dq_bf16_d128_plain_kernel<KIND, DOCS>;
  static hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, PLAIN_LDS_BYTES);
  if (attr != hipSuccess) return set_error(FLEXATTN_ELAUNCH, "hipFuncSetAttribute(dq): %s", hipGetErrorString(attr));
  const int n_wg = a.B * a.Hq * (a.Sq / BM);
  const bool persistent = DOCS ? sorted_schedule_ok(n_wg, a.Sq / BM) : persistent_ok(n_wg, a.Sq / BM);
  const int grid = (persistent && n_wg > 256) ? 256 : n_wg;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(256), PLAIN_LDS_BYTES, stream, a);
  return check_launch("flexattn_bwd_dq bf16");
}

template <int KIND>
static int launch_dq_plain(const BwdArgs& a, hipStream_t stream) {
  return (a.mask.flags & FLEXATTN_MASK_DOC) ? launch_dq_plain_on<KIND, true>(a, stream)
                                            : launch_dq_plain_on<KIND, false>(a, stream);
}

#endif  // FLEXATTN_CUSTOM_ONLY

int bwd_dq_bf16_d128(const BwdArgs& a, hipStream_t stream) {
#ifdef FLEXATTN_CUSTOM_ONLY
  switch (a.score.kind) {
    case FLEXATTN_SCORE_NONE: return launch_dq<FLEXATTN_SCORE_NONE>(a, stream);
    case FLEXATTN_SCORE_CUSTOM: return launch_dq<FLEXATTN_SCORE_CUSTOM>(a, stream);
  }
  return set_error(FLEXATTN_ENOTSUP, "this functor library holds the plain and the compiled score function only (kind %d asked)", a.score.kind);
#else
  // (the generated-stream kernel caches the kv list in LDS)
  // (and has no additive bias)
  // (and folds its scale into bf16 Q where that is harmless, folded_scale_ok; plain scores have a variant that does
  // not fold, the position-bias and softcap streams do not)
  const float fold = a.score.kind == FLEXATTN_SCORE_SOFTCAP ? 2.0f * kLog2e * a.sm_scale / a.score.cap : a.sm_scale * kLog2e;
  const bool stream_ok = !(a.flags & FLEXATTN_FLAG_COMPILED_LOOP) && a.map.nk <= dq_cfg::MAX_LIST && a.score.ab == nullptr;
  const bool fold_ok = folded_scale_ok(fold, a.sm_scale, 128);
  switch (a.score.kind) {
    case FLEXATTN_SCORE_NONE:
      if (stream_ok) return fold_ok ? launch_dq_plain<0>(a, stream) : launch_dq_plain<3>(a, stream);
      return launch_dq<FLEXATTN_SCORE_NONE>(a, stream);
    case FLEXATTN_SCORE_ALIBI:
      return stream_ok && fold_ok ? launch_dq_plain<1>(a, stream) : launch_dq<FLEXATTN_SCORE_ALIBI>(a, stream);
    case FLEXATTN_SCORE_SOFTCAP:
      return stream_ok && fold_ok ? launch_dq_plain<2>(a, stream) : launch_dq<FLEXATTN_SCORE_SOFTCAP>(a, stream);
    case FLEXATTN_SCORE_ALIBI_TILE: return launch_dq<FLEXATTN_SCORE_ALIBI_TILE>(a, stream);
  }
  return set_error(FLEXATTN_EINVAL, "unknown score kind %d", a.score.kind);
#endif
}

// Head dim 256: the kernels with a compiled main loop (two 128-column panels per row), every score kind.
int bwd_dq_bf16_d256(const BwdArgs& a, hipStream_t stream) {
  switch (a.score.kind) {
    case FLEXATTN_SCORE_NONE: return launch_dq<FLEXATTN_SCORE_NONE, 2>(a, stream);
#ifdef FLEXATTN_CUSTOM_ONLY
    case FLEXATTN_SCORE_CUSTOM: return launch_dq<FLEXATTN_SCORE_CUSTOM, 2>(a, stream);
#else
    case FLEXATTN_SCORE_ALIBI: return launch_dq<FLEXATTN_SCORE_ALIBI, 2>(a, stream);
    case FLEXATTN_SCORE_SOFTCAP: return launch_dq<FLEXATTN_SCORE_SOFTCAP, 2>(a, stream);
    case FLEXATTN_SCORE_ALIBI_TILE: return launch_dq<FLEXATTN_SCORE_ALIBI_TILE, 2>(a, stream);
#endif
  }
  return set_error(FLEXATTN_ENOTSUP, "score kind %d is not in this library", a.score.kind);
}

void bwd_dq_bf16_d128_tile(int* bq, int* bk) {
  *bq = dq_cfg::BM;
  *bk = dq_cfg::BN;
}

}  // namespace fa
