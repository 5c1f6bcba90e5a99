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
//
// Full (unmasked) tiles of the plain score run a generated, hand-scheduled instruction stream
// (gen_dkv_tile.py -> bwd_dkv_tile.inc) that software-pipelines MFMA, VALU and LDS work inside the
// wave with a fixed register allocation; partial tiles and score modifications run the C++ path.
#include "fa_common.hpp"
#include "launch.hpp"
#include "tile_io.hpp"

#include <type_traits>

// registers v[68:255] belong to the generated tile streams
#define FA_DKV_TILE_CLOBBERS "v68", "v69", "v70", "v71", "v72", "v73", "v74", "v75", "v76", "v77", "v78", \
  "v79", "v80", "v81", "v82", "v83", "v84", "v85", "v86", "v87", "v88", "v89", "v90", "v91", "v92", "v93", \
  "v94", "v95", "v96", "v97", "v98", "v99", "v100", "v101", "v102", "v103", "v104", "v105", "v106", "v107", \
  "v108", "v109", "v110", "v111", "v112", "v113", "v114", "v115", "v116", "v117", "v118", "v119", "v120", \
  "v121", "v122", "v123", "v124", "v125", "v126", "v127", "v128", "v129", "v130", "v131", "v132", "v133", \
  "v134", "v135", "v136", "v137", "v138", "v139", "v140", "v141", "v142", "v143", "v144", "v145", "v146", \
  "v147", "v148", "v149", "v150", "v151", "v152", "v153", "v154", "v155", "v156", "v157", "v158", "v159", \
  "v160", "v161", "v162", "v163", "v164", "v165", "v166", "v167", "v168", "v169", "v170", "v171", "v172", \
  "v173", "v174", "v175", "v176", "v177", "v178", "v179", "v180", "v181", "v182", "v183", "v184", "v185", \
  "v186", "v187", "v188", "v189", "v190", "v191", "v192", "v193", "v194", "v195", "v196", "v197", "v198", \
  "v199", "v200", "v201", "v202", "v203", "v204", "v205", "v206", "v207", "v208", "v209", "v210", "v211", \
  "v212", "v213", "v214", "v215", "v216", "v217", "v218", "v219", "v220", "v221", "v222", "v223", "v224", \
  "v225", "v226", "v227", "v228", "v229", "v230", "v231", "v232", "v233", "v234", "v235", "v236", "v237", \
  "v238", "v239", "v240", "v241", "v242", "v243", "v244", "v245", "v246", "v247", "v248", "v249", "v250", \
  "v251", "v252", "v253", "v254", "v255"

#include "bwd_dkv_tile.inc"

namespace fa {

namespace dkv_cfg {
constexpr int BNK = 128;  // kv rows per work-group
constexpr int BQ = 128;   // q rows per step (two 64-row LDS tiles)
constexpr int D = 128;
constexpr int LDS_BYTES = 8 * kTileElems * 2 + 4 * BQ * 4;  // (Q, dO) x 2 buffers x 2 tiles, lse x2, delta x2
}  // namespace dkv_cfg

typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

// The register-resident state of the generated tile streams.  Every asm statement that touches it
// names it with the same physical-register constraints, so the values stay where the streams
// expect them and the compiler keeps those registers free of anything else.
struct PinnedState {
  f32x16 dv[4], dk[4];  // a[0:63], a[64:127]
  bf16x8 k[8], v[8];    // a[128:159], a[160:191]
};
#define FA_DKV_PINNED(st)                                                                                   \
  "+{a[0:15]}"(st.dv[0]), "+{a[16:31]}"(st.dv[1]), "+{a[32:47]}"(st.dv[2]), "+{a[48:63]}"(st.dv[3]),        \
      "+{a[64:79]}"(st.dk[0]), "+{a[80:95]}"(st.dk[1]), "+{a[96:111]}"(st.dk[2]), "+{a[112:127]}"(st.dk[3]), \
      "+{a[128:131]}"(st.k[0]), "+{a[132:135]}"(st.k[1]), "+{a[136:139]}"(st.k[2]), "+{a[140:143]}"(st.k[3]), \
      "+{a[144:147]}"(st.k[4]), "+{a[148:151]}"(st.k[5]), "+{a[152:155]}"(st.k[6]), "+{a[156:159]}"(st.k[7]), \
      "+{a[160:163]}"(st.v[0]), "+{a[164:167]}"(st.v[1]), "+{a[168:171]}"(st.v[2]), "+{a[172:175]}"(st.v[3]), \
      "+{a[176:179]}"(st.v[4]), "+{a[180:183]}"(st.v[5]), "+{a[184:187]}"(st.v[6]), "+{a[188:191]}"(st.v[7])

template <int SCORE>
__global__ __launch_bounds__(256, 1) void bwd_dkv_bf16_d128_kernel(BwdArgs a) {
  using namespace dkv_cfg;
  extern __shared__ __attribute__((aligned(1024))) char smem_raw[];
  // step buffer b: Q half 0, Q half 1, dO half 0, dO half 1 (64 KiB); then lse[2][BQ], delta[2][BQ]
  bf16_t* sT = reinterpret_cast<bf16_t*>(smem_raw);
  auto sQ = [&](int buf, int half) { return sT + (4 * buf + half) * kTileElems; };
  auto sDO = [&](int buf, int half) { return sT + (4 * buf + 2 + half) * kTileElems; };
  float* sLse = reinterpret_cast<float*>(sT + 8 * kTileElems);
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

  // Plain score: the dk / dv accumulators (a[0:127]) and the K, V fragments (a[128:191]) live in
  // accumulation registers that only the asm statements of this kernel read or write.
  constexpr bool kAsmTiles = SCORE == FLEXATTN_SCORE_NONE;
  bf16x8 kreg[8], vreg[8];
#pragma unroll
  for (int ks = 0; ks < 8; ++ks) {
    kreg[ks] = *reinterpret_cast<const bf16x8*>(Kg + (size_t)kv_local * D + ks * 16 + hh * 8);
    vreg[ks] = *reinterpret_cast<const bf16x8*>(Vg + (size_t)kv_local * D + ks * 16 + hh * 8);
  }
  PinnedState st;
  if constexpr (kAsmTiles) {
    // the outputs are written by the statement: no ordinary initial value is needed
    asm volatile(FA_DKV_ZERO_ACC
                 : "={a[0:15]}"(st.dv[0]), "={a[16:31]}"(st.dv[1]), "={a[32:47]}"(st.dv[2]), "={a[48:63]}"(st.dv[3]),
                   "={a[64:79]}"(st.dk[0]), "={a[80:95]}"(st.dk[1]), "={a[96:111]}"(st.dk[2]), "={a[112:127]}"(st.dk[3]));
#define FA_PUT(KS, KR, VR)                                                                          \
  {                                                                                                 \
    const u32x4 kw = __builtin_bit_cast(u32x4, kreg[KS]);                                           \
    const u32x4 vw = __builtin_bit_cast(u32x4, vreg[KS]);                                           \
    asm volatile(FA_DKV_PUT_KV_##KS                                                                 \
                 : "={" KR "}"(st.k[KS]), "={" VR "}"(st.v[KS])                                     \
                 : "v"(kw[0]), "v"(kw[1]), "v"(kw[2]), "v"(kw[3]), "v"(vw[0]), "v"(vw[1]), "v"(vw[2]), "v"(vw[3])); \
  }
    FA_PUT(0, "a[128:131]", "a[160:163]") FA_PUT(1, "a[132:135]", "a[164:167]")
    FA_PUT(2, "a[136:139]", "a[168:171]") FA_PUT(3, "a[140:143]", "a[172:175]")
    FA_PUT(4, "a[144:147]", "a[176:179]") FA_PUT(5, "a[148:151]", "a[180:183]")
    FA_PUT(6, "a[152:155]", "a[184:187]") FA_PUT(7, "a[156:159]", "a[188:191]")
#undef FA_PUT
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

  // Iteration `it` covers q tile tile_idx[it % n_tiles] of query head hk*group + it / n_tiles; the
  // quotient and remainders of it, it + 1 and it + 2 are carried along instead of divided out.
  // Its q block index is fetched two iterations ahead, its state one iteration ahead.
  int g_cur = 0, g_nxt = 0, t_nxt = 1, t_n2 = 2;  // it / n_tiles, (it + 1) / n_tiles, (it + 1) % n_tiles, (it + 2) % n_tiles
  if (t_nxt >= n_tiles) { t_nxt -= n_tiles; g_nxt = 1; }
  if (t_n2 >= n_tiles) t_n2 -= n_tiles;
  if (t_n2 >= n_tiles) t_n2 -= n_tiles;
  int qb_cur = 0, qb_nxt = 0, st_cur = 0;
  if (n_iter > 0) qb_cur = tile_idx[0];
  if (n_iter > 1) qb_nxt = tile_idx[t_nxt];
  if (n_iter > 0) st_cur = a.map.state[(size_t)qb_cur * a.map.nk + kb];

  TileLoader<4> loader;
  loader.init(w, lane);
  float l_st = 0.f, m_st = 0.f, dl_st = 0.f;
  // With `tiles_too` false only the per-row values are fetched: the generated tile stream copies
  // the next step's Q / dO tiles itself, spread between its MFMAs.
  size_t next_rbase = 0;
  auto issue_tile = [&](int g, int qb, int buf, bool tiles_too) {
    const size_t rbase = ((size_t)(b * a.Hq + hk * group + g) * a.Sq + (size_t)qb * BQ);
    next_rbase = rbase;
    if (tiles_too) {
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        loader.load(Qall + (rbase + half * kTileRows) * D, sQ(buf, half));
        loader.load(dOall + (rbase + half * kTileRows) * D, sDO(buf, half));
      }
    }
    // raw values only: using them here would make the wave wait for every load issued above
    if (tid < BQ) {
      l_st = a.l[rbase + tid];
      m_st = a.m[rbase + tid];
      dl_st = a.delta[rbase + tid];
    }
  };
  auto store_rows = [&](int buf) {
    if (tid < BQ) {
      sLse[buf * BQ + tid] = (l_st > 0.f) ? __builtin_fmaf(m_st, kLog2e, log2f(l_st)) : __builtin_huge_valf();
      sDl[buf * BQ + tid] = dl_st;
    }
  };
  if (n_iter > 0) {
    issue_tile(0, __builtin_amdgcn_readfirstlane(qb_cur), 0, true);
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
    sm.init(a.score, a.sm_scale, hk * group + g_cur);
    const int q0 = qb * BQ;
    // The lane's keep bits of a partial tile: element e of q block c sits at bit 16 (c & 1) + e of
    // km[c >> 1].  Computed before the next step's loads are issued: the document-id loads would
    // otherwise wait for them.
    unsigned km[2] = {0u, 0u};
    if (kAsmTiles && partial) {
      const bool has_doc = (a.mask.flags & FLEXATTN_MASK_DOC) != 0;
#pragma unroll
      for (int cc = 0; cc < 4; ++cc) {
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4) {
          const int r0 = 32 * cc + 8 * g4 + 4 * hh;
          int di[4] = {0, 0, 0, 0};
          if (has_doc) {
            const auto d4 = *reinterpret_cast<const int __attribute__((ext_vector_type(4)))*>(a.mask.doc_q + q0 + r0);
            di[0] = d4[0]; di[1] = d4[1]; di[2] = d4[2]; di[3] = d4[3];
          }
#pragma unroll
          for (int u = 0; u < 4; ++u) {
            const bool keep = keep_elem(a.mask, q0 + r0 + u, k_idx, di[u], doc_j);
            km[cc >> 1] |= (keep ? 1u : 0u) << (16 * (cc & 1) + 4 * g4 + u);
          }
        }
      }
    }
    const int qb_n2 = (it + 2 < n_iter) ? tile_idx[t_n2] : 0;
    int st_nxt = 0;
    if (it + 1 < n_iter) {
      const int qbn = __builtin_amdgcn_readfirstlane(qb_nxt);
      st_nxt = a.map.state[(size_t)qbn * a.map.nk + kb];
      issue_tile(g_nxt, qbn, buf ^ 1, !kAsmTiles);
    }
    auto tile_cpp = [&]() {
#pragma unroll
    for (int cc = 0; cc < 4; ++cc) {
      const int c = cc & 1;  // 32-row block inside the 64-row LDS tile cc >> 1
      const char* qt = reinterpret_cast<const char*>(sQ(buf, cc >> 1));
      const char* dot = reinterpret_cast<const char*>(sDO(buf, cc >> 1));
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
            float gd = pe * (dp_acc[e] - dl4[u]) * sm.dfactor_unscaled(tv);
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
    };
    if constexpr (kAsmTiles) {
      // byte addresses of the lane's fragments in this step buffer (LDS addresses fit 32 bits)
      const unsigned bbase = (unsigned)(size_t)sQ(buf, 0);
      unsigned ra[8], ta[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        ra[i] = bbase + r_off[i];
        ta[i] = bbase + t_off[i >> 1][i & 1];
      }
      const unsigned la = (unsigned)(size_t)(sLse + buf * BQ + 4 * hh);
      const float c2 = sm.c2;
#define FA_DKV_TILE_ADDRS                                                                                          \
  [r0] "v"(ra[0]), [r1] "v"(ra[1]), [r2] "v"(ra[2]), [r3] "v"(ra[3]), [r4] "v"(ra[4]), [r5] "v"(ra[5]),            \
      [r6] "v"(ra[6]), [r7] "v"(ra[7]), [t0] "v"(ta[0]), [t1] "v"(ta[1]), [t2] "v"(ta[2]), [t3] "v"(ta[3]),        \
      [t4] "v"(ta[4]), [t5] "v"(ta[5]), [t6] "v"(ta[6]), [t7] "v"(ta[7]), [la] "v"(la), [c2] "s"(c2)
      const int partial_flag = __builtin_amdgcn_readfirstlane(partial ? 1 : 0);
      // next step's tiles (after the last step: this step's again, into the idle buffer)
      const bf16_t* gq0 = Qall + next_rbase * D;
      const bf16_t* gq1 = gq0 + kTileRows * D;
      const bf16_t* gd0 = dOall + next_rbase * D;
      const bf16_t* gd1 = gd0 + kTileRows * D;
      const unsigned ldsn = (unsigned)(size_t)sQ(buf ^ 1, 0) + (unsigned)w * 4096u;
      asm volatile(FA_DKV_TILE
                   : FA_DKV_PINNED(st)
                   : FA_DKV_TILE_ADDRS, [m0] "v"(km[0]), [m1] "v"(km[1]), [partial] "s"(partial_flag),
                     [g0] "v"(loader.goff[0]), [g1] "v"(loader.goff[1]), [g2] "v"(loader.goff[2]), [g3] "v"(loader.goff[3]),
                     [gq0] "s"(gq0), [gq1] "s"(gq1), [gd0] "s"(gd0), [gd1] "s"(gd1), [ldsn] "s"(ldsn)
                   : "memory", "scc", "m0", FA_DKV_TILE_CLOBBERS);
#undef FA_DKV_TILE_ADDRS
    } else {
      tile_cpp();
    }

    qb_cur = qb_nxt; qb_nxt = qb_n2;
    g_cur = g_nxt;
    if (++t_nxt == n_tiles) { t_nxt = 0; ++g_nxt; }
    if (++t_n2 == n_tiles) t_n2 = 0;
    st_cur = st_nxt;
    if (it + 1 < n_iter) store_rows(buf ^ 1);
    wait_vmem_all();
    __syncthreads();
  }

  if constexpr (kAsmTiles) {
#define FA_GET(T, SRC, REG, DST)                                                                                   \
  {                                                                                                                \
    float x[16];                                                                                                   \
    asm volatile(FA_DKV_GET_ACC_##T                                                                                \
                 : "=v"(x[0]), "=v"(x[1]), "=v"(x[2]), "=v"(x[3]), "=v"(x[4]), "=v"(x[5]), "=v"(x[6]), "=v"(x[7]), \
                   "=v"(x[8]), "=v"(x[9]), "=v"(x[10]), "=v"(x[11]), "=v"(x[12]), "=v"(x[13]), "=v"(x[14]),        \
                   "=v"(x[15])                                                                                     \
                 : "{" REG "}"(SRC));                                                                              \
    _Pragma("unroll") for (int e = 0; e < 16; ++e) DST[e] = x[e];                                                  \
  }
    FA_GET(0, st.dv[0], "a[0:15]", dv_acc[0]) FA_GET(1, st.dv[1], "a[16:31]", dv_acc[1])
    FA_GET(2, st.dv[2], "a[32:47]", dv_acc[2]) FA_GET(3, st.dv[3], "a[48:63]", dv_acc[3])
    FA_GET(4, st.dk[0], "a[64:79]", dk_acc[0]) FA_GET(5, st.dk[1], "a[80:95]", dk_acc[1])
    FA_GET(6, st.dk[2], "a[96:111]", dk_acc[2]) FA_GET(7, st.dk[3], "a[112:127]", dk_acc[3])
#undef FA_GET
  }
  // the constant part of d(s')/d(raw) was left out of dS: apply it to dk once
  const float dk_scale = sm.dfactor_post_scale(a.sm_scale);
#pragma unroll
  for (int db = 0; db < 4; ++db)
#pragma unroll
    for (int e = 0; e < 16; ++e) dk_acc[db][e] *= dk_scale;

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
