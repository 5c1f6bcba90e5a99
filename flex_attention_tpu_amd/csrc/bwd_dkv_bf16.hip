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
// The plain score runs generated, hand-scheduled instruction streams (gen_dkv_tile.py ->
// bwd_dkv_tile.inc) that software-pipeline MFMA, VALU and LDS work inside the wave with a fixed
// register allocation; score modifications run the compiled C++ kernel.
#include <cstdlib>
#include "fa_common.hpp"
#include "launch.hpp"
#include "tile_io.hpp"

#include <type_traits>

// v[68:199] and a[192:255] belong to the generated tile streams
#define FA_DKV_TILE_CLOBBERS "v68", "v69", "v70", "v71", "v72", "v73", "v74", "v75", "v76", "v77", "v78", "v79", "v80", "v81", "v82", \
  "v83", "v84", "v85", "v86", "v87", "v88", "v89", "v90", "v91", "v92", "v93", "v94", "v95", "v96", "v97", \
  "v98", "v99", "v100", "v101", "v102", "v103", "v104", "v105", "v106", "v107", "v108", "v109", "v110", \
  "v111", "v112", "v113", "v114", "v115", "v116", "v117", "v118", "v119", "v120", "v121", "v122", "v123", \
  "v124", "v125", "v126", "v127", "v128", "v129", "v130", "v131", "v132", "v133", "v134", "v135", "v136", \
  "v137", "v138", "v139", "v140", "v141", "v142", "v143", "v144", "v145", "v146", "v147", "v148", "v149", \
  "v150", "v151", "v152", "v153", "v154", "v155", "v156", "v157", "v158", "v159", "v160", "v161", "v162", \
  "v163", "v164", "v165", "v166", "v167", "v168", "v169", "v170", "v171", "v172", "v173", "v174", "v175", \
  "v176", "v177", "v178", "v179", "v180", "v181", "v182", "v183", "v184", "v185", "v186", "v187", "v188", \
  "v189", "v190", "v191", "v192", "v193", "v194", "v195", "v196", "v197", "v198", "v199", "a192", "a193", \
  "a194", "a195", "a196", "a197", "a198", "a199", "a200", "a201", "a202", "a203", "a204", "a205", "a206", \
  "a207", "a208", "a209", "a210", "a211", "a212", "a213", "a214", "a215", "a216", "a217", "a218", "a219", \
  "a220", "a221", "a222", "a223", "a224", "a225", "a226", "a227", "a228", "a229", "a230", "a231", "a232", \
  "a233", "a234", "a235", "a236", "a237", "a238", "a239", "a240", "a241", "a242", "a243", "a244", "a245", \
  "a246", "a247", "a248", "a249", "a250", "a251", "a252", "a253", "a254", "a255"

// scalar registers of the generated run loop
#define FA_DKV_RUN_SGPRS "s60", "s61", "s62", "s63", "s64", "s65", "s66", "s67", "s68", "s69", "s70", "s71", "s72", "s73", "s74", "s75", "s76", "s77", "s78", "s79", "s80", "s81", "s82", "s83", "s84", "s85", "s86", "s87", "s88", "s89", "s90", "s91", "s92", "s93", "s94", "s95", "s96", "s97", "s98", "s99", "s100"

#include "bwd_dkv_tile.inc"

namespace fa {

namespace dkv_cfg {
constexpr int BNK = 128;  // kv rows per work-group
constexpr int BQ = 128;   // q rows per step (two 64-row LDS tiles)
constexpr size_t kDsBlockBytes = (size_t)BQ * BNK * 2;  // one exported dS block
constexpr int D = 128;
constexpr int MAX_LIST = 2048;       // longest q tile list the plain-score kernel caches in LDS (262144 tokens)
constexpr int PREFETCH_LIST = 1024;  // of which an item's prefetch carries this many in registers; the rest is read when the item starts
// (Q, dO) x 2 buffers x 2 tiles, lse x2, delta x2, run-loop tables, cached q tile list and its partial flags
constexpr int LDS_BYTES = 8 * kTileElems * 2 + 4 * BQ * 4 + 4 * 32 * 4 + MAX_LIST * 5 + kDocStageBytes + kMaxSortedItems * 4;
}  // namespace dkv_cfg


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

// Score modifications: compiled C++ path, one 128 x 128 tile per loop iteration.
// EXPORT: the kernel also writes the tile's bf16 dS (the B operands of the dk product: here with the score function's
// derivative and sm_scale in them) to a.ds, in the block layout of the generated streams' export (see there), for
// the dq pass from dS: a score function is then evaluated in one backward pass instead of two.
template <int SCORE, bool EXPORT = false>
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
  const MaskArgs mk = mask_of_batch(a.mask, b, a.Sq, a.Sk);
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
  if (mk.flags & FLEXATTN_MASK_DOC) doc_j = mk.doc_k[k_idx];

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
    sm.init(a.score, a.sm_scale, hk * group + it / n_tiles, b);
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
        const bool has_doc = MASKED && (mk.flags & FLEXATTN_MASK_DOC) != 0;
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4) {
          const int r0 = 32 * cc + 8 * g4 + 4 * hh;  // the lane's q rows come in runs of 4
          const f32x4 lse4 = *reinterpret_cast<const f32x4*>(sLse + buf * BQ + r0);
          const f32x4 dl4 = *reinterpret_cast<const f32x4*>(sDl + buf * BQ + r0);
          int di[4] = {0, 0, 0, 0};
          if (MASKED && has_doc) {
            const auto d4 = *reinterpret_cast<const int __attribute__((ext_vector_type(4)))*>(mk.doc_q + q0 + r0);
            di[0] = d4[0]; di[1] = d4[1]; di[2] = d4[2]; di[3] = d4[3];
          }
          float pv[4], dsv[4];
#pragma unroll
          for (int u = 0; u < 4; ++u) {
            const int e = 4 * g4 + u;
            const int i = q0 + r0 + u;
            const float tv = sm.to_log2(s_acc[e], i, k_idx);
            float pe = fast_exp2(tv + sm.bias2(i, k_idx) - lse4[u]);
            float gd = pe * (dp_acc[e] - dl4[u]) * sm.dfactor(tv, s_acc[e], i, k_idx);
            if (MASKED) {
              const bool keep = keep_elem(mk, i, k_idx, di[u], doc_j);
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
      if constexpr (EXPORT) {
        // block of (query head, kept tile pair): head a.ds_pairs + a.ds_col[kv tile] + place of the q tile in the kv
        // tile's list; inside it wave w writes 1 KB per (32-row q block cc, 16-row half u), lane L its 8 values
        char* blk = static_cast<char*>(a.ds) +
                    ((size_t)(b * a.Hq + hk * group + it / n_tiles) * (size_t)a.ds_pairs + (size_t)a.ds_col[kb] +
                     (size_t)(it % n_tiles)) * kDsBlockBytes + 8192 * w + 16 * (2 * l32 + hh);
#pragma unroll
        for (int u = 0; u < 2; ++u) *reinterpret_cast<bf16x8*>(blk + 1024 * (2 * cc + u)) = dsb[u];
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

// Head dimension 128 NP, NP >= 2: compiled C++ path.  A row of Q or dO is NP panels of 128 columns, each panel of a
// 64-row tile one LDS tile (tile_io.hpp) at [buffer][panel]; a loop iteration covers 64 q rows (half an entry of the
// kv tile's list: the two buffers of Q and dO panels then take the LDS the 128-row steps take at head dim 128), the
// contractions of S and dP run over the panels, dk^T and dv^T have four accumulators per panel.
template <int SCORE, int NP>
__global__ __launch_bounds__(256, 1) void bwd_dkv_bf16_wide_kernel(BwdArgs a) {
  using namespace dkv_cfg;
  constexpr int D = 128 * NP;
  constexpr int HQ = 64;                  // q rows per iteration
  constexpr int kPanel = kTileElems * 2;  // bytes
  extern __shared__ __attribute__((aligned(1024))) char smem_raw[];
  bf16_t* sQ = reinterpret_cast<bf16_t*>(smem_raw);
  bf16_t* sDO = sQ + 2 * NP * kTileElems;
  float* sLse = reinterpret_cast<float*>(sDO + 2 * NP * kTileElems);
  float* sDl = sLse + 2 * HQ;

  const int nKb = a.Sk / BNK;
  const int nQ = a.map.nq;
  const int n_wg = a.B * a.Hkv * nKb;
  const int wg = xcd_remap(blockIdx.x, n_wg);
  const int bhk = wg / nKb;
  const int kb = wg % nKb;
  const int b = bhk / a.Hkv;
  const MaskArgs mk = mask_of_batch(a.mask, b, a.Sq, a.Sk);
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

  bf16x8 kreg[8 * NP], vreg[8 * NP];
#pragma unroll
  for (int ks = 0; ks < 8 * NP; ++ks) {
    kreg[ks] = *reinterpret_cast<const bf16x8*>(Kg + (size_t)kv_local * D + ks * 16 + hh * 8);
    vreg[ks] = *reinterpret_cast<const bf16x8*>(Vg + (size_t)kv_local * D + ks * 16 + hh * 8);
  }
  int doc_j = 0;
  if (mk.flags & FLEXATTN_MASK_DOC) doc_j = mk.doc_k[k_idx];

  f32x16 dk_acc[4 * NP], dv_acc[4 * NP];
#pragma unroll
  for (int i = 0; i < 4 * NP; ++i)
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      dk_acc[i][e] = 0.f;
      dv_acc[i][e] = 0.f;
    }

  const int n_tiles = a.map.cnt[kb];
  const int* tile_idx = a.map.idx + (size_t)kb * nQ;
  const int n_iter = 2 * n_tiles * group;

  // Iteration `it` covers rows 64 (it & 1) .. of q tile tile_idx[(it / 2) % n_tiles] of query head
  // hk*group + (it / 2) / n_tiles.  Its q block index is fetched two iterations ahead, its state one ahead.
  auto q_block_of = [&](int it) { return tile_idx[(it >> 1) % n_tiles]; };
  int qb_cur = 0, qb_nxt = 0, st_cur = 0;
  if (n_iter > 0) qb_cur = q_block_of(0);
  if (n_iter > 1) qb_nxt = q_block_of(1);
  if (n_iter > 0) st_cur = a.map.state[(size_t)qb_cur * a.map.nk + kb];

  TileLoader<4, D> loader;
  loader.init(w, lane);
  float lse_st = 0.f, dl_st = 0.f;
  auto issue_tile = [&](int it, int qb, int buf) {
    const int g = (it >> 1) / n_tiles;
    const size_t rbase = ((size_t)(b * a.Hq + hk * group + g) * a.Sq + (size_t)qb * BQ + (size_t)(it & 1) * HQ);
#pragma unroll
    for (int pn = 0; pn < NP; ++pn) {
      loader.load(Qall + rbase * D + 128 * pn, sQ + (buf * NP + pn) * kTileElems);
      loader.load(dOall + rbase * D + 128 * pn, sDO + (buf * NP + pn) * kTileElems);
    }
    if (tid < HQ) {
      const float l_i = a.l[rbase + tid], m_i = a.m[rbase + tid];
      lse_st = (l_i > 0.f) ? __builtin_fmaf(m_i, kLog2e, log2f(l_i)) : __builtin_huge_valf();
      dl_st = a.delta[rbase + tid];
    }
  };
  auto store_rows = [&](int buf) {
    if (tid < HQ) {
      sLse[buf * HQ + tid] = lse_st;
      sDl[buf * HQ + tid] = dl_st;
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
    sm.init(a.score, a.sm_scale, hk * group + (it >> 1) / n_tiles, b);
    const int qb_n2 = (it + 2 < n_iter) ? q_block_of(it + 2) : 0;
    int st_nxt = 0;
    if (it + 1 < n_iter) {
      const int qbn = __builtin_amdgcn_readfirstlane(qb_nxt);
      st_nxt = a.map.state[(size_t)qbn * a.map.nk + kb];
      issue_tile(it + 1, qbn, buf ^ 1);
    }
    const int q0 = qb * BQ + (it & 1) * HQ;
    const char* qt = reinterpret_cast<const char*>(sQ + buf * NP * kTileElems);
    const char* dot = reinterpret_cast<const char*>(sDO + buf * NP * kTileElems);
#pragma unroll 1   // (rolled: unrolled, the second block's operand loads are hoisted over the first block's and 72 registers spill; 2.72 -> 2.01 ms on B=4, H=16, S=4096)
    for (int c = 0; c < 2; ++c) {   // 32-row blocks of the 64 rows
      f32x16 s_acc, dp_acc;
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        s_acc[e] = 0.f;
        dp_acc[e] = 0.f;
      }
#pragma unroll
      for (int pn = 0; pn < NP; ++pn) {
        bf16x8 qf[8];
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) qf[ks] = *reinterpret_cast<const bf16x8*>(qt + pn * kPanel + r_off[ks] + c * 32 * kTileD * 2);
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) s_acc = mfma32(qf[ks], kreg[8 * pn + ks], s_acc);
      }
#pragma unroll
      for (int pn = 0; pn < NP; ++pn) {
        bf16x8 df[8];
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) df[ks] = *reinterpret_cast<const bf16x8*>(dot + pn * kPanel + r_off[ks] + c * 32 * kTileD * 2);
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) dp_acc = mfma32(df[ks], vreg[8 * pn + ks], dp_acc);
      }

      bf16x8 pb[2], dsb[2];
      auto elementwise = [&](auto masked) {
        constexpr bool MASKED = decltype(masked)::value;
        const bool has_doc = MASKED && (mk.flags & FLEXATTN_MASK_DOC) != 0;
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4) {
          const int r0 = 32 * c + 8 * g4 + 4 * hh;  // the lane's q rows come in runs of 4
          const f32x4 lse4 = *reinterpret_cast<const f32x4*>(sLse + buf * HQ + r0);
          const f32x4 dl4 = *reinterpret_cast<const f32x4*>(sDl + buf * HQ + r0);
          int di[4] = {0, 0, 0, 0};
          if (MASKED && has_doc) {
            const auto d4 = *reinterpret_cast<const int __attribute__((ext_vector_type(4)))*>(mk.doc_q + q0 + r0);
            di[0] = d4[0]; di[1] = d4[1]; di[2] = d4[2]; di[3] = d4[3];
          }
          float pv[4], dsv[4];
#pragma unroll
          for (int u = 0; u < 4; ++u) {
            const int e = 4 * g4 + u;
            const int i = q0 + r0 + u;
            const float tv = sm.to_log2(s_acc[e], i, k_idx);
            float pe = fast_exp2(tv + sm.bias2(i, k_idx) - lse4[u]);
            float gd = pe * (dp_acc[e] - dl4[u]) * sm.dfactor(tv, s_acc[e], i, k_idx);
            if (MASKED) {
              const bool keep = keep_elem(mk, i, k_idx, di[u], doc_j);
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

      // dv^T += dO^T P, dk^T += Q^T dS, a panel at a time (the transposed fragments of one panel are live at once)
#pragma unroll
      for (int pn = 0; pn < NP; ++pn) {
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          const int off = (32 * c + 16 * u) * kTileD * 2 + pn * kPanel;
          s16x4 dolo[4], dohi[4], qlo[4], qhi[4];
#pragma unroll
          for (int db = 0; db < 4; ++db) {
            dolo[db] = lds_read_tr16(reinterpret_cast<const bf16_t*>(dot + t_off[db][0] + off));
            dohi[db] = lds_read_tr16(reinterpret_cast<const bf16_t*>(dot + t_off[db][1] + off));
            qlo[db] = lds_read_tr16(reinterpret_cast<const bf16_t*>(qt + t_off[db][0] + off));
            qhi[db] = lds_read_tr16(reinterpret_cast<const bf16_t*>(qt + t_off[db][1] + off));
          }
#pragma unroll
          for (int db = 0; db < 4; ++db) {
            dv_acc[4 * pn + db] = mfma32(join_tr(dolo[db], dohi[db]), pb[u], dv_acc[4 * pn + db]);
            dk_acc[4 * pn + db] = mfma32(join_tr(qlo[db], qhi[db]), dsb[u], dk_acc[4 * pn + db]);
          }
          __builtin_amdgcn_sched_barrier(0);   // (keeps the next group's fragments out of this one's registers)
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
  for (int db = 0; db < 4 * NP; ++db) {
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

template <int SCORE, int NP>
static int launch_dkv_wide(const BwdArgs& a, hipStream_t stream) {
  using namespace dkv_cfg;
  constexpr int kLds = 4 * NP * kTileElems * 2 + 4 * 64 * 4;   // (Q, dO) x 2 buffers x NP panels; lse, delta x 2 buffers
  auto kern = bwd_dkv_bf16_wide_kernel<SCORE, NP>;
  static hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, kLds);
  if (attr != hipSuccess) return set_error(FLEXATTN_ELAUNCH, "hipFuncSetAttribute(dkv): %s", hipGetErrorString(attr));
  const int n_wg = a.B * a.Hkv * (a.Sk / BNK);
  hipLaunchKernelGGL(kern, dim3(n_wg), dim3(256), kLds, stream, a);
  return check_launch("flexattn_bwd_dkv bf16");
}

#ifndef FLEXATTN_CUSTOM_ONLY
// ------------------------------------------------------------------------------------------------
// Plain score: the whole main loop runs inside generated asm statements (gen_dkv_tile.py).  One
// statement executes a run of consecutive full tiles, or one partial tile with the lane's keep bits;
// C++ only finds the runs, and builds the keep bits of partial tiles.  The kernel has no static
// shared memory, so the dynamic buffer starts at LDS address 0 (the run loop toggles buffers by
// address bits).
// ------------------------------------------------------------------------------------------------
// ALIBI: the score gets slopes[h] (j - i) added (one query head per kv head only).  With j0 the middle of
// the item's kv tile, exp2(t + a (j - i)) = exp2(t - a (i - j0)) 2^(a (j - j0)): the query's share joins
// -lse in the S chain's accumulator input, the key's share is a factor of whole dk / dv rows that the
// item epilogue applies, so the tile streams are those of the plain score.
// SOFTCAP: s' = cap tanh(s / cap).  The streams turn the chain's result times 2 log2(e) sm_scale / cap, u, into r = 1 / (2^u + 1) (tanh = 1 - 2 r), the exponent (cap' - lse) - 2 cap' r with
// cap' = cap log2(e) (LDS holds cap' - lse) and dS = P dP' r (1 - r); the factor 4 of 1 - tanh^2 = 4 r (1 - r)
// goes into dk with sm_scale.
// DOCS: the mask compares document ids; those of a partial q tile are staged through LDS (stage_doc_ids).
// (A template parameter: the staging code in the kernel costs the other masks registers.)
// EXPORT: the streams also write the step's bf16 dS (without sm_scale, as the dk product takes it) to a.ds, one
// 32 KB block per (query head, kept tile pair) at (head a.ds_pairs + a.ds_col[kv tile] + place of the q tile in the
// kv tile's list) 32 KB (the index of flexattn_build_ds_index: skipped pairs take no room); inside a block wave w
// (kv columns 32 w + L % 32) writes 1 KB per (32-row q block c, 16-row half u) at 8192 w + 1024 (2 c + u), lane L
// its 8 values (rows 8 (e / 4) + 4 (L / 32) + e % 4 of the half) at 16 (2 (L % 32) + L / 32).  bwd_dq_ds.hip reads it.
template <int SCORE, bool DOCS, bool EXPORT = false>
__global__ __launch_bounds__(256, 1) void bwd_dkv_bf16_d128_plain_kernel(BwdArgs a) {
  using namespace dkv_cfg;
  static_assert(!(EXPORT && SCORE == FLEXATTN_SCORE_ALIBI), "the position-bias streams keep the key's share out of dS");
  constexpr bool ALIBI = SCORE == FLEXATTN_SCORE_ALIBI;
  constexpr bool SOFTCAP = SCORE == FLEXATTN_SCORE_SOFTCAP;
  const float cap2 = SOFTCAP ? a.score.cap * kLog2e : 0.f;
  extern __shared__ __attribute__((aligned(1024))) char smem_raw[];
  bf16_t* sT = reinterpret_cast<bf16_t*>(smem_raw);
  float* sLse = reinterpret_cast<float*>(sT + 8 * kTileElems);
  float* sDl = sLse + 2 * BQ;

  const int nKb = a.Sk / BNK;
  const int nQ = a.map.nq;
  const int n_wg = a.B * a.Hkv * nKb;
  const int group = a.Hq / a.Hkv;
  const int tid = threadIdx.x;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  const int l32 = lane & 31;
  const int hh = lane >> 5;

  // One work-group per CU when the launcher found a balanced static schedule (persistent_ok):
  // it then runs n_wg / gridDim.x work items back to back, which saves the gap between the end of a
  // work-group and the start of the next one on the CU (only one fits at a time).
  const int n_items = n_wg / (int)gridDim.x;
  const int kv_local = w * 32 + l32;
  const int row = tid & (BQ - 1);
  // waves 0, 1 turn (l, m) into -lse for rows tid & 127; waves 2, 3 store -delta
  const bool lse_wave = w < 2;
  int* sIdx = reinterpret_cast<int*>(sDl + 2 * BQ) + 4 * 32;
  unsigned char* sPart = reinterpret_cast<unsigned char*>(sIdx + MAX_LIST);  // by q tile: 1 = partial with this kv tile
  TileLoader<4> loader;
  loader.init(w, lane);

  // An item is kv tile kb of (batch, kv head) pair bhk.  Its addresses are cheap to derive from the
  // two numbers, so only those are carried from item to item.
  struct Geometry {
    int bhk, kb;
  };
  const PersistentPlan plan = persistent_plan((int)blockIdx.x, n_wg, nKb);
  // under document masks a persistent work-group takes its items from the longest-first schedule (sorted_items)
  const bool sorted = DOCS && gridDim.x != (unsigned)n_wg;
  int* sItems = reinterpret_cast<int*>(sPart + MAX_LIST) + 4 * 128;
  if (DOCS && sorted)
    sorted_items([&](int t) { return a.map.cnt[t]; }, nKb, n_wg / nKb, 1, (int)blockIdx.x, n_items, tid,
                 reinterpret_cast<int*>(smem_raw), sItems);
  auto geometry = [&](int item) {
    Geometry g;
    if (DOCS && sorted) {
      const int v = sItems[item];
      g.bhk = v >> 16;
      g.kb = v & 0xffff;
    } else {
      persistent_item(plan, (int)blockIdx.x, item, (int)gridDim.x, n_wg, nKb, g.bhk, g.kb);
    }
    g.bhk = __builtin_amdgcn_readfirstlane(g.bhk);
    g.kb = __builtin_amdgcn_readfirstlane(g.kb);
    return g;
  };
  auto kv_offset = [&](const Geometry& g) { return ((size_t)g.bhk * a.Sk + (size_t)g.kb * BNK) * D; };
  // (DOCS) document arrays given per batch entry: the rows of the entry of a (batch, kv head) pair
  auto doc_rows = [&](int bhk, int S) { return (DOCS && a.mask.doc_batched) ? (size_t)(bhk / a.Hkv) * (size_t)S : (size_t)0; };
  // (EXPORT) dS block of the item's kv tile against the first q tile of its list, for the group's first query
  // head: the blocks of a head are ordered kv tile by kv tile (a.ds_col[kb] pairs lie before kv tile kb), and
  // along each kv tile's q list
  auto ds_base = [&](const Geometry& g) {
    const int first = __builtin_amdgcn_readfirstlane(a.ds_col[g.kb]);
    return static_cast<char*>(a.ds) + (((size_t)g.bhk * group) * (size_t)a.ds_pairs + (size_t)first) * kDsBlockBytes;
  };
  // first row of the group's first query head: (b Hq + hk group) Sq with bhk = b Hkv + hk
  auto first_row = [&](const Geometry& g) { return (size_t)g.bhk * group * a.Sq; };

  // Everything an item needs from global memory before its first step is fetched while the previous
  // item runs: plain loads whose values are not touched until that item's last step is done.  (They
  // live in v[192:255] and the low registers, which the run loop leaves alone.)
  constexpr int kListRegs = PREFETCH_LIST / 256;
  struct ItemRegs {
    RowBlock k, v;                 // the wave's 32 K / V rows (full-row layout, see rows_load)
    int doc, n_tiles, qb0;         // list length and its first entry
    int qlo, qhi;                  // (DOCS) first and last q position that carries the column's document id, where known
    float na2;                     // -slopes[head] log2(e) (ALIBI)
    int idx[kListRegs];            // q list entries tid + 256 j
    unsigned char part[kListRegs]; // state of q tile tid + 256 j against this kv tile
  };
  // (opaque(): addresses derived from its result are computed where they are used instead of once
  // before the item loop, where they would have to be kept, spilled, through every run)
  auto opaque = [](int x) {
    asm volatile("" : "+v"(x));
    return x;
  };
  auto fetch = [&](const Geometry& g, ItemRegs& r) {
    const int tid_here = opaque(tid);
    const bf16_t* Kg = static_cast<const bf16_t*>(a.k) + kv_offset(g);
    const bf16_t* Vg = static_cast<const bf16_t*>(a.v) + kv_offset(g);
    rows_load(r.k, Kg + (size_t)(tid_here >> 6) * 32 * D, tid_here & 63);
    rows_load(r.v, Vg + (size_t)(tid_here >> 6) * 32 * D, tid_here & 63);
    const size_t dk_rows = doc_rows(g.bhk, a.Sk);
    r.doc = (a.mask.flags & FLEXATTN_MASK_DOC) ? a.mask.doc_k[dk_rows + g.kb * BNK + kv_local] : 0;
    if constexpr (DOCS) {
      const bool have = a.mask.doc_k_range != nullptr;
      r.qlo = have ? a.mask.doc_k_range[2 * (dk_rows + g.kb * BNK + kv_local)] : 0;
      r.qhi = have ? a.mask.doc_k_range[2 * (dk_rows + g.kb * BNK + kv_local) + 1] : 0;
    }
    const int* tile_idx = a.map.idx + (size_t)g.kb * nQ;
    r.n_tiles = a.map.cnt[g.kb];
    r.qb0 = tile_idx[0];  // (nQ >= 1: always readable; used only if the list is not empty)
    r.na2 = ALIBI ? -a.score.slopes[g.bhk % a.Hkv] * kLog2e : 0.f;
#pragma unroll
    for (int j = 0; j < kListRegs; ++j) {
      const int t = tid_here + 256 * j;
      r.idx[j] = (t < nQ) ? tile_idx[t] : 0;  // (slots past the list length hold no valid entry and are never used)
      r.part[j] = (t < nQ) ? a.map.state[(size_t)t * a.map.nk + g.kb] : 0;
    }
  };
  // What is left of an item's fetched values once its K / V fragments sit in their registers.
  struct ItemHead {
    int doc, n_tiles, qb0, qlo, qhi;
    float na2;
    int idx[kListRegs];
    unsigned char part[kListRegs];
  };
  PinnedState st;
  // The streams multiply the fp32 products Q K^T by c2 (sm_scale * log2(e); softcap: 2 log2(e) sm_scale / cap)
  // on their way into the exponent; K itself goes in as it is.
  const float c2 = SOFTCAP ? 2.f * kLog2e * a.sm_scale / a.score.cap : a.sm_scale * kLog2e;
  auto scaled = [](unsigned two) { return two; };
  // (`stage`: the wave's 16 KB of a free LDS step buffer)
  auto consume = [&](const ItemRegs& r, ItemHead& c, char* stage) {
    u32x4 kw[8], vw[8];
    const int lane_here = opaque(lane);
    rows_to_fragments(r.k, stage, lane_here, kw);
    rows_to_fragments(r.v, stage + 8192, lane_here, vw);
#define FA_PUT(KS, KR, VR)                                                                                    \
  asm volatile(FA_DKV_PUT_KV_##KS                                                                             \
               : "={" KR "}"(st.k[KS]), "={" VR "}"(st.v[KS])                                                 \
               : "v"(scaled(kw[KS][0])), "v"(scaled(kw[KS][1])), "v"(scaled(kw[KS][2])), "v"(scaled(kw[KS][3])), \
                 "v"(vw[KS][0]), "v"(vw[KS][1]), "v"(vw[KS][2]), "v"(vw[KS][3]));
    FA_PUT(0, "a[128:131]", "a[160:163]") FA_PUT(1, "a[132:135]", "a[164:167]")
    FA_PUT(2, "a[136:139]", "a[168:171]") FA_PUT(3, "a[140:143]", "a[172:175]")
    FA_PUT(4, "a[144:147]", "a[176:179]") FA_PUT(5, "a[148:151]", "a[180:183]")
    FA_PUT(6, "a[152:155]", "a[184:187]") FA_PUT(7, "a[156:159]", "a[188:191]")
#undef FA_PUT
    c.doc = r.doc;
    if constexpr (DOCS) { c.qlo = r.qlo; c.qhi = r.qhi; }
    c.n_tiles = __builtin_amdgcn_readfirstlane(r.n_tiles);
    c.qb0 = __builtin_amdgcn_readfirstlane(r.qb0);
    c.na2 = ALIBI ? __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, r.na2))) : 0.f;
#pragma unroll
    for (int j = 0; j < kListRegs; ++j) {
      c.idx[j] = r.idx[j];
      c.part[j] = r.part[j];
    }
  };

  // Byte addresses of the lane's operand fragments and row values in LDS step buffer 0 (see
  // tile_io.hpp); the run loop flips them between the two buffers together with `buf`, across items too.
  const int r_sw = swz(l32);
  const int t_row = 4 * hh + ((lane & 15) >> 2);
  const int t_chunk = 2 * ((lane & 31) >> 4) + ((lane & 3) >> 1);
  const int t_half = 4 * (lane & 1);
  const unsigned base0 = (unsigned)(size_t)sT;
  unsigned ra[8], ta[8];
#pragma unroll
  for (int ks = 0; ks < 8; ++ks) ra[ks] = base0 + (unsigned)(l32 * kTileD + (((2 * ks + hh) ^ r_sw) << 3)) * 2u;
#pragma unroll
  for (int i = 0; i < 8; ++i)
    ta[i] = base0 + (unsigned)(tile_off(t_row + 8 * (i & 1), 4 * (i >> 1) + t_chunk) + t_half) * 2u;
  unsigned la = (unsigned)(size_t)(sLse + 4 * hh);
  unsigned lw = (unsigned)(size_t)((lse_wave ? sLse : sDl) + BQ + row);  // this lane's row value of the NEXT buffer
  int buf = 0;
  bool resident = false;  // the item's first step was already copied into buffer `buf` by the previous item's last step

  ItemRegs pre;
  ItemHead cur;
  Geometry geo = geometry(0);
  fetch(geo, pre);
  consume(pre, cur, reinterpret_cast<char*>(sT + 4 * kTileElems) + w * 16384);

  for (int item = 0; item < n_items; ++item) {
  const int kb = geo.kb;
  const int k_idx = kb * BNK + kv_local;
  const size_t kv_off = kv_offset(geo);
  const size_t rows0 = first_row(geo);
  const bf16_t* Qg = static_cast<const bf16_t*>(a.q) + rows0 * D;
  const bf16_t* dOg = static_cast<const bf16_t*>(a.dout) + rows0 * D;
  const float* rowa = (lse_wave ? a.l : a.delta) + rows0;
  const float* rowb = (lse_wave ? a.m : a.delta) + rows0;
  const int doc_j = cur.doc;
  // (DOCS) with sorted q ids the queries of the column's document are one interval: the keep bits of a partial tile
  // then have a closed form (keep_bits32_range) and no ids are read
  const bool ranged = DOCS && a.mask.doc_k_range != nullptr && keep_bits_have_range(a.mask);
  const int* tile_idx = a.map.idx + (size_t)kb * nQ;
  const int n_tiles = cur.n_tiles;
  const int n_iter = n_tiles * group;
  const float na2 = cur.na2;
  const int kc = kb * BNK + BNK / 2;  // j0
  if (item > 0) __syncthreads();  // the previous item's list and row values are dead from here

  asm volatile(FA_DKV_ZERO_ACC
               : "={a[0:15]}"(st.dv[0]), "={a[16:31]}"(st.dv[1]), "={a[32:47]}"(st.dv[2]), "={a[48:63]}"(st.dv[3]),
                 "={a[64:79]}"(st.dk[0]), "={a[80:95]}"(st.dk[1]), "={a[96:111]}"(st.dk[2]), "={a[112:127]}"(st.dk[3]));

  // The kv tile's q list and which q tiles are partial against it, cached in LDS: finding runs of
  // full tiles then costs no global loads.
  const int tid_p = opaque(tid);  // (fresh per item: see opaque())
#pragma unroll
  for (int j = 0; j < kListRegs; ++j) {
    const int t = tid_p + 256 * j;
    if (t < nQ) {
      sIdx[t] = cur.idx[j];
      sPart[t] = cur.part[j] == 1 ? 1 : 0;
    }
  }
  if (nQ > PREFETCH_LIST) {
    // columns longer than the prefetched part (more than 131072 tokens): the rest straight from global memory
    // (an item is then thousands of steps long: the wait does not show)
    for (int t = PREFETCH_LIST + tid_p; t < nQ; t += 256) {
      sIdx[t] = tile_idx[t];
      sPart[t] = a.map.state[(size_t)t * a.map.nk + kb] == 1 ? 1 : 0;
    }
  }
  if (n_iter > 0 && !resident) {
    // first step into the current buffer: tiles (LDS-direct) and the lane's row value
    const size_t r0 = (size_t)cur.qb0 * BQ;
    bf16_t* dst = sT + (size_t)buf * 4 * kTileElems;
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      loader.load(Qg + (r0 + half * kTileRows) * D, dst + half * kTileElems);
      loader.load(dOg + (r0 + half * kTileRows) * D, dst + (2 + half) * kTileElems);
    }
    const int row_p = tid_p & (BQ - 1);
    const float x = rowa[r0 + row_p], y = rowb[r0 + row_p];
    if (lse_wave) {  // (the streams want -lse: it is the accumulator input of the S chain)
      // (one fused multiply-add, as the streams' turn-around rounds the row values of every later step: an item's
      // results then do not depend on whether its first step was set up here or by the last step of the item before it)
      float neg_lse = (x > 0.f) ? -__builtin_fmaf(y, kLog2e, log2f(x)) : -__builtin_huge_valf();
      if (ALIBI) neg_lse = __builtin_fmaf((float)((int)r0 + row_p - kc), na2, neg_lse);
      if (SOFTCAP) neg_lse += cap2;
      sLse[buf * BQ + row_p] = neg_lse;
    } else {  // (and -delta, for the dP chain)
      sDl[buf * BQ + row_p] = -x;
    }
    wait_vmem_all();
  }
  resident = false;
  __syncthreads();
  // The next item's list lands while this item runs.  (The last item fetches itself again: every
  // path then redefines the fetched registers, so none of them has to live through the run loop.)
  const bool has_next = item + 1 < n_items;
  const Geometry geo_n = has_next ? geometry(item + 1) : geo;
  fetch(geo_n, pre);

  const unsigned tid4 = (unsigned)row * 4u;
  // (EXPORT) first dS block of this item and of the next one
  const size_t ds_item = EXPORT ? (size_t)ds_base(geo) : 0;
  const size_t ds_item_n = EXPORT ? (size_t)ds_base(geo_n) : 0;
  // Work-group constants of the run loop, one 32-dword table per wave behind the row values
  // (order: TABLE in gen_dkv_tile.py; the second half names the next item's first step, see below).
  // Written and read by the same wave: no barrier needed.
  unsigned* tbl = reinterpret_cast<unsigned*>(sDl + 2 * BQ) + w * 32;
  if (lane == 0) {
    tbl[0] = (unsigned)n_tiles;
    tbl[1] = (unsigned)(group - 1);
    tbl[2] = (unsigned)a.Sq;
    tbl[3] = base0 + (unsigned)w * 4096u;  // LDS address of the wave's first 1 KB block in buffer 0
    tbl[4] = __builtin_bit_cast(unsigned, SOFTCAP ? cap2 : na2);
    tbl[5] = lse_wave ? 1u : 0u;
    tbl[6] = (unsigned)(size_t)tile_idx;
    tbl[7] = (unsigned)((size_t)tile_idx >> 32);
    tbl[8] = (unsigned)(size_t)Qg;
    tbl[9] = (unsigned)((size_t)Qg >> 32);
    tbl[10] = (unsigned)(size_t)dOg;
    tbl[11] = (unsigned)((size_t)dOg >> 32);
    tbl[12] = (unsigned)(size_t)rowa;
    tbl[13] = (unsigned)((size_t)rowa >> 32);
    tbl[14] = (unsigned)(size_t)rowb;
    tbl[15] = (unsigned)((size_t)rowb >> 32);
    if (EXPORT) {
      const size_t ds0 = ds_item;
      tbl[28] = (unsigned)ds0;
      tbl[29] = (unsigned)(ds0 >> 32);
      tbl[30] = (unsigned)a.ds_pairs;   // blocks per query head
      tbl[31] = 0u;
    }
  }
  const unsigned tbl_addr = (unsigned)(size_t)tbl;

  // Step `it` is q tile tile_idx[it % n_tiles] of query head it / n_tiles of the group.  Carried:
  // the list positions of steps it + 1 and it + 2, the head of step it + 1, its q block index.
  int it = 0, g1 = 0, p1 = 1, p2 = 2;
  if (p1 >= n_tiles) { p1 -= n_tiles; g1 = 1; }
  if (p2 >= n_tiles) p2 -= n_tiles;
  if (p2 >= n_tiles) p2 -= n_tiles;
  int qb1 = (n_iter > 0) ? __builtin_amdgcn_readfirstlane(sIdx[p1]) : 0;

  while (it < n_iter) {
    // position of step `it` in the list, its q block and state
    int p0 = p1 - 1;
    if (p0 < 0) p0 += n_tiles;
    const int qb = __builtin_amdgcn_readfirstlane(sIdx[p0]);
    const bool partial = __builtin_amdgcn_readfirstlane((int)sPart[qb]) == 1;
    int it_end = it + 1;
    unsigned km[2] = {0u, 0u};
    if (partial) {
      // the lane's keep bits: element e of q block c sits at bit 16 (c & 1) + e of km[c >> 1]
      const int q0 = qb * BQ;
      if constexpr (DOCS) {
        int* sDoc = reinterpret_cast<int*>(sPart + MAX_LIST) + w * 128;  // the wave's stage for document ids
        if (ranged) {
#pragma unroll
          for (int half = 0; half < 2; ++half)
            km[half] = keep_bits32_range<false>(a.mask, k_idx, q0 + 64 * half + 4 * hh, cur.qlo, cur.qhi);
        } else {
          stage_doc_ids(a.mask.doc_q + doc_rows(geo.bhk, a.Sq), q0, q0 + 64, lane, sDoc);
#pragma unroll
          for (int half = 0; half < 2; ++half)
            km[half] = keep_bits32_staged<false>(a.mask, k_idx, q0 + 64 * half + 4 * hh, doc_j, sDoc + 64 * half + 4 * hh);
        }
      } else {
#pragma unroll
        for (int half = 0; half < 2; ++half)
          km[half] = keep_bits32<false>(a.mask, k_idx, q0 + 64 * half + 4 * hh, doc_j, a.mask.doc_q);
      }
    } else {
      // the run of full tiles ends before the next partial one: lanes look 64 steps ahead at a time
      bool found = false;
      while (!found && it_end < n_iter) {
        const int j = it_end + lane;
        bool is_partial = false;
        if (j < n_iter) {
          const int pj = (p0 + (j - it)) % n_tiles;
          is_partial = sPart[sIdx[pj]] == 1;
        }
        const unsigned long long hits = __ballot(is_partial);
        if (hits != 0ull) {
          it_end += __builtin_ctzll(hits);
          found = true;
        } else {
          it_end = (it_end + 64 < n_iter) ? it_end + 64 : n_iter;
        }
      }
    }
    it_end = __builtin_amdgcn_readfirstlane(it_end);
    // The run that ends the item copies the next item's first step during its last step (bit 1 of
    // the flags; the table's second half says where it is).  The fetched values are first touched
    // here, an item's length after their loads were issued.
    int flags = partial ? 1 : 0;
    if (it_end == n_iter && has_next) {
      const int nt = __builtin_amdgcn_readfirstlane(pre.n_tiles);
      if (nt > 0) {
        flags |= 2;
        const int qb0_n = __builtin_amdgcn_readfirstlane(pre.qb0);
        const size_t rows_n = first_row(geo_n);
        const bf16_t* Qg_n = static_cast<const bf16_t*>(a.q) + rows_n * D;
        const bf16_t* dOg_n = static_cast<const bf16_t*>(a.dout) + rows_n * D;
        const float* rowa_n = (lse_wave ? a.l : a.delta) + rows_n;
        const float* rowb_n = (lse_wave ? a.m : a.delta) + rows_n;
        if (lane == 0) {
          tbl[16] = (unsigned)(size_t)Qg_n;
          tbl[17] = (unsigned)((size_t)Qg_n >> 32);
          tbl[18] = (unsigned)(size_t)dOg_n;
          tbl[19] = (unsigned)((size_t)dOg_n >> 32);
          tbl[20] = (unsigned)(size_t)rowa_n;
          tbl[21] = (unsigned)((size_t)rowa_n >> 32);
          tbl[22] = (unsigned)(size_t)rowb_n;
          tbl[23] = (unsigned)((size_t)rowb_n >> 32);
          tbl[24] = (unsigned)qb0_n;
          if (ALIBI) {
            tbl[26] = __builtin_bit_cast(unsigned, pre.na2);
            tbl[27] = (unsigned)(geo_n.kb * BNK + BNK / 2);
          }
          if (EXPORT) {
            const size_t ds_n = ds_item_n;
            tbl[26] = (unsigned)ds_n;
            tbl[27] = (unsigned)(ds_n >> 32);
          }
        }
        resident = true;
      }
    }
    // no scalar operands (see gen_dkv_tile.py): the loop state travels in VGPRs
#define FA_DKV_CALL(RUN, CLOB_MORE, ...)                                                                                 \
  asm volatile(RUN                                                                                               \
               : FA_DKV_PINNED(st), [it] "+v"(it), [p1] "+v"(p1), [g1] "+v"(g1), [p2] "+v"(p2), [qb1] "+v"(qb1), \
                 [buf] "+v"(buf), [r0] "+v"(ra[0]), [r1] "+v"(ra[1]), [r2] "+v"(ra[2]), [r3] "+v"(ra[3]),       \
                 [r4] "+v"(ra[4]), [r5] "+v"(ra[5]), [r6] "+v"(ra[6]), [r7] "+v"(ra[7]), [t0] "+v"(ta[0]),       \
                 [t1] "+v"(ta[1]), [t2] "+v"(ta[2]), [t3] "+v"(ta[3]), [t4] "+v"(ta[4]), [t5] "+v"(ta[5]),       \
                 [t6] "+v"(ta[6]), [t7] "+v"(ta[7]), [la] "+v"(la), [lw] "+v"(lw)                                \
               : [it_end] "v"(it_end), [partial] "v"(flags), [tbl] "v"(tbl_addr), [g0] "v"(loader.goff[0]),      \
                 [g1v] "v"(loader.goff[1]), [g2] "v"(loader.goff[2]), [g3] "v"(loader.goff[3]), [m0] "v"(km[0]), \
                 [m1] "v"(km[1]), [tid4] "v"(tid4), [c2v] "v"(c2), ##__VA_ARGS__                                                \
               : "memory", "scc", "vcc", "m0", FA_DKV_RUN_SGPRS, "v67", FA_DKV_TILE_CLOBBERS CLOB_MORE)
#define FA_DKV_ALIBI_CLOBBERS , "s101"
#define FA_DKV_DS_CLOBBERS , "s52", "s53", "s54", "s55", "s56", "s57", "s58", "s59"
    if constexpr (EXPORT) {
      // dS block of step `it` (head it / n_tiles of the group, place p0 in the q list) and the lane's place in
      // the wave's part
      const size_t ds_cur = ds_item + ((size_t)(it / n_tiles) * (size_t)a.ds_pairs + (size_t)p0) * kDsBlockBytes;
      const unsigned dslo = (unsigned)ds_cur, dshi = (unsigned)(ds_cur >> 32);
      const unsigned dsv = 8192u * (unsigned)w + 4096u + 16u * (unsigned)(2 * l32 + hh);
      if constexpr (SOFTCAP) {
        const float k2 = -2.f * cap2;
        FA_DKV_CALL(FA_DKV_RUN_SOFTCAP_DS, FA_DKV_ALIBI_CLOBBERS FA_DKV_DS_CLOBBERS, [k2] "v"(k2), [dslo] "v"(dslo),
                    [dshi] "v"(dshi), [dsv] "v"(dsv));
      } else {
        FA_DKV_CALL(FA_DKV_RUN_DS, FA_DKV_DS_CLOBBERS, [dslo] "v"(dslo), [dshi] "v"(dshi), [dsv] "v"(dsv));
      }
    } else if constexpr (ALIBI) {
      FA_DKV_CALL(FA_DKV_RUN_ALIBI, FA_DKV_ALIBI_CLOBBERS, [kc] "v"(kc));
    } else if constexpr (SOFTCAP) {
      const float k2 = -2.f * cap2;
      FA_DKV_CALL(FA_DKV_RUN_SOFTCAP, FA_DKV_ALIBI_CLOBBERS, [k2] "v"(k2));
    } else {
      FA_DKV_CALL(FA_DKV_RUN, );
    }
#undef FA_DKV_CALL
#undef FA_DKV_DS_CLOBBERS
#undef FA_DKV_ALIBI_CLOBBERS
    it = __builtin_amdgcn_readfirstlane(it);
    p1 = __builtin_amdgcn_readfirstlane(p1);
    buf = __builtin_amdgcn_readfirstlane(buf);
  }

  // ---- item epilogue ----
  // The next item's K / V fragments go into their registers before this item's stores are issued
  // (their loads are long done; behind the stores the wait would include the stores).
  // (buffer `buf` may hold the next item's first step: the other one is free)
  char* stage = reinterpret_cast<char*>(sT + (size_t)(buf ^ 1) * 4 * kTileElems) + w * 16384;
  consume(pre, cur, stage);

  // dk / dv: bf16 rows staged through the wave's 16 KB of the free LDS step buffer (16-byte chunks XOR-swizzled
  // by row), so that every store instruction writes four complete 256-byte rows.
  {
    const int lane_here = opaque(lane);
    const int row_here = lane_here & 31;
    const unsigned wr = (unsigned)row_here * 256u + 8u * (unsigned)(lane_here >> 5);
#define FA_GET(T, SRC, REG, MAT, DB, SCALE)                                                                        \
  {                                                                                                                \
    float x[16];                                                                                                   \
    asm volatile(FA_DKV_GET_ACC_##T                                                                                \
                 : "=v"(x[0]), "=v"(x[1]), "=v"(x[2]), "=v"(x[3]), "=v"(x[4]), "=v"(x[5]), "=v"(x[6]), "=v"(x[7]), \
                   "=v"(x[8]), "=v"(x[9]), "=v"(x[10]), "=v"(x[11]), "=v"(x[12]), "=v"(x[13]), "=v"(x[14]),        \
                   "=v"(x[15])                                                                                     \
                 : "{" REG "}"(SRC));                                                                              \
    _Pragma("unroll") for (int g = 0; g < 4; ++g) {                                                                \
      const bf16x2 lo = pack_bf16(x[4 * g] * SCALE, x[4 * g + 1] * SCALE);                                         \
      const bf16x2 hi = pack_bf16(x[4 * g + 2] * SCALE, x[4 * g + 3] * SCALE);                                     \
      const bf16x4 out = {lo[0], lo[1], hi[0], hi[1]};                                                             \
      *reinterpret_cast<bf16x4*>(stage + MAT * 8192 + wr + (unsigned)(((4 * DB + g) ^ (row_here & 15)) << 4)) = out; \
    }                                                                                                              \
  }
    // the streams leave the constant sm_scale out of dS: dk takes it here; and both take the key's
    // share of a position bias
    const float ej = ALIBI ? exp2f(-na2 * (float)((lane_here & 31) + 32 * w - BNK / 2)) : 1.f;
    const float ek = (SOFTCAP ? 4.f : 1.f) * a.sm_scale * ej;
    FA_GET(0, st.dv[0], "a[0:15]", 1, 0, ej) FA_GET(1, st.dv[1], "a[16:31]", 1, 1, ej)
    FA_GET(2, st.dv[2], "a[32:47]", 1, 2, ej) FA_GET(3, st.dv[3], "a[48:63]", 1, 3, ej)
    FA_GET(4, st.dk[0], "a[64:79]", 0, 0, ek) FA_GET(5, st.dk[1], "a[80:95]", 0, 1, ek)
    FA_GET(6, st.dk[2], "a[96:111]", 0, 2, ek) FA_GET(7, st.dk[3], "a[112:127]", 0, 3, ek)
#undef FA_GET
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
    bf16_t* dKg = static_cast<bf16_t*>(a.dk) + kv_off + (size_t)(w * 32) * D;
    bf16_t* dVg = static_cast<bf16_t*>(a.dv) + kv_off + (size_t)(w * 32) * D;
    const int chunk = lane_here & 15;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int r = 4 * i + (lane_here >> 4);
      const unsigned rd = (unsigned)r * 256u + (unsigned)((chunk ^ (r & 15)) << 4);
      const u32x4 kx = *reinterpret_cast<const u32x4*>(stage + rd);
      const u32x4 vx = *reinterpret_cast<const u32x4*>(stage + 8192 + rd);
      *reinterpret_cast<u32x4*>(dKg + (size_t)r * D + chunk * 8) = kx;
      *reinterpret_cast<u32x4*>(dVg + (size_t)r * D + chunk * 8) = vx;
    }
  }
  geo = geo_n;
  }  // work items
}

#endif  // FLEXATTN_CUSTOM_ONLY

template <int SCORE, bool EXPORT>
static int launch_dkv_on(const BwdArgs& a, hipStream_t stream) {
  using namespace dkv_cfg;
  auto kern = bwd_dkv_bf16_d128_kernel<SCORE, EXPORT>;
  static hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES);
  if (attr != hipSuccess) return set_error(FLEXATTN_ELAUNCH, "hipFuncSetAttribute(dkv): %s", hipGetErrorString(attr));
  const int n_wg = a.B * a.Hkv * (a.Sk / BNK);
  hipLaunchKernelGGL(kern, dim3(n_wg), dim3(256), LDS_BYTES, stream, a);
  return check_launch("flexattn_bwd_dkv bf16");
}
template <int SCORE>
static int launch_dkv(const BwdArgs& a, hipStream_t stream) {
  return a.ds != nullptr ? launch_dkv_on<SCORE, true>(a, stream) : launch_dkv_on<SCORE, false>(a, stream);
}

#ifndef FLEXATTN_CUSTOM_ONLY
template <int SCORE, bool DOCS, bool EXPORT>
static int launch_dkv_plain_on(const BwdArgs& a, hipStream_t stream) {
  using namespace dkv_cfg;
  auto kern = bwd_dkv_bf16_d128_plain_kernel<SCORE, DOCS, EXPORT>;
  static hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES);
  if (attr != hipSuccess) return set_error(FLEXATTN_ELAUNCH, "hipFuncSetAttribute(dkv): %s", hipGetErrorString(attr));
  const int n_wg = a.B * a.Hkv * (a.Sk / BNK);
  // (persistent_ok's schedule balances masks whose work per tile is linear in the tile index; document
  // masks take the longest-first schedule of sorted_items; what fits neither runs one item per work-group)
  const bool persistent = DOCS ? sorted_schedule_ok(n_wg, a.Sk / BNK) : persistent_ok(n_wg, a.Sk / BNK);
  const int grid = (persistent && n_wg > 256) ? 256 : n_wg;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(256), LDS_BYTES, stream, a);
  return check_launch("flexattn_bwd_dkv bf16");
}

template <int SCORE>
static int launch_dkv_plain(const BwdArgs& a, hipStream_t stream) {
  if constexpr (SCORE != FLEXATTN_SCORE_ALIBI) {
    if (a.ds != nullptr)
      return (a.mask.flags & FLEXATTN_MASK_DOC) ? launch_dkv_plain_on<SCORE, true, true>(a, stream)
                                                : launch_dkv_plain_on<SCORE, false, true>(a, stream);
  }
  return (a.mask.flags & FLEXATTN_MASK_DOC) ? launch_dkv_plain_on<SCORE, true, false>(a, stream)
                                            : launch_dkv_plain_on<SCORE, false, false>(a, stream);
}

#endif  // FLEXATTN_CUSTOM_ONLY

// Whether a request runs the generated-stream dk/dv kernel (else the one with a compiled main loop): the stream
// caches the q tile list in LDS, has no additive bias, serves the global position bias for one query head per kv
// head only, and a functor library of a compiled score function has no streams at all.
bool bwd_dkv_bf16_d128_on_stream(int kind, int flags, int nq, bool has_ab, int Hq, int Hkv) {
#ifdef FLEXATTN_CUSTOM_ONLY
  (void)kind; (void)flags; (void)nq; (void)has_ab; (void)Hq; (void)Hkv;
  return false;
#else
  const bool stream_ok = !(flags & FLEXATTN_FLAG_COMPILED_LOOP) && nq <= dkv_cfg::MAX_LIST && !has_ab;
  switch (kind) {
    case FLEXATTN_SCORE_NONE:
    case FLEXATTN_SCORE_SOFTCAP: return stream_ok;
    case FLEXATTN_SCORE_ALIBI: return stream_ok && Hq == Hkv;
  }
  return false;
#endif
}

int bwd_dkv_bf16_d128(const BwdArgs& a, hipStream_t stream) {
#ifdef FLEXATTN_CUSTOM_ONLY
  switch (a.score.kind) {
    case FLEXATTN_SCORE_NONE: return launch_dkv<FLEXATTN_SCORE_NONE>(a, stream);
    case FLEXATTN_SCORE_CUSTOM: return launch_dkv<FLEXATTN_SCORE_CUSTOM>(a, stream);
  }
  return set_error(FLEXATTN_ENOTSUP, "this functor library holds the plain and the compiled score function only (kind %d asked)", a.score.kind);
#else
  const bool on_stream = bwd_dkv_bf16_d128_on_stream(a.score.kind, a.flags, a.map.nq, a.score.ab != nullptr, a.Hq, a.Hkv);
  switch (a.score.kind) {
    case FLEXATTN_SCORE_NONE:
      return on_stream ? launch_dkv_plain<FLEXATTN_SCORE_NONE>(a, stream) : launch_dkv<FLEXATTN_SCORE_NONE>(a, stream);
    case FLEXATTN_SCORE_ALIBI:
      return on_stream ? launch_dkv_plain<FLEXATTN_SCORE_ALIBI>(a, stream) : launch_dkv<FLEXATTN_SCORE_ALIBI>(a, stream);
    case FLEXATTN_SCORE_SOFTCAP:
      return on_stream ? launch_dkv_plain<FLEXATTN_SCORE_SOFTCAP>(a, stream) : launch_dkv<FLEXATTN_SCORE_SOFTCAP>(a, stream);
    case FLEXATTN_SCORE_ALIBI_TILE: return launch_dkv<FLEXATTN_SCORE_ALIBI_TILE>(a, stream);
  }
  return set_error(FLEXATTN_EINVAL, "unknown score kind %d", a.score.kind);
#endif
}

// Head dim 256: the kernel with a compiled main loop (two 128-column panels per row), every score kind.
int bwd_dkv_bf16_d256(const BwdArgs& a, hipStream_t stream) {
  switch (a.score.kind) {
    case FLEXATTN_SCORE_NONE: return launch_dkv_wide<FLEXATTN_SCORE_NONE, 2>(a, stream);
#ifdef FLEXATTN_CUSTOM_ONLY
    case FLEXATTN_SCORE_CUSTOM: return launch_dkv_wide<FLEXATTN_SCORE_CUSTOM, 2>(a, stream);
#else
    case FLEXATTN_SCORE_ALIBI: return launch_dkv_wide<FLEXATTN_SCORE_ALIBI, 2>(a, stream);
    case FLEXATTN_SCORE_SOFTCAP: return launch_dkv_wide<FLEXATTN_SCORE_SOFTCAP, 2>(a, stream);
    case FLEXATTN_SCORE_ALIBI_TILE: return launch_dkv_wide<FLEXATTN_SCORE_ALIBI_TILE, 2>(a, stream);
#endif
  }
  return set_error(FLEXATTN_ENOTSUP, "score kind %d is not in this library", a.score.kind);
}

void bwd_dkv_bf16_d128_tile(int* bq, int* bk) {
  *bq = dkv_cfg::BQ;
  *bk = dkv_cfg::BNK;
}

}  // namespace fa
