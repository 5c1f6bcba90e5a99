// dq from exported dS (bf16, head dim 128): dq = out_scale * dS K, one contraction per (q tile, kv tile) pair
// instead of the three of the recomputing dq kernel (S = Q K^T, dP = dO V^T, dq += dS K).
//
// The dk/dv stream kernel (bwd_dkv_bf16.hip, EXPORT) leaves every step's bf16 dS in a buffer of 32 KB blocks, one
// per (query head, kept pair of a 128-row q tile and a 128-column kv tile) in the register layout it has there (a
// lane owns one kv column); block of pair (qb, kb) of head bh: bh ds_pairs + ds_rank[qb nk + kb].
// This kernel walks a q tile's row list of the same 128 x 128 block map, copies dS blocks and K tiles
// global -> LDS (global_load_lds_dwordx4, no registers in between) through rings of stages, and reads both
// operands with transposing LDS reads: computed transposed, dq^T[d, i] += sum_j K^T[d, j] dS^T[j, i], the lane
// that owned kv column j in the dk/dv kernel wrote 8 q rows of it contiguously, which is what
// ds_read_b64_tr_b16 turns into "lane owns q row i, 4 consecutive j".  The kernel moves 32 KB of dS and 32 KB of K
// per 32 MFMAs and computing wave; the matrix pipe is busy a quarter of the time and the copies bound the launch.
// On B=4, H=32, S=4096 causal (2.2 GB of dS, as many bytes of K from the L2): 0.51 ms; the same launch without the
// LDS reads and MFMAs 0.50 ms; the dS copies alone 0.41 ms (5.4 TB/s, what 80 KB in flight per CU draw from HBM:
// the rings are the buffer of the bytes in flight and the LDS holds no deeper ones next to the K ring), the K copies
// alone 0.18 ms.  Ring depths of 4-6 (dS) and 3-5 (K) stages time alike; two K stages, or one work-group per CU
// with deeper rings, are 15-20 % slower.
//
// Layout of a dS block (written by the dk/dv kernel): kv columns 32 w' + jj (w' = 0..3), q rows 32 c + 16 u + ii:
// byte 8192 w' + 1024 (2 c + u) + 16 (2 jj + hi) + 8 g + 2 e holds row ii = 8 g + 4 hi + e.
#include "launch.hpp"
#include "tile_io.hpp"

namespace fa {

namespace dqds_cfg {
constexpr int BQ = 128;
constexpr int BNK = 128;
constexpr int D = 128;
constexpr int STAGE_KV = 32;                       // kv columns per pipeline stage: one wave's share of a dS block
constexpr int PARTS = BNK / STAGE_KV;              // stages per kv tile
constexpr int DS_STAGE_BYTES = BQ * STAGE_KV * 2;  // 8 KB
constexpr int K_STAGE_BYTES = STAGE_KV * D * 2;    // 8 KB: 32 rows of a K tile in the layout of tile_io.hpp
#ifndef DQDS_NDS
#define DQDS_NDS 6
#define DQDS_NK 3
#define DQDS_OCC 2
#endif
#ifndef DQDS_PRODUCERS
#define DQDS_PRODUCERS 1
#endif
// Two rings of stages in LDS.  dS comes from HBM and is read once: the rate depends on the bytes in flight per CU
// (a plain streaming read on this GPU: 32 KB in flight per CU 2.9 TB/s, 64 KB 4.8 TB/s, 128 KB and more 6.4 TB/s),
// so its ring is deep; a head's K tiles are shared by the head's q tiles and come from the XCD's L2.
constexpr int NDS = DQDS_NDS;
constexpr int NK = DQDS_NK;
constexpr int OCC = DQDS_OCC;                      // work-groups per CU
// Waves 4-7 of a work-group only copy (4, 5: dS; 6, 7: K) and waves 0-3 only compute: an LDS-direct copy holds the
// wave that issues it until the texture path takes it (about 175 cycles per 1 KB copy when every work-group of the
// CU copies), which the computing waves would otherwise sit out between their MFMAs (2 % of the launch).
constexpr bool PRODUCERS = DQDS_PRODUCERS != 0;
constexpr int THREADS = PRODUCERS ? 512 : 256;
constexpr int MAX_LIST = 1024;
constexpr int K_RING = NDS * DS_STAGE_BYTES;       // LDS offset of the K ring
constexpr int LDS_BYTES = NDS * DS_STAGE_BYTES + NK * K_STAGE_BYTES + MAX_LIST * 4;
constexpr size_t kDsBlockBytes = (size_t)BQ * BNK * 2;
static_assert(NK >= 2 && NDS >= 2 && NDS <= 17 && NK <= 10, "the wait counts are written for up to 15 stages behind");
static_assert(LDS_BYTES <= 160 * 1024 / OCC, "the rings must fit the CU's LDS");
static_assert(NDS * DS_STAGE_BYTES >= 4 * 8192, "the epilogue stages 8 KB per wave in the dS ring");
static_assert(MAX_LIST == 1024, "a list entry packs the kv tile into 10 bits");
}  // namespace dqds_cfg

// s_waitcnt vmcnt(N) (vector-memory operations complete in issue order)
template <int N>
__device__ __forceinline__ void wait_vmem_but() {
  __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 15) | ((N >> 4) << 14));
}

__global__ __launch_bounds__(dqds_cfg::THREADS, dqds_cfg::OCC) void bwd_dq_from_ds_kernel(BwdArgs a, float out_scale) {
  using namespace dqds_cfg;
  extern __shared__ __attribute__((aligned(1024))) char smem_raw[];
  int* sIdx = reinterpret_cast<int*>(smem_raw + NDS * DS_STAGE_BYTES + NK * K_STAGE_BYTES);

  const int nQ = a.map.nq, nK = a.map.nk;
  const int n_wg = a.B * a.Hq * nQ;
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const bool copies = !PRODUCERS || wave >= 4;    // the wave issues copies
  const bool computes = !PRODUCERS || wave < 4;   // the wave runs the MFMAs and stores dq
  const int w = wave & 3;                         // its number among the waves of its kind
  const int lane = tid & 63;
  const int hh = lane >> 5;
  const int l16 = lane & 15;

  // heaviest q tiles of a head first under causal masks; a head's tiles on one XCD (they share its K)
  const int wg = xcd_remap((int)blockIdx.x, n_wg);
  const int bh = wg / nQ;
  const int qb = nQ - 1 - wg % nQ;
  const int group = a.Hq / a.Hkv;
  const int bhk = (bh / a.Hq) * a.Hkv + (bh % a.Hq) / group;

  // the q tile's list in LDS: kv tile (10 bits, nk <= 1024) and the dS block of the pair (22 bits: at most 2^20 pairs)
  const int n_list = a.map.cnt[qb];
  const int* list = a.map.idx + (size_t)qb * nK;
  const int* rank = a.ds_rank + (size_t)qb * nK;
  for (int t = tid; t < n_list; t += THREADS) {
    const int kb = list[t];
    sIdx[t] = kb | (rank[kb] << 10);
  }
  __syncthreads();

  const char* ds_row = static_cast<const char*>(a.ds) + (size_t)bh * (size_t)a.ds_pairs * kDsBlockBytes;
  const bf16_t* Kg = static_cast<const bf16_t*>(a.k) + (size_t)bhk * a.Sk * D;
  const unsigned lds0 = (unsigned)(size_t)(__attribute__((address_space(3))) char*)(smem_raw);
  const unsigned lane16 = (unsigned)lane * 16u;

  // The lane's byte offsets in global memory for the wave's four 1 KB pieces of a stage: dS pieces are copied
  // as they lie; piece p of the K rows = 4 rows in the layout of tile_io.hpp
  unsigned goff[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int piece = 4 * (w & 1) + i;
    const int row = piece * 4 + (lane >> 4);
    // (dS pieces of the odd halves u = piece & 1 go into LDS with their 128-byte halves of every 256 bytes swapped:
    // the two 16-lane groups of a half-wave read pieces u = 0 and u = 1 at the same offset, which would be the same
    // banks; the swap puts them on the two halves of the banks)
    goff[i] = w < 2 ? (unsigned)piece * 1024u + (lane16 ^ (128u * (unsigned)(piece & 1)))
                    : (unsigned)(row * kTileD + (((lane & 15) ^ swz(row)) << 3)) * 2u;
  }

  // stage s = part s % PARTS of the list's kv tile s / PARTS: that part's dS as it lies in the block and its 32 K
  // rows.  A wave's copies complete in issue order, so a copy from the L2 issued behind copies from HBM would
  // wait for those: copying waves 0, 1 copy only dS (four pieces each), 2, 3 only K, and each kind runs as far
  // ahead as its ring allows.
  auto tile_of = [&](int s) { return __builtin_amdgcn_readfirstlane(sIdx[s / PARTS] & 1023); };
  auto block_of = [&](int s) { return __builtin_amdgcn_readfirstlane((int)((unsigned)sIdx[s / PARTS] >> 10)); };
  const bool ds_wave = w < 2;
  auto issue = [&](int s) {
    const char* src;
    unsigned dst;
    if (ds_wave) {
      src = ds_row + (size_t)block_of(s) * kDsBlockBytes + (size_t)(s % PARTS) * DS_STAGE_BYTES;
      dst = lds0 + (unsigned)(s % NDS) * DS_STAGE_BYTES + (unsigned)w * 4096u;
    } else {
      src = reinterpret_cast<const char*>(Kg + ((size_t)tile_of(s) * BNK + (size_t)(s % PARTS) * STAGE_KV) * D);
      dst = lds0 + K_RING + (unsigned)(s % NK) * K_STAGE_BYTES + (unsigned)(w - 2) * 4096u;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (ds_wave)  // (dS is read once: nt keeps it from displacing the head's K in the L2)
        asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1 nt"
                     :
                     : "v"(goff[i]), "s"(src), "s"(dst + 1024u * i)
                     : "memory", "m0", "vcc");
      else
        asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                     :
                     : "v"(goff[i]), "s"(src), "s"(dst + 1024u * i)
                     : "memory", "m0", "vcc");
    }
  };
  const int ring = ds_wave ? NDS : NK;  // the wave's kind of stage is copied ring - 1 stages ahead

  // lane-constant parts of the operand addresses (bytes inside a stage)
  // dS^T fragment of k slice ks (kv columns 16 ks + 8 hh + 0..7), q rows 32 w + (lane & 31):
  //   piece (w' = ks >> 1, c, u = (lane & 31) >> 4); the addressing lane names kv column (l16 >> 2) of the
  //   four it reads and row group l16 & 3 = 2 g + hi
  // (a wave computes 64 q rows x 64 head columns: q blocks 2 (w >> 1) + qi, column blocks 2 (w & 1) + di; with
  // 32 x 128 per wave every MFMA would take 2.5 operand reads from LDS instead of 2, and the LDS reads bound the loop)
  const int wq = w >> 1, wd = w & 1;
  const unsigned ds_u = (unsigned)((lane & 31) >> 4);
  const unsigned ds_in = 32u * (unsigned)(8 * hh + (l16 >> 2)) + 16u * (unsigned)(l16 & 1) + 8u * (unsigned)((l16 & 3) >> 1);
  // (the lane's two reads per fragment, 128 bytes apart; swapped in the pieces of the odd halves, see goff)
  const unsigned ds_off = 1024u * (unsigned)(4 * wq) + 1024u * ds_u + (ds_in ^ (128u * ds_u));
  const unsigned ds_off2 = 1024u * (unsigned)(4 * wq) + 1024u * ds_u + ((ds_in + 128u) ^ (128u * ds_u));
  // K^T fragment: rows 16 ks + 8 hh + (l16 >> 2) (+ 4), columns 32 db + 16 ((lane & 31) >> 4) + 4 (l16 & 3) .. + 4
  const int k_row = 8 * hh + (l16 >> 2);
  const int k_chunk = 2 * ((lane & 31) >> 4) + ((l16 & 3) >> 1);
  const int k_half = 4 * (l16 & 1);

  f32x16 acc[2][2];  // [qi][di]
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[t >> 1][t & 1][i] = 0.f;

  const int n_stages = PARTS * n_list;
  if (copies)
    for (int s = 0; s < ring - 1 && s < n_stages; ++s) issue(s);
  for (int s = 0; s < n_stages; ++s) {
    // the wave's copy of stage s has landed once only its copies of the stages behind it are open
    int behind = n_stages - 1 - s;
    if (behind > ring - 2) behind = ring - 2;
    if (copies) switch (behind) {
      case 0: wait_vmem_but<0>(); break;
      case 1: wait_vmem_but<4>(); break;
      case 2: wait_vmem_but<8>(); break;
      case 3: wait_vmem_but<12>(); break;
      case 4: wait_vmem_but<16>(); break;
      case 5: wait_vmem_but<20>(); break;
      case 6: wait_vmem_but<24>(); break;
      case 7: wait_vmem_but<28>(); break;
      case 8: wait_vmem_but<32>(); break;
      case 9: wait_vmem_but<36>(); break;
      case 10: wait_vmem_but<40>(); break;
      case 11: wait_vmem_but<44>(); break;
      case 12: wait_vmem_but<48>(); break;
      case 13: wait_vmem_but<52>(); break;
      case 14: wait_vmem_but<56>(); break;
      default: wait_vmem_but<60>(); break;
    }
    __syncthreads();  // (also: every wave is done with the slots the next copies go to)
    if (copies && s + ring - 1 < n_stages) issue(s + ring - 1);
    if (!computes) continue;
    const char* st = smem_raw + (s % NDS) * DS_STAGE_BYTES;
    const bf16_t* sK = reinterpret_cast<const bf16_t*>(smem_raw + K_RING + (s % NK) * K_STAGE_BYTES);
#pragma unroll
    for (int ks = 0; ks < STAGE_KV / 16; ++ks) {
      bf16x8 bfrag[2], afrag[2];
#pragma unroll
      for (int qi = 0; qi < 2; ++qi) {
        const char* dsp = st + 8192 * (ks >> 1) + 512 * (ks & 1) + 2048 * qi + ds_off;
        const s16x4 b0 = lds_read_tr16(reinterpret_cast<const bf16_t*>(dsp));
        const s16x4 b1 = lds_read_tr16(reinterpret_cast<const bf16_t*>(dsp - ds_off + ds_off2));
        bfrag[qi] = __builtin_bit_cast(bf16x8, __builtin_shufflevector(b0, b1, 0, 1, 2, 3, 4, 5, 6, 7));
      }
#pragma unroll
      for (int di = 0; di < 2; ++di) {
        const int r = 16 * ks + k_row;
        const int db = 2 * wd + di;
        const s16x4 a0 = lds_read_tr16(sK + tile_off(r, 4 * db + k_chunk) + k_half);
        const s16x4 a1 = lds_read_tr16(sK + tile_off(r + 4, 4 * db + k_chunk) + k_half);
        afrag[di] = __builtin_bit_cast(bf16x8, __builtin_shufflevector(a0, a1, 0, 1, 2, 3, 4, 5, 6, 7));
      }
#pragma unroll
      for (int qi = 0; qi < 2; ++qi)
#pragma unroll
        for (int di = 0; di < 2; ++di) acc[qi][di] = mfma32(afrag[di], bfrag[qi], acc[qi][di]);
    }
  }
  __syncthreads();  // the rings are free: the start of LDS stages the tile's 128 dq rows, 8 KB per 32-row q block

  // dq rows as bf16 through LDS (16-byte chunks XOR-swizzled by row), so that every store instruction writes
  // four complete 256-byte rows; lane: q row lane & 31 of block 2 wq + qi, head columns 32 (2 wd + di) + 8 g + 4 hh + 0..3
  const int row_here = lane & 31;
  const unsigned wr = (unsigned)row_here * 256u + 8u * (unsigned)hh;
  if (computes) {
#pragma unroll
    for (int qi = 0; qi < 2; ++qi)
#pragma unroll
      for (int di = 0; di < 2; ++di)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const f32x16& x = acc[qi][di];
          const bf16x2 lo = pack_bf16(x[4 * g] * out_scale, x[4 * g + 1] * out_scale);
          const bf16x2 hi = pack_bf16(x[4 * g + 2] * out_scale, x[4 * g + 3] * out_scale);
          const bf16x4 out = {lo[0], lo[1], hi[0], hi[1]};
          *reinterpret_cast<bf16x4*>(smem_raw + (2 * wq + qi) * 8192 + wr
                                     + (unsigned)(((4 * (2 * wd + di) + g) ^ (row_here & 15)) << 4)) = out;
        }
  }
  __syncthreads();
  if (!computes) return;
  const char* stage = smem_raw + w * 8192;  // wave w stores q block w
  bf16_t* dQg = static_cast<bf16_t*>(a.dq) + ((size_t)bh * a.Sq + (size_t)qb * BQ + (size_t)w * 32) * D;
  const int chunk = lane & 15;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int r = 4 * i + (lane >> 4);
    const unsigned rd = (unsigned)r * 256u + (unsigned)((chunk ^ (r & 15)) << 4);
    *reinterpret_cast<u32x4*>(dQg + (size_t)r * D + chunk * 8) = *reinterpret_cast<const u32x4*>(stage + rd);
  }
}

// `a.map`: row lists of the block map at the dk/dv kernel's 128 x 128 tiles; `a.ds`: the buffer that kernel filled.
int bwd_dq_from_ds(const BwdArgs& a, float out_scale, hipStream_t stream) {
  using namespace dqds_cfg;
  if (a.map.nk > MAX_LIST) return set_error(FLEXATTN_ENOTSUP, "dq from dS: %d kv tiles, at most %d", a.map.nk, MAX_LIST);
  if (a.ds_rank == nullptr || a.ds_pairs <= 0 || a.ds_pairs > (1ll << 20))
    return set_error(FLEXATTN_EINVAL, "dq from dS: no index of the dS blocks (or more than 2^20 kept tile pairs)");
  auto kern = bwd_dq_from_ds_kernel;
  static hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES);
  if (attr != hipSuccess) return set_error(FLEXATTN_ELAUNCH, "hipFuncSetAttribute(dq from dS): %s", hipGetErrorString(attr));
  const int n_wg = a.B * a.Hq * (a.Sq / BQ);
  hipLaunchKernelGGL(kern, dim3(n_wg), dim3(THREADS), LDS_BYTES, stream, a, out_scale);
  return check_launch("flexattn_bwd_dq (from dS) bf16");
}

}  // namespace fa
