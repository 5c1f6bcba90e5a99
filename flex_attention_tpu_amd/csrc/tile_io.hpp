// LDS tile layout and asynchronous global -> LDS tile loads shared by the bf16 kernels.
//
// A tile is 64 rows x 128 bf16 = 64 rows x 16 chunks of 16 bytes, 16 KB, stored unpadded.  Chunk c
// of row r sits at chunk position c ^ swz(r).  swz permutes the bits of r & 15, so it takes 16 distinct values
// over any 16 consecutive rows and a b128 read of one chunk column over 16 rows (16 lanes, 256 bytes, one LDS
// cycle) is bank-conflict free.  The transposing 8-byte reads take, per half-wave of 32 lanes, 4 consecutive rows
// x two adjacent pairs of chunks (2 x 32 bytes per row): the rows' swizzles differ in bits 2-3 only, so a pair
// of chunks moves by a multiple of two pairs and the eight 32-byte pieces fall on the eight distinct pairs of
// a row, 256 bytes over all 64 banks.  (With the row's low bits in bits 1-2 of the swizzle instead, the two
// pairs of a half-wave fell on the same four positions: every transposing read took two LDS cycles, the 25-32 %
// bank-conflict cycles the counters showed.)
#pragma once
#include "fa_common.hpp"

namespace fa {

constexpr int kTileRows = 64;
constexpr int kTileD = 128;
constexpr int kTileElems = kTileRows * kTileD;  // 8192 bf16 = 16 KB

__host__ __device__ __forceinline__ constexpr int swz(int row) {
  return ((row & 3) << 2) | (((row >> 2) & 1) << 1) | ((row >> 3) & 1);
}

// Element offset of (row, 16-byte chunk) inside a tile.
__host__ __device__ __forceinline__ constexpr int tile_off(int row, int chunk) {
  return row * kTileD + ((chunk ^ swz(row)) << 3);
}

// Asynchronous copy of a 64 x 128 bf16 tile (global row stride ROW elements: 128, or the head dimension where a
// tile is one 128-column panel of wider rows) into LDS with
// global_load_lds_dwordx4: the data never passes through registers.  Each instruction fills one
// contiguous 1 KB block (4 tile rows); lane L's 16 bytes land at block + 16*L, so the swizzle is
// applied on the global side.  The NWAVES waves of a work-group each copy 16/NWAVES blocks.  The
// lane-dependent global offsets are loop invariant and are computed once (TileLoader::init); per
// tile only the uniform base pointers change.  Completion = vmcnt(0) on every wave + barrier.
template <int NWAVES, int ROW = kTileD>
struct TileLoader {
  static constexpr int kBlocks = 16 / NWAVES;  // 1 KB blocks copied per wave
  unsigned goff[kBlocks];  // byte offset of this lane's 16 bytes inside the global tile, per block
  int wave;

  __device__ __forceinline__ void init(int wave_, int lane) {
    wave = wave_;
#pragma unroll
    for (int i = 0; i < kBlocks; ++i) {
      const int row = (wave * kBlocks + i) * 4 + (lane >> 4);
      const int chunk = (lane & 15) ^ swz(row);
      goff[i] = (unsigned)(row * ROW + chunk * 8) * 2u;
    }
  }

  // g_tile and lds_tile must be wave-uniform.  The load is written as inline asm (M0 = LDS
  // destination of the wave's block, SGPR base + per-lane VGPR offset on the global side): issued
  // through the compiler builtin, later LDS reads that the compiler cannot prove disjoint from the
  // destination buffer get a vmcnt(0) wait in front of them, which serialises the prefetch.  The
  // caller orders the copy itself with wait_vmem_all() + barrier before the tile is read.
  __device__ __forceinline__ void load(const bf16_t* g_tile, bf16_t* lds_tile) const {
#pragma unroll
    for (int i = 0; i < kBlocks; ++i) load_block(g_tile, lds_tile, i);
  }

  // One of the wave's kBlocks 1 KB blocks; lets a caller spread the load issue between other work
  // (back-to-back LDS-direct loads occupy the issuing wave for tens of cycles each).
  __device__ __forceinline__ void load_block(const bf16_t* g_tile, bf16_t* lds_tile, int i) const {
    const unsigned lds_base = (unsigned)(size_t)(__attribute__((address_space(3))) char*)(lds_tile);
    const unsigned dst = lds_base + (unsigned)(wave * kBlocks + i) * 1024u;
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                 :
                 : "v"(goff[i]), "s"(g_tile), "s"(dst)
                 : "memory", "m0", "vcc");  // (vcc: else the allocator may hand it out for the address pair,
                                            // which the instruction cannot take as its scalar base)
  }
};

// Waits until every outstanding vector-memory operation of this wave (including LDS-direct loads)
// has completed.
__device__ __forceinline__ void wait_vmem_all() { __builtin_amdgcn_s_waitcnt(0x0F70); }

}  // namespace fa
