// LDS tile layout and asynchronous global -> LDS tile loads shared by the bf16 kernels.
//
// A tile is 64 rows x 128 bf16 = 64 rows x 16 chunks of 16 bytes, 16 KB, stored unpadded.  Chunk c
// of row r sits at chunk position c ^ swz(r).  swz takes 16 distinct values over any 16
// consecutive rows, so a b128 read of one chunk column over 16 rows is bank-conflict free, and
// over 4 consecutive rows it moves a pair of adjacent chunks to 4 distinct pairs, so the
// transposing 8-byte reads (4 rows x 32 bytes per 16 lanes) are conflict free as well.
#pragma once
#include "fa_common.hpp"

namespace fa {

constexpr int kTileRows = 64;
constexpr int kTileD = 128;
constexpr int kTileElems = kTileRows * kTileD;  // 8192 bf16 = 16 KB

__device__ __forceinline__ constexpr int swz(int row) { return ((row & 7) << 1) | ((row >> 3) & 1); }

// Element offset of (row, 16-byte chunk) inside a tile.
__device__ __forceinline__ constexpr int tile_off(int row, int chunk) {
  return row * kTileD + ((chunk ^ swz(row)) << 3);
}

// Asynchronous copy of a 64 x 128 bf16 tile (global row stride 128 elements) into LDS with
// global_load_lds_dwordx4: the data never passes through registers.  Each instruction fills one
// contiguous 1 KB block (4 tile rows); lane L's 16 bytes land at block + 16*L, so the swizzle is
// applied on the global side.  The four waves of a work-group each copy four blocks.  The
// lane-dependent global offsets are loop invariant and are computed once (TileLoader::init); per
// tile only the uniform base pointers change.  Completion = vmcnt(0) on every wave + barrier.
struct TileLoader {
  unsigned goff[4];  // byte offset of this lane's 16 bytes inside the global tile, per block
  int wave;

  __device__ __forceinline__ void init(int wave_, int lane) {
    wave = wave_;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int row = (wave * 4 + i) * 4 + (lane >> 4);
      const int chunk = (lane & 15) ^ swz(row);
      goff[i] = (unsigned)(row * kTileD + chunk * 8) * 2u;
    }
  }

  // g_tile and lds_tile must be wave-uniform.
  __device__ __forceinline__ void load(const bf16_t* g_tile, bf16_t* lds_tile) const {
    const char* g = reinterpret_cast<const char*>(g_tile);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(g + goff[i]),
                                       (__attribute__((address_space(3))) void*)(lds_tile + (wave * 4 + i) * 512),
                                       16, 0, 0);
    }
  }
};

// Waits until every outstanding vector-memory operation of this wave (including LDS-direct loads)
// has completed.
__device__ __forceinline__ void wait_vmem_all() { __builtin_amdgcn_s_waitcnt(0x0F70); }

}  // namespace fa
