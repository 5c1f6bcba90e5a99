// Host-side check of the LDS tile layout in tile_io.hpp (compiled by tests/test_keep_bits.py with
// `hipcc --cuda-host-only`, runs on the CPU): with 64 banks of 4 bytes, the kernels' two read patterns must put
// no two different addresses of one LDS cycle on the same bank.
//   * row reads (ds_read_b128): 16 lanes x 16 bytes per cycle; lane l reads chunk (2 ks + hh) of row l % 32
//   * transposing reads (ds_read_b64_tr_b16): 32 lanes x 8 bytes per cycle; lane l reads 8 bytes at
//     (row 4 hh + (l % 16) / 4 + 8 (i & 1), chunk 4 (i >> 1) + 2 ((l % 32) / 16) + ((l % 4) / 2), half l & 1)
// (the addressing of fwd_bf16.hip, bwd_dq_bf16.hip and bwd_dkv_bf16.hip: ra[] and ta[] there).
#include <cstdio>
#include <map>
#include <set>

#include "tile_io.hpp"

using namespace fa;

static int worst_bank_load(const int* byte_off, int lanes, int bytes) {
  std::map<int, std::set<int>> banks;
  for (int l = 0; l < lanes; ++l)
    for (int b = byte_off[l] / 4; b < (byte_off[l] + bytes) / 4; ++b) banks[b % 64].insert(b);
  int worst = 0;
  for (auto& kv : banks) worst = (int)kv.second.size() > worst ? (int)kv.second.size() : worst;
  return worst;
}

int main() {
  int bad = 0, checked = 0;
  // swz: 16 distinct values over any 16 consecutive rows, period 16 (the streams shift whole 16-row groups with
  // immediate offsets)
  for (int r0 = 0; r0 < 64; ++r0) {
    std::set<int> seen;
    for (int r = r0; r < r0 + 16; ++r) seen.insert(swz(r));
    if (seen.size() != 16 || swz(r0) != swz(r0 + 16) || swz(r0) < 0 || swz(r0) > 15) ++bad;
  }
  int off[64];
  for (int ks = 0; ks < 8; ++ks)
    for (int quarter = 0; quarter < 4; ++quarter) {
      for (int i = 0; i < 16; ++i) {
        const int lane = 16 * quarter + i, l32 = lane & 31, hh = lane >> 5;
        off[i] = 2 * (l32 * kTileD + (((2 * ks + hh) ^ swz(l32)) << 3));
      }
      bad += worst_bank_load(off, 16, 16) != 1;
      ++checked;
    }
  for (int i = 0; i < 8; ++i)
    for (int half = 0; half < 2; ++half) {
      for (int j = 0; j < 32; ++j) {
        const int lane = 32 * half + j, hh = lane >> 5;
        const int t_row = 4 * hh + ((lane & 15) >> 2), t_chunk = 2 * ((lane & 31) >> 4) + ((lane & 3) >> 1), t_half = 4 * (lane & 1);
        off[j] = 2 * (tile_off(t_row + 8 * (i & 1), 4 * (i >> 1) + t_chunk) + t_half);
      }
      bad += worst_bank_load(off, 32, 8) != 1;
      ++checked;
    }
  if (bad) {
    std::printf("FAIL %d of %d access groups put two addresses on one bank\n", bad, checked);
    return 1;
  }
  std::printf("ok %d access groups\n", checked);
  return 0;
}
