// Host-side check of the keep-bit closed forms in fa_common.hpp (compiled by tests/test_keep_bits.py with
// `hipcc --cuda-host-only`, runs on the CPU): keep_bits32 against the element-wise predicate keep_elem
// for every mask flag combination, on both sides (keys varying / queries varying); and keep_bits32_range, the
// interval form for document masks with sorted ids, likewise.
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "fa_common.hpp"

using namespace fa;

template <bool KEYS>
static unsigned brute(const MaskArgs& mk, int fixed, int base, int doc_fixed, const int* doc_var) {
  unsigned bits = 0;
  for (int c = 0; c < 2; ++c)
    for (int g = 0; g < 4; ++g)
      for (int u = 0; u < 4; ++u) {
        const int idx = base + 32 * c + 8 * g + u;
        const int doc = (mk.flags & FLEXATTN_MASK_DOC) ? doc_var[idx] : 0;
        const bool keep = KEYS ? keep_elem(mk, fixed, idx, doc_fixed, doc) : keep_elem(mk, idx, fixed, doc, doc_fixed);
        bits |= (keep ? 1u : 0u) << (16 * c + 4 * g + u);
      }
  return bits;
}

int main() {
  const int S = 2048;
  std::vector<int> doc(S);
  unsigned rng = 12345u;
  auto next = [&]() { rng = rng * 1664525u + 1013904223u; return rng >> 8; };
  for (int i = 0, d = 0; i < S; ++i) {
    if (next() % 97 == 0) ++d;
    doc[i] = d;
  }
  const int flag_sets[] = {FLEXATTN_MASK_CAUSAL, FLEXATTN_MASK_WINDOW, FLEXATTN_MASK_CAUSAL | FLEXATTN_MASK_WINDOW,
                           FLEXATTN_MASK_DOC, FLEXATTN_MASK_DOC | FLEXATTN_MASK_CAUSAL,
                           FLEXATTN_MASK_DOC | FLEXATTN_MASK_CAUSAL | FLEXATTN_MASK_WINDOW, FLEXATTN_MASK_S2};
  long checked = 0;
  for (int flags : flag_sets) {
    for (int trial = 0; trial < 20000; ++trial) {
      MaskArgs mk{};
      mk.flags = flags;
      const int windows[] = {1, 2, 31, 32, 33, 63, 64, 65, 100, 1025, 1 << 30, 0x7fffffff};
      mk.window = windows[next() % 12];
      mk.stride = 1 + (int)(next() % 64);
      mk.doc_q = mk.doc_k = doc.data();
      const int fixed = (int)(next() % S);
      // strips near the fixed index (where the bounds cut) and anywhere
      int base = (trial & 1) ? (int)(next() % (S - 64)) : fixed - 80 + (int)(next() % 160);
      if (base < 0) base = 0;
      if (base > S - 64) base = S - 64;
      base &= ~3;
      const int hh4 = 4 * (int)(next() & 1);
      if (base + hh4 + 60 >= S) continue;
      const int b = base + hh4;
      const unsigned k0 = keep_bits32<true>(mk, fixed, b, doc[fixed], doc.data());
      const unsigned k1 = brute<true>(mk, fixed, b, doc[fixed], doc.data());
      const unsigned q0 = keep_bits32<false>(mk, fixed, b, doc[fixed], doc.data());
      const unsigned q1 = brute<false>(mk, fixed, b, doc[fixed], doc.data());
      if (k0 != k1 || q0 != q1) {
        std::printf("MISMATCH flags=%d window=%d fixed=%d base=%d keys %08x/%08x queries %08x/%08x\n", flags, mk.window, fixed,
                    b, k0, k1, q0, q1);
        return 1;
      }
      checked += 2;
      if (keep_bits_have_range(mk)) {
        // the interval form: positions that carry the fixed index's id (the ids are sorted: one run)
        int rlo = fixed, rhi = fixed;
        while (rlo > 0 && doc[rlo - 1] == doc[fixed]) --rlo;
        while (rhi + 1 < S && doc[rhi + 1] == doc[fixed]) ++rhi;
        const unsigned kr = keep_bits32_range<true>(mk, fixed, b, rlo, rhi);
        const unsigned qr = keep_bits32_range<false>(mk, fixed, b, rlo, rhi);
        if (kr != k1 || qr != q1) {
          std::printf("MISMATCH (range) flags=%d window=%d fixed=%d base=%d keys %08x/%08x queries %08x/%08x\n", flags,
                      mk.window, fixed, b, kr, k1, qr, q1);
          return 1;
        }
        // an id that the other side does not carry at all: nothing is kept
        if (keep_bits32_range<true>(mk, fixed, b, 5, 4) != 0u || keep_bits32_range<false>(mk, fixed, b, 5, 4) != 0u) return 1;
        checked += 2;
      }
    }
  }
  std::printf("ok %ld\n", checked);
  return 0;
}
