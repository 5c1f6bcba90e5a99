// Shared device-side definitions for the gfx950 flex-attention kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "flexattn.h"

// Functor libraries are compiled with FLEXATTN_CUSTOM_HEADER naming a generated header that defines
// fa::custom_score, fa::custom_dscore and fa::custom_keep; the plain library gets the identities.
#ifdef FLEXATTN_CUSTOM_HEADER
#include FLEXATTN_CUSTOM_HEADER
#else
#define FLEXATTN_CUSTOM_TAG ""
#define FLEXATTN_CUSTOM_HAS_SCORE 0
#define FLEXATTN_CUSTOM_HAS_MASK 0
namespace fa {
__host__ __device__ inline float custom_score(float s, int, int, int, int, int, int) { return s; }
__host__ __device__ inline float custom_dscore(float, int, int, int, int, int, int) { return 1.0f; }
__host__ __device__ inline bool custom_keep(int, int) { return true; }
}  // namespace fa
#endif

namespace fa {

typedef __bf16 bf16_t;
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;
constexpr float kNegInf = -__builtin_huge_valf();

// The generated-stream kernels of the forward and dq fold their scale (sm_scale log2 e; softcap: 2 log2 e sm_scale /
// cap) into the bf16 copy of Q they keep in registers, so every logit carries that product's rounding: about
// 2^-9 / sqrt(3) * fold * sqrt(sum_i (q_i k_i)^2) in the exponent, i.e. 0.0011 fold sqrt(D) for unit-variance
// operands.  At the usual sm_scale = 1 / sqrt(D) that is 0.0016, below the 2^-9 the probabilities lose anyway when
// they are rounded to bf16 for the second product.  With sm_scale = 1 on such operands (the reference's own
// drivers) it is 0.018: probabilities off by 1.3 %, lse by 0.06, dq by 2 % in relative L2.  Such calls take the
// kernels with a compiled main loop, which scale the fp32 product.  A power of two folds exactly.  (Softcap: the
// exponent moves by at most cap log2 e / 2 per unit of the chain's result, so the rounding of its fold weighs what
// the plain fold sm_scale log2 e would: the same bound on sm_scale serves.)
inline bool folded_scale_ok(float fold, float sm_scale, int D) {
  int e;
  const float mant = __builtin_frexpf(fold, &e);
  return mant == 0.5f || sm_scale * kLog2e * __builtin_sqrtf((float)D) <= 2.9f;
}

// Kernel-side views of the C ABI structs (pointers already typed).
struct ScoreArgs {
  int kind;
  float cap;
  float slope;
  int mod_q, mod_k;
  const float* slopes;
  // additive bias on the modified logits (the reference's `ab`): element (b, h, i, j) at
  // ab + ((b ab_sb_rows + h ab_sh_rows + i) ab_ld + j) elements, float32 or bf16; NULL = none
  // (strides in rows of ab_ld elements, so that the (batch, head) offset stays in 32-bit scalar arithmetic)
  const void* ab;
  int ab_sb_rows, ab_sh_rows;
  int ab_ld;
  int ab_f32;
};
struct MaskArgs {
  int flags;
  int window;
  int stride;
  const int* doc_q;
  const int* doc_k;
  // For masks whose document ids are sorted on the other side, the positions of the other side that carry a
  // position's id form one interval: (first, last) per position, first > last if there is none; null = unknown.
  const int* doc_q_range;  // [Sq, 2]: kv positions with the id of q position i
  const int* doc_k_range;  // [Sk, 2]: q positions with the id of kv position j
  // Nonzero: the four arrays hold one row per batch entry ([B, Sq], [B, Sk], [B, Sq, 2], [B, Sk, 2]); a kernel
  // masks a batch entry with that entry's rows (mask_of_batch) and the block map is the union over the entries.
  int doc_batched;
};

// The mask of batch entry b: the document arrays advanced to the entry's rows where they are given per entry.
__host__ __device__ __forceinline__ MaskArgs mask_of_batch(const MaskArgs& m, int b, int Sq, int Sk) {
  MaskArgs r = m;
  if (m.doc_batched) {
    r.doc_q += (size_t)b * Sq;
    r.doc_k += (size_t)b * Sk;
    if (r.doc_q_range != nullptr) r.doc_q_range += (size_t)b * Sq * 2;
    if (r.doc_k_range != nullptr) r.doc_k_range += (size_t)b * Sk * 2;
  }
  return r;
}
// One direction of the block map: for "major" block r, idx[r*n_minor + t], t < cnt[r], are the
// minor blocks to visit; state is always indexed [q block][kv block].
struct MapArgs {
  const uint8_t* state;
  const int* cnt;
  const int* idx;
  int nq, nk;
};

struct FwdArgs {
  const void* q; const void* k; const void* v;
  void* o; float* l; float* m;
  int B, Hq, Hkv, Sq, Sk;
  float sm_scale;
  int flags;  // FLEXATTN_FLAG_*
  ScoreArgs score;
  MaskArgs mask;
  MapArgs map;
};

struct BwdArgs {
  const void* q; const void* k; const void* v; const void* dout;
  const float* l; const float* m; const float* delta;
  void* dq; void* dk; void* dv;
  void* ds;   // dS exchange buffer (bf16 kernels that can use one), or null
  // its index over the kept tile pairs of the dk/dv kernel's block map: block of pair (q head bh, q tile qb,
  // kv tile kb) = bh ds_pairs + ds_rank[qb nk + kb], with ds_rank = ds_col[kb] + position of qb in kb's q list
  const int* ds_col;
  const int* ds_rank;
  long long ds_pairs;
  // gradient of the additive bias, float32 [B, Hq, Sq, Sk], or null: the dq kernels with a compiled loop store
  // P (dP - delta) of every element of the tiles they visit (0 where the element mask drops it)
  float* dab;
  // delta computed by the call: with `o` set, the delta kernel runs in front of the pass and writes delta_out
  // (the entry points resolve this before a kernel sees the arguments)
  const void* o;
  float* delta_out;
  int B, Hq, Hkv, Sq, Sk;
  float sm_scale;
  int flags;  // FLEXATTN_FLAG_*
  ScoreArgs score;
  MaskArgs mask;
  MapArgs map;
};

// ------------------------------------------------------------------------------------------
// MFMA wrappers.  v_mfma_f32_32x32x16_bf16: A is 32(M) x 16(K), B is 16(K) x 32(N).
// Lane L supplies A[L%32][8*(L/32) .. +8) and B[8*(L/32) .. +8)[L%32]; it receives
// C[8*(i/4) + 4*(L/32) + i%4][L%32] in accumulator element i.
// ------------------------------------------------------------------------------------------
__device__ __forceinline__ f32x16 mfma32(bf16x8 a, bf16x8 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}

// Row index inside a 32x32 accumulator tile held by (half = lane/32, element i).
__device__ __forceinline__ constexpr int acc_row(int i, int half) { return 8 * (i >> 2) + 4 * half + (i & 3); }

// Transposing LDS read: inside each group of 16 lanes, lane i receives elements j = 0..3 taken
// from the 8-byte chunk addressed by lane 4*j + i/4, at position i%4.
__device__ __forceinline__ s16x4 lds_read_tr16(const bf16_t* p) {
  return __builtin_amdgcn_ds_read_tr16_b64_v4i16(
      (s16x4 __attribute__((address_space(3)))*)(__attribute__((address_space(3))) void*)(p));
}

__device__ __forceinline__ bf16x8 join_tr(s16x4 lo, s16x4 hi) {
  typedef short s16x8 __attribute__((ext_vector_type(8)));
  s16x8 r = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  return __builtin_bit_cast(bf16x8, r);
}

// Reductions across the two 32-lane halves of a wave (lane L with lane L^32).
// v_permlane32_swap exchanges lanes 32-63 of its first register with lanes 0-31 of its second;
// fed two copies of x, every lane ends up holding both halves' values, one in each register, and
// max / sum are symmetric in them.  Written as inline asm: through the compiler builtin the two
// results were folded into one value.  The s_nop cover the VALU-write -> permlane read hazard the
// compiler would otherwise pad itself.
__device__ __forceinline__ void half_pair(float x, float& r0, float& r1) {
  float a = x, b = x;
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
  r0 = a;
  r1 = b;
}
__device__ __forceinline__ float half_max(float x) {
  float r0, r1;
  half_pair(x, r0, r1);
  return fmaxf(r0, r1);
}
__device__ __forceinline__ float half_sum(float x) {
  float r0, r1;
  half_pair(x, r0, r1);
  return r0 + r1;
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_rcp(float x) { return __builtin_amdgcn_rcpf(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }

__device__ __forceinline__ bf16x2 pack_bf16(float a, float b) {
  f32x2 v = {a, b};
  return __builtin_convertvector(v, bf16x2);
}

// ------------------------------------------------------------------------------------------
// Row fragments of a wave's 32 x 128 bf16 block for the transposed MFMA formulations: lane
// (l32 = lane & 31, hh = lane >> 5) needs the 16-byte chunks 2 ks + hh, ks = 0..7, of row l32.
// Loading them directly makes every load instruction touch 32 cache lines; instead the block is
// fetched with full-row loads (rows_load: four complete rows per instruction) and redistributed
// through 8 KB of wave-private LDS when it is needed (rows_to_fragments; 16-byte chunks
// XOR-swizzled by row: conflict-free both ways).
// ------------------------------------------------------------------------------------------
struct RowBlock {
  u32x4 v[8];
};
__device__ __forceinline__ void rows_load(RowBlock& r, const bf16_t* block, int lane) {
#pragma unroll
  for (int i = 0; i < 8; ++i)
    r.v[i] = *reinterpret_cast<const u32x4*>(block + (size_t)(4 * i + (lane >> 4)) * 128 + (lane & 15) * 8);
}
__device__ __forceinline__ void rows_to_fragments(const RowBlock& r, char* stage, int lane, u32x4 (&frag)[8]) {
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int row = 4 * i + (lane >> 4);
    *reinterpret_cast<u32x4*>(stage + row * 256 + (((lane & 15) ^ (row & 15)) << 4)) = r.v[i];
  }
  __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
  __builtin_amdgcn_wave_barrier();
  const int l32 = lane & 31, hh = lane >> 5;
#pragma unroll
  for (int ks = 0; ks < 8; ++ks)
    frag[ks] = *reinterpret_cast<const u32x4*>(stage + l32 * 256 + (((2 * ks + hh) ^ (l32 & 15)) << 4));
  __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
  __builtin_amdgcn_wave_barrier();
}

// ------------------------------------------------------------------------------------------
// Element mask, evaluated only on tiles the block map marks partial.  (Integer code, also callable on the
// host: a CPU test compares the closed forms below with the element-wise predicate.)
// ------------------------------------------------------------------------------------------
__host__ __device__ __forceinline__ bool keep_elem(const MaskArgs& mk, int i, int j, int doc_i, int doc_j) {
  // Branch-free: every term is computed and selected by the (wave-uniform) flag bits.
  const bool f_causal = (mk.flags & FLEXATTN_MASK_CAUSAL) != 0;
  const bool f_window = (mk.flags & FLEXATTN_MASK_WINDOW) != 0;
  const bool f_doc = (mk.flags & FLEXATTN_MASK_DOC) != 0;
  const bool f_s2 = (mk.flags & FLEXATTN_MASK_S2) != 0;
  const int d = i - j;
  const bool in_window = d < mk.window;
  bool keep = (!f_causal | (d >= 0)) & (!f_window | in_window) & (!f_doc | (doc_i == doc_j));
  if (f_s2) keep = keep & (d >= 0) & (in_window | ((j % mk.stride) == 0));
#if FLEXATTN_CUSTOM_HAS_MASK
  if (mk.flags & FLEXATTN_MASK_CUSTOM) keep = keep & custom_keep(i, j);
#endif
  return keep;
}

// Keep bits of a lane's 32 elements in a 64-wide strip of the score matrix, for the generated
// streams: element (c, g, u), c < 2, g < 4, u < 4, lies at offset 32 c + 8 g + u from `base` along the
// varying index (keys when KEYS, the query is then `fixed`; queries otherwise, the key is `fixed`)
// and owns bit 16 c + 4 g + u.  Causal and window masks, the common cases, have a closed form: a
// 64-bit run of ones over the offsets, of which the even nibbles are the lane's elements.  Other
// masks loop over the elements (rolled: the code stays small, these tiles are rare).
__host__ __device__ __forceinline__ unsigned compress_even_nibbles(unsigned long long m) {
  m &= 0x0F0F0F0F0F0F0F0Full;
  m = (m | (m >> 4)) & 0x00FF00FF00FF00FFull;
  m = (m | (m >> 8)) & 0x0000FFFF0000FFFFull;
  m = (m | (m >> 16)) & 0x00000000FFFFFFFFull;
  return (unsigned)m;
}
// Document ids of two 64-index strips, from `first_a` and `first_b` on (multiples of 4), into a
// wave-private LDS stage of 128 ints: lanes 0-31 load and store 16 bytes each.  keep_bits32 then reads
// a strip's ids from LDS (pass `stage [+ 64] - first` as its doc_var) instead of one dependent global
// load per group of four elements.
constexpr int kDocStageBytes = 4 * 128 * 4;  // four waves
__device__ __forceinline__ void stage_doc_ids(const int* doc, int first_a, int first_b, int lane, int* stage) {
  if (lane < 32) {
    const int first = lane < 16 ? first_a : first_b;
    const u32x4 v = *reinterpret_cast<const u32x4*>(doc + first + 4 * (lane & 15));
    *reinterpret_cast<u32x4*>(stage + 4 * lane) = v;
  }
  __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
  __builtin_amdgcn_wave_barrier();
}
template <bool KEYS>
__host__ __device__ __forceinline__ unsigned keep_bits32(const MaskArgs& mk, int fixed, int base, int doc_fixed,
                                                const int* doc_var) {
  if (mk.flags != 0 && (mk.flags & ~(FLEXATTN_MASK_CAUSAL | FLEXATTN_MASK_WINDOW)) == 0) {
    // kept offsets form one interval [lo, hi]: with d = fixed - base, keys keep d - window < off <= d,
    // queries keep d <= off < d + window (the causal bound resp. the window bound, where present)
    const int d = fixed - base;
    const bool causal = (mk.flags & FLEXATTN_MASK_CAUSAL) != 0;
    const bool window = (mk.flags & FLEXATTN_MASK_WINDOW) != 0;
    const int width = mk.window < (1 << 28) ? mk.window : (1 << 28);  // (indices stay far below: no overflow)
    int lo, hi;
    if (KEYS) {
      lo = window ? d - width + 1 : 0;
      hi = causal ? d : 63;
    } else {
      lo = causal ? d : 0;
      hi = window ? width + d - 1 : 63;
    }
    if (lo < 0) lo = 0;
    if (hi > 63) hi = 63;
    if (lo > hi) return 0u;
    const unsigned long long upto = hi == 63 ? ~0ull : ((2ull << hi) - 1ull);
    return compress_even_nibbles(upto & ~((1ull << lo) - 1ull));
  }
  const bool has_doc = (mk.flags & FLEXATTN_MASK_DOC) != 0;
  unsigned bits = 0;
#pragma unroll 1
  for (int cg = 0; cg < 8; ++cg) {
    const int off = 32 * (cg >> 2) + 8 * (cg & 3);
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int idx = base + off + u;
      const int doc = has_doc ? doc_var[idx] : 0;
      const bool keep = KEYS ? keep_elem(mk, fixed, idx, doc_fixed, doc) : keep_elem(mk, idx, fixed, doc, doc_fixed);
      bits |= (keep ? 1u : 0u) << (16 * (cg >> 2) + 4 * (cg & 3) + u);
    }
  }
  return bits;
}

// keep_bits32 for causal / window / document masks when the positions of the varying side that carry the fixed
// index's document id are known to form the interval [rlo, rhi] (MaskArgs::doc_q_range / doc_k_range; empty:
// rlo > rhi): together with the causal and window bounds the kept offsets are still one interval, so a partial
// tile of a document mask costs a dozen integer operations instead of 32 id compares behind a load.
__host__ __device__ __forceinline__ bool keep_bits_have_range(const MaskArgs& mk) {
  return (mk.flags & FLEXATTN_MASK_DOC) != 0 &&
         (mk.flags & ~(FLEXATTN_MASK_CAUSAL | FLEXATTN_MASK_WINDOW | FLEXATTN_MASK_DOC)) == 0;
}
template <bool KEYS>
__host__ __device__ __forceinline__ unsigned keep_bits32_range(const MaskArgs& mk, int fixed, int base, int rlo, int rhi) {
  const int d = fixed - base;
  const bool causal = (mk.flags & FLEXATTN_MASK_CAUSAL) != 0;
  const bool window = (mk.flags & FLEXATTN_MASK_WINDOW) != 0;
  const int width = mk.window < (1 << 28) ? mk.window : (1 << 28);
  int lo, hi;
  if (KEYS) {
    lo = window ? d - width + 1 : 0;
    hi = causal ? d : 63;
  } else {
    lo = causal ? d : 0;
    hi = window ? width + d - 1 : 63;
  }
  const int a = rlo - base, b = rhi - base;
  if (lo < a) lo = a;
  if (hi > b) hi = b;
  if (lo < 0) lo = 0;
  if (hi > 63) hi = 63;
  if (lo > hi) return 0u;
  const unsigned long long upto = hi == 63 ? ~0ull : ((2ull << hi) - 1ull);
  return compress_even_nibbles(upto & ~((1ull << lo) - 1ull));
}

// keep_bits32 for masks with document ids, the strip's ids staged in LDS (stage_doc_ids): `ids` points at
// the id of index `base`.  All 32 ids are read first (eight 16-byte LDS reads in flight at once) and the
// predicate is unrolled: a tenth of the time of the loop above, whose every group waits for its read.
template <bool KEYS>
__device__ __forceinline__ unsigned keep_bits32_staged(const MaskArgs& mk, int fixed, int base, int doc_fixed, const int* ids) {
  u32x4 d[8];
#pragma unroll
  for (int cg = 0; cg < 8; ++cg) d[cg] = *reinterpret_cast<const u32x4*>(ids + 32 * (cg >> 2) + 8 * (cg & 3));
  unsigned bits = 0;
#pragma unroll
  for (int cg = 0; cg < 8; ++cg) {
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int idx = base + 32 * (cg >> 2) + 8 * (cg & 3) + u;
      const int doc = (int)d[cg][u];
      const bool keep = KEYS ? keep_elem(mk, fixed, idx, doc_fixed, doc) : keep_elem(mk, idx, fixed, doc, doc_fixed);
      bits |= (keep ? 1u : 0u) << (16 * (cg >> 2) + 4 * (cg & 3) + u);
    }
  }
  return bits;
}

// ------------------------------------------------------------------------------------------
// Score modification.  `raw` is <q_i, k_j>.  to_log2() returns the modified logit multiplied by
// log2(e) so that probabilities are exp2(t - lse2).  dfactor() returns d(s')/d(raw) given the
// already transformed logit t (log2 domain).
// ------------------------------------------------------------------------------------------
// Internal kind: no score function, but an additive bias.  (The forward with a compiled loop keeps its
// running maximum on the raw dot products when there is no score function at all; with a bias it must
// take the log2-domain route of the score functions.)
constexpr int kScoreBiasOnly = 100;

template <int KIND>
struct ScoreMod {
  float c2;      // sm_scale * log2e
  float scale;   // sm_scale
  float a0, a1;  // kind-specific
  int mod_q, mod_k;
  int bb, hh_;   // batch and head (custom functors)
  const char* ab_base;  // the additive bias, or NULL
  int ab_row0;          // first row of the (batch, head) plane
  int ab_ld, ab_f32;

  __device__ __forceinline__ void init(const ScoreArgs& s, float sm_scale, int head, int batch = 0) {
    bb = batch;
    hh_ = head;
    scale = sm_scale;
    c2 = sm_scale * kLog2e;
    mod_q = s.mod_q;
    mod_k = s.mod_k;
    ab_ld = s.ab_ld;
    ab_f32 = s.ab_f32;
    ab_base = static_cast<const char*>(s.ab);
    ab_row0 = batch * s.ab_sb_rows + head * s.ab_sh_rows;
    if (KIND == FLEXATTN_SCORE_ALIBI) {
      a0 = s.slopes[head] * kLog2e;
    } else if (KIND == FLEXATTN_SCORE_ALIBI_TILE) {
      a0 = s.slope * kLog2e;
    } else if (KIND == FLEXATTN_SCORE_SOFTCAP) {
      a0 = 2.0f * kLog2e * sm_scale / s.cap;  // exponent scale for exp(2 s / cap)
      a1 = s.cap * kLog2e;                    // cap in the log2 domain
    }
  }

  __device__ __forceinline__ float to_log2(float raw, int i, int j) const {
    if (KIND == FLEXATTN_SCORE_NONE || KIND == kScoreBiasOnly) {
      return raw * c2;
    } else if (KIND == FLEXATTN_SCORE_ALIBI) {
      return __builtin_fmaf(raw, c2, a0 * (float)(j - i));
    } else if (KIND == FLEXATTN_SCORE_ALIBI_TILE) {
      int d = (i % mod_q) - (j % mod_k);
      d = d < 0 ? -d : d;
      return __builtin_fmaf(raw, c2, -a0 * (float)d);
    } else if (KIND == FLEXATTN_SCORE_CUSTOM) {
      return custom_score(raw * scale, bb, hh_, i, j, mod_q, mod_k) * kLog2e;
    } else {
      // cap*tanh(x) = cap*(1 - 2/(1 + exp(2x))), x = sm_scale*raw/cap
      float e = fast_exp2(raw * a0);
      float r = fast_rcp(1.0f + e);
      return __builtin_fmaf(-2.0f * a1, r, a1);
    }
  }

  // The additive bias of element (i, j) in the log2 domain (0 without one).  It is added to to_log2()'s
  // result by the kernels, which keep the sum apart from the value they hand to dfactor(): the bias does not
  // depend on the dot product (mha_reference.py:50-51 adds it behind the score function).
  __device__ __forceinline__ bool has_bias() const { return ab_base != nullptr; }
  __device__ __forceinline__ float bias2(int i, int j) const {
    if (ab_base == nullptr) return 0.f;
    const unsigned long long at = (unsigned long long)(unsigned)(ab_row0 + i) * (unsigned)ab_ld + (unsigned)j;
    const float v = ab_f32 ? reinterpret_cast<const float*>(ab_base)[at]
                           : __builtin_bit_cast(float, (unsigned)reinterpret_cast<const unsigned short*>(ab_base)[at] << 16);
    return v * kLog2e;
  }

  // d(s')/d(raw) in natural units, from the log2-domain modified logit t.
  __device__ __forceinline__ float dfactor(float t) const {
    if (KIND == FLEXATTN_SCORE_SOFTCAP) {
      float y = t * fast_rcp(a1);  // tanh
      return scale * (1.0f - y * y);
    }
    return scale;
  }

  // The same for kinds whose derivative depends on more than the transformed logit (compiled closures).
  __device__ __forceinline__ float dfactor(float t, float raw, int i, int j) const {
    if (KIND == FLEXATTN_SCORE_CUSTOM) return scale * custom_dscore(raw * scale, bb, hh_, i, j, mod_q, mod_k);
    return dfactor(t);
  }

  // dfactor() split into an element-wise part and a constant that a kernel may apply once to
  // its accumulated result: dfactor(t) == dfactor_unscaled(t) * dfactor_post_scale(sm_scale).
  __device__ __forceinline__ float dfactor_unscaled(float t) const {
    if (KIND == FLEXATTN_SCORE_SOFTCAP) return dfactor(t);
    return 1.0f;
  }
  __device__ __forceinline__ float dfactor_unscaled(float t, float raw, int i, int j) const {
    if (KIND == FLEXATTN_SCORE_CUSTOM) return dfactor(t, raw, i, j);
    return dfactor_unscaled(t);
  }
  __device__ __forceinline__ float dfactor_post_scale(float sm_scale) const {
    if (KIND == FLEXATTN_SCORE_SOFTCAP || KIND == FLEXATTN_SCORE_CUSTOM) return 1.0f;
    return sm_scale;
  }
};

// XCD-aware work-group remap: consecutive hardware work-group ids go round-robin to the 8 XCDs,
// each with a private L2.  Give every XCD a contiguous range of logical ids so that tiles sharing
// one head's K/V run on the same XCD.
__device__ __forceinline__ int xcd_remap(int wg, int n_wg) {
  constexpr int kXcd = 8;
  if (n_wg % kXcd != 0) return wg;
  return (wg % kXcd) * (n_wg / kXcd) + wg / kXcd;
}

// Static schedule of a generated-stream kernel when it runs one work-group per CU (256 CUs = 8 XCDs x
// 32, consecutive work-group ids go round-robin to the XCDs).  Every XCD takes a contiguous share
// of the (batch, kv head) pairs; its 32 work-groups walk through the share's heads together, so
// they stream the same operand tiles through the XCD's L2, each taking the blocks c, c + 32, ... of a
// head (kv tiles for dk/dv, q tiles for dq).  On every other head the block order is reversed: under
// causal masks the work per block grows or shrinks linearly with its index, so a work-group
// alternates long and short items and all finish together.
__host__ __device__ inline bool persistent_ok(int n_wg, int nKb) {
  if (n_wg % 256 != 0 || (n_wg / 8) % nKb != 0) return false;
  const int heads = n_wg / 8 / nKb;
  if (nKb % 32 == 0) return true;
  return 32 % nKb == 0 && heads % (32 / nKb) == 0;
}
// The work-group's walk through its items with the divisions done once (the kernels locate an item
// three times per item): `base` = first (batch, head) pair of the XCD's share, x, y = (c, blocks per
// head / 32) when a head has at least 32 blocks, else (c / nKb, c % nKb), c = position in the XCD.
struct PersistentPlan {
  int base, x, y;
};
__device__ __forceinline__ PersistentPlan persistent_plan(int j, int n_wg, int nKb) {
  PersistentPlan p;
  const int c = j >> 3;
  p.base = (j & 7) * (n_wg / 8 / nKb);
  if (nKb >= 32) {
    p.x = c;
    p.y = nKb / 32;
  } else {
    p.x = c / nKb;
    p.y = c % nKb;
  }
  return p;
}
// (batch, head) pair and block of item number `item` of work-group j
__device__ __forceinline__ void persistent_item(const PersistentPlan& p, int j, int item, int grid, int n_wg, int nKb,
                                                int& head, int& kb) {
  if (grid == n_wg) {  // one item per work-group, no static schedule
    const int wg = xcd_remap(j, n_wg);
    head = wg / nKb;
    kb = wg % nKb;
    return;
  }
  int hd;
  if (nKb >= 32) {
    hd = p.y == 1 ? item : item / p.y;
    const int kx = p.x + 32 * (item - hd * p.y);
    kb = (hd & 1) ? nKb - 1 - kx : kx;
  } else {
    hd = item * (32 / nKb) + p.x;
    kb = (item & 1) ? nKb - 1 - p.y : p.y;
  }
  head = p.base + hd;
}

// Static schedule for masks whose work per tile is irregular (documents): the tiles are ranked by descending
// work (by comparison, ties by index: every work-group ranks them itself, n_tiles^2 / 256 comparisons per
// thread), the items enumerated rank-major and head-minor, longest first, and dealt to the 256 work-groups
// in rounds of alternating direction, so that every work-group gets one item of every 256 consecutive ones.
// Simulated on the benchmark's document lengths: max / mean load 1.04 forward, 1.01 dq, 1.17 dk/dv (four
// items per work-group there) against 1.41, 1.30, 1.48 of the walk by index above.  Measured against that walk
// and against one item per work-group: up to twice as fast where documents are uneven, 3-9 % slower where
// they are even (an XCD then works on 16 heads at once instead of one).  With fewer than kMinSortedItems items
// per work-group there is too little to balance with: one item per work-group then.
// Writes this work-group's items, head << 16 | tile, to `items`.
// `unit`: heads that share operands through the L2 (the query heads of a kv head in the forward and dq; 1 in
// dk/dv).  When the heads divide into eight shares of whole units, every XCD (work-groups j % 8, consecutive ids
// go round-robin to the XCDs, each with an L2 of its own) takes one share and deals its items, tiles x heads of the
// share, longest first to its 32 work-groups in the same way: the K / V of a kv head (forward, dq) resp. the Q / dO
// of its query heads (dk/dv) then pass through one L2 instead of through all eight.  (Measured on the 16k-token
// document benchmark, GQA 4:1: the forward read 1255 MiB past the L2 for 192 MiB of operands when a head's items
// were dealt over all XCDs.)
constexpr int kMaxSortedItems = 64;
constexpr int kMinSortedItems = 8;
__host__ __device__ inline bool sorted_schedule_ok(int n_wg, int n_tiles) {
  return n_wg % 256 == 0 && n_wg / 256 >= kMinSortedItems && n_wg / 256 <= kMaxSortedItems && n_tiles <= 2048;
}
template <typename WorkFn>
__device__ __forceinline__ void sorted_items(WorkFn work, int n_tiles, int n_heads, int unit, int j, int n_items, int tid,
                                             int* scratch /* LDS: 2 n_tiles ints */, int* items /* LDS: n_items ints */) {
  int* cnt = scratch;
  int* order = scratch + n_tiles;
  for (int t = tid; t < n_tiles; t += 256) cnt[t] = work(t);
  __syncthreads();
  for (int t = tid; t < n_tiles; t += 256) {
    const int c = cnt[t];
    int rank = 0;
    for (int u = 0; u < n_tiles; ++u) {
      const int cu = cnt[u];
      rank += (cu > c || (cu == c && u < t)) ? 1 : 0;
    }
    order[rank] = t;
  }
  __syncthreads();
  if (tid < n_items) {
    if (n_heads % (8 * unit) == 0) {
      const int share = n_heads / 8;            // heads of this work-group's XCD: [(j % 8) share, + share)
      const int c = j >> 3;                     // place among the XCD's 32 work-groups
      const int k = 32 * tid + ((tid & 1) ? 31 - c : c);
      items[tid] = (((j & 7) * share + k % share) << 16) | order[k / share];
    } else {
      const int k = 256 * tid + ((tid & 1) ? 255 - j : j);
      items[tid] = ((k % n_heads) << 16) | order[k / n_heads];
    }
  }
  __syncthreads();
}

}  // namespace fa
