/*
 * flexattn.h -- C ABI of libflexattn.so: flex-attention forward, dq backward, dk/dv backward,
 * delta pre-pass and block-mask builder for AMD MI355X (gfx950), hand-written HIP.
 *
 * The reference project has no FFI: its boundary is three Python functions that hand arrays to
 * `pl.pallas_call`.  Each entry point below replaces one of those device hand-offs; the citation
 * next to it names the reference call site (paths relative to the reference repository).
 *
 * Conventions
 *  - All tensors are contiguous row-major [B, H, S, D] device memory owned by the caller.
 *    Head dimension D: 128 or 256 for bf16, 64 or 128 for float32 (anything else: FLEXATTN_ENOTSUP).
 *    q/o/do/dq have Hq heads, k/v/dk/dv have Hkv heads, Hq % Hkv == 0 (kv head = h / (Hq/Hkv)).
 *  - l, m, delta are float32 [B, Hq, Sq].
 *  - Every function returns FLEXATTN_OK or a negative error code, never throws or aborts, and
 *    records a message readable with flexattn_last_error_string() (thread-local).
 *  - Launches are asynchronous on `stream` (a hipStream_t passed as void*; NULL = default stream).
 *  - Entry points are re-entrant and keep no mutable global state (flexattn_fwd_noalloc excepted: it owns one
 *    device array per GPU, see there).
 */
#ifndef FLEXATTN_H_
#define FLEXATTN_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FLEXATTN_VERSION 104 /* major*10000 + minor*100 + patch */

/* status codes */
#define FLEXATTN_OK 0
#define FLEXATTN_EINVAL (-22)   /* bad argument (null pointer, bad enum, non-divisible shape) */
#define FLEXATTN_ENOTSUP (-95)  /* valid request this build has no kernel for */
#define FLEXATTN_ELAUNCH (-5)   /* HIP reported a launch error */

/* element types */
#define FLEXATTN_BF16 0
#define FLEXATTN_F32 1

/* score modifications: s' = f(sm_scale * <q_i, k_j>, b, h, i, j) with global token indices.
 * Reference: scores.py:3-18 (tile callables traced into the kernels at
 * flex_attention_kernel.py:248-255). */
#define FLEXATTN_SCORE_NONE 0
#define FLEXATTN_SCORE_ALIBI 1      /* s + slopes[h] * (j - i)                     */
#define FLEXATTN_SCORE_SOFTCAP 2    /* cap * tanh(s / cap)            scores.py:13-18 */
#define FLEXATTN_SCORE_ALIBI_TILE 3 /* s - slope * |i % mod_q - j % mod_k|  scores.py:3-11 */
#define FLEXATTN_SCORE_CUSTOM 4     /* the score function compiled into this library (functor libraries only,
                                       see flexattn_custom_tag); mod_q, mod_k: tile edges for tile-local indices */

typedef struct flexattn_score_spec {
  int32_t kind;
  float cap;           /* SOFTCAP */
  float slope;         /* ALIBI_TILE */
  int32_t mod_q;       /* ALIBI_TILE */
  int32_t mod_k;       /* ALIBI_TILE */
  int32_t reserved;
  const float* slopes; /* ALIBI: device float32 [Hq] */
} flexattn_score_spec;

/* element masks (keep = attend), AND-composed.  Reference: masks.py:15-16 (causal),
 * :45-59 (window: i - j < window, no causal bound of its own), :105-110 (document),
 * :146-158 (S2: (0 <= i-j < window) | (j % stride == 0 & i >= j); excludes CAUSAL/WINDOW). */
#define FLEXATTN_MASK_CAUSAL 1
#define FLEXATTN_MASK_WINDOW 2
#define FLEXATTN_MASK_DOC 4
#define FLEXATTN_MASK_S2 8
#define FLEXATTN_MASK_CUSTOM 16 /* AND the mask function compiled into this library (functor libraries only) */

typedef struct flexattn_mask_spec {
  int32_t flags;
  int32_t window;
  int32_t stride;
  /* DOC: 0 or 1: the arrays below hold one row, shared by all batch entries.  B (the call's batch size): they hold
   * one row per batch entry, [B, Sq], [B, Sk], [B, Sq, 2], [B, Sk, 2] (the reference's segment ids of shape [B, S],
   * mha_reference.py:65-73): every entry is masked by its own row; the block map built from such a specification is
   * the union over the entries (a tile runs if it runs for any entry). */
  int32_t doc_batches;
  const int32_t* doc_q; /* DOC: device int32 [Sq]: any ids (they need not be sorted) */
  const int32_t* doc_k; /* DOC: device int32 [Sk] (may equal doc_q) */
  /* DOC, optional (NULL = not known): where the ids of the OTHER side are non-decreasing, the positions there that
   * carry a position's id form one interval, and the kernels then mask partial tiles from these bounds instead of
   * comparing ids element by element (the reference's jagged mask has sorted ids: masks.py:88-110).
   * doc_q_range: device int32 [Sq, 2], for q position i the first and last kv position j with doc_k[j] == doc_q[i]
   * (first > last if there is none); needs doc_k non-decreasing.  doc_k_range: device int32 [Sk, 2], likewise the
   * q positions with the id of kv position j; needs doc_q non-decreasing.  Wrong bounds give wrong results. */
  const int32_t* doc_q_range;
  const int32_t* doc_k_range;
} flexattn_mask_spec;

/* Block-sparsity map at (block_q x block_k) granularity, as produced by
 * flexattn_build_block_mask.  state: 0 = skip, 1 = partial (element mask applied),
 * 2 = full (no element is masked).  kv_idx[qb*nk + t], t < kv_cnt[qb], lists ascending the kv
 * blocks with state != 0 of q block qb; q_idx[kb*nq + t], t < q_cnt[kb], the q blocks of kv block kb. */
typedef struct flexattn_block_map {
  const uint8_t* state; /* [nq, nk] */
  const int32_t* kv_cnt; /* [nq] */
  const int32_t* kv_idx; /* [nq, nk] */
  const int32_t* q_cnt;  /* [nk] */
  const int32_t* q_idx;  /* [nk, nq] */
  int32_t nq, nk, block_q, block_k;
} flexattn_block_map;

/* Additive bias on the logits, the reference's `ab` argument (flex_attention_kernel.py:262-266,
 * flash_attention_dkv_bwd.py:261-263, mha_reference.py:50-51): logits = score_mod(sm_scale <q, k>) + ab,
 * then the mask.  Element (b, h, i, j) lies at ptr + b stride_b + h stride_h + i Sk + j (in elements;
 * a stride of 0 broadcasts over that dimension; strides must be multiples of Sk).  ptr NULL = no bias.  Calls with a bias run the kernels
 * with a compiled main loop.  flexattn_bwd_dq can return the gradient of the bias (flexattn_bwd_params.dab). */
typedef struct flexattn_bias {
  const void* ptr;
  int64_t stride_b, stride_h;
  int32_t dtype; /* FLEXATTN_F32 or FLEXATTN_BF16 */
  int32_t reserved;
} flexattn_bias;

/* Call flags.  The bf16 kernels exist twice: with a generated, hand-scheduled instruction stream as
 * main loop (the default wherever one exists for the request) and with a compiled loop (every
 * score kind and list length).  Both meet the stated tolerances; the flag selects the compiled one
 * for a call, for comparisons and tests. */
#define FLEXATTN_FLAG_COMPILED_LOOP 1

typedef struct flexattn_fwd_params {
  const void* q; const void* k; const void* v; /* in  */
  void* o;                                      /* out [B,Hq,Sq,D], dtype of q */
  float* l; float* m;                           /* out [B,Hq,Sq] or both NULL   */
  int32_t B, Hq, Hkv, Sq, Sk, D;
  int32_t dtype;
  float sm_scale; /* > 0 */
  int32_t flags;  /* FLEXATTN_FLAG_* */
  int32_t reserved;
  flexattn_score_spec score;
  flexattn_mask_spec mask;
  flexattn_block_map map; /* granularity must equal flexattn_tile_shape(FLEXATTN_PASS_FWD, ...) */
  flexattn_bias ab;
} flexattn_fwd_params;

/* Index of the dS exchange buffer (see flexattn_bwd_ds_bytes) over the kept tile pairs of the dk/dv pass's block
 * map, as produced by flexattn_build_ds_index: the buffer holds one 32 KB block per (query head, kept pair),
 * block of (head bh, q tile qb, kv tile kb) = bh * pairs + rank[qb * nk + kb].  The reference's tiled backward
 * kernels keep O(block) state (flex_attention_dq_bwd.py:325-380); this buffer is the one O(kept tiles) object of
 * the build, and it is only as large as the mask leaves it. */
typedef struct flexattn_ds_index {
  const int32_t* col;  /* device [nk + 1]: kept pairs in the kv tiles before kb; col[nk] = pairs */
  const int32_t* rank; /* device [nq, nk]: col[kb] + position of qb in kb's q list; -1 for skipped pairs */
  int64_t pairs;       /* number of kept pairs (the caller reads col[nk] back once per map) */
} flexattn_ds_index;

typedef struct flexattn_bwd_params {
  const void* q; const void* k; const void* v; const void* dout;
  const float* l; const float* m; const float* delta; /* [B,Hq,Sq] */
  void* dq;            /* out of flexattn_bwd_dq  [B,Hq,Sq,D]  */
  void* dk; void* dv;  /* out of flexattn_bwd_dkv [B,Hkv,Sk,D] */
  int32_t B, Hq, Hkv, Sq, Sk, D;
  int32_t dtype;
  float sm_scale; /* > 0 */
  int32_t flags;  /* FLEXATTN_FLAG_* */
  int32_t reserved;
  flexattn_score_spec score;
  flexattn_mask_spec mask;
  flexattn_block_map map; /* granularity of the pass being launched */
  flexattn_bias ab;
  /* dS exchange buffer, or NULL (see flexattn_bwd_ds_bytes): written by flexattn_bwd_dkv, read by flexattn_bwd_dq */
  void* ds;
  int64_t ds_bytes;
  flexattn_ds_index ds_index; /* needed with ds; for the map at the granularity of FLEXATTN_PASS_DKV */
  /* Gradient of the additive bias, or NULL: out of flexattn_bwd_dq, float32 [B, Hq, Sq, Sk] (full shape: the caller
   * sums over the dimensions its bias broadcasts).  dab = P (dP - delta), the gradient with respect to the logits
   * (the reference declares this output next to dk, dv, flash_attention_dkv_bwd.py:103-107,130-138, and its upstream
   * dq kernel writes it, jax_exp.py:1252-1255, there multiplied by sm_scale).  Only the tiles the block map visits
   * are written: clear the buffer first.  A call with dab runs the dq kernel with a compiled main loop; it excludes ds. */
  float* dab;
  /* delta computed by the call, optional: with o ([B,Hq,Sq,D], the forward's output) and delta_out ([B,Hq,Sq]
   * float32) set, `delta` is ignored: delta = sum(o * dout) is taken by the call and written to delta_out (the
   * reference leaves the reduction to its callers, flex_attention_dq_bwd.py:932, and hands `o` to its dq entry
   * point without using it, :163): the delta kernel is launched in front of the pass on the same stream, one call
   * across the boundary instead of two.  A dk/dv call of the same backward then reads delta_out as its `delta`.
   * Excludes ds. */
  const void* o;
  float* delta_out;
} flexattn_bwd_params;

#define FLEXATTN_PASS_FWD 0
#define FLEXATTN_PASS_DQ 1
#define FLEXATTN_PASS_DKV 2

int flexattn_version(void);

/* Message for the calling thread's most recent non-OK return ("" if none). */
const char* flexattn_last_error_string(void);

/* A functor library is this same library compiled against a generated header that defines a score
 * function s' = f(s, b, h, i, j) with its derivative and / or a mask predicate keep(i, j): the successor of
 * the reference's tracing of arbitrary closures into its kernels (flex_attention_kernel.py:248-255,
 * 278-288; util.py:22-189, 196-259).  Returns the hash that names the functor pair, "" for the plain
 * library, which rejects FLEXATTN_SCORE_CUSTOM and FLEXATTN_MASK_CUSTOM with FLEXATTN_ENOTSUP. */
const char* flexattn_custom_tag(void);

/* Tile granularity (block_q, block_k) the kernels of `pass` expect of the block map for this
 * dtype and head dimension (bf16 head dimension 256 runs on the tiles of 128). */
int flexattn_tile_shape(int32_t pass, int32_t dtype, int32_t D, int32_t* block_q, int32_t* block_k);

/* Block-mask builder.  Replaces the per-grid-step evaluation of the `block_mask_fn` closures
 * (masks.py:20-28, 63-81, 113-139, 161-177; consumed at flex_attention_kernel.py:97-106,231-236,
 * flex_attention_dq_bwd.py:167-177,318-323, flash_attention_dkv_bwd.py:76-85,224-230).
 * `state != 0` equals the AND of the reference closures of the flags set, bit for bit.
 * All five output arrays are caller-allocated device memory of the sizes given at
 * flexattn_block_map; any of kv_cnt/kv_idx/q_cnt/q_idx may be NULL in pairs. */
int flexattn_build_block_mask(const flexattn_mask_spec* mask, int32_t Sq, int32_t Sk,
                              int32_t block_q, int32_t block_k, uint8_t* state,
                              int32_t* kv_cnt, int32_t* kv_idx, int32_t* q_cnt, int32_t* q_idx,
                              void* stream);

/* Forward.  Replaces the pallas_call in _flex_attention_impl (flex_attention_kernel.py:173-187). */
int flexattn_fwd(const flexattn_fwd_params* p, void* stream);

/* Forward without any allocation.  No counterpart in the reference; for callers that cannot allocate
 * device memory around the call: code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc.  Same request and same results as flexattn_fwd, except that p->map is ignored: the block map of
 * p->mask is built by the builder kernel into a device array that the library holds per GPU (about 340 KB,
 * from library load to process end) and the forward walks it there, both launched on `stream`.  Limits:
 * Sq / block_q <= 4096 q tiles and (Sq / block_q) * (Sk / block_k) <= 65536 tiles at the granularity of
 * flexattn_tile_shape(FLEXATTN_PASS_FWD, ...) (e.g. 32768 x 32768 tokens); larger requests return
 * FLEXATTN_EINVAL.  Calls no hipMalloc / hipFree; the first call on a device looks up the array's address
 * (make that call outside graph capture).  Every call on a GPU uses that GPU's one array: calls whose
 * execution may overlap on one GPU (different streams, graphs replayed concurrently) race and must be
 * serialised by the caller. */
int flexattn_fwd_noalloc(const flexattn_fwd_params* p, void* stream);

/* delta_i = sum_c o_ic * do_ic in float32.  Replaces the caller-side reduction at
 * flex_attention_dq_bwd.py:932 and flash_attention_dkv_bwd.py:925.  rows = B*Hq*Sq. */
int flexattn_bwd_delta(const void* o, const void* dout, float* delta, int64_t rows, int32_t D,
                       int32_t dtype, void* stream);

/* Builds the index of the dS exchange buffer for a block map at the granularity of FLEXATTN_PASS_DKV (state, q_cnt
 * and q_idx are read): col [nk + 1] and rank [nq * nk] are caller-allocated device int32 arrays.  No counterpart
 * in the reference (its backward kernels exchange nothing). */
int flexattn_build_ds_index(const flexattn_block_map* map, int32_t* col, int32_t* rank, void* stream);

/* dS exchange between the two backward passes.  The reference's dq and dk/dv kernels each recompute S, dP and dS
 * (flex_attention_dq_bwd.py:340-378, flash_attention_dkv_bwd.py:232-302).  Here the dk/dv pass can leave its
 * bf16 dS in a caller-allocated device buffer `ds`, and a dq pass that is given the same buffer computes
 * dq = dS K from it, one contraction instead of three (and a compiled score function is evaluated in one pass
 * instead of two).  Returns the bytes `ds` must hold for the request
 * described by p (B Hq ds_index.pairs 32 KB: one block per query head and kept tile pair; only shapes, dtype, D,
 * flags, score, ab, the map's nq and ds_index.pairs are looked at), or 0 when the kernels of the request exchange
 * nothing (fp32, head dimension 256, the global position bias with one query head per kv head, more than
 * 1024 tiles along a sequence, ds_index.pairs <= 0): then ds must stay NULL.
 * Order: flexattn_bwd_dkv with p->ds set, then flexattn_bwd_dq with the same p->ds on the same stream (or
 * ordered behind it) and the same score, ab and flags (they decide which dk/dv kernel wrote the buffer, and with
 * it whether the values already carry sm_scale); for that dq call p->map is the map at the granularity of
 * FLEXATTN_PASS_DKV with its kv_cnt / kv_idx lists.  With ds == NULL both passes work on their own as before. */
int64_t flexattn_bwd_ds_bytes(const flexattn_bwd_params* p);

/* dq backward.  Replaces the pallas_call in flex_attention_bwd_dq (flex_attention_dq_bwd.py:251-265). */
int flexattn_bwd_dq(const flexattn_bwd_params* p, void* stream);

/* dk/dv backward.  Replaces the pallas_call in flash_attention_bwd_dkv
 * (flex_attention_dkv_kernel.py:158-172; mask-aware twin flash_attention_dkv_bwd.py:164-178). */
int flexattn_bwd_dkv(const flexattn_bwd_params* p, void* stream);

/* The whole backward from one call: delta (when the dq block names `o` and `delta_out`), the dq pass of `dq` and the
 * dk/dv pass of `dkv` (the two blocks describe the same problem, each with the block map of its pass; no dS hand-over),
 * launched one after the other on `stream`.  Replaces the sequence the reference's custom_vjp wiring runs
 * (jax_exp.py:276-321: di, then the dk/dv and the dq kernels) by one call across the boundary: small problems are
 * bound by the host's path to a launch, not by the kernels. */
int flexattn_bwd(const flexattn_bwd_params* dq, const flexattn_bwd_params* dkv, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* FLEXATTN_H_ */
