// C ABI of libflexattn.so: argument validation and dispatch to the gfx950 kernels.
#include <cstdarg>
#include <cstdio>
#include <mutex>

#include "fa_common.hpp"
#include "launch.hpp"

namespace fa {

static thread_local char g_err[512] = "";

int set_error(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return set_error(FLEXATTN_ELAUNCH, "%s: %s", what, hipGetErrorString(e));
  return FLEXATTN_OK;
}

static ScoreArgs to_args(const flexattn_score_spec& s, const flexattn_bias& ab, int Sk) {
  ScoreArgs r;
  r.kind = s.kind;
  r.cap = s.cap;
  r.slope = s.slope;
  r.mod_q = s.mod_q;
  r.mod_k = s.mod_k;
  r.slopes = s.slopes;
  r.ab = ab.ptr;
  r.ab_sb_rows = ab.ptr ? (int)(ab.stride_b / Sk) : 0;
  r.ab_sh_rows = ab.ptr ? (int)(ab.stride_h / Sk) : 0;
  r.ab_ld = Sk;
  r.ab_f32 = ab.dtype == FLEXATTN_F32 ? 1 : 0;
  return r;
}

static int check_bias(const flexattn_bias& ab, int B, int Hq, int Sq, int Sk) {
  if (ab.ptr == nullptr) return FLEXATTN_OK;
  if (ab.dtype != FLEXATTN_F32 && ab.dtype != FLEXATTN_BF16) return set_error(FLEXATTN_EINVAL, "unknown bias dtype %d", ab.dtype);
  if (ab.stride_b < 0 || ab.stride_h < 0) return set_error(FLEXATTN_EINVAL, "negative bias stride");
  if (Sk <= 0 || ab.stride_b % Sk != 0 || ab.stride_h % Sk != 0)
    return set_error(FLEXATTN_EINVAL, "bias strides (%lld, %lld) must be multiples of the row length Sk=%d",
                     (long long)ab.stride_b, (long long)ab.stride_h, Sk);
  const long long rows = (long long)(B - 1) * (ab.stride_b / Sk) + (long long)(Hq - 1) * (ab.stride_h / Sk) + Sq;
  if (rows >= (1ll << 31)) return set_error(FLEXATTN_ENOTSUP, "bias spans %lld rows, at most 2^31 - 1 are addressed", rows);
  return FLEXATTN_OK;
}

static MaskArgs to_args(const flexattn_mask_spec& m) {
  MaskArgs r;
  r.flags = m.flags;
  r.window = m.window;
  r.stride = m.stride;
  r.doc_q = m.doc_q;
  r.doc_k = m.doc_k;
  r.doc_q_range = m.doc_q_range;
  r.doc_k_range = m.doc_k_range;
  r.doc_batched = ((m.flags & FLEXATTN_MASK_DOC) && m.doc_batches > 1) ? 1 : 0;
  return r;
}

// Document arrays given per batch entry must cover the call's batch.
static int check_doc_batches(const flexattn_mask_spec& m, int B) {
  if (!(m.flags & FLEXATTN_MASK_DOC)) return FLEXATTN_OK;
  if (m.doc_batches < 0 || (m.doc_batches > 1 && m.doc_batches != B))
    return set_error(FLEXATTN_EINVAL, "mask DOC: doc_batches=%d, must be 0 or 1 (one row of ids for all) or the batch size %d",
                     m.doc_batches, B);
  return FLEXATTN_OK;
}

static int check_score(const flexattn_score_spec& s) {
  switch (s.kind) {
    case FLEXATTN_SCORE_NONE: return FLEXATTN_OK;
    case FLEXATTN_SCORE_ALIBI:
      if (s.slopes == nullptr) return set_error(FLEXATTN_EINVAL, "score ALIBI needs a per-head slopes array");
      return FLEXATTN_OK;
    case FLEXATTN_SCORE_SOFTCAP:
      if (!(s.cap > 0.f)) return set_error(FLEXATTN_EINVAL, "score SOFTCAP needs cap > 0 (got %g)", (double)s.cap);
      return FLEXATTN_OK;
    case FLEXATTN_SCORE_ALIBI_TILE:
      if (s.mod_q <= 0 || s.mod_k <= 0)
        return set_error(FLEXATTN_EINVAL, "score ALIBI_TILE needs mod_q, mod_k > 0 (got %d, %d)", s.mod_q, s.mod_k);
      return FLEXATTN_OK;
    case FLEXATTN_SCORE_CUSTOM:
      if (!FLEXATTN_CUSTOM_HAS_SCORE)
        return set_error(FLEXATTN_ENOTSUP, "score CUSTOM: this library was built without a compiled score function");
      if (s.mod_q <= 0 || s.mod_k <= 0)
        return set_error(FLEXATTN_EINVAL, "score CUSTOM needs mod_q, mod_k > 0 (got %d, %d)", s.mod_q, s.mod_k);
      return FLEXATTN_OK;
  }
  return set_error(FLEXATTN_EINVAL, "unknown score kind %d", s.kind);
}

static int check_mask(const flexattn_mask_spec& m) {
  const int known = FLEXATTN_MASK_CAUSAL | FLEXATTN_MASK_WINDOW | FLEXATTN_MASK_DOC | FLEXATTN_MASK_S2 | FLEXATTN_MASK_CUSTOM;
  if (m.flags & ~known) return set_error(FLEXATTN_EINVAL, "unknown mask flags 0x%x", m.flags);
  if ((m.flags & FLEXATTN_MASK_CUSTOM) && !FLEXATTN_CUSTOM_HAS_MASK)
    return set_error(FLEXATTN_ENOTSUP, "mask CUSTOM: this library was built without a compiled mask function");
  if ((m.flags & FLEXATTN_MASK_S2) && (m.flags & (FLEXATTN_MASK_CAUSAL | FLEXATTN_MASK_WINDOW)))
    return set_error(FLEXATTN_EINVAL, "mask S2 already contains its window and causal terms; do not combine");
  if ((m.flags & (FLEXATTN_MASK_WINDOW | FLEXATTN_MASK_S2)) && m.window <= 0)
    return set_error(FLEXATTN_EINVAL, "mask window must be > 0 (got %d)", m.window);
  if ((m.flags & FLEXATTN_MASK_S2) && m.stride <= 0)
    return set_error(FLEXATTN_EINVAL, "mask S2 stride must be > 0 (got %d)", m.stride);
  if ((m.flags & FLEXATTN_MASK_DOC) && (m.doc_q == nullptr || m.doc_k == nullptr))
    return set_error(FLEXATTN_EINVAL, "mask DOC needs doc_q and doc_k arrays");
  return FLEXATTN_OK;
}

static int tile_shape(int pass, int dtype, int D, int* bq, int* bk) {
  if (dtype == FLEXATTN_F32) {
    if (D != 64 && D != 128) return set_error(FLEXATTN_ENOTSUP, "fp32: head dim %d not in {64, 128}", D);
    f32_tile(bq, bk);
    return FLEXATTN_OK;
  }
  if (dtype == FLEXATTN_BF16) {
    if (D != 128 && D != 256) return set_error(FLEXATTN_ENOTSUP, "bf16: head dim %d not in {128, 256}", D);
    switch (pass) {   // (head dim 256 runs on the tiles of head dim 128)
      case FLEXATTN_PASS_FWD: fwd_bf16_d128_tile(bq, bk); return FLEXATTN_OK;
      case FLEXATTN_PASS_DQ: bwd_dq_bf16_d128_tile(bq, bk); return FLEXATTN_OK;
      case FLEXATTN_PASS_DKV: bwd_dkv_bf16_d128_tile(bq, bk); return FLEXATTN_OK;
    }
    return set_error(FLEXATTN_EINVAL, "unknown pass %d", pass);
  }
  return set_error(FLEXATTN_EINVAL, "unknown dtype %d", dtype);
}

// sm_scale must be positive (the kernels track maxima of unscaled products and fold the scale into an
// operand); flags must be known.
static int check_scale_flags(float sm_scale, int flags) {
  if (!(sm_scale > 0.f) || !(sm_scale < __builtin_huge_valf()))
    return set_error(FLEXATTN_EINVAL, "sm_scale must be positive and finite (got %g)", (double)sm_scale);
  if (flags & ~FLEXATTN_FLAG_COMPILED_LOOP) return set_error(FLEXATTN_EINVAL, "unknown flags 0x%x", flags);
  return FLEXATTN_OK;
}

// `tile_pass`: the pass whose tile granularity the map must have (the dq pass reads the dk/dv kernel's dS blocks at
// that kernel's tiles)
static int check_shape(int pass, int B, int Hq, int Hkv, int Sq, int Sk, int D, int dtype,
                       const flexattn_block_map& map, int tile_pass = -1) {
  if (B <= 0 || Hq <= 0 || Hkv <= 0 || Sq <= 0 || Sk <= 0 || D <= 0)
    return set_error(FLEXATTN_EINVAL, "non-positive dimension (B=%d Hq=%d Hkv=%d Sq=%d Sk=%d D=%d)", B, Hq, Hkv, Sq, Sk, D);
  if (Hq % Hkv != 0) return set_error(FLEXATTN_EINVAL, "Hq=%d is not a multiple of Hkv=%d", Hq, Hkv);
  int bq = 0, bk = 0;
  int rc = tile_shape(tile_pass >= 0 ? tile_pass : pass, dtype, D, &bq, &bk);
  if (rc != FLEXATTN_OK) return rc;
  if (Sq % bq != 0) return set_error(FLEXATTN_EINVAL, "Sq=%d is not a multiple of the q tile %d", Sq, bq);
  if (Sk % bk != 0) return set_error(FLEXATTN_EINVAL, "Sk=%d is not a multiple of the kv tile %d", Sk, bk);
  if (map.state == nullptr) return set_error(FLEXATTN_EINVAL, "block map state is NULL");
  if (map.block_q != bq || map.block_k != bk || map.nq != Sq / bq || map.nk != Sk / bk)
    return set_error(FLEXATTN_EINVAL, "block map is %dx%d blocks of %dx%d, kernel needs %dx%d blocks of %dx%d",
                     map.nq, map.nk, map.block_q, map.block_k, Sq / bq, Sk / bk, bq, bk);
  if (pass == FLEXATTN_PASS_DKV) {
    if (map.q_cnt == nullptr || map.q_idx == nullptr) return set_error(FLEXATTN_EINVAL, "block map lacks q_cnt/q_idx");
  } else {
    if (map.kv_cnt == nullptr || map.kv_idx == nullptr) return set_error(FLEXATTN_EINVAL, "block map lacks kv_cnt/kv_idx");
  }
  return FLEXATTN_OK;
}

static MapArgs row_view(const flexattn_block_map& m) {
  MapArgs r;
  r.state = m.state; r.cnt = m.kv_cnt; r.idx = m.kv_idx; r.nq = m.nq; r.nk = m.nk;
  return r;
}
static MapArgs col_view(const flexattn_block_map& m) {
  MapArgs r;
  r.state = m.state; r.cnt = m.q_cnt; r.idx = m.q_idx; r.nq = m.nq; r.nk = m.nk;
  return r;
}

// Whether the dk/dv pass of this request runs the generated stream (else the kernel with a compiled main loop).
static bool dkv_on_stream(const flexattn_bwd_params* p) {
  return bwd_dkv_bf16_d128_on_stream(p->score.kind, p->flags, p->map.nq, p->ab.ptr != nullptr, p->Hq, p->Hkv);
}

// Whether the bf16 dk/dv and dq kernels of this request can hand dS over through a buffer: the generated-stream
// dk/dv kernels for plain and softcap scores write it (the position-bias streams keep the key's share of the
// bias out of their dS), and so does the dk/dv kernel with a compiled main loop, for every score (compiled score
// functions among them: the dq pass from dS then evaluates none).  Looks at shapes, score, flags and the map's size.
static bool ds_exchange_ok(const flexattn_bwd_params* p) {
  if (p == nullptr || p->dtype != FLEXATTN_BF16 || p->D != 128) return false;
  if (p->B <= 0 || p->Hq <= 0 || p->Hkv <= 0 || p->Sq <= 0 || p->Sk <= 0) return false;
  if (dkv_on_stream(p) && p->score.kind != FLEXATTN_SCORE_NONE && p->score.kind != FLEXATTN_SCORE_SOFTCAP) return false;
  int bq = 0, bk = 0;
  bwd_dkv_bf16_d128_tile(&bq, &bk);
  if (p->Sq % bq != 0 || p->Sk % bk != 0) return false;
  if (p->ds_index.pairs <= 0 || p->ds_index.pairs > (int64_t)(p->Sq / bq) * (p->Sk / bk)) return false;
  return p->Sq / bq <= 1024 && p->Sk / bk <= 1024;  // (the dq pass from dS caches a tile list in LDS)
}

// What the dq pass multiplies K by: the streams export dS without sm_scale (softcap: without its factor 4 either),
// the kernel with a compiled main loop exports it complete.
static float ds_out_scale(const flexattn_bwd_params* p) {
  if (!dkv_on_stream(p)) return 1.0f;
  return (p->score.kind == FLEXATTN_SCORE_SOFTCAP ? 4.f : 1.f) * p->sm_scale;
}

// one block of block_q x block_k bf16 values per (query head, kept tile pair)
static int64_t ds_bytes_of(const flexattn_bwd_params* p) {
  int bq = 0, bk = 0;
  bwd_dkv_bf16_d128_tile(&bq, &bk);
  return (int64_t)p->B * p->Hq * p->ds_index.pairs * bq * bk * 2;
}

static int check_ds(const flexattn_bwd_params* p) {
  if (p->ds == nullptr) return FLEXATTN_OK;
  if (!ds_exchange_ok(p))
    return set_error(FLEXATTN_EINVAL, "ds given, but the kernels of this request exchange no dS (flexattn_bwd_ds_bytes is 0)");
  if (p->ds_index.col == nullptr || p->ds_index.rank == nullptr)
    return set_error(FLEXATTN_EINVAL, "ds given without ds_index.col / ds_index.rank (flexattn_build_ds_index)");
  if (p->ds_bytes < ds_bytes_of(p))
    return set_error(FLEXATTN_EINVAL, "ds holds %lld bytes, the request needs %lld", (long long)p->ds_bytes,
                     (long long)ds_bytes_of(p));
  return FLEXATTN_OK;
}

static int to_bwd_args(const flexattn_bwd_params* p, int pass, BwdArgs* a) {
  if (p == nullptr) return set_error(FLEXATTN_EINVAL, "params is NULL");
  if (!p->q || !p->k || !p->v || !p->dout || !p->l || !p->m)
    return set_error(FLEXATTN_EINVAL, "a required input pointer is NULL");
  if (p->o != nullptr) {
    if (p->delta_out == nullptr) return set_error(FLEXATTN_EINVAL, "o given without delta_out");
    if (p->ds != nullptr) return set_error(FLEXATTN_EINVAL, "o (delta computed by the call) and ds exclude each other");
  } else if (!p->delta) {
    return set_error(FLEXATTN_EINVAL, "delta is NULL (give delta, or o and delta_out)");
  }
  if (pass == FLEXATTN_PASS_DQ && !p->dq) return set_error(FLEXATTN_EINVAL, "dq is NULL");
  if (pass == FLEXATTN_PASS_DKV && (!p->dk || !p->dv)) return set_error(FLEXATTN_EINVAL, "dk or dv is NULL");
  int rc = check_ds(p);
  if (rc != FLEXATTN_OK) return rc;
  rc = check_shape(pass, p->B, p->Hq, p->Hkv, p->Sq, p->Sk, p->D, p->dtype, p->map, p->ds ? FLEXATTN_PASS_DKV : -1);
  if (rc != FLEXATTN_OK) return rc;
  if ((rc = check_scale_flags(p->sm_scale, p->flags)) != FLEXATTN_OK) return rc;
  if ((rc = check_score(p->score)) != FLEXATTN_OK) return rc;
  if ((rc = check_mask(p->mask)) != FLEXATTN_OK) return rc;
  if ((rc = check_doc_batches(p->mask, p->B)) != FLEXATTN_OK) return rc;
  if ((rc = check_bias(p->ab, p->B, p->Hq, p->Sq, p->Sk)) != FLEXATTN_OK) return rc;
  if (p->dab != nullptr) {
    if (pass != FLEXATTN_PASS_DQ) return set_error(FLEXATTN_EINVAL, "dab is an output of flexattn_bwd_dq");
    if (p->ds != nullptr) return set_error(FLEXATTN_EINVAL, "dab and ds exclude each other (the dq pass from dS recomputes nothing)");
  }
  a->dab = p->dab;
  a->o = p->o;
  a->delta_out = p->delta_out;
  a->ds = p->ds;
  a->ds_col = p->ds_index.col;
  a->ds_rank = p->ds_index.rank;
  a->ds_pairs = p->ds_index.pairs;
  a->q = p->q; a->k = p->k; a->v = p->v; a->dout = p->dout;
  a->l = p->l; a->m = p->m; a->delta = p->delta;
  a->dq = p->dq; a->dk = p->dk; a->dv = p->dv;
  a->B = p->B; a->Hq = p->Hq; a->Hkv = p->Hkv; a->Sq = p->Sq; a->Sk = p->Sk;
  a->sm_scale = p->sm_scale;
  a->flags = p->flags;
  a->score = to_args(p->score, p->ab, p->Sk);
  a->mask = to_args(p->mask);
  a->map = (pass == FLEXATTN_PASS_DKV) ? col_view(p->map) : row_view(p->map);
  return FLEXATTN_OK;
}


// With `o` given the call computes delta itself: the delta kernel runs in front of the pass, on the same stream.
// (Folding the sum into the dq stream kernel was measured and is not done: fetching an item's 32 rows of o along
// with those of Q and dO an item ahead lengthened the dq launch by 0.067 ms on B=4, H=32, S=4096, where the delta
// kernel takes 0.038 ms: the burst of row loads at an item's start is what the CU cannot keep in flight.)
static int delta_first(BwdArgs* a, int D, int dtype, hipStream_t s) {
  if (a->o == nullptr) return FLEXATTN_OK;
  const int rc = bwd_delta(a->o, a->dout, a->delta_out, (int64_t)a->B * a->Hq * a->Sq, D, dtype, s);
  a->delta = a->delta_out;
  a->o = nullptr;
  return rc;
}

static int fwd_with_map(const flexattn_fwd_params* p, const flexattn_block_map& map, hipStream_t s) {
  if (!p->q || !p->k || !p->v || !p->o) return set_error(FLEXATTN_EINVAL, "q, k, v or o is NULL");
  if ((p->l == nullptr) != (p->m == nullptr)) return set_error(FLEXATTN_EINVAL, "l and m must both be given or both NULL");
  int rc = check_shape(FLEXATTN_PASS_FWD, p->B, p->Hq, p->Hkv, p->Sq, p->Sk, p->D, p->dtype, map);
  if (rc != FLEXATTN_OK) return rc;
  if ((rc = check_scale_flags(p->sm_scale, p->flags)) != FLEXATTN_OK) return rc;
  if ((rc = check_score(p->score)) != FLEXATTN_OK) return rc;
  if ((rc = check_mask(p->mask)) != FLEXATTN_OK) return rc;
  if ((rc = check_doc_batches(p->mask, p->B)) != FLEXATTN_OK) return rc;
  if ((rc = check_bias(p->ab, p->B, p->Hq, p->Sq, p->Sk)) != FLEXATTN_OK) return rc;
  FwdArgs a;
  a.q = p->q; a.k = p->k; a.v = p->v; a.o = p->o; a.l = p->l; a.m = p->m;
  a.B = p->B; a.Hq = p->Hq; a.Hkv = p->Hkv; a.Sq = p->Sq; a.Sk = p->Sk;
  a.sm_scale = p->sm_scale;
  a.flags = p->flags;
  a.score = to_args(p->score, p->ab, p->Sk);
  a.mask = to_args(p->mask);
  a.map = row_view(map);
  if (p->dtype == FLEXATTN_BF16) return p->D == 256 ? fwd_bf16_d256(a, s) : fwd_bf16_d128(a, s);
  return (a.flags & FLEXATTN_FLAG_COMPILED_LOOP) ? fwd_f32(a, p->D, s) : fwd_f32_mfma(a, p->D, s);
}

// ---- resident block map of flexattn_fwd_noalloc ---------------------------------------------------------
// The forward walks a block map (tile states, per-row counts and kv lists) that flexattn_fwd's caller
// allocates.  flexattn_fwd_noalloc keeps one in this file-scope device array instead: every GPU the library
// runs on holds its own copy (kScratchBytes, about 340 KB) until the process ends.  The array's name is only a
// host-side handle; its device address is looked up once per device and kept here.
constexpr int kScratchMaxRows = 4096;       // q tiles
constexpr int kScratchMaxTiles = 65536;     // q tiles x kv tiles (e.g. 32768 x 32768 tokens at 128 x 128)
constexpr size_t kScratchStateOff = 0;
constexpr size_t kScratchCntOff = kScratchStateOff + kScratchMaxTiles;
constexpr size_t kScratchIdxOff = kScratchCntOff + (size_t)kScratchMaxRows * 4;
constexpr size_t kScratchBytes = kScratchIdxOff + (size_t)kScratchMaxTiles * 4;
static_assert(kScratchCntOff % 256 == 0 && kScratchIdxOff % 256 == 0, "sub-arrays stay 256-byte aligned");
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

constexpr int kMaxDevices = 64;
static std::mutex g_scratch_mutex;
static unsigned char* g_scratch_ptr[kMaxDevices] = {};

static int scratch_of_current_device(unsigned char** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return set_error(FLEXATTN_ELAUNCH, "hipGetDevice: %s", hipGetErrorString(e));
  if (dev < 0 || dev >= kMaxDevices) return set_error(FLEXATTN_ENOTSUP, "device ordinal %d outside [0, %d)", dev, kMaxDevices);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || ptr == nullptr)
      return set_error(FLEXATTN_ELAUNCH, "hipGetSymbolAddress(scratch) on device %d: %s", dev, hipGetErrorString(e));
    g_scratch_ptr[dev] = static_cast<unsigned char*>(ptr);
  }
  *out = g_scratch_ptr[dev];
  return FLEXATTN_OK;
}

}  // namespace fa

using namespace fa;

extern "C" {

int flexattn_version(void) { return FLEXATTN_VERSION; }

const char* flexattn_last_error_string(void) { return g_err; }

const char* flexattn_custom_tag(void) { return FLEXATTN_CUSTOM_TAG; }

int flexattn_tile_shape(int32_t pass, int32_t dtype, int32_t D, int32_t* block_q, int32_t* block_k) {
  if (block_q == nullptr || block_k == nullptr) return set_error(FLEXATTN_EINVAL, "block_q/block_k is NULL");
  if (pass < FLEXATTN_PASS_FWD || pass > FLEXATTN_PASS_DKV) return set_error(FLEXATTN_EINVAL, "unknown pass %d", pass);
  int bq = 0, bk = 0;
  int rc = tile_shape(pass, dtype, D, &bq, &bk);
  if (rc != FLEXATTN_OK) return rc;
  *block_q = bq;
  *block_k = bk;
  return FLEXATTN_OK;
}

int flexattn_build_block_mask(const flexattn_mask_spec* mask, int32_t Sq, int32_t Sk, int32_t block_q,
                              int32_t block_k, uint8_t* state, int32_t* kv_cnt, int32_t* kv_idx,
                              int32_t* q_cnt, int32_t* q_idx, void* stream) {
  if (mask == nullptr || state == nullptr) return set_error(FLEXATTN_EINVAL, "mask or state is NULL");
  if (Sq <= 0 || Sk <= 0 || block_q <= 0 || block_k <= 0)
    return set_error(FLEXATTN_EINVAL, "non-positive size (Sq=%d Sk=%d block_q=%d block_k=%d)", Sq, Sk, block_q, block_k);
  if (Sq % block_q != 0 || Sk % block_k != 0)
    return set_error(FLEXATTN_EINVAL, "Sq=%d / Sk=%d not divisible by blocks %d / %d", Sq, Sk, block_q, block_k);
  if ((kv_cnt == nullptr) != (kv_idx == nullptr) || (q_cnt == nullptr) != (q_idx == nullptr))
    return set_error(FLEXATTN_EINVAL, "count and index arrays must be given in pairs");
  int rc = check_mask(*mask);
  if (rc != FLEXATTN_OK) return rc;
  if ((mask->flags & FLEXATTN_MASK_DOC) && mask->doc_batches < 0)
    return set_error(FLEXATTN_EINVAL, "mask DOC: doc_batches=%d is negative", mask->doc_batches);
  return build_block_mask(to_args(*mask), mask->doc_batches, Sq, Sk, block_q, block_k, state, kv_cnt, kv_idx, q_cnt, q_idx,
                          static_cast<hipStream_t>(stream));
}

int flexattn_build_ds_index(const flexattn_block_map* map, int32_t* col, int32_t* rank, void* stream) {
  if (map == nullptr || col == nullptr || rank == nullptr) return set_error(FLEXATTN_EINVAL, "map, col or rank is NULL");
  if (map->state == nullptr || map->q_cnt == nullptr || map->q_idx == nullptr)
    return set_error(FLEXATTN_EINVAL, "block map lacks state or q_cnt/q_idx");
  if (map->nq <= 0 || map->nk <= 0) return set_error(FLEXATTN_EINVAL, "block map of %d x %d tiles", map->nq, map->nk);
  return build_ds_index(map->state, map->q_cnt, map->q_idx, map->nq, map->nk, col, rank, static_cast<hipStream_t>(stream));
}

int flexattn_fwd(const flexattn_fwd_params* p, void* stream) {
  if (p == nullptr) return set_error(FLEXATTN_EINVAL, "params is NULL");
  return fwd_with_map(p, p->map, static_cast<hipStream_t>(stream));
}

int flexattn_fwd_noalloc(const flexattn_fwd_params* p, void* stream) {
  if (p == nullptr) return set_error(FLEXATTN_EINVAL, "params is NULL");
  if (p->B <= 0 || p->Hq <= 0 || p->Hkv <= 0 || p->Sq <= 0 || p->Sk <= 0 || p->D <= 0)
    return set_error(FLEXATTN_EINVAL, "non-positive dimension (B=%d Hq=%d Hkv=%d Sq=%d Sk=%d D=%d)", p->B, p->Hq, p->Hkv,
                     p->Sq, p->Sk, p->D);
  int bq = 0, bk = 0;
  int rc = tile_shape(FLEXATTN_PASS_FWD, p->dtype, p->D, &bq, &bk);
  if (rc != FLEXATTN_OK) return rc;
  if (p->Sq % bq != 0) return set_error(FLEXATTN_EINVAL, "Sq=%d is not a multiple of the q tile %d", p->Sq, bq);
  if (p->Sk % bk != 0) return set_error(FLEXATTN_EINVAL, "Sk=%d is not a multiple of the kv tile %d", p->Sk, bk);
  const int nq = p->Sq / bq, nk = p->Sk / bk;
  if (nq > kScratchMaxRows || (long long)nq * nk > kScratchMaxTiles)
    return set_error(FLEXATTN_EINVAL,
                     "flexattn_fwd_noalloc: %d x %d tiles exceed the resident block map (at most %d q tiles and %d tiles "
                     "in all); build a map with flexattn_build_block_mask and call flexattn_fwd",
                     nq, nk, kScratchMaxRows, kScratchMaxTiles);
  if ((rc = check_mask(p->mask)) != FLEXATTN_OK) return rc;
  unsigned char* base = nullptr;
  if ((rc = scratch_of_current_device(&base)) != FLEXATTN_OK) return rc;
  flexattn_block_map map;
  map.state = base + kScratchStateOff;
  map.kv_cnt = reinterpret_cast<const int32_t*>(base + kScratchCntOff);
  map.kv_idx = reinterpret_cast<const int32_t*>(base + kScratchIdxOff);
  map.q_cnt = nullptr;
  map.q_idx = nullptr;
  map.nq = nq; map.nk = nk; map.block_q = bq; map.block_k = bk;
  hipStream_t s = static_cast<hipStream_t>(stream);
  // every state, every count and every list entry below its count is rewritten by the builder: nothing of
  // an earlier call is read, nothing needs clearing
  if ((rc = check_doc_batches(p->mask, p->B)) != FLEXATTN_OK) return rc;
  rc = build_block_mask(to_args(p->mask), p->mask.doc_batches, p->Sq, p->Sk, bq, bk, base + kScratchStateOff,
                        reinterpret_cast<int*>(base + kScratchCntOff), reinterpret_cast<int*>(base + kScratchIdxOff),
                        nullptr, nullptr, s);
  if (rc != FLEXATTN_OK) return rc;
  return fwd_with_map(p, map, s);
}

int flexattn_bwd_delta(const void* o, const void* dout, float* delta, int64_t rows, int32_t D, int32_t dtype,
                       void* stream) {
  if (!o || !dout || !delta) return set_error(FLEXATTN_EINVAL, "o, dout or delta is NULL");
  if (rows <= 0) return set_error(FLEXATTN_EINVAL, "rows=%lld must be positive", (long long)rows);
  return bwd_delta(o, dout, delta, rows, D, dtype, static_cast<hipStream_t>(stream));
}

static int launch_dq(const flexattn_bwd_params* p, BwdArgs a, hipStream_t s) {
  if (p->ds != nullptr) return bwd_dq_from_ds(a, ds_out_scale(p), s);
  if (p->dtype == FLEXATTN_BF16) {
    if (a.dab != nullptr) a.flags |= FLEXATTN_FLAG_COMPILED_LOOP;  // (the generated streams store no bias gradient)
    return p->D == 256 ? bwd_dq_bf16_d256(a, s) : bwd_dq_bf16_d128(a, s);
  }
  return (a.flags & FLEXATTN_FLAG_COMPILED_LOOP) ? bwd_dq_f32(a, p->D, s) : bwd_dq_f32_mfma(a, p->D, s);
}

static int launch_dkv(const flexattn_bwd_params* p, const BwdArgs& a, hipStream_t s) {
  if (p->dtype == FLEXATTN_BF16) return p->D == 256 ? bwd_dkv_bf16_d256(a, s) : bwd_dkv_bf16_d128(a, s);
  return (a.flags & FLEXATTN_FLAG_COMPILED_LOOP) ? bwd_dkv_f32(a, p->D, s) : bwd_dkv_f32_mfma(a, p->D, s);
}

int flexattn_bwd(const flexattn_bwd_params* pq, const flexattn_bwd_params* pkv, void* stream) {
  BwdArgs aq, akv;
  int rc = to_bwd_args(pq, FLEXATTN_PASS_DQ, &aq);
  if (rc != FLEXATTN_OK) return rc;
  if ((rc = to_bwd_args(pkv, FLEXATTN_PASS_DKV, &akv)) != FLEXATTN_OK) return rc;
  if (pq->ds != nullptr || pkv->ds != nullptr)
    return set_error(FLEXATTN_EINVAL, "flexattn_bwd runs the two passes side by side: no dS hand-over (call flexattn_bwd_dkv, then flexattn_bwd_dq)");
  if (pq->B != pkv->B || pq->Hq != pkv->Hq || pq->Hkv != pkv->Hkv || pq->Sq != pkv->Sq || pq->Sk != pkv->Sk || pq->D != pkv->D ||
      pq->dtype != pkv->dtype || pq->q != pkv->q || pq->k != pkv->k || pq->v != pkv->v || pq->dout != pkv->dout)
    return set_error(FLEXATTN_EINVAL, "flexattn_bwd: the two parameter blocks describe different problems");
  hipStream_t s = static_cast<hipStream_t>(stream);
  // delta once, for both passes
  if (pq->o != nullptr) {
    if (pkv->o == nullptr && pkv->delta != pq->delta_out)
      return set_error(FLEXATTN_EINVAL, "flexattn_bwd: the dk/dv block must read the delta that the dq block's call computes");
    if ((rc = delta_first(&aq, pq->D, pq->dtype, s)) != FLEXATTN_OK) return rc;
    akv.delta = aq.delta;
    akv.o = nullptr;
  } else if ((rc = delta_first(&akv, pkv->D, pkv->dtype, s)) != FLEXATTN_OK) {
    return rc;
  }
  // (The two passes do not depend on each other, but running them side by side on two streams does not pay where it
  // could, on problems too small to fill the GPU: those are bound by the host's launch path, and the event record /
  // wait pairs of a fork and a join cost it more than the overlap saves: measured on B=1, H=4, S=512, fp32: 110 us
  // per backward against 65 us for the three launches in a row.)
  if ((rc = launch_dq(pq, aq, s)) != FLEXATTN_OK) return rc;
  return launch_dkv(pkv, akv, s);
}

int64_t flexattn_bwd_ds_bytes(const flexattn_bwd_params* p) { return ds_exchange_ok(p) ? ds_bytes_of(p) : 0; }

int flexattn_bwd_dq(const flexattn_bwd_params* p, void* stream) {
  BwdArgs a;
  int rc = to_bwd_args(p, FLEXATTN_PASS_DQ, &a);
  if (rc != FLEXATTN_OK) return rc;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if ((rc = delta_first(&a, p->D, p->dtype, s)) != FLEXATTN_OK) return rc;
  return launch_dq(p, a, s);   // (ds: checked to be bf16 and a plain or softcap score; the softcap streams leave 4 out of dS)
}

int flexattn_bwd_dkv(const flexattn_bwd_params* p, void* stream) {
  BwdArgs a;
  int rc = to_bwd_args(p, FLEXATTN_PASS_DKV, &a);
  if (rc != FLEXATTN_OK) return rc;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if ((rc = delta_first(&a, p->D, p->dtype, s)) != FLEXATTN_OK) return rc;
  return launch_dkv(p, a, s);
}

}  // extern "C"
