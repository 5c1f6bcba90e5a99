// Block-mask builder: one launch turns a mask specification into the tile state map and the
// compacted per-row / per-column visit lists that the attention kernels walk.
#include "fa_common.hpp"
#include "launch.hpp"

namespace fa {

// State of tile (qb, kb): 0 skip, 1 partial, 2 full.  `run` is the AND of the block predicates
// of the flags set: causal k_start <= q_end; window q_start - k_end < window; document: the id
// ranges read at the block ends overlap (ids are non-decreasing); S2: k_start <= q_end.
// With a compiled mask predicate (FLEXATTN_MASK_CUSTOM) there is no closed form: the element predicate is
// evaluated on every element of the tile, run = any kept, full = all kept, which is what the Python block
// closure of a compiled mask returns (any(mask_fn over the tile)).
__device__ __forceinline__ int tile_state(const MaskArgs& mk, int qb, int kb, int bq, int bk, bool sorted_ids) {
  const int q_start = qb * bq, q_end = q_start + bq - 1;
  const int k_start = kb * bk, k_end = k_start + bk - 1;
#if FLEXATTN_CUSTOM_HAS_MASK
  if (mk.flags & FLEXATTN_MASK_CUSTOM) {
    const bool has_doc = (mk.flags & FLEXATTN_MASK_DOC) != 0;
    bool any = false, all = true;
    for (int i = q_start; i <= q_end; ++i) {
      const int doc_i = has_doc ? mk.doc_q[i] : 0;
      for (int j = k_start; j <= k_end; ++j) {
        const bool keep = keep_elem(mk, i, j, doc_i, has_doc ? mk.doc_k[j] : 0);
        any = any | keep;
        all = all & keep;
      }
    }
    return any ? (all ? 2 : 1) : 0;
  }
#endif
  bool run = true, full = true;
  if (mk.flags & FLEXATTN_MASK_S2) {
    run = k_start <= q_end;
    full = (k_end <= q_start) && (q_end - k_start < mk.window);
  } else {
    if (mk.flags & FLEXATTN_MASK_CAUSAL) {
      run = run && (k_start <= q_end);
      full = full && (k_end <= q_start);
    }
    if (mk.flags & FLEXATTN_MASK_WINDOW) {
      run = run && (q_start - k_end < mk.window);
      full = full && (q_end - k_start < mk.window);
    }
  }
  if (mk.flags & FLEXATTN_MASK_DOC) {
    // smallest and largest id of each block: read at the block ends when the ids are sorted (what the
    // reference's closure does, masks.py:113-139), by a scan of the block otherwise
    int qmin = mk.doc_q[q_start], qmax = mk.doc_q[q_end];
    int kmin = mk.doc_k[k_start], kmax = mk.doc_k[k_end];
    if (!sorted_ids) {
      for (int i = q_start; i <= q_end; ++i) {
        const int d = mk.doc_q[i];
        qmin = d < qmin ? d : qmin;
        qmax = d > qmax ? d : qmax;
      }
      for (int j = k_start; j <= k_end; ++j) {
        const int d = mk.doc_k[j];
        kmin = d < kmin ? d : kmin;
        kmax = d > kmax ? d : kmax;
      }
    }
    const int lo = qmin > kmin ? qmin : kmin;
    const int hi = qmax < kmax ? qmax : kmax;
    run = run && (lo <= hi);
    full = full && (qmin == qmax) && (kmin == kmax) && (qmin == kmin);
  }
  return run ? (full ? 2 : 1) : 0;
}

// Work-groups [0, nq) own one q-block row each: write its states and its ascending kv list.
// Work-groups [nq, nq + nk) own one kv-block column each: write its ascending q list.
// `batches`: number of batch entries the document arrays hold a row for (1: one row for all).  The map is then the
// union over the entries: a tile runs if it runs for any entry and is full only if it is full for every entry (an
// entry that keeps nothing of a tile it visits masks every element of it).
__global__ __launch_bounds__(64) void block_mask_kernel(MaskArgs mk, int batches, int nq, int nk, int bq, int bk,
                                                        uint8_t* state, int* kv_cnt, int* kv_idx,
                                                        int* q_cnt, int* q_idx) {
  const int lane = threadIdx.x;
  // Are the document ids non-decreasing on both sides (of every entry)?  Every work-group checks for itself (the
  // arrays are a few KB): the block ends then bound a block's ids.
  bool sorted_ids = true;
  if (mk.flags & FLEXATTN_MASK_DOC) {
    bool ok = true;
    for (int e = 0; e < batches; ++e) {
      const MaskArgs me = mask_of_batch(mk, e, nq * bq, nk * bk);
      for (int i = lane + 1; i < nq * bq; i += 64) ok = ok && (me.doc_q[i - 1] <= me.doc_q[i]);
      for (int j = lane + 1; j < nk * bk; j += 64) ok = ok && (me.doc_k[j - 1] <= me.doc_k[j]);
    }
    sorted_ids = __ballot(!ok) == 0ull;
  }
  auto tile_state_all = [&](int qb, int kb) {
    int st = tile_state(mk, qb, kb, bq, bk, sorted_ids);
    for (int e = 1; e < batches; ++e) {
      const int se = tile_state(mask_of_batch(mk, e, nq * bq, nk * bk), qb, kb, bq, bk, sorted_ids);
      st = (st == 0 && se == 0) ? 0 : ((st == 2 && se == 2) ? 2 : 1);
    }
    return st;
  };
  const bool is_row = (int)blockIdx.x < nq;
  const int major = is_row ? blockIdx.x : blockIdx.x - nq;
  const int n_minor = is_row ? nk : nq;
  int* cnt = is_row ? kv_cnt : q_cnt;
  int* idx = is_row ? kv_idx : q_idx;
  int total = 0;
  for (int base = 0; base < n_minor; base += 64) {
    const int minor = base + lane;
    int st = 0;
    if (minor < n_minor) {
      st = is_row ? tile_state_all(major, minor) : tile_state_all(minor, major);
      if (is_row) state[(size_t)major * nk + minor] = (uint8_t)st;
    }
    const unsigned long long ballot = __ballot(st != 0);
    if (idx != nullptr && st != 0) {
      const int pos = total + __popcll(ballot & ((1ull << lane) - 1ull));
      idx[(size_t)major * n_minor + pos] = minor;
    }
    total += __popcll(ballot);
  }
  if (cnt != nullptr && lane == 0) cnt[major] = total;
}

// Index of the dS exchange buffer over the kept tile pairs of a block map, counted kv tile by kv tile:
// col[kb] = kept pairs in the kv tiles before kb (col[nk] = all of them), rank[qb, kb] = col[kb] + position of
// qb in kb's q list, -1 for skipped pairs.  Work-group kb < nk owns column kb; work-group nk writes the total.
__global__ __launch_bounds__(256) void ds_index_kernel(const uint8_t* state, const int* q_cnt, const int* q_idx, int nq,
                                                       int nk, int* col, int* rank) {
  __shared__ int part[256];
  const int kb = blockIdx.x;
  const int tid = threadIdx.x;
  int sum = 0;
  for (int k = tid; k < kb; k += 256) sum += q_cnt[k];
  part[tid] = sum;
  __syncthreads();
  for (int step = 128; step > 0; step >>= 1) {
    if (tid < step) part[tid] += part[tid + step];
    __syncthreads();
  }
  const int first = part[0];
  if (tid == 0) col[kb] = first;
  if (kb == nk) return;
  // (skipped pairs and kept pairs are written by disjoint threads: a pair is in the list exactly when its state is not 0)
  for (int qb = tid; qb < nq; qb += 256)
    if (state[(size_t)qb * nk + kb] == 0) rank[(size_t)qb * nk + kb] = -1;
  const int n = q_cnt[kb];
  for (int t = tid; t < n; t += 256) rank[(size_t)q_idx[(size_t)kb * nq + t] * nk + kb] = first + t;
}

int build_ds_index(const uint8_t* state, const int* q_cnt, const int* q_idx, int nq, int nk, int* col, int* rank,
                   hipStream_t stream) {
  hipLaunchKernelGGL(ds_index_kernel, dim3(nk + 1), dim3(256), 0, stream, state, q_cnt, q_idx, nq, nk, col, rank);
  return check_launch("flexattn_build_ds_index");
}

int build_block_mask(const MaskArgs& mask, int doc_batches, int Sq, int Sk, int block_q, int block_k, uint8_t* state,
                     int* kv_cnt, int* kv_idx, int* q_cnt, int* q_idx, hipStream_t stream) {
  const int nq = Sq / block_q, nk = Sk / block_k;
  const bool want_cols = q_cnt != nullptr;
  const int grid = nq + (want_cols ? nk : 0);
  hipLaunchKernelGGL(block_mask_kernel, dim3(grid), dim3(64), 0, stream, mask, doc_batches > 1 ? doc_batches : 1, nq, nk, block_q, block_k,
                     state, kv_cnt, kv_idx, q_cnt, q_idx);
  return check_launch("flexattn_build_block_mask");
}

}  // namespace fa
