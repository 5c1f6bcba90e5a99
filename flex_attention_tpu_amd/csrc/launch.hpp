// Host-side helpers shared by the launch code: error recording and kernel entry declarations.
#pragma once
#include <hip/hip_runtime.h>

#include "fa_common.hpp"

namespace fa {

// Records a printf-style message for flexattn_last_error_string() and returns `code`.
int set_error(int code, const char* fmt, ...);

// Returns FLEXATTN_OK, or records hipGetLastError() under `what`.
int check_launch(const char* what);

// bf16, head dim 128 (MFMA kernels)
int fwd_bf16_d128(const FwdArgs& a, hipStream_t stream);
int fwd_bf16_d256(const FwdArgs& a, hipStream_t stream);   // (same tiles as head dim 128)
void fwd_bf16_d128_tile(int* bq, int* bk);
int bwd_dq_bf16_d128(const BwdArgs& a, hipStream_t stream);
int bwd_dq_bf16_d256(const BwdArgs& a, hipStream_t stream);
void bwd_dq_bf16_d128_tile(int* bq, int* bk);
int bwd_dkv_bf16_d128(const BwdArgs& a, hipStream_t stream);
int bwd_dkv_bf16_d256(const BwdArgs& a, hipStream_t stream);
// (the dk/dv pass of such a request runs the generated stream: its exported dS then lacks sm_scale and the soft-cap's
// factor 4; the kernel with a compiled main loop exports dS complete)
bool bwd_dkv_bf16_d128_on_stream(int kind, int flags, int nq, bool has_ab, int Hq, int Hkv);
void bwd_dkv_bf16_d128_tile(int* bq, int* bk);
// dq = out_scale dS K from the dS blocks that the dk/dv stream kernels wrote to a.ds (a.map: row lists at the
// dk/dv tiles)
int bwd_dq_from_ds(const BwdArgs& a, float out_scale, hipStream_t stream);

// fp32, head dim 64 or 128 (FMA kernels, exact-arithmetic path)
int fwd_f32(const FwdArgs& a, int D, hipStream_t stream);
int bwd_dq_f32(const BwdArgs& a, int D, hipStream_t stream);
int bwd_dkv_f32(const BwdArgs& a, int D, hipStream_t stream);
void f32_tile(int* bq, int* bk);
// the same on the fp32 matrix cores (the default; FLEXATTN_FLAG_COMPILED_LOOP selects the FMA kernels)
int fwd_f32_mfma(const FwdArgs& a, int D, hipStream_t stream);
int bwd_dq_f32_mfma(const BwdArgs& a, int D, hipStream_t stream);
int bwd_dkv_f32_mfma(const BwdArgs& a, int D, hipStream_t stream);

int bwd_delta(const void* o, const void* dout, float* delta, int64_t rows, int D, int dtype, hipStream_t stream);

// (doc_batches: batch entries the mask's document arrays hold a row for; the map is the union over them)
int build_block_mask(const MaskArgs& mask, int doc_batches, int Sq, int Sk, int block_q, int block_k, uint8_t* state,
                     int* kv_cnt, int* kv_idx, int* q_cnt, int* q_idx, hipStream_t stream);

int build_ds_index(const uint8_t* state, const int* q_cnt, const int* q_idx, int nq, int nk, int* col, int* rank,
                   hipStream_t stream);

}  // namespace fa
