// delta_i = sum_c o_ic * do_ic (float32): the row statistic both backward kernels subtract from dP.
// HBM-bound: every lane streams 16 bytes of o and of do; LPR lanes share one row and combine with
// a wavefront butterfly reduction.
#include "fa_common.hpp"
#include "launch.hpp"

namespace fa {

template <typename T, int D>
__global__ __launch_bounds__(256) void delta_kernel(const T* __restrict__ o, const T* __restrict__ dout,
                                                    float* __restrict__ delta, int64_t rows) {
  constexpr int EPL = 16 / sizeof(T);  // elements per lane
  constexpr int LPR = D / EPL;         // lanes per row
  constexpr int RPB = 256 / LPR;       // rows per block
  const int tid = threadIdx.x;
  const int sub = tid % LPR;
  const int64_t n_groups = (rows + RPB - 1) / RPB;
  for (int64_t g = blockIdx.x; g < n_groups; g += gridDim.x) {
    const int64_t row = g * RPB + tid / LPR;
    float acc = 0.f;
    if (row < rows) {
      const u32x4 ov = *reinterpret_cast<const u32x4*>(o + row * D + sub * EPL);
      const u32x4 dv = *reinterpret_cast<const u32x4*>(dout + row * D + sub * EPL);
      if (sizeof(T) == 2) {
        const bf16x8 ob = __builtin_bit_cast(bf16x8, ov);
        const bf16x8 db = __builtin_bit_cast(bf16x8, dv);
#pragma unroll
        for (int e = 0; e < 8; ++e) acc = __builtin_fmaf((float)ob[e], (float)db[e], acc);
      } else {
        const f32x4 of = __builtin_bit_cast(f32x4, ov);
        const f32x4 df = __builtin_bit_cast(f32x4, dv);
#pragma unroll
        for (int e = 0; e < 4; ++e) acc = __builtin_fmaf(of[e], df[e], acc);
      }
    }
#pragma unroll
    for (int off = LPR / 2; off > 0; off >>= 1) acc += __shfl_xor(acc, off);
    if (row < rows && sub == 0) delta[row] = acc;
  }
}

template <typename T, int D>
static int launch_delta(const void* o, const void* dout, float* delta, int64_t rows, hipStream_t stream) {
  constexpr int RPB = 256 / (D / (16 / (int)sizeof(T)));
  int64_t n_groups = (rows + RPB - 1) / RPB;
  int grid = (int)(n_groups < 256 * 32 ? n_groups : 256 * 32);
  if (grid < 1) grid = 1;
  hipLaunchKernelGGL((delta_kernel<T, D>), dim3(grid), dim3(256), 0, stream, static_cast<const T*>(o),
                     static_cast<const T*>(dout), delta, rows);
  return check_launch("flexattn_bwd_delta");
}

int bwd_delta(const void* o, const void* dout, float* delta, int64_t rows, int D, int dtype, hipStream_t stream) {
  if (dtype == FLEXATTN_BF16 && D == 128) return launch_delta<bf16_t, 128>(o, dout, delta, rows, stream);
  if (dtype == FLEXATTN_BF16 && D == 256) return launch_delta<bf16_t, 256>(o, dout, delta, rows, stream);
  if (dtype == FLEXATTN_BF16 && D == 64) return launch_delta<bf16_t, 64>(o, dout, delta, rows, stream);
  if (dtype == FLEXATTN_F32 && D == 128) return launch_delta<float, 128>(o, dout, delta, rows, stream);
  if (dtype == FLEXATTN_F32 && D == 64) return launch_delta<float, 64>(o, dout, delta, rows, stream);
  return set_error(FLEXATTN_ENOTSUP, "delta: unsupported dtype %d / head dim %d", dtype, D);
}

}  // namespace fa
