// Dynamic Tanh in the place of a norm, around the float32 residual stream:
//
//   r = (residual ? residual[src] : 0) + (branch ? branch[src] : 0)       src = rows ? rows[row] : row
//   residual[row] = r                                                     (branch and residual given, no rows)
//   out[row] = tanh(alpha * r) * w + b
//
// alpha is one learned number (read from device memory), w and b vectors. No mean and no variance are computed,
// so nothing crosses a row: a thread an element (four neighbours where the row allows it). All arithmetic is
// float32; branch and out are float32 or bfloat16. The reference's only norm is RMSNorm
// (vllm/kernels/layernorm_kernels.cu:13-38), with the same fused addition (:41-68).
#include "common.h"
#include "entry_points.h"

#include <math.h>

template <typename TB, typename TO, int V>
__global__ __launch_bounds__(256) void dyt_norm_kernel(const TB* __restrict__ branch, float* __restrict__ residual,
                                                       const float* __restrict__ w, const float* __restrict__ b,
                                                       const float* __restrict__ alpha, TO* __restrict__ out,
                                                       const int* __restrict__ rows, int H) {
  const int row = blockIdx.x;
  const long src = rows ? rows[row] : row;
  const int i0 = (blockIdx.y * 256 + threadIdx.x) * V;
  if (i0 >= H) return;
  const float a = alpha[0];
  float r[V];
#pragma unroll
  for (int e = 0; e < V; ++e) {
    r[e] = residual ? residual[src * H + i0 + e] : 0.f;
    if (branch) r[e] += to_f32<TB>(branch[src * H + i0 + e]);
  }
  if (branch && residual && !rows) {
#pragma unroll
    for (int e = 0; e < V; ++e) residual[src * H + i0 + e] = r[e];
  }
#pragma unroll
  for (int e = 0; e < V; ++e) out[(long)row * H + i0 + e] = from_f32<TO>(tanhf(a * r[e]) * w[i0 + e] + b[i0 + e]);
}

extern "C" int lmsf_dyt_norm(const void* branch, int branch_dtype, float* residual, const float* w, const float* b,
                             const float* alpha, void* out, int out_dtype, const int* rows, int n_rows, int H,
                             hipStream_t stream) {
  LMSF_CHECK(w && b && alpha && out, "dyt_norm: null pointer");
  LMSF_CHECK(branch || residual, "dyt_norm: neither a branch nor a residual");
  LMSF_CHECK(n_rows >= 0 && H > 0, "dyt_norm: bad sizes rows=%d H=%d", n_rows, H);
  LMSF_CHECK((branch_dtype == LMSF_F32 || branch_dtype == LMSF_BF16) && (out_dtype == LMSF_F32 || out_dtype == LMSF_BF16),
             "dyt_norm: unknown dtype code");
  if (n_rows == 0) return 0;
  const bool v4 = H % 4 == 0;
  const int per = v4 ? 4 : 1;
  dim3 grid(n_rows, (H / per + 255) / 256), block(256);
#define DYT(TB, TO)                                                                                                    \
  do {                                                                                                                 \
    if (v4)                                                                                                            \
      hipLaunchKernelGGL((dyt_norm_kernel<TB, TO, 4>), grid, block, 0, stream, (const TB*)branch, residual, w, b,      \
                         alpha, (TO*)out, rows, H);                                                                    \
    else                                                                                                               \
      hipLaunchKernelGGL((dyt_norm_kernel<TB, TO, 1>), grid, block, 0, stream, (const TB*)branch, residual, w, b,      \
                         alpha, (TO*)out, rows, H);                                                                    \
  } while (0)
  if (branch_dtype == LMSF_F32 && out_dtype == LMSF_F32) DYT(float, float);
  else if (branch_dtype == LMSF_F32) DYT(float, bf16_t);
  else if (out_dtype == LMSF_F32) DYT(bf16_t, float);
  else DYT(bf16_t, bf16_t);
#undef DYT
  LMSF_LAUNCH_CHECK("dyt_norm");
  return 0;
}
