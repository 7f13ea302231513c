// RMS norm in groups around a float32 residual stream, with the additions that surround it.
//
// A row of W numbers is cut into ``groups`` equal consecutive parts; part g is divided by
// sqrt(mean(part^2) + eps) and the whole row is multiplied by a weight:  gn(x; w)_i = x_i / rms_g(i) * w_i.
// groups = 1 is the plain RMS norm.
//
// One kernel serves the arrangements in which a layer uses such norms; every operand is optional:
//
//   v = branch ? gn(branch[row]; wb) : 0                    the norm *after* a sublayer
//   r = residual ? residual[src] + v : v                    src = rows ? rows[row] : row
//   residual[row] = r                                       (branch, residual, no rows)
//   hist[k][row] = r;  x = sum_{j<=k} mix[j] hist[j][row];  residual[row] = x      (hist: a weighted average over
//                                                           the results of all layers so far, r being the k-th)
//   out[row] = wn ? gn(x; wn) : x                           the norm *before* the next sublayer
//
// All arithmetic is float32; branch and out are float32 or bfloat16, the weights float32. One workgroup a row
// (256 to 1,024 threads), the row kept in LDS between the passes; the stream's row and the earlier results are asked
// for before the first pass, so that the passes do not each wait for memory.
#include "common.h"

#include <math.h>

#define GN_MAX_THREADS 1024
#define GN_THREADS ((int)blockDim.x)

template <typename T>
__device__ __forceinline__ float gn_load(const void* p, long i) { return to_f32<T>(((const T*)p)[i]); }

// divides the row in LDS by its groups' root mean squares and multiplies by w; ``red`` is block_sum's scratch
__device__ __forceinline__ void gn_normalize(float* row, const float* __restrict__ w, int W, int groups, float eps,
                                             float* red) {
  const int gw = W / groups;
  for (int g = 0; g < groups; ++g) {
    float ss = 0.f;
    for (int i = threadIdx.x; i < gw; i += GN_THREADS) {
      const float x = row[g * gw + i];
      ss += x * x;
    }
    ss = block_sum(ss, red);
    const float rms = sqrtf(ss / (float)gw + eps);
    for (int i = threadIdx.x; i < gw; i += GN_THREADS) row[g * gw + i] = row[g * gw + i] / rms * w[g * gw + i];
  }
  __syncthreads();
}

template <typename TB, typename TO>
__global__ __launch_bounds__(GN_MAX_THREADS) void group_norm_kernel(
    const TB* __restrict__ branch, long branch_stride, const float* __restrict__ wb, float* __restrict__ residual,
    float* __restrict__ hist, long hist_stride, int hist_index, const float* __restrict__ mix,
    const float* __restrict__ wn, TO* __restrict__ out, long out_stride, const int* __restrict__ rows, int W,
    int groups, float eps_b, float eps_n) {
  extern __shared__ float row[];   // [W] the row; [W] the stream's row; [W] the earlier results' share of the average
  float* res = row + W;
  float* before = row + 2 * W;
  __shared__ float red[16];
  const int n = blockIdx.x;
  const int src = rows ? rows[n] : n;
  // everything that comes from memory is asked for at once: the passes below would otherwise each wait for their own
  if (residual)
    for (int i = threadIdx.x; i < W; i += GN_THREADS) res[i] = residual[(long)src * W + i];
  if (hist)
    for (int i = threadIdx.x; i < W; i += GN_THREADS) {
      float x = 0.f;
#pragma unroll 8
      for (int j = 0; j < hist_index; ++j) x += mix[j] * hist[(long)j * hist_stride + (long)n * W + i];
      before[i] = x;
    }
  if (branch) {
    for (int i = threadIdx.x; i < W; i += GN_THREADS) row[i] = to_f32<TB>(branch[(long)n * branch_stride + i]);
    __syncthreads();
    gn_normalize(row, wb, W, groups, eps_b, red);
  }
  // (each thread reads back the entries of res and before that it wrote itself)
  if (residual) {
    const bool store = branch && !rows && !hist;
    for (int i = threadIdx.x; i < W; i += GN_THREADS) {
      const float r = res[i] + (branch ? row[i] : 0.f);
      row[i] = r;
      if (store) residual[(long)n * W + i] = r;
    }
  }
  if (hist) {
    for (int i = threadIdx.x; i < W; i += GN_THREADS) {
      const float r = row[i];
      hist[(long)hist_index * hist_stride + (long)n * W + i] = r;
      const float x = before[i] + mix[hist_index] * r;
      row[i] = x;
      residual[(long)n * W + i] = x;
    }
  }
  if (out) {
    __syncthreads();
    if (wn) gn_normalize(row, wn, W, groups, eps_n, red);
    for (int i = threadIdx.x; i < W; i += GN_THREADS) out[(long)n * out_stride + i] = from_f32<TO>(row[i]);
  }
}

template <typename TB, typename TO>
static void gn_launch(int n_rows, size_t smem, hipStream_t stream, const void* branch, long branch_stride,
                      const float* wb, float* residual, float* hist, long hist_stride, int hist_index,
                      const float* mix, const float* wn, void* out, long out_stride, const int* rows, int W,
                      int groups, float eps_b, float eps_n) {
  // few rows: a row's passes wait for memory one after the other, so many threads with few elements each; many
  // rows fill the chip with smaller workgroups
  const int threads = n_rows >= 1024 || W <= 256 ? 256 : W <= 1024 ? 512 : 1024;
  hipLaunchKernelGGL((group_norm_kernel<TB, TO>), dim3(n_rows), dim3(threads), smem, stream, (const TB*)branch,
                     branch_stride, wb, residual, hist, hist_stride, hist_index, mix, wn, (TO*)out, out_stride, rows,
                     W, groups, eps_b, eps_n);
}

extern "C" int lmsf_group_norm(const void* branch, int branch_dtype, long branch_stride, const float* wb,
                               float* residual, float* hist, long hist_stride, int hist_index, const float* mix,
                               const float* wn, void* out, int out_dtype, long out_stride, const int* rows,
                               int n_rows, int W, int groups, float eps_b, float eps_n, hipStream_t stream) {
  LMSF_CHECK(branch || residual, "group_norm: neither a branch nor a residual");
  LMSF_CHECK(W > 0 && groups > 0 && W % groups == 0, "group_norm: %d columns do not split into %d groups", W, groups);
  LMSF_CHECK((size_t)W * 12 <= 160 * 1024 - 256, "group_norm: three rows of %d columns do not fit LDS", W);
  LMSF_CHECK(!branch || wb, "group_norm: a branch needs its weight");
  LMSF_CHECK(!branch || branch_stride >= W, "group_norm: branch rows overlap");
  LMSF_CHECK(!out || out_stride >= W, "group_norm: output rows overlap");
  LMSF_CHECK(!hist || (residual && mix && hist_index >= 0 && hist_stride >= (long)n_rows * W && !rows),
             "group_norm: the running average needs a residual, its weights and whole rows");
  LMSF_CHECK(branch_dtype == LMSF_F32 || branch_dtype == LMSF_BF16, "group_norm: unknown dtype code %d", branch_dtype);
  LMSF_CHECK(out_dtype == LMSF_F32 || out_dtype == LMSF_BF16, "group_norm: unknown dtype code %d", out_dtype);
  if (n_rows <= 0) return 0;
  const size_t smem = (size_t)W * 12;
  if (smem > 64 * 1024) {
    // (once per instantiation would do; the call is cheap)
    hipFuncSetAttribute((const void*)group_norm_kernel<float, float>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    hipFuncSetAttribute((const void*)group_norm_kernel<float, bf16_t>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    hipFuncSetAttribute((const void*)group_norm_kernel<bf16_t, float>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    hipFuncSetAttribute((const void*)group_norm_kernel<bf16_t, bf16_t>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
  }
#define GN_ARGS n_rows, smem, stream, branch, branch_stride, wb, residual, hist, hist_stride, hist_index, mix, wn, out, \
                out_stride, rows, W, groups, eps_b, eps_n
  if (branch_dtype == LMSF_F32 && out_dtype == LMSF_F32) gn_launch<float, float>(GN_ARGS);
  else if (branch_dtype == LMSF_F32) gn_launch<float, bf16_t>(GN_ARGS);
  else if (out_dtype == LMSF_F32) gn_launch<bf16_t, float>(GN_ARGS);
  else gn_launch<bf16_t, bf16_t>(GN_ARGS);
#undef GN_ARGS
  LMSF_LAUNCH_CHECK("group_norm");
  return 0;
}
