// Experts chosen by a table: token id t runs the ``top`` experts table[t, 0 .. top-1], each a gated feed-forward
//     y_e(h) = Wd_e (silu(Wg_e h) * (Wu_e h)),
// and the layer's output is base + weight * sum_k y_{table[t, k]}(h) (base: what runs for every token, or nothing).
// The choice is read on the device from the step's token ids, so a step needs nothing from the host and can be
// replayed from a graph. The experts' matrices lie stacked: Wgu [E, 2 F, W] (gate rows, then up rows), Wd [E, W, F].
//
// Few tokens (decoding): every (token, choice) streams its expert's rows, a wave per output, the token's vector in
// LDS. Accumulation in float32.
#include "common.h"

#include <math.h>

#define MOE_THREADS 256
#define MOE_WAVES (MOE_THREADS / LMSF_WAVE)
#define MOE_OUT_PER_WAVE 4

// act[(n * top + k), f] = silu(Wg_e[f] . h[n]) * (Wu_e[f] . h[n]),  e = table[ids[n], k]
template <typename T>
__global__ __launch_bounds__(MOE_THREADS) void moe_gate_up_kernel(
    const T* __restrict__ h, long h_stride, const T* __restrict__ Wgu, const int* __restrict__ ids,
    const int* __restrict__ table, int vocab, int top, int E, T* __restrict__ act, int F, int W) {
  extern __shared__ float sh[];   // [W]
  const int nk = blockIdx.x, n = nk / top, k = nk - n * top;
  const int id = min(max(ids[n], 0), vocab - 1);
  const int e = min(max(table[(long)id * top + k], 0), E - 1);
  for (int i = threadIdx.x; i < W; i += MOE_THREADS) sh[i] = to_f32<T>(h[(long)n * h_stride + i]);
  __syncthreads();
  const int wave = threadIdx.x / LMSF_WAVE, lane = threadIdx.x % LMSF_WAVE;
  const int f0 = (blockIdx.y * MOE_WAVES + wave) * MOE_OUT_PER_WAVE;
  const T* We = Wgu + (long)e * 2 * F * W;
  for (int f = f0; f < min(F, f0 + MOE_OUT_PER_WAVE); ++f) {
    const T* g = We + (long)f * W;
    const T* u = We + (long)(F + f) * W;
    float ag = 0.f, au = 0.f;
    for (int i = lane; i < W; i += LMSF_WAVE) {
      const float x = sh[i];
      ag += to_f32<T>(g[i]) * x;
      au += to_f32<T>(u[i]) * x;
    }
    ag = wave_sum(ag);
    au = wave_sum(au);
    if (lane == 0) {
      // the two products are rounded as stored activations are, then the activation in float32
      const float gg = to_f32<T>(from_f32<T>(ag)), uu = to_f32<T>(from_f32<T>(au));
      act[(long)nk * F + f] = from_f32<T>(gg / (1.f + expf(-gg)) * uu);
    }
  }
}

// out[n, o] = base[n, o] + weight * sum_k Wd_{e_k}[o] . act[n * top + k]
template <typename T>
__global__ __launch_bounds__(MOE_THREADS) void moe_down_kernel(
    const T* __restrict__ act, const T* __restrict__ Wd, const int* __restrict__ ids, const int* __restrict__ table,
    int vocab, int top, int E, float weight, const T* __restrict__ base, long base_stride, T* __restrict__ out,
    long out_stride, int F, int W) {
  extern __shared__ float sa[];   // [top, F]
  const int n = blockIdx.x;
  const int id = min(max(ids[n], 0), vocab - 1);
  for (int i = threadIdx.x; i < top * F; i += MOE_THREADS) sa[i] = to_f32<T>(act[(long)n * top * F + i]);
  __syncthreads();
  const int wave = threadIdx.x / LMSF_WAVE, lane = threadIdx.x % LMSF_WAVE;
  const int o0 = (blockIdx.y * MOE_WAVES + wave) * MOE_OUT_PER_WAVE;
  for (int o = o0; o < min(W, o0 + MOE_OUT_PER_WAVE); ++o) {
    float total = 0.f;
    for (int k = 0; k < top; ++k) {
      const int e = min(max(table[(long)id * top + k], 0), E - 1);
      const T* wr = Wd + ((long)e * W + o) * F;
      float a = 0.f;
      for (int i = lane; i < F; i += LMSF_WAVE) a += to_f32<T>(wr[i]) * sa[k * F + i];
      total += wave_sum(a);
    }
    if (lane == 0) {
      const float b = base ? to_f32<T>(base[(long)n * base_stride + o]) : 0.f;
      out[(long)n * out_stride + o] = from_f32<T>(b + weight * total);
    }
  }
}

extern "C" int lmsf_table_moe(const void* h, int dtype, long h_stride, const void* Wgu, const void* Wd, const int* ids,
                              const int* table, int vocab, int top, int E, float weight, const void* base,
                              long base_stride, void* act, void* out, long out_stride, int n_tokens, int F, int W,
                              hipStream_t stream) {
  LMSF_CHECK(h && Wgu && Wd && ids && table && act && out, "table_moe: null pointer");
  LMSF_CHECK(dtype == LMSF_F32 || dtype == LMSF_BF16, "table_moe: unknown dtype code %d", dtype);
  LMSF_CHECK(vocab > 0 && top > 0 && E > 0 && F > 0 && W > 0, "table_moe: bad sizes");
  LMSF_CHECK(h_stride >= W && out_stride >= W && (!base || base_stride >= W), "table_moe: rows overlap");
  LMSF_CHECK((size_t)W * 4 <= 64 * 1024 && (size_t)top * F * 4 <= 64 * 1024, "table_moe: a row does not fit LDS");
  LMSF_CHECK((long)n_tokens * top < 2147483647L, "table_moe: too many rows");
  if (n_tokens <= 0) return 0;
  const int per_block = MOE_WAVES * MOE_OUT_PER_WAVE;
  const dim3 g1(n_tokens * top, (F + per_block - 1) / per_block), g2(n_tokens, (W + per_block - 1) / per_block);
  if (dtype == LMSF_F32) {
    hipLaunchKernelGGL((moe_gate_up_kernel<float>), g1, dim3(MOE_THREADS), (size_t)W * 4, stream, (const float*)h,
                       h_stride, (const float*)Wgu, ids, table, vocab, top, E, (float*)act, F, W);
    hipLaunchKernelGGL((moe_down_kernel<float>), g2, dim3(MOE_THREADS), (size_t)top * F * 4, stream, (const float*)act,
                       (const float*)Wd, ids, table, vocab, top, E, weight, (const float*)base, base_stride,
                       (float*)out, out_stride, F, W);
  } else {
    hipLaunchKernelGGL((moe_gate_up_kernel<bf16_t>), g1, dim3(MOE_THREADS), (size_t)W * 4, stream, (const bf16_t*)h,
                       h_stride, (const bf16_t*)Wgu, ids, table, vocab, top, E, (bf16_t*)act, F, W);
    hipLaunchKernelGGL((moe_down_kernel<bf16_t>), g2, dim3(MOE_THREADS), (size_t)top * F * 4, stream,
                       (const bf16_t*)act, (const bf16_t*)Wd, ids, table, vocab, top, E, weight, (const bf16_t*)base,
                       base_stride, (bf16_t*)out, out_stride, F, W);
  }
  LMSF_LAUNCH_CHECK("table_moe");
  return 0;
}
