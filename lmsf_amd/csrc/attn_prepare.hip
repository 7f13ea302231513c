// What an attention layer with separately sized keys and values does to its projections before the paged attention
// kernels run, and to their result afterwards; and the joining of two mixers that ran side by side.
//
// The attention kernels take one head size D for queries, keys and values. A layer whose keys have ``dim`` and whose
// values ``vdim`` entries runs them at D >= max(dim, vdim): queries and keys are padded with zeros (which leave every
// score as it is), values likewise (the padding's outputs are dropped afterwards). The reference's attention has one
// head size (core/src/model_executor/layers/attention.rs:91-103) and rotates and stores in two kernels
// (vllm/kernels/pos_encoding_kernels.cu:12-36, cache_kernels.cu:150-214).
#include "common.h"
#include "entry_points.h"

#include <math.h>

#include <algorithm>

// Per token and head, in this order, each step optional:
//   q, k <- x / sqrt(mean(x^2) + eps) over the head's dim entries                  (unit_norm)
//   q, k <- rotation of the first ``rot`` entries, pairs (i, i + rot/2), by the position's angles (table != null)
//   q    <- q (1 + temp_coef ln(floor((p + 1) / temp_every) + 1))                  (temp_every > 0)
// q goes to q_out [N, H * D]; k to the token's slot of k_pages [pages, G, ps, D], v to v_pages [pages, G, D, ps]
// (a negative slot stores nothing), all padded with zeros to D. A wave a (token, head).
template <typename T>
__global__ __launch_bounds__(256) void attn_prepare_kernel(
    const T* __restrict__ q, long q_stride, const T* __restrict__ k, long k_stride, const T* __restrict__ v,
    long v_stride, const int* __restrict__ positions, const float* __restrict__ table, int rot, int max_pos,
    const int* __restrict__ slots, T* __restrict__ q_out, long qo_stride, T* __restrict__ k_pages,
    T* __restrict__ v_pages, int H, int G, int dim, int vdim, int D, int ps, int unit_norm, float eps, float temp_coef,
    int temp_every) {
  const int t = blockIdx.x;
  const int wave = threadIdx.x / LMSF_WAVE, lane = threadIdx.x % LMSF_WAVE;
  const int p = positions[t];
  const int slot = slots ? slots[t] : -1;
  const int page = slot >= 0 ? slot / ps : 0, off = slot >= 0 ? slot % ps : 0;
  const float* cs = (table && p < max_pos) ? table + (long)p * rot : nullptr;
  const int half = rot / 2;
  const float temp = temp_every > 0 ? 1.f + temp_coef * logf((float)((p + 1) / temp_every) + 1.f) : 1.f;
  // a wave a head of q, k or v: workgroup y takes the heads 4 y .. 4 y + 3 of the row q heads | k heads | v heads
  for (int u = blockIdx.y * (256 / LMSF_WAVE) + wave; u < H + 2 * G; u += gridDim.y * (256 / LMSF_WAVE)) {
    if (u < H + G) {
      const bool is_q = u < H;
      const int head = is_q ? u : u - H;
      if (!is_q && slot < 0) continue;
      const T* src = is_q ? q + (long)t * q_stride + (long)head * dim : k + (long)t * k_stride + (long)head * dim;
      float inv = 1.f;
      if (unit_norm) {
        float ss = 0.f;
        for (int e = lane; e < dim; e += LMSF_WAVE) {
          const float x = to_f32<T>(src[e]);
          ss += x * x;
        }
        ss = wave_sum(ss);
        inv = 1.f / sqrtf(ss / (float)dim + eps);
      }
      const float mul = is_q ? temp : 1.f;
      T* dst = is_q ? q_out + (long)t * qo_stride + (long)head * D
                    : k_pages + (((long)page * G + head) * ps + off) * D;
      for (int e = lane; e < D; e += LMSF_WAVE) {
        float x = 0.f;
        if (e < dim) {
          x = to_f32<T>(src[e]) * inv;
          if (cs && e < rot) {
            const bool first = e < half;
            const float other = to_f32<T>(src[first ? e + half : e - half]) * inv;
            const float c = cs[first ? e : e - half], sn = cs[half + (first ? e : e - half)];
            float a, b;
            if (first) rope_rotate(x, other, c, sn, &a, &b); else rope_rotate(other, x, c, sn, &b, &a);
            x = a;
          }
          x *= mul;
        }
        dst[e] = from_f32<T>(x);
      }
    } else {
      if (slot < 0) continue;
      const int head = u - H - G;
      const T* src = v + (long)t * v_stride + (long)head * vdim;
      T* dst = v_pages + ((long)page * G + head) * D * ps + off;
      for (int e = lane; e < D; e += LMSF_WAVE) dst[(long)e * ps] = e < vdim ? src[e] : from_f32<T>(0.f);
    }
  }
}

extern "C" int lmsf_attn_prepare(const void* q, long q_stride, const void* k, long k_stride, const void* v,
                                 long v_stride, int dtype, const int* positions, const float* table, int rot,
                                 int max_pos, const int* slots, void* q_out, long qo_stride, void* k_pages,
                                 void* v_pages, long num_pages, int n_tokens, int H, int G, int dim, int vdim, int D,
                                 int ps, int unit_norm, float eps, float temp_coef, int temp_every,
                                 hipStream_t stream) {
  LMSF_CHECK(q && k && v && positions && q_out, "attn_prepare: null pointer");
  LMSF_CHECK(dtype == LMSF_F32 || dtype == LMSF_BF16, "attn_prepare: unknown dtype code %d", dtype);
  LMSF_CHECK(H > 0 && G > 0 && H % G == 0 && dim > 0 && vdim > 0 && D >= dim && D >= vdim,
             "attn_prepare: bad sizes H=%d G=%d dim=%d vdim=%d D=%d", H, G, dim, vdim, D);
  LMSF_CHECK(q_stride >= (long)H * dim && k_stride >= (long)G * dim && v_stride >= (long)G * vdim &&
                 qo_stride >= (long)H * D, "attn_prepare: strides too small");
  LMSF_CHECK(!table || (rot > 0 && rot % 2 == 0 && rot <= dim && max_pos > 0), "attn_prepare: bad rotation %d of %d", rot,
             dim);
  LMSF_CHECK(!slots || (k_pages && v_pages && ps > 0 && num_pages > 0), "attn_prepare: slots without pages");
  LMSF_CHECK(temp_every >= 0, "attn_prepare: negative temperature period");
  if (n_tokens == 0) return 0;
  // few tokens: the heads spread over workgroups (8 tokens: 8.4 -> 4.1 us); many: a workgroup a token walks its heads
  // (2,048 tokens: 17.4 us against 23 with the heads spread)
  const dim3 grid(n_tokens, n_tokens >= 256 ? 1 : std::min((H + 2 * G + 3) / 4, 65535));
  if (dtype == LMSF_F32)
    hipLaunchKernelGGL((attn_prepare_kernel<float>), grid, dim3(256), 0, stream, (const float*)q, q_stride,
                       (const float*)k, k_stride, (const float*)v, v_stride, positions, table, rot, max_pos, slots,
                       (float*)q_out, qo_stride, (float*)k_pages, (float*)v_pages, H, G, dim, vdim, D, ps, unit_norm, eps,
                       temp_coef, temp_every);
  else
    hipLaunchKernelGGL((attn_prepare_kernel<bf16_t>), grid, dim3(256), 0, stream, (const bf16_t*)q, q_stride,
                       (const bf16_t*)k, k_stride, (const bf16_t*)v, v_stride, positions, table, rot, max_pos, slots,
                       (bf16_t*)q_out, qo_stride, (bf16_t*)k_pages, (bf16_t*)v_pages, H, G, dim, vdim, D, ps, unit_norm,
                       eps, temp_coef, temp_every);
  LMSF_LAUNCH_CHECK("attn_prepare");
  return 0;
}

// out[n, h * dv + e] = x[n, h * x_head + e] * sigmoid(gate[n, h * dv + e])   (gate null: the plain copy that drops the
// padding behind each head's dv entries)
template <typename T>
__global__ __launch_bounds__(256) void head_gate_kernel(const T* __restrict__ x, long x_stride, int x_head,
                                                        const T* __restrict__ gate, long gate_stride,
                                                        T* __restrict__ out, long out_stride, int H, int dv) {
  const long n = blockIdx.x;
  const int i = blockIdx.y * 256 + threadIdx.x;
  if (i >= H * dv) return;
  const int h = i / dv, e = i % dv;
  float val = to_f32<T>(x[n * x_stride + (long)h * x_head + e]);
  if (gate) val *= 1.f / (1.f + expf(-to_f32<T>(gate[n * gate_stride + i])));
  out[n * out_stride + i] = from_f32<T>(val);
}

extern "C" int lmsf_head_gate(const void* x, int dtype, long x_stride, int x_head, const void* gate, long gate_stride,
                              void* out, long out_stride, int n_tokens, int H, int dv, hipStream_t stream) {
  LMSF_CHECK(x && out, "head_gate: null pointer");
  LMSF_CHECK(dtype == LMSF_F32 || dtype == LMSF_BF16, "head_gate: unknown dtype code %d", dtype);
  LMSF_CHECK(H > 0 && dv > 0 && x_head >= dv && x_stride >= (long)(H - 1) * x_head + dv && out_stride >= (long)H * dv &&
                 (!gate || gate_stride >= (long)H * dv), "head_gate: bad sizes");
  if (n_tokens == 0) return 0;
  dim3 grid(n_tokens, (H * dv + 255) / 256), block(256);
  if (dtype == LMSF_F32)
    hipLaunchKernelGGL((head_gate_kernel<float>), grid, block, 0, stream, (const float*)x, x_stride, x_head,
                       (const float*)gate, gate_stride, (float*)out, out_stride, H, dv);
  else
    hipLaunchKernelGGL((head_gate_kernel<bf16_t>), grid, block, 0, stream, (const bf16_t*)x, x_stride, x_head,
                       (const bf16_t*)gate, gate_stride, (bf16_t*)out, out_stride, H, dv);
  LMSF_LAUNCH_CHECK("head_gate");
  return 0;
}

// out = scale * (a / rms(a) * wa + b / rms(b) * wb), row by row: two mixers that read the same input are each
// normed over the model width and averaged. A workgroup a row; float32 arithmetic.
template <typename T>
__global__ __launch_bounds__(256) void rms_pair_kernel(const T* __restrict__ a, long a_stride, const T* __restrict__ b,
                                                       long b_stride, const float* __restrict__ wa,
                                                       const float* __restrict__ wb, T* __restrict__ out, int W,
                                                       float eps, float scale) {
  __shared__ float red[16];
  const long n = blockIdx.x;
  float sa = 0.f, sb = 0.f;
  for (int i = threadIdx.x; i < W; i += 256) {
    const float x = to_f32<T>(a[n * a_stride + i]), y = to_f32<T>(b[n * b_stride + i]);
    sa += x * x;
    sb += y * y;
  }
  sa = block_sum(sa, red);
  sb = block_sum(sb, red);
  const float ia = 1.f / sqrtf(sa / (float)W + eps), ib = 1.f / sqrtf(sb / (float)W + eps);
  for (int i = threadIdx.x; i < W; i += 256) {
    const float x = to_f32<T>(a[n * a_stride + i]), y = to_f32<T>(b[n * b_stride + i]);
    out[n * W + i] = from_f32<T>(scale * (x * ia * wa[i] + y * ib * wb[i]));
  }
}

extern "C" int lmsf_rms_pair(const void* a, long a_stride, const void* b, long b_stride, int dtype, const float* wa,
                             const float* wb, void* out, int n_rows, int W, float eps, float scale,
                             hipStream_t stream) {
  LMSF_CHECK(a && b && wa && wb && out, "rms_pair: null pointer");
  LMSF_CHECK(dtype == LMSF_F32 || dtype == LMSF_BF16, "rms_pair: unknown dtype code %d", dtype);
  LMSF_CHECK(W > 0 && a_stride >= W && b_stride >= W && n_rows >= 0, "rms_pair: bad sizes");
  if (n_rows == 0) return 0;
  if (dtype == LMSF_F32)
    hipLaunchKernelGGL((rms_pair_kernel<float>), dim3(n_rows), dim3(256), 0, stream, (const float*)a, a_stride,
                       (const float*)b, b_stride, wa, wb, (float*)out, W, eps, scale);
  else
    hipLaunchKernelGGL((rms_pair_kernel<bf16_t>), dim3(n_rows), dim3(256), 0, stream, (const bf16_t*)a, a_stride,
                       (const bf16_t*)b, b_stride, wa, wb, (bf16_t*)out, W, eps, scale);
  LMSF_LAUNCH_CHECK("rms_pair");
  return 0;
}
