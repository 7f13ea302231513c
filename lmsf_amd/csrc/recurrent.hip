// Mixers that carry a fixed-size state from token to token: a short causal convolution per channel, the
// selective scan, and a matrix memory with exponential gates. The reference has no recurrent mixer (its only one is
// attention over a paged cache, core/src/model_executor/layers/attention.rs:91-231).
//
// A step holds segments (a request's next tokens, one after the other in the flat batch); segment s begins at
// flat index seg_starts[s], ends before seg_starts[s + 1], and its request's state lies in row state_slots[s] of a
// float32 state tensor (``state`` points at this mixer's part of row 0, rows are ``state_stride`` floats apart).
// A row is all zeros when a request's first tokens run. A segment's tokens are walked in order by one workgroup
// per (segment, share of the channels or head), the state in registers; the operands of a tile of tokens are
// brought into LDS together, so that the walk waits for memory once a tile and not once a token. Sums over the
// state are taken in an order that does not depend on where a request was cut into steps: the results of a cut
// request equal those of the whole one to the bit. All arithmetic is float32.
#include "common.h"

#include <math.h>

__device__ __forceinline__ float rc_softplus(float z) { return z > 20.f ? z : log1pf(expf(z)); }
__device__ __forceinline__ float rc_sigmoid(float z) { return 1.f / (1.f + expf(-z)); }
__device__ __forceinline__ float rc_logsigmoid(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

// ---------------------------------------------------------------- short causal convolution
// out[t, c] = act(bias[c] + sum_j w[c, j] u[t - taps + 1 + j, c]); an input before the segment's first token is
// the request's earlier input, kept in the state as [C, taps - 1] (oldest first; zeros before the request began).
// ACT 0: none, 1: silu. The state is brought up to date by the second kernel, launched after the first.
template <typename T, int ACT>
__global__ __launch_bounds__(256) void short_conv_kernel(const T* __restrict__ u, long u_stride, const T* __restrict__ w,
                                                         const T* __restrict__ bias, const float* __restrict__ state,
                                                         long state_stride, const int* __restrict__ seg_of,
                                                         const int* __restrict__ seg_starts,
                                                         const int* __restrict__ state_slots, T* __restrict__ out,
                                                         long out_stride, int C, int taps) {
  const int t = blockIdx.x;
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= C) return;
  const int s = seg_of[t];
  const int start = seg_starts[s];
  const float* st = state + (long)state_slots[s] * state_stride + (long)c * (taps - 1);
  float acc = bias ? to_f32<T>(bias[c]) : 0.f;
  for (int j = 0; j < taps; ++j) {
    const int src = t - (taps - 1) + j;
    const float x = src >= start ? to_f32<T>(u[(long)src * u_stride + c]) : st[(taps - 1) + (src - start)];
    acc += to_f32<T>(w[(long)c * taps + j]) * x;
  }
  if (ACT == 1) acc = acc / (1.f + expf(-acc));
  out[(long)t * out_stride + c] = from_f32<T>(acc);
}

// state[c, h] <- the input taps - 1 - h tokens before the segment's end: of this step where the segment is long
// enough, else what the state held that many tokens further on (read before it is overwritten: h rises).
template <typename T>
__global__ __launch_bounds__(256) void short_conv_state_kernel(const T* __restrict__ u, long u_stride,
                                                               float* __restrict__ state, long state_stride,
                                                               const int* __restrict__ seg_starts,
                                                               const int* __restrict__ state_slots, int C, int taps) {
  const int s = blockIdx.x;
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= C) return;
  const int start = seg_starts[s], len = seg_starts[s + 1] - start;
  float* st = state + (long)state_slots[s] * state_stride + (long)c * (taps - 1);
  for (int h = 0; h < taps - 1; ++h) {
    const int idx = len - (taps - 1) + h;
    st[h] = idx >= 0 ? to_f32<T>(u[(long)(start + idx) * u_stride + c]) : st[(taps - 1) + idx];
  }
}

extern "C" int lmsf_short_conv(const void* u, int dtype, long u_stride, const void* w, const void* bias, int act,
                               float* state, long state_stride, const int* seg_of, const int* seg_starts,
                               const int* state_slots, void* out, long out_stride, int n_tokens, int n_segments, int C,
                               int taps, hipStream_t stream) {
  LMSF_CHECK(u && w && out && seg_of && seg_starts && state_slots, "short_conv: null pointer");
  LMSF_CHECK(dtype == LMSF_F32 || dtype == LMSF_BF16, "short_conv: unknown dtype code %d", dtype);
  LMSF_CHECK(C > 0 && taps >= 1 && taps <= 64, "short_conv: bad sizes C=%d taps=%d", C, taps);
  LMSF_CHECK(taps == 1 || state, "short_conv: a convolution over %d taps needs a state", taps);
  LMSF_CHECK(u_stride >= C && out_stride >= C && state_stride >= (long)C * (taps - 1), "short_conv: strides too small");
  LMSF_CHECK(act == 0 || act == 1, "short_conv: unknown activation %d", act);
  LMSF_CHECK(n_tokens >= 0 && n_segments >= 0 && n_segments <= n_tokens, "short_conv: bad counts");
  LMSF_CHECK((C + 255) / 256 <= 65535, "short_conv: too many channels");
  if (n_tokens == 0) return 0;
  dim3 grid(n_tokens, (C + 255) / 256), sgrid(n_segments, (C + 255) / 256), block(256);
#define SC(T, A)                                                                                                      \
  hipLaunchKernelGGL((short_conv_kernel<T, A>), grid, block, 0, stream, (const T*)u, u_stride, (const T*)w,           \
                     (const T*)bias, state, state_stride, seg_of, seg_starts, state_slots, (T*)out, out_stride, C, taps)
  if (dtype == LMSF_F32) {
    if (act) SC(float, 1); else SC(float, 0);
  } else {
    if (act) SC(bf16_t, 1); else SC(bf16_t, 0);
  }
#undef SC
  LMSF_LAUNCH_CHECK("short_conv");
  if (taps > 1) {
    if (dtype == LMSF_F32)
      hipLaunchKernelGGL((short_conv_state_kernel<float>), sgrid, block, 0, stream, (const float*)u, u_stride, state,
                         state_stride, seg_starts, state_slots, C, taps);
    else
      hipLaunchKernelGGL((short_conv_state_kernel<bf16_t>), sgrid, block, 0, stream, (const bf16_t*)u, u_stride, state,
                         state_stride, seg_starts, state_slots, C, taps);
    LMSF_LAUNCH_CHECK("short_conv_state");
  }
  return 0;
}

// ---------------------------------------------------------------- selective scan
// Per channel c and state entry n:  S[c, n] <- exp(dt_c A[c, n]) S[c, n] + dt_c x_c B_n;
// y_c = (sum_n S[c, n] C_n + D_c x_c) * silu(z_c), with dt = softplus(dt_pre) and A = -exp(A_log).
// A workgroup: 16 channels of one segment, 16 lanes a channel, a lane SPL state entries (n = lane + 16 k).
#define SCAN_CH 16

template <typename T, int SPL>
__global__ __launch_bounds__(256) void selective_scan_kernel(
    const T* __restrict__ x, long x_stride, const float* __restrict__ dt_pre, long dt_stride, const T* __restrict__ bc,
    long bc_stride, int b_at, int c_at, const T* __restrict__ z, long z_stride, const float* __restrict__ A_log,
    const float* __restrict__ Dw, float* __restrict__ state, long state_stride, const int* __restrict__ seg_starts,
    const int* __restrict__ state_slots, T* __restrict__ y, long y_stride, int inner, int nstate, int TT) {
  extern __shared__ float lds[];
  float* sx = lds;                      // [TT][16]
  float* sdt = sx + TT * SCAN_CH;       // [TT][16] after softplus
  float* sz = sdt + TT * SCAN_CH;       // [TT][16]
  float* sy = sz + TT * SCAN_CH;        // [TT][16]
  float* sB = sy + TT * SCAN_CH;        // [TT][nstate]
  float* sC = sB + TT * nstate;         // [TT][nstate]
  const int tid = threadIdx.x, ch = tid / 16, ln = tid % 16;
  const int c0 = blockIdx.x * SCAN_CH, c = c0 + ch;
  const int s = blockIdx.y;
  const int start = seg_starts[s], end = seg_starts[s + 1];
  const bool live = c < inner;
  float* st = state + (long)state_slots[s] * state_stride + (long)c * nstate;
  float a[SPL], S[SPL];
#pragma unroll
  for (int k = 0; k < SPL; ++k) {
    const int n = ln + 16 * k;
    const bool ok = live && n < nstate;
    a[k] = ok ? -expf(A_log[(long)c * nstate + n]) : 0.f;
    S[k] = ok ? st[n] : 0.f;
  }
  const float dw = live ? Dw[c] : 0.f;
  for (int t0 = start; t0 < end; t0 += TT) {
    const int nt = min(TT, end - t0);
    for (int i = tid; i < nt * SCAN_CH; i += 256) {
      const int tt = i / SCAN_CH, gc = c0 + i % SCAN_CH;
      const long t = t0 + tt;
      const bool ok = gc < inner;
      sx[i] = ok ? to_f32<T>(x[t * x_stride + gc]) : 0.f;
      sdt[i] = ok ? rc_softplus(dt_pre[t * dt_stride + gc]) : 0.f;
      sz[i] = ok ? to_f32<T>(z[t * z_stride + gc]) : 0.f;
    }
    for (int i = tid; i < nt * nstate; i += 256) {
      const int tt = i / nstate, n = i % nstate;
      const long t = t0 + tt;
      sB[i] = to_f32<T>(bc[t * bc_stride + b_at + n]);
      sC[i] = to_f32<T>(bc[t * bc_stride + c_at + n]);
    }
    __syncthreads();
    for (int tt = 0; tt < nt; ++tt) {
      const float dtv = sdt[tt * SCAN_CH + ch], xv = sx[tt * SCAN_CH + ch];
      const float dx = dtv * xv;
      float acc = 0.f;
#pragma unroll
      for (int k = 0; k < SPL; ++k) {
        const int n = ln + 16 * k;
        if (n < nstate) {
          S[k] = expf(dtv * a[k]) * S[k] + dx * sB[tt * nstate + n];
          acc += S[k] * sC[tt * nstate + n];
        }
      }
      acc += __shfl_xor(acc, 8, LMSF_WAVE);
      acc += __shfl_xor(acc, 4, LMSF_WAVE);
      acc += __shfl_xor(acc, 2, LMSF_WAVE);
      acc += __shfl_xor(acc, 1, LMSF_WAVE);
      if (ln == 0) {
        const float zv = sz[tt * SCAN_CH + ch];
        sy[tt * SCAN_CH + ch] = (acc + dw * xv) * (zv / (1.f + expf(-zv)));
      }
    }
    __syncthreads();
    for (int i = tid; i < nt * SCAN_CH; i += 256) {
      const int tt = i / SCAN_CH, gc = c0 + i % SCAN_CH;
      if (gc < inner) y[(long)(t0 + tt) * y_stride + gc] = from_f32<T>(sy[i]);
    }
  }
  if (live) {
#pragma unroll
    for (int k = 0; k < SPL; ++k) {
      const int n = ln + 16 * k;
      if (n < nstate) st[n] = S[k];
    }
  }
}

extern "C" int lmsf_selective_scan(const void* x, int dtype, long x_stride, const float* dt_pre, long dt_stride,
                                   const void* bc, long bc_stride, int b_at, int c_at, const void* z, long z_stride,
                                   const float* A_log, const float* Dw, float* state, long state_stride,
                                   const int* seg_starts, const int* state_slots, void* y, long y_stride, int n_tokens,
                                   int n_segments, int inner, int nstate, hipStream_t stream) {
  LMSF_CHECK(x && dt_pre && bc && z && A_log && Dw && state && seg_starts && state_slots && y,
             "selective_scan: null pointer");
  LMSF_CHECK(dtype == LMSF_F32 || dtype == LMSF_BF16, "selective_scan: unknown dtype code %d", dtype);
  LMSF_CHECK(inner > 0 && nstate > 0 && nstate <= 256, "selective_scan: bad sizes inner=%d state=%d (state <= 256)", inner,
             nstate);
  LMSF_CHECK(x_stride >= inner && dt_stride >= inner && z_stride >= inner && y_stride >= inner &&
                 bc_stride >= b_at + nstate && bc_stride >= c_at + nstate && b_at >= 0 && c_at >= 0 &&
                 state_stride >= (long)inner * nstate,
             "selective_scan: strides too small");
  LMSF_CHECK(n_tokens >= 0 && n_segments >= 0 && n_segments <= 65535, "selective_scan: bad counts");
  if (n_tokens == 0 || n_segments == 0) return 0;
  const int TT = nstate <= 64 ? 32 : nstate <= 128 ? 16 : 8;
  const size_t smem = (size_t)TT * (4 * SCAN_CH + 2 * nstate) * sizeof(float);
  dim3 grid((inner + SCAN_CH - 1) / SCAN_CH, n_segments), block(256);
#define SCAN(T, SPL)                                                                                                   \
  hipLaunchKernelGGL((selective_scan_kernel<T, SPL>), grid, block, smem, stream, (const T*)x, x_stride, dt_pre,        \
                     dt_stride, (const T*)bc, bc_stride, b_at, c_at, (const T*)z, z_stride, A_log, Dw, state,          \
                     state_stride, seg_starts, state_slots, (T*)y, y_stride, inner, nstate, TT)
#define SCAN_T(T)                        \
  do {                                   \
    if (nstate <= 16) SCAN(T, 1);        \
    else if (nstate <= 32) SCAN(T, 2);   \
    else if (nstate <= 64) SCAN(T, 4);   \
    else if (nstate <= 128) SCAN(T, 8);  \
    else SCAN(T, 16);                    \
  } while (0)
  if (dtype == LMSF_F32) SCAN_T(float); else SCAN_T(bf16_t);
#undef SCAN_T
#undef SCAN
  LMSF_LAUNCH_CHECK("selective_scan");
  return 0;
}

// ---------------------------------------------------------------- matrix memory with exponential gates
// Per head, with log gates i = cap tanh(ipre / cap), f = logsigmoid(cap tanh(fpre / cap)) and a running maximum m
// (0 before the first token):
//   m' = max(f + m, i);  S <- exp(f + m - m') S + exp(i - m') k v^T;  n likewise with k alone;
//   o = S^T q / (max(|n . q|, exp(-m')) + 1e-6),  q times qscale;
//   out = o / rms(o) * w * sigmoid(g)      (rms over the head's dv entries, eps inside the root)
// n is kept as one more column of S (a value entry that is always 1), so that n . q comes out of the same sums as
// S^T q. The state of a slot: S and n as [H, d, dv + 1], then m as [H].
// A workgroup: one head of one segment; thread (rg, vv) owns column vv of the rows rg, rg + RG, ... (RPT of them).
template <typename T, int RPT>
__global__ __launch_bounds__(256) void mlstm_kernel(
    const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v, long qkv_stride,
    const float* __restrict__ gates, long gates_stride, const T* __restrict__ og, long og_stride,
    const float* __restrict__ norm_w, float* __restrict__ state, long state_stride, const int* __restrict__ seg_starts,
    const int* __restrict__ state_slots, T* __restrict__ out, long out_stride, int H, int d, int dv, int VB,
    float qscale, float cap, float eps, int TT) {
  extern __shared__ float lds[];
  const int RG = 256 / VB, dpad = RPT * RG, cols = dv + 1;
  float* sq = lds;                   // [TT][dpad], zeros behind d
  float* sk = sq + TT * dpad;        // [TT][dpad]
  float* sv = sk + TT * dpad;        // [TT][VB]: v, then 1, then zeros
  float* sg = sv + TT * VB;          // [TT][2]: i, f
  float* so = sg + TT * 2;           // [TT][dv]
  float* red = so + TT * dv;         // [RG][VB]
  float* oext = red + RG * VB;       // [VB]
  const int tid = threadIdx.x, vv = tid % VB, rg = tid / VB;
  const int h = blockIdx.x, s = blockIdx.y;
  const int start = seg_starts[s], end = seg_starts[s + 1];
  float* st = state + (long)state_slots[s] * state_stride;
  float* sS = st + (long)h * d * cols;
  float* sm = st + (long)H * d * cols + h;
  float S[RPT];
#pragma unroll
  for (int r = 0; r < RPT; ++r) {
    const int dd = rg + r * RG;
    S[r] = (dd < d && vv < cols) ? sS[(long)dd * cols + vv] : 0.f;
  }
  float m = sm[0];
  for (int t0 = start; t0 < end; t0 += TT) {
    const int nt = min(TT, end - t0);
    for (int i = tid; i < nt * dpad; i += 256) {
      const int tt = i / dpad, dd = i % dpad;
      const long t = t0 + tt;
      sq[i] = dd < d ? to_f32<T>(q[t * qkv_stride + h * d + dd]) * qscale : 0.f;
      sk[i] = dd < d ? to_f32<T>(k[t * qkv_stride + h * d + dd]) : 0.f;
    }
    for (int i = tid; i < nt * VB; i += 256) {
      const int tt = i / VB, e = i % VB;
      sv[i] = e < dv ? to_f32<T>(v[(long)(t0 + tt) * qkv_stride + h * dv + e]) : e == dv ? 1.f : 0.f;
    }
    for (int tt = tid; tt < nt; tt += 256) {
      const float ip = gates[(long)(t0 + tt) * gates_stride + h], fp = gates[(long)(t0 + tt) * gates_stride + H + h];
      sg[tt * 2] = cap * tanhf(ip / cap);
      sg[tt * 2 + 1] = rc_logsigmoid(cap * tanhf(fp / cap));
    }
    __syncthreads();
    for (int tt = 0; tt < nt; ++tt) {
      const float gi = sg[tt * 2], gf = sg[tt * 2 + 1];
      const float m_new = fmaxf(gf + m, gi);
      const float keep = expf(gf + m - m_new), take = expf(gi - m_new);
      m = m_new;
      const float tv = take * sv[tt * VB + vv];
      float acc = 0.f;
#pragma unroll
      for (int r = 0; r < RPT; ++r) {
        const int dd = rg + r * RG;
        S[r] = keep * S[r] + sk[tt * dpad + dd] * tv;
        acc += S[r] * sq[tt * dpad + dd];
      }
      if (RG > 1) {
        red[rg * VB + vv] = acc;
        __syncthreads();
        if (rg == 0) {
          float total = 0.f;
          for (int g = 0; g < RG; ++g) total += red[g * VB + vv];
          oext[vv] = total;
        }
      } else {
        oext[vv] = acc;
      }
      __syncthreads();
      if (tid < dv) so[tt * dv + tid] = oext[tid] / (fmaxf(fabsf(oext[dv]), expf(-m)) + 1e-6f);
      __syncthreads();
    }
    // the heads' norm, the weight and the output gate, a wave a token
    for (int tt = tid / LMSF_WAVE; tt < nt; tt += 256 / LMSF_WAVE) {
      const int lane = tid % LMSF_WAVE;
      float ss = 0.f;
      for (int e = lane; e < dv; e += LMSF_WAVE) ss += so[tt * dv + e] * so[tt * dv + e];
      ss = wave_sum(ss);
      const float inv = 1.f / sqrtf(ss / (float)dv + eps);
      const long t = t0 + tt;
      for (int e = lane; e < dv; e += LMSF_WAVE) {
        const float g = to_f32<T>(og[t * og_stride + h * dv + e]);
        out[t * out_stride + h * dv + e] = from_f32<T>(so[tt * dv + e] * inv * norm_w[h * dv + e] * rc_sigmoid(g));
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int r = 0; r < RPT; ++r) {
    const int dd = rg + r * RG;
    if (dd < d && vv < cols) sS[(long)dd * cols + vv] = S[r];
  }
  if (tid == 0) sm[0] = m;
}

// floats of state a slot needs: S and n as [H, d, dv + 1], m as [H]
extern "C" long lmsf_mlstm_state_floats(int H, int d, int dv) { return (long)H * d * (dv + 1) + H; }

extern "C" int lmsf_mlstm(const void* q, const void* k, const void* v, int dtype, long qkv_stride, const float* gates,
                          long gates_stride, const void* og, long og_stride, const float* norm_w, float* state,
                          long state_stride, const int* seg_starts, const int* state_slots, void* out, long out_stride,
                          int n_tokens, int n_segments, int H, int d, int dv, float qscale, float cap, float eps,
                          hipStream_t stream) {
  LMSF_CHECK(q && k && v && gates && og && norm_w && state && seg_starts && state_slots && out, "mlstm: null pointer");
  LMSF_CHECK(dtype == LMSF_F32 || dtype == LMSF_BF16, "mlstm: unknown dtype code %d", dtype);
  LMSF_CHECK(H > 0 && H <= 65535 && d > 0 && dv > 0 && dv <= 255, "mlstm: bad sizes H=%d d=%d dv=%d (dv <= 255)", H, d, dv);
  LMSF_CHECK(cap > 0.f, "mlstm: the gates' cap must be > 0");
  LMSF_CHECK(gates_stride >= 2 * H && og_stride >= (long)H * dv && out_stride >= (long)H * dv &&
                 state_stride >= lmsf_mlstm_state_floats(H, d, dv),
             "mlstm: strides too small");
  LMSF_CHECK(n_tokens >= 0 && n_segments >= 0 && n_segments <= 65535, "mlstm: bad counts");
  if (n_tokens == 0 || n_segments == 0) return 0;
  int VB = 16;
  while (VB < dv + 1) VB *= 2;
  const int RG = 256 / VB;
  const int rows = (d + RG - 1) / RG;
  LMSF_CHECK(rows <= 128, "mlstm: a head of %d x %d does not fit a workgroup's registers", d, dv);
  const int RPT = rows <= 4 ? 4 : rows <= 8 ? 8 : rows <= 16 ? 16 : rows <= 32 ? 32 : rows <= 64 ? 64 : 128;
  const int dpad = RPT * RG;
  int TT = 16;
  size_t smem = 0;
  for (;; TT /= 2) {
    smem = ((size_t)TT * (2 * dpad + VB + 2 + dv) + (size_t)RG * VB + VB) * sizeof(float);
    if (smem <= 60 * 1024 || TT == 1) break;
  }
  LMSF_CHECK(smem <= 64 * 1024, "mlstm: a head of %d x %d needs %zu bytes of LDS", d, dv, smem);
  dim3 grid(H, n_segments), block(256);
#define ML(T, R)                                                                                                       \
  hipLaunchKernelGGL((mlstm_kernel<T, R>), grid, block, smem, stream, (const T*)q, (const T*)k, (const T*)v,           \
                     qkv_stride, gates, gates_stride, (const T*)og, og_stride, norm_w, state, state_stride, seg_starts, \
                     state_slots, (T*)out, out_stride, H, d, dv, VB, qscale, cap, eps, TT)
#define ML_T(T)                          \
  do {                                   \
    if (RPT == 4) ML(T, 4);              \
    else if (RPT == 8) ML(T, 8);         \
    else if (RPT == 16) ML(T, 16);       \
    else if (RPT == 32) ML(T, 32);       \
    else if (RPT == 64) ML(T, 64);       \
    else ML(T, 128);                     \
  } while (0)
  if (dtype == LMSF_F32) ML_T(float); else ML_T(bf16_t);
#undef ML_T
#undef ML
  LMSF_LAUNCH_CHECK("mlstm");
  return 0;
}
