// Mixers that carry a fixed-size state from token to token: a short causal convolution per channel, the
// selective scan, and a matrix memory with exponential gates. The reference has no recurrent mixer (its only one is
// attention over a paged cache, core/src/model_executor/layers/attention.rs:91-231).
//
// A step holds segments (a request's next tokens, one after the other in the flat batch); segment s begins at
// flat index seg_starts[s], ends before seg_starts[s + 1], and its request's state lies in row state_slots[s] of a
// float32 state tensor (``state`` points at this mixer's part of row 0, rows are ``state_stride`` floats apart).
// A row is all zeros when a request's first tokens run. A segment's tokens are walked in order by one workgroup
// per (segment, share of the channels or head), the state in registers; the operands of a tile of tokens are
// brought into LDS together, so that the walk waits for memory once a tile and not once a token. Long segments
// (portions of prompts) take forms that work on chunks of tokens at once; they and the token-by-token forms agree up
// to rounding. All arithmetic is float32.
#include "common.h"
#include "entry_points.h"

#include <math.h>

__device__ __forceinline__ float rc_softplus(float z) { return z > 20.f ? z : log1pf(expf(z)); }
__device__ __forceinline__ float rc_sigmoid(float z) { return 1.f / (1.f + expf(-z)); }
// exp of a decay's exponent, in the recurrences' inner loops: one multiplication and the hardware's 2^x (relative error
// about |x| 2^-24 beside the instruction's own last bit; an exponent that large forgets within a token)
__device__ __forceinline__ float rc_decay(float x) { return __expf(x); }
__device__ __forceinline__ float rc_logsigmoid(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

// ---------------------------------------------------------------- short causal convolution
// out[t, c] = act(bias[c] + sum_j w[c, j] u[t - taps + 1 + j, c]); an input before the segment's first token is
// the request's earlier input, kept in the state as [C, taps - 1] (oldest first; zeros before the request began).
// ACT 0: none, 1: silu. The state is brought up to date by the second kernel, launched after the first; in a step of
// single tokens (``single``) the thread of a (token, channel) is the only one that reads that channel's state, and
// moves it on itself.
template <typename T, int ACT>
__global__ __launch_bounds__(256) void short_conv_kernel(const T* __restrict__ u, long u_stride, const T* __restrict__ w,
                                                         const T* __restrict__ bias, float* __restrict__ state,
                                                         long state_stride, const int* __restrict__ seg_of,
                                                         const int* __restrict__ seg_starts,
                                                         const int* __restrict__ state_slots, T* __restrict__ out,
                                                         long out_stride, int C, int taps, int single) {
  const int t = blockIdx.x;
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= C) return;
  const int s = seg_of[t];
  const int start = seg_starts[s];
  float* st = state + (long)state_slots[s] * state_stride + (long)c * (taps - 1);
  float acc = bias ? to_f32<T>(bias[c]) : 0.f;
  for (int j = 0; j < taps; ++j) {
    const int src = t - (taps - 1) + j;
    const float x = src >= start ? to_f32<T>(u[(long)src * u_stride + c]) : st[(taps - 1) + (src - start)];
    acc += to_f32<T>(w[(long)c * taps + j]) * x;
    if (single && j > 0) st[j - 1] = x;          // (read above at j, written at j - 1: the state moves on by one token)
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
                               int taps, int single, hipStream_t stream) {
  LMSF_CHECK(u && w && out && seg_of && seg_starts && state_slots, "short_conv: null pointer");
  LMSF_CHECK(dtype == LMSF_F32 || dtype == LMSF_BF16, "short_conv: unknown dtype code %d", dtype);
  LMSF_CHECK(C > 0 && taps >= 1 && taps <= 64, "short_conv: bad sizes C=%d taps=%d", C, taps);
  LMSF_CHECK(taps == 1 || state, "short_conv: a convolution over %d taps needs a state", taps);
  LMSF_CHECK(u_stride >= C && out_stride >= C && state_stride >= (long)C * (taps - 1), "short_conv: strides too small");
  LMSF_CHECK(act == 0 || act == 1, "short_conv: unknown activation %d", act);
  LMSF_CHECK(n_tokens >= 0 && n_segments >= 0 && n_segments <= n_tokens, "short_conv: bad counts");
  LMSF_CHECK(!single || n_segments == n_tokens, "short_conv: a step of single tokens has as many segments as tokens");
  LMSF_CHECK((C + 255) / 256 <= 65535, "short_conv: too many channels");
  if (n_tokens == 0) return 0;
  dim3 grid(n_tokens, (C + 255) / 256), sgrid(n_segments, (C + 255) / 256), block(256);
  // (a form with 16-byte accesses, a thread 8 neighbouring channels of a token, measured slower at 2,048 tokens of 4,096
  // channels, 74 against 60 us, and at 8 tokens, 10.7 against 3.8: its weights' loads lie 64 bytes apart across a wave)
#define SC(T, A)                                                                                                      \
  hipLaunchKernelGGL((short_conv_kernel<T, A>), grid, block, 0, stream, (const T*)u, u_stride, (const T*)w,           \
                     (const T*)bias, state, state_stride, seg_of, seg_starts, state_slots, (T*)out, out_stride, C, taps, \
                     single)
  if (dtype == LMSF_F32) {
    if (act) SC(float, 1); else SC(float, 0);
  } else {
    if (act) SC(bf16_t, 1); else SC(bf16_t, 0);
  }
#undef SC
  LMSF_LAUNCH_CHECK("short_conv");
  if (taps > 1 && !single) {
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
// A workgroup: 16 channels of one chunk of a segment's tokens, 16 lanes a channel, a lane SPL state entries
// (n = lane + 16 k). A segment of up to ``chunk`` tokens is one chunk: its workgroups read the slot's state, walk the
// tokens and write the state back. A longer segment (a prompt's portion) is cut into chunks that run side by side,
// in two launches, because the recurrence is linear in S: over a chunk, S_end = exp(A sum dt) S_begin + L with L the
// end state that the chunk reaches from zero. The first launch (SUMMARY) leaves every chunk's L and sum of dt in
// ``scratch`` (and a copy of the slot's state as the entry before the first chunk); a small kernel folds them into
// every chunk's S_begin; in the last launch every chunk walks its tokens from there and writes y, and the last chunk
// writes the slot's state.
// scratch_base[s] is segment s's first entry of scratch (entries of inner * (nstate + 1) floats: L, then the sums),
// or negative for a segment that is one chunk; null: every segment is one chunk.
#define SCAN_CH 16

template <typename T, int SPL, bool SUMMARY>
__global__ __launch_bounds__(256) void selective_scan_kernel(
    const T* __restrict__ x, long x_stride, const float* __restrict__ dt_pre, long dt_stride, const T* __restrict__ bc,
    long bc_stride, int b_at, int c_at, const T* __restrict__ z, long z_stride, const float* __restrict__ A_log,
    const float* __restrict__ Dw, float* __restrict__ state, long state_stride, const int* __restrict__ seg_starts,
    const int* __restrict__ state_slots, T* __restrict__ y, long y_stride, int inner, int nstate, int TT, int chunk,
    const int* __restrict__ scratch_base, float* __restrict__ scratch) {
  extern __shared__ float lds[];
  float* sx = lds;                      // [TT][16]
  float* sdt = sx + TT * SCAN_CH;       // [TT][16] after softplus
  float* sz = sdt + TT * SCAN_CH;       // [TT][16]
  float* sy = sz + TT * SCAN_CH;        // [TT][16]
  float* sB = sy + TT * SCAN_CH;        // [TT][nstate]
  float* sC = sB + TT * nstate;         // [TT][nstate]
  const int tid = threadIdx.x, ch = tid / 16, ln = tid % 16;
  const int c0 = blockIdx.x * SCAN_CH, c = c0 + ch;
  const int s = blockIdx.z, j = blockIdx.y;
  const int seg_start = seg_starts[s], seg_end = seg_starts[s + 1];
  const int base = scratch_base ? scratch_base[s] : -1;
  if (SUMMARY && base < 0) return;
  const int n_chunks = base < 0 ? 1 : (seg_end - seg_start + chunk - 1) / chunk;
  if (j >= n_chunks) return;
  const int start = base < 0 ? seg_start : seg_start + j * chunk;
  const int end = base < 0 ? seg_end : min(seg_end, start + chunk);
  const bool live = c < inner;
  const long entry = (long)inner * (nstate + 1);
  float* st = state + (long)state_slots[s] * state_stride + (long)c * nstate;
  float a[SPL], S[SPL];
#pragma unroll
  for (int k = 0; k < SPL; ++k) {
    const int n = ln + 16 * k;
    const bool ok = live && n < nstate;
    a[k] = ok ? -expf(A_log[(long)c * nstate + n]) : 0.f;
    S[k] = 0.f;
    if (ok) {
      if (base < 0) {
        S[k] = st[n];
      } else if (SUMMARY) {
        if (j == 0) scratch[(long)base * entry + (long)c * nstate + n] = st[n];       // the entry before the first chunk
      } else {
        S[k] = scratch[(long)(base + j) * entry + (long)c * nstate + n];     // folded by selective_scan_fold_kernel
      }
    }
  }
  if (SUMMARY && j == n_chunks - 1) return;           // nobody folds the last chunk's summary
  const float dw = live ? Dw[c] : 0.f;
  float sum_dt = 0.f;
  for (int t0 = start; t0 < end; t0 += TT) {
    const int nt = min(TT, end - t0);
    __syncthreads();
    for (int i = tid; i < nt * SCAN_CH; i += 256) {
      const int tt = i / SCAN_CH, gc = c0 + i % SCAN_CH;
      const long t = t0 + tt;
      const bool ok = gc < inner;
      sx[i] = ok ? to_f32<T>(x[t * x_stride + gc]) : 0.f;
      sdt[i] = ok ? rc_softplus(dt_pre[t * dt_stride + gc]) : 0.f;
      if (!SUMMARY) sz[i] = ok ? to_f32<T>(z[t * z_stride + gc]) : 0.f;
    }
    for (int i = tid; i < nt * nstate; i += 256) {
      const int tt = i / nstate, n = i % nstate;
      const long t = t0 + tt;
      sB[i] = to_f32<T>(bc[t * bc_stride + b_at + n]);
      if (!SUMMARY) sC[i] = to_f32<T>(bc[t * bc_stride + c_at + n]);
    }
    __syncthreads();
    for (int tt = 0; tt < nt; ++tt) {
      const float dtv = sdt[tt * SCAN_CH + ch], xv = sx[tt * SCAN_CH + ch];
      const float dx = dtv * xv;
      sum_dt += dtv;
      float acc = 0.f;
#pragma unroll
      for (int k = 0; k < SPL; ++k) {
        const int n = ln + 16 * k;
        if (n < nstate) {
          S[k] = rc_decay(dtv * a[k]) * S[k] + dx * sB[tt * nstate + n];
          if (!SUMMARY) acc += S[k] * sC[tt * nstate + n];
        }
      }
      if (!SUMMARY) {
        acc += __shfl_xor(acc, 8, LMSF_WAVE);
        acc += __shfl_xor(acc, 4, LMSF_WAVE);
        acc += __shfl_xor(acc, 2, LMSF_WAVE);
        acc += __shfl_xor(acc, 1, LMSF_WAVE);
        if (ln == 0) {
          const float zv = sz[tt * SCAN_CH + ch];
          sy[tt * SCAN_CH + ch] = (acc + dw * xv) * (zv / (1.f + expf(-zv)));
        }
      }
    }
    if (!SUMMARY) {
      __syncthreads();
      for (int i = tid; i < nt * SCAN_CH; i += 256) {
        const int tt = i / SCAN_CH, gc = c0 + i % SCAN_CH;
        if (gc < inner) y[(long)(t0 + tt) * y_stride + gc] = from_f32<T>(sy[i]);
      }
    }
  }
  if (!live) return;
  if (SUMMARY) {
    float* ent = scratch + (long)(base + j + 1) * entry;
#pragma unroll
    for (int k = 0; k < SPL; ++k) {
      const int n = ln + 16 * k;
      if (n < nstate) ent[(long)c * nstate + n] = S[k];
    }
    if (ln == 0) ent[(long)inner * nstate + c] = sum_dt;
  } else if (j == n_chunks - 1) {
#pragma unroll
    for (int k = 0; k < SPL; ++k) {
      const int n = ln + 16 * k;
      if (n < nstate) st[n] = S[k];
    }
  }
}

// Between the two launches of the chunked form: entry 0 of a segment holds the slot's state, entry e > 0 chunk e - 1's
// end state from zero (L) and its sums of dt. Afterwards entry e holds the state at the beginning of chunk e:
// S_(e) = exp(A sum_dt_(e-1)) S_(e-1) + L_(e-1). A thread a (channel, state entry); the chunks one after the other.
__global__ __launch_bounds__(256) void selective_scan_fold_kernel(const float* __restrict__ A_log,
                                                                  const int* __restrict__ seg_starts,
                                                                  const int* __restrict__ scratch_base,
                                                                  float* __restrict__ scratch, int inner, int nstate,
                                                                  int chunk) {
  const int s = blockIdx.y;
  const int base = scratch_base[s];
  if (base < 0) return;
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= (long)inner * nstate) return;
  const int c = i / nstate;
  const int n_chunks = (seg_starts[s + 1] - seg_starts[s] + chunk - 1) / chunk;
  const long entry = (long)inner * (nstate + 1);
  const float a = -expf(A_log[i]);
  float S = scratch[(long)base * entry + i];
  for (int e = 1; e < n_chunks; ++e) {
    float* ent = scratch + (long)(base + e) * entry;
    S = expf(a * ent[(long)inner * nstate + c]) * S + ent[i];
    ent[i] = S;
  }
}

// The same for states of up to 32 entries: a lane a channel, its whole state in registers, so that nothing crosses
// lanes and every instruction works on 64 channels. B and C of a tile of 8 tokens go through LDS (every lane reads the
// same entry); x, dt and z of the tile are asked for from memory together, a lane its own channel's.
#define SCANL_TT 8

template <typename T, int NS, bool SUMMARY>
__global__ __launch_bounds__(256) void selective_scan_lane_kernel(
    const T* __restrict__ x, long x_stride, const float* __restrict__ dt_pre, long dt_stride, const T* __restrict__ bc,
    long bc_stride, int b_at, int c_at, const T* __restrict__ z, long z_stride, const float* __restrict__ A_log,
    const float* __restrict__ Dw, float* __restrict__ state, long state_stride, const int* __restrict__ seg_starts,
    const int* __restrict__ state_slots, T* __restrict__ y, long y_stride, int inner, int nstate, int chunk,
    const int* __restrict__ scratch_base, float* __restrict__ scratch) {
  __shared__ float sB[SCANL_TT * NS], sC[SCANL_TT * NS];
  const int tid = threadIdx.x;
  const int c = blockIdx.x * 256 + tid;
  const int s = blockIdx.z, j = blockIdx.y;
  const int seg_start = seg_starts[s], seg_end = seg_starts[s + 1];
  const int base = scratch_base ? scratch_base[s] : -1;
  if (SUMMARY && base < 0) return;
  const int n_chunks = base < 0 ? 1 : (seg_end - seg_start + chunk - 1) / chunk;
  if (j >= n_chunks) return;
  if (SUMMARY && j == n_chunks - 1 && j > 0) return;          // nobody folds the last chunk's summary
  const int start = base < 0 ? seg_start : seg_start + j * chunk;
  const int end = base < 0 ? seg_end : min(seg_end, start + chunk);
  const bool live = c < inner;
  const int cc = live ? c : 0;                                 // (a lane beyond the channels computes on channel 0's and stores nothing)
  const long entry = (long)inner * (nstate + 1);
  float* st = state + (long)state_slots[s] * state_stride + (long)cc * nstate;
  float a[NS], S[NS];
#pragma unroll
  for (int n = 0; n < NS; ++n) {
    const bool ok = n < nstate;
    a[n] = ok ? -expf(A_log[(long)cc * nstate + n]) : 0.f;
    S[n] = 0.f;
    if (ok) {
      if (base < 0) {
        S[n] = st[n];
      } else if (SUMMARY) {
        if (j == 0 && live) scratch[(long)base * entry + (long)c * nstate + n] = st[n];     // the entry before the first chunk
      } else {
        S[n] = scratch[(long)(base + j) * entry + (long)cc * nstate + n];    // folded by selective_scan_fold_kernel
      }
    }
  }
  if (SUMMARY && j == n_chunks - 1) return;
  const float dw = Dw[cc];
  float sum_dt = 0.f;
  for (int t0 = start; t0 < end; t0 += SCANL_TT) {
    const int nt = min(SCANL_TT, end - t0);
    float rx[SCANL_TT], rdt[SCANL_TT], rz[SCANL_TT];
#pragma unroll
    for (int tt = 0; tt < SCANL_TT; ++tt) {
      const long t = t0 + (tt < nt ? tt : 0);
      rx[tt] = to_f32<T>(x[t * x_stride + cc]);
      rdt[tt] = dt_pre[t * dt_stride + cc];
      rz[tt] = SUMMARY ? 0.f : to_f32<T>(z[t * z_stride + cc]);
    }
    __syncthreads();
    for (int i = tid; i < nt * NS; i += 256) {
      const int tt = i / NS, n = i % NS;
      const long t = t0 + tt;
      sB[i] = n < nstate ? to_f32<T>(bc[t * bc_stride + b_at + n]) : 0.f;
      if (!SUMMARY) sC[i] = n < nstate ? to_f32<T>(bc[t * bc_stride + c_at + n]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int tt = 0; tt < SCANL_TT; ++tt) {
      if (tt < nt) {
        const float dtv = rc_softplus(rdt[tt]), xv = rx[tt];
        const float dx = dtv * xv;
        sum_dt += dtv;
        float acc = 0.f;
#pragma unroll
        for (int n = 0; n < NS; ++n) {
          S[n] = rc_decay(dtv * a[n]) * S[n] + dx * sB[tt * NS + n];
          if (!SUMMARY) acc += S[n] * sC[tt * NS + n];
        }
        if (!SUMMARY && live) {
          const float zv = rz[tt];
          y[(long)(t0 + tt) * y_stride + c] = from_f32<T>((acc + dw * xv) * (zv / (1.f + expf(-zv))));
        }
      }
    }
  }
  if (!live) return;
  if (SUMMARY) {
    float* ent = scratch + (long)(base + j + 1) * entry;
#pragma unroll
    for (int n = 0; n < NS; ++n)
      if (n < nstate) ent[(long)c * nstate + n] = S[n];
    ent[(long)inner * nstate + c] = sum_dt;
  } else if (j == n_chunks - 1) {
#pragma unroll
    for (int n = 0; n < NS; ++n)
      if (n < nstate) st[n] = S[n];
  }
}

// floats of scratch an entry of the chunked form takes (a chunk's end state from zero and its sums of dt)
extern "C" long lmsf_selective_scan_entry_floats(int inner, int nstate) { return (long)inner * (nstate + 1); }

// ``chunk`` > 0 with ``scratch_base`` and ``scratch``: segments with a non-negative base are cut into chunks of that
// many tokens (``max_chunks``: the most chunks any of them has); otherwise every segment is walked by one workgroup
// per 16 channels.
extern "C" int lmsf_selective_scan(const void* x, int dtype, long x_stride, const float* dt_pre, long dt_stride,
                                   const void* bc, long bc_stride, int b_at, int c_at, const void* z, long z_stride,
                                   const float* A_log, const float* Dw, float* state, long state_stride,
                                   const int* seg_starts, const int* state_slots, void* y, long y_stride, int n_tokens,
                                   int n_segments, int inner, int nstate, int chunk, int max_chunks,
                                   const int* scratch_base, float* scratch, hipStream_t stream) {
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
  const bool chunked = scratch_base != nullptr;
  LMSF_CHECK(!chunked || (scratch && chunk > 0 && max_chunks >= 1 && max_chunks <= 65535),
             "selective_scan: the chunked form needs scratch, a chunk size and the number of chunks");
  if (n_tokens == 0 || n_segments == 0) return 0;
  if (nstate <= 32) {
    dim3 lgrid((inner + 255) / 256, chunked ? max_chunks : 1, n_segments), lblock(256);
#define SCANL(T, NS, SUM)                                                                                              \
  hipLaunchKernelGGL((selective_scan_lane_kernel<T, NS, SUM>), lgrid, lblock, 0, stream, (const T*)x, x_stride, dt_pre, \
                     dt_stride, (const T*)bc, bc_stride, b_at, c_at, (const T*)z, z_stride, A_log, Dw, state,          \
                     state_stride, seg_starts, state_slots, (T*)y, y_stride, inner, nstate, chunk, scratch_base, scratch)
#define SCANL_T(T, SUM)                      \
  do {                                       \
    if (nstate <= 4) SCANL(T, 4, SUM);       \
    else if (nstate <= 8) SCANL(T, 8, SUM);  \
    else if (nstate <= 16) SCANL(T, 16, SUM); \
    else SCANL(T, 32, SUM);                  \
  } while (0)
    if (chunked) {
      if (dtype == LMSF_F32) SCANL_T(float, true); else SCANL_T(bf16_t, true);
      LMSF_LAUNCH_CHECK("selective_scan (chunk summaries)");
      hipLaunchKernelGGL(selective_scan_fold_kernel, dim3((unsigned)(((long)inner * nstate + 255) / 256), n_segments),
                         dim3(256), 0, stream, A_log, seg_starts, scratch_base, scratch, inner, nstate, chunk);
      LMSF_LAUNCH_CHECK("selective_scan (fold)");
    }
    if (dtype == LMSF_F32) SCANL_T(float, false); else SCANL_T(bf16_t, false);
#undef SCANL_T
#undef SCANL
    LMSF_LAUNCH_CHECK("selective_scan");
    return 0;
  }
  const int TT = nstate <= 64 ? 32 : nstate <= 128 ? 16 : 8;
  const size_t smem = (size_t)TT * (4 * SCAN_CH + 2 * nstate) * sizeof(float);
  dim3 grid((inner + SCAN_CH - 1) / SCAN_CH, chunked ? max_chunks : 1, n_segments), block(256);
#define SCAN(T, SPL, SUM)                                                                                              \
  hipLaunchKernelGGL((selective_scan_kernel<T, SPL, SUM>), grid, block, smem, stream, (const T*)x, x_stride, dt_pre,   \
                     dt_stride, (const T*)bc, bc_stride, b_at, c_at, (const T*)z, z_stride, A_log, Dw, state,          \
                     state_stride, seg_starts, state_slots, (T*)y, y_stride, inner, nstate, TT, chunk, scratch_base,   \
                     scratch)
#define SCAN_T(T, SUM)                        \
  do {                                        \
    if (nstate <= 16) SCAN(T, 1, SUM);        \
    else if (nstate <= 32) SCAN(T, 2, SUM);   \
    else if (nstate <= 64) SCAN(T, 4, SUM);   \
    else if (nstate <= 128) SCAN(T, 8, SUM);  \
    else SCAN(T, 16, SUM);                    \
  } while (0)
  if (chunked) {
    if (dtype == LMSF_F32) SCAN_T(float, true); else SCAN_T(bf16_t, true);
    LMSF_LAUNCH_CHECK("selective_scan (chunk summaries)");
    hipLaunchKernelGGL(selective_scan_fold_kernel, dim3((unsigned)(((long)inner * nstate + 255) / 256), n_segments),
                       dim3(256), 0, stream, A_log, seg_starts, scratch_base, scratch, inner, nstate, chunk);
    LMSF_LAUNCH_CHECK("selective_scan (fold)");
  }
  if (dtype == LMSF_F32) SCAN_T(float, false); else SCAN_T(bf16_t, false);
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
// S^T q. The state of a slot: S and n as [H, d, dv + 1], then m as [H, copies] (below).
// Three forms follow: chunks of a segment one after the other or side by side (portions of prompts), and token by
// token with the memory streamed once (steps of single tokens).

// floats of state a slot needs
// m is kept once per block of 32 value columns (all copies equal): workgroups that take different blocks of one head
// then share nothing that any of them writes, whichever of them starts first.
#define MLS_M_COLS 32
__host__ __device__ static inline int mls_m_copies(int dv) { return (dv + MLS_M_COLS - 1) / MLS_M_COLS; }
extern "C" long lmsf_mlstm_state_floats(int H, int d, int dv) {
  return (long)H * d * (dv + 1) + (long)H * mls_m_copies(dv);
}

// ---------------------------------------------------------------- the matrix memory over chunks of tokens
// The same recurrence for segments of many tokens, a chunk of L tokens at a time. With F_t the sum of the log forget
// gates from the chunk's first token to t, g_s = i_s - F_s, M_t = max(m_0, max_{s <= t} g_s) (m_0: the running maximum
// before the chunk), the running maximum is m_t = F_t + M_t and
//   S_t = exp(m_0 - M_t) S_0 + sum_{s <= t} exp(g_s - M_t) k_s v_s^T        (every weight <= 1)
// so that a chunk is three small matrix products: P = (Q K^T) * exp(g_s - M_t) below the diagonal, [O | n.q] = w_0 Q
// [S_0 | n_0] + P [V | 1], and the chunk's last S from K^T (w [V | 1]); O and max(|n.q|, exp(-m_t)) + 1e-6 are left
// in float32 for the kernel that divides and norms the heads. A workgroup of 1,024 threads (four waves a SIMD
// hide one another's waits for LDS): one head of one segment and a block of DVB value columns (n is carried as one more
// column, by the first block); chunks one after the other, a thread an entry of each product.
#define MLC_THREADS 1024

// MODE 0: a segment's chunks one after the other in one workgroup, the state from the slot and back to it.
// Steps with long segments run the chunks side by side instead, in three launches:
// MODE 1: every chunk leaves U = K^T (w [V | 1]) with w_u = exp(g_u - G), G = max_u g_u, and (F_last, G) in scratch;
// mlstm_fold_kernel turns them, chunk after chunk, into every chunk's S_0 (in U's place) and m_0 and writes the slot's S;
// MODE 2: every chunk computes its outputs from its S_0 and m_0 (and the last one writes the slot's m).
// Chunk j of segment s is entry chunk_base[s] + j of the scratch: U as [H, d, dv + 1], fg as [H, 2], m0 as [H].
template <typename T, int MODE>
__global__ __launch_bounds__(MLC_THREADS) void mlstm_chunk_kernel(
    const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v, long qkv_stride,
    const float* __restrict__ gates, long gates_stride, float* __restrict__ state, long state_stride,
    const int* __restrict__ seg_starts, const int* __restrict__ state_slots, float* __restrict__ o_raw, long o_stride,
    int H, int d, int dv, int L, int DVB, float qscale, float cap, int n_vb, const int* __restrict__ chunk_base,
    float* __restrict__ sc_U, float* __restrict__ sc_fg, float* __restrict__ sc_m0, float* __restrict__ den) {
  extern __shared__ float lds[];
  // row lengths in LDS are odd, so that threads that walk down neighbouring rows meet different banks
  const int dp = d | 1, NCp = (DVB + 1) | 1, Lp = L | 1;
  float* sq = lds;                  // [L][dp]
  float* sk = sq + L * dp;          // [L][dp]
  float* sv = sk + L * dp;          // [L][NCp]: the block's values, then 1 (the column of n)
  float* sP = sv + L * NCp;         // [L][Lp]
  float* sS = sP + L * Lp;          // [d][NCp]: S_0's block, then n_0
  float* so = sS + d * NCp;         // [L][NCp]
  float* sF = so + L * NCp;         // [L] F_t;  then [L] g_s;  [L] M_t;  [L] exp(g_s - M_last)
  float* sg = sF + L;
  float* sM = sg + L;
  float* sw = sM + L;
  const int tid = threadIdx.x;
  const int h = blockIdx.x, s = blockIdx.y;
  const int vb = MODE == 0 ? blockIdx.z : blockIdx.z % n_vb, j = MODE == 0 ? 0 : blockIdx.z / n_vb;
  const int e0 = vb * DVB;
  // (n is carried by the first block of columns alone: it is that block's to read and to write, and the other blocks
  // need nothing of it, because the division by max(|n . q|, exp(-m)) + 1e-6 is left to the kernel that follows)
  const int nb = min(DVB, dv - e0), cols = dv + 1, NC = nb + (vb == 0 ? 1 : 0);
  const int seg_start = seg_starts[s], seg_end = seg_starts[s + 1];
  if (MODE != 0 && j * L >= seg_end - seg_start) return;
  const int start = MODE == 0 ? seg_start : seg_start + j * L;
  const int end = MODE == 0 ? seg_end : min(seg_end, start + L);
  const long ent = MODE == 0 ? 0 : (long)chunk_base[s] + j;
  float* st = state + (long)state_slots[s] * state_stride;
  // where S_0 comes from (and, MODE 0, goes back to) and where m_0 lies
  float* gS = MODE == 0 ? st + (long)h * d * cols : sc_U + (ent * H + h) * d * cols;
  float* gm = MODE == 0 ? st + (long)H * d * cols + (long)h * mls_m_copies(dv) + vb : sc_m0 + ent * H + h;
  if (MODE != 1) {
    for (int i = tid; i < d * NC; i += MLC_THREADS) {
      const int dd = i / NC, c = i % NC;
      sS[dd * NCp + c] = c < nb ? gS[(long)dd * cols + e0 + c] : gS[(long)dd * cols + dv];
    }
  }
  float m = MODE == 1 ? -INFINITY : gm[0];
  for (int t0 = start; t0 < end; t0 += L) {
    const int nt = min(L, end - t0);
    __syncthreads();
    for (int i = tid; i < nt * d; i += MLC_THREADS) {
      const int tt = i / d, dd = i % d;
      const long at = (long)(t0 + tt) * qkv_stride + h * d + dd;
      if (MODE != 1) sq[tt * dp + dd] = to_f32<T>(q[at]) * qscale;
      sk[tt * dp + dd] = to_f32<T>(k[at]);
    }
    for (int i = tid; i < nt * NC; i += MLC_THREADS) {
      const int tt = i / NC, c = i % NC;
      sv[tt * NCp + c] = c < nb ? to_f32<T>(v[(long)(t0 + tt) * qkv_stride + h * dv + e0 + c]) : 1.f;
    }
    if (tid < nt) {
      const float ip = gates[(long)(t0 + tid) * gates_stride + h], fp = gates[(long)(t0 + tid) * gates_stride + H + h];
      sg[tid] = cap * tanhf(ip / cap);                              // i_t for now
      sF[tid] = rc_logsigmoid(cap * tanhf(fp / cap));               // f_t for now
    }
    __syncthreads();
    if (tid < LMSF_WAVE) {
      // F_t, g_t = i_t - F_t and M_t = max(m_0, max_{u <= t} g_u): running sums and maxima over a wave's lanes
      float F = tid < nt ? sF[tid] : 0.f;
      for (int o = 1; o < LMSF_WAVE; o <<= 1) {
        const float up = __shfl_up(F, o, LMSF_WAVE);
        if (tid >= o) F += up;
      }
      const float g = tid < nt ? sg[tid] - F : -INFINITY;
      float G = fmaxf(g, m);
      for (int o = 1; o < LMSF_WAVE; o <<= 1) {
        const float up = __shfl_up(G, o, LMSF_WAVE);
        if (tid >= o) G = fmaxf(G, up);
      }
      if (tid < nt) {
        sF[tid] = F;
        sg[tid] = g;
        sM[tid] = G;
      }
    }
    __syncthreads();
    const float M_last = sM[nt - 1];
    if (tid < nt) sw[tid] = expf(sg[tid] - M_last);
    if (MODE != 1) {
      // P[t][u] = (q_t . k_u) exp(g_u - M_t) for u <= t
      for (int i = tid; i < nt * nt; i += MLC_THREADS) {
        const int t = i / nt, u = i % nt;
        float acc = 0.f;
        if (u <= t) {
          const float* qr = sq + t * dp;
          const float* kr = sk + u * dp;
#pragma unroll 8
          for (int dd = 0; dd < d; ++dd) acc += qr[dd] * kr[dd];
          acc *= expf(sg[u] - sM[t]);
        }
        sP[t * Lp + u] = acc;
      }
      __syncthreads();
      // [O | n.q][t][c] = w_0(t) q_t [S_0 | n_0] + P[t] [V | 1]
      for (int i = tid; i < nt * NC; i += MLC_THREADS) {
        const int t = i / NC, c = i % NC;
        float acc = 0.f;
        const float* qr = sq + t * dp;
#pragma unroll 8
        for (int dd = 0; dd < d; ++dd) acc += qr[dd] * sS[dd * NCp + c];
        acc *= expf(m - sM[t]);
        const float* pr = sP + t * Lp;
#pragma unroll 4
        for (int u = 0; u <= t; ++u) acc += pr[u] * sv[u * NCp + c];
        so[t * NCp + c] = acc;
      }
      __syncthreads();
      for (int i = tid; i < nt * nb; i += MLC_THREADS) {
        const int t = i / nb, c = i % nb;
        o_raw[(long)(t0 + t) * o_stride + h * dv + e0 + c] = so[t * NCp + c];
      }
      if (vb == 0 && tid < nt)
        den[(long)(t0 + tid) * H + h] = fmaxf(fabsf(so[tid * NCp + nb]), expf(-(sF[tid] + sM[tid]))) + 1e-6f;
    } else {
      __syncthreads();
    }
    if (MODE == 0) {
      // [S | n] <- exp(m_0 - M_last) [S_0 | n_0] + K^T (w [V | 1])
      const float wl = expf(m - M_last);
      for (int i = tid; i < d * NC; i += MLC_THREADS) {
        const int dd = i / NC, c = i % NC;
        float r = sS[dd * NCp + c] * wl;
#pragma unroll 8
        for (int u = 0; u < nt; ++u) r += sk[u * dp + dd] * sw[u] * sv[u * NCp + c];
        sS[dd * NCp + c] = r;
      }
      m = sF[nt - 1] + M_last;
    }
    if (MODE == 2 && end == seg_end && tid == 0)
      st[(long)H * d * cols + (long)h * mls_m_copies(dv) + vb] = sF[nt - 1] + M_last;      // this block's copy of m
    if (MODE == 1) {
      // U = K^T (w [V | 1]) straight to the scratch; (F_last, G) beside it
      for (int i = tid; i < d * NC; i += MLC_THREADS) {
        const int dd = i / NC, c = i % NC;
        float r = 0.f;
#pragma unroll 8
        for (int u = 0; u < nt; ++u) r += sk[u * dp + dd] * sw[u] * sv[u * NCp + c];
        if (c < nb) gS[(long)dd * cols + e0 + c] = r;
        else if (vb == 0) gS[(long)dd * cols + dv] = r;
      }
      if (tid == 0 && vb == 0) {
        sc_fg[(ent * H + h) * 2] = sF[nt - 1];
        sc_fg[(ent * H + h) * 2 + 1] = M_last;
      }
    }
  }
  if (MODE == 0) {
    __syncthreads();
    for (int i = tid; i < d * NC; i += MLC_THREADS) {
      const int dd = i / NC, c = i % NC;
      if (c < nb) gS[(long)dd * cols + e0 + c] = sS[dd * NCp + c];
      else if (vb == 0) gS[(long)dd * cols + dv] = sS[dd * NCp + c];
    }
    if (tid == 0) gm[0] = m;                     // this block's copy
  }
}

// Chunk after chunk of a segment: the chunk's S_0 and m_0 take U's place and sc_m0, then
//   M = max(m_0, G);  S <- exp(m_0 - M) S + exp(G - M) U;  m <- F_last + M;   at the end S and m go to the slot.
// A thread an entry of [S | n] of one head.
__global__ __launch_bounds__(256) void mlstm_fold_kernel(float* __restrict__ state, long state_stride,
                                                         const int* __restrict__ seg_starts,
                                                         const int* __restrict__ state_slots,
                                                         const int* __restrict__ chunk_base, float* __restrict__ sc_U,
                                                         const float* __restrict__ sc_fg, float* __restrict__ sc_m0,
                                                         int H, int d, int dv, int L) {
  const int h = blockIdx.x, s = blockIdx.y;
  const long per = (long)d * (dv + 1);
  const long i = (long)blockIdx.z * 256 + threadIdx.x;
  if (i >= per) return;
  const int n_chunks = (seg_starts[s + 1] - seg_starts[s] + L - 1) / L;
  float* st = state + (long)state_slots[s] * state_stride;
  float S = st[(long)h * per + i];
  float m = st[(long)H * per + (long)h * mls_m_copies(dv)];      // (copy 0; nobody writes m in this launch)
  const long base = chunk_base[s];
  for (int j = 0; j < n_chunks; ++j) {
    const long ent = (base + j) * H + h;
    const float U = sc_U[ent * per + i];
    const float F = sc_fg[ent * 2], G = sc_fg[ent * 2 + 1];
    sc_U[ent * per + i] = S;
    if (i == 0) sc_m0[ent] = m;
    const float M = fmaxf(m, G);
    S = expf(m - M) * S + expf(G - M) * U;
    m = F + M;
  }
  st[(long)h * per + i] = S;       // (the slot's m is written by the last chunk's workgroup of the launch that follows:
}                                  // here other workgroups of the head may not have read it yet)

// o = num / den[t, h];  out[t, h, e] = o[e] / rms_e(o) * w[h, e] * sigmoid(g[t, h, e]); a wave a (token, head)
template <typename T>
__global__ __launch_bounds__(256) void head_norm_gate_kernel(const float* __restrict__ o, long o_stride,
                                                             const float* __restrict__ den,
                                                             const T* __restrict__ og, long og_stride,
                                                             const float* __restrict__ w, T* __restrict__ out,
                                                             long out_stride, int n_tokens, int H, int dv, float eps) {
  const long unit = (long)blockIdx.x * (256 / LMSF_WAVE) + threadIdx.x / LMSF_WAVE;
  if (unit >= (long)n_tokens * H) return;
  const long t = unit / H;
  const int h = unit % H, lane = threadIdx.x % LMSF_WAVE;
  const float* row = o + t * o_stride + (long)h * dv;
  const float by = 1.f / den[t * H + h];
  float ss = 0.f;
  for (int e = lane; e < dv; e += LMSF_WAVE) ss += (row[e] * by) * (row[e] * by);
  ss = wave_sum(ss);
  const float inv = by / sqrtf(ss / (float)dv + eps);
  for (int e = lane; e < dv; e += LMSF_WAVE) {
    const float g = to_f32<T>(og[t * og_stride + (long)h * dv + e]);
    out[t * out_stride + (long)h * dv + e] = from_f32<T>(row[e] * inv * w[h * dv + e] * rc_sigmoid(g));
  }
}

// The matrix memory for steps of single tokens, where a step is one pass over every request's state and nothing but
// memory counts: a workgroup takes one head of one segment and 64 of its value columns (the first block n as well);
// wave w walks the rows w, w + 4, ..., a lane a column, so that every load of S is 256 consecutive bytes, eight rows
// asked for at a time. S^T q and max(|n . q|, exp(-m)) + 1e-6 are left in float32 for the kernel that divides and
// norms the heads. Segments of more than one token are walked token by token (correct, not fast).
#define MLD_COLS 64

template <typename T>
__global__ __launch_bounds__(256) void mlstm_token_kernel(
    const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v, long qkv_stride,
    const float* __restrict__ gates, long gates_stride, float* __restrict__ state, long state_stride,
    const int* __restrict__ seg_starts, const int* __restrict__ state_slots, float* __restrict__ o_raw, long o_stride,
    float* __restrict__ den, int H, int d, int dv, float qscale, float cap) {
  extern __shared__ float lds[];
  float* sq = lds;               // [d]
  float* sk = sq + d;            // [d]
  float* so = sk + d;            // [4][64]
  const int tid = threadIdx.x, wave = tid / LMSF_WAVE, lane = tid % LMSF_WAVE;
  const int h = blockIdx.x, s = blockIdx.y, e0 = blockIdx.z * MLD_COLS;
  const int cols = dv + 1;
  const bool col_ok = e0 + lane < dv;
  float* st = state + (long)state_slots[s] * state_stride;
  float* gS = st + (long)h * d * cols;
  float* gm = st + (long)H * d * cols + (long)h * mls_m_copies(dv) + blockIdx.z * (MLD_COLS / MLS_M_COLS);
  float m = gm[0];
  for (int t = seg_starts[s]; t < seg_starts[s + 1]; ++t) {
    __syncthreads();
    for (int i = tid; i < d; i += 256) {
      sq[i] = to_f32<T>(q[(long)t * qkv_stride + h * d + i]) * qscale;
      sk[i] = to_f32<T>(k[(long)t * qkv_stride + h * d + i]);
    }
    const float vv = col_ok ? to_f32<T>(v[(long)t * qkv_stride + h * dv + e0 + lane]) : 0.f;
    const float gi = cap * tanhf(gates[(long)t * gates_stride + h] / cap);
    const float gf = rc_logsigmoid(cap * tanhf(gates[(long)t * gates_stride + H + h] / cap));
    const float m_new = fmaxf(gf + m, gi);
    const float keep = expf(gf + m - m_new), take = expf(gi - m_new);
    m = m_new;
    __syncthreads();
    float acc = 0.f;
    for (int d0 = wave; d0 < d; d0 += 4 * 8) {
      float r[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int dd = d0 + 4 * j;
        r[j] = (dd < d && col_ok) ? gS[(long)dd * cols + e0 + lane] : 0.f;
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int dd = d0 + 4 * j;
        if (dd < d && col_ok) {
          const float x = keep * r[j] + take * sk[dd] * vv;
          gS[(long)dd * cols + e0 + lane] = x;
          acc += x * sq[dd];
        }
      }
    }
    so[wave * MLD_COLS + lane] = acc;
    if (wave == 1 && blockIdx.z == 0) {
      // n and n . q, by the first block of columns alone: a lane a row
      float part = 0.f;
      for (int dd = lane; dd < d; dd += LMSF_WAVE) {
        const float x = keep * gS[(long)dd * cols + dv] + take * sk[dd];
        gS[(long)dd * cols + dv] = x;
        part += x * sq[dd];
      }
      part = wave_sum(part);
      if (lane == 0) den[(long)t * H + h] = fmaxf(fabsf(part), expf(-m)) + 1e-6f;
    }
    __syncthreads();
    if (wave == 0 && col_ok)
      o_raw[(long)t * o_stride + h * dv + e0 + lane] =
          so[lane] + so[MLD_COLS + lane] + so[2 * MLD_COLS + lane] + so[3 * MLD_COLS + lane];
  }
  if (tid < MLD_COLS / MLS_M_COLS && e0 + tid * MLS_M_COLS < dv) gm[tid] = m;       // this block's copies of m
}

// the temporary of the forms that leave the division to the heads' kernel: numerators float32 [n_tokens, H * dv], then
// denominators [n_tokens, H]
extern "C" long lmsf_mlstm_chunk_scratch_floats(int n_tokens, int H, int dv) { return (long)n_tokens * H * (dv + 1); }

// tokens of a chunk at heads of d (the most for which a workgroup's operands fit its LDS)
extern "C" int lmsf_mlstm_chunk_tokens(int d) {
  const int DVB = 32, NCp = (DVB + 1) | 1, dp = d | 1;
  for (int L = 64; L >= 4; L /= 2) {
    const size_t smem = ((size_t)2 * L * dp + (size_t)2 * L * NCp + (size_t)L * (L | 1) + (size_t)d * NCp + 4 * L) * sizeof(float);
    if (smem <= 128 * 1024) return L;
  }
  return 0;
}

// floats of scratch a chunk of the side-by-side form takes: U as [H, d, dv + 1], (F_last, G) and m_0 per head
extern "C" long lmsf_mlstm_chunk_entry_floats(int H, int d, int dv) { return (long)H * d * (dv + 1) + 3L * H; }

// ``chunk_base`` null: every segment's chunks one after the other in a workgroup. Otherwise (steps with long
// segments) chunk_base[s] is segment s's first entry of ``entries`` (``n_entries`` of them, each
// lmsf_mlstm_chunk_entry_floats), a segment having ceil(tokens / lmsf_mlstm_chunk_tokens(d)) chunks and the longest
// ``max_chunks``; the chunks then run side by side.
extern "C" int lmsf_mlstm_chunked(const void* q, const void* k, const void* v, int dtype, long qkv_stride,
                                  const float* gates, long gates_stride, const void* og, long og_stride,
                                  const float* norm_w, float* state, long state_stride, const int* seg_starts,
                                  const int* state_slots, void* out, long out_stride, float* o_raw, int n_tokens,
                                  int n_segments, int H, int d, int dv, float qscale, float cap, float eps,
                                  const int* chunk_base, int max_chunks, long n_entries, float* entries,
                                  hipStream_t stream) {
  LMSF_CHECK(q && k && v && gates && og && norm_w && state && seg_starts && state_slots && out && o_raw,
             "mlstm_chunked: null pointer");
  LMSF_CHECK(dtype == LMSF_F32 || dtype == LMSF_BF16, "mlstm_chunked: unknown dtype code %d", dtype);
  LMSF_CHECK(H > 0 && H <= 65535 && d > 0 && dv > 0, "mlstm_chunked: bad sizes H=%d d=%d dv=%d", H, d, dv);
  LMSF_CHECK(cap > 0.f, "mlstm_chunked: the gates' cap must be > 0");
  LMSF_CHECK(gates_stride >= 2 * H && og_stride >= (long)H * dv && out_stride >= (long)H * dv &&
                 state_stride >= lmsf_mlstm_state_floats(H, d, dv),
             "mlstm_chunked: strides too small");
  LMSF_CHECK(n_tokens >= 0 && n_segments >= 0 && n_segments <= 65535, "mlstm_chunked: bad counts");
  LMSF_CHECK(!chunk_base || (entries && max_chunks >= 1 && n_entries >= 1), "mlstm_chunked: chunks without scratch");
  if (n_tokens == 0 || n_segments == 0) return 0;
  const int DVB = MLS_M_COLS, NCp = (DVB + 1) | 1, dp = d | 1;       // (a block of columns owns one copy of m)
  const int L = lmsf_mlstm_chunk_tokens(d);
  LMSF_CHECK(L > 0, "mlstm_chunked: heads of %d entries do not fit a workgroup's LDS", d);
  const size_t smem = ((size_t)2 * L * dp + (size_t)2 * L * NCp + (size_t)L * (L | 1) + (size_t)d * NCp + 4 * L) * sizeof(float);
  const int n_vb = (dv + DVB - 1) / DVB;
  LMSF_CHECK(!chunk_base || (long)n_vb * max_chunks <= 65535, "mlstm_chunked: too many chunks");
#define MLC_RESERVE(T, MODE)                                                                                       \
  do {                                                                                                             \
    static size_t reserved = 0;                                                                                    \
    if (smem > 64 * 1024 && smem > reserved) {                                                                     \
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(mlstm_chunk_kernel<T, MODE>),               \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);                   \
      if (e != hipSuccess) {                                                                                       \
        lmsf_set_error("mlstm_chunked: cannot reserve %zu bytes of LDS: %s", smem, hipGetErrorString(e));          \
        return 2;                                                                                                  \
      }                                                                                                            \
      reserved = smem;                                                                                             \
    }                                                                                                              \
  } while (0)
#define MLC_LAUNCH(T, MODE, GRID)                                                                                  \
  do {                                                                                                             \
    MLC_RESERVE(T, MODE);                                                                                          \
    hipLaunchKernelGGL((mlstm_chunk_kernel<T, MODE>), GRID, dim3(MLC_THREADS), smem, stream, (const T*)q,          \
                       (const T*)k, (const T*)v, qkv_stride, gates, gates_stride, state, state_stride, seg_starts, \
                       state_slots, o_raw, (long)H * dv, H, d, dv, L, DVB, qscale, cap, n_vb, chunk_base, sc_U,    \
                       sc_fg, sc_m0, o_raw + (long)n_tokens * H * dv);                                             \
  } while (0)
  float* sc_U = entries;
  float* sc_fg = entries ? entries + n_entries * H * d * (dv + 1) : nullptr;
  float* sc_m0 = entries ? sc_fg + n_entries * H * 2 : nullptr;
  if (!chunk_base) {
    dim3 grid(H, n_segments, n_vb);
    if (dtype == LMSF_F32) MLC_LAUNCH(float, 0, grid); else MLC_LAUNCH(bf16_t, 0, grid);
    LMSF_LAUNCH_CHECK("mlstm_chunk");
  } else {
    dim3 grid(H, n_segments, n_vb * max_chunks);
    if (dtype == LMSF_F32) MLC_LAUNCH(float, 1, grid); else MLC_LAUNCH(bf16_t, 1, grid);
    LMSF_LAUNCH_CHECK("mlstm_chunk (summaries)");
    const long per = (long)d * (dv + 1);
    hipLaunchKernelGGL(mlstm_fold_kernel, dim3(H, n_segments, (unsigned)((per + 255) / 256)), dim3(256), 0, stream, state,
                       state_stride, seg_starts, state_slots, chunk_base, sc_U, sc_fg, sc_m0, H, d, dv, L);
    LMSF_LAUNCH_CHECK("mlstm_chunk (fold)");
    if (dtype == LMSF_F32) MLC_LAUNCH(float, 2, grid); else MLC_LAUNCH(bf16_t, 2, grid);
    LMSF_LAUNCH_CHECK("mlstm_chunk (outputs)");
  }
#undef MLC_LAUNCH
#undef MLC_RESERVE
  const long units = (long)n_tokens * H;
  dim3 ngrid((unsigned)((units + 3) / 4)), block(256);
  if (dtype == LMSF_F32)
    hipLaunchKernelGGL((head_norm_gate_kernel<float>), ngrid, block, 0, stream, o_raw, (long)H * dv,
                       o_raw + (long)n_tokens * H * dv, (const float*)og,
                       og_stride, norm_w, (float*)out, out_stride, n_tokens, H, dv, eps);
  else
    hipLaunchKernelGGL((head_norm_gate_kernel<bf16_t>), ngrid, block, 0, stream, o_raw, (long)H * dv,
                       o_raw + (long)n_tokens * H * dv, (const bf16_t*)og,
                       og_stride, norm_w, (bf16_t*)out, out_stride, n_tokens, H, dv, eps);
  LMSF_LAUNCH_CHECK("head_norm_gate");
  return 0;
}

// The same function for steps of few tokens a segment (decoding): mlstm_token_kernel, then the heads' norm and gate.
extern "C" int lmsf_mlstm_tokens(const void* q, const void* k, const void* v, int dtype, long qkv_stride,
                                 const float* gates, long gates_stride, const void* og, long og_stride,
                                 const float* norm_w, float* state, long state_stride, const int* seg_starts,
                                 const int* state_slots, void* out, long out_stride, float* o_raw, int n_tokens,
                                 int n_segments, int H, int d, int dv, float qscale, float cap, float eps,
                                 hipStream_t stream) {
  LMSF_CHECK(q && k && v && gates && og && norm_w && state && seg_starts && state_slots && out && o_raw,
             "mlstm_tokens: null pointer");
  LMSF_CHECK(dtype == LMSF_F32 || dtype == LMSF_BF16, "mlstm_tokens: unknown dtype code %d", dtype);
  LMSF_CHECK(H > 0 && H <= 65535 && d > 0 && d <= 4096 && dv > 0, "mlstm_tokens: bad sizes H=%d d=%d dv=%d", H, d, dv);
  LMSF_CHECK(cap > 0.f, "mlstm_tokens: the gates' cap must be > 0");
  LMSF_CHECK(gates_stride >= 2 * H && og_stride >= (long)H * dv && out_stride >= (long)H * dv &&
                 state_stride >= lmsf_mlstm_state_floats(H, d, dv),
             "mlstm_tokens: strides too small");
  LMSF_CHECK(n_tokens >= 0 && n_segments >= 0 && n_segments <= 65535 && (dv + MLD_COLS - 1) / MLD_COLS <= 65535,
             "mlstm_tokens: bad counts");
  if (n_tokens == 0 || n_segments == 0) return 0;
  dim3 grid(H, n_segments, (dv + MLD_COLS - 1) / MLD_COLS), block(256);
  const size_t smem = (size_t)(2 * d + 4 * MLD_COLS) * sizeof(float);
  const long units = (long)n_tokens * H;
  dim3 ngrid((unsigned)((units + 3) / 4));
  if (dtype == LMSF_F32) {
    hipLaunchKernelGGL((mlstm_token_kernel<float>), grid, block, smem, stream, (const float*)q, (const float*)k,
                       (const float*)v, qkv_stride, gates, gates_stride, state, state_stride, seg_starts, state_slots,
                       o_raw, (long)H * dv, o_raw + (long)n_tokens * H * dv, H, d, dv, qscale, cap);
    LMSF_LAUNCH_CHECK("mlstm_tokens");
    hipLaunchKernelGGL((head_norm_gate_kernel<float>), ngrid, block, 0, stream, o_raw, (long)H * dv,
                       o_raw + (long)n_tokens * H * dv, (const float*)og,
                       og_stride, norm_w, (float*)out, out_stride, n_tokens, H, dv, eps);
  } else {
    hipLaunchKernelGGL((mlstm_token_kernel<bf16_t>), grid, block, smem, stream, (const bf16_t*)q, (const bf16_t*)k,
                       (const bf16_t*)v, qkv_stride, gates, gates_stride, state, state_stride, seg_starts, state_slots,
                       o_raw, (long)H * dv, o_raw + (long)n_tokens * H * dv, H, d, dv, qscale, cap);
    LMSF_LAUNCH_CHECK("mlstm_tokens");
    hipLaunchKernelGGL((head_norm_gate_kernel<bf16_t>), ngrid, block, 0, stream, o_raw, (long)H * dv,
                       o_raw + (long)n_tokens * H * dv, (const bf16_t*)og,
                       og_stride, norm_w, (bf16_t*)out, out_stride, n_tokens, H, dv, eps);
  }
  LMSF_LAUNCH_CHECK("head_norm_gate");
  return 0;
}
