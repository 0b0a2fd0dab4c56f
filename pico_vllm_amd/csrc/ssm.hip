// A selective state-space mixer: a short causal convolution per channel and a recurrence whose decay, input and
// output weights depend on the token.
//
//   xc[t][c] = silu(bias[c] + sum_j w[c][j] * x[t - (taps - 1) + j][c])          zeros before a sequence's start
//   dt[t][c] = softplus(dtp[t][c] + dt_bias[c]),   A[c][n] = -exp(A_log[c][n])
//   S[c][n] <- exp(dt A) S + dt xc[t][c] B[t][n];   y[t][c] = sum_n S[c][n] C[t][n] + D[c] xc[t][c]
//   out[t][c] = y[t][c] * silu(z[t][c])
//
// A request's state slot holds, per channel, the N elements of S and behind them the last taps - 1 inputs of the
// convolution (float32 [slots, channels, N + taps - 1]).  Step sizes, decays, the recurrence and its state are
// float32 whatever the storage type of the projections; every sum runs in an order that depends on the sizes alone.
#include "common.h"

#define SSM_MAX_TAPS 16

__device__ __forceinline__ float silu_f(float v) { return v / (1.0f + expf(-v)); }

// grid (T, ceil(C / 256)): one thread per (token, channel).  Inputs before the portion come from the slot's history.
template <typename T>
__global__ __launch_bounds__(256) void causal_conv_kernel(const T* __restrict__ x, int ldx, const float* __restrict__ w,
                                                          const float* __restrict__ bias, const int* __restrict__ token_seq,
                                                          const int* __restrict__ cu_seqlens,
                                                          const int* __restrict__ state_slots, const float* __restrict__ state,
                                                          int num_slots, int C, int N, int taps, T* __restrict__ out) {
  const int t = blockIdx.x, c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int b = token_seq[t], first = cu_seqlens[b];
  const int slot = min(max(state_slots[b], 0), num_slots - 1);
  const float* hist = state + ((size_t)slot * C + c) * (N + taps - 1) + N;
  float acc = bias[c];
  for (int j = 0; j < taps; j++) {
    const int src = t - (taps - 1) + j;                 // token index of this tap's input
    const float v = src >= first ? load_f32(x + (size_t)src * ldx + c) : hist[(taps - 1) + (src - first)];
    acc = fmaf(w[(size_t)c * taps + j], v, acc);
  }
  store_f32(out + (size_t)t * C + c, silu_f(acc));
}

// grid (sequences, ceil(C / 256)): the slot's history becomes the last taps - 1 inputs behind this step's tokens.
template <typename T>
__global__ __launch_bounds__(256) void conv_history_kernel(const T* __restrict__ x, int ldx, const int* __restrict__ cu_seqlens,
                                                           const int* __restrict__ state_slots, float* __restrict__ state,
                                                           int num_slots, int C, int N, int taps) {
  const int b = blockIdx.x, c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int first = cu_seqlens[b], n = cu_seqlens[b + 1] - first, slot = state_slots[b];
  if (n <= 0 || slot < 0 || slot >= num_slots) return;
  float* hist = state + ((size_t)slot * C + c) * (N + taps - 1) + N;
  float keep[SSM_MAX_TAPS];
  for (int k = 0; k < taps - 1; k++) {
    const int at = n + k;                               // index in [old history | this step's inputs]
    keep[k] = at < taps - 1 ? hist[at] : load_f32(x + (size_t)(first + at - (taps - 1)) * ldx + c);
  }
  for (int k = 0; k < taps - 1; k++) hist[k] = keep[k];
}

extern "C" int pico_causal_conv(const void* x, int ldx, int dtype, const float* w, const float* bias, const int* token_seq,
                                const int* cu_seqlens, const int* state_slots, float* state, int num_slots, int T, int B,
                                int C, int N, int taps, void* out, hipStream_t stream) {
  PICO_REQUIRE(T >= 0 && B >= 0 && C > 0 && N > 0 && taps >= 1 && taps <= SSM_MAX_TAPS && ldx >= C && num_slots > 0,
               "pico_causal_conv: bad sizes (1 to %d taps)", SSM_MAX_TAPS);
  if (T == 0 || B == 0) return 0;
  const int cb = (C + 255) / 256;
  PICO_REQUIRE(cb <= 65535, "pico_causal_conv: too many channels");
  if (dtype == PICO_DTYPE_F32) {
    causal_conv_kernel<float><<<dim3(T, cb), 256, 0, stream>>>((const float*)x, ldx, w, bias, token_seq, cu_seqlens, state_slots,
                                                               state, num_slots, C, N, taps, (float*)out);
    if (taps > 1)
      conv_history_kernel<float><<<dim3(B, cb), 256, 0, stream>>>((const float*)x, ldx, cu_seqlens, state_slots, state, num_slots, C, N, taps);
  } else if (dtype == PICO_DTYPE_BF16) {
    causal_conv_kernel<bf16_t><<<dim3(T, cb), 256, 0, stream>>>((const bf16_t*)x, ldx, w, bias, token_seq, cu_seqlens, state_slots,
                                                                state, num_slots, C, N, taps, (bf16_t*)out);
    if (taps > 1)
      conv_history_kernel<bf16_t><<<dim3(B, cb), 256, 0, stream>>>((const bf16_t*)x, ldx, cu_seqlens, state_slots, state, num_slots, C, N, taps);
  } else {
    PICO_REQUIRE(false, "pico_causal_conv: unknown dtype %d", dtype);
  }
  PICO_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------
// The recurrence.  grid (sequences, ceil(C / channels a workgroup)); LPC lanes (a power of two, at most 64) share a
// channel, lane l of them owns state elements l, l + LPC, .. (NPL of them); the sum over n is a lane's chain and then
// a butterfly over the LPC lanes.  Tokens are taken SSM_TB at a time so that their loads travel together.
// ---------------------------------------------------------------------------
#define SSM_TB 8

template <typename T, int NPL>
__global__ __launch_bounds__(256) void selective_scan_kernel(const T* __restrict__ xc, const float* __restrict__ dtp,
                                                             const float* __restrict__ dt_bias, const T* __restrict__ bc,
                                                             int ldbc, int b_col, int c_col, const float* __restrict__ A_log,
                                                             const float* __restrict__ D, const T* __restrict__ z, int ldz,
                                                             const int* __restrict__ cu_seqlens,
                                                             const int* __restrict__ state_slots, float* __restrict__ state,
                                                             int num_slots, int C, int N, int hist, int LPC,
                                                             T* __restrict__ out) {
  const int b = blockIdx.x;
  const int per = blockDim.x / LPC;                      // channels a workgroup
  const int c = blockIdx.y * per + threadIdx.x / LPC, l = threadIdx.x % LPC;
  const int t_begin = cu_seqlens[b], t_end = cu_seqlens[b + 1], slot = state_slots[b];
  if (slot < 0 || slot >= num_slots || t_end <= t_begin) return;
  const bool c_ok = c < C;
  const int ci = min(c, C - 1);
  float* sp = state + ((size_t)slot * C + ci) * (N + hist);
  float S[NPL], A[NPL];
  int ni[NPL];
  bool n_ok[NPL];
#pragma unroll
  for (int j = 0; j < NPL; j++) {
    const int n = l + j * LPC;
    n_ok[j] = n < N;
    ni[j] = min(n, N - 1);
    S[j] = n_ok[j] ? sp[ni[j]] : 0.f;
    A[j] = -expf(A_log[(size_t)ci * N + ni[j]]);
  }
  const float bias = dt_bias[ci], Dc = D[ci];
  for (int t0 = t_begin; t0 < t_end; t0 += SSM_TB) {
    const int nb = min(SSM_TB, t_end - t0);
    float xv[SSM_TB], dv[SSM_TB], zv[SSM_TB], Bv[SSM_TB][NPL], Cv[SSM_TB][NPL];
#pragma unroll
    for (int k = 0; k < SSM_TB; k++) {
      const size_t t = (size_t)(t0 + min(k, nb - 1));
      xv[k] = load_f32(xc + t * C + ci);
      dv[k] = dtp[t * C + ci];
      zv[k] = load_f32(z + t * ldz + ci);
#pragma unroll
      for (int j = 0; j < NPL; j++) {
        Bv[k][j] = load_f32(bc + t * ldbc + b_col + ni[j]);
        Cv[k][j] = load_f32(bc + t * ldbc + c_col + ni[j]);
      }
    }
#pragma unroll
    for (int k = 0; k < SSM_TB; k++) {
      if (k >= nb) break;
      const float pre = dv[k] + bias;
      const float dt = pre > 20.f ? pre : log1pf(expf(pre));
      const float dx = dt * xv[k];
      float y = 0.f;
#pragma unroll
      for (int j = 0; j < NPL; j++) {
        S[j] = n_ok[j] ? fmaf(expf(dt * A[j]), S[j], dx * Bv[k][j]) : 0.f;
        y = fmaf(S[j], Cv[k][j], y);
      }
      for (int off = LPC >> 1; off > 0; off >>= 1) y += __shfl_xor(y, off, 64);
      if (l == 0 && c_ok) store_f32(out + (size_t)(t0 + k) * C + c, fmaf(Dc, xv[k], y) * silu_f(zv[k]));
    }
  }
  if (c_ok) {
#pragma unroll
    for (int j = 0; j < NPL; j++)
      if (n_ok[j]) sp[ni[j]] = S[j];
  }
}

extern "C" int pico_selective_scan(const void* xc, const float* dtp, const float* dt_bias, const void* bc, int ldbc, int b_col,
                                   int c_col, const float* A_log, const float* D, const void* z, int ldz, int dtype,
                                   const int* cu_seqlens, const int* state_slots, float* state, int num_slots, int B, int T,
                                   int C, int N, int hist, void* out, hipStream_t stream) {
  PICO_REQUIRE(B >= 0 && T >= 0 && C > 0 && N > 0 && N <= 256 && hist >= 0 && num_slots > 0 && ldz >= C &&
                   b_col >= 0 && c_col >= 0 && ldbc >= b_col + N && ldbc >= c_col + N,
               "pico_selective_scan: bad sizes (at most 256 state elements a channel)");
  if (B == 0 || T == 0) return 0;
  int lpc = 1;
  while (lpc < N && lpc < 64) lpc *= 2;
  const int npl = (N + lpc - 1) / lpc;                   // 1, 2 or 4 (3 runs as 4)
  const int per = 256 / lpc;
  const dim3 grid(B, (C + per - 1) / per);
  PICO_REQUIRE(grid.y <= 65535, "pico_selective_scan: too many channels");
#define SSM_ARGS(TT)                                                                                                    \
  (const TT*)xc, dtp, dt_bias, (const TT*)bc, ldbc, b_col, c_col, A_log, D, (const TT*)z, ldz, cu_seqlens, state_slots, \
      state, num_slots, C, N, hist, lpc, (TT*)out
#define SSM_LAUNCH(TT)                                                                                    \
  do {                                                                                                    \
    if (npl == 1) selective_scan_kernel<TT, 1><<<grid, 256, 0, stream>>>(SSM_ARGS(TT));                   \
    else if (npl == 2) selective_scan_kernel<TT, 2><<<grid, 256, 0, stream>>>(SSM_ARGS(TT));              \
    else selective_scan_kernel<TT, 4><<<grid, 256, 0, stream>>>(SSM_ARGS(TT));                            \
  } while (0)
  if (dtype == PICO_DTYPE_F32) SSM_LAUNCH(float);
  else if (dtype == PICO_DTYPE_BF16) SSM_LAUNCH(bf16_t);
  else PICO_REQUIRE(false, "pico_selective_scan: unknown dtype %d", dtype);
#undef SSM_LAUNCH
#undef SSM_ARGS
  PICO_LAUNCH_CHECK();
  return 0;
}
