// A selective state-space mixer: a short causal convolution per channel and a recurrence whose decay, input and
// output weights depend on the token.
//
//   xc[t][c] = silu(bias[c] + sum_j w[j][c] * x[t - (taps - 1) + j][c])          zeros before a sequence's start; w is kept
//                                                                            tap by tap, [taps, C]: neighbours read neighbours
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
// the decay exp(dt A) of an element: the library's exponential in the 32-bit engine; with bfloat16 storage the
// hardware's (exp2 of the argument times log2 e; the argument is at most 0, the relative error a few 1e-7)
template <typename T> __device__ __forceinline__ float decay_exp(float v);
template <> __device__ __forceinline__ float decay_exp<float>(float v) { return expf(v); }
template <> __device__ __forceinline__ float decay_exp<bf16_t>(float v) { return __expf(v); }

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
  float acc = bias ? bias[c] : 0.f;
  for (int j = 0; j < taps; j++) {
    const int src = t - (taps - 1) + j;                 // token index of this tap's input
    const float v = src >= first ? load_f32(x + (size_t)src * ldx + c) : hist[(taps - 1) + (src - first)];
    acc = fmaf(w[(size_t)j * C + c], v, acc);
  }
  store_f32(out + (size_t)t * C + c, silu_f(acc));
}

// The same for bfloat16 with eight neighbouring channels a thread (16-byte accesses; C and the row stride multiples of 8).
// grid (T, ceil(C / 8 / 256)).
__global__ __launch_bounds__(256) void causal_conv8_kernel(const bf16_t* __restrict__ x, int ldx, const float* __restrict__ w,
                                                           const float* __restrict__ bias, const int* __restrict__ token_seq,
                                                           const int* __restrict__ cu_seqlens,
                                                           const int* __restrict__ state_slots, const float* __restrict__ state,
                                                           int num_slots, int C, int N, int taps, bf16_t* __restrict__ out) {
  const int t = blockIdx.x, c0 = (blockIdx.y * blockDim.x + threadIdx.x) * 8;
  if (c0 >= C) return;
  const int b = token_seq[t], first = cu_seqlens[b];
  const int slot = min(max(state_slots[b], 0), num_slots - 1);
  float acc[8];
#pragma unroll
  for (int i = 0; i < 8; i++) acc[i] = bias ? bias[c0 + i] : 0.f;
  for (int j = 0; j < taps; j++) {
    const int src = t - (taps - 1) + j;
    float v[8];
    if (src >= first) {
      const uint4 r = *reinterpret_cast<const uint4*>(x + (size_t)src * ldx + c0);
      v[0] = __uint_as_float(r.x << 16); v[1] = __uint_as_float(r.x & 0xffff0000u);
      v[2] = __uint_as_float(r.y << 16); v[3] = __uint_as_float(r.y & 0xffff0000u);
      v[4] = __uint_as_float(r.z << 16); v[5] = __uint_as_float(r.z & 0xffff0000u);
      v[6] = __uint_as_float(r.w << 16); v[7] = __uint_as_float(r.w & 0xffff0000u);
    } else {
#pragma unroll
      for (int i = 0; i < 8; i++) v[i] = state[((size_t)slot * C + c0 + i) * (N + taps - 1) + N + (taps - 1) + (src - first)];
    }
    const float4 w0 = *reinterpret_cast<const float4*>(w + (size_t)j * C + c0), w1 = *reinterpret_cast<const float4*>(w + (size_t)j * C + c0 + 4);
    acc[0] = fmaf(w0.x, v[0], acc[0]); acc[1] = fmaf(w0.y, v[1], acc[1]); acc[2] = fmaf(w0.z, v[2], acc[2]); acc[3] = fmaf(w0.w, v[3], acc[3]);
    acc[4] = fmaf(w1.x, v[4], acc[4]); acc[5] = fmaf(w1.y, v[5], acc[5]); acc[6] = fmaf(w1.z, v[6], acc[6]); acc[7] = fmaf(w1.w, v[7], acc[7]);
  }
  uint4 o;
  o.x = pack2_bf16(silu_f(acc[0]), silu_f(acc[1]));
  o.y = pack2_bf16(silu_f(acc[2]), silu_f(acc[3]));
  o.z = pack2_bf16(silu_f(acc[4]), silu_f(acc[5]));
  o.w = pack2_bf16(silu_f(acc[6]), silu_f(acc[7]));
  *reinterpret_cast<uint4*>(out + (size_t)t * C + c0) = o;
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

// Every sequence brings ONE token (a decode step): convolution and history in one launch, a thread per (sequence,
// channel), which reads its history before it writes it.  grid (sequences, ceil(C / 256)).
template <typename T>
__global__ __launch_bounds__(256) void causal_conv_step_kernel(const T* __restrict__ x, int ldx, const float* __restrict__ w,
                                                               const float* __restrict__ bias, const int* __restrict__ cu_seqlens,
                                                               const int* __restrict__ state_slots, float* __restrict__ state,
                                                               int num_slots, int C, int N, int taps, T* __restrict__ out) {
  const int b = blockIdx.x, c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int t = cu_seqlens[b], slot = state_slots[b];
  if (cu_seqlens[b + 1] != t + 1 || slot < 0 || slot >= num_slots) return;
  float* hist = state + ((size_t)slot * C + c) * (N + taps - 1) + N;
  const float xv = load_f32(x + (size_t)t * ldx + c);
  float acc = bias ? bias[c] : 0.f;
  float keep[SSM_MAX_TAPS];
  for (int j = 0; j < taps - 1; j++) {
    keep[j] = hist[j];
    acc = fmaf(w[(size_t)j * C + c], keep[j], acc);
  }
  acc = fmaf(w[(size_t)(taps - 1) * C + c], xv, acc);
  for (int j = 0; j + 1 < taps - 1; j++) hist[j] = keep[j + 1];
  if (taps > 1) hist[taps - 2] = xv;
  store_f32(out + (size_t)t * C + c, silu_f(acc));
}

extern "C" int pico_causal_conv(const void* x, int ldx, int dtype, const float* w, const float* bias, const int* token_seq,
                                const int* cu_seqlens, const int* state_slots, float* state, int num_slots, int T, int B,
                                int C, int N, int taps, void* out, int single, hipStream_t stream) {
  PICO_REQUIRE(T >= 0 && B >= 0 && C > 0 && N >= 0 && taps >= 1 && taps <= SSM_MAX_TAPS && ldx >= C && num_slots > 0,
               "pico_causal_conv: bad sizes (1 to %d taps)", SSM_MAX_TAPS);
  if (T == 0 || B == 0) return 0;
  const int cb = (C + 255) / 256;
  PICO_REQUIRE(cb <= 65535, "pico_causal_conv: too many channels");
  if (single) {               // one token a sequence (the caller says so; a sequence of another length is left alone)
    PICO_REQUIRE(T == B, "pico_causal_conv: a step of single tokens has as many tokens as sequences");
    if (dtype == PICO_DTYPE_F32)
      causal_conv_step_kernel<float><<<dim3(B, cb), 256, 0, stream>>>((const float*)x, ldx, w, bias, cu_seqlens, state_slots, state,
                                                                      num_slots, C, N, taps, (float*)out);
    else if (dtype == PICO_DTYPE_BF16)
      causal_conv_step_kernel<bf16_t><<<dim3(B, cb), 256, 0, stream>>>((const bf16_t*)x, ldx, w, bias, cu_seqlens, state_slots, state,
                                                                       num_slots, C, N, taps, (bf16_t*)out);
    else
      PICO_REQUIRE(false, "pico_causal_conv: unknown dtype %d", dtype);
    PICO_LAUNCH_CHECK();
    return 0;
  }
  if (dtype == PICO_DTYPE_F32) {
    causal_conv_kernel<float><<<dim3(T, cb), 256, 0, stream>>>((const float*)x, ldx, w, bias, token_seq, cu_seqlens, state_slots,
                                                               state, num_slots, C, N, taps, (float*)out);
    if (taps > 1)
      conv_history_kernel<float><<<dim3(B, cb), 256, 0, stream>>>((const float*)x, ldx, cu_seqlens, state_slots, state, num_slots, C, N, taps);
  } else if (dtype == PICO_DTYPE_BF16) {
    if (C % 8 == 0 && ldx % 8 == 0 && (uintptr_t)x % 16 == 0 && (uintptr_t)out % 16 == 0 && (uintptr_t)w % 16 == 0)
      causal_conv8_kernel<<<dim3(T, (C / 8 + 255) / 256), 256, 0, stream>>>((const bf16_t*)x, ldx, w, bias, token_seq, cu_seqlens,
                                                                            state_slots, state, num_slots, C, N, taps, (bf16_t*)out);
    else
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
// The recurrence.  grid (sequences, ceil(C / channels a workgroup)); LPC lanes (a power of two: 1 up to 16 state
// elements, so that a lane owns at most 16) share a channel, lane l of them owns state elements l, l + LPC, .. (NPL of
// them); the sum over n is a lane's chain and then a butterfly over the LPC lanes.  Tokens are taken SSM_TB at a time:
// a thread's own values (its channel's input, step size and gate: neighbouring threads read neighbouring channels)
// travel together in registers, and the tokens' B and C rows, which all channels share, are staged in LDS.
// ---------------------------------------------------------------------------
#define SSM_TB 16
#define SSM_WHOLE 0
#define SSM_LOCAL 1
#define SSM_FROM 2

// Long portions are cut into chunks of `chunk` tokens that run side by side (the recurrence is linear in the state):
//   SSM_LOCAL: every chunk from a state of zero, no outputs; leaves its state in ws[chunk] and the sum of its step
//              sizes in ws_dt[chunk] (the chunk's decay of element n is exp(A[c][n] * that sum))
//   (ssm_combine_kernel walks a sequence's chunks: ws[j] <- the state in front of chunk j, and the slot's final state)
//   SSM_FROM:  every chunk again from ws[chunk], writing the outputs
// SSM_WHOLE is the plain walk from the slot's state.  blockIdx.x = sequence * max_chunks + chunk.
template <typename T, int NPL, int MODE>
__global__ __launch_bounds__(256) void selective_scan_kernel(const T* __restrict__ xc, const float* __restrict__ dtp,
                                                             const float* __restrict__ dt_bias, const T* __restrict__ bc,
                                                             int ldbc, int b_col, int c_col, const float* __restrict__ A_log,
                                                             const float* __restrict__ D, const T* __restrict__ z, int ldz,
                                                             const int* __restrict__ cu_seqlens,
                                                             const int* __restrict__ state_slots, float* __restrict__ state,
                                                             int num_slots, int C, int N, int hist, int LPC,
                                                             T* __restrict__ out, int chunk, int max_chunks,
                                                             float* __restrict__ ws, float* __restrict__ ws_dt) {
  extern __shared__ float bcs[];                         // [SSM_TB][2 N]: the block's B and C rows, shared by all channels
  const int b = MODE == SSM_WHOLE ? blockIdx.x : blockIdx.x / max_chunks;
  const int per = blockDim.x / LPC;                      // channels a workgroup
  const int c = blockIdx.y * per + threadIdx.x / LPC, l = threadIdx.x % LPC;
  int t_begin = cu_seqlens[b], t_end = cu_seqlens[b + 1];
  const int slot = state_slots[b];
  if (MODE != SSM_WHOLE) {
    t_begin += (blockIdx.x % max_chunks) * chunk;
    t_end = min(t_end, t_begin + chunk);
  }
  if (slot < 0 || slot >= num_slots || t_end <= t_begin) return;      // the whole workgroup alike
  const bool c_ok = c < C;
  const int ci = min(c, C - 1);
  float* sp = MODE == SSM_WHOLE ? state + ((size_t)slot * C + ci) * (N + hist) : ws + ((size_t)blockIdx.x * C + ci) * N;
  float S[NPL], A[NPL];
  int ni[NPL];
  bool n_ok[NPL];
#pragma unroll
  for (int j = 0; j < NPL; j++) {
    const int n = l + j * LPC;
    n_ok[j] = n < N;
    ni[j] = min(n, N - 1);
    S[j] = (MODE != SSM_LOCAL && n_ok[j]) ? sp[ni[j]] : 0.f;
    A[j] = -expf(A_log[(size_t)ci * N + ni[j]]);
  }
  const float bias = dt_bias[ci], Dc = D[ci];
  float dt_sum = 0.f;
  for (int t0 = t_begin; t0 < t_end; t0 += SSM_TB) {
    const int nb = min(SSM_TB, t_end - t0);
    // a thread's own values of the block's tokens travel while the B and C rows are staged
    float xv[SSM_TB], dv[SSM_TB], zv[SSM_TB];
#pragma unroll
    for (int k = 0; k < SSM_TB; k++) {
      const size_t t = (size_t)(t0 + min(k, nb - 1));
      xv[k] = load_f32(xc + t * C + ci);
      dv[k] = dtp[t * C + ci];
      zv[k] = MODE != SSM_LOCAL ? load_f32(z + t * ldz + ci) : 0.f;
    }
    __syncthreads();                                     // the last block's rows have been read
    for (int i = threadIdx.x; i < nb * 2 * N; i += blockDim.x) {
      const int k = i / (2 * N), e = i % (2 * N);
      bcs[i] = load_f32(bc + (size_t)(t0 + k) * ldbc + (e < N ? b_col + e : c_col + e - N));
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < SSM_TB; k++) {
      if (k >= nb) break;
      const float pre = dv[k] + bias;
      const float dt = pre > 20.f ? pre : log1pf(expf(pre));
      const float dx = dt * xv[k];
      dt_sum += dt;
      const float* Bk = bcs + k * 2 * N;
      float y = 0.f;
#pragma unroll
      for (int j = 0; j < NPL; j++) {
        S[j] = n_ok[j] ? fmaf(decay_exp<T>(dt * A[j]), S[j], dx * Bk[ni[j]]) : 0.f;
        if (MODE != SSM_LOCAL) y = fmaf(S[j], Bk[N + ni[j]], y);
      }
      if (MODE != SSM_LOCAL) {
        for (int off = LPC >> 1; off > 0; off >>= 1) y += __shfl_xor(y, off, 64);
        if (l == 0 && c_ok) store_f32(out + (size_t)(t0 + k) * C + c, fmaf(Dc, xv[k], y) * silu_f(zv[k]));
      }
    }
  }
  if (c_ok && MODE != SSM_FROM) {
#pragma unroll
    for (int j = 0; j < NPL; j++)
      if (n_ok[j]) sp[ni[j]] = S[j];
    if (MODE == SSM_LOCAL && l == 0) ws_dt[(size_t)blockIdx.x * C + c] = dt_sum;
  }
}

// The walk over a sequence's chunks, one thread per state element: ws[j] becomes the state in front of chunk j, the
// slot gets the state behind the last chunk.  grid (sequences, ceil(C N / 256)).
__global__ __launch_bounds__(256) void ssm_combine_kernel(const int* __restrict__ cu_seqlens, const int* __restrict__ state_slots,
                                                          float* __restrict__ state, float* __restrict__ ws,
                                                          const float* __restrict__ ws_dt, const float* __restrict__ A_log,
                                                          int num_slots, int C, int N, int hist, int chunk, int max_chunks) {
  const int b = blockIdx.x, e = blockIdx.y * 256 + threadIdx.x;
  if (e >= C * N) return;
  const int slot = state_slots[b], n_tok = cu_seqlens[b + 1] - cu_seqlens[b];
  if (slot < 0 || slot >= num_slots || n_tok <= 0) return;
  const int c = e / N, n = e % N;
  const float A = -expf(A_log[e]);
  float* sp = state + ((size_t)slot * C + c) * (N + hist) + n;
  float S = *sp;
  const int chunks = (n_tok + chunk - 1) / chunk;
  for (int j = 0; j < chunks; j++) {
    const size_t at = (size_t)b * max_chunks + j;
    float* w = ws + (at * C + c) * N + n;
    const float local = *w;
    *w = S;
    S = fmaf(expf(A * ws_dt[at * C + c]), S, local);
  }
  *sp = S;
}

// chunk == 0: every sequence walked whole from its slot.  chunk > 0: sequences cut into chunks of that many tokens that
// run side by side (three launches); ws float32 [num_seqs * max_chunks, C, N], ws_dt [num_seqs * max_chunks, C],
// max_chunks at least the chunks of the longest sequence.
extern "C" int pico_selective_scan(const void* xc, const float* dtp, const float* dt_bias, const void* bc, int ldbc, int b_col,
                                   int c_col, const float* A_log, const float* D, const void* z, int ldz, int dtype,
                                   const int* cu_seqlens, const int* state_slots, float* state, int num_slots, int B, int T,
                                   int C, int N, int hist, void* out, int chunk, int max_chunks, float* ws, float* ws_dt,
                                   hipStream_t stream) {
  PICO_REQUIRE(B >= 0 && T >= 0 && C > 0 && N > 0 && N <= 256 && hist >= 0 && num_slots > 0 && ldz >= C &&
                   b_col >= 0 && c_col >= 0 && ldbc >= b_col + N && ldbc >= c_col + N,
               "pico_selective_scan: bad sizes (at most 256 state elements a channel)");
  PICO_REQUIRE(chunk == 0 || (chunk > 0 && max_chunks > 0 && ws != nullptr && ws_dt != nullptr &&
                              (long long)max_chunks * chunk >= T && (long long)B * max_chunks < (1ll << 31)),
               "pico_selective_scan: chunks need room for their states and must cover the step's tokens");
  if (B == 0 || T == 0) return 0;
  int lpc = 1;
  while (lpc * 16 < N) lpc *= 2;                         // up to 16 state elements a lane
  const int need = (N + lpc - 1) / lpc;
  const int npl = need <= 1 ? 1 : need <= 2 ? 2 : need <= 4 ? 4 : need <= 8 ? 8 : 16;
  const size_t lds = (size_t)SSM_TB * 2 * N * sizeof(float);
  const int per = 256 / lpc;
  const int gy = (C + per - 1) / per;
  PICO_REQUIRE(gy <= 65535 && ((long long)C * N + 255) / 256 <= 65535, "pico_selective_scan: too many channels");
#define SSM_ARGS(TT)                                                                                                    \
  (const TT*)xc, dtp, dt_bias, (const TT*)bc, ldbc, b_col, c_col, A_log, D, (const TT*)z, ldz, cu_seqlens, state_slots, \
      state, num_slots, C, N, hist, lpc, (TT*)out, chunk, max_chunks, ws, ws_dt
#define SSM_LAUNCH(TT, MODE, GX)                                                                              \
  do {                                                                                                        \
    if (npl == 1) selective_scan_kernel<TT, 1, MODE><<<dim3(GX, gy), 256, lds, stream>>>(SSM_ARGS(TT));       \
    else if (npl == 2) selective_scan_kernel<TT, 2, MODE><<<dim3(GX, gy), 256, lds, stream>>>(SSM_ARGS(TT));  \
    else if (npl == 4) selective_scan_kernel<TT, 4, MODE><<<dim3(GX, gy), 256, lds, stream>>>(SSM_ARGS(TT));  \
    else if (npl == 8) selective_scan_kernel<TT, 8, MODE><<<dim3(GX, gy), 256, lds, stream>>>(SSM_ARGS(TT));  \
    else selective_scan_kernel<TT, 16, MODE><<<dim3(GX, gy), 256, lds, stream>>>(SSM_ARGS(TT));               \
  } while (0)
#define SSM_RUN(TT)                                                                                                        \
  if (chunk == 0) {                                                                                                        \
    SSM_LAUNCH(TT, SSM_WHOLE, B);                                                                                          \
  } else {                                                                                                                 \
    SSM_LAUNCH(TT, SSM_LOCAL, B * max_chunks);                                                                             \
    ssm_combine_kernel<<<dim3(B, (C * N + 255) / 256), 256, 0, stream>>>(cu_seqlens, state_slots, state, ws, ws_dt, A_log, \
                                                                         num_slots, C, N, hist, chunk, max_chunks);        \
    SSM_LAUNCH(TT, SSM_FROM, B * max_chunks);                                                                              \
  }
  if (dtype == PICO_DTYPE_F32) {
    SSM_RUN(float)
  } else if (dtype == PICO_DTYPE_BF16) {
    SSM_RUN(bf16_t)
  } else {
    PICO_REQUIRE(false, "pico_selective_scan: unknown dtype %d", dtype);
  }
#undef SSM_RUN
#undef SSM_LAUNCH
#undef SSM_ARGS
  PICO_LAUNCH_CHECK();
  return 0;
}
