// Gated linear attention: a recurrent mixer whose state is a matrix per head.
//
//   per head, with key channels c and value channels v:
//     S_t[c][v] = alpha_t[c] * S_(t-1)[c][v] + k_t[c] * v_t[v]          (a decay per key channel)
//     o_t[v]    = sum_c S_t[c][v] * q_t[c] * qscale
//   alpha_t = sigmoid(z_t)^(1 / tau),  z_t = A2 (A1 h_t) + b           (a low-rank projection; A1 h_t comes with q, k, v)
//   out_t = rmsnorm_v(o_t) * w * silu(g_t)                             (every head by itself, one weight for all heads)
//
// The state lives in float32, one [heads, dk, dv] block per state slot; decays, their logarithms, the recurrence and
// the head norm are float32 whatever the storage type T of the projections.  Every sum runs in an order that depends
// on the sizes alone, so a token's output does not depend on how its sequence was cut into steps.
#include "common.h"

// ---------------------------------------------------------------------------
// Logarithm of the decay: out[t][c] = log(sigmoid(z)) / tau, z = sum_r a2[c][r] * x[t][r] + b[c].
// x: the low-rank activations (columns of a wider row, stride ldx); a2 [C, R]; b float32 [C].  grid (T), any C and R.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void gla_decay_kernel(const T* __restrict__ x, int ldx, const T* __restrict__ a2,
                                                        const float* __restrict__ b, float inv_tau, float* __restrict__ out,
                                                        int C, int R) {
  extern __shared__ float xs[];
  const int t = blockIdx.x;
  for (int r = threadIdx.x; r < R; r += blockDim.x) xs[r] = load_f32(x + (size_t)t * ldx + r);
  __syncthreads();
  for (int c = threadIdx.x; c < C; c += blockDim.x) {
    const T* w = a2 + (size_t)c * R;
    float z = b ? b[c] : 0.f;
    for (int r = 0; r < R; r++) z = fmaf(load_f32(w + r), xs[r], z);
    // log(sigmoid(z)) = -log(1 + e^-z), without overflow on either side
    const float ls = z >= 0.f ? -log1pf(expf(-z)) : z - log1pf(expf(z));
    out[(size_t)t * C + c] = ls * inv_tau;
  }
}

extern "C" int pico_gla_decay(const void* x, int ldx, int dtype, const void* a2, const float* b, float tau, float* out,
                              int T, int C, int R, hipStream_t stream) {
  PICO_REQUIRE(T >= 0 && C > 0 && R > 0 && ldx >= R && R <= 8192, "pico_gla_decay: bad sizes");
  PICO_REQUIRE(tau > 0.f, "pico_gla_decay: tau must be positive");
  if (T == 0) return 0;
  const size_t lds = (size_t)R * sizeof(float);
  if (dtype == PICO_DTYPE_F32)
    gla_decay_kernel<float><<<T, 256, lds, stream>>>((const float*)x, ldx, (const float*)a2, b, 1.0f / tau, out, C, R);
  else if (dtype == PICO_DTYPE_BF16)
    gla_decay_kernel<bf16_t><<<T, 256, lds, stream>>>((const bf16_t*)x, ldx, (const bf16_t*)a2, b, 1.0f / tau, out, C, R);
  else
    PICO_REQUIRE(false, "pico_gla_decay: unknown dtype %d", dtype);
  PICO_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------
// The recurrence, token by token.  grid (sequences, heads, ceil(dv / 64 VPL)); a workgroup owns 64 VPL value channels of
// one head of one sequence; wave w of its ceil(dk / GLA_CPT) waves owns key channels GLA_CPT w .., lane l value channels
// l, l + 64, .. (VPL of them: 2 where a head has more than 64):
// a thread keeps GLA_CPT state elements in registers over all tokens of the step.  Tokens are taken TB (8 or 16) at a
// time: their q, k and decays are staged in LDS (every thread reads all of its channels' from there) while the next
// block's travel from memory in registers; the waves' partial outputs meet in LDS and are summed in wave order.
//
// Long portions are cut into chunks of `chunk` tokens that run side by side (the recurrence is linear in the state):
//   GLA_LOCAL:  every chunk from a state of zero, no outputs; leaves its state in ws[chunk] and the sum of its decays'
//               logarithms in ws_decay[chunk]
//   (gla_combine_kernel walks a sequence's chunks: ws[j] <- the state in front of chunk j, and the slot's final state)
//   GLA_FROM:   every chunk again from ws[chunk], writing the outputs
// GLA_WHOLE is the plain walk from the slot's state (a sequence is one chunk).  blockIdx.x = sequence * max_chunks + chunk.
// ---------------------------------------------------------------------------
#define GLA_CPT 32
#define GLA_WHOLE 0
#define GLA_LOCAL 1
#define GLA_FROM 2

// FUSED: the decays are made inside the walk (log_decay is null) instead of read.
template <typename T, int MODE, int TB, int VPL, bool FUSED>
__global__ __launch_bounds__(TB == 16 ? 256 : 512) void gla_scan_kernel(const T* __restrict__ x, int ldx, int q_col, int k_col, int v_col,
                                                       const float* __restrict__ log_decay,
                                                       const int* __restrict__ cu_seqlens,
                                                       const int* __restrict__ state_slots, float* __restrict__ state,
                                                       float* __restrict__ out, int H, int dk, int dv, float qscale,
                                                       int num_slots, int chunk, int max_chunks, float* __restrict__ ws,
                                                       float* __restrict__ ws_decay, const T* __restrict__ a2,
                                                       const float* __restrict__ a2_bias, int a_col, int R, float inv_tau,
                                                       const float* __restrict__ head_decay) {
  extern __shared__ float lds[];
  // head_decay given: every key channel of head h decays by the constant head_decay[h] at every token (log_decay, a2
  // are not read); the decay is multiplied in as it is, no logarithm and exponential between
  const float fixed = head_decay ? head_decay[blockIdx.y] : 0.f;
  const int nw = blockDim.x >> 6, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int CP = nw * GLA_CPT;                          // key channels with padding
  float* qs = lds;                                      // [TB][CP]
  float* ks = qs + TB * CP;
  float* as = ks + TB * CP;
  float* po = as + TB * CP;                             // [TB][nw][64 VPL]
  // a lane owns VPL value channels, 64 apart: what it reads of a token's q, k and decays out of LDS serves them all
  // (every wave of a compute unit reads the same staged values, and LDS hands each lane its own copy)
  constexpr int VW = 64 * VPL;
  const int b = MODE == GLA_WHOLE ? blockIdx.x : blockIdx.x / max_chunks, h = blockIdx.y, v = blockIdx.z * VW + lane;
  bool v_ok[VPL];
  int v_in[VPL];                                        // a value channel that exists, else the head's last one
#pragma unroll
  for (int j = 0; j < VPL; j++) {
    v_ok[j] = v + 64 * j < dv;
    v_in[j] = min(v + 64 * j, dv - 1) - v;
  }
  int t_begin = cu_seqlens[b], t_end = cu_seqlens[b + 1];
  if (MODE != GLA_WHOLE) {
    t_begin += (blockIdx.x % max_chunks) * chunk;
    t_end = min(t_end, t_begin + chunk);
  }
  const int slot = state_slots[b];
  if (slot < 0 || slot >= num_slots || t_end <= t_begin) return;
  const int c0 = wave * GLA_CPT;
  float* sp = MODE == GLA_WHOLE ? state + (((size_t)slot * H + h) * dk + c0) * dv + v
                                : ws + (((size_t)blockIdx.x * H + h) * dk + c0) * dv + v;
  // Every load below is unconditional, from an address clamped into the tensor, and what must not count is cleared
  // afterwards: a load inside a branch is waited for inside that branch, and a thread's loads of a block then queue
  // one behind the other's latency instead of travelling together.
  float S[VPL][GLA_CPT];
  if (MODE != GLA_LOCAL) {
#pragma unroll
    for (int j = 0; j < VPL; j++)
#pragma unroll
      for (int c = 0; c < GLA_CPT; c++) S[j][c] = sp[(size_t)(min(c0 + c, dk - 1) - c0) * dv + v_in[j]];
  }
#pragma unroll
  for (int j = 0; j < VPL; j++)
#pragma unroll
    for (int c = 0; c < GLA_CPT; c++) S[j][c] = (MODE != GLA_LOCAL && v_ok[j] && c0 + c < dk) ? S[j][c] : 0.f;
  if (MODE == GLA_LOCAL && blockIdx.z == 0) {
    // the chunk's decays multiplied up, as the sum of their logarithms, for the walk over the chunks
    for (int c = threadIdx.x; c < dk; c += blockDim.x) {
      float sum = 0.f;
      if (head_decay) sum = (float)(t_end - t_begin) * logf(fixed);
      else
        for (int t = t_begin; t < t_end; t++) sum += log_decay[(size_t)t * H * dk + (size_t)h * dk + c];
      ws_decay[((size_t)blockIdx.x * H + h) * dk + c] = sum;
    }
  }
  // A thread stages TB / 2 elements (token tt, channel c) of a block: i = threadIdx.x + j * blockDim.x.  The next
  // block's values travel in registers while this block is walked.
  constexpr int NL = TB / 2;
  const int tt0 = (int)threadIdx.x >= CP ? 1 : 0, cc = (int)threadIdx.x - tt0 * CP;
  T rq[NL], rk[NL], rv[VPL][TB];
  float ra[NL];
  const int c_in = min(cc, dk - 1);
  auto fetch = [&](int t0) {
    const int nb = min(TB, t_end - t0);
#pragma unroll
    for (int j = 0; j < NL; j++) {
      const int tt = min(tt0 + 2 * j, nb - 1);
      const T* row = x + (size_t)(t0 + tt) * ldx + (size_t)h * dk + c_in;
      rq[j] = MODE != GLA_LOCAL ? row[q_col] : row[k_col];
      rk[j] = row[k_col];
      if (head_decay) {
        ra[j] = 0.f;
      } else if (!FUSED) {
        ra[j] = log_decay[(size_t)(t0 + tt) * H * dk + (size_t)h * dk + c_in];
      } else if (tt0 + 2 * j >= nb) {
        ra[j] = 0.f;                                    // no such token in this block: nothing to work out
      } else {
        // the decay's logarithm made here from the low-rank activations (as gla_decay_kernel does): one launch less
        const T* xa = x + (size_t)(t0 + tt) * ldx + a_col;
        const T* w = a2 + ((size_t)h * dk + c_in) * R;
        float z = a2_bias ? a2_bias[h * dk + c_in] : 0.f;
        for (int r = 0; r < R; r++) z = fmaf(load_f32(w + r), load_f32(xa + r), z);
        const float ls = z >= 0.f ? -log1pf(expf(-z)) : z - log1pf(expf(z));
        ra[j] = ls * inv_tau;
      }
    }
#pragma unroll
    for (int j = 0; j < VPL; j++)
#pragma unroll
      for (int tt = 0; tt < TB; tt++) rv[j][tt] = x[(size_t)(t0 + min(tt, nb - 1)) * ldx + v_col + (size_t)h * dv + v + v_in[j]];
  };
  fetch(t_begin);
  for (int t0 = t_begin; t0 < t_end; t0 += TB) {
    const int nb = min(TB, t_end - t0);
    __syncthreads();                                    // the last block's staged values and partial outputs have been read
#pragma unroll
    for (int j = 0; j < NL; j++) {
      const int tt = tt0 + 2 * j, c = cc, i = tt * CP + c;      // = threadIdx.x + j * blockDim.x: a workgroup has 2 CP threads
      const bool in = tt < nb && c < dk;
      qs[i] = (in && MODE != GLA_LOCAL) ? load_f32(&rq[j]) * qscale : 0.f;
      ks[i] = in ? load_f32(&rk[j]) : 0.f;
      as[i] = in ? (head_decay ? fixed : expf(ra[j])) : 1.f;
    }
    float vv[VPL][TB];
#pragma unroll
    for (int j = 0; j < VPL; j++)
#pragma unroll
      for (int tt = 0; tt < TB; tt++) vv[j][tt] = (tt < nb && v_ok[j]) ? load_f32(&rv[j][tt]) : 0.f;
    __syncthreads();
    if (t0 + TB < t_end) fetch(t0 + TB);
#pragma unroll
    for (int tt = 0; tt < TB; tt++) {
      if (tt >= nb) break;
      const float4* a4 = reinterpret_cast<const float4*>(as + tt * CP + c0);
      const float4* k4 = reinterpret_cast<const float4*>(ks + tt * CP + c0);
      const float4* q4 = reinterpret_cast<const float4*>(qs + tt * CP + c0);
      // four partial sums over the channels (c mod 4), added at the end: four short chains instead of one long one
      float acc0[VPL], acc1[VPL], acc2[VPL], acc3[VPL];
#pragma unroll
      for (int j = 0; j < VPL; j++) acc0[j] = acc1[j] = acc2[j] = acc3[j] = 0.f;
#pragma unroll
      for (int c = 0; c < GLA_CPT / 4; c++) {
        const float4 av = a4[c], kv = k4[c];
        float4 qv = make_float4(0.f, 0.f, 0.f, 0.f);
        if (MODE != GLA_LOCAL) qv = q4[c];
#pragma unroll
        for (int j = 0; j < VPL; j++) {
          const float vt = vv[j][tt];
          S[j][4 * c + 0] = fmaf(av.x, S[j][4 * c + 0], kv.x * vt);
          S[j][4 * c + 1] = fmaf(av.y, S[j][4 * c + 1], kv.y * vt);
          S[j][4 * c + 2] = fmaf(av.z, S[j][4 * c + 2], kv.z * vt);
          S[j][4 * c + 3] = fmaf(av.w, S[j][4 * c + 3], kv.w * vt);
          if (MODE != GLA_LOCAL) {
            acc0[j] = fmaf(S[j][4 * c + 0], qv.x, acc0[j]);
            acc1[j] = fmaf(S[j][4 * c + 1], qv.y, acc1[j]);
            acc2[j] = fmaf(S[j][4 * c + 2], qv.z, acc2[j]);
            acc3[j] = fmaf(S[j][4 * c + 3], qv.w, acc3[j]);
          }
        }
      }
      if (MODE != GLA_LOCAL) {
#pragma unroll
        for (int j = 0; j < VPL; j++) po[(tt * nw + wave) * VW + 64 * j + lane] = (acc0[j] + acc1[j]) + (acc2[j] + acc3[j]);
      }
    }
    if (MODE == GLA_LOCAL) continue;
    __syncthreads();
    for (int i = threadIdx.x; i < nb * VW; i += blockDim.x) {
      const int tt = i / VW, l = i % VW, vo = blockIdx.z * VW + l;
      if (vo >= dv) continue;
      float sum = 0.f;
      for (int w = 0; w < nw; w++) sum += po[(tt * nw + w) * VW + l];
      out[(size_t)(t0 + tt) * H * dv + (size_t)h * dv + vo] = sum;
    }
  }
  if (MODE != GLA_FROM) {
#pragma unroll
    for (int j = 0; j < VPL; j++)
#pragma unroll
      for (int c = 0; c < GLA_CPT; c++)
        if (v_ok[j] && c0 + c < dk) sp[(size_t)c * dv + 64 * j] = S[j][c];
  }
}

// The walk over a sequence's chunks, one thread per state element: ws[j] becomes the state in front of chunk j, the
// slot gets the state behind the last chunk.  grid (sequences, heads, ceil(dk dv / 256)).
__global__ __launch_bounds__(256) void gla_combine_kernel(const int* __restrict__ cu_seqlens,
                                                          const int* __restrict__ state_slots, float* __restrict__ state,
                                                          float* __restrict__ ws, const float* __restrict__ ws_decay, int H,
                                                          int dk, int dv, int num_slots, int chunk, int max_chunks) {
  const int b = blockIdx.x, h = blockIdx.y, e = blockIdx.z * 256 + threadIdx.x;
  if (e >= dk * dv) return;
  const int slot = state_slots[b], n = cu_seqlens[b + 1] - cu_seqlens[b];
  if (slot < 0 || slot >= num_slots || n <= 0) return;
  const int c = e / dv;
  float* sp = state + ((size_t)slot * H + h) * dk * dv + e;
  float S = *sp;
  const int chunks = (n + chunk - 1) / chunk;
  for (int j = 0; j < chunks; j++) {
    const size_t at = (size_t)b * max_chunks + j;
    float* w = ws + (at * H + h) * dk * dv + e;
    const float local = *w;
    *w = S;
    S = fmaf(expf(ws_decay[(at * H + h) * dk + c]), S, local);
  }
  *sp = S;
}

// log_decay null (chunk == 0 only): the decays are made inside the walk from x[:, a_col : a_col + R], a2 [H dk, R] and
// a2_bias, as pico_gla_decay makes them.
// chunk == 0: every sequence walked whole from its slot.  chunk > 0: sequences cut into chunks of that many tokens that
// run side by side (three launches); ws float32 [num_seqs * max_chunks, H, dk, dv], ws_decay [num_seqs * max_chunks, H, dk],
// max_chunks at least the chunks of the longest sequence.
extern "C" int pico_gla_scan(const void* x, int ldx, int dtype, int q_col, int k_col, int v_col, const float* log_decay,
                             const int* cu_seqlens, const int* state_slots, float* state, float* out, int num_seqs,
                             int T, int H, int dk, int dv, float qscale, int num_slots, int chunk, int max_chunks,
                             float* ws, float* ws_decay, const void* a2, const float* a2_bias, int a_col, int R, float tau,
                             const float* head_decay, hipStream_t stream) {
  PICO_REQUIRE(head_decay != nullptr || log_decay != nullptr || (chunk == 0 && a2 != nullptr && R > 0 && a_col >= 0 && ldx >= a_col + R && tau > 0.f),
               "pico_gla_scan: without the decays' logarithms the walk needs what makes them, and runs whole");
  PICO_REQUIRE(num_seqs >= 0 && T >= 0 && H > 0 && dk > 0 && dv > 0 && num_slots > 0, "pico_gla_scan: bad sizes");
  PICO_REQUIRE(dk <= 8 * GLA_CPT, "pico_gla_scan: at most %d key channels a head, got %d", 8 * GLA_CPT, dk);
  PICO_REQUIRE(q_col >= 0 && k_col >= 0 && v_col >= 0 && ldx >= q_col + H * dk && ldx >= k_col + H * dk && ldx >= v_col + H * dv,
               "pico_gla_scan: the row of %d columns does not hold q, k and v", ldx);
  PICO_REQUIRE(H <= 65535 && (dv + 63) / 64 <= 65535 && (dk * dv + 255) / 256 <= 65535, "pico_gla_scan: sizes beyond the grid");
  PICO_REQUIRE(chunk == 0 || (chunk > 0 && max_chunks > 0 && ws != nullptr && ws_decay != nullptr &&
                              (long long)max_chunks * chunk >= T && (long long)num_seqs * max_chunks < (1ll << 31)),
               "pico_gla_scan: chunks need room for their states and must cover the step's tokens");
  if (num_seqs == 0 || T == 0) return 0;
  const int nw = (dk + GLA_CPT - 1) / GLA_CPT;
  // tokens of a block: 16 where the staged values fit (up to 128 key channels), else 8
  const int tb = nw <= 4 ? 16 : 8;
  // value channels a lane: one.  (Two, where a head has more than 64, halve what is read out of LDS for the same
  // arithmetic, but a wave then takes nearly twice as long and half as many fill the chip: 136 against 100 us for the
  // chunks of a 2,048-token prompt with 12 heads of 64 x 128.)
  const int vpl = 1;
  const size_t lds = (size_t)(3 * tb * nw * GLA_CPT + tb * nw * 64 * vpl) * sizeof(float);
  PICO_REQUIRE(lds <= 64 * 1024, "pico_gla_scan: key channels beyond the staging memory");
  const int vb = (dv + 64 * vpl - 1) / (64 * vpl);
#define GLA_ARGS(TT)                                                                                                       \
  (const TT*)x, ldx, q_col, k_col, v_col, log_decay, cu_seqlens, state_slots, state, out, H, dk, dv, qscale, num_slots,   \
      chunk, max_chunks, ws, ws_decay, (const TT*)a2, a2_bias, a_col, R, 1.0f / (tau > 0.f ? tau : 1.f), head_decay
#define GLA_LAUNCH(TT, MODE, GX)                                                                                           \
  do {                                                                                                                     \
    constexpr bool fused = MODE == GLA_WHOLE;     /* with FUSED the launch below is taken only when log_decay is null */ \
    if (log_decay == nullptr && head_decay == nullptr && fused) {                                                                                   \
      if (tb == 16)                                                                                                        \
        gla_scan_kernel<TT, MODE, 16, 1, fused><<<dim3(GX, H, vb), 64 * nw, lds, stream>>>(GLA_ARGS(TT));                  \
      else                                                                                                                 \
        gla_scan_kernel<TT, MODE, 8, 1, fused><<<dim3(GX, H, vb), 64 * nw, lds, stream>>>(GLA_ARGS(TT));                   \
    } else if (tb == 16 && vpl == 2)                                                                                       \
      gla_scan_kernel<TT, MODE, 16, 2, false><<<dim3(GX, H, vb), 64 * nw, lds, stream>>>(GLA_ARGS(TT));                    \
    else if (tb == 16)                                                                                                     \
      gla_scan_kernel<TT, MODE, 16, 1, false><<<dim3(GX, H, vb), 64 * nw, lds, stream>>>(GLA_ARGS(TT));                    \
    else if (vpl == 2)                                                                                                     \
      gla_scan_kernel<TT, MODE, 8, 2, false><<<dim3(GX, H, vb), 64 * nw, lds, stream>>>(GLA_ARGS(TT));                     \
    else                                                                                                                   \
      gla_scan_kernel<TT, MODE, 8, 1, false><<<dim3(GX, H, vb), 64 * nw, lds, stream>>>(GLA_ARGS(TT));                     \
  } while (0)
#define GLA_RUN(TT)                                                                                                        \
  if (chunk == 0) {                                                                                                        \
    GLA_LAUNCH(TT, GLA_WHOLE, num_seqs);                                                                                   \
  } else {                                                                                                                 \
    GLA_LAUNCH(TT, GLA_LOCAL, num_seqs * max_chunks);                                                                      \
    gla_combine_kernel<<<dim3(num_seqs, H, (dk * dv + 255) / 256), 256, 0, stream>>>(cu_seqlens, state_slots, state, ws,   \
                                                                                     ws_decay, H, dk, dv, num_slots, chunk, \
                                                                                     max_chunks);                          \
    GLA_LAUNCH(TT, GLA_FROM, num_seqs * max_chunks);                                                                       \
  }
  if (dtype == PICO_DTYPE_F32) {
    GLA_RUN(float)
  } else if (dtype == PICO_DTYPE_BF16) {
    GLA_RUN(bf16_t)
  } else {
    PICO_REQUIRE(false, "pico_gla_scan: unknown dtype %d", dtype);
  }
#undef GLA_RUN
#undef GLA_LAUNCH
#undef GLA_ARGS
  PICO_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------
// Head norm and gate: out[t][h][v] = o[t][h][v] / sqrt(mean_v(o^2) + eps) * w[v] * silu(g[t][h][v]).
// o float32 [T, H dv]; g: columns of a wider row of type T (stride ldg); out type T [T, H dv].  grid (T, H), one wave.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(64) void gla_out_kernel(const float* __restrict__ o, const T* __restrict__ g, int ldg,
                                                     const float* __restrict__ w, float eps, T* __restrict__ out, int H,
                                                     int dv, int sigmoid_gate) {
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const float* orow = o + ((size_t)t * H + h) * dv;
  float ss = 0.f;
  for (int v = lane; v < dv; v += 64) ss = fmaf(orow[v], orow[v], ss);
  ss = wave_sum(ss);
  const float r = 1.0f / sqrtf(ss / (float)dv + eps);
  const T* grow = g + (size_t)t * ldg + (size_t)h * dv;
  T* dst = out + ((size_t)t * H + h) * dv;
  for (int v = lane; v < dv; v += 64) {
    const float gv = load_f32(grow + v);
    // the gate: silu(g), or sigmoid(g)
    store_f32(dst + v, orow[v] * r * w[v] * ((sigmoid_gate ? 1.0f : gv) / (1.0f + expf(-gv))));
  }
}

extern "C" int pico_gla_out(const float* o, const void* g, int ldg, int dtype, const float* w, float eps, void* out, int T,
                            int H, int dv, int sigmoid_gate, hipStream_t stream) {
  PICO_REQUIRE(T >= 0 && H > 0 && dv > 0 && ldg >= H * dv && H <= 65535, "pico_gla_out: bad sizes");
  if (T == 0) return 0;
  const dim3 grid(T, H);
  if (dtype == PICO_DTYPE_F32)
    gla_out_kernel<float><<<grid, 64, 0, stream>>>(o, (const float*)g, ldg, w, eps, (float*)out, H, dv, sigmoid_gate);
  else if (dtype == PICO_DTYPE_BF16)
    gla_out_kernel<bf16_t><<<grid, 64, 0, stream>>>(o, (const bf16_t*)g, ldg, w, eps, (bf16_t*)out, H, dv, sigmoid_gate);
  else
    PICO_REQUIRE(false, "pico_gla_out: unknown dtype %d", dtype);
  PICO_LAUNCH_CHECK();
  return 0;
}
