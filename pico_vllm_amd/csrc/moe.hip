// A routed feed-forward (mixture of experts): the choice of experts and the experts' products.
//
//   scores s = sigmoid(z) of the router logits z (float32); a token's `top` experts are those with the largest z
//   (the lowest index among equal ones), its weights their scores as they are
//   expert e on a row x: g = min(Wg_e x, limit), u = clamp(Wu_e x, -limit, limit),
//                        y = g * sigmoid(alpha g) * (u + 1), out = Wd_e y
//   a token's output: sum over its experts of expert_e(w_e * x)     (the weight scales the expert's INPUT)
//
// A second family (MOE_MODE_SOFTMAX_SWIGLU): scores s = softmax(z) over all router outputs; the `top` largest of
// s + correction are chosen; weights = the chosen s over their sum, times a constant; an expert is
// Wd_e (silu(Wg_e x) * (Wu_e x)) and the weight scales its OUTPUT (here: y, in front of the linear Wd_e); router outputs
// from E on stand for experts that hand their input on unchanged.
//
// Expert matrices are stacked: gate_up [E, 2 F, D] (an expert's gate rows, then its up rows), down [E, D, F].
// This file holds the plain kernels (one wave per output element, any sizes, float32 or bfloat16 storage, every sum
// in float32 and in an order that depends on the sizes alone); the matrix-core kernels for many rows stand behind them.
#include "common.h"

// ---------------------------------------------------------------------------
// Routing: one thread per token.
// ---------------------------------------------------------------------------
#define MOE_MAX_TOP 16

// the `top` largest of a row's E logits z (the lowest index among equal ones) and their sigmoids
__device__ __forceinline__ void route_row(const float* z, int E, int top, int* __restrict__ experts,
                                          float* __restrict__ weights);

__global__ __launch_bounds__(64) void moe_route_kernel(const float* __restrict__ logits, int T, int E, int top,
                                                       int* __restrict__ experts, float* __restrict__ weights) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= T) return;
  route_row(logits + (size_t)t * E, E, top, experts + (size_t)t * top, weights + (size_t)t * top);
}

__device__ __forceinline__ void route_row(const float* z, int E, int top, int* __restrict__ experts,
                                          float* __restrict__ weights) {
  int chosen[MOE_MAX_TOP];
  for (int k = 0; k < top; k++) {
    int best = -1;
    float bz = 0.f;
    for (int e = 0; e < E; e++) {
      bool taken = false;
      for (int j = 0; j < k; j++) taken |= chosen[j] == e;
      if (taken) continue;
      const float v = z[e];
      if (best < 0 || v > bz) { best = e; bz = v; }     // NaN never wins over a number; the first of equals stays
    }
    chosen[k] = best;
    experts[k] = best;
    weights[k] = 1.0f / (1.0f + expf(-bz));
  }
}

// ---------------------------------------------------------------------------
// Router logits z = x Wr^T in float32 (Wr float32 [E, D]; x float32 or bfloat16).  A wave makes one expert's logit of
// ROUTER_TOKENS tokens: its lanes split k (four k a lane and turn where D is a multiple of 4, else one: a chain a lane,
// then the wave's tree, an order that depends on D alone).  grid (ceil(T / ROUTER_TOKENS), ceil(E / 4)).
// ---------------------------------------------------------------------------
#define ROUTER_TOKENS 4

template <typename T> __device__ __forceinline__ void load4_f32(const T* p, float* o);
template <> __device__ __forceinline__ void load4_f32<float>(const float* p, float* o) {
  const float4 v = *reinterpret_cast<const float4*>(p);
  o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w;
}
template <> __device__ __forceinline__ void load4_f32<bf16_t>(const bf16_t* p, float* o) {
  const uint2 v = *reinterpret_cast<const uint2*>(p);
  o[0] = __uint_as_float(v.x << 16); o[1] = __uint_as_float(v.x & 0xffff0000u);
  o[2] = __uint_as_float(v.y << 16); o[3] = __uint_as_float(v.y & 0xffff0000u);
}

template <typename T, bool VEC>
__global__ __launch_bounds__(256) void moe_logits_kernel(const T* __restrict__ x, int ldx, const float* __restrict__ Wr,
                                                         int Tn, int E, int D, float* __restrict__ z) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int t0 = blockIdx.x * ROUTER_TOKENS, e = blockIdx.y * 4 + wave;
  if (e >= E) return;
  const float* w = Wr + (size_t)e * D;
  const T* xr[ROUTER_TOKENS];
  float acc[ROUTER_TOKENS];
#pragma unroll
  for (int i = 0; i < ROUTER_TOKENS; i++) {
    xr[i] = x + (size_t)min(t0 + i, Tn - 1) * ldx;
    acc[i] = 0.f;
  }
  if (VEC) {
#pragma unroll 2
    for (int k = lane * 4; k < D; k += 256) {
      float wv[4], xv[4];
      load4_f32<float>(w + k, wv);
#pragma unroll
      for (int i = 0; i < ROUTER_TOKENS; i++) {
        load4_f32<T>(xr[i] + k, xv);
#pragma unroll
        for (int j = 0; j < 4; j++) acc[i] = fmaf(xv[j], wv[j], acc[i]);
      }
    }
  } else {
    for (int k = lane; k < D; k += 64) {
      const float wv = w[k];
#pragma unroll
      for (int i = 0; i < ROUTER_TOKENS; i++) acc[i] = fmaf(load_f32(xr[i] + k), wv, acc[i]);
    }
  }
#pragma unroll
  for (int i = 0; i < ROUTER_TOKENS; i++) {
    const float s = wave_sum(acc[i]);
    if (lane == 0 && t0 + i < Tn) z[(size_t)(t0 + i) * E + e] = s;
  }
}

// router logits into z [T, E], then the choice: two launches
__global__ void moe_route_softmax_kernel(const float* __restrict__ logits, const float* __restrict__ correction, int T,
                                         int E, int top, float scale, int* __restrict__ experts,
                                         float* __restrict__ weights);

static int moe_router_impl(const void* x, int ldx, int dtype, const float* Wr, int T, int E, int D, int top, float* z,
                           int* experts, float* weights, int softmax, const float* correction, float scale,
                           hipStream_t stream);

extern "C" int pico_moe_router(const void* x, int ldx, int dtype, const float* Wr, int T, int E, int D, int top,
                               float* z, int* experts, float* weights, hipStream_t stream) {
  return moe_router_impl(x, ldx, dtype, Wr, T, E, D, top, z, experts, weights, 0, nullptr, 1.f, stream);
}

// router logits, then the choice by softmax scores plus correction (see moe_route_softmax_kernel)
extern "C" int pico_moe_router_softmax(const void* x, int ldx, int dtype, const float* Wr, const float* correction, int T,
                                       int E, int D, int top, float scale, float* z, int* experts, float* weights,
                                       hipStream_t stream) {
  return moe_router_impl(x, ldx, dtype, Wr, T, E, D, top, z, experts, weights, 1, correction, scale, stream);
}

static int moe_router_impl(const void* x, int ldx, int dtype, const float* Wr, int T, int E, int D, int top, float* z,
                           int* experts, float* weights, int softmax, const float* correction, float scale,
                           hipStream_t stream) {
  PICO_REQUIRE(T >= 0 && E > 0 && D > 0 && ldx >= D && top > 0 && top <= E && top <= MOE_MAX_TOP,
               "pico_moe_router: %d of %d experts per token is outside what the kernel takes (at most %d)", top, E, MOE_MAX_TOP);
  PICO_REQUIRE(dtype == PICO_DTYPE_F32 || dtype == PICO_DTYPE_BF16, "pico_moe_router: unknown dtype %d", dtype);
  if (T == 0) return 0;
  const dim3 grid((T + ROUTER_TOKENS - 1) / ROUTER_TOKENS, (E + 3) / 4);
  PICO_REQUIRE(grid.y <= 65535, "pico_moe_router: too many experts");
  const size_t esz = dtype == PICO_DTYPE_F32 ? 4 : 2;
  const bool vec = D % 4 == 0 && ldx % 4 == 0 && (uintptr_t)x % (4 * esz) == 0 && (uintptr_t)Wr % 16 == 0;
#define LAUNCH(TT, V) moe_logits_kernel<TT, V><<<grid, 256, 0, stream>>>((const TT*)x, ldx, Wr, T, E, D, z)
  if (dtype == PICO_DTYPE_F32) { if (vec) LAUNCH(float, true); else LAUNCH(float, false); }
  else { if (vec) LAUNCH(bf16_t, true); else LAUNCH(bf16_t, false); }
#undef LAUNCH
  if (softmax)
    moe_route_softmax_kernel<<<(T + 3) / 4, 256, 0, stream>>>(z, correction, T, E, top, scale, experts, weights);
  else
    moe_route_kernel<<<(T + 63) / 64, 64, 0, stream>>>(z, T, E, top, experts, weights);
  PICO_LAUNCH_CHECK();
  return 0;
}

extern "C" int pico_moe_route(const float* logits, int T, int E, int top, int* experts, float* weights,
                              hipStream_t stream) {
  PICO_REQUIRE(T >= 0 && E > 0 && top > 0 && top <= E && top <= MOE_MAX_TOP,
               "pico_moe_route: %d of %d experts per token is outside what the kernel takes (at most %d)", top, E, MOE_MAX_TOP);
  if (T == 0) return 0;
  moe_route_kernel<<<(T + 63) / 64, 64, 0, stream>>>(logits, T, E, top, experts, weights);
  PICO_LAUNCH_CHECK();
  return 0;
}

#define MOE_MODE_CLIPPED 0
#define MOE_MODE_SOFTMAX_SWIGLU 1

// mode 0: the clipped activation, the row's weight w already in the input; mode 1: w silu(g) u
__device__ __forceinline__ float expert_act(float g, float u, float limit, float alpha, int mode, float w) {
  if (mode == MOE_MODE_SOFTMAX_SWIGLU) return w * (g / (1.0f + expf(-g))) * u;
  g = fminf(g, limit);
  u = fminf(fmaxf(u, -limit), limit);
  return g / (1.0f + expf(-alpha * g)) * (u + 1.0f);
}

// ---------------------------------------------------------------------------
// Choice by softmax scores with a correction: one wave per token, lane l looks after router outputs l, l + 64, ...
// z [T, E] float32 router logits (E counts every router output); correction [E] or null.  Sums and maxima run over the
// wave in a fixed order; among equal choice scores the lowest output wins.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void moe_route_softmax_kernel(const float* __restrict__ logits,
                                                                const float* __restrict__ correction, int T, int E, int top,
                                                                float scale, int* __restrict__ experts,
                                                                float* __restrict__ weights) {
  const int t = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (t >= T) return;
  const float* z = logits + (size_t)t * E;
  float mx = -INFINITY;
  for (int e = lane; e < E; e += 64) mx = fmaxf(mx, z[e]);
  mx = wave_max(mx);
  float den = 0.f;
  for (int e = lane; e < E; e += 64) den += expf(z[e] - mx);
  const float inv = 1.0f / wave_sum(den);
  int chosen[MOE_MAX_TOP];
  float score[MOE_MAX_TOP];
  float total = 0.f;
  for (int k = 0; k < top; k++) {
    float bc = -INFINITY;
    int best = 0x7fffffff;
    for (int e = lane; e < E; e += 64) {
      bool taken = false;
      for (int j = 0; j < k; j++) taken |= chosen[j] == e;
      if (taken) continue;
      const float c = expf(z[e] - mx) * inv + (correction ? correction[e] : 0.f);
      if (c > bc || best == 0x7fffffff) { best = e; bc = c; }     // a lane's outputs come in ascending order: the first of equals stays
    }
    wave_first_max(bc, best);
    chosen[k] = best;
    score[k] = expf(z[min(best, E - 1)] - mx) * inv;
    total += score[k];
  }
  const float f = scale / (total + 1e-20f);
  if (lane < top) {
    // (chosen and score are the same in every lane)
    for (int k = 0; k < top; k++)
      if (k == lane) {
        experts[(size_t)t * top + k] = chosen[k];
        weights[(size_t)t * top + k] = score[k] * f;
      }
  }
}

// ---------------------------------------------------------------------------
// Router outputs from E on are experts that hand their input on: for every (token, slot) with such an expert,
// stacked: out[slot][t][:] = w h[t][:] (the slab rows that no expert's product writes); else out[t][:] += w h[t][:].
// grid (T).
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void moe_identity_kernel(const T* __restrict__ h, int ldh, const int* __restrict__ experts,
                                                           const float* __restrict__ weights, float* __restrict__ out,
                                                           int Tn, int top, int E, int D, int stacked) {
  const int t = blockIdx.x;
  const T* x = h + (size_t)t * ldh;
  if (stacked) {
    for (int k = 0; k < top; k++) {
      if (experts[(size_t)t * top + k] < E) continue;
      const float w = weights[(size_t)t * top + k];
      float* o = out + ((size_t)k * Tn + t) * D;
      for (int j = threadIdx.x; j < D; j += blockDim.x) o[j] = w * load_f32(x + j);
    }
    return;
  }
  float w = 0.f;
  for (int k = 0; k < top; k++)
    if (experts[(size_t)t * top + k] >= E) w += weights[(size_t)t * top + k];
  if (w == 0.f) return;
  float* o = out + (size_t)t * D;
  for (int j = threadIdx.x; j < D; j += blockDim.x) o[j] = fmaf(w, load_f32(x + j), o[j]);
}

extern "C" int pico_moe_identity(const void* h, int ldh, int dtype, const int* experts, const float* weights, float* out,
                                 int T, int top, int E, int D, int stacked, hipStream_t stream) {
  PICO_REQUIRE(T >= 0 && top > 0 && E >= 0 && D > 0 && ldh >= D, "pico_moe_identity: bad sizes");
  if (T == 0) return 0;
  if (dtype == PICO_DTYPE_F32)
    moe_identity_kernel<float><<<T, 256, 0, stream>>>((const float*)h, ldh, experts, weights, out, T, top, E, D, stacked);
  else if (dtype == PICO_DTYPE_BF16)
    moe_identity_kernel<bf16_t><<<T, 256, 0, stream>>>((const bf16_t*)h, ldh, experts, weights, out, T, top, E, D, stacked);
  else
    PICO_REQUIRE(false, "pico_moe_identity: unknown dtype %d", dtype);
  PICO_LAUNCH_CHECK();
  return 0;
}

// the input of an expert: the token's row times its weight, rounded to the storage type as a product's operand is
template <typename T> __device__ __forceinline__ float scaled_input(const T* p, float w);
template <> __device__ __forceinline__ float scaled_input<float>(const float* p, float w) { return *p * w; }
template <> __device__ __forceinline__ float scaled_input<bf16_t>(const bf16_t* p, float w) {
  return bf16_to_f32(f32_to_bf16(bf16_to_f32(*p) * w));
}

// ---------------------------------------------------------------------------
// Plain first half: y[r, f] = act(gate_e[f] . x, up_e[f] . x) for row r = (token, slot), x = w_r * h[token].
// grid (rows, ceil(F / 16)); four waves, each four outputs; the lanes of a wave split k.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void moe_up_plain_kernel(const T* __restrict__ h, int ldh, const T* __restrict__ gate_up,
                                                           const int* __restrict__ experts, const float* __restrict__ weights,
                                                           T* __restrict__ y, int top, int E, int F, int D, float limit,
                                                           float alpha, int mode) {
  const int r = blockIdx.x, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int e = experts[r];
  if (e < 0 || e >= E) return;
  const float wr = weights[r];
  const float w = mode == MOE_MODE_SOFTMAX_SWIGLU ? 1.f : wr;
  const T* x = h + (size_t)(r / top) * ldh;
  const T* We = gate_up + (size_t)e * 2 * F * D;
  for (int i = 0; i < 4; i++) {
    const int f = blockIdx.y * 16 + wave * 4 + i;
    if (f >= F) break;
    const T* wg = We + (size_t)f * D;
    const T* wu = We + (size_t)(F + f) * D;
    float g = 0.f, u = 0.f;
    for (int j = lane; j < D; j += 64) {
      const float xv = mode == MOE_MODE_SOFTMAX_SWIGLU ? load_f32(x + j) : scaled_input<T>(x + j, w);
      g = fmaf(load_f32(wg + j), xv, g);
      u = fmaf(load_f32(wu + j), xv, u);
    }
    g = wave_sum(g);
    u = wave_sum(u);
    if (lane == 0) store_f32(y + (size_t)r * F + f, expert_act(g, u, limit, alpha, mode, wr));
  }
}

// ---------------------------------------------------------------------------
// Plain second half: out[t, n] = sum over the token's slots (in slot order) of down_e[n] . y[(t, slot)], float32.
// grid (tokens, ceil(D / 16)).
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void moe_down_plain_kernel(const T* __restrict__ y, const T* __restrict__ down,
                                                             const int* __restrict__ experts, float* __restrict__ out,
                                                             int top, int E, int F, int D) {
  const int t = blockIdx.x, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  for (int i = 0; i < 4; i++) {
    const int n = blockIdx.y * 16 + wave * 4 + i;
    if (n >= D) break;
    float total = 0.f;
    for (int k = 0; k < top; k++) {
      const int r = t * top + k, e = experts[r];
      if (e < 0 || e >= E) continue;
      const T* wd = down + ((size_t)e * D + n) * F;
      const T* yr = y + (size_t)r * F;
      float s = 0.f;
      for (int j = lane; j < F; j += 64) s = fmaf(load_f32(wd + j), load_f32(yr + j), s);
      total += wave_sum(s);
    }
    if (lane == 0) out[(size_t)t * D + n] = total;
  }
}

extern "C" int pico_moe_experts_plain(const void* h, int ldh, int dtype, const void* gate_up, const void* down,
                                      const int* experts, const float* weights, void* y, float* out, int T, int top,
                                      int E, int F, int D, float limit, float alpha, int mode, hipStream_t stream) {
  PICO_REQUIRE(T >= 0 && top > 0 && E > 0 && F > 0 && D > 0 && ldh >= D, "pico_moe_experts_plain: bad sizes");
  PICO_REQUIRE(mode == MOE_MODE_CLIPPED || mode == MOE_MODE_SOFTMAX_SWIGLU, "pico_moe_experts_plain: unknown mode %d", mode);
  if (T == 0) return 0;
  const dim3 g1(T * top, (F + 15) / 16), g2(T, (D + 15) / 16);
  PICO_REQUIRE(g1.y <= 65535 && g2.y <= 65535, "pico_moe_experts_plain: sizes beyond the grid");
  if (dtype == PICO_DTYPE_F32) {
    moe_up_plain_kernel<float><<<g1, 256, 0, stream>>>((const float*)h, ldh, (const float*)gate_up, experts, weights,
                                                       (float*)y, top, E, F, D, limit, alpha, mode);
    moe_down_plain_kernel<float><<<g2, 256, 0, stream>>>((const float*)y, (const float*)down, experts, out, top, E, F, D);
  } else if (dtype == PICO_DTYPE_BF16) {
    moe_up_plain_kernel<bf16_t><<<g1, 256, 0, stream>>>((const bf16_t*)h, ldh, (const bf16_t*)gate_up, experts, weights,
                                                        (bf16_t*)y, top, E, F, D, limit, alpha, mode);
    moe_down_plain_kernel<bf16_t><<<g2, 256, 0, stream>>>((const bf16_t*)y, (const bf16_t*)down, experts, out, top, E, F, D);
  } else {
    PICO_REQUIRE(false, "pico_moe_experts_plain: unknown dtype %d", dtype);
  }
  PICO_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------
// A third way of choosing: logits z = x Wr^T + bias; the `top` largest logits are chosen (the lowest index among equal
// ones) and the weights are the softmax over the chosen logits only.  Wr may hold `extra` rows behind the E experts'
// whose logits are made in the same launch and take no part in the choice (a gate of the layer, say): z is
// [T, E + extra], and what the choice reads of it has the bias added.
// ---------------------------------------------------------------------------
// A wave a token, four tokens a workgroup; lane l looks after logits l, l + 64, ..: it keeps them (bias added) in LDS,
// where it alone reads and writes them, so the waves never wait for one another.
__global__ __launch_bounds__(256) void moe_route_top_softmax_kernel(float* __restrict__ z, const float* __restrict__ bias,
                                                                    int T, int E, int ldz, int top,
                                                                    int* __restrict__ experts, float* __restrict__ weights) {
  extern __shared__ float zs[];                          // [4][E]
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, t = blockIdx.x * 4 + wave;
  if (t >= T) return;
  float* row = z + (size_t)t * ldz;
  float* mine = zs + (size_t)wave * E;
  for (int e = lane; e < E; e += 64) {
    const float v = row[e] + (bias ? bias[e] : 0.f);
    row[e] = v;
    mine[e] = v;
  }
  float wk = 0.f, largest = 0.f, sum = 0.f;              // lane k keeps the k-th chosen logit's weight
  int ek = 0;
  for (int k = 0; k < top; k++) {
    float mx = -INFINITY;
    int mi = 0x7fffffff;
    for (int e = lane; e < E; e += 64) {
      const float v = mine[e];
      if (v > mx || mi == 0x7fffffff) { mx = v; mi = e; }      // the first of equals stays; NaN never wins over a number
    }
    wave_first_max(mx, mi);                              // the lowest index among equal values, in every lane
    if (k == 0) largest = mx;
    const float w = expf(mx - largest);
    sum += w;
    if (lane == k) { wk = w; ek = mi; }
    if ((mi & 63) == lane) mine[mi] = -INFINITY;         // taken
  }
  if (lane < top) {
    experts[(size_t)t * top + lane] = ek;
    weights[(size_t)t * top + lane] = wk / sum;
  }
}

extern "C" int pico_moe_router_top_softmax(const void* x, int ldx, int dtype, const float* Wr, const float* bias, int T,
                                           int E, int extra, int D, int top, float* z, int* experts, float* weights,
                                           hipStream_t stream) {
  PICO_REQUIRE(T >= 0 && E > 0 && extra >= 0 && D > 0 && ldx >= D && top > 0 && top <= E && top <= MOE_MAX_TOP,
               "pico_moe_router_top_softmax: %d of %d experts per token is outside what the kernel takes (at most %d)", top, E, MOE_MAX_TOP);
  PICO_REQUIRE(dtype == PICO_DTYPE_F32 || dtype == PICO_DTYPE_BF16, "pico_moe_router_top_softmax: unknown dtype %d", dtype);
  if (T == 0) return 0;
  const int rows = E + extra;
  const dim3 grid((T + ROUTER_TOKENS - 1) / ROUTER_TOKENS, (rows + 3) / 4);
  PICO_REQUIRE(grid.y <= 65535, "pico_moe_router_top_softmax: too many experts");
  const size_t esz = dtype == PICO_DTYPE_F32 ? 4 : 2;
  const bool vec = D % 4 == 0 && ldx % 4 == 0 && (uintptr_t)x % (4 * esz) == 0 && (uintptr_t)Wr % 16 == 0;
#define LAUNCH(TT, V) moe_logits_kernel<TT, V><<<grid, 256, 0, stream>>>((const TT*)x, ldx, Wr, T, rows, D, z)
  if (dtype == PICO_DTYPE_F32) { if (vec) LAUNCH(float, true); else LAUNCH(float, false); }
  else { if (vec) LAUNCH(bf16_t, true); else LAUNCH(bf16_t, false); }
#undef LAUNCH
  PICO_REQUIRE(E <= 8192, "pico_moe_router_top_softmax: at most 8192 experts");
  moe_route_top_softmax_kernel<<<(T + 3) / 4, 256, (size_t)4 * E * sizeof(float), stream>>>(z, bias, T, E, rows, top, experts, weights);
  PICO_LAUNCH_CHECK();
  return 0;
}
