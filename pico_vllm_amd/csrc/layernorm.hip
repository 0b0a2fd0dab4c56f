// Layer norm with weight and bias, with the residual sum in front of it, and a sum into the residual stream whose
// addend is scaled element by element.
//
//   x = resid[row] (+ scale * (delta_0[row] + delta_1[row] + ..))          scale: a vector [H], or none (ones)
//   out = (x - mean(x)) / sqrt(mean((x - mean)^2) + eps) * w + b
//
// Everything in float32; the variance from the deviations (two passes over a row kept in LDS).
#include "common.h"

#define LN_MAX_SLABS 16

// One workgroup a row.  VEC: four elements a thread and turn with 16-byte accesses (H a multiple of 4, everything
// aligned); the row is kept in LDS between the passes.
template <typename TD> __device__ __forceinline__ float4 ln_load4(const TD* p);
template <> __device__ __forceinline__ float4 ln_load4<float>(const float* p) { return *reinterpret_cast<const float4*>(p); }
template <> __device__ __forceinline__ float4 ln_load4<bf16_t>(const bf16_t* p) {
  const uint2 v = *reinterpret_cast<const uint2*>(p);
  return make_float4(__uint_as_float(v.x << 16), __uint_as_float(v.x & 0xffff0000u), __uint_as_float(v.y << 16),
                     __uint_as_float(v.y & 0xffff0000u));
}
template <typename TO> __device__ __forceinline__ void ln_store4(TO* p, float4 v);
template <> __device__ __forceinline__ void ln_store4<float>(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
template <> __device__ __forceinline__ void ln_store4<bf16_t>(bf16_t* p, float4 v) {
  *reinterpret_cast<uint2*>(p) = make_uint2(pack2_bf16(v.x, v.y), pack2_bf16(v.z, v.w));
}

template <typename TD, typename TO, bool VEC>
__global__ __launch_bounds__(1024) void add_layernorm_kernel(float* __restrict__ resid, const TD* __restrict__ delta, int slabs,
                                                             size_t slab_stride, const float* __restrict__ dscale,
                                                             const float* __restrict__ w, const float* __restrict__ b,
                                                             TO* __restrict__ out, const int* __restrict__ rows, int H,
                                                             float eps) {
  extern __shared__ float xs[];          // [H] the row, then 16 floats of scratch
  float* scratch = xs + H;
  const int row = rows ? rows[blockIdx.x] : blockIdx.x;
  float* x = resid + (size_t)row * H;
  const TD* dl = delta ? delta + (size_t)row * H : nullptr;
  TO* o = out + (size_t)blockIdx.x * H;
  float s = 0.f;
  if (VEC) {
    for (int i = threadIdx.x * 4; i < H; i += blockDim.x * 4) {
      float4 v = *reinterpret_cast<const float4*>(x + i);
      if (dl) {
        float4 d = ln_load4<TD>(dl + i);
        for (int k = 1; k < slabs; k++) {
          const float4 e = ln_load4<TD>(dl + k * slab_stride + i);
          d.x += e.x; d.y += e.y; d.z += e.z; d.w += e.w;
        }
        if (dscale) {
          const float4 c = *reinterpret_cast<const float4*>(dscale + i);
          d.x *= c.x; d.y *= c.y; d.z *= c.z; d.w *= c.w;
        }
        v.x += d.x; v.y += d.y; v.z += d.z; v.w += d.w;
        if (!rows) *reinterpret_cast<float4*>(x + i) = v;
      }
      *reinterpret_cast<float4*>(xs + i) = v;
      s += (v.x + v.y) + (v.z + v.w);
    }
  } else {
    for (int i = threadIdx.x; i < H; i += blockDim.x) {
      float v = x[i];
      if (dl) {
        float d = load_f32(dl + i);
        for (int k = 1; k < slabs; k++) d += load_f32(dl + k * slab_stride + i);
        v += dscale ? dscale[i] * d : d;
        if (!rows) x[i] = v;
      }
      xs[i] = v;
      s += v;
    }
  }
  const float mean = block_sum(s, scratch) / (float)H;
  float q = 0.f;
  if (VEC) {
    for (int i = threadIdx.x * 4; i < H; i += blockDim.x * 4) {
      const float4 v = *reinterpret_cast<const float4*>(xs + i);
      const float d0 = v.x - mean, d1 = v.y - mean, d2 = v.z - mean, d3 = v.w - mean;
      q += (d0 * d0 + d1 * d1) + (d2 * d2 + d3 * d3);
    }
  } else {
    for (int i = threadIdx.x; i < H; i += blockDim.x) {
      const float d = xs[i] - mean;
      q = fmaf(d, d, q);
    }
  }
  const float r = 1.0f / sqrtf(block_sum(q, scratch) / (float)H + eps);
  if (VEC) {
    for (int i = threadIdx.x * 4; i < H; i += blockDim.x * 4) {
      const float4 v = *reinterpret_cast<const float4*>(xs + i);
      const float4 g = *reinterpret_cast<const float4*>(w + i), c = *reinterpret_cast<const float4*>(b + i);
      ln_store4<TO>(o + i, make_float4((v.x - mean) * r * g.x + c.x, (v.y - mean) * r * g.y + c.y, (v.z - mean) * r * g.z + c.z,
                                       (v.w - mean) * r * g.w + c.w));
    }
  } else {
    for (int i = threadIdx.x; i < H; i += blockDim.x) store_f32(o + i, (xs[i] - mean) * r * w[i] + b[i]);
  }
}

extern "C" int pico_add_layernorm(float* resid, const void* delta, int delta_dtype, int slabs, long long slab_stride,
                                  const float* dscale, const float* w, const float* b, void* out, int out_dtype,
                                  const int* rows, int T, int H, float eps, hipStream_t stream) {
  PICO_REQUIRE(T >= 0 && H > 0 && H <= 15360, "pico_add_layernorm: bad sizes T=%d H=%d (a row of at most 15360)", T, H);
  PICO_REQUIRE(slabs >= 1 && slabs <= LN_MAX_SLABS && slab_stride >= 0, "pico_add_layernorm: 1 to %d slabs, got %d", LN_MAX_SLABS, slabs);
  PICO_REQUIRE(eps > 0.f && w != nullptr && b != nullptr, "pico_add_layernorm: eps must be positive, weight and bias given");
  if (T == 0) return 0;
  const size_t lds = (size_t)(H + 16) * sizeof(float);
  const bool vec = H % 4 == 0 && slab_stride % 4 == 0 && (uintptr_t)resid % 16 == 0 && (uintptr_t)delta % 16 == 0 &&
                   (uintptr_t)dscale % 16 == 0 && (uintptr_t)w % 16 == 0 && (uintptr_t)b % 16 == 0 && (uintptr_t)out % 16 == 0;
  const int threads = vec ? min(1024, max(64, (H / 4 + 63) / 64 * 64)) : min(1024, max(64, (H + 63) / 64 * 64));
#define LAUNCH(TD, TO)                                                                                                    \
  do {                                                                                                                    \
    if (vec)                                                                                                              \
      add_layernorm_kernel<TD, TO, true><<<T, threads, lds, stream>>>(resid, (const TD*)delta, slabs, (size_t)slab_stride, \
                                                                      dscale, w, b, (TO*)out, rows, H, eps);              \
    else                                                                                                                  \
      add_layernorm_kernel<TD, TO, false><<<T, threads, lds, stream>>>(resid, (const TD*)delta, slabs, (size_t)slab_stride, \
                                                                       dscale, w, b, (TO*)out, rows, H, eps);             \
  } while (0)
  if (delta_dtype == PICO_DTYPE_F32 && out_dtype == PICO_DTYPE_F32) LAUNCH(float, float);
  else if (delta_dtype == PICO_DTYPE_BF16 && out_dtype == PICO_DTYPE_BF16) LAUNCH(bf16_t, bf16_t);
  else if (delta_dtype == PICO_DTYPE_F32 && out_dtype == PICO_DTYPE_BF16) LAUNCH(float, bf16_t);
  else if (delta_dtype == PICO_DTYPE_BF16 && out_dtype == PICO_DTYPE_F32) LAUNCH(bf16_t, float);
  else PICO_REQUIRE(false, "pico_add_layernorm: unknown dtypes %d %d", delta_dtype, out_dtype);
#undef LAUNCH
  PICO_LAUNCH_CHECK();
  return 0;
}

// resid[t][i] += scale[i] * (a_0[t][i] + a_1[t][i] + .. + sigmoid(gate[t * gate_stride]) * b[t][i])
// a: `slabs` addends of type TA (or none); b of type TB with a gate logit per row (or none; no gate: b as it is);
// scale [H] or none.
template <typename TA, typename TB>
__global__ __launch_bounds__(256) void scaled_add_kernel(float* __restrict__ resid, const TA* __restrict__ a, int slabs,
                                                         size_t slab_stride, const TB* __restrict__ b,
                                                         const float* __restrict__ gate, int gate_stride,
                                                         const float* __restrict__ scale, int H, size_t n) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int col = (int)(i % H);
  float d = 0.f;
  if (a) {
    d = load_f32(a + i);
    for (int k = 1; k < slabs; k++) d += load_f32(a + k * slab_stride + i);
  }
  if (b) {
    float bv = load_f32(b + i);
    if (gate) bv *= 1.0f / (1.0f + expf(-gate[(i / H) * (size_t)gate_stride]));
    d += bv;
  }
  resid[i] += scale ? scale[col] * d : d;
}

extern "C" int pico_scaled_add(float* resid, const void* a, int a_dtype, int slabs, long long slab_stride, const void* b,
                               int b_dtype, const float* gate, int gate_stride, const float* scale, int T, int H,
                               hipStream_t stream) {
  PICO_REQUIRE(T >= 0 && H > 0 && slabs >= 1 && slab_stride >= 0, "pico_scaled_add: bad sizes");
  PICO_REQUIRE(a != nullptr || b != nullptr, "pico_scaled_add: nothing to add");
  if (T == 0) return 0;
  const size_t n = (size_t)T * H;
  const unsigned grid = (unsigned)((n + 255) / 256);
#define LAUNCH(TA, TB)                                                                                               \
  scaled_add_kernel<TA, TB><<<grid, 256, 0, stream>>>(resid, (const TA*)a, slabs, (size_t)slab_stride, (const TB*)b, \
                                                      gate, gate_stride, scale, H, n)
  const int ad = a ? a_dtype : PICO_DTYPE_F32, bd = b ? b_dtype : PICO_DTYPE_F32;
  if (ad == PICO_DTYPE_F32 && bd == PICO_DTYPE_F32) LAUNCH(float, float);
  else if (ad == PICO_DTYPE_F32 && bd == PICO_DTYPE_BF16) LAUNCH(float, bf16_t);
  else if (ad == PICO_DTYPE_BF16 && bd == PICO_DTYPE_F32) LAUNCH(bf16_t, float);
  else if (ad == PICO_DTYPE_BF16 && bd == PICO_DTYPE_BF16) LAUNCH(bf16_t, bf16_t);
  else PICO_REQUIRE(false, "pico_scaled_add: unknown dtypes %d %d", a_dtype, b_dtype);
#undef LAUNCH
  PICO_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------
// An embedding of token pairs on the residual stream: resid[t] += table[row(t)],
//   row = (previous token * mul_prev + token * mul_cur) mod buckets,    or `buckets` (the table's last row) at position 0.
// The previous token of a portion's first token is what the sequence's state slot holds (last[slot]); a second launch
// writes every sequence's last token of this step there (after all reads: a launch of its own).
// ---------------------------------------------------------------------------
template <typename TT>
__global__ __launch_bounds__(256) void pair_embed_kernel(float* __restrict__ resid, const TT* __restrict__ table,
                                                         const int* __restrict__ tokens, const int* __restrict__ positions,
                                                         const int* __restrict__ token_seq, const int* __restrict__ cu_seqlens,
                                                         const int* __restrict__ state_slots, const int* __restrict__ last,
                                                         int num_slots, long long mul_prev, long long mul_cur, int buckets, int H) {
  const int t = blockIdx.x;
  int row = buckets;
  if (positions[t] > 0) {
    const int b = token_seq[t];
    int prev;
    if (t > cu_seqlens[b]) prev = tokens[t - 1];
    else {
      const int slot = state_slots[b];
      prev = (slot >= 0 && slot < num_slots) ? last[slot] : 0;
    }
    long long r = ((long long)prev * mul_prev + (long long)tokens[t] * mul_cur) % buckets;
    if (r < 0) r += buckets;
    row = (int)r;
  }
  const TT* src = table + (size_t)row * H;
  float* x = resid + (size_t)t * H;
  for (int i = threadIdx.x; i < H; i += blockDim.x) x[i] += load_f32(src + i);
}

__global__ void last_token_kernel(const int* __restrict__ tokens, const int* __restrict__ cu_seqlens,
                                  const int* __restrict__ state_slots, int* __restrict__ last, int num_slots, int B) {
  const int b = blockIdx.x * blockDim.x + threadIdx.x;
  if (b >= B) return;
  const int lo = cu_seqlens[b], hi = cu_seqlens[b + 1], slot = state_slots[b];
  if (hi > lo && slot >= 0 && slot < num_slots) last[slot] = tokens[hi - 1];
}

extern "C" int pico_pair_embed(float* resid, const void* table, int dtype, const int* tokens, const int* positions,
                               const int* token_seq, const int* cu_seqlens, const int* state_slots, int* last,
                               int num_slots, long long mul_prev, long long mul_cur, int buckets, int T, int B, int H,
                               hipStream_t stream) {
  PICO_REQUIRE(T >= 0 && B >= 0 && H > 0 && buckets > 0 && num_slots > 0, "pico_pair_embed: bad sizes");
  if (T == 0 || B == 0) return 0;
  if (dtype == PICO_DTYPE_F32)
    pair_embed_kernel<float><<<T, 256, 0, stream>>>(resid, (const float*)table, tokens, positions, token_seq, cu_seqlens,
                                                    state_slots, last, num_slots, mul_prev, mul_cur, buckets, H);
  else if (dtype == PICO_DTYPE_BF16)
    pair_embed_kernel<bf16_t><<<T, 256, 0, stream>>>(resid, (const bf16_t*)table, tokens, positions, token_seq, cu_seqlens,
                                                     state_slots, last, num_slots, mul_prev, mul_cur, buckets, H);
  else
    PICO_REQUIRE(false, "pico_pair_embed: unknown dtype %d", dtype);
  last_token_kernel<<<(B + 63) / 64, 64, 0, stream>>>(tokens, cu_seqlens, state_slots, last, num_slots, B);
  PICO_LAUNCH_CHECK();
  return 0;
}
