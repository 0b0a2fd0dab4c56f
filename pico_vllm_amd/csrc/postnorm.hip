// Norms of a layer that norms what a sublayer RETURNS (x <- x + norm(sublayer(x))), and of the stream itself.
//
//   pico_norm_add:        x[t] += rms(y[t]) * w                          (y: the sublayer's output)
//                         or, with two outputs a and b and a weight each,
//                         x[t] += rms( (rms(a[t]) * wa + rms(b[t]) * wb) / 2 ) * w
//   pico_stream_rmsnorm:  x[t] <- rms(x[t]) * w
//   rms(v) = v / sqrt(mean(v^2) + eps).  Both can leave a copy of the new x in the activations' storage type, which is
//   what the next sublayer reads.
//
// x is the float32 residual stream.  An output may be [T, H] in float32 or bfloat16, or a float32 stack [S, T, H] of
// partial sums of the product that made it, which are added up first (in the order of the stack).  All arithmetic is
// float32; a row's sums run in an order that depends on H alone.  One workgroup a row, the row kept in LDS.
#include "common.h"

#define POSTNORM_MAX_SLABS 8

// The slabs' entries added up in the order of the stack; all loads are issued before the first sum waits for one.
template <typename T>
__device__ __forceinline__ float summed(const T* __restrict__ y, int slabs, size_t slab_stride, size_t at) {
  float part[POSTNORM_MAX_SLABS];
#pragma unroll
  for (int s = 0; s < POSTNORM_MAX_SLABS; s++) part[s] = load_f32(y + (size_t)min(s, slabs - 1) * slab_stride + at);
  float v = part[0];
#pragma unroll
  for (int s = 1; s < POSTNORM_MAX_SLABS; s++) v += s < slabs ? part[s] : 0.f;
  return v;
}

// TA, TB: the types of a and b; TO: the type of the copy.
template <typename TA, typename TB, typename TO>
__global__ __launch_bounds__(1024) void norm_add_kernel(float* __restrict__ x, const TA* __restrict__ a, int a_slabs,
                                                       const float* __restrict__ wa, const TB* __restrict__ b, int b_slabs,
                                                       const float* __restrict__ wb, size_t slab_stride,
                                                       const float* __restrict__ w, float eps, TO* __restrict__ copy, int H) {
  extern __shared__ float row[];          // [H] (and [H] more with b)
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  const size_t base = (size_t)t * H;
  float ss = 0.f;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    const float v = summed(a, a_slabs, slab_stride, base + i);
    row[i] = v;
    ss = fmaf(v, v, ss);
  }
  const float ra = 1.0f / sqrtf(block_sum(ss, scratch) / (float)H + eps);
  if (b) {
    float* rb_row = row + H;
    float sb = 0.f;
    for (int i = threadIdx.x; i < H; i += blockDim.x) {
      const float v = summed(b, b_slabs, slab_stride, base + i);
      rb_row[i] = v;
      sb = fmaf(v, v, sb);
    }
    const float rb = 1.0f / sqrtf(block_sum(sb, scratch) / (float)H + eps);
    float sm = 0.f;
    for (int i = threadIdx.x; i < H; i += blockDim.x) {
      const float v = 0.5f * (row[i] * ra * wa[i] + rb_row[i] * rb * wb[i]);
      row[i] = v;
      sm = fmaf(v, v, sm);
    }
    const float rm = 1.0f / sqrtf(block_sum(sm, scratch) / (float)H + eps);
    for (int i = threadIdx.x; i < H; i += blockDim.x) {
      const float v = x[base + i] + row[i] * rm * w[i];
      x[base + i] = v;
      if (copy) store_f32(copy + base + i, v);
    }
    return;
  }
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    const float v = x[base + i] + row[i] * ra * w[i];
    x[base + i] = v;
    if (copy) store_f32(copy + base + i, v);
  }
}

template <typename TO>
__global__ __launch_bounds__(256) void stream_rmsnorm_kernel(float* __restrict__ x, const float* __restrict__ w, float eps,
                                                             TO* __restrict__ copy, int H) {
  extern __shared__ float row[];
  __shared__ float scratch[16];
  const size_t base = (size_t)blockIdx.x * H;
  float ss = 0.f;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    const float v = x[base + i];
    row[i] = v;
    ss = fmaf(v, v, ss);
  }
  const float r = 1.0f / sqrtf(block_sum(ss, scratch) / (float)H + eps);
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    const float v = row[i] * r * w[i];
    x[base + i] = v;
    if (copy) store_f32(copy + base + i, v);
  }
}

template <typename T>
__global__ __launch_bounds__(256) void cast_rows_kernel(const float* __restrict__ x, T* __restrict__ out, long long n) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) store_f32(out + i, x[i]);
}

#define POSTNORM_MAX_H 16384     // floats of LDS a workgroup may ask for (64 KB)

extern "C" int pico_norm_add(float* x, const void* a, int a_dtype, int a_slabs, const float* wa, const void* b, int b_dtype,
                             int b_slabs, const float* wb, long long slab_stride, const float* w, float eps, void* copy, int copy_dtype,
                             int T, int H, hipStream_t stream) {
  PICO_REQUIRE(T >= 0 && H > 0 && H * (b ? 2 : 1) <= POSTNORM_MAX_H, "pico_norm_add: a width of 1 to %d (half with two outputs), got %d", POSTNORM_MAX_H, H);
  PICO_REQUIRE(a != nullptr && a_slabs >= 1 && (b == nullptr || (b_slabs >= 1 && wa && wb)), "pico_norm_add: bad operands");
  PICO_REQUIRE(a_slabs <= POSTNORM_MAX_SLABS && b_slabs <= POSTNORM_MAX_SLABS, "pico_norm_add: at most %d partial sums an output", POSTNORM_MAX_SLABS);
  PICO_REQUIRE((a_slabs == 1 || a_dtype == PICO_DTYPE_F32) && (b == nullptr || b_slabs == 1 || b_dtype == PICO_DTYPE_F32),
               "pico_norm_add: partial sums are float32");
  if (b == nullptr) b_dtype = a_dtype;
  if (copy == nullptr) copy_dtype = PICO_DTYPE_F32;
  if (T == 0) return 0;
  const size_t lds = (size_t)H * sizeof(float) * (b ? 2 : 1);
  // few rows: as many threads as the row has entries (up to 1,024), so that a thread's loads are one turn and travel
  // together; many rows fill the chip with four waves each
  const int threads = T >= 64 ? 256 : min(1024, max(256, (H + 63) / 64 * 64));
#define LAUNCH(TA, TB, TO)                                                                                                   \
  norm_add_kernel<TA, TB, TO><<<T, threads, lds, stream>>>(x, (const TA*)a, a_slabs, wa, (const TB*)b, b_slabs, wb,              \
                                                       (size_t)slab_stride, w, eps, (TO*)copy, H)
  const int key = (a_dtype == PICO_DTYPE_BF16 ? 4 : 0) | (b_dtype == PICO_DTYPE_BF16 ? 2 : 0) | (copy_dtype == PICO_DTYPE_BF16 ? 1 : 0);
  PICO_REQUIRE((a_dtype | 1) == 1 && (b_dtype | 1) == 1 && (copy_dtype | 1) == 1, "pico_norm_add: unknown dtype");
  switch (key) {
    case 0: LAUNCH(float, float, float); break;
    case 1: LAUNCH(float, float, bf16_t); break;
    case 2: LAUNCH(float, bf16_t, float); break;
    case 3: LAUNCH(float, bf16_t, bf16_t); break;
    case 4: LAUNCH(bf16_t, float, float); break;
    case 5: LAUNCH(bf16_t, float, bf16_t); break;
    case 6: LAUNCH(bf16_t, bf16_t, float); break;
    default: LAUNCH(bf16_t, bf16_t, bf16_t); break;
  }
#undef LAUNCH
  PICO_LAUNCH_CHECK();
  return 0;
}

extern "C" int pico_stream_rmsnorm(float* x, const float* w, float eps, void* copy, int copy_dtype, int T, int H,
                                   hipStream_t stream) {
  PICO_REQUIRE(T >= 0 && H > 0 && H <= POSTNORM_MAX_H, "pico_stream_rmsnorm: a width of 1 to %d, got %d", POSTNORM_MAX_H, H);
  if (T == 0) return 0;
  const size_t lds = (size_t)H * sizeof(float);
  if (copy == nullptr || copy_dtype == PICO_DTYPE_F32)
    stream_rmsnorm_kernel<float><<<T, 256, lds, stream>>>(x, w, eps, (float*)copy, H);
  else if (copy_dtype == PICO_DTYPE_BF16)
    stream_rmsnorm_kernel<bf16_t><<<T, 256, lds, stream>>>(x, w, eps, (bf16_t*)copy, H);
  else
    PICO_REQUIRE(false, "pico_stream_rmsnorm: unknown dtype %d", copy_dtype);
  PICO_LAUNCH_CHECK();
  return 0;
}

extern "C" int pico_cast_rows(const float* x, void* out, int dtype, long long n, hipStream_t stream) {
  PICO_REQUIRE(n >= 0 && dtype == PICO_DTYPE_BF16, "pico_cast_rows: float32 to bfloat16 only");
  if (n == 0) return 0;
  cast_rows_kernel<bf16_t><<<(unsigned)((n + 255) / 256), 256, 0, stream>>>(x, (bf16_t*)out, n);
  PICO_LAUNCH_CHECK();
  return 0;
}
