// Attention through low-rank latents: what stands between the down projections and the attention kernel.
//
// A row of the first product holds [query latent (q_rank) | key/value latent (kv_rank) | rotated key part (rot)].
//   cq = rmsnorm(query latent) * wq                      -> its own tensor, for the queries' up projection
//   c  = rmsnorm(key/value latent) * wkv
//   kr = the rotated key part turned by the token's angles (neighbouring pairs)
// The cache keeps per token the key row [c | kr] (one kv head of size kv_rank + rot) and c again as the value column
// (V pages are [dv, page]), so that the attention kernels of this package serve it as attention with one kv head:
// a head's query is [its unrotated query times its key matrix (kv_rank) | its rotated query (rot)], and a head's
// output in the latent's space goes through its value matrix afterwards.
// Norms and rotation are float32.
#include "common.h"

template <typename T>
__global__ __launch_bounds__(256) void latent_prepare_kernel(const T* __restrict__ y, int ldy, int q_rank, int kv_rank,
                                                             int rot, const float* __restrict__ wq,
                                                             const float* __restrict__ wkv, float eps,
                                                             const float* __restrict__ cos_sin,
                                                             const int* __restrict__ slots, T* __restrict__ cq,
                                                             T* __restrict__ k_cache, T* __restrict__ v_cache, int P,
                                                             int num_pages) {
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  const T* row = y + (size_t)t * ldy;
  float ss = 0.f;
  for (int i = threadIdx.x; i < q_rank; i += blockDim.x) { const float v = load_f32(row + i); ss = fmaf(v, v, ss); }
  const float rq = 1.0f / sqrtf(block_sum(ss, scratch) / (float)q_rank + eps);
  for (int i = threadIdx.x; i < q_rank; i += blockDim.x) store_f32(cq + (size_t)t * q_rank + i, load_f32(row + i) * rq * wq[i]);
  const int slot = slots[t];
  if (slot < 0 || slot >= num_pages * P) return;        // a token that keeps nothing (padding of a recorded step)
  const T* lat = row + q_rank;
  ss = 0.f;
  for (int i = threadIdx.x; i < kv_rank; i += blockDim.x) { const float v = load_f32(lat + i); ss = fmaf(v, v, ss); }
  const float rk = 1.0f / sqrtf(block_sum(ss, scratch) / (float)kv_rank + eps);
  const int page = slot / P, off = slot % P, dk = kv_rank + rot;
  T* kdst = k_cache + ((size_t)page * P + off) * dk;
  T* vdst = v_cache + (size_t)page * kv_rank * P + off;
  for (int i = threadIdx.x; i < kv_rank; i += blockDim.x) {
    const float c = load_f32(lat + i) * rk * wkv[i];
    store_f32(kdst + i, c);
    store_f32(vdst + (size_t)i * P, c);
  }
  const float* cs = cos_sin + (size_t)t * rot;           // [rot / 2][cos, sin]
  for (int i = threadIdx.x; i < rot / 2; i += blockDim.x) {
    const float u = load_f32(lat + kv_rank + 2 * i), v = load_f32(lat + kv_rank + 2 * i + 1);
    const float c = cs[2 * i], s = cs[2 * i + 1];
    store_f32(kdst + kv_rank + 2 * i, u * c - v * s);
    store_f32(kdst + kv_rank + 2 * i + 1, v * c + u * s);
  }
}

extern "C" int pico_latent_prepare(const void* y, int ldy, int dtype, int q_rank, int kv_rank, int rot, const float* wq,
                                   const float* wkv, float eps, const float* cos_sin, const int* slots, void* cq,
                                   void* k_cache, void* v_cache, int T, int P, int num_pages, hipStream_t stream) {
  PICO_REQUIRE(T >= 0 && q_rank > 0 && kv_rank > 0 && rot >= 0 && rot % 2 == 0 && ldy >= q_rank + kv_rank + rot && P > 0 && num_pages > 0,
               "pico_latent_prepare: bad sizes");
  PICO_REQUIRE(eps > 0.f, "pico_latent_prepare: eps must be positive");
  if (T == 0) return 0;
  if (dtype == PICO_DTYPE_F32)
    latent_prepare_kernel<float><<<T, 256, 0, stream>>>((const float*)y, ldy, q_rank, kv_rank, rot, wq, wkv, eps, cos_sin,
                                                        slots, (float*)cq, (float*)k_cache, (float*)v_cache, P, num_pages);
  else if (dtype == PICO_DTYPE_BF16)
    latent_prepare_kernel<bf16_t><<<T, 256, 0, stream>>>((const bf16_t*)y, ldy, q_rank, kv_rank, rot, wq, wkv, eps, cos_sin,
                                                         slots, (bf16_t*)cq, (bf16_t*)k_cache, (bf16_t*)v_cache, P, num_pages);
  else
    PICO_REQUIRE(false, "pico_latent_prepare: unknown dtype %d", dtype);
  PICO_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------
// Rotation in place: the `rot` entries from column col0 + head * head_stride of every row of x are turned by the
// token's angles cos_sin [T, rot / 2, 2].  halves = 0: entry 2i goes with 2i + 1;  1: entry i goes with i + rot / 2.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void rope_inplace_kernel(T* __restrict__ x, int ldx, int col0, int heads, int head_stride,
                                                           int rot, int halves, const float* __restrict__ cos_sin) {
  const int t = blockIdx.x, half = rot / 2;
  const float* cs = cos_sin + (size_t)t * rot;
  for (int i = threadIdx.x; i < heads * half; i += blockDim.x) {
    const int h = i / half, p = i % half;
    T* base = x + (size_t)t * ldx + col0 + (size_t)h * head_stride;
    T* a = halves ? base + p : base + 2 * p;
    T* b = halves ? base + p + half : base + 2 * p + 1;
    const float u = load_f32(a), v = load_f32(b), c = cs[2 * p], s = cs[2 * p + 1];
    store_f32(a, u * c - v * s);
    store_f32(b, v * c + u * s);
  }
}

extern "C" int pico_rope_inplace(void* x, int ldx, int dtype, int col0, int heads, int head_stride, int rot, int halves,
                                 const float* cos_sin, int T, hipStream_t stream) {
  PICO_REQUIRE(T >= 0 && heads > 0 && rot >= 0 && rot % 2 == 0 && head_stride >= rot && col0 >= 0 &&
                   ldx >= col0 + (heads - 1) * head_stride + rot, "pico_rope_inplace: the heads do not fit the row");
  if (T == 0 || rot == 0) return 0;
  if (dtype == PICO_DTYPE_F32)
    rope_inplace_kernel<float><<<T, 256, 0, stream>>>((float*)x, ldx, col0, heads, head_stride, rot, halves, cos_sin);
  else if (dtype == PICO_DTYPE_BF16)
    rope_inplace_kernel<bf16_t><<<T, 256, 0, stream>>>((bf16_t*)x, ldx, col0, heads, head_stride, rot, halves, cos_sin);
  else
    PICO_REQUIRE(false, "pico_rope_inplace: unknown dtype %d", dtype);
  PICO_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------
// A product per head: out[t][h][o] = sum_i x[t][h][i] * W[h][i][o]        (W [heads, in, out]: a head's matrix with the
// inner index first, so that neighbouring threads read neighbouring addresses)
// x: head h of row t at x + t ldx + x_col + h x_head;  out likewise.  grid (T, heads, tiles of 64 outputs); the sum's order
// depends on `in` alone.
// `copy` > 0: the `copy` entries behind a head's `in` inputs are handed on behind its `out` outputs (a rotated part
// that goes on as it is, or is turned on the way).
// ---------------------------------------------------------------------------
#define HEAD_LINEAR_TILE 64
#define HEAD_LINEAR_SLICES 4
// A workgroup makes HEAD_LINEAR_TILE outputs of one head of one token; its four waves take a quarter of the inner
// index each (so that a matrix's loads travel side by side, not one behind the other) and their partial sums meet in
// LDS and are added in the waves' order: the sum's order depends on `in` alone.
template <typename T>
__global__ __launch_bounds__(HEAD_LINEAR_TILE* HEAD_LINEAR_SLICES) void head_linear_kernel(
    const T* __restrict__ x, int ldx, int x_col, int x_head, const T* __restrict__ W, T* __restrict__ out, int ldo, int o_col,
    int o_head, int in, int outn, int copy, const float* __restrict__ cos_sin) {
  extern __shared__ float xs[];                           // [in + copy], then [slices][tile] partial sums
  const int t = blockIdx.x, h = blockIdx.y;
  const T* xr = x + (size_t)t * ldx + x_col + (size_t)h * x_head;
  const int extra = blockIdx.z == 0 ? copy : 0;          // the first tile of a head hands the copied entries on
  for (int i = threadIdx.x; i < in + extra; i += blockDim.x) xs[i] = load_f32(xr + i);
  __syncthreads();
  float* part = xs + in + copy;
  const T* w = W + (size_t)h * in * outn;
  T* o = out + (size_t)t * ldo + o_col + (size_t)h * o_head;
  const int cx = threadIdx.x % HEAD_LINEAR_TILE, slice = threadIdx.x / HEAD_LINEAR_TILE;
  const int c = blockIdx.z * HEAD_LINEAR_TILE + cx, cc = min(c, outn - 1);
  const int per = (in + HEAD_LINEAR_SLICES - 1) / HEAD_LINEAR_SLICES;
  const int i0 = slice * per, i1 = min(in, i0 + per);
  float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
  int i = i0;
#pragma unroll 2
  for (; i + 3 < i1; i += 4) {
    a0 = fmaf(xs[i], load_f32(w + (size_t)i * outn + cc), a0);
    a1 = fmaf(xs[i + 1], load_f32(w + (size_t)(i + 1) * outn + cc), a1);
    a2 = fmaf(xs[i + 2], load_f32(w + (size_t)(i + 2) * outn + cc), a2);
    a3 = fmaf(xs[i + 3], load_f32(w + (size_t)(i + 3) * outn + cc), a3);
  }
  for (; i < i1; i++) a0 = fmaf(xs[i], load_f32(w + (size_t)i * outn + cc), a0);
  part[slice * HEAD_LINEAR_TILE + cx] = (a0 + a1) + (a2 + a3);
  __syncthreads();
  if (slice == 0 && c < outn)
    store_f32(o + c, (part[cx] + part[HEAD_LINEAR_TILE + cx]) + (part[2 * HEAD_LINEAR_TILE + cx] + part[3 * HEAD_LINEAR_TILE + cx]));
  // the copied entries as they are, or (cos_sin given: [T, copy / 2, 2]) turned by the token's angles, neighbours in pairs
  const float* cs = cos_sin ? cos_sin + (size_t)t * copy : nullptr;
  for (int k = threadIdx.x; k < extra; k += blockDim.x) {
    float v = xs[in + k];
    if (cs) {
      const int p = k >> 1;
      const float a = xs[in + 2 * p], b = xs[in + 2 * p + 1], c = cs[2 * p], sn = cs[2 * p + 1];
      v = (k & 1) ? b * c + a * sn : a * c - b * sn;
    }
    store_f32(o + outn + k, v);
  }
}

extern "C" int pico_head_linear(const void* x, int ldx, int x_col, int x_head, const void* W, void* out, int ldo, int o_col,
                                int o_head, int dtype, int T, int heads, int in, int outn, int copy, const float* cos_sin,
                                hipStream_t stream) {
  PICO_REQUIRE(cos_sin == nullptr || copy % 2 == 0, "pico_head_linear: a part that is turned has an even number of entries");
  PICO_REQUIRE(T >= 0 && heads > 0 && heads <= 65535 && in > 0 && outn > 0 && copy >= 0 && in + copy <= 12288,
               "pico_head_linear: bad sizes");
  PICO_REQUIRE(ldx >= x_col + (heads - 1) * x_head + in + copy && ldo >= o_col + (heads - 1) * o_head + outn + copy,
               "pico_head_linear: the heads do not fit the rows");
  if (T == 0) return 0;
  const size_t lds = (size_t)(in + copy + HEAD_LINEAR_TILE * HEAD_LINEAR_SLICES) * sizeof(float);
  const int tiles = (outn + HEAD_LINEAR_TILE - 1) / HEAD_LINEAR_TILE;
  if (dtype == PICO_DTYPE_F32)
    head_linear_kernel<float><<<dim3(T, heads, tiles), HEAD_LINEAR_TILE * HEAD_LINEAR_SLICES, lds, stream>>>((const float*)x, ldx, x_col, x_head, (const float*)W,
                                                                    (float*)out, ldo, o_col, o_head, in, outn, copy, cos_sin);
  else if (dtype == PICO_DTYPE_BF16)
    head_linear_kernel<bf16_t><<<dim3(T, heads, tiles), HEAD_LINEAR_TILE * HEAD_LINEAR_SLICES, lds, stream>>>((const bf16_t*)x, ldx, x_col, x_head, (const bf16_t*)W,
                                                                     (bf16_t*)out, ldo, o_col, o_head, in, outn, copy, cos_sin);
  else
    PICO_REQUIRE(false, "pico_head_linear: unknown dtype %d", dtype);
  PICO_LAUNCH_CHECK();
  return 0;
}
