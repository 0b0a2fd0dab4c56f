// Attention with a linear distance penalty, a query temperature that grows with the position, and keys and
// values of different sizes, over the paged cache; and the store of its keys and values.
//
//   query head h reads kv head h / (nq / nkv)
//   s_ij = (q_i . k_j) * scale * temp(i) - slope_h * (i - j),   keys j <= i, with a window only i - j < window
//   temp(i) = 1 + coef * ln(floor((i + 1) / every) + 1)         (every == 0: 1)
//   slope_h = 2^(-span * (h + 1) / nq)                          (span == 0: no penalty)
//   optionally s_ij <- cap * tanh(s_ij / cap); with a window, the first `keep_first` positions of a sequence stay
//   visible to every later query (at their true distance); optionally o_i is multiplied element by element with
//   sigmoid(gate_i) before it is written
//   softmax over the visible keys, o_i = sum_j p_ij v_j
//   instead of a window, chunks: key j <= i is seen iff floor(i / chunk) == floor(j / chunk), chunks counted from
//   position 0; optionally a sink (a key of score 0 without a value: the softmax's denominator gains a 1); the gate may be
//   one number a head; several kv heads (of keys) may share one head of values (v_div of them each)
//
// A page holds k as [kv heads, page, dk] and v as [kv heads, dv, page].  Scores, softmax and the sums over keys are
// float32 whatever the storage type.  This file holds the plain kernel (one wave per query token and head, any sizes,
// float32 or bfloat16 storage): the attention of the 32-bit engine and the fallback of the bfloat16 engine.
#include "common.h"

struct BiasParams {
  float scale, temp_coef, slope_span;
  int temp_every, window;
  float softcap;      // 0: none
  int keep_first;     // with a window: keys below this position are seen whatever their distance
  int chunk;          // > 0: position i sees key j <= i only if floor(i / chunk) == floor(j / chunk) (instead of a window)
  int sink;           // != 0: one more key of score 0 and no value, p_j = exp(s_j) / (1 + sum exp(s))
  int gate_heads;     // != 0: the gate holds one number a head (gate[t][h]) instead of one an output element
  int v_div;          // kv head g's values are value head g / v_div (several kv heads of keys over one head of values)
};

__device__ __forceinline__ float query_scale(const BiasParams& p, int pos) {
  if (p.temp_every <= 0) return p.scale;
  return p.scale * (1.0f + p.temp_coef * logf((float)((pos + 1) / p.temp_every + 1)));
}

__device__ __forceinline__ float head_slope(const BiasParams& p, int h, int nq) {
  return p.slope_span > 0.f ? exp2f(-p.slope_span * (float)(h + 1) / (float)nq) : 0.f;
}

// ---------------------------------------------------------------------------
// Store of a step's keys and values: token t's k and v (columns k_col.. and v_col.. of its row of `qkv`) go to slot
// slots[t] (page * P + offset; negative: nothing is stored).  With `v_first` the value is mixed first:
// v <- (1 - lambda) v + lambda v_first[t] in float32, and the mixed value is what the cache gets.
// One workgroup per token.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void kv_mix_store_kernel(const T* __restrict__ qkv, int ld, int k_col, int v_col,
                                                           const T* __restrict__ v_first, int ld_first, float lambda,
                                                           const int* __restrict__ slots, T* __restrict__ k_cache,
                                                           T* __restrict__ v_cache, int nkv, int dk, int dv, int P,
                                                           int num_pages) {
  const int t = blockIdx.x;
  const int slot = slots[t];
  if (slot < 0) return;
  const int page = slot / P, off = slot % P;
  if (page >= num_pages) return;
  const T* row = qkv + (size_t)t * ld;
  for (int i = threadIdx.x; i < nkv * dk; i += blockDim.x) {
    const int g = i / dk, j = i % dk;
    k_cache[(((size_t)page * nkv + g) * P + off) * dk + j] = row[k_col + i];
  }
  for (int i = threadIdx.x; i < nkv * dv; i += blockDim.x) {
    const int g = i / dv, j = i % dv;
    T* dst = v_cache + (((size_t)page * nkv + g) * dv + j) * P + off;
    if (v_first) {
      const float v = load_f32(row + v_col + i), f = load_f32(v_first + (size_t)t * ld_first + i);
      store_f32(dst, (1.0f - lambda) * v + lambda * f);
    } else {
      *dst = row[v_col + i];
    }
  }
}

extern "C" int pico_kv_mix_store(const void* qkv, int dtype, int ld, int k_col, int v_col, const void* v_first,
                                 int ld_first, float lambda, const int* slots, void* k_cache, void* v_cache, int T,
                                 int nkv, int dk, int dv, int P, int num_pages, hipStream_t stream) {
  PICO_REQUIRE(T >= 0 && nkv > 0 && dk > 0 && dv > 0 && P > 0 && num_pages > 0, "pico_kv_mix_store: bad sizes");
  PICO_REQUIRE(k_col >= 0 && v_col >= 0 && ld >= k_col + nkv * dk && ld >= v_col + nkv * dv,
               "pico_kv_mix_store: the row of %d columns does not hold the keys and values", ld);
  PICO_REQUIRE(v_first == nullptr || ld_first >= nkv * dv, "pico_kv_mix_store: the rows of the first values are too short");
  if (T == 0) return 0;
  if (dtype == PICO_DTYPE_F32)
    kv_mix_store_kernel<float><<<T, 256, 0, stream>>>((const float*)qkv, ld, k_col, v_col, (const float*)v_first, ld_first,
                                                      lambda, slots, (float*)k_cache, (float*)v_cache, nkv, dk, dv, P,
                                                      num_pages);
  else if (dtype == PICO_DTYPE_BF16)
    kv_mix_store_kernel<bf16_t><<<T, 256, 0, stream>>>((const bf16_t*)qkv, ld, k_col, v_col, (const bf16_t*)v_first,
                                                       ld_first, lambda, slots, (bf16_t*)k_cache, (bf16_t*)v_cache, nkv,
                                                       dk, dv, P, num_pages);
  else
    PICO_REQUIRE(false, "pico_kv_mix_store: unknown dtype %d", dtype);
  PICO_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------
// The plain kernel.  Keys are visited in blocks of 64 aligned to absolute positions, so the result at a position does
// not depend on how the sequence was cut into steps.
// ---------------------------------------------------------------------------
template <typename T, int NV>
__global__ __launch_bounds__(64) void attn_bias_plain_kernel(
    const T* __restrict__ q, int q_stride, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const int* __restrict__ block_table, int max_pages, const int* __restrict__ positions,
    const int* __restrict__ token_seq, T* __restrict__ out, int nq, int nkv, int dk, int dv, int P, BiasParams bp,
    int num_pages, const T* __restrict__ gate, int gate_stride, float* __restrict__ out32) {
  extern __shared__ float lds[];
  float* qs = lds;        // [dk]
  float* ps = lds + dk;   // [64]
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int g = h / (nq / nkv);
  const int pos = positions[t];
  const int* bt = block_table + (size_t)token_seq[t] * max_pages;
  const int lo = bp.chunk > 0 ? pos / bp.chunk * bp.chunk : bp.window > 0 ? max(0, pos - bp.window + 1) : 0;
  const int gv = g / bp.v_div, nv = nkv / bp.v_div;        // the head of values, and how many there are
  const float qscale = query_scale(bp, pos), slope = head_slope(bp, h, nq);
  const T* qrow = q + (size_t)t * q_stride + (size_t)h * dk;
  for (int j = lane; j < dk; j += 64) qs[j] = load_f32(qrow + j);
  __syncthreads();

  float m = -INFINITY, l = 0.f;
  float acc[NV];
#pragma unroll
  for (int i = 0; i < NV; i++) acc[i] = 0.f;
  // blocks of 64 keys aligned to absolute positions: first those that hold kept first positions in front of the
  // window, then the window's; a block that holds both is visited once
  const int keep = bp.window > 0 ? min(bp.keep_first, lo) : 0;      // keys below `keep` are seen although the window has passed them
  const int win0 = (lo / 64) * 64;
  const float inv_cap = bp.softcap > 0.f ? 1.0f / bp.softcap : 0.f;
  for (int c0 = 0; c0 <= pos; c0 += 64) {
    if (c0 >= keep && c0 < win0) { c0 = win0 - 64; continue; }
    const int key = c0 + lane;
    const bool valid = key <= pos && (key >= lo || key < keep);
    float s = -INFINITY;
    if (valid) {
      int page = bt[key / P];
      page = min(max(page, 0), num_pages - 1);
      const T* kp = k_cache + (((size_t)page * nkv + g) * P + key % P) * dk;
      float dot = 0.f;
      for (int j = 0; j < dk; j++) dot = fmaf(qs[j], load_f32(kp + j), dot);
      s = dot * qscale - slope * (float)(pos - key);
      if (bp.softcap > 0.f) s = bp.softcap * tanhf(s * inv_cap);
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float alpha = expf(m - m_new);
    const float p = valid ? expf(s - m_new) : 0.f;
    l = l * alpha + wave_sum(p);
    __syncthreads();
    ps[lane] = p;
    __syncthreads();
    float blk[NV];
#pragma unroll
    for (int i = 0; i < NV; i++) blk[i] = 0.f;
    const int kend = min(64, pos - c0 + 1);
    for (int kk = 0; kk < kend; kk++) {
      const int kpos = c0 + kk;
      if (kpos < lo && kpos >= keep) continue;
      int page = bt[kpos / P];
      page = min(max(page, 0), num_pages - 1);
      const T* vp = v_cache + ((size_t)page * nv + gv) * dv * P + kpos % P;
      const float pk = ps[kk];
#pragma unroll
      for (int i = 0; i < NV; i++) {
        const int dim = lane + 64 * i;
        if (dim < dv) blk[i] = fmaf(pk, load_f32(vp + (size_t)dim * P), blk[i]);
      }
    }
#pragma unroll
    for (int i = 0; i < NV; i++) acc[i] = fmaf(acc[i], alpha, blk[i]);
    m = m_new;
  }
  if (bp.sink) l += expf(-m);                              // the sink's exp(0 - m); the query's own key is always seen
  T* o = out + ((size_t)t * nq + h) * dv;
#pragma unroll
  for (int i = 0; i < NV; i++) {
    const int dim = lane + 64 * i;
    if (dim >= dv) continue;
    float v = acc[i] / l;
    if (gate) v *= 1.0f / (1.0f + expf(-load_f32(gate + (size_t)t * gate_stride + (bp.gate_heads ? (size_t)h : (size_t)h * dv + dim))));
    if (out32) out32[((size_t)t * nq + h) * dv + dim] = v;
    else store_f32(o + dim, v);
  }
}

extern "C" int pico_attn_bias_plain(const void* q, int q_stride, int dtype, const void* k_cache, const void* v_cache,
                                    const int* block_table, int max_pages, const int* positions, const int* token_seq,
                                    void* out, int T, int nq, int nkv, int dk, int dv, int P, int window, float scale,
                                    float temp_coef, int temp_every, float slope_span, int num_pages,
                                    float softcap, int keep_first, const void* gate, int gate_stride, int chunk, int sink,
                                    int gate_heads, int v_div, int out_f32, hipStream_t stream) {
  PICO_REQUIRE(T >= 0 && nq > 0 && nkv > 0 && dk > 0 && dv > 0 && P > 0 && max_pages > 0 && num_pages > 0,
               "pico_attn_bias_plain: bad sizes");
  PICO_REQUIRE(nq % nkv == 0, "pico_attn_bias_plain: %d query heads are not a multiple of %d kv heads", nq, nkv);
  PICO_REQUIRE(dk <= 1024 && dv <= 512, "pico_attn_bias_plain: key size %d (at most 1024) or value size %d (at most 512) too large", dk, dv);
  PICO_REQUIRE(nq <= 65535, "pico_attn_bias_plain: too many heads");
  PICO_REQUIRE(q_stride >= nq * dk, "pico_attn_bias_plain: query row stride too small");
  PICO_REQUIRE(window >= 0 && temp_every >= 0 && slope_span >= 0.f, "pico_attn_bias_plain: window, interval and span must not be negative");
  PICO_REQUIRE(softcap >= 0.f && keep_first >= 0, "pico_attn_bias_plain: cap and kept first positions must not be negative");
  PICO_REQUIRE(gate == nullptr || gate_stride >= (gate_heads ? nq : nq * dv), "pico_attn_bias_plain: gate row stride too small");
  PICO_REQUIRE(chunk >= 0 && (chunk == 0 || window == 0), "pico_attn_bias_plain: chunks or a window, not both");
  PICO_REQUIRE(v_div >= 1 && nkv % v_div == 0, "pico_attn_bias_plain: %d kv heads do not share values %d each", nkv, v_div);
  if (T == 0) return 0;
  const BiasParams bp{scale, temp_coef, slope_span, temp_every, window, softcap, keep_first, chunk, sink, gate_heads, v_div};
  float* out32 = out_f32 ? (float*)out : nullptr;
  dim3 grid(T, nq);
  const size_t lds = (size_t)(dk + 64) * sizeof(float);
  if (dtype == PICO_DTYPE_F32) {
    if (dv <= 256)
      attn_bias_plain_kernel<float, 4><<<grid, 64, lds, stream>>>(
          (const float*)q, q_stride, (const float*)k_cache, (const float*)v_cache, block_table, max_pages, positions,
          token_seq, (float*)out, nq, nkv, dk, dv, P, bp, num_pages, (const float*)gate, gate_stride, out32);
    else
      attn_bias_plain_kernel<float, 8><<<grid, 64, lds, stream>>>(
          (const float*)q, q_stride, (const float*)k_cache, (const float*)v_cache, block_table, max_pages, positions,
          token_seq, (float*)out, nq, nkv, dk, dv, P, bp, num_pages, (const float*)gate, gate_stride, out32);
  }
  else if (dtype == PICO_DTYPE_BF16) {
    if (dv <= 256)
      attn_bias_plain_kernel<bf16_t, 4><<<grid, 64, lds, stream>>>(
          (const bf16_t*)q, q_stride, (const bf16_t*)k_cache, (const bf16_t*)v_cache, block_table, max_pages, positions,
          token_seq, (bf16_t*)out, nq, nkv, dk, dv, P, bp, num_pages, (const bf16_t*)gate, gate_stride, out32);
    else
      attn_bias_plain_kernel<bf16_t, 8><<<grid, 64, lds, stream>>>(
          (const bf16_t*)q, q_stride, (const bf16_t*)k_cache, (const bf16_t*)v_cache, block_table, max_pages, positions,
          token_seq, (bf16_t*)out, nq, nkv, dk, dv, P, bp, num_pages, (const bf16_t*)gate, gate_stride, out32);
  }
  else
    PICO_REQUIRE(false, "pico_attn_bias_plain: unknown dtype %d", dtype);
  PICO_LAUNCH_CHECK();
  return 0;
}
