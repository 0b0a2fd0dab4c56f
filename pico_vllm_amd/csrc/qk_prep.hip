// What stands between the q/k/v product and the attention kernel for attentions that norm their queries and keys:
//
//   pico_qk_norm_store:  RMS norm of q and k, either unit by unit (a unit = one head, or one map of a head that has
//                        several; one weight [dk] for all units) or over the whole row (all heads at once; a weight of
//                        the row's size); then the first `rot` entries of every unit turned (entry i with entry
//                        i + rot / 2, by the angles of a table [T, rot / 2, (cos, sin)]); the queries go to `q_out`, the
//                        keys and the values into the pages (k [nk, page, dk], v [nv, dv, page]).  The values are
//                        columns of the same row as they are: with v_col = k_col they are the keys as projected.
//   pico_diff_combine:   two attention maps of a head into one output:  o = a1 - lambda a2;  o / rms(o) * mult.
//
// Units of q with `maps` > 1 (head h holds maps units [map 0 | map 1 | ..]) leave in the order (kv group g, map m, head
// in group) so that unit ((g maps + m) R + r) reads kv unit g maps + m, the usual grouping of an attention kernel whose
// kv heads are the (group, map) pairs; R = heads a group.  Norms and angles are float32.
#include "common.h"

#define QK_NORM_NONE 0
#define QK_NORM_UNIT 1
#define QK_NORM_ROW 2

template <typename T>
__global__ __launch_bounds__(1024) void qk_norm_store_kernel(
    const T* __restrict__ x, int ld, int q_col, int k_col, int v_col, int nq, int nk, int nv, int dk, int dv, int maps,
    int norm_mode, const float* __restrict__ wq, const float* __restrict__ wk, float eps, const float* __restrict__ cos_sin,
    int rot, const int* __restrict__ slots, T* __restrict__ q_out, T* __restrict__ k_cache, T* __restrict__ v_cache, int P,
    int num_pages) {
  __shared__ float scratch[16];
  const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  const T* row = x + (size_t)t * ld;
  float row_q = 1.f, row_k = 1.f;
  if (norm_mode == QK_NORM_ROW) {
    float sq = 0.f, sk = 0.f;
    for (int i = threadIdx.x; i < nq * dk; i += blockDim.x) { const float v = load_f32(row + q_col + i); sq = fmaf(v, v, sq); }
    for (int i = threadIdx.x; i < nk * dk; i += blockDim.x) { const float v = load_f32(row + k_col + i); sk = fmaf(v, v, sk); }
    row_q = 1.0f / sqrtf(block_sum(sq, scratch) / (float)(nq * dk) + eps);
    row_k = 1.0f / sqrtf(block_sum(sk, scratch) / (float)(nk * dk) + eps);
  }
  const int slot = slots ? slots[t] : -1;
  const int page = slot >= 0 ? slot / P : -1, off = slot >= 0 ? slot % P : 0;
  const bool store = page >= 0 && page < num_pages;
  const int half = rot / 2;
  const float* cs = cos_sin ? cos_sin + (size_t)t * half * 2 : nullptr;
  const int qheads = nq / maps, R = max(1, qheads / max(1, nk / maps));      // heads a kv group
  for (int u = wave; u < nq + nk; u += nw) {
    const bool is_q = u < nq;
    const int un = is_q ? u : u - nq;
    const T* src = row + (is_q ? q_col : k_col) + (size_t)un * dk;
    float r = is_q ? row_q : row_k;
    if (norm_mode == QK_NORM_UNIT) {
      float ss = 0.f;
      for (int i = lane; i < dk; i += 64) { const float v = load_f32(src + i); ss = fmaf(v, v, ss); }
      r = 1.0f / sqrtf(wave_sum(ss) / (float)dk + eps);
    }
    const float* w = norm_mode == QK_NORM_NONE ? nullptr : (is_q ? wq : wk) + (norm_mode == QK_NORM_ROW ? (size_t)un * dk : 0);
    T* dst;
    if (is_q) {
      int place = un;
      if (maps > 1) {
        const int h = un / maps, m = un % maps, g = h / R, rr = h % R;
        place = (g * maps + m) * R + rr;
      }
      dst = q_out + ((size_t)t * nq + place) * dk;
    } else {
      if (!store) continue;
      dst = k_cache + (((size_t)page * nk + un) * P + off) * dk;
    }
    for (int i = lane; i < dk; i += 64) {
      float v = load_f32(src + i) * r * (w ? w[i] : 1.f);
      if (i < rot) {
        const int j = i < half ? i + half : i - half, f = i < half ? i : i - half;
        const float o = load_f32(src + j) * r * (w ? w[j] : 1.f);
        const float c = cs[2 * f], s = cs[2 * f + 1];
        v = i < half ? v * c - o * s : v * c + o * s;
      }
      store_f32(dst + i, v);
    }
  }
  if (store && v_cache) {
    for (int i = threadIdx.x; i < nv * dv; i += blockDim.x) {
      const int g = i / dv, j = i % dv;
      v_cache[(((size_t)page * nv + g) * dv + j) * P + off] = row[v_col + i];
    }
  }
}

extern "C" int pico_qk_norm_store(const void* x, int dtype, int ld, int q_col, int k_col, int v_col, int nq, int nk, int nv,
                                  int dk, int dv, int maps, int norm_mode, const float* wq, const float* wk, float eps,
                                  const float* cos_sin, int rot, const int* slots, void* q_out, void* k_cache, void* v_cache,
                                  int T, int P, int num_pages, hipStream_t stream) {
  PICO_REQUIRE(T >= 0 && nq > 0 && nk > 0 && nv >= 0 && dk > 0 && dv > 0 && maps >= 1 && nq % maps == 0 && nk % maps == 0,
               "pico_qk_norm_store: bad sizes");
  PICO_REQUIRE((nq / maps) % (nk / maps) == 0, "pico_qk_norm_store: %d query heads are not a multiple of %d kv heads", nq / maps, nk / maps);
  PICO_REQUIRE(norm_mode >= 0 && norm_mode <= 2 && (norm_mode == 0 || (wq && wk)), "pico_qk_norm_store: a norm needs its weights");
  PICO_REQUIRE(rot >= 0 && rot % 2 == 0 && rot <= dk && (rot == 0 || cos_sin), "pico_qk_norm_store: %d turned entries of %d", rot, dk);
  PICO_REQUIRE(ld >= q_col + nq * dk && ld >= k_col + nk * dk && ld >= v_col + nv * dv, "pico_qk_norm_store: the rows do not hold q, k and v");
  PICO_REQUIRE(k_cache == nullptr || (P > 0 && num_pages > 0 && slots), "pico_qk_norm_store: a cache needs pages and slots");
  if (T == 0) return 0;
  if (k_cache == nullptr) { slots = nullptr; v_cache = nullptr; P = 1; num_pages = 0; }
  // few tokens: a wave a unit, up to sixteen waves, so that a token's units wait for their norms side by side and not one
  // behind the other; many tokens fill the chip with four waves each
  const int threads = T >= 64 ? 256 : 64 * min(16, max(4, nq + nk));
  if (dtype == PICO_DTYPE_F32)
    qk_norm_store_kernel<float><<<T, threads, 0, stream>>>((const float*)x, ld, q_col, k_col, v_col, nq, nk, nv, dk, dv, maps, norm_mode,
                                                       wq, wk, eps, cos_sin, rot, slots, (float*)q_out, (float*)k_cache,
                                                       (float*)v_cache, P, num_pages);
  else if (dtype == PICO_DTYPE_BF16)
    qk_norm_store_kernel<bf16_t><<<T, threads, 0, stream>>>((const bf16_t*)x, ld, q_col, k_col, v_col, nq, nk, nv, dk, dv, maps,
                                                        norm_mode, wq, wk, eps, cos_sin, rot, slots, (bf16_t*)q_out,
                                                        (bf16_t*)k_cache, (bf16_t*)v_cache, P, num_pages);
  else
    PICO_REQUIRE(false, "pico_qk_norm_store: unknown dtype %d", dtype);
  PICO_LAUNCH_CHECK();
  return 0;
}

// a: float32 [T, groups * 2 * R * dv], the maps' outputs in the order (group, map, head in group); out [T, heads * dv]
// in the order of the heads.  One wave a (token, head).
template <typename T>
__global__ __launch_bounds__(64) void diff_combine_kernel(const float* __restrict__ a, float lambda, float eps, float mult,
                                                          T* __restrict__ out, int H, int R, int dv) {
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int g = h / R, r = h % R;
  const float* a1 = a + ((size_t)t * 2 * H + (size_t)(g * 2) * R + r) * dv;
  const float* a2 = a1 + (size_t)R * dv;
  float ss = 0.f;
  for (int i = lane; i < dv; i += 64) {
    const float o = a1[i] - lambda * a2[i];
    ss = fmaf(o, o, ss);
  }
  const float s = mult / sqrtf(wave_sum(ss) / (float)dv + eps);
  T* dst = out + ((size_t)t * H + h) * dv;
  for (int i = lane; i < dv; i += 64) store_f32(dst + i, (a1[i] - lambda * a2[i]) * s);
}

extern "C" int pico_diff_combine(const float* a, float lambda, float eps, float mult, void* out, int dtype, int T, int H,
                                 int G, int dv, hipStream_t stream) {
  PICO_REQUIRE(T >= 0 && H > 0 && G > 0 && H % G == 0 && dv > 0 && H <= 65535, "pico_diff_combine: bad sizes");
  if (T == 0) return 0;
  const dim3 grid(T, H);
  if (dtype == PICO_DTYPE_F32)
    diff_combine_kernel<float><<<grid, 64, 0, stream>>>(a, lambda, eps, mult, (float*)out, H, H / G, dv);
  else if (dtype == PICO_DTYPE_BF16)
    diff_combine_kernel<bf16_t><<<grid, 64, 0, stream>>>(a, lambda, eps, mult, (bf16_t*)out, H, H / G, dv);
  else
    PICO_REQUIRE(false, "pico_diff_combine: unknown dtype %d", dtype);
  PICO_LAUNCH_CHECK();
  return 0;
}
