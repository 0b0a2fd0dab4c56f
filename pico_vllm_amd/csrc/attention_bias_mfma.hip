// Matrix-core kernel of the attention with a distance penalty (see attention_bias.hip for the formulas), bfloat16,
// compiled for one pair of sizes: -DPICO_DK=<key size, a multiple of 32> -DPICO_DV=<value size, a multiple of 16>.
//
// One kernel serves prompt portions and single tokens alike.  The unit of work is a block of 16 query COLUMNS that
// share their keys: columns are (token, head) pairs of one sequence and one kv group, token-major; with R heads a
// group a block holds floor(16 / R) consecutive tokens with all their heads (R > 16: one token and 16 of its heads).
// A wave computes S^T = K Q^T for 32 keys a step (two v_mfma_f32_16x16x32_bf16 tiles whose rows are ordered so that
// the lanes of quarter kq hold the 8 consecutive keys 8 kq .. 8 kq + 7), adds the penalty and the masks per column
// (every lane owns one column: its position, temperature and slope are lane scalars), keeps an online softmax per
// column, and feeds P^T from registers as the B operand of O^T += V^T P^T, whose A operand is 16 contiguous bytes of
// V^T as the pages hold it.  Scores, softmax statistics and sums are float32; P is rounded to bfloat16 for the product.
//
// Two shapes of workgroup (four waves): SPLIT, one block whose key range the waves share in steps of 32 and merge
// through LDS (few blocks: decoding, short portions); or four neighbouring blocks, one a wave, whose key ranges
// overlap so that their loads meet in the first-level cache (long portions).
#include "common.h"

#ifndef PICO_DK
#error "compile with -DPICO_DK=<key size> -DPICO_DV=<value size>"
#endif
constexpr int DK = PICO_DK, DV = PICO_DV;
static_assert(DK % 32 == 0 && DK >= 32 && DK <= 512, "key size: a multiple of 32 up to 512");
static_assert(DV % 16 == 0 && DV >= 16 && DV <= 256, "value size: a multiple of 16 up to 256");
constexpr int KS = DK / 32;     // contraction steps of a score tile
constexpr int DT = DV / 16;     // 16-wide tiles of the value dimension

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

extern "C" int pico_attnb_key_dim() { return DK; }
extern "C" int pico_attnb_value_dim() { return DV; }

struct BiasArgs {
  const bf16_t* q;
  int q_stride;
  const bf16_t* k_cache;
  const bf16_t* v_cache;
  const int* block_table;
  int max_pages;
  const int* cu_seqlens;       // [B + 1] first flat token of every sequence
  const int* positions;        // [T]
  bf16_t* out;                 // [T, nq * DV]
  int num_seqs, nq, nkv, P, num_pages, window, temp_every;
  float scale, temp_coef, slope_span;
  // chunks > 1 (SPLIT only): workgroup z of a block takes the z-th piece of the block's keys and leaves its sums
  // unnormalised in parts_o [chunks][columns][DV] and its (maximum, sum) in parts_ml [chunks][columns][2]
  int chunks, ncols;
  float* parts_o;
  float* parts_ml;
  // scores <- softcap tanh(scores / softcap) (0: none); with a window, keys below keep_first are seen at any distance;
  // gate (or null): the output is multiplied element by element with sigmoid(gate[t][head * DV + d])
  float softcap;
  int keep_first;
  const bf16_t* gate;
  int gate_stride;
  // chunk > 0 (instead of a window): key j <= i is seen iff floor(i / chunk) == floor(j / chunk); sink: the softmax's
  // denominator gains exp(0) (a key of score 0 without a value); gate_heads: the gate holds one number a head;
  // v_div: kv head g reads value head g / v_div; out_f32: `out` is float32
  int chunk, sink, gate_heads, v_div, out_f32;
};

__device__ __forceinline__ float sigmoid_f32(float x) { return 1.0f / (1.0f + __expf(-x)); }

template <bool SPLIT>
__global__ __launch_bounds__(256, 2) void attn_bias_kernel(const BiasArgs a) {
  __shared__ float xo[SPLIT ? 3 : 1][SPLIT ? DV : 1][16];
  __shared__ float xml[SPLIT ? 3 : 1][2][16];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, col = lane & 15, kq = lane >> 4;
  const int g = blockIdx.y;
  const int R = a.nq / a.nkv;
  const int tpb = R >= 16 ? 1 : 16 / R;                 // tokens a block
  const int hb = R > 16 ? (R + 15) / 16 : 1;            // blocks a token (R > 16)
  // which block of which sequence: blocks are counted sequence by sequence
  int tile = SPLIT ? (int)blockIdx.x : 4 * (int)blockIdx.x + wave;
  int b = 0, t_begin = 0, t_end = 0;
  bool found = false;
  for (; b < a.num_seqs; b++) {
    t_begin = a.cu_seqlens[b];
    t_end = a.cu_seqlens[b + 1];
    const int tiles = (t_end - t_begin + tpb - 1) / tpb * hb;
    if (tile < tiles) { found = true; break; }
    tile -= tiles;
  }
  if (!found) {
    if (SPLIT) return;          // the whole workgroup
    t_begin = t_end = 0;        // this wave has nothing; it still meets no barrier below
  }
  const int t0 = t_begin + (tile / hb) * tpb;           // first token of the block
  const int ntok = found ? min(tpb, t_end - t0) : 0;
  const int hc = tile % hb;                             // which 16 heads of the token (R > 16)
  const int my_tok = R >= 16 ? 0 : col / R, my_h = R >= 16 ? 16 * hc + col : col % R;
  const bool col_ok = my_tok < ntok && my_h < R;
  const int t = t0 + (col_ok ? my_tok : 0);
  const int head = g * R + (col_ok ? my_h : 0);
  const int p0 = found ? a.positions[t0] : 0;           // the block's first position; its tokens follow one another
  const int my_pos = p0 + (col_ok ? my_tok : 0);
  const int hi = p0 + ntok;                             // keys below hi are read
  const int lo = a.chunk > 0 ? p0 / a.chunk * a.chunk : a.window > 0 ? max(0, p0 - a.window + 1) : 0;
  const int my_lo = a.chunk > 0 ? my_pos / a.chunk * a.chunk : a.window > 0 ? max(0, my_pos - a.window + 1) : 0;
  const int gv = g / a.v_div, nv = a.nkv / a.v_div;      // the head of values, and how many there are
  const int keep = a.window > 0 ? a.keep_first : 0;     // keys below are seen although a window has passed them
  const float inv_cap = a.softcap > 0.f ? 1.0f / a.softcap : 0.f;
  const int* bt = a.block_table + (size_t)b * a.max_pages;
  float qscale = a.scale, slope = 0.f;
  if (a.temp_every > 0) qscale *= 1.0f + a.temp_coef * logf((float)((my_pos + 1) / a.temp_every + 1));
  if (a.slope_span > 0.f) slope = exp2f(-a.slope_span * (float)(head + 1) / (float)a.nq);

  bf16x8 qf[KS];
  {
    const bf16_t* qrow = a.q + (size_t)t * a.q_stride + (size_t)head * DK + 8 * kq;
#pragma unroll
    for (int st = 0; st < KS; st++) {
      uint4 v = make_uint4(0, 0, 0, 0);
      if (col_ok) v = *reinterpret_cast<const uint4*>(qrow + 32 * st);
      qf[st] = __builtin_bit_cast(bf16x8, v);
    }
  }
  float m = -INFINITY, l = 0.f;
  f32x4 o[DT];
#pragma unroll
  for (int tt = 0; tt < DT; tt++) o[tt] = f32x4{0.f, 0.f, 0.f, 0.f};

  const int pshift = 31 - __clz(a.P);                   // page sizes are powers of two
  const int stride = SPLIT ? 128 : 32;
  int begin = lo & ~31, end = hi;
  if (SPLIT && a.chunks > 1) {
    // pieces of whole turns of the four waves (128 keys), so the tiles are those of the uncut loop
    const int piece = ((hi - begin + a.chunks - 1) / a.chunks + 127) & ~127;
    begin += (int)blockIdx.z * piece;
    end = min(hi, begin + piece);
  }
  // kept first keys in front of the window's first tile: tiles of their own, taken by the first piece (those inside
  // the window's tiles are let through by the mask below)
  const int sink_end = min(keep, lo & ~31);
  const bool sinks = sink_end > 0 && (!SPLIT || blockIdx.z == 0);
  const int first = begin + (SPLIT ? 32 * wave : 0);
  if (ntok > 0 && (first < end || sinks)) {
    const int last_key = hi - 1, last_group = last_key / 8 * 8;
    const int row_key = 8 * (col >> 2) + (col & 3);     // key of this lane's row in tile 0; tile 1: 4 more
    int key0 = sinks ? (SPLIT ? 32 * wave : 0) : first;
    bool in_sinks = sinks;
    if (in_sinks && key0 >= sink_end) { in_sinks = false; key0 = first; }
    while (in_sinks || key0 < end) {
      uint4 kr[2][KS];
      uint4 vr[DT];
      // positions beyond the range are clamped to its last key (group of 8, which lies in one page as pages hold at
      // least 8 keys): the page exists, the scores are masked
#pragma unroll
      for (int tl = 0; tl < 2; tl++) {
        const int pos = min(key0 + row_key + 4 * tl, last_key);
        const int page = min(max(bt[pos >> pshift], 0), a.num_pages - 1);
        const bf16_t* kp = a.k_cache + ((((size_t)page * a.nkv + g) << pshift) + (pos & (a.P - 1))) * DK + 8 * kq;
#pragma unroll
        for (int st = 0; st < KS; st++) kr[tl][st] = *reinterpret_cast<const uint4*>(kp + 32 * st);
      }
      {
        const int pos = min(key0 + 8 * kq, last_group);
        const int page = min(max(bt[pos >> pshift], 0), a.num_pages - 1);
        const bf16_t* vp = a.v_cache + ((((size_t)page * nv + gv) * DV + col) << pshift) + (pos & (a.P - 1));
#pragma unroll
        for (int tt = 0; tt < DT; tt++) vr[tt] = *reinterpret_cast<const uint4*>(vp + ((size_t)tt * 16 << pshift));
      }
      f32x4 s0 = f32x4{0.f, 0.f, 0.f, 0.f}, s1 = s0;
#pragma unroll
      for (int st = 0; st < KS; st++) {
        s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, kr[0][st]), qf[st], s0, 0, 0, 0);
        s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, kr[1][st]), qf[st], s1, 0, 0, 0);
      }
      float sv[8];
      float mx = -INFINITY;
#pragma unroll
      for (int r = 0; r < 8; r++) {
        const int key = key0 + 8 * kq + r;
        float v = (r < 4 ? s0[r & 3] : s1[r & 3]) * qscale - slope * (float)(my_pos - key);
        if (a.softcap > 0.f) v = a.softcap * tanhf(v * inv_cap);
        if (key > my_pos || (key < my_lo && key >= keep)) v = -INFINITY;
        sv[r] = v;
        mx = fmaxf(mx, v);
      }
      mx = max_across_16(mx);
      mx = max_across_32(mx);
      const float m_new = fmaxf(m, mx);
      const float m_use = m_new == -INFINITY ? 0.f : m_new;     // a column that has seen no key yet
      const float alpha = __expf(m - m_use);
      float sum = 0.f;
#pragma unroll
      for (int r = 0; r < 8; r++) {
        sv[r] = __expf(sv[r] - m_use);
        sum += sv[r];
      }
      sum = sum_across_16(sum);
      sum = sum_across_32(sum);
      l = l * alpha + sum;
      m = m_new;
      const bf16x8 pb = __builtin_bit_cast(bf16x8, make_uint4(pack2_bf16(sv[0], sv[1]), pack2_bf16(sv[2], sv[3]),
                                                               pack2_bf16(sv[4], sv[5]), pack2_bf16(sv[6], sv[7])));
      if (key0 + 32 > hi || key0 < lo) {
        // values of keys outside the range hold whatever the page held before: make them zero (0 * NaN is NaN)
        // this lane's eight keys: a key counts if it lies below hi and either inside the block's window or among
        // the kept first ones
        uint32_t live[4];
#pragma unroll
        for (int w = 0; w < 4; w++) {
          const int k0 = key0 + 8 * kq + 2 * w, k1 = k0 + 1;
          const bool v0 = k0 < hi && (k0 >= lo || k0 < keep), v1 = k1 < hi && (k1 >= lo || k1 < keep);
          live[w] = (v0 ? 0x0000ffffu : 0u) | (v1 ? 0xffff0000u : 0u);
        }
#pragma unroll
        for (int tt = 0; tt < DT; tt++) {
          vr[tt].x &= live[0];
          vr[tt].y &= live[1];
          vr[tt].z &= live[2];
          vr[tt].w &= live[3];
        }
      }
#pragma unroll
      for (int tt = 0; tt < DT; tt++) {
        o[tt] *= alpha;
        o[tt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, vr[tt]), pb, o[tt], 0, 0, 0);
      }
      key0 += stride;
      if (in_sinks && key0 >= sink_end) { in_sinks = false; key0 = first; }
    }
  }
  float a0 = 1.f, L = l, M_all = m;
  if (SPLIT) {
    // merge the four waves; lane (col, kq) of wave 0 holds value dimensions 16 tt + 4 kq + r of column `col`
    if (wave > 0) {
#pragma unroll
      for (int tt = 0; tt < DT; tt++)
#pragma unroll
        for (int r = 0; r < 4; r++) xo[wave - 1][16 * tt + 4 * kq + r][col] = o[tt][r];
      if (kq == 0) { xml[wave - 1][0][col] = m; xml[wave - 1][1][col] = l; }
    }
    __syncthreads();
    if (wave != 0) return;
    float M = m;
#pragma unroll
    for (int w = 0; w < 3; w++) M = fmaxf(M, xml[w][0][col]);
    const float m_use = (M == -INFINITY) ? 0.f : M;
    M_all = M;
    a0 = __expf(m - m_use);
    float aw[3];
    L = l * a0;
#pragma unroll
    for (int w = 0; w < 3; w++) {
      aw[w] = __expf(xml[w][0][col] - m_use);
      L += xml[w][1][col] * aw[w];
    }
#pragma unroll
    for (int tt = 0; tt < DT; tt++)
#pragma unroll
      for (int r = 0; r < 4; r++) {
        float acc = o[tt][r] * a0;
#pragma unroll
        for (int w = 0; w < 3; w++) acc += xo[w][16 * tt + 4 * kq + r][col] * aw[w];
        o[tt][r] = acc;
      }
  }
  if (!col_ok) return;
  if (SPLIT && a.chunks > 1) {
    const size_t c = (size_t)blockIdx.z * a.ncols + (size_t)t * a.nq + head;
    float* po = a.parts_o + c * DV + 4 * kq;
#pragma unroll
    for (int tt = 0; tt < DT; tt++) *reinterpret_cast<f32x4*>(po + 16 * tt) = o[tt];
    if (kq == 0) { a.parts_ml[2 * c] = M_all; a.parts_ml[2 * c + 1] = L; }
    return;
  }
  if (a.sink) L += __expf(-M_all);                        // the column's own key is always seen: M_all is finite
  float inv = 1.0f / L;
  if (a.gate && a.gate_heads) inv *= sigmoid_f32(bf16_to_f32(a.gate[(size_t)t * a.gate_stride + head]));
  bf16_t* orow = a.out + ((size_t)t * a.nq + head) * DV + 4 * kq;
  const bf16_t* grow = a.gate && !a.gate_heads ? a.gate + (size_t)t * a.gate_stride + (size_t)head * DV + 4 * kq : nullptr;
#pragma unroll
  for (int tt = 0; tt < DT; tt++) {
    float g0 = inv, g1 = inv, g2 = inv, g3 = inv;
    if (a.out_f32) {
      float* o32 = reinterpret_cast<float*>(a.out) + ((size_t)t * a.nq + head) * DV + 4 * kq + 16 * tt;
      *reinterpret_cast<f32x4*>(o32) = f32x4{o[tt][0] * g0, o[tt][1] * g1, o[tt][2] * g2, o[tt][3] * g3};
      continue;
    }
    if (grow) {
      const uint2 gv = *reinterpret_cast<const uint2*>(grow + 16 * tt);
      g0 *= sigmoid_f32(__uint_as_float(gv.x << 16));
      g1 *= sigmoid_f32(__uint_as_float(gv.x & 0xffff0000u));
      g2 *= sigmoid_f32(__uint_as_float(gv.y << 16));
      g3 *= sigmoid_f32(__uint_as_float(gv.y & 0xffff0000u));
    }
    uint2 w;
    w.x = pack2_bf16(o[tt][0] * g0, o[tt][1] * g1);
    w.y = pack2_bf16(o[tt][2] * g2, o[tt][3] * g3);
    *reinterpret_cast<uint2*>(orow + 16 * tt) = w;
  }
}

#define MAX_PIECES 64
// The pieces of a column's keys put together: out = sum_z o_z e^(m_z - M) / sum_z l_z e^(m_z - M), z in ascending order.
__global__ __launch_bounds__(DV <= 64 ? 64 : DV <= 128 ? 128 : 256) void attn_bias_merge_kernel(
    const float* __restrict__ parts_o, const float* __restrict__ parts_ml, int chunks, int ncols, bf16_t* __restrict__ out,
    const bf16_t* __restrict__ gate, int gate_stride, int nq, int sink, int gate_heads, int out_f32) {
  // the pieces' maxima and sums once into LDS (one load a thread, all in flight together), then every thread its sum
  __shared__ float ms[MAX_PIECES], ws[MAX_PIECES];
  const int c = blockIdx.x, d = threadIdx.x;
  for (int z = d; z < chunks; z += blockDim.x) {
    const float2 ml = *reinterpret_cast<const float2*>(parts_ml + 2 * ((size_t)z * ncols + c));
    ms[z] = ml.x;
    ws[z] = ml.y;
  }
  __syncthreads();
  if (d >= DV) return;
  float M = -INFINITY;
  for (int z = 0; z < chunks; z++) M = fmaxf(M, ms[z]);
  float L = 0.f, acc = 0.f;
#pragma unroll 8
  for (int z = 0; z < chunks; z++) {
    const float w = ms[z] == -INFINITY ? 0.f : __expf(ms[z] - M);
    L += ws[z] * w;
    acc += parts_o[((size_t)z * ncols + c) * DV + d] * w;
  }
  if (sink) L += __expf(-M);
  float v = acc / L;
  if (gate) v *= sigmoid_f32(bf16_to_f32(gate[(size_t)(c / nq) * gate_stride + (gate_heads ? (size_t)(c % nq) : (size_t)(c % nq) * DV + d)]));
  if (out_f32) reinterpret_cast<float*>(out)[(size_t)c * DV + d] = v;
  else out[(size_t)c * DV + d] = f32_to_bf16(v);
}

// split != 0: one block of 16 columns a workgroup, its keys shared by the four waves; else four blocks a workgroup.
extern "C" int pico_attnb(const void* q, int q_stride, const void* k_cache, const void* v_cache, const int* block_table,
                          int max_pages, const int* cu_seqlens, const int* positions, int num_seqs, int T, void* out,
                          int nq, int nkv, int dk, int dv, int P, int num_pages, float scale, int window, float temp_coef,
                          int temp_every, float slope_span, int split, int chunks, float* parts_o, float* parts_ml,
                          float softcap, int keep_first, const void* gate, int gate_stride, int chunk, int sink,
                          int gate_heads, int v_div, int out_f32, hipStream_t stream) {
  PICO_REQUIRE(dk == DK && dv == DV, "pico_attnb: built for keys of %d and values of %d, asked for %d and %d", DK, DV, dk, dv);
  PICO_REQUIRE(T >= 0 && num_seqs > 0 && nq > 0 && nkv > 0 && nq % nkv == 0 && max_pages > 0 && num_pages > 0,
               "pico_attnb: bad sizes");
  PICO_REQUIRE(P >= 8 && (P & (P - 1)) == 0, "pico_attnb: the page size must be a power of two of at least 8, got %d", P);
  PICO_REQUIRE(q_stride >= nq * DK && q_stride % 8 == 0 && (uintptr_t)q % 16 == 0, "pico_attnb: query rows must be 16-byte aligned");
  PICO_REQUIRE(nkv <= 65535 && window >= 0 && temp_every >= 0 && slope_span >= 0.f, "pico_attnb: bad constants");
  PICO_REQUIRE(chunks >= 1 && chunks <= MAX_PIECES && (chunks == 1 || (split && parts_o && parts_ml)),
               "pico_attnb: pieces of the keys go with one block a workgroup and need room for the parts");
  PICO_REQUIRE(softcap >= 0.f && keep_first >= 0, "pico_attnb: cap and kept first positions must not be negative");
  PICO_REQUIRE(gate == nullptr || (gate_heads ? gate_stride >= nq : (gate_stride >= nq * DV && gate_stride % 4 == 0 && (uintptr_t)gate % 8 == 0)),
               "pico_attnb: gate rows must be 8-byte aligned and hold all heads");
  PICO_REQUIRE(chunk >= 0 && (chunk == 0 || window == 0), "pico_attnb: chunks or a window, not both");
  PICO_REQUIRE(v_div >= 1 && nkv % v_div == 0, "pico_attnb: %d kv heads do not share values %d each", nkv, v_div);
  if (T == 0) return 0;
  const int R = nq / nkv;
  const int tpb = R >= 16 ? 1 : 16 / R, hb = R > 16 ? (R + 15) / 16 : 1;
  // every sequence's last block may be partly empty
  const long long tiles = ((long long)(T + tpb - 1) / tpb + num_seqs) * hb;
  PICO_REQUIRE(tiles < (1ll << 30), "pico_attnb: too many blocks");
  BiasArgs a{(const bf16_t*)q, q_stride, (const bf16_t*)k_cache, (const bf16_t*)v_cache, block_table, max_pages,
             cu_seqlens, positions, (bf16_t*)out, num_seqs, nq, nkv, P, num_pages, window, temp_every, scale, temp_coef,
             slope_span, chunks, T * nq, parts_o, parts_ml, softcap, keep_first, (const bf16_t*)gate, gate_stride,
             chunk, sink, gate_heads, v_div, out_f32};
  if (split) {
    attn_bias_kernel<true><<<dim3((unsigned)tiles, nkv, chunks), 256, 0, stream>>>(a);
    if (chunks > 1)
      attn_bias_merge_kernel<<<T * nq, DV <= 64 ? 64 : DV <= 128 ? 128 : 256, 0, stream>>>(parts_o, parts_ml, chunks, T * nq,
                                                                                           (bf16_t*)out, (const bf16_t*)gate,
                                                                                           gate_stride, nq, sink, gate_heads, out_f32);
  } else
    attn_bias_kernel<false><<<dim3((unsigned)((tiles + 3) / 4), nkv), 256, 0, stream>>>(a);
  PICO_LAUNCH_CHECK();
  return 0;
}
