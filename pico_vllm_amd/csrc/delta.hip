// Recurrent mixers whose state is a matrix S [dk, dv] per head and request, walked token by token:
//
//     S <- diag(g_t) S                        (g_t: a decay per key channel, or one per head)
//     u  = beta_t (v_t - S^T k_t)             (the delta rule; without it u = beta_t v_t)
//     S <- S + k_t u^T
//     o_t = S^T q_t                           (the read-out sees the token's own write)
//
// The gated delta rule uses it as it stands; a state-space (duality) layer is the same walk without the correction, with
// k = B, q = C, beta = dt and one decay exp(-a dt) a head.  Query/key heads may be shared by several value heads (head
// h reads q/k head h / (H / KVH)).  Everything here is float32: the state, the decays, beta, the unit norms; only the
// values come in the activations' storage type.
//
//   pico_delta_prep:   unit vectors q, k per head (x / sqrt(sum x^2 + 1e-6), q times qscale), beta = sigmoid(.),
//                      g = exp(-exp(A_log_h) softplus(a2 (a1 h) + dt_bias)) per head and key channel
//   pico_ssd_prep:     dt = softplus(dt_raw + dt_bias), g = exp(-exp(A_log_h) dt) per head; B and C widened to float32
//   pico_delta_scan:   the walk.  A value channel's column of S does not depend on the other columns, so a wave takes
//                      64 / KS columns with the key channels of each cut over KS lanes (KPL channels a lane, in
//                      registers for the whole step); the two sums over key channels meet across those lanes.
//   pico_gated_group_norm: (y + D_h x) silu(z), RMS-normed in equal parts of the row, times a weight
#include "common.h"

__device__ __forceinline__ float softplus_f(float z) { return z > 20.f ? z : log1pf(expf(z)); }
__device__ __forceinline__ float sigmoid_f(float z) { return 1.0f / (1.0f + expf(-z)); }

// grid (T); x: the convolved q | k (columns q_col .., k_col .., KVH heads of dk each); y: the row that holds beta's
// logits (b_col, H of them) and the low-rank activations (a_col, R of them); a2 [H * dk, R].
template <typename T>
__global__ __launch_bounds__(1024) void delta_prep_kernel(const T* __restrict__ x, int ldx, int q_col, int k_col,
                                                         const T* __restrict__ y, int ldy, int b_col, int a_col,
                                                         const T* __restrict__ a2, const float* __restrict__ dt_bias,
                                                         const float* __restrict__ a_log, float qscale, float* __restrict__ qn,
                                                         float* __restrict__ kn, float* __restrict__ g, float* __restrict__ beta,
                                                         int H, int KVH, int dk, int R) {
  extern __shared__ float low[];           // [R]
  const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  const T* yr = y + (size_t)t * ldy;
  for (int r = threadIdx.x; r < R; r += blockDim.x) low[r] = load_f32(yr + a_col + r);
  __syncthreads();
  for (int u = wave; u < 2 * KVH; u += nw) {
    const bool is_q = u < KVH;
    const int hh = is_q ? u : u - KVH;
    const T* src = x + (size_t)t * ldx + (is_q ? q_col : k_col) + (size_t)hh * dk;
    float ss = 0.f;
    for (int i = lane; i < dk; i += 64) { const float v = load_f32(src + i); ss = fmaf(v, v, ss); }
    const float r = (is_q ? qscale : 1.0f) / sqrtf(wave_sum(ss) + 1e-6f);
    float* dst = (is_q ? qn : kn) + ((size_t)t * KVH + hh) * dk;
    for (int i = lane; i < dk; i += 64) dst[i] = load_f32(src + i) * r;
  }
  for (int c = threadIdx.x; c < H * dk; c += blockDim.x) {
    const T* w = a2 + (size_t)c * R;
    float z = dt_bias[c];
    for (int r = 0; r < R; r++) z = fmaf(load_f32(w + r), low[r], z);
    g[(size_t)t * H * dk + c] = expf(-expf(a_log[c / dk]) * softplus_f(z));
  }
  for (int h = threadIdx.x; h < H; h += blockDim.x) beta[(size_t)t * H + h] = sigmoid_f(load_f32(yr + b_col + h));
}

extern "C" int pico_delta_prep(const void* x, int ldx, int q_col, int k_col, const void* y, int ldy, int b_col, int a_col,
                               int dtype, const void* a2, const float* dt_bias, const float* a_log, float qscale, float* qn,
                               float* kn, float* g, float* beta, int T, int H, int KVH, int dk, int R, hipStream_t stream) {
  PICO_REQUIRE(T >= 0 && H > 0 && KVH > 0 && H % KVH == 0 && dk > 0 && R > 0 && R <= 8192, "pico_delta_prep: bad sizes");
  PICO_REQUIRE(ldx >= q_col + KVH * dk && ldx >= k_col + KVH * dk && ldy >= b_col + H && ldy >= a_col + R,
               "pico_delta_prep: the rows do not hold what is read");
  if (T == 0) return 0;
  const size_t lds = (size_t)R * sizeof(float);
  const int threads = T >= 64 ? 256 : 1024;       // few tokens: a thread a decay, so that their sums run side by side
  if (dtype == PICO_DTYPE_F32)
    delta_prep_kernel<float><<<T, threads, lds, stream>>>((const float*)x, ldx, q_col, k_col, (const float*)y, ldy, b_col, a_col,
                                                      (const float*)a2, dt_bias, a_log, qscale, qn, kn, g, beta, H, KVH, dk, R);
  else if (dtype == PICO_DTYPE_BF16)
    delta_prep_kernel<bf16_t><<<T, threads, lds, stream>>>((const bf16_t*)x, ldx, q_col, k_col, (const bf16_t*)y, ldy, b_col, a_col,
                                                       (const bf16_t*)a2, dt_bias, a_log, qscale, qn, kn, g, beta, H, KVH, dk, R);
  else
    PICO_REQUIRE(false, "pico_delta_prep: unknown dtype %d", dtype);
  PICO_LAUNCH_CHECK();
  return 0;
}

// grid (T); bc: the convolved B | C (columns b_col .., c_col .., n each); dt_raw: H columns of y from dt_col.
template <typename T>
__global__ __launch_bounds__(256) void ssd_prep_kernel(const T* __restrict__ bc, int ldb, int b_col, int c_col, int n,
                                                       const T* __restrict__ y, int ldy, int dt_col,
                                                       const float* __restrict__ dt_bias, const float* __restrict__ a_log,
                                                       float* __restrict__ bf, float* __restrict__ cf, float* __restrict__ g,
                                                       float* __restrict__ dt, int H) {
  const int t = blockIdx.x;
  const T* br = bc + (size_t)t * ldb;
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    bf[(size_t)t * n + i] = load_f32(br + b_col + i);
    cf[(size_t)t * n + i] = load_f32(br + c_col + i);
  }
  for (int h = threadIdx.x; h < H; h += blockDim.x) {
    const float d = softplus_f(load_f32(y + (size_t)t * ldy + dt_col + h) + dt_bias[h]);
    dt[(size_t)t * H + h] = d;
    g[(size_t)t * H + h] = expf(-expf(a_log[h]) * d);
  }
}

extern "C" int pico_ssd_prep(const void* bc, int ldb, int b_col, int c_col, int n, const void* y, int ldy, int dt_col, int dtype,
                             const float* dt_bias, const float* a_log, float* bf, float* cf, float* g, float* dt, int T, int H,
                             hipStream_t stream) {
  PICO_REQUIRE(T >= 0 && H > 0 && n > 0 && ldb >= b_col + n && ldb >= c_col + n && ldy >= dt_col + H, "pico_ssd_prep: bad sizes");
  if (T == 0) return 0;
  if (dtype == PICO_DTYPE_F32)
    ssd_prep_kernel<float><<<T, 256, 0, stream>>>((const float*)bc, ldb, b_col, c_col, n, (const float*)y, ldy, dt_col, dt_bias,
                                                  a_log, bf, cf, g, dt, H);
  else if (dtype == PICO_DTYPE_BF16)
    ssd_prep_kernel<bf16_t><<<T, 256, 0, stream>>>((const bf16_t*)bc, ldb, b_col, c_col, n, (const bf16_t*)y, ldy, dt_col, dt_bias,
                                                   a_log, bf, cf, g, dt, H);
  else
    PICO_REQUIRE(false, "pico_ssd_prep: unknown dtype %d", dtype);
  PICO_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------
// The walk.  grid (sequences, heads, column tiles); a workgroup of up to four waves owns a tile of value columns of one
// head of one sequence.  In a wave VC = 64 / KS lanes stand side by side over columns and KS lanes share a column, each
// with KPL of its key channels; a lane owns VPL columns (VC apart), so what it reads of a token's k, g and q serves them
// all: a thread keeps KPL * VPL state elements in registers for the whole step.  Tokens are taken TB at a time: their k,
// q, decays, beta and the tile's values are staged in LDS by the whole workgroup (every load unconditional, from a
// clamped address).  The sums over key channels are added lane-locally in channel order and then across the KS lanes
// of a column in a fixed tree: a token's output does not depend on how its sequence was cut into steps or on what else
// the step holds.
//
// Long portions are cut into chunks of `chunk` tokens that run side by side.  A chunk maps the state in front of it to
// the state behind it as S -> P S + L, with P [dk, dk] and L [dk, dv] that depend on the chunk's tokens alone:
//   DS_LOCAL:  every chunk from a state of zero with its values: L.  With the delta rule P = prod_t (I - beta k k^T) diag(g)
//              is no diagonal matrix; its column e is what the walk makes of the unit vector e with values of zero, so
//              the same walk takes dk more columns (a state of [0 | I], values [v | 0]) and leaves [L | P].  Without the
//              delta rule P is the product of the chunk's decays, a number a key channel.
//   (the combine kernels walk a sequence's chunks: ws_S[c] <- the state in front of chunk c, and the slot's final state)
//   DS_FROM:   every chunk again from ws_S[chunk], writing the outputs
// DS_WHOLE is the plain walk from the slot's state.  blockIdx.x = sequence * max_chunks + chunk in the chunked modes.
// ---------------------------------------------------------------------------
#define DS_WHOLE 0
#define DS_LOCAL 1
#define DS_FROM 2

template <typename TV, int KPL, int VPL, bool DELTA, int MODE>
__global__ __launch_bounds__(256) void delta_scan_kernel(const float* __restrict__ q, const float* __restrict__ k,
                                                         const TV* __restrict__ v, int ldv, const float* __restrict__ g,
                                                         int g_channels, const float* __restrict__ beta,
                                                         const int* __restrict__ cu_seqlens, const int* __restrict__ state_slots,
                                                         float* __restrict__ state, float* __restrict__ out, int H, int KVH,
                                                         int dk, int dv, int KS, int TB, int num_slots, int chunk,
                                                         int max_chunks, float* __restrict__ ws_S, float* __restrict__ ws_P) {
  extern __shared__ float lds[];
  const int b = MODE == DS_WHOLE ? blockIdx.x : blockIdx.x / max_chunks, h = blockIdx.y;
  const int nw = blockDim.x >> 6, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int VC = 64 / KS, vc = lane % VC, ks = lane / VC;
  const int DKP = KS * KPL;                            // key channels with padding
  const int tile = nw * VC * VPL;                      // columns of the workgroup
  float* ks_ = lds;                                    // [TB][DKP]
  float* qs_ = ks_ + TB * DKP;
  float* gs_ = qs_ + TB * DKP;
  float* vs_ = gs_ + TB * DKP;                         // [TB][tile]
  float* bs_ = vs_ + TB * tile;                        // [TB]
  int t_begin = cu_seqlens[b], t_end = cu_seqlens[b + 1];
  if (MODE != DS_WHOLE) {
    t_begin += (blockIdx.x % max_chunks) * chunk;
    t_end = min(t_end, t_begin + chunk);
  }
  const int slot = state_slots[b];
  if (slot < 0 || slot >= num_slots || t_end <= t_begin) return;          // the whole workgroup
  const int ncols = (MODE == DS_LOCAL && DELTA) ? dv + dk : dv;           // the unit vectors' columns behind the values'
  const int col0 = blockIdx.z * tile, lcol0 = wave * VC * VPL + vc;       // the tile's first column; this lane's first in the tile
  const int c0 = ks * KPL;
  const int kvh = h / (H / KVH);
  float* sbase = MODE == DS_WHOLE ? state + (((size_t)slot * H + h) * dk) * dv
                                  : ws_S + (((size_t)blockIdx.x * H + h) * dk) * dv;
  // The state's loads are unconditional, from addresses clamped into the tensor, and what must not count is cleared in a
  // loop of its own: a load whose value is selected right behind it is waited for there, and a thread's loads then queue
  // one behind the other's latency instead of travelling together.
  float S[VPL][KPL];
  if (MODE != DS_LOCAL) {
#pragma unroll
    for (int j = 0; j < VPL; j++)
#pragma unroll
      for (int i = 0; i < KPL; i++)
        S[j][i] = sbase[(size_t)min(c0 + i, dk - 1) * dv + min(col0 + lcol0 + j * VC, dv - 1)];
  }
#pragma unroll
  for (int j = 0; j < VPL; j++) {
    const int col = col0 + lcol0 + j * VC;
#pragma unroll
    for (int i = 0; i < KPL; i++) {
      if (MODE == DS_LOCAL) S[j][i] = (col >= dv && col < ncols && c0 + i == col - dv) ? 1.f : 0.f;
      else S[j][i] = (c0 + i < dk && col < dv) ? S[j][i] : 0.f;
    }
  }
  float gprod[KPL];                                    // DS_LOCAL without the delta rule: the chunk's decays multiplied up
#pragma unroll
  for (int i = 0; i < KPL; i++) gprod[i] = 1.f;
  for (int t0 = t_begin; t0 < t_end; t0 += TB) {
    const int nb = min(TB, t_end - t0);
    __syncthreads();                                   // the last block's staged values have been read
    for (int idx = threadIdx.x; idx < nb * DKP; idx += blockDim.x) {      // only the block's tokens: a single token is one turn
      const int tt = idx / DKP, c = idx % DKP;
      const int t = t0 + min(tt, nb - 1), cc = min(c, dk - 1);
      const bool in = tt < nb && c < dk;
      const float kx = k[((size_t)t * KVH + kvh) * dk + cc];
      const float qx = MODE == DS_LOCAL ? 0.f : q[((size_t)t * KVH + kvh) * dk + cc];
      const float gx = g_channels ? g[((size_t)t * H + h) * dk + cc] : g[(size_t)t * H + h];
      ks_[idx] = in ? kx : 0.f;
      qs_[idx] = in ? qx : 0.f;
      gs_[idx] = in ? gx : 1.f;
    }
    for (int idx = threadIdx.x; idx < nb * tile; idx += blockDim.x) {
      const int tt = idx / tile, col = col0 + idx % tile;
      const float x = load_f32(v + (size_t)(t0 + min(tt, nb - 1)) * ldv + (size_t)h * dv + min(col, dv - 1));
      vs_[idx] = (tt < nb && col < dv) ? x : 0.f;       // the unit vectors' columns have values of zero
    }
    if ((int)threadIdx.x < TB) bs_[threadIdx.x] = beta[(size_t)(t0 + min((int)threadIdx.x, nb - 1)) * H + h];
    __syncthreads();
    for (int tt = 0; tt < nb; tt++) {
      const float4* k4 = reinterpret_cast<const float4*>(ks_ + tt * DKP + c0);
      const float4* g4 = reinterpret_cast<const float4*>(gs_ + tt * DKP + c0);
      const float4* q4 = reinterpret_cast<const float4*>(qs_ + tt * DKP + c0);
      const float bt = bs_[tt];
      float kc[KPL], u[VPL];
#pragma unroll
      for (int j = 0; j < VPL; j++) u[j] = 0.f;
#pragma unroll
      for (int i = 0; i < KPL / 4; i++) {
        const float4 kv = k4[i], gv = g4[i];
        kc[4 * i] = kv.x; kc[4 * i + 1] = kv.y; kc[4 * i + 2] = kv.z; kc[4 * i + 3] = kv.w;
        if (MODE == DS_LOCAL && !DELTA) { gprod[4 * i] *= gv.x; gprod[4 * i + 1] *= gv.y; gprod[4 * i + 2] *= gv.z; gprod[4 * i + 3] *= gv.w; }
#pragma unroll
        for (int j = 0; j < VPL; j++) {
          S[j][4 * i] *= gv.x; S[j][4 * i + 1] *= gv.y; S[j][4 * i + 2] *= gv.z; S[j][4 * i + 3] *= gv.w;
          if (DELTA) {
            u[j] = fmaf(S[j][4 * i], kv.x, u[j]); u[j] = fmaf(S[j][4 * i + 1], kv.y, u[j]);
            u[j] = fmaf(S[j][4 * i + 2], kv.z, u[j]); u[j] = fmaf(S[j][4 * i + 3], kv.w, u[j]);
          }
        }
      }
#pragma unroll
      for (int j = 0; j < VPL; j++) {
        const float vt = vs_[tt * tile + lcol0 + j * VC];
        if (DELTA) {
          float sk = u[j];
          for (int o = VC; o < 64; o <<= 1) sk += __shfl_xor(sk, o);
          u[j] = bt * (vt - sk);
        } else {
          u[j] = bt * vt;
        }
      }
      if (MODE == DS_LOCAL) {
#pragma unroll
        for (int j = 0; j < VPL; j++)
#pragma unroll
          for (int i = 0; i < KPL; i++) S[j][i] = fmaf(kc[i], u[j], S[j][i]);
        continue;
      }
      float so[VPL];
#pragma unroll
      for (int j = 0; j < VPL; j++) so[j] = 0.f;
#pragma unroll
      for (int i = 0; i < KPL / 4; i++) {
        const float4 qv = q4[i];
#pragma unroll
        for (int j = 0; j < VPL; j++) {
          S[j][4 * i] = fmaf(kc[4 * i], u[j], S[j][4 * i]); so[j] = fmaf(S[j][4 * i], qv.x, so[j]);
          S[j][4 * i + 1] = fmaf(kc[4 * i + 1], u[j], S[j][4 * i + 1]); so[j] = fmaf(S[j][4 * i + 1], qv.y, so[j]);
          S[j][4 * i + 2] = fmaf(kc[4 * i + 2], u[j], S[j][4 * i + 2]); so[j] = fmaf(S[j][4 * i + 2], qv.z, so[j]);
          S[j][4 * i + 3] = fmaf(kc[4 * i + 3], u[j], S[j][4 * i + 3]); so[j] = fmaf(S[j][4 * i + 3], qv.w, so[j]);
        }
      }
#pragma unroll
      for (int j = 0; j < VPL; j++) {
        float x = so[j];
        for (int o = VC; o < 64; o <<= 1) x += __shfl_xor(x, o);
        const int col = col0 + lcol0 + j * VC;
        if (ks == 0 && col < dv) out[((size_t)(t0 + tt) * H + h) * dv + col] = x;
      }
    }
  }
  if (MODE == DS_FROM) return;
#pragma unroll
  for (int j = 0; j < VPL; j++) {
    const int col = col0 + lcol0 + j * VC;
    if (col >= ncols) continue;
    if (col >= dv) {                                   // DS_LOCAL with the delta rule: column col - dv of P
      float* pp = ws_P + (((size_t)blockIdx.x * H + h) * dk) * dk + (col - dv);
#pragma unroll
      for (int i = 0; i < KPL; i++)
        if (c0 + i < dk) pp[(size_t)(c0 + i) * dk] = S[j][i];
      continue;
    }
#pragma unroll
    for (int i = 0; i < KPL; i++)
      if (c0 + i < dk) sbase[(size_t)(c0 + i) * dv + col] = S[j][i];
    if (MODE == DS_LOCAL && !DELTA && col == 0) {
#pragma unroll
      for (int i = 0; i < KPL; i++)
        if (c0 + i < dk) ws_P[((size_t)blockIdx.x * H + h) * dk + c0 + i] = gprod[i];
    }
  }
}

// The walk over a sequence's chunks without the delta rule, one thread per state element: ws_S[c] becomes the state in
// front of chunk c, the slot gets the state behind the last chunk.  grid (sequences, heads, ceil(dk dv / 256)).
__global__ __launch_bounds__(256) void decay_combine_kernel(const int* __restrict__ cu_seqlens, const int* __restrict__ state_slots,
                                                            float* __restrict__ state, float* __restrict__ ws_S,
                                                            const float* __restrict__ ws_P, int H, int dk, int dv, int num_slots,
                                                            int chunk, int max_chunks) {
  const int b = blockIdx.x, h = blockIdx.y, e = blockIdx.z * 256 + threadIdx.x;
  if (e >= dk * dv) return;
  const int slot = state_slots[b], n = cu_seqlens[b + 1] - cu_seqlens[b];
  if (slot < 0 || slot >= num_slots || n <= 0) return;
  const int i = e / dv;
  float* sp = state + ((size_t)slot * H + h) * dk * dv + e;
  float s = *sp;
  const int chunks = (n + chunk - 1) / chunk;
  for (int c = 0; c < chunks; c++) {
    const size_t blk = (size_t)b * max_chunks + c;
    float* lp = ws_S + (blk * H + h) * dk * dv + e;
    const float local = *lp, p = ws_P[(blk * H + h) * dk + i];
    *lp = s;
    s = fmaf(p, s, local);
  }
  *sp = s;
}

// The same with the delta rule: S <- P S + L with a full matrix P [dk, dk] a chunk.  grid (sequences, heads,
// ceil(dv / 16)); a workgroup of 256 threads owns 16 value columns, thread (r, j) the rows r, r + 16, .. of column j.
// The tile of the state and, ET columns at a time, the chunk's P stand in LDS for the products.  The walk is a chain of
// as many steps as the sequence has chunks, so a step must not wait for memory: the next tile of P (at most 16 floats a
// thread) and the next chunk's L travel in registers while this tile's products run.
#define DC_ROWS 32          // rows a thread: 512 key channels at most
#define DC_TILE 16          // floats of a tile of P a thread holds on their way to LDS
__global__ __launch_bounds__(256) void delta_combine_kernel(const int* __restrict__ cu_seqlens, const int* __restrict__ state_slots,
                                                            float* __restrict__ state, float* __restrict__ ws_S,
                                                            const float* __restrict__ ws_P, int H, int dk, int dv, int num_slots,
                                                            int chunk, int max_chunks, int ET) {
  extern __shared__ float sh[];           // [dk + 3][16] the state's tile (three rows of zeros behind it), then [dk][ET] of P
  float* pt = sh + (dk + 3) * 16;          // ET is a multiple of 4: the columns behind the last of P hold zeros
  if (threadIdx.x < 48) sh[dk * 16 + threadIdx.x] = 0.f;
  const int b = blockIdx.x, h = blockIdx.y, j = threadIdx.x & 15, r = threadIdx.x >> 4;
  const int col = blockIdx.z * 16 + j, cin = min(col, dv - 1);
  const int slot = state_slots[b], n = cu_seqlens[b + 1] - cu_seqlens[b];
  if (slot < 0 || slot >= num_slots || n <= 0) return;          // the whole workgroup
  const int rows = (dk - r + 15) / 16;                          // rows r, r + 16, .. below dk
  const int ntile = (dk + ET - 1) / ET;
  const int chunks = (n + chunk - 1) / chunk;
  float s[DC_ROWS], acc[DC_ROWS], lnext[DC_ROWS], pre[DC_TILE];
  float* sp = state + ((size_t)slot * H + h) * dk * dv + cin;
  // every load is unconditional, from a clamped address; what must not count is never used
  auto load_local = [&](int c) {
    const float* lp = ws_S + ((((size_t)b * max_chunks + c) * H + h) * dk) * dv + cin;
#pragma unroll
    for (int x = 0; x < DC_ROWS; x++)
      if (x < rows) lnext[x] = lp[(size_t)min(r + 16 * x, dk - 1) * dv];
  };
  // ET is a power of two: a thread's place in a tile is a shift and a mask away
  const int eshift = 31 - __clz(ET);
  auto fetch_tile = [&](int c, int tile) {
    const float* pm = ws_P + ((((size_t)b * max_chunks + c) * H + h) * dk) * dk;
    const int e0 = tile * ET;
#pragma unroll
    for (int m = 0; m < DC_TILE; m++) {
      const int idx = (int)threadIdx.x + 256 * m, i = idx >> eshift, ee = idx & (ET - 1);
      pre[m] = pm[(size_t)min(i, dk - 1) * dk + min(e0 + ee, dk - 1)];
    }
  };
  auto store_tile = [&](int tile) {
    const int e0 = tile * ET, ne = min(ET, dk - e0);
#pragma unroll
    for (int m = 0; m < DC_TILE; m++) {
      const int idx = (int)threadIdx.x + 256 * m, i = idx >> eshift, ee = idx & (ET - 1);
      if (i < dk) pt[idx] = ee < ne ? pre[m] : 0.f;
    }
  };
#pragma unroll
  for (int x = 0; x < DC_ROWS; x++)
    if (x < rows) s[x] = sp[(size_t)(r + 16 * x) * dv];
  load_local(0);
  fetch_tile(0, 0);
  for (int c = 0; c < chunks; c++) {
    float* lp = ws_S + ((((size_t)b * max_chunks + c) * H + h) * dk) * dv + cin;
    __syncthreads();                                            // the last chunk's products have read the tiles
#pragma unroll
    for (int x = 0; x < DC_ROWS; x++) {
      if (x < rows) {
        sh[(r + 16 * x) * 16 + j] = s[x];
        acc[x] = lnext[x];                                      // what the chunk makes of a state of zero
      }
    }
    for (int tile = 0; tile < ntile; tile++) {
      const int e0 = tile * ET, ne4 = (min(ET, dk - e0) + 3) & ~3;
      if (tile > 0) __syncthreads();                            // the last tile's products have read it
      store_tile(tile);
      __syncthreads();                                          // the state's tile and this tile of P are written
      // everything that goes to or comes from memory is issued here, behind the barrier (which waits for what is under
      // way) and in front of the products, under which it travels
      if (tile + 1 < ntile) fetch_tile(c, tile + 1);
      else if (c + 1 < chunks) fetch_tile(c + 1, 0);
      if (tile == 0) {
        if (col < dv) {
#pragma unroll
          for (int x = 0; x < DC_ROWS; x++)
            if (x < rows) lp[(size_t)(r + 16 * x) * dv] = s[x];  // the state in front of this chunk
        }
        if (c + 1 < chunks) load_local(c + 1);
      }
      // four columns of P a turn: the state's four entries serve all rows of the thread, whose sums do not wait for one another
      const float* sc = sh + e0 * 16 + j;
#pragma unroll 2
      for (int ee = 0; ee < ne4; ee += 4) {
        const float s0 = sc[ee * 16], s1 = sc[(ee + 1) * 16], s2 = sc[(ee + 2) * 16], s3 = sc[(ee + 3) * 16];
#pragma unroll
        for (int x = 0; x < DC_ROWS; x++) {
          if (x >= rows) break;
          const float4 p4 = *reinterpret_cast<const float4*>(pt + (r + 16 * x) * ET + ee);
          acc[x] = fmaf(p4.w, s3, fmaf(p4.z, s2, fmaf(p4.y, s1, fmaf(p4.x, s0, acc[x]))));
        }
      }
    }
#pragma unroll
    for (int x = 0; x < DC_ROWS; x++)
      if (x < rows) s[x] = acc[x];
  }
  if (col < dv) {
#pragma unroll
    for (int x = 0; x < DC_ROWS; x++)
      if (x < rows) sp[(size_t)(r + 16 * x) * dv] = s[x];
  }
}

#define DELTA_MAX_KEY_DIM 512

extern "C" int pico_delta_scan(const float* q, const float* k, const void* v, int ldv, int v_dtype, const float* g,
                               int g_channels, const float* beta, const int* cu_seqlens, const int* state_slots, float* state,
                               float* out, int num_seqs, int T, int H, int KVH, int dk, int dv, int num_slots, int delta, int chunk,
                               int max_chunks, float* ws_S, float* ws_P, hipStream_t stream) {
  PICO_REQUIRE(num_seqs >= 0 && H > 0 && KVH > 0 && H % KVH == 0 && dk > 0 && dk <= DELTA_MAX_KEY_DIM && dv > 0 && num_slots > 0,
               "pico_delta_scan: bad sizes (at most %d key channels a head)", DELTA_MAX_KEY_DIM);
  PICO_REQUIRE(ldv >= H * dv && H <= 65535, "pico_delta_scan: the rows do not hold the values");
  PICO_REQUIRE(chunk >= 0 && (chunk == 0 || (max_chunks > 0 && ws_S && ws_P)), "pico_delta_scan: chunks need their workspace");
  if (num_seqs == 0) return 0;
  // key channels a lane: the fewest of 4, 8, 16, 32 with which at most 4 lanes share a column; beyond 128 channels
  // more lanes a column.  Two columns a lane where a head has 32 or more; as many waves (up to four) as the columns ask for.
  int kpl = 4;
  while (kpl < 32 && 4 * kpl < dk) kpl *= 2;
  int KS = 1;
  while (KS * kpl < dk) KS *= 2;
  const int VC = 64 / KS, DKP = KS * kpl;
  // A step of single tokens is the state read and written once: one column a lane and one wave a workgroup there, four
  // times the workgroups with a quarter of the loads each in front of the one token's arithmetic.  (A column's sums are
  // the same whatever the tiling.)
  const bool few = chunk == 0 && T <= 2 * num_seqs;
  const int vpl = dv >= 32 && !few ? 2 : 1;
  const int TB = DKP > 256 ? 8 : 16;
  const unsigned nblk = (unsigned)(num_seqs * (chunk ? max_chunks : 1));
  auto waves = [&](int cols) { return few ? 1 : min(4, max(1, (cols + VC * vpl - 1) / (VC * vpl))); };
  auto lds_bytes = [&](int nw) { return (size_t)(3 * TB * DKP + TB * nw * VC * vpl + TB) * sizeof(float); };
  auto tiles = [&](int cols, int nw) { return (unsigned)((cols + nw * VC * vpl - 1) / (nw * VC * vpl)); };
  // columns of P in LDS at a time: a power of two from 4, as many as a workgroup's threads carry 16 floats each of
  int ET = 4;
  while (2 * ET * dk <= 256 * DC_TILE && ET < dk) ET *= 2;
  const int cols_local = delta ? dv + dk : dv;
  const int nw_v = waves(dv), nw_l = waves(cols_local);
  PICO_REQUIRE(tiles(cols_local, nw_l) <= 65535 && (dv + 15) / 16 <= 65535 && ((size_t)dk * dv + 255) / 256 <= 65535,
               "pico_delta_scan: too many value channels");
#define ARGS(TV) q, k, (const TV*)v, ldv, g, g_channels, beta, cu_seqlens, state_slots, state, out, H, KVH, dk, dv, KS, TB, num_slots, \
                 chunk, max_chunks, ws_S, ws_P
#define GO(TV, KPL, VPL, D)                                                                                                  \
  do {                                                                                                                       \
    if (chunk == 0) {                                                                                                        \
      delta_scan_kernel<TV, KPL, VPL, D, DS_WHOLE><<<dim3(nblk, H, tiles(dv, nw_v)), 64 * nw_v, lds_bytes(nw_v), stream>>>(ARGS(TV)); \
    } else {                                                                                                                 \
      delta_scan_kernel<TV, KPL, VPL, D, DS_LOCAL><<<dim3(nblk, H, tiles(cols_local, nw_l)), 64 * nw_l, lds_bytes(nw_l), stream>>>(ARGS(TV)); \
      if (D)                                                                                                                 \
        delta_combine_kernel<<<dim3(num_seqs, H, (dv + 15) / 16), 256, ((size_t)dk * (16 + ET) + 48) * sizeof(float), stream>>>( \
            cu_seqlens, state_slots, state, ws_S, ws_P, H, dk, dv, num_slots, chunk, max_chunks, ET);                        \
      else                                                                                                                   \
        decay_combine_kernel<<<dim3(num_seqs, H, (dk * dv + 255) / 256), 256, 0, stream>>>(                                  \
            cu_seqlens, state_slots, state, ws_S, ws_P, H, dk, dv, num_slots, chunk, max_chunks);                            \
      delta_scan_kernel<TV, KPL, VPL, D, DS_FROM><<<dim3(nblk, H, tiles(dv, nw_v)), 64 * nw_v, lds_bytes(nw_v), stream>>>(ARGS(TV)); \
    }                                                                                                                        \
  } while (0)
#define PICK2(TV, KPL, D)                  \
  do {                                     \
    if (vpl == 2) GO(TV, KPL, 2, D);       \
    else GO(TV, KPL, 1, D);                \
  } while (0)
#define PICK(TV, D)                       \
  do {                                    \
    if (kpl == 4) PICK2(TV, 4, D);        \
    else if (kpl == 8) PICK2(TV, 8, D);   \
    else if (kpl == 16) PICK2(TV, 16, D); \
    else PICK2(TV, 32, D);                \
  } while (0)
  if (v_dtype == PICO_DTYPE_F32) { if (delta) PICK(float, true); else PICK(float, false); }
  else if (v_dtype == PICO_DTYPE_BF16) { if (delta) PICK(bf16_t, true); else PICK(bf16_t, false); }
  else PICO_REQUIRE(false, "pico_delta_scan: unknown dtype %d", v_dtype);
#undef PICK
#undef PICK2
#undef GO
#undef ARGS
  PICO_LAUNCH_CHECK();
  return 0;
}

// out[t] = norm_groups( (y[t] + D_h x[t]) * silu(z[t]) ) * w: the row of H * dv entries is cut into `groups` equal parts,
// each over its own root mean square.  grid (T, groups); y float32 [T, H * dv]; x, z columns of wider rows.
template <typename T>
__global__ __launch_bounds__(1024) void gated_group_norm_kernel(const float* __restrict__ y, const T* __restrict__ x, int ldx,
                                                               const T* __restrict__ z, int ldz, const float* __restrict__ D,
                                                               const float* __restrict__ w, float eps, T* __restrict__ out,
                                                               int H, int dv, int groups) {
  extern __shared__ float part[];
  __shared__ float scratch[16];
  const int t = blockIdx.x, gi = blockIdx.y, n = H * dv / groups, base = gi * n;
  float ss = 0.f;
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    const int c = base + i;
    const float zz = load_f32(z + (size_t)t * ldz + c);
    const float val = fmaf(D[c / dv], load_f32(x + (size_t)t * ldx + c), y[(size_t)t * H * dv + c]) * (zz / (1.0f + expf(-zz)));
    part[i] = val;
    ss = fmaf(val, val, ss);
  }
  const float r = 1.0f / sqrtf(block_sum(ss, scratch) / (float)n + eps);
  for (int i = threadIdx.x; i < n; i += blockDim.x) store_f32(out + (size_t)t * H * dv + base + i, part[i] * r * w[base + i]);
}

extern "C" int pico_gated_group_norm(const float* y, const void* x, int ldx, const void* z, int ldz, int dtype, const float* D,
                                     const float* w, float eps, void* out, int T, int H, int dv, int groups,
                                     hipStream_t stream) {
  PICO_REQUIRE(T >= 0 && H > 0 && dv > 0 && groups > 0 && (H * dv) % groups == 0 && groups <= 65535, "pico_gated_group_norm: bad sizes");
  PICO_REQUIRE(H * dv / groups <= 16384 && ldx >= H * dv && ldz >= H * dv, "pico_gated_group_norm: a part of at most 16384 entries");
  if (T == 0) return 0;
  const size_t lds = (size_t)(H * dv / groups) * sizeof(float);
  const dim3 grid(T, groups);
  const int threads = T >= 64 ? 256 : 1024;       // few tokens: a thread's loads are one turn and travel together
  if (dtype == PICO_DTYPE_F32)
    gated_group_norm_kernel<float><<<grid, threads, lds, stream>>>(y, (const float*)x, ldx, (const float*)z, ldz, D, w, eps, (float*)out, H, dv, groups);
  else if (dtype == PICO_DTYPE_BF16)
    gated_group_norm_kernel<bf16_t><<<grid, threads, lds, stream>>>(y, (const bf16_t*)x, ldx, (const bf16_t*)z, ldz, D, w, eps, (bf16_t*)out, H, dv, groups);
  else
    PICO_REQUIRE(false, "pico_gated_group_norm: unknown dtype %d", dtype);
  PICO_LAUNCH_CHECK();
  return 0;
}
