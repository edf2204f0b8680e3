// A feed-forward made of many small experts, of which every token uses a few:
//   route    scores of the router's logits, the choice of experts within the best groups, weights
//   sort     the (token, choice) pairs listed by expert
//   products x W_e^T for every expert's pairs: gate|up with the gated activation, then down
//   combine  the weighted sum of a token's experts, plus what a shared expert gave
// float32 and bfloat16 storage; scores, weights and sums are float32.  A pair is p = token * top + choice.
#include "common.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float sigmoid_f(float z) { return 1.0f / (1.0f + expf(-z)); }

// ---------------------------------------------------------------------------------------
// Router.  z [N, E] float32 logits.  s = sigmoid(z) (score_fn 0) or softmax(z) over the experts
// (score_fn 1).  Experts e with the same e / (E / groups) are one group, ranked by the sum of its
// top two s (its only one, if it has one member); the choice is the `top` highest s among the members
// of the `keep` highest-ranked groups (ties: the lower index).  Weights: the
// chosen s divided by (their sum + floor) if `normalize`, times `scale`.
// One wave per token; E <= 512, groups <= 64.
// ---------------------------------------------------------------------------------------
#define MOE_MAX_E 512

__global__ __launch_bounds__(256) void moe_route_kernel(const float* __restrict__ z, int* __restrict__ ids,
                                                        float* __restrict__ wts, int N, int E, int top, int groups,
                                                        int keep, float scale, int score_fn, int normalize,
                                                        float floor_) {
  __shared__ float s_all[4][MOE_MAX_E];
  __shared__ float g_all[4][64];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int n = blockIdx.x * 4 + wave;
  if (n >= N) return;
  float* s = s_all[wave];
  float* gs = g_all[wave];
  const float* zr = z + (size_t)n * E;
  if (score_fn == 1) {
    float mx = -INFINITY;
    for (int e = lane; e < E; e += 64) mx = fmaxf(mx, zr[e]);
    mx = wave_max(mx);
    float sum = 0.f;
    for (int e = lane; e < E; e += 64) {
      const float v = expf(zr[e] - mx);
      s[e] = v;
      sum += v;
    }
    sum = wave_sum(sum);
    for (int e = lane; e < E; e += 64) s[e] = s[e] / sum;
  } else {
    for (int e = lane; e < E; e += 64) s[e] = sigmoid_f(zr[e]);
  }
  __builtin_amdgcn_wave_barrier();
  const int per = E / groups;
  if (lane < groups) {
    float a = -INFINITY, b = -INFINITY;   // the two largest
    for (int i = 0; i < per; ++i) {
      const float v = s[lane * per + i];
      if (v > a) { b = a; a = v; }
      else if (v > b) b = v;
    }
    gs[lane] = per > 1 ? a + b : a;
  }
  __builtin_amdgcn_wave_barrier();
  bool allowed_group = false;
  if (lane < groups) {
    int ahead = 0;
    const float mine = gs[lane];
    for (int g = 0; g < groups; ++g) ahead += (gs[g] > mine || (gs[g] == mine && g < lane)) ? 1 : 0;
    allowed_group = ahead < keep;
  }
  const unsigned long long allowed = __ballot(allowed_group);
  // this lane's experts: e = lane + 64 i; a score of -1 can never be chosen before an allowed one
  float cand[MOE_MAX_E / 64];
#pragma unroll
  for (int i = 0; i < MOE_MAX_E / 64; ++i) {
    const int e = lane + 64 * i;
    cand[i] = (e < E && ((allowed >> (e / per)) & 1ull)) ? s[e] : -1.0f;
  }
  float total = 0.f;
  float my_w = 0.f;   // lane t keeps the weight of choice t (top <= 64)
  int my_id = 0;
  for (int t = 0; t < top; ++t) {
    float best = -2.0f;
    int at = 0x7fffffff;
#pragma unroll
    for (int i = 0; i < MOE_MAX_E / 64; ++i)
      if (cand[i] > best) { best = cand[i]; at = lane + 64 * i; }
    // the wave's best: larger score first, then the lower index
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ob = __shfl_xor(best, o, QVL_WAVE);
      const int oa = __shfl_xor(at, o, QVL_WAVE);
      if (ob > best || (ob == best && oa < at)) { best = ob; at = oa; }
    }
    if ((at & 63) == lane) {
#pragma unroll
      for (int i = 0; i < MOE_MAX_E / 64; ++i)
        if (at == lane + 64 * i) cand[i] = -3.0f;
    }
    total += best;
    if (lane == t) { my_w = best; my_id = at; }
  }
  if (lane < top) {
    const float w = normalize ? my_w / (total + floor_) : my_w;
    ids[(size_t)n * top + lane] = my_id;
    wts[(size_t)n * top + lane] = w * scale;
  }
}

extern "C" int qvl_moe_route(const void* z, void* ids, void* wts, int N, int E, int top, int groups, int keep,
                             float scale, int score_fn, int normalize, float floor_, hipStream_t stream) {
  if (N <= 0) return QVL_OK;
  if (E <= 0 || top <= 0 || groups <= 0 || keep <= 0 || keep > groups || E % groups || top > keep * (E / groups))
    return QVL_ERR_SHAPE;
  if (E > MOE_MAX_E || groups > 64 || top > 64) return QVL_ERR_LIMIT;
  hipLaunchKernelGGL(moe_route_kernel, dim3((N + 3) / 4), dim3(256), 0, stream, (const float*)z, (int*)ids, (float*)wts, N,
                     E, top, groups, keep, scale, score_fn, normalize, floor_);
  return qvl_launch_status();
}

// ---------------------------------------------------------------------------------------
// Pairs listed by expert: offsets[e] .. offsets[e + 1] of `sorted` hold the pairs that chose expert
// e (in no fixed order: a pair's row of a product does not depend on its neighbours).  One block.
// ---------------------------------------------------------------------------------------
__global__ __launch_bounds__(1024) void moe_sort_kernel(const int* __restrict__ ids, int* __restrict__ sorted,
                                                        int* __restrict__ offsets, int P, int E) {
  __shared__ int count[MOE_MAX_E + 1];
  __shared__ int start[MOE_MAX_E + 1];
  for (int e = threadIdx.x; e <= E; e += blockDim.x) count[e] = 0;
  __syncthreads();
  for (int p = threadIdx.x; p < P; p += blockDim.x) {
    const int e = ids[p];
    if (e >= 0 && e < E) atomicAdd(&count[e], 1);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int at = 0;
    for (int e = 0; e < E; ++e) {
      start[e] = at;
      at += count[e];
    }
    start[E] = at;
  }
  __syncthreads();
  for (int e = threadIdx.x; e <= E; e += blockDim.x) {
    offsets[e] = start[e];
    count[e] = 0;
  }
  __syncthreads();
  for (int p = threadIdx.x; p < P; p += blockDim.x) {
    const int e = ids[p];
    if (e >= 0 && e < E) sorted[start[e] + atomicAdd(&count[e], 1)] = p;
  }
}

extern "C" int qvl_moe_sort(const void* ids, void* sorted, void* offsets, int P, int E, hipStream_t stream) {
  if (P <= 0) return QVL_OK;
  if (E <= 0) return QVL_ERR_SHAPE;
  if (E > MOE_MAX_E) return QVL_ERR_LIMIT;
  hipLaunchKernelGGL(moe_sort_kernel, dim3(1), dim3(1024), 0, stream, (const int*)ids, (int*)sorted, (int*)offsets, P, E);
  return qvl_launch_status();
}

// ---------------------------------------------------------------------------------------
// The experts' products.  For the pair p at place i of `sorted` (expert e by `offsets`):
//   in = x[p / div, :]            (div = top for the first product, whose rows are tokens; 1 for the second)
//   plain:  out[p, c] = in . W[e, c, :]
//   gated:  g = min(in . W[e, c, :], limit), u = clamp(in . W[e, R + c, :], -limit, limit)  (no clamps if limit <= 0)
//           out[p, c] = g * sigmoid(alpha g) * (u + shift)            (W[e] holds R gate rows, then R up rows)
//   plain with act 1:  out[p, c] = max(in . W[e, c, :], 0)^2
// Any sizes and both storage types: one wave per output value, lanes split K (the sum's order is fixed).
// ---------------------------------------------------------------------------------------
struct ExpertArgs {
  const void* x;
  long long ldx;
  const void* w;        // [E, rows_w, K]
  const int* sorted;
  const int* offsets;
  void* out;            // [P, R], rows ldo values apart
  long long ldo;
  int P, E, R, K, div, gated;
  int act;              // on a plain product's values: 0 none, 1 the square of relu
  float alpha, limit, shift;
};

__device__ __forceinline__ float gated_value(float g, float u, float alpha, float limit, float shift) {
  if (limit > 0.f) {
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
  }
  return g * sigmoid_f(alpha * g) * (u + shift);
}

__device__ __forceinline__ float plain_value(float v, int act) {
  if (act == 1) {
    v = fmaxf(v, 0.f);
    v *= v;
  }
  return v;
}

__device__ __forceinline__ int expert_of(const int* offsets, int E, int i) {
  int e = 0;
  while (e + 1 < E && offsets[e + 1] <= i) ++e;
  return e;
}

template <typename T, typename TO>
__global__ __launch_bounds__(256) void moe_rows_kernel(ExpertArgs a) {
  const int i = blockIdx.x, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int e = expert_of(a.offsets, a.E, i);
  const int p = a.sorted[i];
  const T* xr = (const T*)a.x + (size_t)(p / a.div) * a.ldx;
  const int rows_w = a.gated ? 2 * a.R : a.R;
  const T* we = (const T*)a.w + (size_t)e * rows_w * a.K;
  for (int c = blockIdx.y * 4 + wave; c < a.R; c += gridDim.y * 4) {
    const T* wg = we + (size_t)c * a.K;
    float g = 0.f, u = 0.f;
    for (int k = lane; k < a.K; k += 64) g += ldf<T>(xr + k) * ldf<T>(wg + k);
    g = wave_sum(g);
    if (a.gated) {
      const T* wu = we + (size_t)(a.R + c) * a.K;
      for (int k = lane; k < a.K; k += 64) u += ldf<T>(xr + k) * ldf<T>(wu + k);
      u = wave_sum(u);
      g = gated_value(g, u, a.alpha, a.limit, a.shift);
    } else {
      g = plain_value(g, a.act);
    }
    if (lane == 0) stf<TO>((TO*)a.out + (size_t)p * a.ldo + c, g);
  }
}

// bfloat16 on the matrix cores, few pairs an expert (a decode step: the experts' weights are read once
// each and that is the time it takes).  A block of four waves owns 16 MT pairs of one expert and 64 output
// columns; a wave takes 16 of the columns (rows of W: the instruction's first operand, straight from
// memory: nobody else in the block reads them) and all MT tiles of 16 pairs (rows of x: the second
// operand).  K in steps of 32, a multiple of 8.  Which expert a block serves follows from the
// offsets: tile t of the grid is the (t - tiles before e)-th tile of 16 MT pairs of expert e.
template <int MT, typename TO>
__global__ __launch_bounds__(256) void moe_mfma_kernel(ExpertArgs a) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, lg = lane >> 4, r = lane & 15;
  constexpr int TM = 16 * MT;
  int tile = blockIdx.x, e = 0, first = 0, last = 0;
  for (; e < a.E; ++e) {
    first = a.offsets[e];
    last = a.offsets[e + 1];
    const int nt = (last - first + TM - 1) / TM;
    if (tile < nt) break;
    tile -= nt;
  }
  if (e >= a.E) return;
  first += tile * TM;
  const int c0 = (blockIdx.y * 4 + wave) * 16;     // this wave's output columns
  if (c0 >= a.R) return;
  const int rows_w = a.gated ? 2 * a.R : a.R;
  const bf16_t* we = (const bf16_t*)a.w + (size_t)e * rows_w * a.K;
  const bool col_ok = c0 + r < a.R;
  const bf16_t* wg = we + (size_t)(col_ok ? c0 + r : 0) * a.K + 8 * lg;
  const bf16_t* wu = wg + (size_t)a.R * a.K;      // only read if gated
  const bf16_t* xr[MT];
  int pair[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int i = first + 16 * t + r;
    pair[t] = i < last ? a.sorted[i] : -1;
    xr[t] = (const bf16_t*)a.x + (size_t)(pair[t] < 0 ? 0 : pair[t] / a.div) * a.ldx + 8 * lg;
  }
  f32x4_t accg[MT], accu[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    accg[t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    accu[t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  }
  // No load stands inside a branch (the compiler would wait for each before the next): what does not
  // exist is read from a place that does (column 0 of the step, row 0) and replaced by zeros.
  const bf16x8_t zero = __builtin_bit_cast(bf16x8_t, uint4{0u, 0u, 0u, 0u});
  if (!a.gated) wu = wg;
#pragma unroll 2
  for (int k = 0; k < a.K; k += 32) {
    const bool k_ok = k + 8 * lg < a.K;
    const int at = k_ok ? k : k - 8 * lg;
    bf16x8_t fg = *reinterpret_cast<const bf16x8_t*>(wg + at);
    bf16x8_t fu = *reinterpret_cast<const bf16x8_t*>(wu + at);
    bf16x8_t fx[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) fx[t] = *reinterpret_cast<const bf16x8_t*>(xr[t] + at);
    fg = (k_ok && col_ok) ? fg : zero;
    fu = (k_ok && col_ok) ? fu : zero;
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      const bf16x8_t f = (k_ok && pair[t] >= 0) ? fx[t] : zero;
      accg[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fg, f, accg[t], 0, 0, 0);
      if (a.gated) accu[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fu, f, accu[t], 0, 0, 0);
    }
  }
  // a lane holds, of tile t, pair r and columns c0 + 4 lg .. + 3
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    if (pair[t] < 0) continue;
    TO* o = (TO*)a.out + (size_t)pair[t] * a.ldo + c0 + 4 * lg;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (c0 + 4 * lg + j >= a.R) break;
      float v = accg[t][j];
      if (a.gated) v = gated_value(v, accu[t][j], a.alpha, a.limit, a.shift);
      else v = plain_value(v, a.act);
      stf<TO>(o + j, v);
    }
  }
}

// Many pairs an expert: tiles of TILE_M pairs x TILE_N rows of W (gated: TILE_N / 2 gate rows and the up rows
// of the same outputs), K in steps of TILE_K through LDS.  The 256 threads fetch the next step's values of x
// (gathered rows) and of W into registers while the step in LDS is multiplied, then put them into the other
// of two buffers; the 16-byte chunks of a row are exchanged by bits of the row number, so that the 16 lanes
// that read one chunk of 16 rows hit all 64 banks.  The four waves stand 2 x 2: each owns 64 pairs and
// 16 NW rows of W (gated: 8 NW gate rows and their up rows): 4 NW products of 16 x 16 x 32 a step from
// 4 + NW operand reads.
// Measured on 12,288 pairs over 32 experts, K 3,584, 2 x 2,368 rows (gate|up): TILE_K 64, NW 4: 1,000 us; TILE_K 32:
// 1,030; NW 8 (tiles of 128 x 256: fewer operand reads and fetched bytes a product, but the sums leave
// room for one wave a SIMD): 1,220 (TILE_K 64), 1,420 (TILE_K 32); fetching two steps ahead into a
// second set of registers: 1,230.
#ifndef TILE_K
#define TILE_K 64
#endif
#ifndef NW
#define NW 4                                           // tiles of 16 rows of W a wave multiplies
#endif
#define TILE_M 128
#define TILE_N (32 * NW)
#define ROW_CHUNKS (TILE_K / 8)                        // 16-byte chunks of a row of a tile
#define X_CHUNKS (TILE_M * ROW_CHUNKS / 256)           // chunks of x a thread fetches a step
#define W_CHUNKS (TILE_N * ROW_CHUNKS / 256)           // and of W

__device__ __forceinline__ int lds_slot(int row, int chunk) {
#if TILE_K == 64
  return row * 8 + (chunk ^ ((row >> 1) & 7));
#else
  return row * 4 + (chunk ^ ((row >> 2) & 3));
#endif
}

template <bool GATED, typename TO>
__global__ __launch_bounds__(256) void moe_tile_kernel(ExpertArgs a, int tiles_m, int tiles_n) {
  __shared__ __attribute__((aligned(16))) uint4 s_x[2][TILE_M * ROW_CHUNKS];
  __shared__ __attribute__((aligned(16))) uint4 s_w[2][TILE_N * ROW_CHUNKS];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, lg = lane >> 4, r = lane & 15;
  const int wm = wave >> 1, wn = wave & 1;
  // Blocks go to the XCDs in turn (block b to XCD b mod 8, each with an L2 of its own).  The 32 blocks that
  // an XCD's compute units hold at a time are made 4 tiles of pairs x 8 tiles of rows of W: they walk K at
  // about the same pace, so a slice of x is fetched into that L2 once for 8 blocks and a slice of W once for 4.
  const int xcd = blockIdx.x & 7, idx = blockIdx.x >> 3;
  const int super = (idx >> 5) * 8 + xcd, inner = idx & 31;
  const int supers_m = (tiles_m + 3) / 4;
  const int tile_n = (super / supers_m) * 8 + (inner >> 2);
  int tile = (super % supers_m) * 4 + (inner & 3);
  if (tile >= tiles_m || tile_n >= tiles_n) return;
  int e = 0, first = 0, last = 0;
  for (; e < a.E; ++e) {
    first = a.offsets[e];
    last = a.offsets[e + 1];
    const int nt = (last - first + TILE_M - 1) / TILE_M;
    if (tile < nt) break;
    tile -= nt;
  }
  if (e >= a.E) return;
  first += tile * TILE_M;
  constexpr int HALF = TILE_N / 2;
  constexpr int OUT_COLS = GATED ? HALF : TILE_N;           // output columns of a block
  const int c0 = tile_n * OUT_COLS;
  const int rows_w = GATED ? 2 * a.R : a.R;
  const bf16_t* we = (const bf16_t*)a.w + (size_t)e * rows_w * a.K;

  // what this thread fetches each step: chunks of 16 bytes of x and of W.  No load stands inside a branch
  // (the compiler would wait for each before the next): a chunk that does not exist is read from one
  // that does (row 0, column 0 of the step) and replaced by zeros.
  const bf16_t* gx[X_CHUNKS];
  const bf16_t* gw[W_CHUNKS];
  bool x_ok[X_CHUNKS], w_ok[W_CHUNKS];
#pragma unroll
  for (int j = 0; j < X_CHUNKS; ++j) {
    const int id = threadIdx.x + 256 * j, row = id / ROW_CHUNKS, ch = id % ROW_CHUNKS;
    const int i = first + row;
    const int pair = i < last ? a.sorted[i] : -1;
    x_ok[j] = pair >= 0;
    gx[j] = (const bf16_t*)a.x + (size_t)(pair < 0 ? 0 : pair / a.div) * a.ldx + 8 * ch;
  }
#pragma unroll
  for (int j = 0; j < W_CHUNKS; ++j) {
    const int id = threadIdx.x + 256 * j, row = id / ROW_CHUNKS, ch = id % ROW_CHUNKS;
    int wrow;                                               // row of W_e behind row `row` of the tile
    if (GATED) wrow = row < HALF ? c0 + row : a.R + c0 + (row - HALF);
    else wrow = c0 + row;
    w_ok[j] = GATED ? (c0 + (row % HALF) < a.R) : (wrow < a.R);
    gw[j] = we + (size_t)(w_ok[j] ? wrow : 0) * a.K + 8 * ch;
  }
  uint4 rx[X_CHUNKS], rw[W_CHUNKS];
  auto fetch = [&](int k) {
    const int ch = threadIdx.x % ROW_CHUNKS;                // 256 is a multiple of ROW_CHUNKS: the same for every j
    const bool k_ok = k + 8 * ch < a.K;
    const int at = k_ok ? k : k - 8 * ch;
#pragma unroll
    for (int j = 0; j < X_CHUNKS; ++j) {
      const uint4 v = *reinterpret_cast<const uint4*>(gx[j] + at);
      const bool ok = x_ok[j] && k_ok;
      rx[j] = uint4{ok ? v.x : 0u, ok ? v.y : 0u, ok ? v.z : 0u, ok ? v.w : 0u};
    }
#pragma unroll
    for (int j = 0; j < W_CHUNKS; ++j) {
      const uint4 v = *reinterpret_cast<const uint4*>(gw[j] + at);
      const bool ok = w_ok[j] && k_ok;
      rw[j] = uint4{ok ? v.x : 0u, ok ? v.y : 0u, ok ? v.z : 0u, ok ? v.w : 0u};
    }
  };
  auto put = [&](int buf) {
#pragma unroll
    for (int j = 0; j < X_CHUNKS; ++j) {
      const int id = threadIdx.x + 256 * j;
      s_x[buf][lds_slot(id / ROW_CHUNKS, id % ROW_CHUNKS)] = rx[j];
    }
#pragma unroll
    for (int j = 0; j < W_CHUNKS; ++j) {
      const int id = threadIdx.x + 256 * j;
      s_w[buf][lds_slot(id / ROW_CHUNKS, id % ROW_CHUNKS)] = rw[j];
    }
  };
  f32x4_t acc[NW][4];    // [tile of 16 rows of W][tile of 16 pairs]
#pragma unroll
  for (int n = 0; n < NW; ++n)
#pragma unroll
    for (int m = 0; m < 4; ++m) acc[n][m] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  // rows of the W tile this wave multiplies: gated, its gate rows and the up rows of the same outputs
  constexpr int PER_WAVE = GATED ? 8 * NW : 16 * NW;        // output columns of a wave
  int wrow0[NW];
#pragma unroll
  for (int n = 0; n < NW; ++n)
    wrow0[n] = GATED ? (n < NW / 2 ? wn * PER_WAVE + n * 16 : HALF + wn * PER_WAVE + (n - NW / 2) * 16) : wn * PER_WAVE + n * 16;

  fetch(0);
  put(0);
  __syncthreads();
  int buf = 0;
  for (int k = 0; k < a.K; k += TILE_K) {
    const bool more = k + TILE_K < a.K;
    if (more) fetch(k + TILE_K);
#pragma unroll
    for (int kk = 0; kk < TILE_K / 32; ++kk) {
      bf16x8_t fx[4];
#pragma unroll
      for (int m = 0; m < 4; ++m) fx[m] = __builtin_bit_cast(bf16x8_t, s_x[buf][lds_slot(wm * 64 + m * 16 + r, 4 * kk + lg)]);
#pragma unroll
      for (int n = 0; n < NW; ++n) {
        const bf16x8_t fw = __builtin_bit_cast(bf16x8_t, s_w[buf][lds_slot(wrow0[n] + r, 4 * kk + lg)]);
#pragma unroll
        for (int m = 0; m < 4; ++m) acc[n][m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fw, fx[m], acc[n][m], 0, 0, 0);
      }
    }
    if (more) put(buf ^ 1);
    __syncthreads();
    buf ^= 1;
  }
  // a lane holds, of (n, m): pair wm 64 + 16 m + r, W rows wrow0[n] + 4 lg .. + 3
#pragma unroll
  for (int m = 0; m < 4; ++m) {
    const int i = first + wm * 64 + m * 16 + r;
    if (i >= last) continue;
    const int pair = a.sorted[i];
    TO* o = (TO*)a.out + (size_t)pair * a.ldo;
#pragma unroll
    for (int n = 0; n < (GATED ? NW / 2 : NW); ++n) {
      const int c = c0 + wn * PER_WAVE + n * 16 + 4 * lg;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (c + j >= a.R) break;
        float v = acc[n][m][j];
        if (GATED) v = gated_value(v, acc[n + NW / 2][m][j], a.alpha, a.limit, a.shift);
        else v = plain_value(v, a.act);
        stf<TO>(o + c + j, v);
      }
    }
  }
}

// The same product with the fetches going straight from memory into LDS (global_load_lds_dwordx4: lane l
// of a wave puts its 16 bytes at M0 + 16 l), up to ST_STAGES - 1 steps of K ahead of the step that is
// multiplied, through ST_STAGES stages of LDS.  No register holds data on its way, so the waves can carry 128 x 256 tiles (8 tiles
// of 16 rows of W each: 32 products from 12 operand reads a step) and a fetch is hidden by the steps before
// it rather than by other waves.  Chunk c of row rho lies at place c ^ ((rho >> 2) & 3) of the row (the 16
// lanes of an operand read hit all banks), so the lane that fills place s of row rho fetches chunk
// s ^ ((rho >> 2) & 3).  Nothing can be replaced by zeros on this way: rows that do not exist are read from
// rows that do (their sums are not stored), and K must be a multiple of 32.  Offsets within x and within an
// expert's W are 32-bit.
#define ST_K 32
#define ST_NW 8
#define ST_M 128
#define ST_N (32 * ST_NW)
#ifndef ST_STAGES
#define ST_STAGES 5                                    // steps of K in LDS: one being multiplied, the others on their way
#endif
#define ST_X_SLOTS (ST_M * 4)                          // 16-byte places of x in a stage
#define ST_SLOTS ((ST_M + ST_N) * 4)                   // and of x and W together
#define ST_WAVE_LOADS (ST_SLOTS / 64 / 4)              // loads of 1 KB a wave issues a step

__device__ __forceinline__ void fetch16_to_lds(const void* base, uint32_t lane_bytes, uint32_t lds_at) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(lane_bytes), "s"(base), "s"(lds_at)
               : "memory", "m0");
}
// Wait until at most N of this wave's fetches are outstanding (they finish in order).
template <int N>
__device__ __forceinline__ void wait_fetches() {
  __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | 0x0f70);
}

template <bool GATED, typename TO>
__global__ __launch_bounds__(256) void moe_stream_kernel(ExpertArgs a, int tiles_m, int tiles_n) {
  __shared__ __attribute__((aligned(16))) uint4 stage[ST_STAGES][ST_SLOTS];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63, lg = lane >> 4, r = lane & 15;
  const int wm = wave >> 1, wn = wave & 1;
  const int xcd = blockIdx.x & 7, idx = blockIdx.x >> 3;
  const int super = (idx >> 5) * 8 + xcd, inner = idx & 31;
  const int supers_m = (tiles_m + 3) / 4;
  const int tile_n = (super / supers_m) * 8 + (inner >> 2);
  int tile = (super % supers_m) * 4 + (inner & 3);
  if (tile >= tiles_m || tile_n >= tiles_n) return;
  int e = 0, first = 0, last = 0;
  for (; e < a.E; ++e) {
    first = a.offsets[e];
    last = a.offsets[e + 1];
    const int nt = (last - first + ST_M - 1) / ST_M;
    if (tile < nt) break;
    tile -= nt;
  }
  if (e >= a.E) return;
  first += tile * ST_M;
  constexpr int HALF = ST_N / 2;
  constexpr int OUT_COLS = GATED ? HALF : ST_N;
  const int c0 = tile_n * OUT_COLS;
  const int rows_w = GATED ? 2 * a.R : a.R;
  const bf16_t* we = (const bf16_t*)a.w + (size_t)e * rows_w * a.K;

  // this wave's fetches of a step: places wave * ST_WAVE_LOADS * 64 ... of the stage, 64 a fetch
  uint32_t from[ST_WAVE_LOADS];      // byte offset of this lane's 16 bytes at K = 0, within x or within W_e
#pragma unroll
  for (int j = 0; j < ST_WAVE_LOADS; ++j) {
    const int place = (wave * ST_WAVE_LOADS + j) * 64 + lane;
    if (place < ST_X_SLOTS) {
      const int row = place >> 2, ch = (place & 3) ^ ((row >> 2) & 3);
      const int i = first + row;
      const int pair = a.sorted[i < last ? i : first];
      from[j] = (uint32_t)(((size_t)(pair / a.div) * a.ldx + 8 * ch) * 2);
    } else {
      const int row = (place - ST_X_SLOTS) >> 2, ch = (place & 3) ^ ((row >> 2) & 3);
      int wrow;
      if (GATED) wrow = row < HALF ? c0 + row : a.R + c0 + (row - HALF);
      else wrow = c0 + row;
      const bool ok = GATED ? (c0 + (row % HALF) < a.R) : (wrow < a.R);
      from[j] = (uint32_t)(((size_t)(ok ? wrow : 0) * a.K + 8 * ch) * 2);
    }
  }
  const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void*)&stage[0][0];
  auto issue = [&](int step) {
    const uint32_t at = lds0 + (uint32_t)(step % ST_STAGES) * (ST_SLOTS * 16) + (uint32_t)wave * (ST_WAVE_LOADS * 1024);
    const uint32_t k_bytes = (uint32_t)step * (ST_K * 2);
#pragma unroll
    for (int j = 0; j < ST_WAVE_LOADS; ++j) {
      // a fetch lies wholly in x's places or wholly in W's: the same base for all its lanes
      const bool is_x = (wave * ST_WAVE_LOADS + j) * 64 < ST_X_SLOTS;
      fetch16_to_lds(is_x ? (const void*)a.x : (const void*)we, from[j] + k_bytes, at + j * 1024);
    }
  };
  f32x4_t acc[ST_NW][4];
#pragma unroll
  for (int n = 0; n < ST_NW; ++n)
#pragma unroll
    for (int m = 0; m < 4; ++m) acc[n][m] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  constexpr int PER_WAVE = GATED ? 8 * ST_NW : 16 * ST_NW;
  int wrow0[ST_NW];
#pragma unroll
  for (int n = 0; n < ST_NW; ++n)
    wrow0[n] = GATED ? (n < ST_NW / 2 ? wn * PER_WAVE + n * 16 : HALF + wn * PER_WAVE + (n - ST_NW / 2) * 16) : wn * PER_WAVE + n * 16;

  const int steps = a.K / ST_K;
#pragma unroll
  for (int i = 0; i < ST_STAGES - 1; ++i)
    if (i < steps) issue(i);
  for (int s = 0; s < steps; ++s) {
    // the steps after s that have been asked for may still be on their way: ST_STAGES - 2 of them, fewer at the end
    const int ahead = steps - 1 - s < ST_STAGES - 2 ? steps - 1 - s : ST_STAGES - 2;
    if (ahead >= 3) wait_fetches<3 * ST_WAVE_LOADS>();
    else if (ahead == 2) wait_fetches<2 * ST_WAVE_LOADS>();
    else if (ahead == 1) wait_fetches<ST_WAVE_LOADS>();
    else wait_fetches<0>();
    __syncthreads();                                    // every wave's part of step s is there, and step s - 1 has been multiplied
    if (s + ST_STAGES - 1 < steps) issue(s + ST_STAGES - 1);
    const uint4* sx = stage[s % ST_STAGES];
    const uint4* sw = sx + ST_X_SLOTS;
    bf16x8_t fx[4];
#pragma unroll
    for (int m = 0; m < 4; ++m) {
      const int row = wm * 64 + m * 16 + r;
      fx[m] = __builtin_bit_cast(bf16x8_t, sx[row * 4 + (lg ^ ((row >> 2) & 3))]);
    }
#pragma unroll
    for (int n = 0; n < ST_NW; ++n) {
      const int row = wrow0[n] + r;
      const bf16x8_t fw = __builtin_bit_cast(bf16x8_t, sw[row * 4 + (lg ^ ((row >> 2) & 3))]);
#pragma unroll
      for (int m = 0; m < 4; ++m) acc[n][m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fw, fx[m], acc[n][m], 0, 0, 0);
    }
  }
#pragma unroll
  for (int m = 0; m < 4; ++m) {
    const int i = first + wm * 64 + m * 16 + r;
    if (i >= last) continue;
    const int pair = a.sorted[i];
    TO* o = (TO*)a.out + (size_t)pair * a.ldo;
#pragma unroll
    for (int n = 0; n < (GATED ? ST_NW / 2 : ST_NW); ++n) {
      const int c = c0 + wn * PER_WAVE + n * 16 + 4 * lg;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (c + j >= a.R) break;
        float v = acc[n][m][j];
        if (GATED) v = gated_value(v, acc[n + ST_NW / 2][m][j], a.alpha, a.limit, a.shift);
        else v = plain_value(v, a.act);
        stf<TO>(o + c + j, v);
      }
    }
  }
}

// x_dtype / out_dtype: 0 float32, 1 bfloat16.  float32 operands write float32; bfloat16 operands
// write either.  The matrix-core kernel runs for bfloat16 with K a multiple of 8 and rows of x on
// 16-byte boundaries; `big_tiles` asks for the kernel with tiles of 128 pairs through LDS (many pairs an expert).
extern "C" int qvl_moe_experts(const void* x, long long ldx, int x_dtype, const void* w, const void* sorted,
                               const void* offsets, void* out, long long ldo, int out_dtype, int P, int E, int R, int K,
                               int div,
                               int gated, float alpha, float limit, float shift, int act, int big_tiles,
                               hipStream_t stream) {
  if (P <= 0) return QVL_OK;
  if (E <= 0 || R <= 0 || K <= 0 || div <= 0 || ldx < K || ldo < R || !x || !w || !sorted || !offsets || !out) return QVL_ERR_SHAPE;
  ExpertArgs a;
  a.x = x; a.ldx = ldx; a.w = w; a.sorted = (const int*)sorted; a.offsets = (const int*)offsets; a.out = out; a.ldo = ldo;
  a.P = P; a.E = E; a.R = R; a.K = K; a.div = div; a.gated = gated; a.act = gated ? 0 : act; a.alpha = alpha; a.limit = limit; a.shift = shift;
  if (x_dtype == 1 && K % 8 == 0 && ldx % 8 == 0 && ((uintptr_t)x % 16) == 0 && ((uintptr_t)w % 16) == 0) {
    if (out_dtype != 0 && out_dtype != 1) return QVL_ERR_DTYPE;
#ifndef MOE_NO_STREAM
    const unsigned long long x_rows = (unsigned long long)((P + div - 1) / div);
    if (big_tiles && K % ST_K == 0 && x_rows * (unsigned long long)ldx * 2 < 0xffffff00ull &&
        (unsigned long long)(gated ? 2 * R : R) * K * 2 < 0xffffff00ull) {
      const int cols = gated ? ST_N / 2 : ST_N;
      const int tiles_m = P / ST_M + (E < P ? E : P), tiles_n = (R + cols - 1) / cols;
      if ((long long)tiles_m * tiles_n > 0x7ffffff0ll) return QVL_ERR_LIMIT;
      const int supers = ((tiles_m + 3) / 4) * ((tiles_n + 7) / 8);
      const dim3 tgrid((unsigned)((supers + 7) / 8) * 8 * 32);
      if (gated && out_dtype == 1)
        hipLaunchKernelGGL((moe_stream_kernel<true, bf16_t>), tgrid, dim3(256), 0, stream, a, tiles_m, tiles_n);
      else if (gated) hipLaunchKernelGGL((moe_stream_kernel<true, float>), tgrid, dim3(256), 0, stream, a, tiles_m, tiles_n);
      else if (out_dtype == 1)
        hipLaunchKernelGGL((moe_stream_kernel<false, bf16_t>), tgrid, dim3(256), 0, stream, a, tiles_m, tiles_n);
      else hipLaunchKernelGGL((moe_stream_kernel<false, float>), tgrid, dim3(256), 0, stream, a, tiles_m, tiles_n);
      return qvl_launch_status();
    }
#endif
    if (big_tiles) {
      const int cols = gated ? TILE_N / 2 : TILE_N;
      const int tiles_m = P / TILE_M + (E < P ? E : P), tiles_n = (R + cols - 1) / cols;
      if ((long long)tiles_m * tiles_n > 0x7ffffff0ll) return QVL_ERR_LIMIT;
      // whole groups of 4 x 8 tiles, 8 groups (one per XCD) at a time
      const int supers = ((tiles_m + 3) / 4) * ((tiles_n + 7) / 8);
      const dim3 tgrid((unsigned)((supers + 7) / 8) * 8 * 32);
      if (gated && out_dtype == 1)
        hipLaunchKernelGGL((moe_tile_kernel<true, bf16_t>), tgrid, dim3(256), 0, stream, a, tiles_m, tiles_n);
      else if (gated) hipLaunchKernelGGL((moe_tile_kernel<true, float>), tgrid, dim3(256), 0, stream, a, tiles_m, tiles_n);
      else if (out_dtype == 1)
        hipLaunchKernelGGL((moe_tile_kernel<false, bf16_t>), tgrid, dim3(256), 0, stream, a, tiles_m, tiles_n);
      else hipLaunchKernelGGL((moe_tile_kernel<false, float>), tgrid, dim3(256), 0, stream, a, tiles_m, tiles_n);
      return qvl_launch_status();
    }
    const int tiles = P / 16 + (E < P ? E : P);
    const dim3 grid(tiles, (R + 63) / 64);
    if (grid.y > 65535) return QVL_ERR_LIMIT;
    if (out_dtype == 1) hipLaunchKernelGGL((moe_mfma_kernel<1, bf16_t>), grid, dim3(256), 0, stream, a);
    else if (out_dtype == 0) hipLaunchKernelGGL((moe_mfma_kernel<1, float>), grid, dim3(256), 0, stream, a);
    else return QVL_ERR_DTYPE;
    return qvl_launch_status();
  }
  int by = (R + 3) / 4;
  if (by > 64) by = 64;
  const dim3 grid(P, by);
  if (x_dtype == 0 && out_dtype == 0) hipLaunchKernelGGL((moe_rows_kernel<float, float>), grid, dim3(256), 0, stream, a);
  else if (x_dtype == 1 && out_dtype == 1) hipLaunchKernelGGL((moe_rows_kernel<bf16_t, bf16_t>), grid, dim3(256), 0, stream, a);
  else if (x_dtype == 1 && out_dtype == 0) hipLaunchKernelGGL((moe_rows_kernel<bf16_t, float>), grid, dim3(256), 0, stream, a);
  else return QVL_ERR_DTYPE;
  return qvl_launch_status();
}

// ---------------------------------------------------------------------------------------
// out[n, :] = sum over k of wts[n, k] * y[n top + k, :], in the order of k, plus `extra[n, :]` (what
// a shared expert gave: float32 or bfloat16, or float32 slabs added in order; null: nothing).
// ---------------------------------------------------------------------------------------
// four consecutive values as float32
template <typename T> __device__ __forceinline__ float4 ld4(const T* p);
template <> __device__ __forceinline__ float4 ld4<float>(const float* p) { return *reinterpret_cast<const float4*>(p); }
template <> __device__ __forceinline__ float4 ld4<bf16_t>(const bf16_t* p) {
  const uint2 v = *reinterpret_cast<const uint2*>(p);
  return float4{__uint_as_float(v.x << 16), __uint_as_float(v.x & 0xffff0000u), __uint_as_float(v.y << 16),
                __uint_as_float(v.y & 0xffff0000u)};
}

// VEC 4: a thread owns four neighbouring columns of one token (H a multiple of 4); VEC 1: one column.
// Its loads are all on their way before the first is used.
template <typename TY, typename TX, int VEC>
__global__ __launch_bounds__(256) void moe_combine_kernel(const TY* __restrict__ y, const float* __restrict__ wts,
                                                          const TX* __restrict__ extra, int nslabs, long long slab_stride,
                                                          float* __restrict__ out, int top, int H) {
  const size_t n = blockIdx.x;
  const int c = (blockIdx.y * 256 + threadIdx.x) * VEC;
  if (c >= H) return;
  const float* wr = wts + n * top;
  if (VEC == 4) {
    float4 v = float4{0.f, 0.f, 0.f, 0.f};
#pragma unroll 8
    for (int k = 0; k < top; ++k) {
      const float4 t = ld4<TY>(y + (n * top + k) * (size_t)H + c);
      const float w = wr[k];
      v.x += w * t.x; v.y += w * t.y; v.z += w * t.z; v.w += w * t.w;
    }
    if (extra) {
      float4 x = ld4<TX>(extra + n * H + c);
      for (int s = 1; s < nslabs; ++s) {
        const float4 t = ld4<TX>(extra + (size_t)s * slab_stride + n * H + c);
        x.x += t.x; x.y += t.y; x.z += t.z; x.w += t.w;
      }
      v.x += x.x; v.y += x.y; v.z += x.z; v.w += x.w;
    }
    *reinterpret_cast<float4*>(out + n * H + c) = v;
  } else {
    float v = 0.f;
#pragma unroll 8
    for (int k = 0; k < top; ++k) v += wr[k] * ldf<TY>(y + (n * top + k) * (size_t)H + c);
    if (extra) {
      float x = ldf<TX>(extra + n * H + c);
      for (int s = 1; s < nslabs; ++s) x += ldf<TX>(extra + (size_t)s * slab_stride + n * H + c);
      v += x;
    }
    out[n * H + c] = v;
  }
}

extern "C" int qvl_moe_combine(const void* y, int y_dtype, const void* wts, const void* extra, int extra_dtype,
                               int nslabs, long long slab_stride, void* out, int N, int top, int H, hipStream_t stream) {
  if (N <= 0) return QVL_OK;
  if (top <= 0 || H <= 0 || nslabs < 1 || (nslabs > 1 && extra_dtype != 0)) return QVL_ERR_SHAPE;
#define LAUNCH(TY, TX)                                                                                         \
  if (vec4)                                                                                                        \
    hipLaunchKernelGGL((moe_combine_kernel<TY, TX, 4>), dim3(N, (H / 4 + 255) / 256), dim3(256), 0, stream,          \
                       (const TY*)y, (const float*)wts, (const TX*)extra, nslabs, slab_stride, (float*)out, top, H); \
  else                                                                                                             \
    hipLaunchKernelGGL((moe_combine_kernel<TY, TX, 1>), dim3(N, (H + 255) / 256), dim3(256), 0, stream,              \
                       (const TY*)y, (const float*)wts, (const TX*)extra, nslabs, slab_stride, (float*)out, top, H)
  const bool vec4 = H % 4 == 0 && slab_stride % 4 == 0 && ((uintptr_t)y % 16) == 0 && ((uintptr_t)extra % 16) == 0 &&
                    ((uintptr_t)out % 16) == 0;
  if (y_dtype == 0 && extra_dtype == 0) { LAUNCH(float, float); }
  else if (y_dtype == 0 && extra_dtype == 1) { LAUNCH(float, bf16_t); }
  else if (y_dtype == 1 && extra_dtype == 0) { LAUNCH(bf16_t, float); }
  else if (y_dtype == 1 && extra_dtype == 1) { LAUNCH(bf16_t, bf16_t); }
  else return QVL_ERR_DTYPE;
#undef LAUNCH
  return qvl_launch_status();
}
