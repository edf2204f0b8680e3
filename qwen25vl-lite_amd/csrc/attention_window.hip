// Paged attention on the matrix cores for what the other matrix-core kernel does not take: a sliding
// window that also keeps a request's first keys visible, values of another width than keys, and a softmax
// whose denominator holds one more term per query head, exp(sink), with no key and no value behind it.
// bfloat16 storage, float32 scores, softmax and sums.  Compiled per key size HD and value size VD.
//
// A column is a (token, query head of one key/value head's group) pair; a tile has 16 of them.  A
// tile's keys are walked in blocks of 32 by absolute index: the blocks that hold kept first keys
// (below min(keep_first, the tile's lowest window start)), then those from the lowest window start to
// the tile's last key; every column masks for itself.  Per block:
//   S^T = K Q^T   two products of 16 keys x 16 columns (v_mfma_f32_16x16x32_bf16 over the channels).
//                 Row rho of product t holds key 8 (rho / 4) + 4 t + rho % 4 of the block, so that a lane
//                 ends up with the scores of keys 8 lg .. 8 lg + 7 of its column, which is what the
//                 second product's operand wants;
//   softmax       running maximum and sum per column (the four lanes of a column exchange theirs);
//   O^T += V^T P^T   per 16 value channels one product; V^T rows are 8 consecutive keys of a channel,
//                 one 16-byte load from the transposed value pages.
// Many tiles: a wave per entry of two neighbouring tiles (every fetched key and value fragment is used
// for both), four entries a block.  Few tiles (decoded tokens): the four waves of a block share a tile,
// wave w taking blocks w, w + 4, ..., and merge through LDS.
#include "common.h"

#ifndef HD
#define HD 128
#endif
#ifndef VD
#define VD HD
#endif
#if HD % 8 || HD > 256 || VD > 256
#error "key size: a multiple of 8 up to 256; value size: up to 256"
#endif

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

#define KS ((HD + 31) / 32)   // 32-channel steps of the first product
#define NT ((VD + 15) / 16)   // 16-channel tiles of the second

__device__ __forceinline__ bf16x8_t zero8() { return __builtin_bit_cast(bf16x8_t, uint4{0u, 0u, 0u, 0u}); }
__device__ __forceinline__ bf16x8_t load8(const bf16_t* p) { return *reinterpret_cast<const bf16x8_t*>(p); }

struct WindowArgs {
  const bf16_t* q;        // [N, nq, HD]
  const bf16_t* kc;       // [pages, nkv, ps, HD]
  const bf16_t* vc;       // [pages, nkv, VD, ps]
  const int* bt;          // [R, table_width]
  int table_width;
  const int* cu_q;        // [R + 1], or null: request r brings token r only
  const int* ctx_len;     // [R]
  const int* tile_req;    // [tiles], or null: tile i is request i's only tile
  const int* tile_ct;
  int num_tiles;
  bf16_t* out;            // [N, nq, VD]
  int nq, nkv, ps, window, keep_first;
  float scale;
  const float* sinks;     // [nq] float32, or null
};

// W: waves that share an entry's key blocks (1 or 4).  CT: column tiles of an entry, all carried by the
// same wave: a key or value fragment that has been fetched is multiplied with each of them, and what a
// kernel of this kind waits for is its fetches (its keys and values come from L2 for every entry anew).
template <int W, int CT>
__global__ __launch_bounds__(256) void attn_window_kernel(WindowArgs a) {
  __shared__ float s_m[3][CT][16], s_l[3][CT][16];
  __shared__ __attribute__((aligned(16))) float s_acc[W > 1 ? 3 : 1][W > 1 ? CT * NT : 1][64][4];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, lg = lane >> 4, r = lane & 15;
  const int entry = W == 1 ? blockIdx.x * 4 + wave : blockIdx.x;
  const int part = W == 1 ? 0 : wave;
  if (entry >= a.num_tiles) return;          // W > 1: the whole block leaves
  const int kvh = blockIdx.y, g = a.nq / a.nkv;
  const int req = a.tile_req ? a.tile_req[entry] : entry;
  const int ct0 = (a.tile_ct ? a.tile_ct[entry] : 0) * CT;
  const int q0 = a.cu_q ? a.cu_q[req] : req;
  const int qlen = a.cu_q ? a.cu_q[req + 1] - q0 : 1;
  const int ctx = a.ctx_len[req];
  const int my_kept = a.window > 0 ? a.keep_first : 0;
  bool valid[CT];
  int token[CT], head[CT], my_p[CT], my_lo[CT];
  bf16x8_t qb[CT][KS];
#pragma unroll
  for (int c = 0; c < CT; ++c) {
    const int col = (ct0 + c) * 16 + r, i_col = col / g;
    valid[c] = i_col < qlen;
    token[c] = q0 + (valid[c] ? i_col : 0);
    head[c] = kvh * g + (col - i_col * g);
    const int p = ctx - qlen + (valid[c] ? i_col : 0);
    my_p[c] = valid[c] ? p : -1;
    my_lo[c] = (a.window > 0 && p - a.window + 1 > 0) ? p - a.window + 1 : 0;
    const bf16_t* qrow = a.q + ((size_t)token[c] * a.nq + head[c]) * HD;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int d = ks * 32 + 8 * lg;
      qb[c][ks] = (valid[c] && d < HD) ? load8(qrow + d) : zero8();
    }
  }
  const int i_first = (ct0 * 16) / g;
  int i_last = ((ct0 + CT) * 16 - 1) / g;
  i_last = i_last < qlen - 1 ? i_last : qlen - 1;
  const int p_first = ctx - qlen + i_first, hi_tile = ctx - qlen + i_last;
  const int lo_tile = (a.window > 0 && p_first - a.window + 1 > 0) ? p_first - a.window + 1 : 0;
  const int kept_tile = a.window > 0 ? (a.keep_first < lo_tile ? a.keep_first : lo_tile) : 0;
  const int n_kept = (kept_tile + 31) / 32;
  const int b_start = lo_tile / 32 > n_kept ? lo_tile / 32 : n_kept;
  const int n_blocks = n_kept + hi_tile / 32 - b_start + 1;
  const int* btr = a.bt + (size_t)req * a.table_width;
  float m[CT], l[CT];
  f32x4_t acc[CT][NT];
#pragma unroll
  for (int c = 0; c < CT; ++c) {
    m[c] = -INFINITY;
    l[c] = 0.f;
#pragma unroll
    for (int dt = 0; dt < NT; ++dt) acc[c][dt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  }

  for (int b = part; b < n_blocks; b += W) {
    const int k0 = (b < n_kept ? b : b - n_kept + b_start) * 32;
    // No load stands inside a branch (the compiler would wait for each before the next): channels past a
    // head's end are read from its start and replaced by zeros.
    f32x4_t s[CT][2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      int key = k0 + 8 * (r >> 2) + 4 * t + (r & 3);
      key = key > hi_tile ? hi_tile : key;                 // beyond the entry's last key: masked below, read something that exists
      const int pg = btr[key / a.ps];
      const size_t page = (size_t)(pg < 0 ? 0 : pg);       // a page that was given back holds no visible key
      const bf16_t* krow = a.kc + ((page * a.nkv + kvh) * a.ps + (size_t)(key % a.ps)) * HD;
#pragma unroll
      for (int c = 0; c < CT; ++c) s[c][t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const int d = ks * 32 + 8 * lg;
        const bool d_ok = (HD % 32 == 0) || d < HD;
        bf16x8_t kf = load8(krow + (d_ok ? d : 0));
        kf = d_ok ? kf : zero8();
#pragma unroll
        for (int c = 0; c < CT; ++c) s[c][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qb[c][ks], s[c][t], 0, 0, 0);
      }
    }
    // this lane: keys k0 + 8 lg + 4 t + i of column r of each tile
    float alpha[CT];
    bf16x8_t pb[CT];
#pragma unroll
    for (int c = 0; c < CT; ++c) {
      float mx = -INFINITY;
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int j = k0 + 8 * lg + 4 * t + i;
          const bool see = j <= my_p[c] && (j >= my_lo[c] || j < my_kept);
          const float v = see ? s[c][t][i] * a.scale : -INFINITY;
          s[c][t][i] = v;
          mx = fmaxf(mx, v);
        }
      mx = fmaxf(mx, __shfl_xor(mx, 16, QVL_WAVE));
      mx = fmaxf(mx, __shfl_xor(mx, 32, QVL_WAVE));
      const float m_new = fmaxf(m[c], mx);
      const float m_safe = m_new == -INFINITY ? 0.f : m_new;
      alpha[c] = expf(m[c] - m_safe);                      // nothing seen before: exp(-inf) = 0
      float psum = 0.f;
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float pv = expf(s[c][t][i] - m_safe);
          psum += pv;
          pb[c][4 * t + i] = (__bf16)pv;
        }
      psum += __shfl_xor(psum, 16, QVL_WAVE);
      psum += __shfl_xor(psum, 32, QVL_WAVE);
      l[c] = l[c] * alpha[c] + psum;
      m[c] = m_new;
    }
    int key0 = k0 + 8 * lg;
    key0 = key0 > hi_tile ? k0 : key0;                     // all eight masked: read the block's first keys instead
    const int pg = btr[key0 / a.ps];
    const size_t page = (size_t)(pg < 0 ? 0 : pg);
    const bf16_t* vbase = a.vc + (page * a.nkv + kvh) * (size_t)VD * a.ps + (size_t)(key0 % a.ps);
#pragma unroll
    for (int dt = 0; dt < NT; ++dt) {
      const int ch = dt * 16 + r;
      const bool c_ok = (VD % 16 == 0) || ch < VD;
      bf16x8_t vf = load8(vbase + (size_t)(c_ok ? ch : 0) * a.ps);
      vf = c_ok ? vf : zero8();
#pragma unroll
      for (int c = 0; c < CT; ++c) {
        acc[c][dt] *= alpha[c];
        acc[c][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pb[c], acc[c][dt], 0, 0, 0);
      }
    }
  }

  if (W > 1) {
    // waves 1 .. 3 hand their maxima, sums and sums of values to wave 0
    if (wave > 0) {
#pragma unroll
      for (int c = 0; c < CT; ++c) {
        if (lg == 0) {
          s_m[wave - 1][c][r] = m[c];
          s_l[wave - 1][c][r] = l[c];
        }
#pragma unroll
        for (int dt = 0; dt < NT; ++dt) *reinterpret_cast<f32x4_t*>(s_acc[wave - 1][c * NT + dt][lane]) = acc[c][dt];
      }
    }
    __syncthreads();
    if (wave > 0) return;
#pragma unroll
    for (int c = 0; c < CT; ++c) {
      float m_all = m[c];
      for (int w = 0; w < 3; ++w) m_all = fmaxf(m_all, s_m[w][c][r]);
      const float m_safe = m_all == -INFINITY ? 0.f : m_all;
      float f = expf(m[c] - m_safe);
      l[c] *= f;
#pragma unroll
      for (int dt = 0; dt < NT; ++dt) acc[c][dt] *= f;
      for (int w = 0; w < 3; ++w) {
        f = expf(s_m[w][c][r] - m_safe);
        l[c] += s_l[w][c][r] * f;
#pragma unroll
        for (int dt = 0; dt < NT; ++dt) acc[c][dt] += *reinterpret_cast<const f32x4_t*>(s_acc[w][c * NT + dt][lane]) * f;
      }
      m[c] = m_safe;                                       // what the sums now refer to
    }
  }
#pragma unroll
  for (int c = 0; c < CT; ++c) {
    if (!valid[c]) continue;
    if (a.sinks) {
      const float sk = a.sinks[head[c]];
      const float m_all = fmaxf(m[c], sk);
      const float f = expf(m[c] - m_all);
      l[c] = l[c] * f + expf(sk - m_all);
#pragma unroll
      for (int dt = 0; dt < NT; ++dt) acc[c][dt] *= f;
    }
    const float inv = 1.0f / l[c];
    bf16_t* o = a.out + ((size_t)token[c] * a.nq + head[c]) * VD;
#pragma unroll
    for (int dt = 0; dt < NT; ++dt)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int ch = dt * 16 + 4 * lg + i;
        if (ch < VD) o[ch] = f32_to_bf16(acc[c][dt][i] * inv);
      }
  }
}

// column tiles an entry of the tile list has when a wave owns an entry (`share` == 0)
#if HD <= 128 && VD <= 128
#define WIDE_CT 2
#else
#define WIDE_CT 1
#endif
extern "C" int qvl_attn_window_entry_tiles() { return WIDE_CT; }

extern "C" int qvl_attn_window_sizes(int* hd, int* vd) {
  *hd = HD;
  *vd = VD;
  return QVL_OK;
}

// share != 0: the four waves of a block share an entry of one column tile (few tiles); else a wave per
// entry of qvl_attn_window_entry_tiles() column tiles (tile_ct counts in such entries).
extern "C" int qvl_attn_window(const void* q, const void* kc, const void* vc, const void* bt, int table_width,
                               const void* cu_q, const void* ctx_len, const void* tile_req, const void* tile_ct,
                               int num_tiles, void* out, int nq, int nkv, int ps, int window, int keep_first, float scale,
                               const void* sinks, int share, hipStream_t stream) {
  if (num_tiles <= 0) return QVL_OK;
  if (nq <= 0 || nkv <= 0 || nq % nkv || ps <= 0 || ps % 8 || table_width <= 0 || window < 0 || keep_first < 0)
    return QVL_ERR_SHAPE;
  if ((tile_req == nullptr) != (tile_ct == nullptr) || (!tile_req && (nq / nkv > 16 || !share))) return QVL_ERR_SHAPE;
  if (nkv > 65535) return QVL_ERR_LIMIT;
  WindowArgs a;
  a.q = (const bf16_t*)q; a.kc = (const bf16_t*)kc; a.vc = (const bf16_t*)vc; a.bt = (const int*)bt;
  a.table_width = table_width; a.cu_q = (const int*)cu_q; a.ctx_len = (const int*)ctx_len;
  a.tile_req = (const int*)tile_req; a.tile_ct = (const int*)tile_ct; a.num_tiles = num_tiles; a.out = (bf16_t*)out;
  a.nq = nq; a.nkv = nkv; a.ps = ps; a.window = window; a.keep_first = keep_first; a.scale = scale;
  a.sinks = (const float*)sinks;
  if (share) hipLaunchKernelGGL((attn_window_kernel<4, 1>), dim3(num_tiles, nkv), dim3(256), 0, stream, a);
  else hipLaunchKernelGGL((attn_window_kernel<1, WIDE_CT>), dim3((num_tiles + 3) / 4, nkv), dim3(256), 0, stream, a);
  return qvl_launch_status();
}
