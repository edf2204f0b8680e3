// Row-wise kernels of gated and normed sublayers: a residual add, a clamped gated activation, a
// norm over groups of channels with a gate, a per-head output gate, a per-head norm + rotation +
// cache write for attention whose values may be its unrotated keys, and a soft cap on logits.
// float32 and bfloat16 storage; all arithmetic is float32.
#include "common.h"

__device__ __forceinline__ float sigmoid_f(float z) { return 1.0f / (1.0f + expf(-z)); }

// four consecutive values as float32
template <typename T> __device__ __forceinline__ float4 ldv4(const T* p);
template <> __device__ __forceinline__ float4 ldv4<float>(const float* p) { return *reinterpret_cast<const float4*>(p); }
template <> __device__ __forceinline__ float4 ldv4<bf16_t>(const bf16_t* p) {
  const uint2 v = *reinterpret_cast<const uint2*>(p);
  return float4{__uint_as_float(v.x << 16), __uint_as_float(v.x & 0xffff0000u), __uint_as_float(v.y << 16),
                __uint_as_float(v.y & 0xffff0000u)};
}
template <typename T> __device__ __forceinline__ void stv4(T* p, float4 v);
template <> __device__ __forceinline__ void stv4<float>(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
template <> __device__ __forceinline__ void stv4<bf16_t>(bf16_t* p, float4 v) {
  uint2 o;
  o.x = (uint32_t)f32_to_bf16(v.x) | ((uint32_t)f32_to_bf16(v.y) << 16);
  o.y = (uint32_t)f32_to_bf16(v.z) | ((uint32_t)f32_to_bf16(v.w) << 16);
  *reinterpret_cast<uint2*>(p) = o;
}

// ---------------------------------------------------------------------------------------
// h[n, :] += delta[n, :]   (float32 sum; delta float32 or bfloat16, or float32 slabs added in order)
// ---------------------------------------------------------------------------------------
template <typename TD>
__global__ void residual_add_kernel(float* __restrict__ h, const TD* __restrict__ delta, long long total, int nslabs,
                                    long long slab_stride) {
  const long long step = (long long)gridDim.x * blockDim.x;
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += step) {
    float d = ldf<TD>(delta + i);
    for (int c = 1; c < nslabs; ++c) d += ldf<TD>(delta + (size_t)c * slab_stride + i);
    h[i] += d;
  }
}

extern "C" int qvl_residual_add(void* h, const void* delta, long long total, int delta_dtype, int nslabs,
                                long long slab_stride, hipStream_t stream) {
  if (total <= 0) return QVL_OK;
  if (nslabs < 1 || (nslabs > 1 && delta_dtype != 0)) return QVL_ERR_SHAPE;
  const int blocks = (int)((total + 255) / 256 > 4096 ? 4096 : (total + 255) / 256);
  if (delta_dtype == 0)
    hipLaunchKernelGGL(residual_add_kernel<float>, dim3(blocks), dim3(256), 0, stream, (float*)h, (const float*)delta,
                       total, nslabs, slab_stride);
  else if (delta_dtype == 1)
    hipLaunchKernelGGL(residual_add_kernel<bf16_t>, dim3(blocks), dim3(256), 0, stream, (float*)h,
                       (const bf16_t*)delta, total, nslabs, slab_stride);
  else
    return QVL_ERR_DTYPE;
  return qvl_launch_status();
}

// ---------------------------------------------------------------------------------------
// Gated activation with clamps: x [N, 2 I] holds the gate branch in columns [0, I) and the linear
// branch in [I, 2 I);  g = min(gate, limit), u = clamp(lin, -limit, limit) (no clamps if limit <= 0)
//   out = g * sigmoid(alpha * g) * (u + shift)
// alpha 1, shift 0, no limit is SwiGLU.
// ---------------------------------------------------------------------------------------
template <typename T>
__global__ void gated_act_kernel(const T* __restrict__ x, T* __restrict__ out, int I, float alpha, float limit,
                                 float shift) {
  const size_t n = blockIdx.y;
  const T* xr = x + n * 2 * (size_t)I;
  T* o = out + n * (size_t)I;
  for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < I; i += gridDim.x * blockDim.x) {
    float g = ldf<T>(xr + i), u = ldf<T>(xr + I + i);
    if (limit > 0.f) {
      g = fminf(g, limit);
      u = fminf(fmaxf(u, -limit), limit);
    }
    stf<T>(o + i, g * sigmoid_f(alpha * g) * (u + shift));
  }
}

// The same, four values a thread (I a multiple of 4): one grid-stride loop over all rows.
template <typename T>
__global__ __launch_bounds__(256) void gated_act_vec_kernel(const T* __restrict__ x, T* __restrict__ out, int I,
                                                            long long vectors, float alpha, float limit, float shift) {
  const int per_row = I >> 2;
  const long long step = (long long)gridDim.x * blockDim.x;
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < vectors; i += step) {
    const long long n = i / per_row;
    const int c = (int)(i % per_row) << 2;
    const T* xr = x + n * 2 * (size_t)I + c;
    float4 g = ldv4<T>(xr), u = ldv4<T>(xr + I), y;
    float* gp = &g.x; float* up = &u.x; float* yp = &y.x;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      float gg = gp[k], uu = up[k];
      if (limit > 0.f) {
        gg = fminf(gg, limit);
        uu = fminf(fmaxf(uu, -limit), limit);
      }
      yp[k] = gg * sigmoid_f(alpha * gg) * (uu + shift);
    }
    stv4<T>(out + n * (size_t)I + c, y);
  }
}

extern "C" int qvl_gated_act(const void* x, void* out, int N, int I, int dtype, float alpha, float limit, float shift,
                             hipStream_t stream) {
  if (N <= 0 || I <= 0) return QVL_OK;
  if (I % 4 == 0 && (dtype == 0 || dtype == 1)) {
    const long long vectors = (long long)N * (I >> 2);
    const int blocks = (int)((vectors + 255) / 256 > 16384 ? 16384 : (vectors + 255) / 256);
    if (dtype == 0)
      hipLaunchKernelGGL(gated_act_vec_kernel<float>, dim3(blocks), dim3(256), 0, stream, (const float*)x, (float*)out,
                         I, vectors, alpha, limit, shift);
    else
      hipLaunchKernelGGL(gated_act_vec_kernel<bf16_t>, dim3(blocks), dim3(256), 0, stream, (const bf16_t*)x,
                         (bf16_t*)out, I, vectors, alpha, limit, shift);
    return qvl_launch_status();
  }
  if (N > 65535 * 16) return QVL_ERR_LIMIT;
  // rows go to blockIdx.y (at most 65,535): more rows are launched in pieces
  const int bx = (I + 255) / 256 > 64 ? 64 : (I + 255) / 256;
  for (int at = 0; at < N; at += 65535) {
    const int rows = N - at < 65535 ? N - at : 65535;
    if (dtype == 0)
      hipLaunchKernelGGL(gated_act_kernel<float>, dim3(bx, rows), dim3(256), 0, stream,
                         (const float*)x + (size_t)at * 2 * I, (float*)out + (size_t)at * I, I, alpha, limit, shift);
    else if (dtype == 1)
      hipLaunchKernelGGL(gated_act_kernel<bf16_t>, dim3(bx, rows), dim3(256), 0, stream,
                         (const bf16_t*)x + (size_t)at * 2 * I, (bf16_t*)out + (size_t)at * I, I, alpha, limit, shift);
    else
      return QVL_ERR_DTYPE;
  }
  return qvl_launch_status();
}

// ---------------------------------------------------------------------------------------
// logits = cap * tanh(logits / cap), in place, float32
// ---------------------------------------------------------------------------------------
__global__ void softcap_kernel(float* __restrict__ x, long long total, float cap) {
  const long long step = (long long)gridDim.x * blockDim.x;
  const float inv = 1.0f / cap;
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += step)
    x[i] = cap * tanhf(x[i] * inv);
}

extern "C" int qvl_softcap(void* x, long long total, float cap, hipStream_t stream) {
  if (total <= 0) return QVL_OK;
  if (!(cap > 0.f)) return QVL_ERR_SHAPE;
  const int blocks = (int)((total + 255) / 256 > 4096 ? 4096 : (total + 255) / 256);
  hipLaunchKernelGGL(softcap_kernel, dim3(blocks), dim3(256), 0, stream, (float*)x, total, cap);
  return qvl_launch_status();
}

// ---------------------------------------------------------------------------------------
// Norm over groups of `span` consecutive channels, then a gate:
//   y = x / sqrt(mean_group(x^2) + eps) * w[c % wlen] * act(gate[n, c])
// x float32 [N, C] (C a multiple of span), or `nslabs` such arrays `slab_stride` apart whose sum, taken
// in slab order, is x; gate is read from rows of `gate_stride` values starting at its own pointer;
// act: 0 no gate, 1 sigmoid, 2 silu.  One block per (group, token).
// ---------------------------------------------------------------------------------------
template <typename TG, typename TO>
__global__ void group_norm_gate_kernel(const float* __restrict__ x, const float* __restrict__ w, int wlen,
                                       const TG* __restrict__ gate, long long gate_stride, TO* __restrict__ out,
                                       int C, int span, float eps, int act, int nslabs, long long slab_stride) {
  __shared__ float red[17];
  const size_t n = blockIdx.y;
  const int c0 = blockIdx.x * span;
  const float* xr = x + n * (size_t)C + c0;
  auto x_at = [&](int i) {
    float v = xr[i];
    for (int s = 1; s < nslabs; ++s) v += xr[(size_t)s * slab_stride + i];
    return v;
  };
  float ss = 0.f;
  for (int i = threadIdx.x; i < span; i += blockDim.x) {
    const float v = x_at(i);
    ss += v * v;
  }
  const float rs = 1.0f / sqrtf(block_sum(ss, red) / (float)span + eps);
  TO* o = out + n * (size_t)C + c0;
  const TG* gr = gate ? gate + n * (size_t)gate_stride + c0 : nullptr;
  for (int i = threadIdx.x; i < span; i += blockDim.x) {
    float y = (x_at(i) * rs) * w[(c0 + i) % wlen];
    if (act) {
      const float g = ldf<TG>(gr + i);
      y *= act == 1 ? sigmoid_f(g) : g * sigmoid_f(g);
    }
    stf<TO>(o + i, y);
  }
}

// The same with a team of TEAM threads (a wave, or the block) per group, four values at a time, the
// group's values held in registers between the two passes: span a multiple of 4 and at most
// TEAM * 4 * GN_VEC.  Blocks of 256 threads; blockIdx.x counts teams over all (token, group) pairs.
#define GN_VEC 4

template <typename TG, typename TO, int TEAM>
__global__ __launch_bounds__(256) void group_norm_gate_vec_kernel(
    const float* __restrict__ x, const float* __restrict__ w, int wlen, const TG* __restrict__ gate,
    long long gate_stride, TO* __restrict__ out, int C, int span, float eps, int act, int nslabs,
    long long slab_stride, long long items) {
  __shared__ float red[17];
  const int team = threadIdx.x / TEAM, lane = threadIdx.x % TEAM;
  const long long item = (long long)blockIdx.x * (256 / TEAM) + team;
  const bool live = item < items;               // a whole team at once
  const int groups = C / span;
  const size_t n = live ? (size_t)(item / groups) : 0;
  const int c0 = live ? (int)(item % groups) * span : 0;
  const float* xr = x + n * (size_t)C + c0;
  const int nvec = span >> 2;
  float4 v[GN_VEC];
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < GN_VEC; ++j) {
    const int i = lane + TEAM * j;
    v[j] = float4{0.f, 0.f, 0.f, 0.f};
    if (live && i < nvec) {
      v[j] = ldv4<float>(xr + 4 * i);
      for (int s = 1; s < nslabs; ++s) {
        const float4 a = ldv4<float>(xr + (size_t)s * slab_stride + 4 * i);
        v[j].x += a.x; v[j].y += a.y; v[j].z += a.z; v[j].w += a.w;
      }
      ss += v[j].x * v[j].x + v[j].y * v[j].y + v[j].z * v[j].z + v[j].w * v[j].w;
    }
  }
  const float total = TEAM == 64 ? wave_sum(ss) : block_sum(ss, red);
  if (!live) return;
  const float rs = 1.0f / sqrtf(total / (float)span + eps);
  TO* o = out + n * (size_t)C + c0;
  const TG* gr = gate ? gate + n * (size_t)gate_stride + c0 : nullptr;
#pragma unroll
  for (int j = 0; j < GN_VEC; ++j) {
    const int i = lane + TEAM * j;
    if (i < nvec) {
      const int wc = (c0 + 4 * i) % wlen;       // wlen is a multiple of 4 here, so the four stay in one period
      const float4 ww = ldv4<float>(w + wc);
      float4 y{(v[j].x * rs) * ww.x, (v[j].y * rs) * ww.y, (v[j].z * rs) * ww.z, (v[j].w * rs) * ww.w};
      if (act) {
        const float4 g = ldv4<TG>(gr + 4 * i);
        if (act == 1) { y.x *= sigmoid_f(g.x); y.y *= sigmoid_f(g.y); y.z *= sigmoid_f(g.z); y.w *= sigmoid_f(g.w); }
        else { y.x *= g.x * sigmoid_f(g.x); y.y *= g.y * sigmoid_f(g.y); y.z *= g.z * sigmoid_f(g.z); y.w *= g.w * sigmoid_f(g.w); }
      }
      stv4<TO>(o + 4 * i, y);
    }
  }
}

extern "C" int qvl_group_norm_gate(const void* x, const void* w, int wlen, const void* gate, long long gate_stride,
                                   int gate_dtype, void* out, int out_dtype, int N, int C, int span, float eps, int act,
                                   int nslabs, long long slab_stride, hipStream_t stream) {
  if (N <= 0 || C <= 0) return QVL_OK;
  if (span <= 0 || C % span || wlen <= 0 || (act && !gate) || act < 0 || act > 2 || nslabs < 1) return QVL_ERR_SHAPE;
  if (C / span > 65535 * 16) return QVL_ERR_LIMIT;
  // the vector kernel: widths, strides and addresses in steps of four values (16 bytes of float32)
  const int gbytes = gate_dtype == 0 ? 4 : 2;
  const bool vec = span % 4 == 0 && wlen % 4 == 0 && span <= 256 * 4 * GN_VEC && slab_stride % 4 == 0 &&
                   (uintptr_t)x % 16 == 0 && (uintptr_t)w % 16 == 0 && (uintptr_t)out % 16 == 0 &&
                   (!gate || (gate_stride % 4 == 0 && (uintptr_t)gate % (4 * gbytes) == 0));
  if (vec) {
    const long long items = (long long)N * (C / span);
    const bool wave = span <= 64 * 4 * GN_VEC;
    const long long blocks = wave ? (items + 3) / 4 : items;
    if (blocks > 0x7fffffffLL) return QVL_ERR_LIMIT;
#define LAUNCHV(TG, TO, TEAM)                                                                                      \
    hipLaunchKernelGGL((group_norm_gate_vec_kernel<TG, TO, TEAM>), dim3((unsigned)blocks), dim3(256), 0, stream,   \
                       (const float*)x, (const float*)w, wlen, (const TG*)gate, gate_stride, (TO*)out, C, span,    \
                       eps, act, nslabs, slab_stride, items)
#define BY_TEAM(TG, TO) if (wave) LAUNCHV(TG, TO, 64); else LAUNCHV(TG, TO, 256)
    if (gate_dtype == 0 && out_dtype == 0) { BY_TEAM(float, float); }
    else if (gate_dtype == 1 && out_dtype == 1) { BY_TEAM(bf16_t, bf16_t); }
    else if (gate_dtype == 0 && out_dtype == 1) { BY_TEAM(float, bf16_t); }
    else return QVL_ERR_DTYPE;
#undef BY_TEAM
#undef LAUNCHV
    return qvl_launch_status();
  }
  const int threads = span >= 1024 ? 1024 : (span + 63) / 64 * 64;
#define LAUNCH(TG, TO)                                                                                            \
  for (int at = 0; at < N; at += 65535) {                                                                         \
    const int rows = N - at < 65535 ? N - at : 65535;                                                             \
    hipLaunchKernelGGL((group_norm_gate_kernel<TG, TO>), dim3(C / span, rows), dim3(threads), 0, stream,          \
                       (const float*)x + (size_t)at * C, (const float*)w, wlen,                                   \
                       gate ? (const TG*)gate + (size_t)at * gate_stride : (const TG*)nullptr, gate_stride,       \
                       (TO*)out + (size_t)at * C, C, span, eps, act, nslabs, slab_stride);                        \
  }
  if (gate_dtype == 0 && out_dtype == 0) { LAUNCH(float, float) }
  else if (gate_dtype == 1 && out_dtype == 1) { LAUNCH(bf16_t, bf16_t) }
  else if (gate_dtype == 0 && out_dtype == 1) { LAUNCH(float, bf16_t) }
  else return QVL_ERR_DTYPE;
#undef LAUNCH
  return qvl_launch_status();
}

// ---------------------------------------------------------------------------------------
// Per-head output gate: o[n, h, :] *= sigmoid(gate[n, h]);  gate float32 with a row stride.
// ---------------------------------------------------------------------------------------
template <typename T>
__global__ void head_gate_kernel(T* __restrict__ o, const float* __restrict__ gate, long long gate_stride, int nh,
                                 int hd) {
  const size_t n = blockIdx.x;
  T* orow = o + n * (size_t)nh * hd;
  const float* g = gate + n * (size_t)gate_stride;
  for (int i = threadIdx.x; i < nh * hd; i += blockDim.x) stf<T>(orow + i, ldf<T>(orow + i) * sigmoid_f(g[i / hd]));
}

extern "C" int qvl_head_gate(void* o, const void* gate, long long gate_stride, int N, int nh, int hd, int dtype,
                             hipStream_t stream) {
  if (N <= 0) return QVL_OK;
  if (nh <= 0 || hd <= 0 || gate_stride < nh) return QVL_ERR_SHAPE;
  if (dtype == 0)
    hipLaunchKernelGGL(head_gate_kernel<float>, dim3(N), dim3(256), 0, stream, (float*)o, (const float*)gate,
                       gate_stride, nh, hd);
  else if (dtype == 1)
    hipLaunchKernelGGL(head_gate_kernel<bf16_t>, dim3(N), dim3(256), 0, stream, (bf16_t*)o, (const float*)gate,
                       gate_stride, nh, hd);
  else
    return QVL_ERR_DTYPE;
  return qvl_launch_status();
}

// ---------------------------------------------------------------------------------------
// Queries and keys of attention with a per-head norm before or after the rotation:
//   x [N, stride] float32: nq query heads and nkv key heads of hd channels, then nkv value heads of
//   vd channels (none if the values are the keys as projected: `v_from_k`).  `bias` (or null) is
//   added to every column first.
//   head vector a -> a / sqrt(mean(a^2) + eps) * nw (nw = qw for query heads, kw for key heads; a
//   null weight is a gain of one) -> rotation of the first 2 rot_half channels by the angles whose
//   cosines and sines are cs[n, f]: pair (2f, 2f+1) if `interleaved`, else (f, f + rot_half).
//   norm_mode 0: no norm; 1: the norm comes before the rotation; 2: after it; 3: before it and over all
//   query heads of a token together (and all its key heads together): the two inverse root mean squares
//   come in `row_rs` [N, 2] (row_inv_rms below forms them) and the weights span all heads' columns.
//   Queries go to q_out [N, nq hd]; keys into k_cache [pages, nkv, ps, hd] at slots[n]; values
//   (the key head before norm and rotation, or the value head) into v_cache [pages, nkv, vd, ps].
// One wave per (token, head); a block holds 4 of them.  hd, vd <= 512.
// ---------------------------------------------------------------------------------------
#define QKN_MAX_HD 512

template <typename T>
__global__ __launch_bounds__(256) void qk_norm_rope_write_kernel(
    const float* __restrict__ x, long long x_stride, const float* __restrict__ bias, const float* __restrict__ qw,
    const float* __restrict__ kw, const float2* __restrict__ cs, const int* __restrict__ slots, T* __restrict__ q_out,
    T* __restrict__ k_cache, T* __restrict__ v_cache, int N, int nq, int nkv, int hd, int vd, int rot_half, int ps,
    float eps, int interleaved, int v_from_k, int write_kv, int norm_mode, const float* __restrict__ row_rs) {
  __shared__ float buf[4][QKN_MAX_HD];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int heads = nq + (write_kv ? (v_from_k ? nkv : 2 * nkv) : 0);
  const long long item = (long long)blockIdx.x * 4 + wave;
  if (item >= (long long)N * heads) return;
  const int n = (int)(item / heads), head = (int)(item % heads);
  const int kind = head < nq ? 0 : (head < nq + nkv ? 1 : 2);   // query, key, value head
  const size_t col = kind == 2 ? (size_t)(nq + nkv) * hd + (size_t)(head - nq - nkv) * vd : (size_t)head * hd;
  const float* a = x + (size_t)n * x_stride + col;
  const float* b = bias ? bias + col : nullptr;
  float* mine = buf[wave];
  const int slot = (head >= nq && write_kv) ? slots[n] : -1;
  if (kind != 0 && slot < 0) return;                            // a padding row writes nowhere
  const size_t page = slot >= 0 ? (size_t)(slot / ps) : 0;
  const int in_page = slot >= 0 ? slot % ps : 0;
  if (kind == 2) {
    const int kvh = head - nq - nkv;
    T* vrow = v_cache + ((page * nkv + kvh) * vd) * (size_t)ps + in_page;
    for (int c = lane; c < vd; c += 64) stf<T>(vrow + (size_t)c * ps, a[c] + (b ? b[c] : 0.f));
    return;
  }
  float ss = 0.f;
  for (int c = lane; c < hd; c += 64) {
    const float v = a[c] + (b ? b[c] : 0.f);
    mine[c] = v;
    ss += v * v;
  }
  const float* nw = kind == 0 ? qw : kw;
  if (kind == 1 && v_from_k) {
    const int kvh = head - nq;
    T* vrow = v_cache + ((page * nkv + kvh) * vd) * (size_t)ps + in_page;
    for (int c = lane; c < hd; c += 64) stf<T>(vrow + (size_t)c * ps, mine[c]);
  }
  if (norm_mode == 1) {
    const float rs = 1.0f / sqrtf(wave_sum(ss) / (float)hd + eps);
    for (int c = lane; c < hd; c += 64) mine[c] = nw ? (mine[c] * rs) * nw[c] : mine[c] * rs;
  } else if (norm_mode == 3) {
    const float rs = row_rs[2 * (size_t)n + kind];
    const float* nwh = nw ? nw + (size_t)(kind == 0 ? head : head - nq) * hd : nullptr;
    for (int c = lane; c < hd; c += 64) mine[c] = nwh ? (mine[c] * rs) * nwh[c] : mine[c] * rs;
  }
  __builtin_amdgcn_wave_barrier();
  T* dst = kind == 0 ? q_out + ((size_t)n * nq + head) * hd
                     : k_cache + ((page * nkv + (head - nq)) * ps + in_page) * (size_t)hd;
  const float2* csn = cs + (size_t)n * rot_half;
  float turned[QKN_MAX_HD / 64];
  float ss2 = 0.f;
#pragma unroll
  for (int i = 0; i < QKN_MAX_HD / 64; ++i) {
    const int c = lane + 64 * i;
    float v = 0.f;
    if (c < hd) {
      v = mine[c];
      if (c < 2 * rot_half) {
        int f, partner;
        bool first;
        if (interleaved) { f = c >> 1; first = !(c & 1); partner = c ^ 1; }
        else { first = c < rot_half; f = first ? c : c - rot_half; partner = first ? c + rot_half : c - rot_half; }
        const float2 t = csn[f];
        const float p = mine[partner];
        v = first ? v * t.x - p * t.y : v * t.x + p * t.y;
      }
    }
    turned[i] = v;
    ss2 += v * v;
  }
  const float rs2 = norm_mode == 2 ? 1.0f / sqrtf(wave_sum(ss2) / (float)hd + eps) : 1.0f;
#pragma unroll
  for (int i = 0; i < QKN_MAX_HD / 64; ++i) {
    const int c = lane + 64 * i;
    if (c < hd) {
      float v = turned[i];
      if (norm_mode == 2) v = nw ? (v * rs2) * nw[c] : v * rs2;
      stf<T>(dst + c, v);
    }
  }
}

extern "C" int qvl_qk_norm_rope_write(const void* x, long long x_stride, const void* bias, const void* qw,
                                      const void* kw, const void* cs, const void* slots, void* q_out, void* k_cache,
                                      void* v_cache, int N, int nq, int nkv, int hd, int vd, int rot_half, int ps,
                                      float eps, int interleaved, int v_from_k, int write_kv, int norm_mode,
                                      const void* row_rs, int dtype, hipStream_t stream) {
  if (N <= 0) return QVL_OK;
  if (nq <= 0 || nkv < 0 || hd <= 0 || vd <= 0 || rot_half < 0 || 2 * rot_half > hd || ps <= 0) return QVL_ERR_SHAPE;
  if (write_kv && (!slots || !k_cache || !v_cache || nkv <= 0)) return QVL_ERR_SHAPE;
  if (norm_mode < 0 || norm_mode > 3 || (norm_mode == 3 && !row_rs) || (v_from_k && vd != hd)) return QVL_ERR_SHAPE;
  if (hd > QKN_MAX_HD || vd > QKN_MAX_HD) return QVL_ERR_LIMIT;
  const int heads = nq + (write_kv ? (v_from_k ? nkv : 2 * nkv) : 0);
  const long long items = (long long)N * heads;
  const unsigned blocks = (unsigned)((items + 3) / 4);
#define LAUNCH(T)                                                                                                  \
  hipLaunchKernelGGL(qk_norm_rope_write_kernel<T>, dim3(blocks), dim3(256), 0, stream, (const float*)x, x_stride,   \
                     (const float*)bias, (const float*)qw, (const float*)kw, (const float2*)cs, (const int*)slots, \
                     (T*)q_out, (T*)k_cache, (T*)v_cache, N, nq, nkv, hd, vd, rot_half, ps, eps, interleaved,      \
                     v_from_k, write_kv, norm_mode, (const float*)row_rs)
  if (dtype == 0) LAUNCH(float);
  else if (dtype == 1) LAUNCH(bf16_t);
  else return QVL_ERR_DTYPE;
#undef LAUNCH
  return qvl_launch_status();
}

// ---------------------------------------------------------------------------------------
// Inverse root mean squares of two neighbouring column ranges of every row:
//   out[n, 0] = 1 / sqrt(mean((x[n, 0 .. c0) + bias)^2) + eps),  out[n, 1] the same over [c0, c0 + c1)
// (c1 may be 0: then out[n, 1] is 1).  One block per row; the order of the sums depends on the sizes only.
// ---------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void row_inv_rms_kernel(const float* __restrict__ x, long long x_stride,
                                                          const float* __restrict__ bias, int c0, int c1, float eps,
                                                          float* __restrict__ out) {
  __shared__ float red[17];
  const size_t n = blockIdx.x;
  const float* row = x + n * x_stride;
  float s0 = 0.f, s1 = 0.f;
  for (int c = threadIdx.x; c < c0; c += blockDim.x) {
    const float v = row[c] + (bias ? bias[c] : 0.f);
    s0 += v * v;
  }
  for (int c = threadIdx.x; c < c1; c += blockDim.x) {
    const float v = row[c0 + c] + (bias ? bias[c0 + c] : 0.f);
    s1 += v * v;
  }
  const float t0 = block_sum(s0, red);
  __syncthreads();
  const float t1 = c1 > 0 ? block_sum(s1, red) : 0.f;
  if (threadIdx.x == 0) {
    out[2 * n] = 1.0f / sqrtf(t0 / (float)c0 + eps);
    out[2 * n + 1] = c1 > 0 ? 1.0f / sqrtf(t1 / (float)c1 + eps) : 1.0f;
  }
}

extern "C" int qvl_row_inv_rms(const void* x, long long x_stride, const void* bias, int c0, int c1, float eps, void* out,
                               int N, hipStream_t stream) {
  if (N <= 0) return QVL_OK;
  if (c0 <= 0 || c1 < 0 || x_stride < (long long)c0 + c1 || !x || !out) return QVL_ERR_SHAPE;
  hipLaunchKernelGGL(row_inv_rms_kernel, dim3(N), dim3(256), 0, stream, (const float*)x, x_stride, (const float*)bias,
                     c0, c1, eps, (float*)out);
  return qvl_launch_status();
}

// ---------------------------------------------------------------------------------------
// The sum of a residual stream whose sublayers are normed on their way in:
//   h[n, :] += factor * (y[n, :] / sqrt(mean(y[n]^2) + eps_y)) * gain + vec
// (y float32 or bfloat16, or float32 slabs added in order; a null gain adds y as it is; a null y
// adds nothing; vec, or null, is one vector for every row), and, if `out` is given, the next norm
//   out[m, :] = h[n, :] / sqrt(mean(h[n]^2) + eps) * w
// and, if `out2` is given, the same rows under a second gain, out2[m, :] = ... * w2 (two sublayers that
// read the same sum through norms of their own)
// With `rows`, n = rows[m] and h is only read (the sum is formed for the rows asked for).
// One block per row; a thread keeps its values of the row in registers between the passes.
// ---------------------------------------------------------------------------------------
#define SN_VPT 16

template <typename TY, typename TO, int VPT>
__global__ void sandwich_norm_kernel(float* __restrict__ h, const TY* __restrict__ y, int nslabs, long long slab_stride,
                                     const float* __restrict__ gain, float eps_y, float factor,
                                     const float* __restrict__ vec, const float* __restrict__ w, float eps,
                                     TO* __restrict__ out, const int* __restrict__ rows, int H,
                                     const float* __restrict__ w2, TO* __restrict__ out2) {
  __shared__ float red[17];
  const int m = blockIdx.x, n = rows ? rows[m] : m;
  float* hr = h + (size_t)n * H;
  // Everything a thread needs of the row is asked for before the first sum is waited for, and no load
  // stands inside a branch (the compiler would wait for each before the next): a column past the row's
  // end reads column 0 and counts as zero.
  float val[VPT], hv[VPT], gv[VPT], wv[VPT];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int c = threadIdx.x + i * blockDim.x;
    const bool ok = c < H;
    const int cc = ok ? c : 0;
    float v = y ? ldf<TY>(y + (size_t)n * H + cc) : 0.f;
    for (int s = 1; s < nslabs; ++s) v += ldf<TY>(y + (size_t)s * slab_stride + (size_t)n * H + cc);
    float add = vec ? vec[cc] : 0.f;
    hv[i] = ok ? hr[cc] + add : 0.f;
    gv[i] = gain ? gain[cc] : 1.f;
    wv[i] = w ? w[cc] : 1.f;
    v = ok ? v : 0.f;
    val[i] = v;
    ss += v * v;
  }
  float rs = 1.0f;
  if (y && gain) rs = factor / sqrtf(block_sum(ss, red) / (float)H + eps_y);
  float ss2 = 0.f;
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int c = threadIdx.x + i * blockDim.x;
    float v = hv[i];
    if (y) v += gain ? (val[i] * rs) * gv[i] : val[i];
    if (c < H && !rows && (y || vec)) hr[c] = v;
    val[i] = v;
    ss2 += v * v;
  }
  if (!out) return;
  const float rs2 = 1.0f / sqrtf(block_sum(ss2, red) / (float)H + eps);
  TO* o = out + (size_t)m * H;
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int c = threadIdx.x + i * blockDim.x;
    if (c < H) stf<TO>(o + c, (val[i] * rs2) * wv[i]);
  }
  if (!out2) return;
  TO* o2 = out2 + (size_t)m * H;
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int c = threadIdx.x + i * blockDim.x;
    if (c < H) stf<TO>(o2 + c, (val[i] * rs2) * w2[c]);
  }
}

// The same for rows of up to 4,096 values whose width is a multiple of 4: a thread owns four neighbouring
// columns and asks for them 16 bytes at a time (8 of a bfloat16 addend).
template <typename TY, typename TO>
__global__ void sandwich_norm_vec4_kernel(float* __restrict__ h, const TY* __restrict__ y, int nslabs, long long slab_stride,
                                          const float* __restrict__ gain, float eps_y, float factor,
                                          const float* __restrict__ vec, const float* __restrict__ w, float eps,
                                          TO* __restrict__ out, const int* __restrict__ rows, int H,
                                          const float* __restrict__ w2, TO* __restrict__ out2) {
  __shared__ float red[17];
  const int m = blockIdx.x, n = rows ? rows[m] : m;
  const int c = 4 * threadIdx.x;
  const bool ok = c < H;
  const int cc = ok ? c : 0;            // a thread past the row's end reads its start and counts as zero
  float* hr = h + (size_t)n * H;
  float4 v = float4{0.f, 0.f, 0.f, 0.f};
  if (y) {
    v = ldv4<TY>(y + (size_t)n * H + cc);
    for (int s = 1; s < nslabs; ++s) {
      const float4 t = ldv4<TY>(y + (size_t)s * slab_stride + (size_t)n * H + cc);
      v.x += t.x; v.y += t.y; v.z += t.z; v.w += t.w;
    }
  }
  float4 hv = ldv4<float>(hr + cc);
  const float4 add = vec ? ldv4<float>(vec + cc) : float4{0.f, 0.f, 0.f, 0.f};
  const float4 gv = gain ? ldv4<float>(gain + cc) : float4{1.f, 1.f, 1.f, 1.f};
  const float4 wv = w ? ldv4<float>(w + cc) : float4{1.f, 1.f, 1.f, 1.f};
  const float4 wv2 = w2 ? ldv4<float>(w2 + cc) : float4{1.f, 1.f, 1.f, 1.f};
  if (!ok) { v = float4{0.f, 0.f, 0.f, 0.f}; hv = v; }
  float rs = 1.0f;
  if (y && gain) rs = factor / sqrtf(block_sum(v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w, red) / (float)H + eps_y);
  float4 t;
  if (y && gain) t = float4{(v.x * rs) * gv.x, (v.y * rs) * gv.y, (v.z * rs) * gv.z, (v.w * rs) * gv.w};
  else t = v;
  t = float4{hv.x + add.x + t.x, hv.y + add.y + t.y, hv.z + add.z + t.z, hv.w + add.w + t.w};
  if (!ok) t = float4{0.f, 0.f, 0.f, 0.f};
  if (ok && !rows && (y || vec)) stv4<float>(hr + c, t);
  if (!out) return;
  const float rs2 = 1.0f / sqrtf(block_sum(t.x * t.x + t.y * t.y + t.z * t.z + t.w * t.w, red) / (float)H + eps);
  if (ok) stv4<TO>(out + (size_t)m * H + c, float4{(t.x * rs2) * wv.x, (t.y * rs2) * wv.y, (t.z * rs2) * wv.z, (t.w * rs2) * wv.w});
  if (ok && out2)
    stv4<TO>(out2 + (size_t)m * H + c, float4{(t.x * rs2) * wv2.x, (t.y * rs2) * wv2.y, (t.z * rs2) * wv2.z, (t.w * rs2) * wv2.w});
}

extern "C" int qvl_sandwich_norm(void* h, const void* y, int y_dtype, int nslabs, long long slab_stride, const void* gain,
                                 float eps_y, float factor, const void* vec, const void* w, float eps, void* out,
                                 int out_dtype, const void* rows, int M, int H, const void* w2, void* out2,
                                 hipStream_t stream) {
  if (M <= 0) return QVL_OK;
  if (H <= 0 || nslabs < 1 || (nslabs > 1 && y_dtype != 0) || (out && !w) || (out2 && (!w2 || !out))) return QVL_ERR_SHAPE;
  if (H > 1024 * SN_VPT) return QVL_ERR_LIMIT;
  // rows up to 4,096 wide: four values a thread (few rows are a chain of waits, and short chains end sooner)
  const int vpt = H <= 4096 ? 4 : SN_VPT;
  int threads = ((H + vpt - 1) / vpt + 63) / 64 * 64;
  const bool vec4 = H % 4 == 0 && H <= 4096 && slab_stride % 4 == 0 &&
                    (((uintptr_t)h | (uintptr_t)y | (uintptr_t)gain | (uintptr_t)vec | (uintptr_t)w | (uintptr_t)out |
                      (uintptr_t)w2 | (uintptr_t)out2) & 15) == 0;
#define LAUNCH(TY, TO)                                                                                              \
  if (vec4)                                                                                                         \
    hipLaunchKernelGGL((sandwich_norm_vec4_kernel<TY, TO>), dim3(M), dim3((H / 4 + 63) / 64 * 64), 0, stream,       \
                       (float*)h, (const TY*)y, nslabs, slab_stride, (const float*)gain, eps_y, factor,             \
                       (const float*)vec, (const float*)w, eps, (TO*)out, (const int*)rows, H, (const float*)w2,    \
                       (TO*)out2);                                                                                  \
  else if (vpt == 4)                                                                                                \
    hipLaunchKernelGGL((sandwich_norm_kernel<TY, TO, 4>), dim3(M), dim3(threads), 0, stream, (float*)h,             \
                       (const TY*)y, nslabs, slab_stride, (const float*)gain, eps_y, factor, (const float*)vec,     \
                       (const float*)w, eps, (TO*)out, (const int*)rows, H, (const float*)w2, (TO*)out2);           \
  else                                                                                                              \
    hipLaunchKernelGGL((sandwich_norm_kernel<TY, TO, SN_VPT>), dim3(M), dim3(threads), 0, stream, (float*)h,        \
                       (const TY*)y, nslabs, slab_stride, (const float*)gain, eps_y, factor, (const float*)vec,     \
                       (const float*)w, eps, (TO*)out, (const int*)rows, H, (const float*)w2, (TO*)out2)
  if (y_dtype == 0 && out_dtype == 0) { LAUNCH(float, float); }
  else if (y_dtype == 0 && out_dtype == 1) { LAUNCH(float, bf16_t); }
  else if (y_dtype == 1 && out_dtype == 1) { LAUNCH(bf16_t, bf16_t); }
  else if (y_dtype == 1 && out_dtype == 0) { LAUNCH(bf16_t, float); }
  else return QVL_ERR_DTYPE;
#undef LAUNCH
  return qvl_launch_status();
}
