// Row-wise kernels of layers whose norm stands behind the sublayer, and of feed-forwards whose activation
// is a sum of normed powers or a squared relu.  float32 and bfloat16 storage; all arithmetic is float32.
//
//   layer norm     y = (v - mean(v)) / sqrt(mean((v - mean(v))^2) + eps) * w      (no bias; two passes: the
//                  deviations are formed from the mean, not from a sum of squares)
//   normed powers  out = a z / rms(z) + b z^2 / rms(z^2) + c z^3 / rms(z^3) + e,  rms(u) = sqrt(mean(u^2) + eps),
//                  powers taken element by element over a row
//   squared relu   out = max(z, 0)^2
//
// A block of 256 threads owns a row.  Rows of up to 256 * 32 values stay in registers between the
// passes (PER values, or groups of four values, a thread); longer rows are read again.
#include "common.h"

#define RN_THREADS 256

// four neighbouring values at once (16 bytes of float32, 8 of bfloat16)
template <typename T> __device__ __forceinline__ float4 ld4v(const T* p);
template <> __device__ __forceinline__ float4 ld4v<float>(const float* p) { return *reinterpret_cast<const float4*>(p); }
template <> __device__ __forceinline__ float4 ld4v<bf16_t>(const bf16_t* p) {
  const uint2 v = *reinterpret_cast<const uint2*>(p);
  return float4{__uint_as_float(v.x << 16), __uint_as_float(v.x & 0xffff0000u), __uint_as_float(v.y << 16),
                __uint_as_float(v.y & 0xffff0000u)};
}
template <typename T> __device__ __forceinline__ void st4v(T* p, float4 v);
template <> __device__ __forceinline__ void st4v<float>(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
template <> __device__ __forceinline__ void st4v<bf16_t>(bf16_t* p, float4 v) {
  uint2 o;
  o.x = (uint32_t)f32_to_bf16(v.x) | ((uint32_t)f32_to_bf16(v.y) << 16);
  o.y = (uint32_t)f32_to_bf16(v.z) | ((uint32_t)f32_to_bf16(v.w) << 16);
  *reinterpret_cast<uint2*>(p) = o;
}

// A row's values as a block's threads hold them between the passes.  VEC 4 (H a multiple of 4, rows on 16-byte
// boundaries): a thread owns the columns 4 g .. 4 g + 3 for g = thread + 256 i, i < PER, all of them in
// registers, fetched with one load each; the loads of a pass are all on their way before the first value is
// used, slab by slab.  VEC 1: one column a load; PER > 0: the row lives in v[]; PER == 0: it is read again
// where it is needed.  Which form runs depends on H and the alignment alone, so the order of a row's sums
// does not depend on what else the step holds.
template <typename TS, int PER, int VEC>
struct RowValues {
  float v[PER > 0 ? PER * VEC : 1];
  const TS* src;
  int nslabs;
  long long slab_stride;
  int H;
  __device__ __forceinline__ float fetch(int c) const {
    float x = ldf<TS>(src + c);
    for (int s = 1; s < nslabs; ++s) x += ldf<TS>(src + (size_t)s * slab_stride + c);
    return x;
  }
  __device__ __forceinline__ void load() {
    if (VEC == 4) {
#pragma unroll
      for (int i = 0; i < (PER > 0 ? PER : 1); ++i) {
        const int c = (threadIdx.x + i * RN_THREADS) * 4;
        const float4 x = c < H ? ld4v<TS>(src + c) : float4{0.f, 0.f, 0.f, 0.f};
        v[4 * i] = x.x; v[4 * i + 1] = x.y; v[4 * i + 2] = x.z; v[4 * i + 3] = x.w;
      }
      for (int s = 1; s < nslabs; ++s) {
        const TS* slab = src + (size_t)s * slab_stride;
#pragma unroll
        for (int i = 0; i < (PER > 0 ? PER : 1); ++i) {
          const int c = (threadIdx.x + i * RN_THREADS) * 4;
          const float4 x = c < H ? ld4v<TS>(slab + c) : float4{0.f, 0.f, 0.f, 0.f};
          v[4 * i] += x.x; v[4 * i + 1] += x.y; v[4 * i + 2] += x.z; v[4 * i + 3] += x.w;
        }
      }
    } else if (PER > 0) {
#pragma unroll
      for (int i = 0; i < (PER > 0 ? PER : 1); ++i) {
        const int c = threadIdx.x + i * RN_THREADS;
        v[i] = c < H ? fetch(c) : 0.f;
      }
    }
  }
  // f(value, column) for every column this thread owns
  template <typename F> __device__ __forceinline__ void each(F f) const {
    if (VEC == 4) {
#pragma unroll
      for (int i = 0; i < (PER > 0 ? PER : 1); ++i) {
        const int c = (threadIdx.x + i * RN_THREADS) * 4;
        if (c < H) {
#pragma unroll
          for (int j = 0; j < 4; ++j) f(v[4 * i + j], c + j);
        }
      }
    } else if (PER > 0) {
#pragma unroll
      for (int i = 0; i < (PER > 0 ? PER : 1); ++i) {
        const int c = threadIdx.x + i * RN_THREADS;
        if (c < H) f(v[i], c);
      }
    } else {
      for (int c = threadIdx.x; c < H; c += RN_THREADS) f(fetch(c), c);
    }
  }
  // g(four values, first column) -> four values, for every group of four this thread owns (VEC 4 only)
  template <typename G> __device__ __forceinline__ void each4(G g) const {
#pragma unroll
    for (int i = 0; i < (PER > 0 ? PER : 1); ++i) {
      const int c = (threadIdx.x + i * RN_THREADS) * 4;
      if (c < H) g(float4{v[4 * i], v[4 * i + 1], v[4 * i + 2], v[4 * i + 3]}, c);
    }
  }
};

// src [rows, H] (or float32 slabs of it, added in order).  y = layer norm of row `rows[m]` (or m) times w.
// add != null: add[row] += y in float32 and y stands for the new sum from there on.  out != null: out[m] = y.
template <typename TS, typename TO, int PER, int VEC>
__global__ __launch_bounds__(RN_THREADS) void layer_norm_kernel(const TS* __restrict__ src, int nslabs,
                                                                long long slab_stride, const float* __restrict__ w,
                                                                float eps, float* __restrict__ add, TO* __restrict__ out,
                                                                const int* __restrict__ rows, int H) {
  __shared__ float red[17];
  const size_t m = blockIdx.x;
  const size_t row = rows ? (size_t)rows[m] : m;
  RowValues<TS, PER, VEC> r;
  r.src = src + row * H; r.nslabs = nslabs; r.slab_stride = slab_stride; r.H = H;
  r.load();
  float sum = 0.f;
  r.each([&](float x, int) { sum += x; });
  const float mean = block_sum(sum, red) / (float)H;
  float sq = 0.f;
  r.each([&](float x, int) { const float d = x - mean; sq += d * d; });
  const float inv = 1.0f / sqrtf(block_sum(sq, red) / (float)H + eps);
  float* arow = add ? add + row * H : nullptr;
  TO* orow = out ? out + m * H : nullptr;
  if (VEC == 4) {
    r.each4([&](float4 x, int c) {
      const float4 g = ld4v<float>(w + c);
      float4 y{(x.x - mean) * inv * g.x, (x.y - mean) * inv * g.y, (x.z - mean) * inv * g.z, (x.w - mean) * inv * g.w};
      if (arow) {
        const float4 a = ld4v<float>(arow + c);
        y.x += a.x; y.y += a.y; y.z += a.z; y.w += a.w;
        st4v<float>(arow + c, y);
      }
      if (orow) st4v<TO>(orow + c, y);
    });
    return;
  }
  r.each([&](float x, int c) {
    float y = (x - mean) * inv * w[c];
    if (arow) {
      y += arow[c];
      arow[c] = y;
    }
    if (orow) stf<TO>(orow + c, y);
  });
}

static inline bool aligned16(const void* p) { return ((uintptr_t)p & 15) == 0; }

template <typename TS, typename TO>
static int launch_layer_norm(const void* src, int nslabs, long long slab_stride, const void* w, float eps, void* add,
                             void* out, const void* rows, int M, int H, hipStream_t stream) {
#define LN_LAUNCH(PER, VEC)                                                                                           \
  hipLaunchKernelGGL((layer_norm_kernel<TS, TO, PER, VEC>), dim3(M), dim3(RN_THREADS), 0, stream, (const TS*)src,     \
                     nslabs, slab_stride, (const float*)w, eps, (float*)add, (TO*)out, (const int*)rows, H)
  if (H % 4 == 0 && H <= RN_THREADS * 4 * 32 && slab_stride % 4 == 0 && aligned16(src) && aligned16(w) && aligned16(add) &&
      aligned16(out)) {
    const int per = (H / 4 + RN_THREADS - 1) / RN_THREADS;
    if (per <= 1) LN_LAUNCH(1, 4);
    else if (per <= 2) LN_LAUNCH(2, 4);
    else if (per <= 4) LN_LAUNCH(4, 4);
    else if (per <= 8) LN_LAUNCH(8, 4);
    else if (per <= 16) LN_LAUNCH(16, 4);
    else LN_LAUNCH(32, 4);
    return qvl_launch_status();
  }
  const int per = (H + RN_THREADS - 1) / RN_THREADS;
  if (per <= 1) LN_LAUNCH(1, 1);
  else if (per <= 2) LN_LAUNCH(2, 1);
  else if (per <= 4) LN_LAUNCH(4, 1);
  else if (per <= 8) LN_LAUNCH(8, 1);
  else if (per <= 16) LN_LAUNCH(16, 1);
  else if (per <= 32) LN_LAUNCH(32, 1);
  else LN_LAUNCH(0, 1);
#undef LN_LAUNCH
  return qvl_launch_status();
}

// src_dtype / out_dtype: 0 float32, 1 bfloat16.  Slabs (nslabs > 1) are float32.  `add` (float32 [rows, H], may
// be null) and `out` ([M, H], may be null) as above; `rows` (int32 [M], may be null) picks rows of src.
extern "C" int qvl_layer_norm(const void* src, int src_dtype, int nslabs, long long slab_stride, const void* w, float eps,
                              void* add, void* out, int out_dtype, const void* rows, int M, int H, hipStream_t stream) {
  if (M <= 0) return QVL_OK;
  if (H <= 0 || !src || !w || nslabs < 1 || (nslabs > 1 && src_dtype != 0) || (!add && !out)) return QVL_ERR_SHAPE;
  if (src_dtype == 0 && (out_dtype == 0 || !out))
    return launch_layer_norm<float, float>(src, nslabs, slab_stride, w, eps, add, out, rows, M, H, stream);
  if (src_dtype == 0 && out_dtype == 1)
    return launch_layer_norm<float, bf16_t>(src, nslabs, slab_stride, w, eps, add, out, rows, M, H, stream);
  if (src_dtype == 1 && (out_dtype == 0 || !out))
    return launch_layer_norm<bf16_t, float>(src, nslabs, slab_stride, w, eps, add, out, rows, M, H, stream);
  if (src_dtype == 1 && out_dtype == 1)
    return launch_layer_norm<bf16_t, bf16_t>(src, nslabs, slab_stride, w, eps, add, out, rows, M, H, stream);
  return QVL_ERR_DTYPE;
}

// ---------------------------------------------------------------------------------------
// A sum of normed powers over the rows of z [N, I]; coeff float32 [4] = (a, b, c, e).
// ---------------------------------------------------------------------------------------
template <typename TS, typename TO, int PER, int VEC>
__global__ __launch_bounds__(RN_THREADS) void normed_powers_kernel(const TS* __restrict__ z, const float* __restrict__ coeff,
                                                                   float eps, TO* __restrict__ out, int I) {
  __shared__ float red[17];
  const size_t n = blockIdx.x;
  RowValues<TS, PER, VEC> r;
  r.src = z + n * I; r.nslabs = 1; r.slab_stride = 0; r.H = I;
  r.load();
  float s2 = 0.f, s4 = 0.f, s6 = 0.f;
  r.each([&](float x, int) {
    const float x2 = x * x;
    s2 += x2;
    s4 += x2 * x2;
    s6 += x2 * x2 * x2;
  });
  const float inv_i = 1.0f / (float)I;
  const float r1 = 1.0f / sqrtf(block_sum(s2, red) * inv_i + eps);
  const float r2 = 1.0f / sqrtf(block_sum(s4, red) * inv_i + eps);
  const float r3 = 1.0f / sqrtf(block_sum(s6, red) * inv_i + eps);
  const float a = coeff[0] * r1, b = coeff[1] * r2, c3 = coeff[2] * r3, e = coeff[3];
  TO* orow = out + n * I;
  if (VEC == 4) {
    r.each4([&](float4 x, int c) {
      st4v<TO>(orow + c, float4{((c3 * x.x + b) * x.x + a) * x.x + e, ((c3 * x.y + b) * x.y + a) * x.y + e,
                                ((c3 * x.z + b) * x.z + a) * x.z + e, ((c3 * x.w + b) * x.w + a) * x.w + e});
    });
    return;
  }
  r.each([&](float x, int c) { stf<TO>(orow + c, ((c3 * x + b) * x + a) * x + e); });
}

extern "C" int qvl_normed_powers(const void* z, int z_dtype, const void* coeff, float eps, void* out, int out_dtype, int N,
                                 int I, hipStream_t stream) {
  if (N <= 0) return QVL_OK;
  if (I <= 0 || !z || !coeff || !out) return QVL_ERR_SHAPE;
#define NP_LAUNCH(TS, TO, PER, VEC)                                                                                 \
  hipLaunchKernelGGL((normed_powers_kernel<TS, TO, PER, VEC>), dim3(N), dim3(RN_THREADS), 0, stream, (const TS*)z, \
                     (const float*)coeff, eps, (TO*)out, I)
#define NP_BY_SIZE(TS, TO)                                                                                          \
  if (vec) {                                                                                                        \
    const int per = (I / 4 + RN_THREADS - 1) / RN_THREADS;                                                          \
    if (per <= 1) NP_LAUNCH(TS, TO, 1, 4);                                                                          \
    else if (per <= 2) NP_LAUNCH(TS, TO, 2, 4);                                                                     \
    else if (per <= 4) NP_LAUNCH(TS, TO, 4, 4);                                                                     \
    else if (per <= 8) NP_LAUNCH(TS, TO, 8, 4);                                                                     \
    else if (per <= 12) NP_LAUNCH(TS, TO, 12, 4);                                                                   \
    else if (per <= 16) NP_LAUNCH(TS, TO, 16, 4);                                                                   \
    else if (per <= 20) NP_LAUNCH(TS, TO, 20, 4);                                                                   \
    else if (per <= 24) NP_LAUNCH(TS, TO, 24, 4);                                                                   \
    else NP_LAUNCH(TS, TO, 32, 4);                                                                                  \
  } else {                                                                                                          \
    const int per = (I + RN_THREADS - 1) / RN_THREADS;                                                              \
    if (per <= 1) NP_LAUNCH(TS, TO, 1, 1);                                                                          \
    else if (per <= 2) NP_LAUNCH(TS, TO, 2, 1);                                                                     \
    else if (per <= 4) NP_LAUNCH(TS, TO, 4, 1);                                                                     \
    else if (per <= 8) NP_LAUNCH(TS, TO, 8, 1);                                                                     \
    else if (per <= 16) NP_LAUNCH(TS, TO, 16, 1);                                                                   \
    else if (per <= 32) NP_LAUNCH(TS, TO, 32, 1);                                                                   \
    else NP_LAUNCH(TS, TO, 0, 1);                                                                                   \
  }
  const bool vec = I % 4 == 0 && I <= RN_THREADS * 4 * 32 && aligned16(z) && aligned16(out);
  if (z_dtype == 0 && out_dtype == 0) NP_BY_SIZE(float, float)
  else if (z_dtype == 0 && out_dtype == 1) NP_BY_SIZE(float, bf16_t)
  else if (z_dtype == 1 && out_dtype == 1) NP_BY_SIZE(bf16_t, bf16_t)
  else if (z_dtype == 1 && out_dtype == 0) NP_BY_SIZE(bf16_t, float)
  else return QVL_ERR_DTYPE;
#undef NP_BY_SIZE
#undef NP_LAUNCH
  return qvl_launch_status();
}

// ---------------------------------------------------------------------------------------
// out = max(z, 0)^2, element by element (out may be z)
// ---------------------------------------------------------------------------------------
template <typename T>
__global__ void squared_relu_kernel(const T* z, T* out, long long total) {
  const long long step = (long long)gridDim.x * blockDim.x;
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += step) {
    const float x = fmaxf(ldf<T>(z + i), 0.f);
    stf<T>(out + i, x * x);
  }
}

extern "C" int qvl_squared_relu(const void* z, void* out, long long total, int dtype, hipStream_t stream) {
  if (total <= 0) return QVL_OK;
  const int blocks = (int)((total + 255) / 256 > 16384 ? 16384 : (total + 255) / 256);
  if (dtype == 0)
    hipLaunchKernelGGL(squared_relu_kernel<float>, dim3(blocks), dim3(256), 0, stream, (const float*)z, (float*)out, total);
  else if (dtype == 1)
    hipLaunchKernelGGL(squared_relu_kernel<bf16_t>, dim3(blocks), dim3(256), 0, stream, (const bf16_t*)z, (bf16_t*)out,
                       total);
  else
    return QVL_ERR_DTYPE;
  return qvl_launch_status();
}
