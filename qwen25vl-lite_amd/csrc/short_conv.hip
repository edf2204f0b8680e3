// A short causal convolution over time on every channel, added to its input or standing alone:
//   out[t, c] = [x[t, c] +] sum_j w[j, c] * x[t - taps + 1 + j, c],   j = 0 .. taps - 1   (w is [taps, C])
// over the tokens of one request; inputs before the request's first token are zeros.  Rows of x may lie
// further apart than C values (the first C columns of a wider product).  The last taps - 1
// inputs of a request are its state (float32 [slots, taps - 1, C], oldest first), read by the first tokens
// of the request's next run and replaced at the end of this one.  x is the float32 residual; the result is
// written in the run's storage type or in float32.
//
// Grid (N + R, channel blocks); a thread owns one channel, or four neighbouring ones where 4 divides C.
// Rows below N are tokens: a token that stands at least taps - 1 tokens into its run reads only x.  The last R rows are requests: the thread of a channel forms the outputs of the
// run's first taps - 1 tokens from the old state and then writes the new one, so nobody else reads or
// writes that channel of the slot in this launch.
#include "common.h"

// VEC neighbouring channels a thread (4 with C a multiple of 4: 16-byte loads of x and of the state)
template <int VEC> struct Chan { float v[VEC]; };
template <int VEC> __device__ __forceinline__ Chan<VEC> ld_chan(const float* p) {
  Chan<VEC> o;
  if (VEC == 4) {
    const float4 t = *reinterpret_cast<const float4*>(p);
    o.v[0] = t.x; o.v[VEC > 1 ? 1 : 0] = t.y; o.v[VEC > 2 ? 2 : 0] = t.z; o.v[VEC > 3 ? 3 : 0] = t.w;
  } else {
    o.v[0] = *p;
  }
  return o;
}
template <int VEC> __device__ __forceinline__ void st_chan(float* p, const Chan<VEC>& a) {
  if (VEC == 4) *reinterpret_cast<float4*>(p) = float4{a.v[0], a.v[VEC > 1 ? 1 : 0], a.v[VEC > 2 ? 2 : 0], a.v[VEC > 3 ? 3 : 0]};
  else *p = a.v[0];
}
template <typename TO, int VEC> __device__ __forceinline__ void st_out(TO* p, const Chan<VEC>& a) {
  if (VEC == 4 && sizeof(TO) == 2) {            // four bfloat16 values: one 8-byte store (rows of out are C values apart)
    uint2 o;
    o.x = (uint32_t)f32_to_bf16(a.v[0]) | ((uint32_t)f32_to_bf16(a.v[VEC > 1 ? 1 : 0]) << 16);
    o.y = (uint32_t)f32_to_bf16(a.v[VEC > 2 ? 2 : 0]) | ((uint32_t)f32_to_bf16(a.v[VEC > 3 ? 3 : 0]) << 16);
    *reinterpret_cast<uint2*>(p) = o;
    return;
  }
#pragma unroll
  for (int u = 0; u < VEC; ++u) stf<TO>(p + u, a.v[u]);
}

// MAXT: up to this many taps a token's loads are issued together
template <typename TO, int VEC, int MAXT>
__global__ __launch_bounds__(256) void short_conv_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                         float* __restrict__ state, const int* __restrict__ cu_q,
                                                         const int* __restrict__ req_slots,
                                                         const int* __restrict__ token_req, TO* __restrict__ out, int N,
                                                         int C, int taps, long long xs, int plus) {
  const int c = (blockIdx.y * blockDim.x + threadIdx.x) * VEC;
  if (c >= C) return;
  const float* wc = w + c;                      // tap j of channels c ..: wc[j * C]
  const int keep = taps - 1;
  if ((int)blockIdx.x < N) {
    const int t = blockIdx.x;
    const int i = t - cu_q[token_req[t]];
    if (i < keep) return;                       // the request's row forms it from the state
    if (taps <= MAXT) {
      // every load is on its way before the first is used: tap j >= taps reads tap taps - 1 again and counts zero
      Chan<VEC> xv[MAXT];
      float wv[VEC][MAXT];
#pragma unroll
      for (int j = 0; j < MAXT; ++j) {
        const int jj = j < taps ? j : keep;
        xv[j] = ld_chan<VEC>(x + (size_t)(t - keep + jj) * xs + c);
        const Chan<VEC> wj = ld_chan<VEC>(wc + (size_t)jj * C);
#pragma unroll
        for (int u = 0; u < VEC; ++u) wv[u][j] = wj.v[u];
      }
      Chan<VEC> acc = xv[MAXT - 1];              // x[t]
      if (!plus) {
#pragma unroll
        for (int u = 0; u < VEC; ++u) acc.v[u] = 0.f;
      }
#pragma unroll
      for (int j = 0; j < MAXT; ++j)
#pragma unroll
        for (int u = 0; u < VEC; ++u) acc.v[u] += (j < taps ? wv[u][j] : 0.f) * xv[j].v[u];
      st_out<TO, VEC>(out + (size_t)t * C + c, acc);
      return;
    }
    Chan<VEC> acc = ld_chan<VEC>(x + (size_t)t * xs + c);
    if (!plus) {
#pragma unroll
      for (int u = 0; u < VEC; ++u) acc.v[u] = 0.f;
    }
    for (int j = 0; j < taps; ++j) {
      const Chan<VEC> v = ld_chan<VEC>(x + (size_t)(t - keep + j) * xs + c);
      const Chan<VEC> wj = ld_chan<VEC>(wc + (size_t)j * C);
#pragma unroll
      for (int u = 0; u < VEC; ++u) acc.v[u] += wj.v[u] * v.v[u];
    }
    st_out<TO, VEC>(out + (size_t)t * C + c, acc);
    return;
  }
  const int r = blockIdx.x - N;
  const int begin = cu_q[r], n = cu_q[r + 1] - begin;
  if (n <= 0) return;
  float* st = state + (size_t)req_slots[r] * keep * C + c;      // st[k * C]: input number k of the kept ones
  const int first = n < keep ? n : keep;
  for (int i = 0; i < first; ++i) {
    Chan<VEC> acc = ld_chan<VEC>(x + (size_t)(begin + i) * xs + c);
    if (!plus) {
#pragma unroll
      for (int u = 0; u < VEC; ++u) acc.v[u] = 0.f;
    }
    for (int j = 0; j < taps; ++j) {
      const int src = i - keep + j;             // index into this run; negative: the kept inputs
      const Chan<VEC> v = src >= 0 ? ld_chan<VEC>(x + (size_t)(begin + src) * xs + c) : ld_chan<VEC>(st + (size_t)(keep + src) * C);
      const Chan<VEC> wj = ld_chan<VEC>(wc + (size_t)j * C);
#pragma unroll
      for (int u = 0; u < VEC; ++u) acc.v[u] += wj.v[u] * v.v[u];
    }
    st_out<TO, VEC>(out + (size_t)(begin + i) * C + c, acc);
  }
  // the last `keep` inputs of (kept inputs, this run); entry k comes from a place behind k, so ascending order
  // never reads what it has overwritten
  for (int k = 0; k < keep; ++k) {
    const int at = n + k;                       // index into (kept inputs, this run)
    st_chan<VEC>(st + (size_t)k * C, at < keep ? ld_chan<VEC>(st + (size_t)at * C) : ld_chan<VEC>(x + (size_t)(begin + at - keep) * xs + c));
  }
}

// x float32 [N, C] with rows x_stride values apart (plus_input 0: the convolution without its input added); w float32 [taps, C] (tap j of every channel side by side); state float32 [slots, taps - 1, C] (unused with taps == 1);
// cu_q [R + 1], req_slots [R], token_req [N] int32; out [N, C] of out_dtype (0 float32, 1 bfloat16).
extern "C" int qvl_short_conv(const void* x, const void* w, void* state, const void* cu_q, const void* req_slots,
                              const void* token_req, void* out, int out_dtype, int N, int R, int C, int taps,
                              long long x_stride, int plus_input, hipStream_t stream) {
  if (N <= 0) return QVL_OK;
  if (R <= 0 || C <= 0 || taps < 1 || !x || !w || !out || !cu_q || !token_req) return QVL_ERR_SHAPE;
  if (taps > 1 && (!state || !req_slots)) return QVL_ERR_SHAPE;
  if (x_stride < C) return QVL_ERR_SHAPE;
  const long long rows = (long long)N + (taps > 1 ? R : 0);
  if (rows > 0x7fffffffll || (C + 255) / 256 > 65535) return QVL_ERR_LIMIT;
  const bool vec = C % 4 == 0 && x_stride % 4 == 0 && ((uintptr_t)x & 15) == 0 && ((uintptr_t)w & 15) == 0 && ((uintptr_t)state & 15) == 0 && ((uintptr_t)out & 15) == 0;
  const int per_block = vec ? 1024 : 256;
  const dim3 grid((unsigned)rows, (C + per_block - 1) / per_block);
#define SC_LAUNCH(TO, VEC)                                                                                          \
  hipLaunchKernelGGL((short_conv_kernel<TO, VEC, 4>), grid, dim3(256), 0, stream, (const float*)x, (const float*)w,     \
                     (float*)state, (const int*)cu_q, (const int*)req_slots, (const int*)token_req, (TO*)out, N, C, taps, x_stride, plus_input)
  if (out_dtype == 0) { if (vec) SC_LAUNCH(float, 4); else SC_LAUNCH(float, 1); }
  else if (out_dtype == 1) { if (vec) SC_LAUNCH(bf16_t, 4); else SC_LAUNCH(bf16_t, 1); }
  else return QVL_ERR_DTYPE;
#undef SC_LAUNCH
  return qvl_launch_status();
}
