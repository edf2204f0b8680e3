// Row-wise kernels of attention through a latent.  A token's down projections arrive as one row
//   [ query latent (q_rank) | key/value latent (kv_rank) | shared rotated key part (rot_dim) ]
// (the last two are absent in a layer that reads another layer's cache).  All arithmetic is float32.
//
// latent_down: the query latent is RMS-normed (weight wq) and written out for the up projection; the
//   key/value latent is RMS-normed (weight wkv) and, with the rotated key part behind it, becomes the
//   token's one cached key [kv_rank + rot_dim]; the normed latent alone is its cached value.  Keys lie
//   in pages [pages, 1, page_size, kv_rank + rot_dim], values transposed [pages, 1, kv_rank, page_size].
// latent_query: a head's query is [dim plain | rot_dim rotated]; the plain part has been multiplied
//   into the latent's space by the caller (into columns [0, kv_rank) of the head's slot of the output);
//   this kernel rotates the other part into columns [kv_rank, kv_rank + rot_dim).
// Rotation: of the first 2 * half channels of a rotated part, channel i is paired with channel i + half
// (or, `interleaved`, channel 2i with channel 2i + 1) and the pair turned by the angle whose (cos, sin)
// is cs[token, i]; the remaining channels pass.
// A layer whose queries do not pass a latent has q_rank 0: latent_down then only forms the cached key.
#include "common.h"

__device__ __forceinline__ float turned(const float* cs, int half, int ch, float self, float other_lo, float other_hi) {
  // ch < half: u' = u cos - v sin (other = v);   half <= ch < 2 half: v' = v cos + u sin (other = u)
  if (ch < half) return self * cs[2 * ch] - other_hi * cs[2 * ch + 1];
  if (ch < 2 * half) return self * cs[2 * (ch - half)] + other_lo * cs[2 * (ch - half) + 1];
  return self;
}

// channel ch of the rotated part `rot` (rot_dim channels) after the turn, in either pairing
template <typename T>
__device__ __forceinline__ float turned_at(const T* rot, const float* cs, int half, int ch, int interleaved) {
  const float self = ldf<T>(rot + ch);
  if (interleaved) {
    if (ch >= 2 * half) return self;
    const float other = ldf<T>(rot + (ch ^ 1));
    const float c = cs[2 * (ch >> 1)], s = cs[2 * (ch >> 1) + 1];
    return (ch & 1) ? self * c + other * s : self * c - other * s;
  }
  const float lo = ch >= half && ch < 2 * half ? ldf<T>(rot + ch - half) : 0.f;
  const float hi = ch < half ? ldf<T>(rot + ch + half) : 0.f;
  return turned(cs, half, ch, self, lo, hi);
}

template <typename TP, typename TO>
__global__ __launch_bounds__(256) void latent_down_kernel(const TP* __restrict__ proj, long long proj_stride, int q_rank,
                                                          int kv_rank, int rot_dim, const float* __restrict__ wq,
                                                          const float* __restrict__ wkv, float eps,
                                                          const float* __restrict__ cs, int half,
                                                          const int* __restrict__ slots, TO* __restrict__ cq,
                                                          TO* __restrict__ kc, TO* __restrict__ vc, int ps,
                                                          int interleaved) {
  __shared__ float red[17];
  const size_t n = blockIdx.x;
  const TP* row = proj + n * proj_stride;
  float sq = 0.f;
  if (q_rank > 0) {
    for (int c = threadIdx.x; c < q_rank; c += blockDim.x) {
      const float x = ldf<TP>(row + c);
      sq += x * x;
    }
    const float inv_q = 1.0f / sqrtf(block_sum(sq, red) / (float)q_rank + eps);
    for (int c = threadIdx.x; c < q_rank; c += blockDim.x) stf<TO>(cq + n * q_rank + c, ldf<TP>(row + c) * inv_q * wq[c]);
  }
  if (!kc) return;
  const int slot = slots[n];
  const TP* lat = row + q_rank;
  sq = 0.f;
  for (int c = threadIdx.x; c < kv_rank; c += blockDim.x) {
    const float x = ldf<TP>(lat + c);
    sq += x * x;
  }
  const float inv_c = 1.0f / sqrtf(block_sum(sq, red) / (float)kv_rank + eps);
  if (slot < 0) return;                         // a padding row: nothing is kept
  const size_t page = slot / ps, off = slot % ps;
  const int hd = kv_rank + rot_dim;
  TO* krow = kc + (page * ps + off) * hd;
  TO* vcol = vc + page * (size_t)kv_rank * ps + off;
  for (int c = threadIdx.x; c < kv_rank; c += blockDim.x) {
    const float y = ldf<TP>(lat + c) * inv_c * wkv[c];
    stf<TO>(krow + c, y);
    stf<TO>(vcol + (size_t)c * ps, y);
  }
  const TP* rot = lat + kv_rank;
  const float* csn = cs + n * 2 * half;
  for (int ch = threadIdx.x; ch < rot_dim; ch += blockDim.x)
    stf<TO>(krow + kv_rank + ch, turned_at<TP>(rot, csn, half, ch, interleaved));
}

template <typename TQ, typename TO>
__global__ __launch_bounds__(256) void latent_query_kernel(const TQ* __restrict__ q, long long q_stride, int heads, int dim,
                                                           int rot_dim, int kv_rank, const float* __restrict__ cs,
                                                           int half, TO* __restrict__ out, int interleaved) {
  const size_t n = blockIdx.x;
  const float* csn = cs + n * 2 * half;
  const int hd = kv_rank + rot_dim;
  for (int i = threadIdx.x; i < heads * rot_dim; i += blockDim.x) {
    const int h = i / rot_dim, ch = i % rot_dim;
    const TQ* rot = q + n * q_stride + (size_t)h * (dim + rot_dim) + dim;
    stf<TO>(out + (n * heads + h) * hd + kv_rank + ch, turned_at<TQ>(rot, csn, half, ch, interleaved));
  }
}

// proj [N, >= q_rank (+ kv_rank + rot_dim)] of proj_dtype with rows proj_stride apart; wq float32 [q_rank];
// cq [N, q_rank] of out_dtype (q_rank 0: neither).  With kc (and vc, wkv, slots, cs): the cache write as above; slots int32 [N], -1:
// the row keeps nothing; cs float32 [N, half, 2] with 2 * half <= rot_dim.
extern "C" int qvl_latent_down(const void* proj, long long proj_stride, int proj_dtype, int q_rank, int kv_rank,
                               int rot_dim, const void* wq, const void* wkv, float eps, const void* cs, int half,
                               const void* slots, void* cq, void* kc, void* vc, int ps, int out_dtype, int N,
                               int interleaved, hipStream_t stream) {
  if (N <= 0) return QVL_OK;
  if (q_rank < 0 || !proj || (q_rank > 0 && (!wq || !cq)) || (q_rank == 0 && !kc)) return QVL_ERR_SHAPE;
  if (kc && (kv_rank <= 0 || rot_dim < 0 || 2 * half > rot_dim || half < 0 || !vc || !wkv || !slots || ps <= 0 ||
             (half > 0 && !cs) || proj_stride < q_rank + kv_rank + rot_dim))
    return QVL_ERR_SHAPE;
#define LD_LAUNCH(TP, TO)                                                                                           \
  hipLaunchKernelGGL((latent_down_kernel<TP, TO>), dim3(N), dim3(256), 0, stream, (const TP*)proj, proj_stride, q_rank, \
                     kv_rank, rot_dim, (const float*)wq, (const float*)wkv, eps, (const float*)cs, half,            \
                     (const int*)slots, (TO*)cq, (TO*)kc, (TO*)vc, ps, interleaved)
  if (proj_dtype == 0 && out_dtype == 0) LD_LAUNCH(float, float);
  else if (proj_dtype == 0 && out_dtype == 1) LD_LAUNCH(float, bf16_t);
  else if (proj_dtype == 1 && out_dtype == 1) LD_LAUNCH(bf16_t, bf16_t);
  else return QVL_ERR_DTYPE;
#undef LD_LAUNCH
  return qvl_launch_status();
}

// q [N, heads * (dim + rot_dim)] of q_dtype, rows q_stride apart; out [N, heads, kv_rank + rot_dim] of out_dtype:
// only columns [kv_rank, kv_rank + rot_dim) of every head are written.
extern "C" int qvl_latent_query(const void* q, long long q_stride, int q_dtype, int heads, int dim, int rot_dim,
                                int kv_rank, const void* cs, int half, void* out, int out_dtype, int N,
                                int interleaved, hipStream_t stream) {
  if (N <= 0 || rot_dim == 0) return QVL_OK;
  if (heads <= 0 || dim < 0 || rot_dim < 0 || kv_rank <= 0 || half < 0 || 2 * half > rot_dim || !q || !out ||
      (half > 0 && !cs))
    return QVL_ERR_SHAPE;
#define LQ_LAUNCH(TQ, TO)                                                                                            \
  hipLaunchKernelGGL((latent_query_kernel<TQ, TO>), dim3(N), dim3(256), 0, stream, (const TQ*)q, q_stride, heads, dim, \
                     rot_dim, kv_rank, (const float*)cs, half, (TO*)out, interleaved)
  if (q_dtype == 0 && out_dtype == 0) LQ_LAUNCH(float, float);
  else if (q_dtype == 0 && out_dtype == 1) LQ_LAUNCH(float, bf16_t);
  else if (q_dtype == 1 && out_dtype == 1) LQ_LAUNCH(bf16_t, bf16_t);
  else return QVL_ERR_DTYPE;
#undef LQ_LAUNCH
  return qvl_launch_status();
}
