// Linear attention with a decayed outer-product state, one head at a time:
//   S_t = diag(a_t) S_(t-1) + k_t v_t^T,   o_t = S_t^T q_t
// S is [LA_DIM, vdim] float32 per (request slot, head).  The decay a_t is one constant per head, or
// one value per key channel and token: a_t = sigmoid(z_t)^(1/tau) from float32 z, or a forget gate with a
// floor, a_t = l + (1 - l) sigmoid(z_t + b) with l and b per key channel, whose complement is the key,
// k_t = 1 - a_t (no key is read then).  q, k and v are columns of the projection's rows (float32 or
// bfloat16), with an optional silu on each (`act`: bit 0 q, bit 1 k, bit 2 v) and a scale on q applied in
// float32 as they are read.  Compiled per key size (-DLA_DIM=...).
//
// The scan: a block of four waves owns 64 value channels of one head of one request and walks the
// request's tokens of this step in order, starting from the state its slot holds and leaving the
// new state there.  Lane = value channel; each wave keeps LA_DIM / 4 rows of S in registers (a key
// size that four does not divide is shared by two waves, or kept by one).
// Tokens are staged LA_TB at a time: q, k and the decays go to LDS (every lane reads the same
// word), the four partial sums of o meet in LDS.  The order of every sum is fixed by the sizes
// alone, so a token's result does not depend on how its sequence was cut into steps or on what
// else the batch holds.
//
// One prompt alone has only heads x vdim / 64 such blocks.  With G > 1 the key channels are cut
// into G groups, each with blocks of its own (four waves of LA_DIM / (4 G) rows); a group's sums of
// o go to its own slab of the output, [G, N, heads * vdim], and whoever reads the output adds the
// slabs in order (the norm that follows does).
#include "common.h"

#ifndef LA_DIM
#define LA_DIM 64
#endif
// waves of a block: four share the rows of S where the key size divides by four, else two or one
#define LA_WAVES (LA_DIM % 4 == 0 ? 4 : (LA_DIM % 2 == 0 ? 2 : 1))
#define LA_THREADS (64 * LA_WAVES)
#define LA_TB (LA_DIM > 256 ? 4 : (LA_DIM > 128 ? 8 : 16))


__device__ __forceinline__ float la_act(float z, int act) { return act ? z / (1.0f + expf(-z)) : z; }

// how the decay is given: a constant per head; sigmoid(z)^(1/tau); a floored forget gate whose complement is the key
#define LA_HEAD 0
#define LA_CHANNEL 1
#define LA_FORGET 2
// the complement of the floored forget gate, (1 - l) (1 - sigmoid(z)) = (1 - l) / (1 + exp(z)): this is the key,
// and the decay is 1 minus it
__device__ __forceinline__ float la_forget_key(float z, float lower) { return (1.0f - lower) / (1.0f + expf(z)); }

// log(sigmoid(z)) = min(z, 0) - log1p(exp(-|z|))
__device__ __forceinline__ float la_decay(float z, float inv_tau) {
  return expf((fminf(z, 0.f) - log1pf(expf(-fabsf(z)))) * inv_tau);
}

template <typename TP, int MODE, int G>
__global__ __launch_bounds__(LA_THREADS) void la_scan_kernel(
    const TP* __restrict__ proj, long long proj_stride, int q_off, int k_off, int v_off,
    const float* __restrict__ head_decay, const float* __restrict__ z, long long z_stride, float inv_tau,
    const float* __restrict__ lower, const float* __restrict__ zbias,
    float* __restrict__ state, const int* __restrict__ cu_q, const int* __restrict__ req_slots,
    float* __restrict__ out, long long out_slab, int H, int vdim, int act, float q_scale) {
  // key channels of this block's group (a G that does not divide the rows among the waves is never launched)
  constexpr int DG = LA_DIM % (LA_WAVES * G) == 0 ? LA_DIM / G : LA_DIM;
  constexpr int LA_ROWS = DG / LA_WAVES;    // rows of S a wave keeps
  __shared__ float qs[LA_TB][DG];
  __shared__ float ks[LA_TB][DG];
  constexpr bool CHANNEL_DECAY = MODE != LA_HEAD;
  __shared__ float as[CHANNEL_DECAY ? LA_TB : 1][DG];
  __shared__ float po[LA_TB][LA_WAVES][64];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int head = blockIdx.y, req = blockIdx.z;
  const int vtile = blockIdx.x / G, group = blockIdx.x % G;
  const int d0 = group * DG;
  const int vcol = vtile * 64 + lane;
  const bool live = vcol < vdim;
  const int begin = cu_q[req], end = cu_q[req + 1];
  if (begin >= end) return;
  out += (size_t)group * out_slab;
  float* srow = state + (((size_t)req_slots[req] * H + head) * LA_DIM + d0 + (size_t)wave * LA_ROWS) * vdim + vcol;
  float S[LA_ROWS];
#pragma unroll
  for (int i = 0; i < LA_ROWS; ++i) S[i] = live ? srow[(size_t)i * vdim] : 0.f;
  const float fixed = CHANNEL_DECAY ? 1.f : head_decay[head];

  for (int t0 = begin; t0 < end; t0 += LA_TB) {
    const int nt = end - t0 < LA_TB ? end - t0 : LA_TB;
    for (int idx = tid; idx < nt * DG; idx += LA_THREADS) {
      const int t = idx / DG, d = idx % DG;
      const TP* row = proj + (size_t)(t0 + t) * proj_stride + (size_t)head * LA_DIM + d0 + d;
      qs[t][d] = la_act(ldf<TP>(row + q_off), act & 1) * q_scale;
      if (MODE == LA_FORGET) {
        const int hd = head * LA_DIM + d0 + d;
        const float zz = z[(size_t)(t0 + t) * z_stride + hd] + (zbias ? zbias[hd] : 0.f);
        const float key = la_forget_key(zz, lower[hd]);
        ks[t][d] = key;
        as[t][d] = 1.0f - key;
      } else {
        ks[t][d] = la_act(ldf<TP>(row + k_off), act & 2);
        if (MODE == LA_CHANNEL)
          as[t][d] = la_decay(z[(size_t)(t0 + t) * z_stride + (size_t)head * LA_DIM + d0 + d], inv_tau);
      }
    }
    float vt[LA_TB];
#pragma unroll
    for (int t = 0; t < LA_TB; ++t)
      vt[t] = (live && t < nt)
                  ? la_act(ldf<TP>(proj + (size_t)(t0 + t) * proj_stride + v_off + (size_t)head * vdim + vcol), act & 4)
                  : 0.f;
    __syncthreads();
#pragma unroll
    for (int t = 0; t < LA_TB; ++t) {
      if (t < nt) {
        float acc = 0.f;
#pragma unroll
        for (int i = 0; i < LA_ROWS; ++i) {
          const int d = wave * LA_ROWS + i;
          const float a = CHANNEL_DECAY ? as[t][d] : fixed;
          S[i] = a * S[i] + ks[t][d] * vt[t];
          acc += S[i] * qs[t][d];
        }
        po[t][wave][lane] = acc;
      }
    }
    __syncthreads();
    for (int idx = tid; idx < nt * 64; idx += LA_THREADS) {
      const int t = idx >> 6, l = idx & 63;
      const int c = vtile * 64 + l;
      if (c < vdim) {
        float sum = po[t][0][l];
#pragma unroll
        for (int w = 1; w < LA_WAVES; ++w) sum += po[t][w][l];
        out[((size_t)(t0 + t) * H + head) * vdim + c] = sum;
      }
    }
    __syncthreads();
  }
  if (live) {
#pragma unroll
    for (int i = 0; i < LA_ROWS; ++i) srow[(size_t)i * vdim] = S[i];
  }
}

// ---------------------------------------------------------------------------------------
// Long runs, cut into chunks that are scanned side by side.  With P_t = a_c0 * ... * a_t (per key
// channel, from the chunk's first token c0 to t, t included) and S' the state before the chunk:
//   o_t = (scan from a zero state)_t + S'^T (q_t * P_t),      S_end = diag(P_last) S' + U
// where U is the state the scan from zero ends with.  The scan above runs every chunk as if it were a
// request (from zeroed rows of a scratch tensor); the kernels below form q_t * P_t and P_last, carry
// the state from chunk to chunk, and put the second term, a plain float32 matrix product per (chunk,
// head) done by the caller, back into token order.
// ---------------------------------------------------------------------------------------

// grid (chunks, H), LA_DIM * LA_PARTS threads: qp [chunks, H, chunk_len, LA_DIM] (rows past the chunk's end
// stay as they are), last [chunks, H, LA_DIM].  The chunk's tokens are cut into LA_PARTS ranges; a thread
// sums the logarithms of its channel's decays over its range, learns through LDS what the ranges before
// it add up to, and walks its range again to write q_t * P_t.
#define LA_PARTS (LA_DIM <= 64 ? 8 : (LA_DIM <= 128 ? 4 : (LA_DIM <= 256 ? 2 : 1)))

template <typename TP, int MODE>
__global__ void la_prefix_kernel(const TP* __restrict__ proj, long long proj_stride, int q_off,
                                 const float* __restrict__ head_decay, const float* __restrict__ z,
                                 long long z_stride, float inv_tau, const float* __restrict__ lower,
                                 const float* __restrict__ zbias, const int* __restrict__ chunk_cu,
                                 float* __restrict__ qp, float* __restrict__ last, int H, int chunk_len, int act,
                                 float q_scale) {
  __shared__ float part_sum[LA_PARTS][LA_DIM];
  const int c = blockIdx.x, head = blockIdx.y, d = threadIdx.x % LA_DIM, part = threadIdx.x / LA_DIM;
  const int begin = chunk_cu[c], end = chunk_cu[c + 1];
  const int per = (end - begin + LA_PARTS - 1) / LA_PARTS;
  const int lo = begin + part * per < end ? begin + part * per : end;
  const int hi = lo + per < end ? lo + per : end;
  const float fixed_log = MODE != LA_HEAD ? 0.f : logf(head_decay[head]);
  const float my_lower = MODE == LA_FORGET ? lower[head * LA_DIM + d] : 0.f;
  const float my_bias = (MODE == LA_FORGET && zbias) ? zbias[head * LA_DIM + d] : 0.f;
  auto log_decay = [&](int t) {
    if (MODE == LA_HEAD) return fixed_log;
    const float zz = z[(size_t)t * z_stride + (size_t)head * LA_DIM + d];
    if (MODE == LA_FORGET) return log1pf(-la_forget_key(zz + my_bias, my_lower));
    return (fminf(zz, 0.f) - log1pf(expf(-fabsf(zz)))) * inv_tau;
  };
  float mine = 0.f;
  for (int t = lo; t < hi; ++t) mine += log_decay(t);
  part_sum[part][d] = mine;
  __syncthreads();
  float acc = 0.f;     // log of the running product, from the chunk's first token on
  for (int p = 0; p < part; ++p) acc += part_sum[p][d];
  float* row = qp + ((size_t)c * H + head) * chunk_len * LA_DIM + d;
  for (int t = lo; t < hi; ++t) {
    acc += log_decay(t);
    const float q = la_act(ldf<TP>(proj + (size_t)t * proj_stride + q_off + (size_t)head * LA_DIM + d), act & 1) * q_scale;
    row[(size_t)(t - begin) * LA_DIM] = q * expf(acc);
  }
  if (part == LA_PARTS - 1) last[((size_t)c * H + head) * LA_DIM + d] = expf(acc);
}

// One thread per element of a head's state: for the request's chunks in order, scratch[c] (the chunk's
// U) is replaced by the state before the chunk, and the request's slot gets the state after its last.
__global__ void la_carry_kernel(float* __restrict__ scratch, const float* __restrict__ last, float* __restrict__ state,
                                const int* __restrict__ req_first, const int* __restrict__ req_slots, int H, int vdim) {
  const int req = blockIdx.y;
  const long long per_slot = (long long)H * LA_DIM * vdim;
  const long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= per_slot) return;
  const long long hd = e / vdim;      // head * LA_DIM + d
  float* mine = state + (size_t)req_slots[req] * per_slot + e;
  float S = *mine;
  for (int c = req_first[req]; c < req_first[req + 1]; ++c) {
    float* u = scratch + (size_t)c * per_slot + e;
    const float before = S;
    S = last[(size_t)c * H * LA_DIM + hd] * S + *u;
    *u = before;
  }
  *mine = S;
}

// corr [chunks, H, chunk_len, vdim] -> out [N, H * vdim]
__global__ void la_gather_kernel(const float* __restrict__ corr, const int* __restrict__ chunk_cu,
                                 float* __restrict__ out, int H, int chunk_len, int vdim) {
  const int c = blockIdx.x, head = blockIdx.y;
  const int begin = chunk_cu[c], n = chunk_cu[c + 1] - begin;
  const float* src = corr + ((size_t)c * H + head) * chunk_len * vdim;
  for (int i = threadIdx.x; i < n * vdim; i += blockDim.x) {
    const int t = i / vdim, v = i % vdim;
    out[((size_t)(begin + t) * H + head) * vdim + v] = src[i];
  }
}

extern "C" int qvl_la_prefix(const void* proj, long long proj_stride, int q_off, int proj_dtype, const void* head_decay,
                             const void* z, long long z_stride, float inv_tau, const void* lower, const void* zbias,
                             const void* chunk_cu, void* qp,
                             void* last, int chunks, int H, int dim, int chunk_len, int act, float q_scale,
                             hipStream_t stream) {
  if (chunks <= 0) return QVL_OK;
  if (dim != LA_DIM || H <= 0 || chunk_len <= 0 || (!head_decay && !z) || (lower && !z)) return QVL_ERR_SHAPE;
  if (H > 65535 || LA_DIM * LA_PARTS > 1024) return QVL_ERR_LIMIT;
#define LAUNCH(TP, MODE)                                                                                            \
  hipLaunchKernelGGL((la_prefix_kernel<TP, MODE>), dim3(chunks, H), dim3(LA_DIM * LA_PARTS), 0, stream, (const TP*)proj, \
                     proj_stride, q_off, (const float*)head_decay, (const float*)z, z_stride, inv_tau,               \
                     (const float*)lower, (const float*)zbias, (const int*)chunk_cu, (float*)qp, (float*)last, H,    \
                     chunk_len, act, q_scale)
#define BY_MODE(TP) { if (lower) LAUNCH(TP, LA_FORGET); else if (z) LAUNCH(TP, LA_CHANNEL); else LAUNCH(TP, LA_HEAD); }
  if (proj_dtype == 0) BY_MODE(float)
  else if (proj_dtype == 1) BY_MODE(bf16_t)
  else return QVL_ERR_DTYPE;
#undef BY_MODE
#undef LAUNCH
  return qvl_launch_status();
}

extern "C" int qvl_la_carry(void* scratch, const void* last, void* state, const void* req_first, const void* req_slots,
                            int R, int H, int dim, int vdim, hipStream_t stream) {
  if (R <= 0) return QVL_OK;
  if (dim != LA_DIM || H <= 0 || vdim <= 0) return QVL_ERR_SHAPE;
  if (R > 65535) return QVL_ERR_LIMIT;
  const long long per_slot = (long long)H * LA_DIM * vdim;
  hipLaunchKernelGGL(la_carry_kernel, dim3((unsigned)((per_slot + 255) / 256), R), dim3(256), 0, stream, (float*)scratch,
                     (const float*)last, (float*)state, (const int*)req_first, (const int*)req_slots, H, vdim);
  return qvl_launch_status();
}

extern "C" int qvl_la_gather(const void* corr, const void* chunk_cu, void* out, int chunks, int H, int chunk_len,
                             int vdim, hipStream_t stream) {
  if (chunks <= 0) return QVL_OK;
  if (H <= 0 || H > 65535 || chunk_len <= 0 || vdim <= 0) return QVL_ERR_SHAPE;
  hipLaunchKernelGGL(la_gather_kernel, dim3(chunks, H), dim3(256), 0, stream, (const float*)corr, (const int*)chunk_cu,
                     (float*)out, H, chunk_len, vdim);
  return qvl_launch_status();
}

extern "C" int qvl_la_key_size() { return LA_DIM; }

// proj: rows of `proj_stride` values holding q (H * LA_DIM columns from q_off), k (from k_off) and v
// (H * vdim columns from v_off).  head_decay [H] float32, or z float32 rows (H * LA_DIM columns) with
// inv_tau, or z with lower (and zbias, which may be null) float32 [H * LA_DIM]: the floored forget gate, whose
// complement is the key (k_off is not read).  state [slots, H, LA_DIM, vdim] float32; cu_q [R + 1], req_slots [R]; out float32
// [groups, N, H * vdim] (groups 1, 2, 4 or 8 with LA_DIM a multiple of 4 * groups), slabs `out_slab` apart.
extern "C" int qvl_la_scan(const void* proj, long long proj_stride, int q_off, int k_off, int v_off, int proj_dtype,
                           const void* head_decay, const void* z, long long z_stride, float inv_tau,
                           const void* lower, const void* zbias, void* state, const void* cu_q, const void* req_slots, void* out, long long out_slab, int groups, int R,
                           int H, int dim, int vdim, int act, float q_scale, hipStream_t stream) {
  if (R <= 0) return QVL_OK;
  if (dim != LA_DIM || H <= 0 || vdim <= 0 || (!head_decay && !z) || (lower && !z)) return QVL_ERR_SHAPE;
  if (groups != 1 && groups != 2 && groups != 4 && groups != 8) return QVL_ERR_SHAPE;
  if (LA_DIM % (LA_WAVES * groups)) return QVL_ERR_SHAPE;
  if (H > 65535 || R > 65535) return QVL_ERR_LIMIT;
  const dim3 grid(((vdim + 63) / 64) * groups, H, R);
#define LAUNCH(TP, CH, G)                                                                                           \
  hipLaunchKernelGGL((la_scan_kernel<TP, CH, G>), grid, dim3(LA_THREADS), 0, stream, (const TP*)proj, proj_stride, q_off,   \
                     k_off, v_off, (const float*)head_decay, (const float*)z, z_stride, inv_tau,                    \
                     (const float*)lower, (const float*)zbias, (float*)state, (const int*)cu_q, (const int*)req_slots, (float*)out, out_slab, H, vdim, act, q_scale)
#define BY_GROUPS(TP, CH)                                                                                           \
  switch (groups) {                                                                                                 \
    case 1: LAUNCH(TP, CH, 1); break;                                                                               \
    case 2: LAUNCH(TP, CH, 2); break;                                                                               \
    case 4: LAUNCH(TP, CH, 4); break;                                                                               \
    default: LAUNCH(TP, CH, 8); break;                                                                              \
  }
#define BY_MODE(TP)                                                                                                 \
  {                                                                                                                 \
    if (lower) { BY_GROUPS(TP, LA_FORGET) }                                                                         \
    else if (z) { BY_GROUPS(TP, LA_CHANNEL) }                                                                       \
    else { BY_GROUPS(TP, LA_HEAD) }                                                                                 \
  }
  if (proj_dtype == 0) BY_MODE(float)
  else if (proj_dtype == 1) BY_MODE(bf16_t)
  else return QVL_ERR_DTYPE;
#undef BY_MODE
#undef BY_GROUPS
#undef LAUNCH
  return qvl_launch_status();
}
