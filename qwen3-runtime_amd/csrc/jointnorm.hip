// Queries and keys normed over their whole projection, on their way into attention.
//
// From the columns q | k (| v) of one product, per token: biases are added (float32); the
// token's value of key head h is that head's key as it then is (`values_are_keys`), or the v
// columns; all nq * d query elements are divided by their one root mean square (eps inside
// the root) and multiplied by a weight vector of that whole size, and likewise the nkv * d key
// elements; the queries are then multiplied by the temperature of the token's position p,
// 1 + coef * ln(floor((p + 1) / every) + 1). Queries go to q_out [T, nq * d], keys and values
// into the paged cache (keys [page, head, offset, d], values [page, head, d, offset]). Sums,
// norms and the temperature are float32. One block per token; the biased row waits in LDS
// between the two passes over it. In steps of many tokens the values are stored by blocks of
// their own, one per (eight tokens in a row, key head): where the eight have neighbouring places
// in one page, a value element's eight tokens leave as one 16-byte piece of the transposed
// page (two pieces in float32) instead of eight 2-byte stores 2 * page_size bytes apart.
#include "common.h"
#include <math.h>

struct JointNormArgs {
  const void* qk; long row;            // [T, row]: q at column 0, k at nq * d, v behind it
  const float* bias;                   // over the same columns, or null
  const float* q_weight; const float* k_weight;
  const int* positions;
  void* q_out;
  const int* slots; void* k_cache; void* v_cache; int page_size;  // slots null: nothing is stored
  int nq, nkv, d;
  int values_are_keys;
  float eps, temp_coef; int temp_every;  // temp_every 0: no temperature
  int num_tokens;
  int group_values;  // the values are stored by the blocks behind the tokens' own, eight tokens each
  int wide;          // rows, projections and heads are whole 16-byte pieces: a piece a load and a store
};

// Block `b` of the value blocks: key head b % nkv of tokens 8 (b / nkv) .. + 7.
template <typename T>
__device__ __forceinline__ void store_values_of_group(const JointNormArgs& a, int b) {
  const int g = b / a.nkv, h = b - g * a.nkv;
  const int t0 = g * 8, nt = min(8, a.num_tokens - t0);
  const int wq = a.nq * a.d, wk = a.nkv * a.d;
  const int col0 = (a.values_are_keys ? wq : wq + wk) + h * a.d;
  int slot[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) slot[i] = a.slots[t0 + min(i, nt - 1)];
  bool together = nt == 8 && (slot[0] & 7) == 0 && (a.page_size & 7) == 0;
#pragma unroll
  for (int i = 1; i < 8; ++i) together = together && slot[i] == slot[0] + i;
  const T* qk = (const T*)a.qk;
  T* vc = (T*)a.v_cache;
  for (int e = threadIdx.x; e < a.d; e += blockDim.x) {
    __attribute__((aligned(16))) T vals[8];
    const float bias = a.bias ? a.bias[col0 + e] : 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i)
      vals[i] = from_f32<T>(to_f32<T>(qk[(size_t)(t0 + min(i, nt - 1)) * a.row + col0 + e]) + bias);
    if (together) {
      const int page = slot[0] / a.page_size, off = slot[0] - page * a.page_size;
      T* dst = vc + (((size_t)page * a.nkv + h) * a.d + e) * a.page_size + off;
#pragma unroll
      for (int piece = 0; piece < (int)(sizeof(T) * 8 / 16); ++piece) ((u32x4_t*)dst)[piece] = ((const u32x4_t*)vals)[piece];
    } else {
      for (int i = 0; i < nt; ++i) {
        const int page = slot[i] / a.page_size, off = slot[i] - page * a.page_size;
        vc[(((size_t)page * a.nkv + h) * a.d + e) * a.page_size + off] = vals[i];
      }
    }
  }
}

// Two sums over a block of up to 1,024 threads at once; every thread gets both, added in the same order.
__device__ __forceinline__ void block_sum_pair(float& x, float& y, float* red) {
  x = wave_sum(x);
  y = wave_sum(y);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int nw = (blockDim.x + 63) >> 6;
  if (lane == 0) { red[wave] = x; red[16 + wave] = y; }
  __syncthreads();
  x = y = 0.f;
  for (int i = 0; i < nw; ++i) { x += red[i]; y += red[16 + i]; }
}

// THREADS a block: 1,024 for steps of few tokens (a token's row is then through in one or two
// rounds of loads), 256 for many.
template <typename T, int THREADS>
__global__ __launch_bounds__(THREADS) void joint_norm_kernel(JointNormArgs a) {
  extern __shared__ __align__(16) float sm[];  // [(nq + nkv) * d], then 32 for the sums
  if ((int)blockIdx.x >= a.num_tokens) {  // a value block: the whole block turns here, before any barrier
    store_values_of_group<T>(a, blockIdx.x - a.num_tokens);
    return;
  }
  const int t = blockIdx.x;
  const int wq = a.nq * a.d, wk = a.nkv * a.d;
  float* red = sm + wq + wk;
  const T* row = (const T*)a.qk + (size_t)t * a.row;
  constexpr int V = 16 / sizeof(T);  // elements of a 16-byte piece
  typedef T piece_t __attribute__((ext_vector_type(V)));
  // whole pieces: heads, projections and rows begin at multiples of a piece (the host checks the bases)
  const bool wide = a.wide;
  float sq = 0.f, sk = 0.f;
  if (wide) {
    for (int c = threadIdx.x * V; c < wq + wk; c += THREADS * V) {
      const piece_t x = *(const piece_t*)(row + c);
      float v[V];
#pragma unroll
      for (int j = 0; j < V; j += 4) {
        const f32x4_t b = a.bias ? *(const f32x4_t*)(a.bias + c + j) : f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int k = 0; k < 4; ++k) v[j + k] = to_f32<T>(x[j + k]) + b[k];
      }
      float ss = 0.f;
#pragma unroll
      for (int j = 0; j < V; ++j) ss += v[j] * v[j];
      if (c < wq) sq += ss; else sk += ss;
#pragma unroll
      for (int j = 0; j < V; j += 4) *(f32x4_t*)(sm + c + j) = f32x4_t{v[j], v[j + 1], v[j + 2], v[j + 3]};
    }
  } else {
    for (int i = threadIdx.x; i < wq + wk; i += THREADS) {
      const float v = to_f32<T>(row[i]) + (a.bias ? a.bias[i] : 0.f);
      sm[i] = v;
      if (i < wq) sq += v * v; else sk += v * v;
    }
  }
  block_sum_pair(sq, sk, red);
  const float iq = 1.0f / sqrtf(sq / (float)wq + a.eps);
  const float ik = 1.0f / sqrtf(sk / (float)wk + a.eps);
  float temp = 1.0f;
  if (a.temp_every > 0) temp = 1.0f + a.temp_coef * logf((float)((a.positions[t] + 1) / a.temp_every + 1));
  T* qo = (T*)a.q_out + (size_t)t * wq;
  if (wide) {
    for (int c = threadIdx.x * V; c < wq; c += THREADS * V) {
      piece_t out;
#pragma unroll
      for (int j = 0; j < V; j += 4) {
        const f32x4_t w = *(const f32x4_t*)(a.q_weight + c + j), x = *(const f32x4_t*)(sm + c + j);
#pragma unroll
        for (int k = 0; k < 4; ++k) out[j + k] = from_f32<T>(x[k] * iq * w[k] * temp);
      }
      *(piece_t*)(qo + c) = out;
    }
  } else {
    for (int i = threadIdx.x; i < wq; i += THREADS) qo[i] = from_f32<T>(sm[i] * iq * a.q_weight[i] * temp);
  }
  if (!a.slots) return;
  const int slot = a.slots[t];
  const int page = slot / a.page_size, off = slot - page * a.page_size;
  T* kc = (T*)a.k_cache;
  T* vc = (T*)a.v_cache;
  if (wide) {
    for (int c = threadIdx.x * V; c < wk; c += THREADS * V) {
      const int h = c / a.d, e = c - h * a.d;
      piece_t out;
#pragma unroll
      for (int j = 0; j < V; j += 4) {
        const f32x4_t w = *(const f32x4_t*)(a.k_weight + c + j), x = *(const f32x4_t*)(sm + wq + c + j);
#pragma unroll
        for (int k = 0; k < 4; ++k) out[j + k] = from_f32<T>(x[k] * ik * w[k]);
      }
      *(piece_t*)(kc + (((size_t)page * a.nkv + h) * a.page_size + off) * a.d + e) = out;
    }
  }
  for (int i = threadIdx.x; i < wk; i += THREADS) {
    const int h = i / a.d, e = i - h * a.d;
    const size_t head = (size_t)page * a.nkv + h;
    if (!wide) kc[(head * a.page_size + off) * a.d + e] = from_f32<T>(sm[wq + i] * ik * a.k_weight[i]);
    if (a.group_values) continue;
    const float v = a.values_are_keys ? sm[wq + i]
                                      : to_f32<T>(row[wq + wk + i]) + (a.bias ? a.bias[wq + wk + i] : 0.f);
    vc[(head * a.d + e) * a.page_size + off] = from_f32<T>(v);
  }
}

extern "C" int qrt_qk_joint_norm_store(const JointNormArgs* args, int dtype, int num_tokens, long num_pages,
                                       hipStream_t stream) {
  JointNormArgs a = *args;
  QRT_CHECK(num_tokens >= 0 && a.nq > 0 && a.nkv > 0 && a.d > 0, "qk_joint_norm_store: bad sizes");
  const long need = (long)(a.nq + (a.values_are_keys ? 1 : 2) * a.nkv) * a.d;
  QRT_CHECK(a.row >= need, "qk_joint_norm_store: rows of %ld for %ld columns", a.row, need);
  QRT_CHECK(a.q_weight && a.k_weight && a.q_out && a.qk, "qk_joint_norm_store: no weights or no output");
  QRT_CHECK(a.temp_every >= 0 && (a.temp_every == 0 || a.positions), "qk_joint_norm_store: a temperature without positions");
  QRT_CHECK(!a.slots || (a.k_cache && a.v_cache && a.page_size > 0 && num_pages > 0), "qk_joint_norm_store: no cache");
  const size_t smem = ((size_t)(a.nq + a.nkv) * a.d + 32) * sizeof(float);
  QRT_CHECK(smem <= 64 * 1024, "qk_joint_norm_store: a token's %d query and key elements do not fit the block's memory",
            (a.nq + a.nkv) * a.d);
  if (num_tokens == 0) return 0;
  const bool few = num_tokens <= 256;
  a.num_tokens = num_tokens;
  a.group_values = !few && a.slots;
  const int piece = dtype == QRT_F32 ? 4 : 8;
  a.wide = a.d % piece == 0 && a.row % piece == 0 && ((uintptr_t)a.qk & 15) == 0 && ((uintptr_t)a.q_out & 15) == 0 &&
           ((uintptr_t)a.k_cache & 15) == 0 && ((uintptr_t)a.bias & 15) == 0 && ((uintptr_t)a.q_weight & 15) == 0 &&
           ((uintptr_t)a.k_weight & 15) == 0;
  const int blocks = num_tokens + (a.group_values ? (num_tokens + 7) / 8 * a.nkv : 0);
  if (dtype == QRT_F32) {
    if (few) joint_norm_kernel<float, 1024><<<blocks, 1024, smem, stream>>>(a);
    else joint_norm_kernel<float, 256><<<blocks, 256, smem, stream>>>(a);
  } else if (dtype == QRT_BF16) {
    if (few) joint_norm_kernel<bf16_t, 1024><<<blocks, 1024, smem, stream>>>(a);
    else joint_norm_kernel<bf16_t, 256><<<blocks, 256, smem, stream>>>(a);
  } else return qrt_fail("qk_joint_norm_store: unknown dtype %d", dtype);
  QRT_LAUNCH_CHECK("qk_joint_norm_store");
  return 0;
}
