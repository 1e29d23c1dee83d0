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
// between the two passes over it.
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
};

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
  extern __shared__ float sm[];  // [(nq + nkv) * d], then 32 for the sums
  const int t = blockIdx.x;
  const int wq = a.nq * a.d, wk = a.nkv * a.d;
  float* red = sm + wq + wk;
  const T* row = (const T*)a.qk + (size_t)t * a.row;
  float sq = 0.f, sk = 0.f;
  for (int i = threadIdx.x; i < wq + wk; i += THREADS) {
    const float v = to_f32<T>(row[i]) + (a.bias ? a.bias[i] : 0.f);
    sm[i] = v;
    if (i < wq) sq += v * v; else sk += v * v;
  }
  block_sum_pair(sq, sk, red);
  const float iq = 1.0f / sqrtf(sq / (float)wq + a.eps);
  const float ik = 1.0f / sqrtf(sk / (float)wk + a.eps);
  float temp = 1.0f;
  if (a.temp_every > 0) temp = 1.0f + a.temp_coef * logf((float)((a.positions[t] + 1) / a.temp_every + 1));
  T* qo = (T*)a.q_out + (size_t)t * wq;
  for (int i = threadIdx.x; i < wq; i += THREADS) qo[i] = from_f32<T>(sm[i] * iq * a.q_weight[i] * temp);
  if (!a.slots) return;
  const int slot = a.slots[t];
  const int page = slot / a.page_size, off = slot - page * a.page_size;
  T* kc = (T*)a.k_cache;
  T* vc = (T*)a.v_cache;
  for (int i = threadIdx.x; i < wk; i += THREADS) {
    const int h = i / a.d, e = i - h * a.d;
    const size_t head = (size_t)page * a.nkv + h;
    kc[(head * a.page_size + off) * a.d + e] = from_f32<T>(sm[wq + i] * ik * a.k_weight[i]);
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
  if (dtype == QRT_F32) {
    if (few) joint_norm_kernel<float, 1024><<<num_tokens, 1024, smem, stream>>>(a);
    else joint_norm_kernel<float, 256><<<num_tokens, 256, smem, stream>>>(a);
  } else if (dtype == QRT_BF16) {
    if (few) joint_norm_kernel<bf16_t, 1024><<<num_tokens, 1024, smem, stream>>>(a);
    else joint_norm_kernel<bf16_t, 256><<<num_tokens, 256, smem, stream>>>(a);
  } else return qrt_fail("qk_joint_norm_store: unknown dtype %d", dtype);
  QRT_LAUNCH_CHECK("qk_joint_norm_store");
  return 0;
}
