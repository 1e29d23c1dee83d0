// Routed mixture of SwiGLU experts: the router, and the experts' products for
// (token, chosen expert) pairs taken one by one.
//
// Router: logits z[e] = x . W_r[e] + b[e] in float32 (the router's matrix is held in float32
// in every mode), the `top` largest per token (ties: the lower index), softmax over those; or,
// with sigmoid scores, the `top` largest sigmoid(z), which weigh the experts as they are; or, with
// softmax scores over all experts (`sigmoid_scores` = 2), the `top` largest of those, likewise. With
// scores, a `correction` per expert may be added for the choice alone, the chosen scores may be
// divided by their sum (+ 1e-20, `renormalise`), and the weights are multiplied by `weight_scale`. Experts
// may form equal groups of neighbours of which only the `keep` best (by the sum of a group's two
// largest entries, or with `group_max` by its largest) stay in the choice.
// Experts: pair p = (token t, its j-th expert e) computes act[p] = silu(G_e x) * (U_e x) (or the
// clamped activation of common.h) with
// gate_up [E, 2I, H] (gate rows, then up rows), then out[t] = sum_j w[t, j] * D_e act[p] with
// down [E, H, I], float32 out. Every output element is one wave's sum over its row in a fixed
// order: it depends on neither the batch nor the other pairs. This form streams an expert's
// matrices once per pair and suits steps of few tokens (decoding).
#include "common.h"
#include <math.h>

// sum over lanes of x[c] * w[c], c < n: 16-byte loads of w where the row allows them
template <typename T>
__device__ __forceinline__ float lane_dot(const T* __restrict__ w, const float* __restrict__ xs, int n, int lane, bool wide) {
  constexpr int VEC = 16 / sizeof(T);
  typedef T vec_t __attribute__((ext_vector_type(VEC)));
  float acc = 0.f;
  if (wide) {
#pragma unroll 4
    for (int c = lane * VEC; c < n; c += 64 * VEC) {
      const vec_t v = *(const vec_t*)(w + c);
#pragma unroll
      for (int e = 0; e < VEC; ++e) acc = fmaf(xs[c + e], to_f32<T>(v[e]), acc);
    }
  } else {
    for (int c = lane; c < n; c += 64) acc = fmaf(xs[c], to_f32<T>(w[c]), acc);
  }
  return acc;
}

// An expert's activation: the gated ones of common.h, or, for experts without a gate, the square
// of relu of the one product (`u` unused).
#define QRT_ACT_RELU2 2
__device__ __forceinline__ float expert_act(float g, float u, int kind, float limit) {
  if (kind == QRT_ACT_RELU2) {
    g = fmaxf(g, 0.f);
    return g * g;
  }
  return gated_act(g, u, kind, limit);
}

// ------------------------------------------------------------------- router
#define MAX_EXPERTS 1024
// One block of 16 waves per token. A wave takes the experts wave, wave + 16, ...: its lanes read
// the token's row and the expert's row straight from memory, several 16-byte pieces in flight
// each, so that a router of 16 experts costs about two rounds of memory latency.
template <typename T>
__global__ __launch_bounds__(1024) void route_top_kernel(const T* __restrict__ x, const float* __restrict__ router,
                                                         const float* __restrict__ bias, int* __restrict__ index,
                                                         float* __restrict__ weight, int hidden, int experts, int top,
                                                         int sigmoid_scores, int groups, int keep, int group_max,
                                                         const float* __restrict__ correction, int renormalise,
                                                         float weight_scale) {
  __shared__ float logit[MAX_EXPERTS];
  __shared__ float score[MAX_EXPERTS];
  const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const T* xr = x + (size_t)t * hidden;
  const bool wide = hidden % 4 == 0;
  for (int e = wave; e < experts; e += 16) {
    const float* wr = router + (size_t)e * hidden;
    float acc = 0.f;
    if (wide) {
      typedef T xvec_t __attribute__((ext_vector_type(4)));
#pragma unroll 8
      for (int c = lane * 4; c < hidden; c += 256) {
        const f32x4_t wv = *(const f32x4_t*)(wr + c);
        const xvec_t xv = *(const xvec_t*)(xr + c);
#pragma unroll
        for (int k = 0; k < 4; ++k) acc = fmaf(to_f32<T>(xv[k]), wv[k], acc);
      }
    } else {
      for (int c = lane; c < hidden; c += 64) acc = fmaf(to_f32<T>(xr[c]), wr[c], acc);
    }
    const float z = wave_sum(acc);
    if (lane == 0) logit[e] = z + (bias ? bias[e] : 0.f);
  }
  __syncthreads();
  if (wave != 0) return;
  if (sigmoid_scores == 1) {
    // scores sigmoid(z) take the logits' place: the choice goes by them, and they are the weights
    for (int e = lane; e < experts; e += 64) score[e] = logit[e] = 1.0f / (1.0f + expf(-logit[e]));
    __builtin_amdgcn_wave_barrier();
  } else if (sigmoid_scores == 2) {
    // the softmax over all experts likewise; maximum and sum in the same order in every lane
    float mx = -INFINITY, sum = 0.f;
    for (int e = 0; e < experts; ++e) mx = fmaxf(mx, logit[e]);
    for (int e = 0; e < experts; ++e) sum += expf(logit[e] - mx);
    __builtin_amdgcn_wave_barrier();
    for (int e = lane; e < experts; e += 64) score[e] = logit[e] = expf(logit[e] - mx) / sum;
    __builtin_amdgcn_wave_barrier();
  }
  if (correction) {
    // the choice goes by score + correction; the weights stay the scores
    for (int e = lane; e < experts; e += 64) logit[e] += correction[e];
    __builtin_amdgcn_wave_barrier();
  }
  if (groups > 1 && keep < groups) {
    // experts form `groups` equal groups of neighbours; a group's score is the sum of its two
    // largest entries (of its one, if it has one); only the `keep` best groups stay in the choice
    const int per = experts / groups;
    float mine = -INFINITY;  // lane g holds group g's score (groups <= 64)
    if (lane < groups) {
      float a = -INFINITY, b = -INFINITY;
      for (int e = lane * per; e < (lane + 1) * per; ++e) {
        const float z = logit[e];
        if (z > a) { b = a; a = z; } else if (z > b) b = z;
      }
      mine = (per > 1 && !group_max) ? a + b : a;
    }
    bool kept = false;
    for (int j = 0; j < keep; ++j) {
      float best = kept ? -INFINITY : mine;
      int at = (kept || lane >= groups) ? 0x7fffffff : lane;
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) {
        const float ob = __shfl_xor(best, o, 64);
        const int oa = __shfl_xor(at, o, 64);
        if (ob > best || (ob == best && oa < at)) { best = ob; at = oa; }
      }
      if (lane == at) kept = true;
    }
    const unsigned long long mask = __ballot(kept);
    for (int e = lane; e < experts; e += 64)
      if (!((mask >> (e / per)) & 1ull)) logit[e] = -INFINITY;
    __builtin_amdgcn_wave_barrier();
  }
  // `top` rounds of "largest that is left", ties to the lower index
  float chosen = 0.f, first = 0.f, denom = 0.f;
  for (int j = 0; j < top; ++j) {
    float best = -INFINITY;
    int at = 0x7fffffff;
    for (int e = lane; e < experts; e += 64) {
      const float z = logit[e];
      if (z > best) { best = z; at = e; }  // ascending e: the first of equals stays
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ob = __shfl_xor(best, o, 64);
      const int oa = __shfl_xor(at, o, 64);
      if (ob > best || (ob == best && oa < at)) { best = ob; at = oa; }
    }
    at = min(at, experts - 1);  // logits that are not numbers compare false throughout: still an expert
    if (j == 0) first = best;
    const float p = sigmoid_scores ? score[at] : expf(best - first);
    denom += p;
    if (lane == j) chosen = p;
    if (lane == 0) {
      index[(size_t)t * top + j] = at;
      logit[at] = -INFINITY;
    }
    __builtin_amdgcn_wave_barrier();
  }
  if (lane < top) {
    float w = sigmoid_scores ? chosen : chosen / denom;
    if (renormalise) w = w / (denom + 1e-20f);  // denom: the chosen scores' sum, in the order of the choice
    weight[(size_t)t * top + lane] = w * weight_scale;
  }
}

extern "C" int qrt_route_top(const void* x, int x_dtype, const float* router, const float* bias, int* index,
                             float* weight, int num_tokens, int hidden, int experts, int top, int sigmoid_scores,
                             int groups, int keep, int group_max, const float* correction, int renormalise,
                             float weight_scale, hipStream_t stream) {
  QRT_CHECK(groups >= 1 && groups <= 64 && experts % groups == 0 && keep >= 1 && keep <= groups &&
            (long)keep * (experts / groups) >= top,
            "route_top: %d groups of which %d stay do not fit %d experts of which %d are chosen", groups, keep, experts, top);
  QRT_CHECK(num_tokens >= 0 && hidden > 0, "route_top: bad sizes T=%d H=%d", num_tokens, hidden);
  QRT_CHECK(sigmoid_scores != 0 || (!correction && !renormalise),
            "route_top: a correction of the choice and renormalised weights go with scores over all experts");
  QRT_CHECK(experts >= 1 && experts <= MAX_EXPERTS && top >= 1 && top <= experts && top <= 64,
            "route_top: %d of %d experts (at most %d experts, 64 chosen)", top, experts, MAX_EXPERTS);
  if (num_tokens == 0) return 0;
  dim3 grid(num_tokens), block(1024);
  if (x_dtype == QRT_F32)
    route_top_kernel<float><<<grid, block, 0, stream>>>((const float*)x, router, bias, index, weight, hidden, experts, top, sigmoid_scores, groups, keep, group_max, correction, renormalise, weight_scale);
  else if (x_dtype == QRT_BF16)
    route_top_kernel<bf16_t><<<grid, block, 0, stream>>>((const bf16_t*)x, router, bias, index, weight, hidden, experts, top, sigmoid_scores, groups, keep, group_max, correction, renormalise, weight_scale);
  else return qrt_fail("route_top: unknown dtype %d", x_dtype);
  QRT_LAUNCH_CHECK("route_top");
  return 0;
}

// ------------------------------------------- experts, pair by pair (few tokens)
#define ROWS_PER_WAVE 4
template <typename T>
__global__ __launch_bounds__(256) void moe_gate_up_kernel(const T* __restrict__ x, const T* __restrict__ gate_up,
                                                          const int* __restrict__ index, T* __restrict__ act,
                                                          int hidden, int inter, int top, int act_kind, float limit) {
  extern __shared__ float xs[];  // [hidden]
  const int p = blockIdx.x, t = p / top;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int e = index[p];
  for (int c = threadIdx.x; c < hidden; c += 256) xs[c] = to_f32<T>(x[(size_t)t * hidden + c]);
  __syncthreads();
  const bool wide = hidden % (16 / sizeof(T)) == 0;
  const bool gated = act_kind != QRT_ACT_RELU2;  // without a gate an expert's rows are the up rows alone
  const T* w = gate_up + (size_t)e * (gated ? 2 : 1) * inter * hidden;
  const int i0 = (blockIdx.y * 4 + wave) * ROWS_PER_WAVE;
#pragma unroll
  for (int r = 0; r < ROWS_PER_WAVE; ++r) {
    const int i = i0 + r;
    if (i >= inter) break;
    const float g = wave_sum(lane_dot<T>(w + (size_t)i * hidden, xs, hidden, lane, wide));
    const float u = gated ? wave_sum(lane_dot<T>(w + (size_t)(inter + i) * hidden, xs, hidden, lane, wide)) : 0.f;
    if (lane == 0) act[(size_t)p * inter + i] = from_f32<T>(expert_act(g, u, act_kind, limit));
  }
}

template <typename T>
__global__ __launch_bounds__(256) void moe_down_kernel(const T* __restrict__ act, const T* __restrict__ down,
                                                       const int* __restrict__ index, const float* __restrict__ weight,
                                                       float* __restrict__ out, int hidden, int inter, int top) {
  extern __shared__ float as[];  // [top, inter]
  const int t = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int c = threadIdx.x; c < top * inter; c += 256) as[c] = to_f32<T>(act[(size_t)t * top * inter + c]);
  __syncthreads();
  const bool wide = inter % (16 / sizeof(T)) == 0;
  const int n0 = (blockIdx.y * 4 + wave) * ROWS_PER_WAVE;
#pragma unroll
  for (int r = 0; r < ROWS_PER_WAVE; ++r) {
    const int n = n0 + r;
    if (n >= hidden) break;
    float sum = 0.f;
    for (int j = 0; j < top; ++j) {
      const int e = index[(size_t)t * top + j];
      const float d = wave_sum(lane_dot<T>(down + ((size_t)e * hidden + n) * inter, as + (size_t)j * inter, inter, lane, wide));
      sum = fmaf(weight[(size_t)t * top + j], d, sum);
    }
    if (lane == 0) out[(size_t)t * hidden + n] = sum;
  }
}

extern "C" int qrt_moe_pairs(const void* x, const void* gate_up, const void* down, const int* index,
                             const float* weight, void* act, float* out, int dtype, int num_tokens, int hidden,
                             int inter, int experts, int top, int act_kind, float limit, hipStream_t stream) {
  QRT_CHECK(num_tokens >= 0 && hidden > 0 && inter > 0 && experts > 0 && top > 0, "moe: bad sizes");
  QRT_CHECK(act_kind == QRT_ACT_SWIGLU || act_kind == QRT_ACT_CLAMPED || act_kind == QRT_ACT_RELU2, "moe: unknown activation %d", act_kind);
  QRT_CHECK((size_t)hidden * 4 <= 64 * 1024 && (size_t)top * inter * 4 <= 64 * 1024,
            "moe: a token's row (%d) or its experts' inner rows (%d x %d) do not fit", hidden, top, inter);
  QRT_CHECK(dtype == QRT_F32 || dtype == QRT_BF16, "moe: unknown dtype %d", dtype);
  if (num_tokens == 0) return 0;
  const int per_block = 4 * ROWS_PER_WAVE;
  dim3 g1(num_tokens * top, (inter + per_block - 1) / per_block), g2(num_tokens, (hidden + per_block - 1) / per_block);
  QRT_CHECK(g1.y <= 65535 && g2.y <= 65535, "moe: rows too wide for one launch");
  if (dtype == QRT_F32) {
    moe_gate_up_kernel<float><<<g1, 256, hidden * 4, stream>>>((const float*)x, (const float*)gate_up, index, (float*)act, hidden, inter, top, act_kind, limit);
    moe_down_kernel<float><<<g2, 256, top * inter * 4, stream>>>((const float*)act, (const float*)down, index, weight, out, hidden, inter, top);
  } else {
    moe_gate_up_kernel<bf16_t><<<g1, 256, hidden * 4, stream>>>((const bf16_t*)x, (const bf16_t*)gate_up, index, (bf16_t*)act, hidden, inter, top, act_kind, limit);
    moe_down_kernel<bf16_t><<<g2, 256, top * inter * 4, stream>>>((const bf16_t*)act, (const bf16_t*)down, index, weight, out, hidden, inter, top);
  }
  QRT_LAUNCH_CHECK("moe_pairs");
  return 0;
}

// --------------------------------- experts, expert by expert (many tokens)
// With many tokens each expert multiplies a matrix of its own tokens once: the pairs are put in
// the order of their experts (group), the tokens' rows gathered in that order, the experts'
// products run on their stretches of rows (the host's loop over the engine's own matrix
// products, or one batched library product over stretches padded to equal length), and the
// results weighted and summed per token (combine), pair by pair in the order of the router's
// choice, without atomics on the output.
//
// group: order[i] = the pair at place i, place[p] = the place of pair p, offsets[e] = the first
// place of expert e (offsets[E] = P). One block. Which of an expert's pairs gets which of its
// places is left to the order in which the atomics arrive; no result depends on it, since
// every row is computed by itself.
__global__ __launch_bounds__(1024) void moe_group_kernel(const int* __restrict__ index, int* __restrict__ order,
                                                         int* __restrict__ place, int* __restrict__ offsets,
                                                         int pairs, int experts) {
  __shared__ int count[MAX_EXPERTS + 1];
  for (int e = threadIdx.x; e <= experts; e += blockDim.x) count[e] = 0;
  __syncthreads();
  for (int p = threadIdx.x; p < pairs; p += blockDim.x) atomicAdd(&count[index[p]], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int at = 0;
    for (int e = 0; e < experts; ++e) {
      const int n = count[e];
      count[e] = at;
      offsets[e] = at;
      at += n;
    }
    offsets[experts] = at;
  }
  __syncthreads();
  for (int p = threadIdx.x; p < pairs; p += blockDim.x) {
    const int at = atomicAdd(&count[index[p]], 1);
    order[at] = p;
    place[p] = at;
  }
}

// The row of place `at` among the experts' rows: the place itself, or, where every expert has a
// stretch of `padded` rows of its own (one batched product over all experts), the expert's
// stretch plus the place within the expert.
__device__ __forceinline__ size_t moe_row(int at, int expert, const int* __restrict__ offsets, int padded) {
  return padded > 0 ? (size_t)expert * padded + (at - offsets[expert]) : (size_t)at;
}

template <typename T>
__global__ void moe_gather_kernel(const T* __restrict__ x, const int* __restrict__ order, const int* __restrict__ index,
                                  const int* __restrict__ offsets, int padded, T* __restrict__ xs, int hidden, int top) {
  const int p = order[blockIdx.x];
  const T* src = x + (size_t)(p / top) * hidden;
  T* dst = xs + moe_row(blockIdx.x, index[p], offsets, padded) * hidden;
  for (int c = threadIdx.x; c < hidden; c += blockDim.x) dst[c] = src[c];
}

template <typename T>
__global__ void moe_combine_kernel(const T* __restrict__ y, const int* __restrict__ place, const int* __restrict__ index,
                                   const int* __restrict__ offsets, int padded, const float* __restrict__ weight,
                                   float* __restrict__ out, int hidden, int top) {
  const int t = blockIdx.x;
  for (int c = threadIdx.x; c < hidden; c += blockDim.x) {
    float sum = 0.f;
    for (int j = 0; j < top; ++j) {
      const size_t p = (size_t)t * top + j;
      sum = fmaf(weight[p], to_f32<T>(y[moe_row(place[p], index[p], offsets, padded) * hidden + c]), sum);
    }
    out[(size_t)t * hidden + c] = sum;
  }
}

extern "C" int qrt_moe_group(const int* index, int* order, int* place, int* offsets, int pairs, int experts,
                             hipStream_t stream) {
  QRT_CHECK(pairs > 0 && experts >= 1 && experts <= MAX_EXPERTS, "moe_group: bad sizes");
  moe_group_kernel<<<1, 1024, 0, stream>>>(index, order, place, offsets, pairs, experts);
  QRT_LAUNCH_CHECK("moe_group");
  return 0;
}

extern "C" int qrt_moe_gather(const void* x, const int* order, const int* index, const int* offsets, int padded,
                              void* xs, int dtype, int pairs, int hidden, int top, hipStream_t stream) {
  QRT_CHECK(pairs > 0 && hidden > 0 && top > 0 && padded >= 0, "moe_gather: bad sizes");
  if (dtype == QRT_F32) moe_gather_kernel<float><<<pairs, 256, 0, stream>>>((const float*)x, order, index, offsets, padded, (float*)xs, hidden, top);
  else if (dtype == QRT_BF16) moe_gather_kernel<bf16_t><<<pairs, 256, 0, stream>>>((const bf16_t*)x, order, index, offsets, padded, (bf16_t*)xs, hidden, top);
  else return qrt_fail("moe_gather: unknown dtype %d", dtype);
  QRT_LAUNCH_CHECK("moe_gather");
  return 0;
}

extern "C" int qrt_moe_combine(const void* y, const int* place, const int* index, const int* offsets, int padded,
                               const float* weight, float* out, int dtype, int num_tokens, int hidden, int top,
                               hipStream_t stream) {
  QRT_CHECK(num_tokens > 0 && hidden > 0 && top > 0 && padded >= 0, "moe_combine: bad sizes");
  if (dtype == QRT_F32) moe_combine_kernel<float><<<num_tokens, 256, 0, stream>>>((const float*)y, place, index, offsets, padded, weight, out, hidden, top);
  else if (dtype == QRT_BF16) moe_combine_kernel<bf16_t><<<num_tokens, 256, 0, stream>>>((const bf16_t*)y, place, index, offsets, padded, weight, out, hidden, top);
  else return qrt_fail("moe_combine: unknown dtype %d", dtype);
  QRT_LAUNCH_CHECK("moe_combine");
  return 0;
}

// ------------------- experts, expert by expert, without the host (decoding in batches)
// Once several tokens share an expert, the pair-by-pair form reads that expert's matrices once
// per token. Here the pairs are grouped by expert on the device (moe_group above) and a block
// owns a few rows of one expert's matrix: it brings them into LDS once and multiplies them
// with every token of that expert, a token per wave at a time, the token's row read from
// memory in 16-byte pieces. Blocks of experts that nobody chose leave at once. No count ever
// reaches the host, so the form can be captured into a graph. MODE 1 (gated): the rows are R gate
// rows and the R up rows that go with them, the input is the tokens' matrix and the output
// silu(gate) * up by pair; MODE 2: R up rows of experts without a gate, the output their
// activation by pair; MODE 0: R rows of the down matrix, the input by pair and the
// output by place (moe_combine weighs and sums it). Every output element is one wave's sum in a
// fixed order.
template <typename T, int R, int MODE>
__global__ __launch_bounds__(256) void moe_rows_by_expert_kernel(const T* __restrict__ in, const T* __restrict__ w,
                                                                 const int* __restrict__ order,
                                                                 const int* __restrict__ offsets, T* __restrict__ out,
                                                                 int K, int N, int top, int act_kind, float limit) {
  constexpr int VEC = 16 / sizeof(T);
  constexpr bool GATED = MODE == 1;
  constexpr bool FIRST = MODE != 0;  // the experts' first product: input by token, output by pair
  constexpr int NR = GATED ? 2 * R : R;
  typedef T vec_t __attribute__((ext_vector_type(VEC)));
  extern __shared__ __align__(16) unsigned char smem_raw[];
  T* rows = (T*)smem_raw;  // [NR, K]
  const int e = blockIdx.x, n0 = blockIdx.y * R;
  const int first = offsets[e], count = offsets[e + 1] - first;
  if (count == 0) return;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const T* we = w + (size_t)e * (GATED ? 2 : 1) * N * K;
  // all NR rows' pieces of a column range are asked for before the first is stored: NR loads in
  // flight a thread, and a row of 2,560 elements is through in two such rounds
  for (int c = threadIdx.x * VEC; c < K; c += 256 * VEC) {
    vec_t piece[NR];
#pragma unroll
    for (int r = 0; r < NR; ++r) {
      const int n = min(n0 + (r % R), N - 1) + (GATED && r >= R ? N : 0);  // beyond the matrix: its last row, dropped below
      piece[r] = *(const vec_t*)(we + (size_t)n * K + c);
    }
#pragma unroll
    for (int r = 0; r < NR; ++r) *(vec_t*)(rows + (size_t)r * K + c) = piece[r];
  }
  __syncthreads();
  for (int i = wave; i < count; i += 4) {
    const int p = order[first + i];
    const T* xr = in + (size_t)(FIRST ? p / top : p) * K;
    float acc[NR];
#pragma unroll
    for (int r = 0; r < NR; ++r) acc[r] = 0.f;
#pragma unroll 2
    for (int c = lane * VEC; c < K; c += 64 * VEC) {
      const vec_t xv = *(const vec_t*)(xr + c);
      float xf[VEC];
#pragma unroll
      for (int k = 0; k < VEC; ++k) xf[k] = to_f32<T>(xv[k]);
#pragma unroll
      for (int r = 0; r < NR; ++r) {
        const vec_t wv = *(const vec_t*)(rows + (size_t)r * K + c);
#pragma unroll
        for (int k = 0; k < VEC; ++k) acc[r] = fmaf(xf[k], to_f32<T>(wv[k]), acc[r]);
      }
    }
#pragma unroll
    for (int r = 0; r < NR; ++r) acc[r] = wave_sum(acc[r]);
    if (lane == 0) {
#pragma unroll
      for (int r = 0; r < R; ++r) {
        if (n0 + r >= N) break;
        if (FIRST) out[(size_t)p * N + n0 + r] = from_f32<T>(expert_act(acc[r], GATED ? acc[NR - R + r] : 0.f, act_kind, limit));
        else out[(size_t)(first + i) * N + n0 + r] = from_f32<T>(acc[r]);
      }
    }
  }
}

template <typename T, int R, int MODE>
static void moe_rows_launch(const void* in, const void* w, const int* order, const int* offsets, void* out, int K, int N,
                            int experts, int top, int act_kind, float limit, hipStream_t stream) {
  dim3 grid(experts, (N + R - 1) / R);
  const size_t smem = (size_t)(MODE == 1 ? 2 * R : R) * K * sizeof(T);
  moe_rows_by_expert_kernel<T, R, MODE><<<grid, 256, smem, stream>>>((const T*)in, (const T*)w, order, offsets, (T*)out, K, N, top, act_kind, limit);
}

template <typename T, int MODE>
static int moe_rows_pick(const void* in, const void* w, const int* order, const int* offsets, void* out, int K, int N,
                         int experts, int top, int act_kind, float limit, hipStream_t stream) {
  // as many rows a block as 48 KB of LDS hold, eight at most
  const size_t row_bytes = (size_t)(MODE == 1 ? 2 : 1) * K * sizeof(T);
  const int fit = (int)(48 * 1024 / row_bytes);
  if (fit >= 8) moe_rows_launch<T, 8, MODE>(in, w, order, offsets, out, K, N, experts, top, act_kind, limit, stream);
  else if (fit >= 4) moe_rows_launch<T, 4, MODE>(in, w, order, offsets, out, K, N, experts, top, act_kind, limit, stream);
  else if (fit >= 2) moe_rows_launch<T, 2, MODE>(in, w, order, offsets, out, K, N, experts, top, act_kind, limit, stream);
  else if (fit >= 1) moe_rows_launch<T, 1, MODE>(in, w, order, offsets, out, K, N, experts, top, act_kind, limit, stream);
  else return qrt_fail("moe: rows of %d elements do not fit the block's memory", K);
  return 0;
}

// x [T, H] -> act [pairs, I] (by pair) -> y [pairs, H] (by place); order and offsets from qrt_moe_group
extern "C" int qrt_moe_by_expert(const void* x, const void* gate_up, const void* down, const int* order,
                                 const int* offsets, void* act, void* y, int dtype, int hidden, int inter, int experts,
                                 int top, int act_kind, float limit, hipStream_t stream) {
  QRT_CHECK(hidden > 0 && inter > 0 && experts >= 1 && experts <= MAX_EXPERTS && top > 0, "moe: bad sizes");
  QRT_CHECK(act_kind == QRT_ACT_SWIGLU || act_kind == QRT_ACT_CLAMPED || act_kind == QRT_ACT_RELU2, "moe: unknown activation %d", act_kind);
  QRT_CHECK(dtype == QRT_F32 || dtype == QRT_BF16, "moe: unknown dtype %d", dtype);
  const int vec = dtype == QRT_F32 ? 4 : 8;
  QRT_CHECK(hidden % vec == 0 && inter % vec == 0, "moe: widths %d and %d are no multiples of %d", hidden, inter, vec);
  QRT_CHECK((inter + 0) / 1 <= 65535 * 8 && hidden <= 65535 * 8, "moe: rows too many for one launch");
  int rc;
  if (dtype == QRT_F32) {
    rc = act_kind == QRT_ACT_RELU2
             ? moe_rows_pick<float, 2>(x, gate_up, order, offsets, act, hidden, inter, experts, top, act_kind, limit, stream)
             : moe_rows_pick<float, 1>(x, gate_up, order, offsets, act, hidden, inter, experts, top, act_kind, limit, stream);
    if (rc == 0) rc = moe_rows_pick<float, 0>(act, down, order, offsets, y, inter, hidden, experts, top, act_kind, limit, stream);
  } else {
    rc = act_kind == QRT_ACT_RELU2
             ? moe_rows_pick<bf16_t, 2>(x, gate_up, order, offsets, act, hidden, inter, experts, top, act_kind, limit, stream)
             : moe_rows_pick<bf16_t, 1>(x, gate_up, order, offsets, act, hidden, inter, experts, top, act_kind, limit, stream);
    if (rc == 0) rc = moe_rows_pick<bf16_t, 0>(act, down, order, offsets, y, inter, hidden, experts, top, act_kind, limit, stream);
  }
  if (rc != 0) return rc;
  QRT_LAUNCH_CHECK("moe_by_expert");
  return 0;
}

// ------------------------------------------------ sigmoid gate on a matrix
// out[t, c] *= sigmoid(gate[t, c]), gate rows `gate_stride` elements apart
template <typename T>
__global__ void sigmoid_gate_kernel(T* __restrict__ out, const T* __restrict__ gate, long gate_stride, int width) {
  const int t = blockIdx.x;
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    const float g = to_f32<T>(gate[(size_t)t * gate_stride + c]);
    out[(size_t)t * width + c] = from_f32<T>(to_f32<T>(out[(size_t)t * width + c]) / (1.0f + expf(-g)));
  }
}

extern "C" int qrt_sigmoid_gate(void* out, const void* gate, long gate_stride, int dtype, int num_tokens, int width,
                                hipStream_t stream) {
  QRT_CHECK(num_tokens >= 0 && width > 0 && gate_stride >= width, "sigmoid_gate: bad sizes");
  if (num_tokens == 0) return 0;
  if (dtype == QRT_F32) sigmoid_gate_kernel<float><<<num_tokens, 256, 0, stream>>>((float*)out, (const float*)gate, gate_stride, width);
  else if (dtype == QRT_BF16) sigmoid_gate_kernel<bf16_t><<<num_tokens, 256, 0, stream>>>((bf16_t*)out, (const bf16_t*)gate, gate_stride, width);
  else return qrt_fail("sigmoid_gate: unknown dtype %d", dtype);
  QRT_LAUNCH_CHECK("sigmoid_gate");
  return 0;
}
