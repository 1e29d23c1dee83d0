// Steps of attention through a latent, each over packed tokens:
//
// * the RMS norm of some columns of a wider matrix (a latent that a fused product left beside
//   other things), float32 inside, out in the matrix's type;
// * the write of the cached row: columns [first, first + rank) RMS-normed are the latent c, the
//   rot_dim columns behind them, rotated, the key part all heads share; the key row of the one
//   key/value head is [c | k_rot], its value row [c | 0] (keys [page, 1, offset, W], values
//   [page, 1, W, offset], W = rank + rot_dim);
// * a copy of `width` elements per (token, head) from one strided layout to another with the
//   first 2 n of them turned, element i against element i + n (the "rotate half" layout), or,
//   with `neighbours`, element 2i against element 2i + 1, by position * freq[i] (angles, sines
//   and cosines float32; sines and cosines times `magnitude`); the cached row's rotated part
//   takes the same two options;
// * a product per head, out[t, h, :] = W[h] x[t, h, :], on strided rows: W [heads, N, K].
#include "common.h"
#include <math.h>

// Element i of a vector whose first 2 `pairs` elements turn: its partner and the pair's number.
// Half layout: i against i + pairs; neighbours: 2j against 2j + 1. `first` says whether i is the
// pair's first element (x cos - other sin) or its second (x cos + other sin).
__device__ __forceinline__ void rotation_partner(int i, int pairs, int neighbours, int* pair, int* other, bool* first) {
  if (neighbours) {
    *pair = i >> 1;
    *first = (i & 1) == 0;
    *other = i ^ 1;
  } else {
    *first = i < pairs;
    *pair = *first ? i : i - pairs;
    *other = *first ? i + pairs : i - pairs;
  }
}

// ---------------------------------------------------------------- norm of some columns
template <typename T>
__global__ __launch_bounds__(256) void rmsnorm_columns_kernel(const T* __restrict__ y, long stride, int first, int width,
                                                              const float* __restrict__ weight, float eps,
                                                              T* __restrict__ out) {
  __shared__ float red[32];
  const T* row = y + (size_t)blockIdx.x * stride + first;
  float ss = 0.f;
  for (int i = threadIdx.x; i < width; i += 256) {
    const float v = to_f32<T>(row[i]);
    ss += v * v;
  }
  ss = block_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)width + eps);
  for (int i = threadIdx.x; i < width; i += 256)
    out[(size_t)blockIdx.x * width + i] = from_f32<T>(to_f32<T>(row[i]) * inv * weight[i]);
}

extern "C" int qrt_rmsnorm_columns(const void* y, long stride, int first, int width, const float* weight, float eps,
                                   void* out, int dtype, int num_tokens, hipStream_t stream) {
  QRT_CHECK(num_tokens >= 0 && width > 0 && first >= 0 && (long)first + width <= stride, "rmsnorm_columns: bad sizes");
  if (num_tokens == 0) return 0;
  if (dtype == QRT_F32)
    rmsnorm_columns_kernel<float><<<num_tokens, 256, 0, stream>>>((const float*)y, stride, first, width, weight, eps, (float*)out);
  else if (dtype == QRT_BF16)
    rmsnorm_columns_kernel<bf16_t><<<num_tokens, 256, 0, stream>>>((const bf16_t*)y, stride, first, width, weight, eps, (bf16_t*)out);
  else return qrt_fail("rmsnorm_columns: unknown dtype %d", dtype);
  QRT_LAUNCH_CHECK("rmsnorm_columns");
  return 0;
}

// ---------------------------------------------------------------- the cached row
template <typename T>
__global__ __launch_bounds__(256) void latent_store_kernel(const T* __restrict__ y, long stride, int first, int rank,
                                                           int rot_dim, const float* __restrict__ weight, float eps,
                                                           const int* __restrict__ positions, const float* __restrict__ freq,
                                                           int pairs, const int* __restrict__ slots, T* __restrict__ k_cache,
                                                           T* __restrict__ v_cache, int page_size, int neighbours,
                                                           float magnitude) {
  __shared__ float red[32];
  const int t = blockIdx.x;
  const T* row = y + (size_t)t * stride + first;
  const int slot = slots[t];
  const int page = slot / page_size, off = slot - page * page_size;
  const int w = rank + rot_dim;
  T* kr = k_cache + (size_t)slot * w;
  T* vr = v_cache + (size_t)page * w * page_size + off;
  float ss = 0.f;
  for (int i = threadIdx.x; i < rank; i += 256) {
    const float v = to_f32<T>(row[i]);
    ss += v * v;
  }
  ss = block_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)rank + eps);
  for (int i = threadIdx.x; i < rank; i += 256) {
    const T c = from_f32<T>(to_f32<T>(row[i]) * inv * weight[i]);
    kr[i] = c;
    vr[(size_t)i * page_size] = c;
  }
  const float pos = (float)positions[t];
  const T* rot = row + rank;
  for (int i = threadIdx.x; i < rot_dim; i += 256) {
    float x = to_f32<T>(rot[i]);
    if (i < 2 * pairs) {
      int j, o;
      bool first;
      rotation_partner(i, pairs, neighbours, &j, &o, &first);
      float sn, cs;
      sincos_angle(pos * freq[j], &sn, &cs);
      sn *= magnitude;
      cs *= magnitude;
      const float other = to_f32<T>(rot[o]);
      x = first ? x * cs - other * sn : x * cs + other * sn;
    }
    kr[rank + i] = from_f32<T>(x);
    vr[(size_t)(rank + i) * page_size] = from_f32<T>(0.f);
  }
}

extern "C" int qrt_latent_store(const void* y, long stride, int first, int rank, int rot_dim, const float* weight, float eps,
                                const int* positions, const float* freq, int pairs, const int* slots, void* k_cache,
                                void* v_cache, int page_size, long num_pages, int dtype, int num_tokens, int neighbours,
                                float magnitude, hipStream_t stream) {
  QRT_CHECK(num_tokens >= 0 && rank > 0 && rot_dim >= 0 && first >= 0 && (long)first + rank + rot_dim <= stride,
            "latent_store: bad sizes");
  QRT_CHECK(pairs >= 0 && 2 * pairs <= rot_dim && (pairs == 0 || freq), "latent_store: %d pairs in %d elements", pairs, rot_dim);
  QRT_CHECK(page_size > 0 && num_pages > 0 && slots && positions, "latent_store: no cache");
  if (num_tokens == 0) return 0;
  if (dtype == QRT_F32)
    latent_store_kernel<float><<<num_tokens, 256, 0, stream>>>((const float*)y, stride, first, rank, rot_dim, weight, eps, positions,
                                                               freq, pairs, slots, (float*)k_cache, (float*)v_cache, page_size, neighbours, magnitude);
  else if (dtype == QRT_BF16)
    latent_store_kernel<bf16_t><<<num_tokens, 256, 0, stream>>>((const bf16_t*)y, stride, first, rank, rot_dim, weight, eps, positions,
                                                                freq, pairs, slots, (bf16_t*)k_cache, (bf16_t*)v_cache, page_size, neighbours, magnitude);
  else return qrt_fail("latent_store: unknown dtype %d", dtype);
  QRT_LAUNCH_CHECK("latent_store");
  return 0;
}

// ---------------------------------------------------------------- rotate half, from one layout to another
struct RotateArgs {
  const void* x; long x_row; int in_stride, in_offset;
  void* out; long out_row; int out_stride, out_offset;
  int heads, width, pairs;
  const int* positions; const float* freq;
  int scale_from_head; float scale;  // heads from this one on are multiplied by `scale` after turning
  int neighbours; float magnitude;   // pairs of neighbours instead of halves; what multiplies sines and cosines
};

template <typename TI, typename TO>
__global__ __launch_bounds__(256) void rotate_half_kernel(RotateArgs a) {
  const int t = blockIdx.x;
  const float pos = a.pairs ? (float)a.positions[t] : 0.f;
  const TI* xr = (const TI*)a.x + (size_t)t * a.x_row + a.in_offset;
  TO* orow = (TO*)a.out + (size_t)t * a.out_row + a.out_offset;
  const int total = a.heads * a.width;
  for (int e = blockIdx.y * 256 + threadIdx.x; e < total; e += 256 * gridDim.y) {
    const int h = e / a.width, i = e - h * a.width;
    const TI* src = xr + (size_t)h * a.in_stride;
    float x = to_f32<TI>(src[i]);
    if (i < 2 * a.pairs) {
      int j, o;
      bool first;
      rotation_partner(i, a.pairs, a.neighbours, &j, &o, &first);
      float sn, cs;
      sincos_angle(pos * a.freq[j], &sn, &cs);
      sn *= a.magnitude;
      cs *= a.magnitude;
      const float other = to_f32<TI>(src[o]);
      x = first ? x * cs - other * sn : x * cs + other * sn;
    }
    if (h >= a.scale_from_head) x *= a.scale;
    orow[(size_t)h * a.out_stride + i] = from_f32<TO>(x);
  }
}

extern "C" int qrt_rotate_half(const RotateArgs* args, int in_dtype, int out_dtype, int num_tokens, hipStream_t stream) {
  RotateArgs a = *args;
  QRT_CHECK(num_tokens >= 0 && a.heads > 0 && a.width > 0 && a.pairs >= 0 && 2 * a.pairs <= a.width, "rotate_half: bad sizes");
  QRT_CHECK(a.in_offset >= 0 && a.in_offset + a.width <= a.in_stride && (long)a.heads * a.in_stride <= a.x_row &&
            a.out_offset >= 0 && a.out_offset + a.width <= a.out_stride && (long)a.heads * a.out_stride <= a.out_row,
            "rotate_half: heads of %d at %d in rows of %ld, to heads of %d at %d in rows of %ld", a.in_stride, a.in_offset,
            a.x_row, a.out_stride, a.out_offset, a.out_row);
  QRT_CHECK(a.pairs == 0 || (a.freq && a.positions), "rotate_half: no angles");
  if (num_tokens == 0) return 0;
  const int total = a.heads * a.width;
  const dim3 grid(num_tokens, num_tokens >= 512 ? 1 : min((total + 255) / 256, 64));
  if (in_dtype == QRT_F32 && out_dtype == QRT_F32) rotate_half_kernel<float, float><<<grid, 256, 0, stream>>>(a);
  else if (in_dtype == QRT_BF16 && out_dtype == QRT_BF16) rotate_half_kernel<bf16_t, bf16_t><<<grid, 256, 0, stream>>>(a);
  else if (in_dtype == QRT_BF16 && out_dtype == QRT_F32) rotate_half_kernel<bf16_t, float><<<grid, 256, 0, stream>>>(a);
  else return qrt_fail("rotate_half: no form for types %d -> %d", in_dtype, out_dtype);
  QRT_LAUNCH_CHECK("rotate_half");
  return 0;
}

// ---------------------------------------------------------------- a product per head
// One block of four waves per (token, head): the head's input in LDS as float32, each wave takes
// outputs wave, wave + 4, ...; an output is one wave's sum over K in a fixed order, whatever else is
// in the batch. For few tokens and for float32; many tokens in bfloat16 go to a batched library product.
template <typename T>
__global__ __launch_bounds__(256) void heads_linear_kernel(const T* __restrict__ x, long x_row, int in_stride, int in_offset,
                                                           const T* __restrict__ w, int n, int k, T* __restrict__ out,
                                                           long out_row, int out_stride, int out_offset) {
  extern __shared__ float xs[];
  const int t = blockIdx.x, h = blockIdx.y;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const T* xr = x + (size_t)t * x_row + (size_t)h * in_stride + in_offset;
  for (int i = threadIdx.x; i < k; i += 256) xs[i] = to_f32<T>(xr[i]);
  __syncthreads();
  const T* wh = w + (size_t)h * n * k;
  T* o = out + (size_t)t * out_row + (size_t)h * out_stride + out_offset;
  for (int j = wave; j < n; j += 4) {
    const T* wr = wh + (size_t)j * k;
    float acc = 0.f;
    for (int c = lane; c < k; c += 64) acc = fmaf(xs[c], to_f32<T>(wr[c]), acc);
    acc = wave_sum(acc);
    if (lane == 0) o[j] = from_f32<T>(acc);
  }
}

// Few tokens: one block per (64 outputs of a head), all tokens of the step at once, so that the
// head's weights are read once a step. Lane j of every wave owns output j of the block's 64 and
// walks its weight row; the four waves take a quarter of K each, and their partial sums meet in
// LDS in a fixed order. A token's sum is the same sequence of operations whatever else is in the
// batch. Tokens go in groups of HL_TOKENS with the inputs in LDS as float32.
#define HL_TOKENS 8
template <typename T>
__global__ __launch_bounds__(256) void heads_linear_rows_kernel(const T* __restrict__ x, long x_row, int in_stride, int in_offset,
                                                                const T* __restrict__ w, int n, int k, T* __restrict__ out,
                                                                long out_row, int out_stride, int out_offset, int num_tokens) {
  extern __shared__ float sm[];
  float* xs = sm;                        // [HL_TOKENS][k]
  float* red = sm + HL_TOKENS * k;       // [4][HL_TOKENS][64]
  const int h = blockIdx.y, j0 = blockIdx.x * 64;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int j = min(j0 + lane, n - 1);
  const T* wr = w + ((size_t)h * n + j) * k;
  const int per = (k + 3) / 4, c0 = min(wave * per, k), c1 = min(k, c0 + per);
  for (int t0 = 0; t0 < num_tokens; t0 += HL_TOKENS) {
    const int nt = min(HL_TOKENS, num_tokens - t0);
    __syncthreads();
    for (int i = threadIdx.x; i < HL_TOKENS * k; i += 256) {
      const int t = i / k, c = i - t * k;
      xs[i] = t < nt ? to_f32<T>(x[(size_t)(t0 + t) * x_row + (size_t)h * in_stride + in_offset + c]) : 0.f;
    }
    __syncthreads();
    float acc[HL_TOKENS];
#pragma unroll
    for (int t = 0; t < HL_TOKENS; ++t) acc[t] = 0.f;
    if (sizeof(T) == 2 && (k & 31) == 0 && ((uintptr_t)w & 15) == 0) {
      // bfloat16 rows whose quarters are whole 16-byte pieces: eight weights a load
      for (int c = c0; c < c1; c += 8) {
        const bf16x8_t w8 = *(const bf16x8_t*)((const bf16_t*)wr + c);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float wv = (float)w8[e];
#pragma unroll
          for (int t = 0; t < HL_TOKENS; ++t) acc[t] = fmaf(xs[t * k + c + e], wv, acc[t]);
        }
      }
    } else {
      for (int c = c0; c < c1; ++c) {
        const float wv = to_f32<T>(wr[c]);
#pragma unroll
        for (int t = 0; t < HL_TOKENS; ++t) acc[t] = fmaf(xs[t * k + c], wv, acc[t]);
      }
    }
#pragma unroll
    for (int t = 0; t < HL_TOKENS; ++t) red[(wave * HL_TOKENS + t) * 64 + lane] = acc[t];
    __syncthreads();
    for (int i = threadIdx.x; i < nt * 64; i += 256) {
      const int t = i >> 6, l = i & 63;
      if (j0 + l < n) {
        const float sum = ((red[(0 * HL_TOKENS + t) * 64 + l] + red[(1 * HL_TOKENS + t) * 64 + l]) +
                           red[(2 * HL_TOKENS + t) * 64 + l]) + red[(3 * HL_TOKENS + t) * 64 + l];
        out[(size_t)(t0 + t) * out_row + (size_t)h * out_stride + out_offset + j0 + l] = from_f32<T>(sum);
      }
    }
  }
}

extern "C" int qrt_heads_linear(const void* x, long x_row, int in_stride, int in_offset, const void* w, int heads, int n, int k,
                                void* out, long out_row, int out_stride, int out_offset, int dtype, int num_tokens,
                                hipStream_t stream) {
  QRT_CHECK(num_tokens >= 0 && heads > 0 && heads <= 65535 && n > 0 && k > 0 && k <= 16384, "heads_linear: bad sizes");
  QRT_CHECK(in_offset >= 0 && in_offset + k <= in_stride && (long)heads * in_stride <= x_row && out_offset >= 0 &&
            out_offset + n <= out_stride && (long)heads * out_stride <= out_row, "heads_linear: heads do not fit their rows");
  if (num_tokens == 0) return 0;
  if (num_tokens <= 64 && k <= 1024) {  // the head's weights once a step
    const dim3 rows_grid((n + 63) / 64, heads);
    const size_t rows_lds = (size_t)(HL_TOKENS * k + 4 * HL_TOKENS * 64) * sizeof(float);
    if (dtype == QRT_F32)
      heads_linear_rows_kernel<float><<<rows_grid, 256, rows_lds, stream>>>((const float*)x, x_row, in_stride, in_offset, (const float*)w,
                                                                            n, k, (float*)out, out_row, out_stride, out_offset, num_tokens);
    else if (dtype == QRT_BF16)
      heads_linear_rows_kernel<bf16_t><<<rows_grid, 256, rows_lds, stream>>>((const bf16_t*)x, x_row, in_stride, in_offset, (const bf16_t*)w,
                                                                             n, k, (bf16_t*)out, out_row, out_stride, out_offset, num_tokens);
    else return qrt_fail("heads_linear: unknown dtype %d", dtype);
    QRT_LAUNCH_CHECK("heads_linear_rows");
    return 0;
  }
  const dim3 grid(num_tokens, heads);
  const size_t lds = (size_t)k * sizeof(float);
  if (dtype == QRT_F32)
    heads_linear_kernel<float><<<grid, 256, lds, stream>>>((const float*)x, x_row, in_stride, in_offset, (const float*)w, n, k,
                                                           (float*)out, out_row, out_stride, out_offset);
  else if (dtype == QRT_BF16)
    heads_linear_kernel<bf16_t><<<grid, 256, lds, stream>>>((const bf16_t*)x, x_row, in_stride, in_offset, (const bf16_t*)w, n, k,
                                                            (bf16_t*)out, out_row, out_stride, out_offset);
  else return qrt_fail("heads_linear: unknown dtype %d", dtype);
  QRT_LAUNCH_CHECK("heads_linear");
  return 0;
}
