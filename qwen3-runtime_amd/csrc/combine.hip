// Small float32 steps between sub-layers that are neither a product nor a plain norm:
// the mean of several outputs each RMS-normed first (mixers side by side), the residual
// stream joined with the embedding for a product that re-enters it (a looped span's entry),
// a sum of two sub-layer outputs (routed and shared experts), and gated activations other than
// SwiGLU. Inputs that are sub-layer outputs may be one matrix [T, H] (float32 or bfloat16) or
// float32 planes [P, T, H] whose sum they are.
#include "common.h"
#include <math.h>

struct Planes {
  const void* p; int code; int planes; long plane_stride;
};

// Up to eight planes are asked for together (a plane that is not there: the first one again, dropped),
// so that an element costs one trip to memory however many planes it has; they are added in order.
__device__ __forceinline__ float planes_at(const Planes& y, size_t i) {
  if (y.code == QRT_BF16) return (float)((const bf16_t*)y.p)[i];
  const float* p = (const float*)y.p;
  if (y.planes == 1) return p[i];
  float part[8];
#pragma unroll
  for (int k = 0; k < 8; ++k) part[k] = p[(size_t)(k < y.planes ? k : 0) * y.plane_stride + i];
  float v = 0.f;
#pragma unroll
  for (int k = 0; k < 8; ++k) v += k < y.planes ? part[k] : 0.f;
  for (int k = 8; k < y.planes; ++k) v += p[(size_t)k * y.plane_stride + i];
  return v;
}

// Two sums over a block of up to 1,024 threads at once; every thread gets both.
__device__ __forceinline__ void block_sum2(float& a, float& b, float* red) {
  a = wave_sum(a);
  b = wave_sum(b);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int nw = (blockDim.x + 63) >> 6;
  if (lane == 0) { red[wave] = a; red[16 + wave] = b; }
  __syncthreads();
  a = b = 0.f;
  for (int i = 0; i < nw; ++i) { a += red[i]; b += red[16 + i]; }  // the same order in every thread
}

// out[t] = (1/2) (a[t] / rms(a[t]) * wa + b[t] / rms(b[t]) * wb), rms with eps inside the root.
// One block of 1,024 threads per token; a thread keeps its elements of both rows in registers
// (rows up to 4,096 wide; wider rows are read a second time), and asks for all of them, and for
// the weights, before the first use: a token costs one round of memory latency.
#define NM_KEEP 4
__global__ __launch_bounds__(1024) void norm_mean_kernel(Planes ya, Planes yb, const float* __restrict__ wa,
                                                         const float* __restrict__ wb, float* __restrict__ out,
                                                         int hidden, float eps) {
  __shared__ float red[32];
  const size_t row = (size_t)blockIdx.x * hidden;
  float va[NM_KEEP], vb[NM_KEEP], ua[NM_KEEP], ub[NM_KEEP];
#pragma unroll
  for (int j = 0; j < NM_KEEP; ++j) {
    const int i = min((int)threadIdx.x + 1024 * j, hidden - 1);  // beyond the row: its last element, dropped below
    va[j] = planes_at(ya, row + i);
    vb[j] = planes_at(yb, row + i);
    ua[j] = wa[i];
    ub[j] = wb[i];
  }
  float sa = 0.f, sb = 0.f;
#pragma unroll
  for (int j = 0; j < NM_KEEP; ++j)
    if ((int)threadIdx.x + 1024 * j < hidden) {
      sa += va[j] * va[j];
      sb += vb[j] * vb[j];
    }
  for (int i = threadIdx.x + 1024 * NM_KEEP; i < hidden; i += 1024) {
    const float x = planes_at(ya, row + i), y = planes_at(yb, row + i);
    sa += x * x;
    sb += y * y;
  }
  block_sum2(sa, sb, red);
  const float ia = 1.0f / sqrtf(sa / (float)hidden + eps);
  const float ib = 1.0f / sqrtf(sb / (float)hidden + eps);
#pragma unroll
  for (int j = 0; j < NM_KEEP; ++j) {
    const int i = threadIdx.x + 1024 * j;
    if (i < hidden) out[row + i] = 0.5f * (va[j] * ia * ua[j] + vb[j] * ib * ub[j]);
  }
  for (int i = threadIdx.x + 1024 * NM_KEEP; i < hidden; i += 1024)
    out[row + i] = 0.5f * (planes_at(ya, row + i) * ia * wa[i] + planes_at(yb, row + i) * ib * wb[i]);
}

extern "C" int qrt_norm_mean(const void* a, int a_code, int a_planes, const void* b, int b_code, int b_planes,
                             const float* wa, const float* wb, float* out, int num_tokens, int hidden, float eps,
                             hipStream_t stream) {
  QRT_CHECK(num_tokens >= 0 && hidden > 0 && a_planes >= 1 && b_planes >= 1, "norm_mean: bad sizes");
  QRT_CHECK((a_code == QRT_F32 || (a_code == QRT_BF16 && a_planes == 1)) && (b_code == QRT_F32 || (b_code == QRT_BF16 && b_planes == 1)),
            "norm_mean: planes are float32");
  if (num_tokens == 0) return 0;
  const long stride = (long)num_tokens * hidden;
  norm_mean_kernel<<<dim3(num_tokens), 1024, 0, stream>>>(Planes{a, a_code, a_planes, stride}, Planes{b, b_code, b_planes, stride},
                                                         wa, wb, out, hidden, eps);
  QRT_LAUNCH_CHECK("norm_mean");
  return 0;
}

// out[t] = [ residual[t] + scale * delta[t] | origin[t] ]   (2H wide, in the products' type)
template <typename TO>
__global__ void add_concat_kernel(const float* __restrict__ residual, Planes delta, float scale,
                                  const float* __restrict__ origin, TO* __restrict__ out, int hidden) {
  const size_t row = (size_t)blockIdx.x * hidden;
  TO* o = out + 2 * row;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    float v = residual[row + i];
    if (delta.p) v = fmaf(scale, planes_at(delta, row + i), v);
    o[i] = from_f32<TO>(v);
    o[hidden + i] = from_f32<TO>(origin[row + i]);
  }
}

extern "C" int qrt_add_concat(const float* residual, const void* delta, int d_code, int d_planes, float scale,
                              const float* origin, void* out, int out_dtype, int num_tokens, int hidden,
                              hipStream_t stream) {
  QRT_CHECK(num_tokens >= 0 && hidden > 0 && d_planes >= 1, "add_concat: bad sizes");
  QRT_CHECK(!delta || d_code == QRT_F32 || (d_code == QRT_BF16 && d_planes == 1), "add_concat: planes are float32");
  if (num_tokens == 0) return 0;
  const Planes d{delta, d_code, d_planes, (long)num_tokens * hidden};
  if (out_dtype == QRT_F32) add_concat_kernel<float><<<dim3(num_tokens), 256, 0, stream>>>(residual, d, scale, origin, (float*)out, hidden);
  else if (out_dtype == QRT_BF16) add_concat_kernel<bf16_t><<<dim3(num_tokens), 256, 0, stream>>>(residual, d, scale, origin, (bf16_t*)out, hidden);
  else return qrt_fail("add_concat: unknown dtype %d", out_dtype);
  QRT_LAUNCH_CHECK("add_concat");
  return 0;
}

// acc[t] += y[t]
__global__ void accumulate_kernel(float* __restrict__ acc, Planes y, long n) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) acc[i] += planes_at(y, (size_t)i);
}

extern "C" int qrt_accumulate(float* acc, const void* y, int y_code, int y_planes, long n, hipStream_t stream) {
  QRT_CHECK(n >= 0 && y_planes >= 1, "accumulate: bad sizes");
  QRT_CHECK(y_code == QRT_F32 || (y_code == QRT_BF16 && y_planes == 1), "accumulate: planes are float32");
  if (n == 0) return 0;
  accumulate_kernel<<<dim3((unsigned)((n + 255) / 256)), 256, 0, stream>>>(acc, Planes{y, y_code, y_planes, n}, n);
  QRT_LAUNCH_CHECK("accumulate");
  return 0;
}

// out[t, i] = act(gu[t, i], gu[t, I + i]) for the gated activations of common.h
template <typename T>
__global__ void gated_act_kernel(const T* __restrict__ gu, T* __restrict__ out, int inter, int kind, float limit) {
  const T* row = gu + (size_t)blockIdx.x * 2 * inter;
  for (int i = threadIdx.x; i < inter; i += blockDim.x)
    out[(size_t)blockIdx.x * inter + i] = from_f32<T>(gated_act(to_f32<T>(row[i]), to_f32<T>(row[inter + i]), kind, limit));
}

extern "C" int qrt_gated_act(const void* gu, void* out, int dtype, int num_tokens, int inter, int kind, float limit,
                             hipStream_t stream) {
  QRT_CHECK(num_tokens >= 0 && inter > 0, "gated_act: bad sizes");
  QRT_CHECK(kind == QRT_ACT_SWIGLU || kind == QRT_ACT_CLAMPED, "gated_act: unknown activation %d", kind);
  if (num_tokens == 0) return 0;
  if (dtype == QRT_F32) gated_act_kernel<float><<<dim3(num_tokens), 256, 0, stream>>>((const float*)gu, (float*)out, inter, kind, limit);
  else if (dtype == QRT_BF16) gated_act_kernel<bf16_t><<<dim3(num_tokens), 256, 0, stream>>>((const bf16_t*)gu, (bf16_t*)out, inter, kind, limit);
  else return qrt_fail("gated_act: unknown dtype %d", dtype);
  QRT_LAUNCH_CHECK("gated_act");
  return 0;
}

// ------------------------------------------------ a sub-layer output with a norm of its own
// r = rows ? rows[b] : b
// d = y[r] / rms(y[r]) * w_after;  x = residual[r] + d  (written back without `rows`);
// out[b] = x / rms(x) * w.  Both rms with their eps inside the root, everything float32.
// One block of 1,024 threads per row; a thread keeps its elements in registers (rows up to 4,096
// wide; the rest of a wider row is read again), all of them and the weights asked for first.
template <typename TO>
__global__ __launch_bounds__(1024) void norm_add_rmsnorm_kernel(float* __restrict__ residual, Planes y,
                                                                const float* __restrict__ w_after, float eps_after,
                                                                const float* __restrict__ weight, float eps,
                                                                const int* __restrict__ rows, TO* __restrict__ out, int hidden) {
  __shared__ float red[32];
  const int b = blockIdx.x;
  const int r = rows ? rows[b] : b;
  const size_t row = (size_t)r * hidden;
  float vy[NM_KEEP], vx[NM_KEEP], wa[NM_KEEP], wn[NM_KEEP];
#pragma unroll
  for (int j = 0; j < NM_KEEP; ++j) {
    const int i = min((int)threadIdx.x + 1024 * j, hidden - 1);
    vy[j] = planes_at(y, row + i);
    vx[j] = residual[row + i];
    wa[j] = w_after[i];
    wn[j] = weight[i];
  }
  float sy = 0.f;
#pragma unroll
  for (int j = 0; j < NM_KEEP; ++j)
    if ((int)threadIdx.x + 1024 * j < hidden) sy += vy[j] * vy[j];
  for (int i = threadIdx.x + 1024 * NM_KEEP; i < hidden; i += 1024) {
    const float v = planes_at(y, row + i);
    sy += v * v;
  }
  sy = block_sum(sy, red);
  const float iy = 1.0f / sqrtf(sy / (float)hidden + eps_after);
  float sx = 0.f;
#pragma unroll
  for (int j = 0; j < NM_KEEP; ++j) {
    const int i = threadIdx.x + 1024 * j;
    if (i < hidden) {
      vx[j] += vy[j] * iy * wa[j];
      sx += vx[j] * vx[j];
      if (!rows) residual[row + i] = vx[j];
    }
  }
  for (int i = threadIdx.x + 1024 * NM_KEEP; i < hidden; i += 1024) {
    const float x = residual[row + i] + planes_at(y, row + i) * iy * w_after[i];
    sx += x * x;
    if (!rows) residual[row + i] = x;
  }
  sx = block_sum(sx, red);
  const float ix = 1.0f / sqrtf(sx / (float)hidden + eps);
#pragma unroll
  for (int j = 0; j < NM_KEEP; ++j) {
    const int i = threadIdx.x + 1024 * j;
    if (i < hidden) out[(size_t)b * hidden + i] = from_f32<TO>(vx[j] * ix * wn[j]);
  }
  for (int i = threadIdx.x + 1024 * NM_KEEP; i < hidden; i += 1024) {
    const float x = rows ? residual[row + i] + planes_at(y, row + i) * iy * w_after[i] : residual[row + i];
    out[(size_t)b * hidden + i] = from_f32<TO>(x * ix * weight[i]);
  }
}

extern "C" int qrt_norm_add_rmsnorm(float* residual, const void* y, int y_code, int y_planes, long plane_stride,
                                    const float* w_after, float eps_after, const float* weight, float eps, const int* rows,
                                    void* out, int out_dtype, int num_out, int hidden, hipStream_t stream) {
  QRT_CHECK(num_out >= 0 && hidden > 0 && y_planes >= 1, "norm_add_rmsnorm: bad sizes");
  QRT_CHECK(y_code == QRT_F32 || (y_code == QRT_BF16 && y_planes == 1), "norm_add_rmsnorm: planes are float32");
  if (num_out == 0) return 0;
  const Planes yp{y, y_code, y_planes, plane_stride};
  if (out_dtype == QRT_F32)
    norm_add_rmsnorm_kernel<float><<<num_out, 1024, 0, stream>>>(residual, yp, w_after, eps_after, weight, eps, rows, (float*)out, hidden);
  else if (out_dtype == QRT_BF16)
    norm_add_rmsnorm_kernel<bf16_t><<<num_out, 1024, 0, stream>>>(residual, yp, w_after, eps_after, weight, eps, rows, (bf16_t*)out, hidden);
  else return qrt_fail("norm_add_rmsnorm: unknown dtype %d", out_dtype);
  QRT_LAUNCH_CHECK("norm_add_rmsnorm");
  return 0;
}

// ------------------------------------------------ a sum of scaled sub-layer outputs, then the norm
// x = residual[r] + sum_i s_i * y_i[r]  (element by element; written back without `rows`);
// out[b] = x / rms(x) * w.  Everything float32. One block of 1,024 threads per row; a thread keeps
// its elements in registers (rows up to 4,096 wide; the rest of a wider row is computed again),
// all terms, vectors and weights asked for before the first is used. The terms are added in order.
#define SA_TERMS 4
struct ScaledTerms {
  Planes y[SA_TERMS];
  const float* scale[SA_TERMS];
  int count;
};

template <int N>
__device__ __forceinline__ float scaled_sum_at(const ScaledTerms& s, float x, size_t at, int i) {
  float part[N], sc[N];
#pragma unroll
  for (int k = 0; k < N; ++k) {
    part[k] = planes_at(s.y[k], at);
    sc[k] = s.scale[k][i];
  }
#pragma unroll
  for (int k = 0; k < N; ++k) x = fmaf(sc[k], part[k], x);
  return x;
}

template <typename TO, int N>
__global__ __launch_bounds__(1024) void scaled_add_rmsnorm_kernel(float* __restrict__ residual, ScaledTerms s,
                                                                  const float* __restrict__ weight, float eps,
                                                                  const int* __restrict__ rows, TO* __restrict__ out,
                                                                  int hidden) {
  __shared__ float red[32];
  const int b = blockIdx.x;
  const int r = rows ? rows[b] : b;
  const size_t row = (size_t)r * hidden;
  float vx[NM_KEEP], wn[NM_KEEP];
#pragma unroll
  for (int j = 0; j < NM_KEEP; ++j) {
    const int i = min((int)threadIdx.x + 1024 * j, hidden - 1);
    vx[j] = scaled_sum_at<N>(s, residual[row + i], row + i, i);
    wn[j] = weight[i];
  }
  float sx = 0.f;
#pragma unroll
  for (int j = 0; j < NM_KEEP; ++j) {
    const int i = threadIdx.x + 1024 * j;
    if (i < hidden) {
      sx += vx[j] * vx[j];
      if (!rows) residual[row + i] = vx[j];
    }
  }
  for (int i = threadIdx.x + 1024 * NM_KEEP; i < hidden; i += 1024) {
    const float x = scaled_sum_at<N>(s, residual[row + i], row + i, i);
    sx += x * x;
    if (!rows) residual[row + i] = x;
  }
  sx = block_sum(sx, red);
  const float ix = 1.0f / sqrtf(sx / (float)hidden + eps);
#pragma unroll
  for (int j = 0; j < NM_KEEP; ++j) {
    const int i = threadIdx.x + 1024 * j;
    if (i < hidden) out[(size_t)b * hidden + i] = from_f32<TO>(vx[j] * ix * wn[j]);
  }
  for (int i = threadIdx.x + 1024 * NM_KEEP; i < hidden; i += 1024) {
    const float x = rows ? scaled_sum_at<N>(s, residual[row + i], row + i, i) : residual[row + i];
    out[(size_t)b * hidden + i] = from_f32<TO>(x * ix * weight[i]);
  }
}

// y, y_code, y_planes, scale: `count` entries each; all planes [P, T, H] lie `plane_stride` elements apart
extern "C" int qrt_scaled_add_rmsnorm(float* residual, const void* const* y, const int* y_code, const int* y_planes,
                                      const float* const* scale, int count, long plane_stride, const float* weight,
                                      float eps, const int* rows, void* out, int out_dtype, int num_out, int hidden,
                                      hipStream_t stream) {
  QRT_CHECK(num_out >= 0 && hidden > 0 && count >= 1 && count <= SA_TERMS, "scaled_add_rmsnorm: %d terms (1..%d)", count, SA_TERMS);
  ScaledTerms s;
  s.count = count;
  for (int k = 0; k < SA_TERMS; ++k) {
    const int kk = k < count ? k : 0;
    QRT_CHECK(y[kk] && scale[kk] && y_planes[kk] >= 1, "scaled_add_rmsnorm: term %d is not there", kk);
    QRT_CHECK(y_code[kk] == QRT_F32 || (y_code[kk] == QRT_BF16 && y_planes[kk] == 1), "scaled_add_rmsnorm: planes are float32");
    s.y[k] = Planes{y[kk], y_code[kk], y_planes[kk], plane_stride};
    s.scale[k] = scale[kk];
  }
  if (num_out == 0) return 0;
  QRT_CHECK(out_dtype == QRT_F32 || out_dtype == QRT_BF16, "scaled_add_rmsnorm: unknown dtype %d", out_dtype);
#define SA_LAUNCH(N)                                                                                                          \
  if (out_dtype == QRT_F32)                                                                                                   \
    scaled_add_rmsnorm_kernel<float, N><<<num_out, 1024, 0, stream>>>(residual, s, weight, eps, rows, (float*)out, hidden);   \
  else                                                                                                                        \
    scaled_add_rmsnorm_kernel<bf16_t, N><<<num_out, 1024, 0, stream>>>(residual, s, weight, eps, rows, (bf16_t*)out, hidden)
  if (count == 1) { SA_LAUNCH(1); }
  else if (count == 2) { SA_LAUNCH(2); }
  else if (count == 3) { SA_LAUNCH(3); }
  else { SA_LAUNCH(4); }
#undef SA_LAUNCH
  QRT_LAUNCH_CHECK("scaled_add_rmsnorm");
  return 0;
}

// ------------------------------------------------ small elementwise steps
// x *= factor, float32, in place (logits times a constant)
__global__ void scale_kernel(float* __restrict__ x, float factor, long n) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i < n) x[i] *= factor;
}

extern "C" int qrt_scale(float* x, float factor, long n, hipStream_t stream) {
  QRT_CHECK(n >= 0, "scale: bad size");
  if (n == 0) return 0;
  scale_kernel<<<dim3((unsigned)((n + 255) / 256)), 256, 0, stream>>>(x, factor, n);
  QRT_LAUNCH_CHECK("scale");
  return 0;
}

// activations without a gate, float32 inside. RELU2: max(x, 0)^2.
#define QRT_UNARY_RELU2 0
template <typename T>
__global__ void unary_act_kernel(const T* __restrict__ x, T* __restrict__ out, long n, int kind) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i < n) {
    const float v = fmaxf(to_f32<T>(x[i]), 0.f);
    out[i] = from_f32<T>(v * v);
  }
}

extern "C" int qrt_unary_act(const void* x, void* out, int dtype, long n, int kind, hipStream_t stream) {
  QRT_CHECK(n >= 0 && kind == QRT_UNARY_RELU2, "unary_act: unknown activation %d", kind);
  if (n == 0) return 0;
  const dim3 grid((unsigned)((n + 255) / 256));
  if (dtype == QRT_F32) unary_act_kernel<float><<<grid, 256, 0, stream>>>((const float*)x, (float*)out, n, kind);
  else if (dtype == QRT_BF16) unary_act_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)x, (bf16_t*)out, n, kind);
  else return qrt_fail("unary_act: unknown dtype %d", dtype);
  QRT_LAUNCH_CHECK("unary_act");
  return 0;
}
