// Paged attention in true 32-bit, any head size: the check path.
//
// One wave per (query token, query head). The wave walks the keys its query may
// see in chunks of 64 (one key per lane for the scores), keeps a running
// maximum and sum (online softmax, float32), and accumulates the context with
// each lane owning head elements lane, lane + 64, ... Query head h reads key
// head h / g. The query at position p sees keys j <= p, and j > p - window when
// a window is set, or j >= p - p % chunk when a chunk size is. Scores are
// dot * scale, then, with a cap, cap * tanh(score / cap). Values may have another
// size Dv than keys; with a gate the output is multiplied by sigmoid(gate). Beside a window the
// first keep_first keys of the sequence stay visible to every later query (their pages stay in the
// table; the pages between them and the window may be gone and are not touched). With a sink the
// softmax's denominator has one more term of score 0: p_j = exp(s_j) / (1 + sum exp(s_j)). Cache
// layout: keys [page, head, offset, D], values [page, head, Dv, offset].
#include "common.h"
#include <math.h>

struct AttnArgs {
  const void* q;         // [T, nq * D]
  void* out;             // [T, nq * D]
  const void* k_cache;
  const void* v_cache;
  const int* positions;  // [T] position of each query token
  const int* seq_of_token;  // [T]
  const int* block_table;   // [S, table_width]
  int table_width;
  int num_tokens, nq, nkv, head_dim, page_size, window;  // window 0: none
  float scale;
  int chunk;       // 0: none
  float softcap;   // 0: none
  int value_dim;   // 0: head_dim
  const void* gate;  // [T, gate_stride] with nq * Dv columns used, or null
  long gate_stride;
  int keep_first;  // with a window: keys j < keep_first are seen too
  int sink;        // 1: one more term exp(0) in the denominator
};

#define MAX_D 1024

template <typename T>
__global__ __launch_bounds__(64) void attention_f32_kernel(AttnArgs a) {
  __shared__ float qs[MAX_D];
  const int lane = threadIdx.x;
  const int t = blockIdx.x, h = blockIdx.y;
  const int D = a.head_dim, ps = a.page_size, Dv = a.value_dim;
  const int kvh = h / (a.nq / a.nkv);
  const int pos = a.positions[t];
  const int* table = a.block_table + (size_t)a.seq_of_token[t] * a.table_width;
  const T* q = (const T*)a.q + ((size_t)t * a.nq + h) * D;
  for (int i = lane; i < D; i += 64) qs[i] = to_f32<T>(q[i]);
  __syncthreads();

  const int lo = a.window > 0 ? max(0, pos - a.window + 1) : (a.chunk > 0 ? pos - pos % a.chunk : 0);
  float m = -INFINITY, l = 0.f;
  float acc[MAX_D / 64];
#pragma unroll
  for (int i = 0; i < MAX_D / 64; ++i) acc[i] = 0.f;

  const T* kc = (const T*)a.k_cache;
  const T* vc = (const T*)a.v_cache;
  // two stretches of keys: the kept first ones that lie before the window, then the window
  const int kept_end = a.window > 0 ? min(a.keep_first, lo) : 0;
  for (int seg = kept_end > 0 ? 0 : 1; seg < 2; ++seg) {
  const int seg_begin = seg == 0 ? 0 : lo, seg_last = seg == 0 ? kept_end - 1 : pos;
  for (int j0 = seg_begin; j0 <= seg_last; j0 += 64) {
    const int j = j0 + lane;
    const bool valid = j <= seg_last;
    float s = -INFINITY;
    int page = 0, off = 0;
    if (valid) {
      page = table[j / ps];
      off = j % ps;
      const T* kr = kc + (((size_t)page * a.nkv + kvh) * ps + off) * D;
      float dot = 0.f;
      for (int d = 0; d < D; ++d) dot = fmaf(qs[d], to_f32<T>(kr[d]), dot);
      s = dot * a.scale;
      if (a.softcap > 0.f) s = a.softcap * tanhf(s / a.softcap);
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float p = valid ? expf(s - m_new) : 0.f;
    const float corr = expf(m - m_new);  // m = -inf at the first chunk: exp(-inf) = 0
    l = l * corr + wave_sum(p);
    m = m_new;
#pragma unroll
    for (int i = 0; i < MAX_D / 64; ++i) acc[i] *= corr;
    const int n = min(64, seg_last - j0 + 1);
    for (int jj = 0; jj < n; ++jj) {
      const float pj = __shfl(p, jj, 64);
      const int pg = __shfl(page, jj, 64);
      const int of = __shfl(off, jj, 64);
      const T* vr = vc + ((size_t)pg * a.nkv + kvh) * Dv * ps + of;
#pragma unroll
      for (int i = 0; i < MAX_D / 64; ++i) {
        const int d = lane + 64 * i;
        if (d < Dv) acc[i] = fmaf(pj, to_f32<T>(vr[(size_t)d * ps]), acc[i]);
      }
    }
  }
  }
  if (a.sink) {  // the sink: a key of score 0 without a value
    const float m_new = fmaxf(m, 0.f);
    const float corr = expf(m - m_new);
    l = l * corr + expf(-m_new);
#pragma unroll
    for (int i = 0; i < MAX_D / 64; ++i) acc[i] *= corr;
  }
  T* o = (T*)a.out + ((size_t)t * a.nq + h) * Dv;
  const T* gate = a.gate ? (const T*)a.gate + (size_t)t * a.gate_stride + (size_t)h * Dv : nullptr;
  const float inv = l > 0.f ? 1.0f / l : 0.f;
#pragma unroll
  for (int i = 0; i < MAX_D / 64; ++i) {
    const int d = lane + 64 * i;
    if (d < Dv) {
      float v = acc[i] * inv;
      if (gate) v *= 1.0f / (1.0f + expf(-to_f32<T>(gate[d])));
      o[d] = from_f32<T>(v);
    }
  }
}

extern "C" int qrt_attention_f32(const AttnArgs* args, int dtype, hipStream_t stream) {
  AttnArgs a = *args;
  QRT_CHECK(a.num_tokens >= 0 && a.nq > 0 && a.nkv > 0 && a.nq % a.nkv == 0,
            "attention: %d query heads do not divide into %d key heads", a.nq, a.nkv);
  QRT_CHECK(a.head_dim > 0 && a.head_dim <= MAX_D, "attention: head size %d is above %d", a.head_dim, MAX_D);
  QRT_CHECK(a.page_size > 0 && a.table_width > 0 && a.window >= 0, "attention: bad page size, table width or window");
  if (a.value_dim == 0) a.value_dim = a.head_dim;
  QRT_CHECK(a.value_dim > 0 && a.value_dim <= MAX_D, "attention: value size %d is above %d", a.value_dim, MAX_D);
  QRT_CHECK(a.chunk >= 0 && !(a.chunk > 0 && a.window > 0), "attention: a window or a chunk size, not both");
  QRT_CHECK(a.softcap >= 0.f, "attention: negative score cap");
  QRT_CHECK(a.keep_first >= 0 && (a.keep_first == 0 || a.window > 0), "attention: first keys are kept beside a window");
  QRT_CHECK(a.nq <= 65535, "attention: too many heads");
  if (a.num_tokens == 0) return 0;
  dim3 grid(a.num_tokens, a.nq), block(64);
  if (dtype == QRT_F32) attention_f32_kernel<float><<<grid, block, 0, stream>>>(a);
  else if (dtype == QRT_BF16) attention_f32_kernel<bf16_t><<<grid, block, 0, stream>>>(a);
  else return qrt_fail("attention: unknown dtype %d", dtype);
  QRT_LAUNCH_CHECK("attention_f32");
  return 0;
}
