// Retention: the recurrence of linear attention with a constant decay per head, float32.
//
//   S <- decay_h S + k v^T;   o = S^T q          (S [dim, vdim] per sequence and head)
//
// over each sequence's tokens of the step, from the state in the sequence's slot, which is left
// there for the next step: [slots, heads, vdim, dim], a value channel's column of S contiguous.
// q, k, v come as float32 [T, 2 heads dim + heads vdim] (queries, keys, values; rotated and
// scaled by whoever made them). A block of 256 threads owns 16 columns of one head's state for
// one sequence; 16 neighbouring lanes share a column, each holding rows lane, lane + 16, ... in
// registers, so the sum over rows that a read-out needs ends in a sum over a row of 16 lanes.
// Tokens are staged through LDS 16 at a time. The order of the float32 operations per token
// does not depend on how the tokens are cut into steps, tiles or batches.
#include "common.h"
#include <math.h>

struct RetentionArgs {
  const float* qkv; int channels, q_first, k_first, v_first;
  const float* decay;     // [heads]
  float* state;           // [slots, heads, vdim, dim]
  float* out;             // [T, heads, vdim]
  const int* cu_q; const int* state_slots;
  int heads, dim, vdim;
};

#define RT_TILE 16   // tokens per LDS tile
#define RT_COLS 16   // columns of the state per block

template <int R>
__global__ __launch_bounds__(256) void retention_kernel(RetentionArgs a) {
  extern __shared__ float lds[];
  const int seq = blockIdx.x, head = blockIdx.y, col0 = blockIdx.z * RT_COLS;
  const int t0 = a.cu_q[seq], t1 = a.cu_q[seq + 1];
  if (t1 <= t0) return;
  const int dim = a.dim, vdim = a.vdim;
  const int sub = threadIdx.x & 15, colg = threadIdx.x >> 4;  // lane within its column, column of the block
  const int col = col0 + colg;
  const bool col_ok = col < vdim;
  float* qs = lds;                       // [RT_TILE][dim]
  float* ks = qs + RT_TILE * dim;        // [RT_TILE][dim]
  float* vs = ks + RT_TILE * dim;        // [RT_TILE][RT_COLS]
  const float decay = a.decay[head];
  float* st = a.state + (((size_t)a.state_slots[seq] * a.heads + head) * vdim + min(col, vdim - 1)) * dim;
  float s[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int d = sub + 16 * r;
    s[r] = (d < dim && col_ok) ? st[d] : 0.f;
  }
  for (int base = t0; base < t1; base += RT_TILE) {
    const int n = min(RT_TILE, t1 - base);
    __syncthreads();
    for (int e = threadIdx.x; e < n * dim; e += 256) {
      const int i = e / dim, d = e - i * dim;
      const float* row = a.qkv + (size_t)(base + i) * a.channels;
      qs[e] = row[a.q_first + head * dim + d];
      ks[e] = row[a.k_first + head * dim + d];
    }
    for (int e = threadIdx.x; e < n * RT_COLS; e += 256) {
      const int i = e / RT_COLS, c = e - i * RT_COLS;
      vs[e] = col0 + c < vdim ? a.qkv[(size_t)(base + i) * a.channels + a.v_first + head * vdim + col0 + c] : 0.f;
    }
    __syncthreads();
    for (int i = 0; i < n; ++i) {
      const float v = vs[i * RT_COLS + colg];
      float acc = 0.f;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const int d = sub + 16 * r;
        const float kd = d < dim ? ks[i * dim + d] : 0.f;
        const float qd = d < dim ? qs[i * dim + d] : 0.f;
        s[r] = fmaf(decay, s[r], kd * v);
        acc = fmaf(s[r], qd, acc);
      }
      acc += __shfl_xor(acc, 8, 64);
      acc += __shfl_xor(acc, 4, 64);
      acc += __shfl_xor(acc, 2, 64);
      acc += __shfl_xor(acc, 1, 64);
      if (sub == 0 && col_ok) a.out[((size_t)(base + i) * a.heads + head) * vdim + col] = acc;
    }
  }
  if (col_ok) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int d = sub + 16 * r;
      if (d < dim) st[d] = s[r];
    }
  }
}

extern "C" int qrt_retention(const RetentionArgs* args, int num_tokens, int num_seqs, int num_slots, hipStream_t stream) {
  RetentionArgs a = *args;
  QRT_CHECK(num_tokens >= 0 && num_seqs >= 0 && num_slots > 0, "retention: bad counts");
  QRT_CHECK(a.heads > 0 && a.heads <= 65535 && a.dim > 0 && a.dim <= 512 && a.vdim > 0, "retention: %d heads of %d x %d", a.heads, a.dim, a.vdim);
  QRT_CHECK(a.channels >= 2 * a.heads * a.dim + a.heads * a.vdim, "retention: %d channels hold no q, k and v", a.channels);
  if (num_tokens == 0 || num_seqs == 0) return 0;
  const dim3 grid(num_seqs, a.heads, (a.vdim + RT_COLS - 1) / RT_COLS);
  const size_t lds = (size_t)(2 * RT_TILE * a.dim + RT_TILE * RT_COLS) * sizeof(float);
  const int rows = (a.dim + 15) / 16;
  if (rows <= 2) retention_kernel<2><<<grid, 256, lds, stream>>>(a);
  else if (rows <= 4) retention_kernel<4><<<grid, 256, lds, stream>>>(a);
  else if (rows <= 8) retention_kernel<8><<<grid, 256, lds, stream>>>(a);
  else if (rows <= 16) retention_kernel<16><<<grid, 256, lds, stream>>>(a);
  else retention_kernel<32><<<grid, 256, lds, stream>>>(a);
  QRT_LAUNCH_CHECK("retention");
  return 0;
}
