// Retention: the recurrence of linear attention with a constant decay per head, float32.
//
//   S <- decay_h S + k v^T;   o = S^T q          (S [dim, vdim] per sequence and head)
//
// over each sequence's tokens of the step, from the state in the sequence's slot, which is left
// there for the next step: [slots, heads, vdim, dim], a value channel's column of S contiguous.
// q, k, v come as float32 [T, 2 heads dim + heads vdim] (queries, keys, values; rotated and
// scaled by whoever made them). A block of 256 threads owns 16 columns of one head's state for
// one sequence; 16 neighbouring lanes share a column, each holding its rows in registers four
// neighbours at a time (rows 4 (lane + 16 g) .. + 3 of group g), so that state, keys and queries
// move 16 bytes a lane and the sum over rows that a read-out needs ends in a DPP sum inside a row
// of 16 lanes. Tokens are staged through LDS 16 at a time; the next tile's global loads are in
// flight while a tile is walked, the walk has no global access and no branch between tokens, and
// the tile's read-outs leave together afterwards. The order of the float32 operations per token
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

#define RT_COLS 16   // columns of the state per block

// the sum over the 16 lanes of a row (every lane gets it)
__device__ __forceinline__ float row16_sum(float x) {
  int v = __builtin_bit_cast(int, x);
  x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xF, 0xF, true));   // quad_perm [1,0,3,2]
  v = __builtin_bit_cast(int, x);
  x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xF, 0xF, true));   // quad_perm [2,3,0,1]
  v = __builtin_bit_cast(int, x);
  x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, v, 0x141, 0xF, 0xF, true));  // row_half_mirror
  v = __builtin_bit_cast(int, x);
  x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, v, 0x140, 0xF, 0xF, true));  // row_mirror
  return x;
}

// G groups of four rows a lane: heads of up to 64 G key elements (padded with zero rows). RT_TILE
// tokens a tile: 16 (8 for the widest heads: what fits 64 KB), or 4 for steps of single tokens,
// whose blocks then are all resident at once with a quarter of the LDS and of the loads.
template <int G, int RT_TILE>
__global__ __launch_bounds__(256) void retention_kernel(RetentionArgs a) {
  constexpr int DP = 64 * G;                          // rows staged
  constexpr int NQK = 2 * RT_TILE * DP / 256;         // q and k elements a thread fetches per tile
  __shared__ __attribute__((aligned(16))) float qs[RT_TILE * DP];
  __shared__ __attribute__((aligned(16))) float ks[RT_TILE * DP];
  __shared__ float vs[RT_TILE * RT_COLS];
  __shared__ float os[RT_TILE * RT_COLS];
  const int seq = blockIdx.x, head = blockIdx.y, col0 = blockIdx.z * RT_COLS;
  const int t0 = a.cu_q[seq], t1 = a.cu_q[seq + 1];
  if (t1 <= t0) return;
  const int dim = a.dim, vdim = a.vdim;
  const int sub = threadIdx.x & 15, colg = threadIdx.x >> 4;  // lane within its column, column of the block
  const int col = col0 + colg;
  const bool col_ok = col < vdim;
  const float decay = a.decay[head];
  float* st = a.state + (((size_t)a.state_slots[seq] * a.heads + head) * vdim + min(col, vdim - 1)) * dim;
  const bool vec = (dim & 3) == 0;  // a lane's four rows are 16 aligned bytes of the column
  float s[G][4];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    const int d = 4 * (sub + 16 * g);
    if (vec && d < dim && col_ok) {
      const float4 x = *(const float4*)(st + d);
      s[g][0] = x.x; s[g][1] = x.y; s[g][2] = x.z; s[g][3] = x.w;
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) s[g][j] = (d + j < dim && col_ok) ? st[d + j] : 0.f;
    }
  }
  // what this thread fetches of a tile: elements threadIdx.x + 256 i of q | k ([which][token][row]), one of v
  float pre[NQK], pre_v;
  auto fetch = [&](int base) {
    const int n = min(RT_TILE, t1 - base);
#pragma unroll
    for (int i = 0; i < NQK; ++i) {
      const int e = threadIdx.x + 256 * i;
      const int which = e / (RT_TILE * DP), tok = (e / DP) % RT_TILE, d = e % DP;
      const bool ok = tok < n && d < dim;
      const float* row = a.qkv + (size_t)(base + min(tok, n - 1)) * a.channels + (which ? a.k_first : a.q_first) + head * dim;
      pre[i] = ok ? row[d] : 0.f;
    }
    const int tok = min((int)threadIdx.x / RT_COLS, RT_TILE - 1), c = threadIdx.x % RT_COLS;
    pre_v = (tok < n && col0 + c < vdim) ? a.qkv[(size_t)(base + tok) * a.channels + a.v_first + head * vdim + col0 + c] : 0.f;
  };
  fetch(t0);
  for (int base = t0; base < t1; base += RT_TILE) {
    const int n = min(RT_TILE, t1 - base);
    __syncthreads();  // the tile before has been walked and its read-outs have left
#pragma unroll
    for (int i = 0; i < NQK; ++i) {
      const int e = threadIdx.x + 256 * i;
      if (e < RT_TILE * DP) qs[e] = pre[i];
      else ks[e - RT_TILE * DP] = pre[i];
    }
    if (threadIdx.x < RT_TILE * RT_COLS) vs[threadIdx.x] = pre_v;
    __syncthreads();
    if (base + RT_TILE < t1) fetch(base + RT_TILE);  // on its way during the walk
    if (n == RT_TILE) {
#pragma unroll 4
      for (int i = 0; i < RT_TILE; ++i) {
        const float v = vs[i * RT_COLS + colg];
        float acc = 0.f;
#pragma unroll
        for (int g = 0; g < G; ++g) {
          const float4 kd = *(const float4*)(ks + i * DP + 4 * (sub + 16 * g));
          const float4 qd = *(const float4*)(qs + i * DP + 4 * (sub + 16 * g));
          s[g][0] = fmaf(decay, s[g][0], kd.x * v); acc = fmaf(s[g][0], qd.x, acc);
          s[g][1] = fmaf(decay, s[g][1], kd.y * v); acc = fmaf(s[g][1], qd.y, acc);
          s[g][2] = fmaf(decay, s[g][2], kd.z * v); acc = fmaf(s[g][2], qd.z, acc);
          s[g][3] = fmaf(decay, s[g][3], kd.w * v); acc = fmaf(s[g][3], qd.w, acc);
        }
        acc = row16_sum(acc);
        if (sub == 0) os[i * RT_COLS + colg] = acc;
      }
    } else {
      for (int i = 0; i < n; ++i) {
        const float v = vs[i * RT_COLS + colg];
        float acc = 0.f;
#pragma unroll
        for (int g = 0; g < G; ++g) {
          const float4 kd = *(const float4*)(ks + i * DP + 4 * (sub + 16 * g));
          const float4 qd = *(const float4*)(qs + i * DP + 4 * (sub + 16 * g));
          s[g][0] = fmaf(decay, s[g][0], kd.x * v); acc = fmaf(s[g][0], qd.x, acc);
          s[g][1] = fmaf(decay, s[g][1], kd.y * v); acc = fmaf(s[g][1], qd.y, acc);
          s[g][2] = fmaf(decay, s[g][2], kd.z * v); acc = fmaf(s[g][2], qd.z, acc);
          s[g][3] = fmaf(decay, s[g][3], kd.w * v); acc = fmaf(s[g][3], qd.w, acc);
        }
        acc = row16_sum(acc);
        if (sub == 0) os[i * RT_COLS + colg] = acc;
      }
    }
    __syncthreads();
    {  // the tile's read-outs: thread (token, column)
      const int tok = threadIdx.x / RT_COLS, c = threadIdx.x % RT_COLS;
      if (tok < n && tok < RT_TILE && col0 + c < vdim) a.out[((size_t)(base + tok) * a.heads + head) * vdim + col0 + c] = os[threadIdx.x];
    }
  }
  if (col_ok) {
#pragma unroll
    for (int g = 0; g < G; ++g) {
      const int d = 4 * (sub + 16 * g);
      if (vec && d < dim) {
        *(float4*)(st + d) = make_float4(s[g][0], s[g][1], s[g][2], s[g][3]);
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j)
          if (d + j < dim) st[d + j] = s[g][j];
      }
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
  const int groups = (a.dim + 63) / 64;
  if (num_tokens <= 2 * num_seqs) {  // decoded tokens, mostly
    if (groups <= 1) retention_kernel<1, 4><<<grid, 256, 0, stream>>>(a);
    else if (groups <= 2) retention_kernel<2, 4><<<grid, 256, 0, stream>>>(a);
    else if (groups <= 4) retention_kernel<4, 4><<<grid, 256, 0, stream>>>(a);
    else retention_kernel<8, 4><<<grid, 256, 0, stream>>>(a);
  } else if (groups <= 1) retention_kernel<1, 16><<<grid, 256, 0, stream>>>(a);
  else if (groups <= 2) retention_kernel<2, 16><<<grid, 256, 0, stream>>>(a);
  else if (groups <= 4) retention_kernel<4, 16><<<grid, 256, 0, stream>>>(a);
  else retention_kernel<8, 8><<<grid, 256, 0, stream>>>(a);
  QRT_LAUNCH_CHECK("retention");
  return 0;
}
