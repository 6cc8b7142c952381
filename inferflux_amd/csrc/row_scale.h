// A norm's factor per row, applied by the matrix product that follows the norm to its sums instead of to its input
// (shared by the weight-streaming products of gemm_bf16.hip and gemm_wide.hip).
#pragma once
#include "common.h"

typedef __attribute__((__vector_size__(4 * sizeof(float)))) float rs_floatx4;

// A normalisation whose factor per row is applied to the product's results instead of to its input:
// row m of x stands for x[m] * rsqrt(sum_j pieces[j][m] / width + eps).  ``pieces`` is [n][16]
// (16 rows whatever M is): piece j is the sum of squares of a run of consecutive elements of the row before it was
// weighted (runs of 16 from the stream epilogue of gemm_bf16.hip, longer ones from the embedding kernel).
struct RowScale {
  const float* pieces;  // null: no factor
  int n;
  float width, eps;
};

// The factor of row lane % 16, computed by one wave.  The pieces are read as float4s (rows 4 (c % 4) ... + 3 of
// piece c / 4 in float4 number c), lane l taking numbers l, l + 64, ...: sixteen loads are in flight at a time
// (one after the other they would cost a trip to the L2 each), a lane always meets the same four rows, and the
// sums are added in a fixed order.
__device__ __forceinline__ float row_factor(const RowScale& s, int lane) {
  const int chunks = 4 * s.n;
  rs_floatx4 t{0.f, 0.f, 0.f, 0.f};
  for (int base = lane; base < chunks; base += WAVE * 16) {
    rs_floatx4 v[16];
#pragma unroll
    for (int u = 0; u < 16; ++u) {
      const int c = base + WAVE * u;
      v[u] = c < chunks ? *(const rs_floatx4*)(s.pieces + (size_t)4 * c) : rs_floatx4{0.f, 0.f, 0.f, 0.f};
    }
#pragma unroll
    for (int u = 0; u < 16; ++u)
#pragma unroll
      for (int r = 0; r < 4; ++r) t[r] += v[u][r];
  }
#pragma unroll
  for (int off = 4; off < WAVE; off <<= 1)
#pragma unroll
    for (int r = 0; r < 4; ++r) t[r] += __shfl_xor(t[r], off);
  // every lane with lane % 4 == q now holds the sums of rows 4 q ... 4 q + 3
  const int col = lane & 15;
  float sum = 0.f;
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const float from = __shfl(t[r], col >> 2);
    if ((col & 3) == r) sum = from;
  }
  return rsqrtf(sum / s.width + s.eps);
}

// The same sums gathered by a whole workgroup of ``threads`` threads (a multiple of 64): thread ``tid`` takes float4
// numbers tid, tid + threads, ... (a thread always meets the same four rows).  row_sums_ask asks for the thread's first
// four, to be called before the kernel's own first loads so that the pieces arrive ahead of them and cost no trip of
// their own; row_sums_of_thread adds them up (and fetches what lies beyond four a thread, a stream wider than any
// model's); row_sums_of_wave leaves, in lanes 0-3 of each wave, the wave's share of the sums of rows 4 lane ... 4 lane + 3.
// The caller puts the shares into LDS, adds them in wave order and takes rsqrt(sum / width + eps).
struct RowSumsEarly {
  rs_floatx4 v[4];
};
__device__ __forceinline__ void row_sums_ask(const RowScale& s, int tid, int threads, RowSumsEarly& e) {
  const int chunks = 4 * s.n;
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const int c = tid + threads * u;
    e.v[u] = c < chunks ? *(const rs_floatx4*)(s.pieces + (size_t)4 * c) : rs_floatx4{0.f, 0.f, 0.f, 0.f};
  }
}
__device__ __forceinline__ rs_floatx4 row_sums_of_thread(const RowScale& s, int tid, int threads, const RowSumsEarly& e) {
  const int chunks = 4 * s.n;
  rs_floatx4 t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int u = 0; u < 4; ++u)
#pragma unroll
    for (int r = 0; r < 4; ++r) t[r] += e.v[u][r];
  for (int c = tid + 4 * threads; c < chunks; c += threads) {
    const rs_floatx4 v = *(const rs_floatx4*)(s.pieces + (size_t)4 * c);
#pragma unroll
    for (int r = 0; r < 4; ++r) t[r] += v[r];
  }
  return t;
}
__device__ __forceinline__ rs_floatx4 row_sums_of_wave(rs_floatx4 t) {
#pragma unroll
  for (int off = 4; off < WAVE; off <<= 1)
#pragma unroll
    for (int r = 0; r < 4; ++r) t[r] += __shfl_xor(t[r], off);
  return t;
}
