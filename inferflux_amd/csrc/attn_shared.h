// What the matrix-core attention kernels share: operand vector types, the exponent, reductions over the four
// lanes that hold one query column, and the merge of split key ranges.
#pragma once
#include "common.h"

#ifndef HEAD_DIM
#error "compile with -DHEAD_DIM=<multiple of 16>"
#endif
constexpr int D = HEAD_DIM;
constexpr int KS = (D + 31) / 32;  // 32-wide steps of the QK product (the last one half empty when D % 32 == 16)
constexpr int DT = D / 16;         // 16-wide tiles of the output's head dimension


typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

__device__ __forceinline__ bf16x8 zero8() {
  bf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = (__bf16)0.f;
  return z;
}

__device__ __forceinline__ bf16x8 join4(bf16x4 a, bf16x4 b) {
  bf16x8 r;
#pragma unroll
  for (int i = 0; i < 4; ++i) { r[i] = a[i]; r[i + 4] = b[i]; }
  return r;
}

__device__ __forceinline__ bf16x4 zero4() {
  bf16x4 z;
#pragma unroll
  for (int i = 0; i < 4; ++i) z[i] = (__bf16)0.f;
  return z;
}

// 2^x on the hardware's exponent unit.  Arguments are <= 0 here and results below the smallest
// normal float may flush to zero, which a softmax weight of that size may.
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// The four lanes that hold the same query column are lane, lane^16, lane^32, lane^48: one lane of each
// row of 16.  gfx950 exchanges rows between two registers in one VALU instruction (permlane16_swap: odd
// rows of the first with even rows of the second; permlane32_swap: rows 2, 3 of the first with rows 0, 1
// of the second); given the same value twice, the two results hold v and v from the partner lane.
__device__ __forceinline__ void swap16(float v, float& a, float& b) {
  const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  a = __uint_as_float(r[0]); b = __uint_as_float(r[1]);
}
__device__ __forceinline__ void swap32(float v, float& a, float& b) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  a = __uint_as_float(r[0]); b = __uint_as_float(r[1]);
}
__device__ __forceinline__ float col_max(float v) {
  float a, b;
  swap16(v, a, b); v = fmaxf(a, b);
  swap32(v, a, b); return fmaxf(a, b);
}
__device__ __forceinline__ float col_sum(float v) {
  float a, b;
  swap16(v, a, b); v = a + b;
  swap32(v, a, b); return a + b;
}

// =======================================================================================
// split key ranges: partial results and their merge
// =======================================================================================
struct RowArgs {
  const bf16_t* q;        // [T, nH, D]
  const bf16_t* k_cache;  // [pages, nKV, P, D]
  const bf16_t* v_cache;  // [pages, nKV, D, P]
  const int* rows;        // [n_rows] rows of the batch this launch handles (nullptr: rows 0..n_rows-1)
  const int* row_req;     // [T]
  const int* positions;   // [T]
  const int* block_table; // [R, max_blocks], -1 where no page
  float* part_o;          // [n_rows, nH, max_splits, D]
  float* part_ml;         // [n_rows, nH, max_splits, 2]
  bf16_t* out;            // [T, nH * D]
  int max_blocks, n_rows, nH, nKV, P, window, chunk, max_splits;
  float scale_log2e;
  int part_by_row;        // partial results lie at the batch row's number (the tile kernel's), not at its place in ``rows``
  int waves;              // the row kernel that takes a (row, kv head) whole: waves per workgroup
  int req_is_row;         // row_req[r] == r for every row (a step of single tokens): table lookups need not wait for it
};

// out[row, head] = sum_s 2^(m_s - M) O_s / sum_s 2^(m_s - M) l_s over the row's splits, M = max m_s.
// One workgroup per (row, head).  A wave takes a run of consecutive splits: lane s first weighs split s of the run,
// then every lane sums its elements over the run's splits in ascending order.  The partial results of the first
// MERGE_EARLY splits of a run are asked for together with the maxima and sums, before their weights are known (a
// kernel this short is a chain of trips to the L2: maxima, then weights, then the partial results cost three; so it
// is one for runs of up to 32 splits).  Rows of up to MERGE_RUN splits are one wave's; longer rows (one request over
// tens of thousands of keys: hundreds of splits, which a single wave would walk for 25-50 us) are shared by up to
// MERGE_MAX_WAVES waves, whose results meet in LDS and are added in wave order.
constexpr int MERGE_EARLY = 32, MERGE_RUN = 32, MERGE_MAX_WAVES = 8;

// Waves per workgroup of the merge launch for rows of up to ``max_splits`` splits.
static inline int merge_waves(int max_splits) {
  const int w = (max_splits + MERGE_RUN - 1) / MERGE_RUN;
  return w < 1 ? 1 : (w > MERGE_MAX_WAVES ? MERGE_MAX_WAVES : w);
}

__global__ __launch_bounds__(WAVE * MERGE_MAX_WAVES) void attn_rows_merge_kernel(RowArgs a) {
  constexpr int C = (D + WAVE - 1) / WAVE;
  __shared__ float ml_w[MERGE_MAX_WAVES][2];
  __shared__ float acc_w[MERGE_MAX_WAVES][C * WAVE];
  const int ri = blockIdx.x, head = blockIdx.y, lane = threadIdx.x % WAVE, wid = threadIdx.x / WAVE, nw = blockDim.x / WAVE;
  const int row = a.rows ? a.rows[ri] : ri;
  const int pos = a.positions[row];
  const int lo = a.window > 0 ? max(0, pos - a.window + 1) : 0;
  const int first = lo / a.chunk, last = pos / a.chunk;  // first and last split that hold a visible key
  // this wave's run of them: runs of MERGE_RUN, longer ones only for rows that MERGE_MAX_WAVES such runs do not cover.
  // How a row is cut depends on the row alone, not on how many waves the launch has (it has enough: merge_waves), so
  // a row's result is the same bits in every launch that holds it.
  const int n_splits = last - first + 1;
  const int per = max(MERGE_RUN, (n_splits + MERGE_MAX_WAVES - 1) / MERGE_MAX_WAVES);
  const int s0 = first + wid * per, s1 = min(last, s0 + per - 1);
  const size_t pi = a.part_by_row ? row : ri;
  const float* po = a.part_o + (pi * a.nH + head) * a.max_splits * D;
  const float* pml = a.part_ml + (pi * a.nH + head) * a.max_splits * 2;
  float acc[C];
#pragma unroll
  for (int c = 0; c < C; ++c) acc[c] = 0.f;
  float L = 0.f, M = -INFINITY;
  if (s0 <= s1) {
    // Lane s of a round holds split sb + s; runs of more than 64 splits take further rounds.  The first
    // round's maxima and sums are kept from the pass that finds the maximum (the usual case is one round).
    const int n_first = min(WAVE, s1 - s0 + 1);
    const float2 ml_first = lane < n_first ? *(const float2*)(pml + 2 * (s0 + lane)) : float2{-INFINITY, 0.f};
    // A split that saw no key has weight 0 and its partial result may hold anything: what was read of it is
    // dropped by a select below, never multiplied.
    float early[MERGE_EARLY][C];
#pragma unroll
    for (int u = 0; u < MERGE_EARLY; ++u)
#pragma unroll
      for (int c = 0; c < C; ++c) {
        const int e = lane + c * WAVE;
        early[u][c] = (u < n_first && e < D) ? po[(size_t)(s0 + u) * D + e] : 0.f;
      }
    M = ml_first.x;
    for (int sb = s0 + WAVE; sb <= s1; sb += WAVE) {
      const int s = sb + lane;
      M = fmaxf(M, s <= s1 ? pml[2 * s] : -INFINITY);
    }
    M = wave_max(M);
    for (int sb = s0; sb <= s1; sb += WAVE) {
      const int s = sb + lane;
      float ms = ml_first.x, ls = ml_first.y;
      if (sb != s0) {
        const float2 ml = s <= s1 ? *(const float2*)(pml + 2 * s) : float2{-INFINITY, 0.f};
        ms = ml.x; ls = ml.y;
      }
      const float w = ms == -INFINITY ? 0.f : exp2f(ms - M);   // lane u's is the weight of split sb + u
      L += w * ls;
      const int n = min(WAVE, s1 - sb + 1);
      int i = 0;
      if (sb == s0) {
#pragma unroll
        for (int u = 0; u < MERGE_EARLY; ++u) {
          const float wu = u < n ? __shfl(w, u, WAVE) : 0.f;
#pragma unroll
          for (int c = 0; c < C; ++c) acc[c] = fmaf(wu, wu != 0.f ? early[u][c] : 0.f, acc[c]);
        }
        i = MERGE_EARLY;
      }
      // the rest sixteen splits at a time, so that their loads are in flight together
      for (; i < n; i += 16) {
        float wi[16], val[16][C];
#pragma unroll
        for (int u = 0; u < 16; ++u) {
          wi[u] = __shfl(w, min(i + u, WAVE - 1), WAVE);
          if (i + u >= n) wi[u] = 0.f;
#pragma unroll
          for (int c = 0; c < C; ++c) {
            const int e = lane + c * WAVE;
            val[u][c] = (wi[u] != 0.f && e < D) ? po[(size_t)(sb + i + u) * D + e] : 0.f;
          }
        }
#pragma unroll
        for (int u = 0; u < 16; ++u)
#pragma unroll
          for (int c = 0; c < C; ++c) acc[c] = fmaf(wi[u], val[u][c], acc[c]);
      }
    }
    L = wave_sum(L);
  }
  if (nw > 1) {   // the waves' results, relative to their own maxima, are added in wave order by the first
    if (lane == 0) { ml_w[wid][0] = M; ml_w[wid][1] = L; }
#pragma unroll
    for (int c = 0; c < C; ++c) acc_w[wid][lane + c * WAVE] = acc[c];
    __syncthreads();
    if (wid > 0) return;
    float Mall = -INFINITY;
    for (int w = 0; w < nw; ++w) Mall = fmaxf(Mall, ml_w[w][0]);
    L = 0.f;
#pragma unroll
    for (int c = 0; c < C; ++c) acc[c] = 0.f;
    for (int w = 0; w < nw; ++w) {
      const float mw = ml_w[w][0];
      if (mw == -INFINITY) continue;
      const float f = exp2f(mw - Mall);
      L = fmaf(f, ml_w[w][1], L);
#pragma unroll
      for (int c = 0; c < C; ++c) acc[c] = fmaf(f, acc_w[w][lane + c * WAVE], acc[c]);
    }
  }
  const float inv = L > 0.f ? 1.f / L : 0.f;
#pragma unroll
  for (int c = 0; c < C; ++c) {
    const int e = lane + c * WAVE;
    if (e < D) a.out[((size_t)row * a.nH + head) * D + e] = (bf16_t)(acc[c] * inv);
  }
}
