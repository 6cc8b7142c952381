// Weight-streaming matrix product for few rows:  out[M,N] = x[M,K] * W[N,K]^T,  M <= 64,
// bf16 in, float accumulate on the matrix cores (16x16x32), out bf16 or float.
//
// At decode sizes the product is bound by reading W once from HBM, so the kernel is built around
// that stream: a wave owns NT tiles of 16 weight rows and walks K in blocks of 64; each lane reads
// 32 contiguous bytes of a row per block (four lanes cover one 128-byte line), which serve two
// MFMA steps.  Which 8 k-values a lane group feeds to which MFMA step does not matter for a sum
// over k as long as x is read with the same rule, so x is read the same way (from L2: it is
// small and shared by every workgroup).  The waves of a workgroup split K round-robin and add
// their accumulators through LDS in a fixed order, so the result does not depend on timing.
// U blocks are loaded before the first is consumed, to keep enough bytes in flight.
//
// The weight may also come pre-tiled for exactly this walk (TILED): tile (t, kt) holds the 16 rows
// 16 t .. 16 t + 15 at k = 32 kt .. 32 kt + 31 as 64 pieces of 16 bytes, piece 16 g + col = row
// 16 t + col at k = 32 kt + 8 g; tiles follow each other along k, then along t, and the tensor is
// padded with zeros to whole tiles and to an even number of tiles along k.  A wave's load then
// covers 1 KB of contiguous memory instead of 16 half-used lines, and x is read in runs of 64
// contiguous bytes per row; measured on 7B shapes this takes 15-25 % off the time.
//
// The reference sends these products to cuBLAS (runtime/backends/cuda/native/cublas_gemm.cpp:
// 99-117) and measured 30-44 % of its roofline there (docs/benchmarks.md:180-183).
#include "common.h"
#include "row_scale.h"

IFX_DEFINE_LAST_ERROR()

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

constexpr int UNITS = 256;   // compute units of the chip that the launch plans below are measured on

__device__ __forceinline__ bf16x8 zero8() {
  bf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = (__bf16)0.f;
  return z;
}

// EPI 2: the product is added to the float stream [M, N] in place, and what the norm that follows needs is
// written beside it: rows[m, n] = bf16(stream[m, n] * norm_w[n]) and pieces[n / 16][m] (see RowScale).
struct StreamOut {
  float* stream;
  const bf16_t* norm_w;
  bf16_t* rows;
  float* pieces;
};

// Sum over the four lanes col, col + 16, col + 32, col + 48, the same in all four.
__device__ __forceinline__ float sum_over_groups(float v) {
  v += __shfl_xor(v, 16);
  v += __shfl_xor(v, 32);
  return v;
}

// The sums of one workgroup: acc[nt][mt] = W tile (first_tile + nt) times x rows 16 mt ..., K split over
// the workgroup's waves and added through LDS in wave order.  Returns true in the wave that holds the
// sums (wave 0); the others are done.
template <int MT, int NT, int U, bool TILED>
__device__ __forceinline__ bool skinny_accumulate(const bf16_t* __restrict__ x, const bf16_t* __restrict__ W, int M, int N,
                                                  int K, int k_tiles, int first_tile, floatx4 (&acc)[NT][MT], float* red,
                                                  int tile_rows = 16) {
  const int wid = threadIdx.x / WAVE, nw = blockDim.x / WAVE, lane = threadIdx.x % WAVE;
  const int col = lane & 15, g = lane >> 4;
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[nt][mt] = floatx4{0.f, 0.f, 0.f, 0.f};

  const bf16_t* wrow[NT];  // rows (tiles) past N are read again, never stored
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
    wrow[nt] = TILED ? W + ((size_t)min(first_tile + nt, (N - 1) / tile_rows) * k_tiles * 4 * tile_rows + tile_rows * g + col) * 8
                     : W + (size_t)min(16 * (first_tile + nt) + col, N - 1) * K;
  const bool row_held = !TILED || col < tile_rows;   // a tile of the copy holds tile_rows rows: the other lanes' rows are zeros
  const bf16_t* xrow[MT];
  bool xok[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    xok[mt] = 16 * mt + col < M;
    xrow[mt] = x + (size_t)(xok[mt] ? 16 * mt + col : 0) * K;
  }

  const int nkb = (K + 63) / 64;
  for (int kb0 = wid * U; kb0 < nkb; kb0 += nw * U) {
    bf16x8 wa[U][NT][2], xa[U][MT][2];
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        // the lane's 8 k-values of step h of block kb0 + u, and where its piece of W lies
        const int k = TILED ? (kb0 + u) * 64 + 32 * h + 8 * g : (kb0 + u) * 64 + 16 * g + 8 * h;
        const size_t w_off = TILED ? (size_t)(2 * (kb0 + u) + h) * 4 * tile_rows * 8 : (size_t)k;
        const bool blk = kb0 + u < nkb && row_held, kok = kb0 + u < nkb && k < K;
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
          // Tiles are read once, in whole lines: a streaming load keeps them from pushing x out of the L2.
          // (Rows are read in half lines by two loads; there the hint costs more than it gives.)
          const bf16x8* wp = (const bf16x8*)(wrow[nt] + w_off);
          wa[u][nt][h] = TILED ? (blk ? __builtin_nontemporal_load(wp) : zero8()) : (kok ? *wp : zero8());
        }
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) xa[u][mt][h] = (kok && xok[mt]) ? *(const bf16x8*)(xrow[mt] + k) : zero8();
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
            acc[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa[u][nt][h], xa[u][mt][h], acc[nt][mt], 0, 0, 0);
  }

  if (nw > 1) {
    if (wid > 0) {
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          *(floatx4*)(red + ((size_t)((wid - 1) * NT * MT + nt * MT + mt) * WAVE + lane) * 4) = acc[nt][mt];
    }
    __syncthreads();
    if (wid > 0) return false;
    for (int w = 1; w < nw; ++w)
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          const floatx4 o = *(const floatx4*)(red + ((size_t)((w - 1) * NT * MT + nt * MT + mt) * WAVE + lane) * 4);
#pragma unroll
          for (int r = 0; r < 4; ++r) acc[nt][mt][r] += o[r];
        }
  }
  return true;
}

// EPI 0: out[m, n] = acc.  EPI 1: the rows of W alternate gate, up, gate, up ...; a lane holds two
// such pairs of one output row and writes silu(gate) * up to out[m, n / 2] (out is [M, N / 2]).
// EPI 2 (up to 16 rows, N a multiple of 4): see StreamOut; ``out`` is not used.
// ``order`` (tiled copies only): tile t of the copy holds the weight's rows 16 order[t] ...; null: in order.
// ``scale`` (up to 16 rows): the results of row m are multiplied by the row's factor first.
typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4;
typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2;
typedef __attribute__((__vector_size__(2 * sizeof(float)))) float floatx2;

template <int MT, int NT, int U, typename TO, int EPI, bool TILED>
__global__ void skinny_gemm_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ W, TO* __restrict__ out,
                                   int M, int N, int K, int k_tiles, const int* __restrict__ order, RowScale scale,
                                   StreamOut so, int tile_rows) {
  extern __shared__ float red[];  // [(waves - 1)][NT * MT][64 lanes][4]
  const int lane = threadIdx.x % WAVE, col = lane & 15, g = lane >> 4;
  const int first_tile = blockIdx.x * NT, n_tiles = (N + tile_rows - 1) / tile_rows;
  const bool first_wave = threadIdx.x < WAVE;
  float rs = 1.f;
  if (MT == 1 && scale.pieces && first_wave) rs = row_factor(scale, lane);
  // The lane's four sums of a tile are rows 4 g ... 4 g + 3 of it, handled as two pairs: tile_rows is even, so a
  // pair is held or not as a whole, and a pair's first column is even.
  // EPI 2: what the epilogue reads is asked for before the stream of weights, not after it
  floatx2 was[NT][2];
  bf16x2 nw[NT][2];
  if (EPI == 2 && first_wave) {
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int q = 0; q < 2; ++q) {
        const int n = tile_rows * (first_tile + nt) + 4 * g + 2 * q;
        const bool ok = 4 * g + 2 * q < tile_rows && n < N && col < M;
        was[nt][q] = ok ? *(const floatx2*)(so.stream + (size_t)col * N + n) : floatx2{0.f, 0.f};
        if (ok) nw[nt][q] = *(const bf16x2*)(so.norm_w + n);
      }
  }
  floatx4 acc[NT][MT];
  if (!skinny_accumulate<MT, NT, U, TILED>(x, W, M, N, K, k_tiles, first_tile, acc, red, tile_rows)) return;
  // acc[nt][mt][r] = out[m = 16 mt + col][n = tile_rows (row tile of the weight) + 4 g + r], for 4 g + r < tile_rows
  if (EPI == 2) {
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      if (first_tile + nt >= n_tiles) continue;   // the same for the whole wave
      float sq = 0.f;
#pragma unroll
      for (int q = 0; q < 2; ++q) {
        const int n = tile_rows * (first_tile + nt) + 4 * g + 2 * q;
        if (4 * g + 2 * q < tile_rows && n < N && col < M) {
          floatx2 v;
          bf16x2 y;
#pragma unroll
          for (int r = 0; r < 2; ++r) {
            v[r] = was[nt][q][r] + acc[nt][0][2 * q + r] * rs;
            y[r] = (__bf16)(v[r] * (float)nw[nt][q][r]);
            sq += v[r] * v[r];
          }
          *(floatx2*)(so.stream + (size_t)col * N + n) = v;
          *(bf16x2*)(so.rows + (size_t)col * N + n) = y;
        }
      }
      sq = sum_over_groups(sq);
      if (g == 0) so.pieces[(size_t)(first_tile + nt) * 16 + col] = sq;
    }
    return;
  }
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    if (first_tile + nt >= n_tiles) continue;
    const int n0 = tile_rows * ((TILED && order) ? order[first_tile + nt] : first_tile + nt);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const int m = 16 * mt + col;
      if (m >= M) continue;
      if (EPI == 0) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int n = n0 + 4 * g + r;
          if (4 * g + r < tile_rows && n < N) out[(size_t)m * N + n] = from_f<TO>(acc[nt][mt][r] * rs);
        }
      } else {
#pragma unroll
        for (int r = 0; r < 4; r += 2) {
          const int n = n0 + 4 * g + r;  // even: gate at n, up at n + 1
          const float gt = acc[nt][mt][r] * rs, up = acc[nt][mt][r + 1] * rs;
          if (4 * g + r < tile_rows && n + 1 < N) out[(size_t)m * (N / 2) + n / 2] = from_f<TO>(gt / (1.0f + expf(-gt)) * up);
        }
      }
    }
  }
}

// The q/k/v projection of up to 16 tokens with what follows it as the epilogue: bias, rotation of q and
// k by the token's position (split-half pairs over the whole head), q to q_out, k and v into the paged
// cache at the token's slot.  The tiled copy is ordered so that consecutive tiles hold the two halves of
// 16 rotation pairs: tile 2 w is rows h d + 16 j ... of head h, tile 2 w + 1 rows h d + d/2 + 16 j ...,
// with w = h (d / 32) + j; a lane then holds both elements of its four pairs.  Heads are numbered over
// the concatenated weight: q heads, then k heads, then v heads.
struct QkvArgs {
  const void* bias;       // [(nH + 2 nKV) d] or null
  int bias_dtype;
  const int* slots;       // [M] page * page_size + offset, < 0: nothing is written; null: queries only
  const float* cs;        // [M, d / 2]
  const float* sn;
  bf16_t* q_out;          // [M, nH * d]
  bf16_t* k_cache;        // [pages, nKV, P, d]
  bf16_t* v_cache;        // [pages, nKV, d, P]
  int nH, nKV, d, P;
};

template <int U>
__global__ void qkv_rope_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ W, int M, int N, int K, int k_tiles,
                                QkvArgs a, RowScale scale) {
  extern __shared__ float red[];
  const int lane = threadIdx.x % WAVE, col = lane & 15, g = lane >> 4;
  float rs = 1.f;
  if (scale.pieces && threadIdx.x < WAVE) rs = row_factor(scale, lane);
  floatx4 acc[2][1];
  if (!skinny_accumulate<1, 2, U, true>(x, W, M, N, K, k_tiles, 2 * blockIdx.x, acc, red)) return;
  const int m = col;
  if (m >= M) return;
  const int d = a.d, half = d / 2, per_head = d / 32;
  const int head = blockIdx.x / per_head, i0 = 16 * (blockIdx.x % per_head) + 4 * g;   // the lane's pairs: i0 + r and i0 + r + half
  float x0[4], x1[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    x0[r] = acc[0][0][r] * rs;
    x1[r] = acc[1][0][r] * rs;
    if (a.bias) {
      x0[r] += load_dyn(a.bias, a.bias_dtype, (size_t)head * d + i0 + r);
      x1[r] += load_dyn(a.bias, a.bias_dtype, (size_t)head * d + half + i0 + r);
    }
  }
  const bool is_v = head >= a.nH + a.nKV;
  if (!is_v) {
    const floatx4 cs = *(const floatx4*)(a.cs + (size_t)m * half + i0), sn = *(const floatx4*)(a.sn + (size_t)m * half + i0);
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const float y0 = x0[r] * cs[r] - x1[r] * sn[r], y1 = x0[r] * sn[r] + x1[r] * cs[r];
      x0[r] = y0;
      x1[r] = y1;
    }
  }
  bf16x4 lo, hi;
#pragma unroll
  for (int r = 0; r < 4; ++r) { lo[r] = (__bf16)x0[r]; hi[r] = (__bf16)x1[r]; }
  if (head < a.nH) {
    bf16_t* dst = a.q_out + ((size_t)m * a.nH + head) * d + i0;
    *(bf16x4*)dst = lo;
    *(bf16x4*)(dst + half) = hi;
    return;
  }
  const int slot = a.slots ? a.slots[m] : -1;
  if (slot < 0) return;
  const int page = slot / a.P, off = slot % a.P;
  if (!is_v) {
    bf16_t* dst = a.k_cache + (((size_t)page * a.nKV + (head - a.nH)) * a.P + off) * d + i0;
    *(bf16x4*)dst = lo;
    *(bf16x4*)(dst + half) = hi;
  } else {
    bf16_t* dst = a.v_cache + (((size_t)page * a.nKV + (head - a.nH - a.nKV)) * d + i0) * a.P + off;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      dst[(size_t)r * a.P] = lo[r];
      dst[(size_t)(half + r) * a.P] = hi[r];
    }
  }
}

template <int MT, int NT, int U, bool TILED>
static int launch(const void* x, const void* W, void* out, int out_dtype, int M, int N, int K, int k_tiles, int waves, int epi,
                  const int* order, const RowScale& scale, const StreamOut& so, int tile_rows, hipStream_t s) {
  const int groups = ((N + tile_rows - 1) / tile_rows + NT - 1) / NT;
  const size_t lds = (size_t)(waves - 1) * NT * MT * WAVE * 4 * sizeof(float);
  IFX_REQUIRE(lds <= 64 * 1024, "skinny_gemm: %d waves of %dx%d tiles need %zu bytes of LDS", waves, NT, MT, lds);
#define GO(TO_, EPI_)                                                                                              \
  hipLaunchKernelGGL((skinny_gemm_kernel<MT, NT, U, TO_, EPI_, TILED>), dim3(groups), dim3(waves * WAVE), lds, s,  \
                     (const bf16_t*)x, (const bf16_t*)W, (TO_*)out, M, N, K, k_tiles, order, scale, so, tile_rows)
  if (epi == 2) {
    if constexpr (MT == 1) GO(float, 2);
    else IFX_FAIL("skinny_gemm: the stream epilogue takes at most 16 rows");
  } else if (out_dtype == DT_BF16 && epi == 0) GO(bf16_t, 0);
  else if (out_dtype == DT_BF16) GO(bf16_t, 1);
  else if (epi == 0) GO(float, 0);
  else GO(float, 1);
#undef GO
  IFX_LAUNCH_CHECK();
}

// The tiled form of an [N, K] weight: row tiles of ``tile_rows`` rows (even, 8 to 16; the last one padded with
// zeros), k in whole tiles of 32, an even number of them.  Piece ((t k_tiles + kt) 4 + g) tile_rows + col
// (16 bytes) holds the 8 k-values from 32 kt + 8 g of row tile t's row col: a wave reads a (t, kt) as 64 tile_rows
// contiguous bytes, lane 16 g + col taking that piece (lanes with col >= tile_rows none), which is its share of
// the 16x32 operand of the matrix core, rows past tile_rows being zeros.  Fewer than 16 rows to a tile are for
// weights with so few rows that 16-row tiles would leave compute units without a tile (see ops.choose_tile_rows).
extern "C" int ifx_tiled_rows(int N) { return (N + 15) / 16 * 16; }
extern "C" int ifx_tiled_cols(int K) { return (K + 63) / 64 * 64; }
extern "C" long long ifx_tiled_size(int N, int K, int tile_rows) {   // elements of the copy
  return (long long)((N + tile_rows - 1) / tile_rows) * tile_rows * ifx_tiled_cols(K);
}

__global__ void tile_weights_kernel(const bf16_t* __restrict__ W, bf16_t* __restrict__ Wt, int N, int K, int k_tiles, size_t pieces,
                                    const int* __restrict__ order, int tile_rows) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;   // piece number: ((t * k_tiles + kt) * 4 + g) * tile_rows + col
  if (i >= pieces) return;
  const int col = (int)(i % tile_rows), g = (int)(i / tile_rows % 4);
  const size_t tile = i / (4 * tile_rows);
  const int t = (int)(tile / k_tiles), kt = (int)(tile % k_tiles);
  const int n = (order ? order[t] : t) * tile_rows + col, k = 32 * kt + 8 * g;
  *(bf16x8*)(Wt + i * 8) = (n < N && k < K) ? *(const bf16x8*)(W + (size_t)n * K + k) : zero8();
}

// Wt [ifx_tiled_size(N, K, tile_rows)] = the tiled form of W [N, K] (K a multiple of 8).  ``order``
// [ceil(N / tile_rows)] (or null): row tile t of the copy is row tile order[t] of W (a permutation,
// checked by the caller).
extern "C" int ifx_tile_weights(const void* W, void* Wt, int N, int K, const int* order, int tile_rows, void* stream) {
  IFX_REQUIRE(N > 0 && K > 0 && K % 8 == 0, "tile_weights: N=%d K=%d (K must be a multiple of 8)", N, K);
  IFX_REQUIRE(tile_rows >= 8 && tile_rows <= 16 && tile_rows % 2 == 0, "tile_weights: %d rows to a tile (8 to 16, even)", tile_rows);
  const int k_tiles = ifx_tiled_cols(K) / 32;
  const size_t pieces = (size_t)((N + tile_rows - 1) / tile_rows) * k_tiles * 4 * tile_rows;
  hipLaunchKernelGGL(tile_weights_kernel, dim3((unsigned)((pieces + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                     (const bf16_t*)W, (bf16_t*)Wt, N, K, k_tiles, pieces, order, tile_rows);
  IFX_LAUNCH_CHECK();
}

// The q/k/v projection of M <= 16 tokens from the pair-ordered tiled copy Wt of the concatenated weight
// [(nH + 2 nKV) d, K], with bias, rotation and the cache write as its epilogue (see qkv_rope_kernel).
// With slots null only the nH query heads are projected (the copy then holds those rows only).
// scale_pieces [n_scale_pieces][16] (or null), scale_width, scale_eps: a factor per row of x, see RowScale.
extern "C" int ifx_qkv_rope(const void* x, const void* Wt, int M, int K, const void* bias, int bias_dtype, const int* slots,
                            const float* cs, const float* sn, int nH, int nKV, int d, int page_size, void* q_out,
                            void* k_cache, void* v_cache, int waves, int unroll, const float* scale_pieces,
                            int n_scale_pieces, float scale_width, float scale_eps, void* stream) {
  IFX_REQUIRE(!scale_pieces || (n_scale_pieces > 0 && scale_width > 0.f), "qkv_rope: bad row factors (%d pieces, width %g)",
              n_scale_pieces, (double)scale_width);
  IFX_REQUIRE(M >= 0 && M <= 16 && K > 0 && K % 8 == 0, "qkv_rope: M=%d must be at most 16, K=%d a multiple of 8", M, K);
  IFX_REQUIRE(nH > 0 && nKV >= 0 && d > 0 && d % 32 == 0, "qkv_rope: head size %d must be a multiple of 32 (nH=%d nKV=%d)", d, nH, nKV);
  IFX_REQUIRE(cs && sn && q_out, "qkv_rope: needs the rotation table and an output");
  IFX_REQUIRE(!slots || (page_size > 0 && k_cache && v_cache), "qkv_rope: cache write without cache");
  IFX_REQUIRE(bias_dtype == DT_BF16 || bias_dtype == DT_F32 || !bias, "qkv_rope: unknown bias dtype %d", bias_dtype);
  if (M == 0) return 0;
  const int heads = nH + (slots ? 2 * nKV : 0), N = heads * d, groups = N / 32;
  const int nkb = (K + 63) / 64, k_tiles = ifx_tiled_cols(K) / 32;
  if (unroll == 0) unroll = 2;
  if (waves == 0) {
    waves = 1;
    while (waves < 16 && groups * waves < 1024) waves *= 2;
    while (waves > 1 && nkb < waves * 2) waves /= 2;
  }
  IFX_REQUIRE(waves >= 1 && waves <= 16 && (unroll == 2 || unroll == 4), "qkv_rope: waves=%d unroll=%d", waves, unroll);
  const size_t lds = (size_t)(waves - 1) * 2 * WAVE * 4 * sizeof(float);
  QkvArgs a{bias, bias_dtype, slots, cs, sn, (bf16_t*)q_out, (bf16_t*)k_cache, (bf16_t*)v_cache, nH, slots ? nKV : 0, d, page_size};
  const RowScale scale{scale_pieces, n_scale_pieces, scale_width, scale_eps};
  hipStream_t s = (hipStream_t)stream;
  if (unroll == 2) hipLaunchKernelGGL(qkv_rope_kernel<2>, dim3(groups), dim3(waves * WAVE), lds, s, (const bf16_t*)x, (const bf16_t*)Wt, M, N, K, k_tiles, a, scale);
  else hipLaunchKernelGGL(qkv_rope_kernel<4>, dim3(groups), dim3(waves * WAVE), lds, s, (const bf16_t*)x, (const bf16_t*)Wt, M, N, K, k_tiles, a, scale);
  IFX_LAUNCH_CHECK();
}

// nt, waves, unroll = 0: chosen here from the shape.
// epi 1: gate/up rows interleaved in W, out = silu(gate) * up, [M, N / 2].
// epi 2: the product is added to ``stream`` [M, N] (float, in place), rows_out [M, N] = bf16(stream * norm_w) and
//        pieces_out [ceil(N / 16)][16] = sums of squares of the stream in runs of 16, for the norm that follows
//        (M <= 16, N a multiple of 4, norm_w bfloat16 [N]); ``out`` is not used.
// tiled 1 or 16: W is the tiled form written by ifx_tile_weights, with the row-tile order it was given (or null);
//        8 to 14 (even): that form with so many rows to a tile (no order).
// scale_pieces [n_scale_pieces][16] (or null), scale_width, scale_eps: a factor per row of x (M <= 16), see RowScale.
extern "C" int ifx_skinny_gemm(const void* x, const void* W, void* out, int out_dtype, int M, int N, int K, int nt,
                               int waves, int unroll, int epi, int tiled, const int* order, const float* scale_pieces,
                               int n_scale_pieces, float scale_width, float scale_eps, float* stream_io,
                               const void* norm_w, void* rows_out, float* pieces_out, void* stream) {
  IFX_REQUIRE(tiled == 0 || tiled == 1 || (tiled >= 8 && tiled <= 16 && tiled % 2 == 0), "skinny_gemm: tiled=%d (0, 1, or 8 to 16 rows to a tile)", tiled);
  const int tile_rows = tiled >= 8 ? tiled : 16;
  IFX_REQUIRE((tiled && tile_rows == 16) || !order, "skinny_gemm: a tile order goes with a tiled copy of 16-row tiles");
  IFX_REQUIRE(epi == 0 || !order, "skinny_gemm: only the plain epilogue takes a tile order");
  IFX_REQUIRE(epi == 0 || (epi == 1 && N % 2 == 0) || (epi == 2 && N % 4 == 0), "skinny_gemm: epilogue %d with N=%d", epi, N);
  IFX_REQUIRE(epi != 2 || (M <= 16 && stream_io && norm_w && rows_out && pieces_out),
              "skinny_gemm: the stream epilogue takes at most 16 rows (M=%d) and needs the stream, the norm's weight and two outputs", M);
  IFX_REQUIRE(!scale_pieces || (M <= 16 && n_scale_pieces > 0 && scale_width > 0.f),
              "skinny_gemm: row factors take at most 16 rows (M=%d, %d pieces, width %g)", M, n_scale_pieces, (double)scale_width);
  IFX_REQUIRE(M >= 0 && M <= 64 && N > 0 && K > 0, "skinny_gemm: M=%d must be at most 64 (N=%d K=%d)", M, N, K);
  IFX_REQUIRE(K % 8 == 0, "skinny_gemm: K=%d must be a multiple of 8", K);
  IFX_REQUIRE(out_dtype == DT_BF16 || out_dtype == DT_F32, "skinny_gemm: unknown out dtype %d", out_dtype);
  if (M == 0) return 0;
  const int mt = (M + 15) / 16;
  const int nkb = (K + 63) / 64;
  // Choices measured on the 7B shapes at 1-16 rows: two row tiles per wave pay off only for very tall
  // weights; deeper unrolling than 4 blocks spills; about 1500-2500 waves fill the chip.
  if (tiled && mt == 1) {
    // Measured on the tiled copy (shapes of the 0.5B to 72B models, 1-16 rows).  Two row tiles per wave halve the
    // reads of x; they win where they leave 128 workgroups or more and do not make the fullest compute unit fuller
    // (every workgroup of a launch is resident at once, so what counts is how many tiles the unit with the most gets:
    // 1,728 tiles are 7 to a unit one by one and 8 in pairs), except up to 4 rows of x for weights of more than 512
    // tiles, where x is little to read.  Tall weights want 8 waves per workgroup up to 8 rows of x and one beyond;
    // the others enough waves to have 1,536 in flight up to 4 rows (4,096 for weights of more than 512 tiles) and
    // 1,200 beyond (fewer waves split K less and read less of x), at most 8 to a workgroup of tile pairs.  Against one rule for all (pairs from 256 tiles on,
    // 1,536 waves) gate/up of the 0.5B, 1.5B, 3B and 14B shapes takes 10-15 % less time at 1-16 rows.
    const bool tall = N >= 32768;
    const int n_tiles = (N + tile_rows - 1) / tile_rows;
    auto fullest_unit = [&](int nt_) { return ((n_tiles + nt_ - 1) / nt_ + UNITS - 1) / UNITS * nt_; };
    if (nt == 0) {
      const bool pairs_fit = tile_rows == 16 && (n_tiles + 1) / 2 >= 128 && fullest_unit(2) <= fullest_unit(1);
      nt = tall ? (M <= 4 ? 1 : 2) : (pairs_fit && (M > 4 || n_tiles <= 512) ? 2 : 1);
    }
    if (unroll == 0) unroll = (nt == 1 && M <= 4) ? 4 : 2;
    if (waves == 0) {
      const int groups = (n_tiles + nt - 1) / nt;
      waves = 1;
      if (tall) waves = M <= 8 ? 8 : 1;
      else
        while (waves < (nt == 2 ? 8 : 16) && groups * waves < (M > 4 ? 1200 : n_tiles > 512 ? 4096 : 1536)) waves *= 2;
      while (waves > 1 && nkb < waves * 2) waves /= 2;
    }
  }
  if (nt == 0) nt = (N >= 32768 && mt <= 2) ? 2 : 1;
  if (unroll == 0) unroll = (mt * nt >= 2) ? 2 : 4;
  if (waves == 0) {
    const int groups = (N + tile_rows * nt - 1) / (tile_rows * nt);
    waves = 1;
    if (groups < 1024)
      while (waves < 16 && groups * waves < 1536 && nkb >= waves * 2) waves *= 2;
  }
  while (waves > 1 && (size_t)(waves - 1) * nt * mt * WAVE * 16 > 64 * 1024) waves /= 2;
  IFX_REQUIRE(waves >= 1 && waves <= 16, "skinny_gemm: waves=%d outside 1..16", waves);
  if (epi == 2 && nt == 2 && unroll == 4) unroll = 2;   // that instantiation spills
  hipStream_t s = (hipStream_t)stream;
  const int k_tiles = ifx_tiled_cols(K) / 32;
  const RowScale scale{scale_pieces, n_scale_pieces, scale_width, scale_eps};
  const StreamOut so{stream_io, (const bf16_t*)norm_w, (bf16_t*)rows_out, pieces_out};
#define CASE(MT_, NT_, U_)                                                                                             \
  if (mt == MT_ && nt == NT_ && unroll == U_)                                                                          \
    return tiled ? launch<MT_, NT_, U_, true>(x, W, out, out_dtype, M, N, K, k_tiles, waves, epi, order, scale, so, tile_rows, s)  \
                 : launch<MT_, NT_, U_, false>(x, W, out, out_dtype, M, N, K, k_tiles, waves, epi, order, scale, so, 16, s)
  // (the combinations left out need more than the 128 registers a workgroup of 16 waves leaves a lane)
  CASE(1, 1, 4); CASE(1, 2, 4); CASE(1, 1, 2); CASE(1, 2, 2);
  CASE(2, 1, 4); CASE(2, 2, 2); CASE(2, 1, 2);
  CASE(3, 1, 2); CASE(3, 2, 2);
  CASE(4, 1, 2);
#undef CASE
  IFX_FAIL("skinny_gemm: no kernel for m-tiles=%d n-tiles=%d unroll=%d", mt, nt, unroll);
}


// =======================================================================================
// The same product for up to 64 rows with x staged in LDS.
//
// A workgroup of 4 waves owns 64 weight rows (one 16-row tile per wave) and one slice of K.  The
// rows of x that belong to the current 128-wide piece of K are copied to LDS once and read from
// there by all four waves, so x crosses the L2 once per 64 weight rows instead of once per 16;
// at 64 rows of x that is the difference between x traffic of four times the weights and x
// traffic equal to the weights.  The weight stream is as above: 32 contiguous bytes per lane per
// 64 k-values, U pieces in flight.  With more than one slice of K, slices write float partial
// sums that a second kernel adds in slice order (a fixed order: the result does not depend on
// timing).
// =======================================================================================
#define KC 128
#define XPAD 8

template <int MT, int U, typename TO, int EPI>
__global__ __launch_bounds__(256) void staged_gemm_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ W,
                                                          TO* __restrict__ out, float* __restrict__ part, int M, int N,
                                                          int K, int chunks_per_slice) {
  __shared__ __attribute__((aligned(16))) bf16_t xs[2][MT * 16][KC + XPAD];
  const int tid = threadIdx.x, wid = tid / WAVE, lane = tid % WAVE, col = lane & 15, g = lane >> 4;
  const int n_base = blockIdx.x * 64 + 16 * wid;
  const int n_chunks = (K + KC - 1) / KC;
  const int c_begin = blockIdx.y * chunks_per_slice, n = min(n_chunks, c_begin + chunks_per_slice) - c_begin;
  const bf16_t* wrow = W + (size_t)min(n_base + col, N - 1) * K;  // rows past N are read again, never stored
  floatx4 acc[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) acc[mt] = floatx4{0.f, 0.f, 0.f, 0.f};
  bf16x8 wreg[U][4], xr[MT];

  auto load_w = [&](int c, bf16x8* w) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {  // q = 2 * (64-block of the piece) + (half of the lane's 16 values)
      const int k = c * KC + (q >> 1) * 64 + 16 * g + 8 * (q & 1);
      w[q] = k < K ? *(const bf16x8*)(wrow + k) : zero8();
    }
  };
  auto load_x = [&](int c) {
#pragma unroll
    for (int i = 0; i < MT; ++i) {
      const int p = tid + 256 * i, row = p >> 4, k = c * KC + 8 * (p & 15);
      xr[i] = (row < M && k < K) ? *(const bf16x8*)(x + (size_t)row * K + k) : zero8();
    }
  };
  auto store_x = [&](int buf) {
#pragma unroll
    for (int i = 0; i < MT; ++i) {
      const int p = tid + 256 * i;
      *(bf16x8*)&xs[buf][p >> 4][8 * (p & 15)] = xr[i];
    }
  };

#pragma unroll
  for (int u = 0; u < U; ++u)
    if (u < n) load_w(c_begin + u, wreg[u]);
  if (n > 0) {
    load_x(c_begin);
    store_x(0);
  }
  __syncthreads();
  for (int i0 = 0; i0 < n; i0 += U) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int i = i0 + u;
      if (i >= n) break;  // the same for every thread
      if (i + 1 < n) load_x(c_begin + i + 1);
#pragma unroll
      for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          const bf16x8 xb = *(const bf16x8*)&xs[u & 1][16 * mt + col][(q >> 1) * 64 + 16 * g + 8 * (q & 1)];
          acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wreg[u][q], xb, acc[mt], 0, 0, 0);
        }
      if (i + U < n) load_w(c_begin + i + U, wreg[u]);
      if (i + 1 < n) store_x((u + 1) & 1);
      __syncthreads();
    }
  }
  // acc[mt][r] = out[m = 16 mt + col][n = n_base + 4 g + r]
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = 16 * mt + col;
    if (m >= M) continue;
    if (gridDim.y > 1) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int nn = n_base + 4 * g + r;
        if (nn < N) part[((size_t)blockIdx.y * M + m) * N + nn] = acc[mt][r];
      }
    } else if (EPI == 0) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int nn = n_base + 4 * g + r;
        if (nn < N) out[(size_t)m * N + nn] = from_f<TO>(acc[mt][r]);
      }
    } else {
#pragma unroll
      for (int r = 0; r < 4; r += 2) {
        const int nn = n_base + 4 * g + r;  // even: gate at nn, up at nn + 1
        const float gt = acc[mt][r], up = acc[mt][r + 1];
        if (nn + 1 < N) out[(size_t)m * (N / 2) + nn / 2] = from_f<TO>(gt / (1.0f + expf(-gt)) * up);
      }
    }
  }
}

template <typename TO>
__global__ void sum_slices_kernel(const float* __restrict__ part, TO* __restrict__ out, int S, size_t n) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  float a = 0.f;
  for (int s = 0; s < S; ++s) a += part[(size_t)s * n + i];
  out[i] = from_f<TO>(a);
}

template <int MT, int U>
static int launch_staged(const void* x, const void* W, void* out, int out_dtype, float* part, int M, int N, int K,
                         int slices, int cps, int epi, hipStream_t s) {
  const dim3 grid((N + 63) / 64, slices);
#define GO(TO_, EPI_)                                                                                         \
  hipLaunchKernelGGL((staged_gemm_kernel<MT, U, TO_, EPI_>), grid, dim3(256), 0, s, (const bf16_t*)x,         \
                     (const bf16_t*)W, (TO_*)out, part, M, N, K, cps)
  if (out_dtype == DT_BF16 && epi == 0) GO(bf16_t, 0);
  else if (out_dtype == DT_BF16) GO(bf16_t, 1);
  else if (epi == 0) GO(float, 0);
  else GO(float, 1);
#undef GO
  if (slices > 1) {
    const size_t n = (size_t)M * N;
    const unsigned blocks = (unsigned)((n + 255) / 256);
    if (out_dtype == DT_BF16) hipLaunchKernelGGL(sum_slices_kernel<bf16_t>, dim3(blocks), dim3(256), 0, s, part, (bf16_t*)out, slices, n);
    else hipLaunchKernelGGL(sum_slices_kernel<float>, dim3(blocks), dim3(256), 0, s, part, (float*)out, slices, n);
  }
  IFX_LAUNCH_CHECK();
}

// Largest number of K slices ifx_staged_gemm will use for a shape: the caller sizes ``part``
// (slices * M * N floats) by it.
extern "C" int ifx_staged_gemm_slices(int M, int N, int K, int slices) {
  const int n_chunks = (K + KC - 1) / KC;
  if (slices <= 0) {
    const int groups = (N + 63) / 64;
    slices = groups >= 512 ? 1 : (1024 + groups - 1) / groups;
    if (slices > n_chunks / 4) slices = n_chunks / 4;
  }
  if (slices < 1) slices = 1;
  if (slices > n_chunks) slices = n_chunks;
  const int cps = (n_chunks + slices - 1) / slices;
  return (n_chunks + cps - 1) / cps;
}

extern "C" int ifx_staged_gemm(const void* x, const void* W, void* out, int out_dtype, float* part, int M, int N, int K,
                               int slices, int unroll, int epi, void* stream) {
  IFX_REQUIRE(M >= 0 && M <= 64 && N > 0 && K > 0, "staged_gemm: M=%d must be at most 64 (N=%d K=%d)", M, N, K);
  IFX_REQUIRE(K % 8 == 0, "staged_gemm: K=%d must be a multiple of 8", K);
  IFX_REQUIRE(out_dtype == DT_BF16 || out_dtype == DT_F32, "staged_gemm: unknown out dtype %d", out_dtype);
  IFX_REQUIRE(epi == 0 || (epi == 1 && N % 2 == 0), "staged_gemm: epilogue %d with N=%d", epi, N);
  if (M == 0) return 0;
  const int mt = (M + 15) / 16;
  const int n_chunks = (K + KC - 1) / KC;
  if (epi != 0) slices = 1;
  slices = ifx_staged_gemm_slices(M, N, K, slices);
  IFX_REQUIRE(slices == 1 || part, "staged_gemm: %d slices of K need a scratch buffer", slices);
  const int cps = (n_chunks + slices - 1) / slices;
  if (unroll == 0) unroll = 4;
  hipStream_t s = (hipStream_t)stream;
#define CASE(MT_, U_) if (mt == MT_ && unroll == U_) return launch_staged<MT_, U_>(x, W, out, out_dtype, part, M, N, K, slices, cps, epi, s)
  CASE(1, 4); CASE(2, 4); CASE(3, 4); CASE(4, 4);
  CASE(1, 2); CASE(2, 2); CASE(3, 2); CASE(4, 2);
  CASE(1, 6); CASE(2, 6); CASE(3, 6); CASE(4, 6);
#undef CASE
  IFX_FAIL("staged_gemm: no kernel for m-tiles=%d unroll=%d", mt, unroll);
}
