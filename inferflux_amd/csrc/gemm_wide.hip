// Weight-streaming matrix product for 17-128 rows (and for 9-16 rows of large tall weights):  out[M,N] = x[M,K] * W[N,K]^T
// from the tiled copy of W (layout: gemm_bf16.hip), bf16 in, float accumulate on the matrix cores (16x16x32), out bf16 or
// float; up to 16 rows may come with a norm's factor per row, applied to the sums (row_scale.h).
//
// At these sizes the product is still bound by reading W once, but every tile of W now meets two to eight
// tiles of x, and a wave that fetched those from the L2 itself would move more bytes of x than of W.  A
// workgroup of 8-16 waves therefore owns one tile of 16 weight rows per wave and one slice of K, and the
// rows of x for the next 128 k-values are copied to LDS once per workgroup (two buffers, one barrier per
// round of 128) and read from there by every wave.  Each wave streams its own tile row of W, one
// contiguous kilobyte per load with streaming loads, DEPTH rounds ahead of the arithmetic; the rows of x are
// asked for as far ahead and wait in registers (a round's arithmetic is much shorter than a trip to the L2).
//
// How many waves and slices: what a compute unit can have on its way from memory is bounded, so the time is
// set by the unit with the most bytes to fetch, x included.  Measured on the 7B shapes, the best launch has
// about one workgroup for each of the 256 units, as many waves in it as that takes (8-16), and K cut into
// slices where the weight has too few rows for that (ifx_wide_gemm_plan).
//
// x in LDS: the 16-byte piece (row r, k-piece j of the round's 16) lies at slot j R + (r + j) % R of the
// buffer (R = 16 MT rows).  A wave reads its B operand of (k-tile kt, x tile mt) as 16-byte pieces
// j = 4 kt + g of rows 16 mt + col: sixteen consecutive slots per group of 16 lanes, no bank conflict; the
// shift by j keeps the stores of 16 consecutive pieces of one row apart as well.
//
// More than 64 rows (five to eight tiles of x, 170 registers a wave) run as workgroups of exactly 8 waves.  That is
// worth it where the weight has few rows and K is cut into slices (down, o, q/k/v of the 7B shape at 65-128 rows:
// 37-50, 15-21 and 16-22 us against the library's 58-66, 30-34 and 30-37); a tall weight such as gate/up would need
// more than one workgroup of 8 waves per compute unit and is left to the library there (115 against 64 us at 128
// rows).  The caller decides (ops._small_m_kernel).
//
// With more than one slice of K the slices write float partial sums and a second kernel adds them in slice
// order; the result never depends on timing.
//
// The reference sends these products to cuBLAS (runtime/backends/cuda/native/cublas_gemm.cpp:99-117).
#include "common.h"
#include "row_scale.h"

IFX_DEFINE_LAST_ERROR()

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;
typedef __attribute__((__vector_size__(2 * sizeof(float)))) float floatx2;

constexpr int DEPTH = 3;                                           // rounds of W and x on their way
constexpr int MIN_WAVES = 8, MAX_WAVES = 16;                     // of the kernel's usual form
constexpr int FEW_WAVES = 4;                                       // of its form for workgroups of 4-7 waves (up to MANY_ROWS rows)
constexpr int MAX_ROWS = 128, MANY_ROWS = 64;                     // beyond MANY_ROWS a workgroup has exactly MIN_WAVES waves
constexpr int WK = 128, WK_TILES = WK / 32, WK_PIECES = WK / 8;   // k-values, k-tiles and 16-byte pieces of a round

__device__ __forceinline__ bf16x8 zero8() {
  bf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = (__bf16)0.f;
  return z;
}

// (float results are logits, 39 MB at 64 rows of a 152,064-token vocabulary, read again only by the sampler: written
// with streaming stores they do not push the rows of x out of the L2: the 7B head at 64 rows 206 -> 189 us, 14B 288 -> 263)
__device__ __forceinline__ void store4(float* p, floatx4 v) { __builtin_nontemporal_store(v, (floatx4*)p); }
__device__ __forceinline__ void store4(bf16_t* p, floatx4 v) {
  typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4;
  bf16x4 w;
#pragma unroll
  for (int r = 0; r < 4; ++r) w[r] = (__bf16)v[r];
  *(bf16x4*)p = w;
}
__device__ __forceinline__ void store2(float* p, float a, float b) { *(float2*)p = float2{a, b}; }
__device__ __forceinline__ void store2(bf16_t* p, float a, float b) {
  typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2;
  bf16x2 w;
  w[0] = (__bf16)a; w[1] = (__bf16)b;
  *(bf16x2*)p = w;
}

// EPI 0: out[m, n] = sum.  EPI 1: the rows of W alternate gate, up, ...: out[m, n / 2] = silu(gate) * up.
// ``order``: tile t of the copy holds the weight's rows 16 order[t] ...; null: in order.
// ``MINW``: the fewest waves a workgroup of this form may have (each thread then copies more pieces of x to LDS and
// holds them in more registers, which a workgroup of at most 8 waves has).
// ``scale`` (up to 16 rows): the sums of row m are multiplied by the row's factor (see RowScale).  Every thread asks for
// its few of the pieces before the first rounds of W and x, so that they arrive first and cost no trip of their own; the
// waves' shares of the rows' sums meet in LDS.
template <int MT, typename TO, int EPI, int MINW>
__global__ __launch_bounds__((16 * MT > MANY_ROWS || MINW < MIN_WAVES ? MIN_WAVES : MAX_WAVES) * WAVE) void wide_gemm_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ Wt,
                                                                     TO* __restrict__ out, float* __restrict__ part, int M,
                                                                     int N, int K, int k_tiles, int rounds_per_slice,
                                                                     const int* __restrict__ order, int tile_rows, RowScale scale) {
  constexpr int R = MT * 16;                                  // rows of x in LDS
  constexpr int X_PIECES = R * WK_PIECES;                     // 16-byte pieces of a round's x
  constexpr int X_PER_THREAD = (X_PIECES + MINW * WAVE - 1) / (MINW * WAVE);
  __shared__ __attribute__((aligned(16))) bf16x8 xs[2][X_PIECES];
  __shared__ __attribute__((aligned(16))) float row_sums[MAX_WAVES][16];
  const int tid = threadIdx.x, threads = blockDim.x, waves = threads / WAVE;
  const int wid = tid / WAVE, lane = tid % WAVE, col = lane & 15, g = lane >> 4;
  const bool scaled = MT == 1 && scale.pieces != nullptr;
  RowSumsEarly pieces_asked;
  if (scaled) row_sums_ask(scale, tid, threads, pieces_asked);
  const int tile = blockIdx.x * waves + wid, n_tiles = (N + tile_rows - 1) / tile_rows;
  const int n_rounds = (K + WK - 1) / WK;
  const int r_begin = blockIdx.y * rounds_per_slice, n = min(n_rounds, r_begin + rounds_per_slice) - r_begin;
  // a wave whose tile lies past N reads the last tile again and stores nothing
  // (a tile of the copy holds tile_rows rows, 64 tile_rows bytes per k-tile: see gemm_bf16.hip; the lanes of the other rows hold zeros)
  const bf16_t* wtile = Wt + ((size_t)min(tile, n_tiles - 1) * k_tiles * 4 * tile_rows + tile_rows * g + col) * 8;
  const bool row_held = col < tile_rows;
  floatx4 acc[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) acc[mt] = floatx4{0.f, 0.f, 0.f, 0.f};
  bf16x8 wreg[DEPTH][WK_TILES];
  bf16x8 xreg[DEPTH][X_PER_THREAD];

  auto load_w = [&](int r, bf16x8 (&w)[WK_TILES]) {
#pragma unroll
    for (int kt = 0; kt < WK_TILES; ++kt) {
      const int t = r * WK_TILES + kt;
      w[kt] = (t < k_tiles && row_held) ? __builtin_nontemporal_load((const bf16x8*)(wtile + (size_t)t * 4 * tile_rows * 8)) : zero8();
    }
  };
  auto load_x = [&](int r, bf16x8 (&xp)[X_PER_THREAD]) {
#pragma unroll
    for (int i = 0; i < X_PER_THREAD; ++i) {
      const int p = tid + threads * i, row = p / WK_PIECES, k = r * WK + 8 * (p % WK_PIECES);
      xp[i] = (p < X_PIECES && row < M && k < K) ? *(const bf16x8*)(x + (size_t)row * K + k) : zero8();
    }
  };
  auto store_x = [&](int buf, const bf16x8 (&xp)[X_PER_THREAD]) {
#pragma unroll
    for (int i = 0; i < X_PER_THREAD; ++i) {
      const int p = tid + threads * i, row = p / WK_PIECES, j = p % WK_PIECES;
      if (p < X_PIECES) xs[buf][j * R + (row + j) % R] = xp[i];
    }
  };
  auto compute = [&](const bf16x8 (&w)[WK_TILES], int buf) {
#pragma unroll
    for (int kt = 0; kt < WK_TILES; ++kt) {
      const int j = 4 * kt + g;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
        acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[kt], xs[buf][j * R + (16 * mt + col + j) % R], acc[mt], 0, 0, 0);
    }
  };
  // register set d holds W and x of the rounds c with c % DEPTH == d
  if (n > 0) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d)
      if (d < n) {
        load_x(r_begin + d, xreg[d]);
        load_w(r_begin + d, wreg[d]);
      }
    store_x(0, xreg[0]);
    if (DEPTH < n) load_x(r_begin + DEPTH, xreg[0]);
  }
  if (scaled) {
    const rs_floatx4 sums = row_sums_of_wave(row_sums_of_thread(scale, tid, threads, pieces_asked));
    if (lane < 4) *(rs_floatx4*)&row_sums[wid][4 * lane] = sums;
  }
  __syncthreads();
  for (int c0 = 0; c0 < n; c0 += 2 * DEPTH) {   // unrolled over the register sets and the two LDS buffers
#pragma unroll
    for (int dd = 0; dd < 2 * DEPTH; ++dd) {
      const int c = c0 + dd;
      if (c >= n) break;   // the same for every thread
      compute(wreg[dd % DEPTH], dd & 1);
      if (c + DEPTH < n) load_w(r_begin + c + DEPTH, wreg[dd % DEPTH]);
      if (c + 1 < n) {     // the other buffer was last read in round c - 1, which every wave has left
        store_x((dd + 1) & 1, xreg[(dd + 1) % DEPTH]);
        if (c + 1 + DEPTH < n) load_x(r_begin + c + 1 + DEPTH, xreg[(dd + 1) % DEPTH]);
      }
      __syncthreads();
    }
  }
  if (tile >= n_tiles) return;
  // acc[mt][r] = out[m = 16 mt + col][n = tile_rows (row tile of the weight) + 4 g + r], for 4 g + r < tile_rows
  const int n0 = tile_rows * (order ? order[tile] : tile) + 4 * g;
  const int held = min(4, tile_rows - 4 * g);      // how many of the lane's four rows the tile holds (even, may be <= 0)
  // A lane's four sums are four consecutive columns of one output row.  Where the tile holds all four and rows start at
  // multiples of four columns they go out as one store (16 bytes of float, 8 of bf16) instead of four: the head's
  // 39 MB of logits at 64 rows otherwise arrive as 4-byte pieces 600 KB apart.
  const bool whole = held == 4 && n0 + 3 < N && ((N | n0) & 3) == 0;
  if (scaled) {   // (the shares were written before the first barrier above, which every wave has passed)
    float sum = 0.f;
    for (int w = 0; w < waves; ++w) sum += row_sums[w][col];
    const float f = rsqrtf(sum / scale.width + scale.eps);
#pragma unroll
    for (int r = 0; r < 4; ++r) acc[0][r] *= f;
  }
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = 16 * mt + col;
    if (m >= M) continue;
    if (gridDim.y > 1) {
      float* dst = part + ((size_t)blockIdx.y * M + m) * N + n0;
      if (whole) {
        *(floatx4*)dst = acc[mt];
      } else if (((N | n0) & 1) == 0) {   // (tiles of 10 or 14 rows start at even columns: pairs go out as 8 bytes; plain
                                           //  stores: the kernel that adds the slices reads them next, and streaming ones
                                           //  cost a decode step of 64 requests 2 %)
#pragma unroll
        for (int r = 0; r < 4; r += 2)
          if (r < held && n0 + r < N) *(floatx2*)(dst + r) = floatx2{acc[mt][r], acc[mt][r + 1]};
      } else {
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (r < held && n0 + r < N) dst[r] = acc[mt][r];
      }
    } else if (EPI == 0) {
      TO* dst = out + (size_t)m * N + n0;
      if (whole) {
        store4(dst, acc[mt]);
      } else {
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (r < held && n0 + r < N) dst[r] = from_f<TO>(acc[mt][r]);
      }
    } else {
      TO* dst = out + (size_t)m * (N / 2) + n0 / 2;
      float v[2];
#pragma unroll
      for (int r = 0; r < 4; r += 2) {   // even: gate at n0 + r, up at n0 + r + 1
        const float gt = acc[mt][r], up = acc[mt][r + 1];
        v[r / 2] = gt / (1.0f + expf(-gt)) * up;
      }
      if (whole) {
        store2(dst, v[0], v[1]);
      } else {
#pragma unroll
        for (int r = 0; r < 4; r += 2)
          if (r < held && n0 + r + 1 < N) dst[r / 2] = from_f<TO>(v[r / 2]);
      }
    }
  }
}

template <typename TO>
__global__ void wide_sum_slices_kernel(const float* __restrict__ part, TO* __restrict__ out, int S, size_t n) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  float a = 0.f;
  for (int s = 0; s < S; ++s) a += part[(size_t)s * n + i];
  out[i] = from_f<TO>(a);
}

// out [n] = part [S][n] added in slice order.
extern "C" int ifx_sum_slices(const float* part, void* out, int out_dtype, int S, long long n, void* stream) {
  IFX_REQUIRE(S >= 1 && n >= 0 && (out_dtype == DT_BF16 || out_dtype == DT_F32), "sum_slices: %d slices of %lld, out dtype %d", S, n, out_dtype);
  if (n == 0) return 0;
  const unsigned blocks = (unsigned)((n + 255) / 256);
  if (out_dtype == DT_BF16) hipLaunchKernelGGL(wide_sum_slices_kernel<bf16_t>, dim3(blocks), dim3(256), 0, (hipStream_t)stream, part, (bf16_t*)out, S, (size_t)n);
  else hipLaunchKernelGGL(wide_sum_slices_kernel<float>, dim3(blocks), dim3(256), 0, (hipStream_t)stream, part, (float*)out, S, (size_t)n);
  IFX_LAUNCH_CHECK();
}

// Waves per workgroup and slices of K for a shape.  ``waves`` / ``slices`` 0: chosen here (about one workgroup
// for each of the 256 compute units: as many waves as that takes; 8 waves for more than 64 rows; then slices of at
// least two rounds, at most eight); the gate/up epilogue takes one slice.  Returns waves * 256 + slices.
// Where even 16 waves leave several workgroups to a unit (the head: 9,500 tiles), what counts is how many tiles the
// fullest unit gets and how often x is staged: 8, 10 and 14 waves give the fullest unit 40, 40 and 42 tiles, the numbers
// between 44-48.  Measured on the heads of the 0.5B-72B shapes: 10 waves up to 32 rows (7B 179 -> 172 us at 17 rows, 3B
// 122 -> 99, 72B 399 -> 374; K below 2,048 gains nothing), 8 beyond, except for K a multiple of 2,048, where 8 waves
// are markedly slower at every number of rows (3B at 64 rows 131 us with 8 waves, 116 with 14; the tiles a workgroup's
// waves stream together then lie a power of two apart in memory, which may be why).
// Fewer than 8 waves are chosen for the gate/up epilogue at 33-64 rows only: there the tall weights of narrow models
// (600-1,700 tiles) take 4-17 % less time with one workgroup of 4-7 waves on every unit than with 8 waves on two thirds
// of them; up to 32 rows the form for few waves is the slower one at every shape measured, and the other products
// fill the chip with slices of K.
extern "C" int ifx_wide_gemm_plan(int rows, int N, int K, int waves, int slices, int epi, int tile_rows) {
  if (tile_rows < 8 || tile_rows > 16) tile_rows = 16;
  const int n_tiles = (N + tile_rows - 1) / tile_rows, n_rounds = (K + WK - 1) / WK;
  if (waves <= 0) {
    if (n_tiles > 256 * MAX_WAVES) waves = rows <= 32 ? (K >= 2048 ? 10 : MIN_WAVES) : (K % 2048 == 0 ? 14 : MIN_WAVES);
    else waves = (n_tiles + 255) / 256;
    if (waves < MIN_WAVES && (rows <= 32 || epi == 0)) waves = MIN_WAVES;   // (products that may be cut into slices of K fill the chip that way)
  }
  const int fewest = rows > MANY_ROWS ? MIN_WAVES : FEW_WAVES;
  waves = waves < fewest ? fewest : (waves > MAX_WAVES ? MAX_WAVES : waves);
  if (rows > MANY_ROWS) waves = MIN_WAVES;
  const int groups = (n_tiles + waves - 1) / waves;
  if (epi != 0) slices = 1;
  if (slices <= 0) {
    slices = 256 / groups;
    if (slices > 8) slices = 8;
    if (slices > n_rounds / 2) slices = n_rounds / 2;
  }
  if (slices < 1) slices = 1;
  if (slices > n_rounds) slices = n_rounds;
  const int rps = (n_rounds + slices - 1) / slices;
  return waves * 256 + (n_rounds + rps - 1) / rps;
}

template <int MT>
static int launch_wide(const void* x, const void* Wt, void* out, int out_dtype, float* part, int M, int N, int K, int waves,
                       int slices, int rps, int epi, const int* order, bool add_slices, int tile_rows, RowScale scale, hipStream_t s) {
  const int n_tiles = (N + tile_rows - 1) / tile_rows;
  const dim3 grid((n_tiles + waves - 1) / waves, slices);
  const int k_tiles = (K + 63) / 64 * 2;
#define GO(TO_, EPI_, MINW_)                                                                                       \
  hipLaunchKernelGGL((wide_gemm_kernel<MT, TO_, EPI_, MINW_>), grid, dim3(waves * WAVE), 0, s, (const bf16_t*)x,   \
                     (const bf16_t*)Wt, (TO_*)out, part, M, N, K, k_tiles, rps, order, tile_rows, scale)
#define GO_ALL(MINW_)                                    \
  if (out_dtype == DT_BF16 && epi == 0) GO(bf16_t, 0, MINW_); \
  else if (out_dtype == DT_BF16) GO(bf16_t, 1, MINW_);        \
  else if (epi == 0) GO(float, 0, MINW_);                     \
  else GO(float, 1, MINW_)
  if (waves >= MIN_WAVES) {
    GO_ALL(MIN_WAVES);
  } else {
    if constexpr (16 * MT <= MANY_ROWS) { GO_ALL(FEW_WAVES); }
    else IFX_FAIL("wide_gemm: more than %d rows take workgroups of %d waves", MANY_ROWS, MIN_WAVES);
  }
#undef GO_ALL
#undef GO
  if (slices > 1 && add_slices) {
    const size_t n = (size_t)M * N;
    const unsigned blocks = (unsigned)((n + 255) / 256);
    if (out_dtype == DT_BF16) hipLaunchKernelGGL(wide_sum_slices_kernel<bf16_t>, dim3(blocks), dim3(256), 0, s, part, (bf16_t*)out, slices, n);
    else hipLaunchKernelGGL(wide_sum_slices_kernel<float>, dim3(blocks), dim3(256), 0, s, part, (float*)out, slices, n);
  }
  IFX_LAUNCH_CHECK();
}

// x [M <= 128, K] times the tiled copy Wt of W [N, K], transposed.  ``waves``, ``slices``: as ifx_wide_gemm_plan
// returned them; ``part``: slices * M * N floats when there is more than one slice.
// epi 1: gate/up rows interleaved in W, out = silu(gate) * up, [M, N / 2] (one slice, no tile order).
// order: the row-tile order the copy was written with (or null); tile_rows: the rows to a tile it was written with.
// ``out`` null with more than one slice: the partial sums are left in ``part`` for a kernel that adds them itself
// (ifx_add_rmsnorm, ifx_rope_append).
// scale_pieces [n_scale_pieces][16] (or null), scale_width, scale_eps: a factor per row of x (M <= 16), see RowScale.
extern "C" int ifx_wide_gemm(const void* x, const void* Wt, void* out, int out_dtype, float* part, int M, int N, int K,
                             int waves, int slices, int epi, const int* order, int tile_rows, const float* scale_pieces,
                             int n_scale_pieces, float scale_width, float scale_eps, void* stream) {
  IFX_REQUIRE(out || slices > 1, "wide_gemm: no output");
  IFX_REQUIRE(tile_rows >= 8 && tile_rows <= 16 && tile_rows % 2 == 0 && (tile_rows == 16 || !order),
              "wide_gemm: %d rows to a tile (8 to 16, even; a tile order goes with 16)", tile_rows);
  IFX_REQUIRE(M >= 0 && M <= MAX_ROWS && N > 0 && K > 0, "wide_gemm: M=%d must be at most %d (N=%d K=%d)", M, MAX_ROWS, N, K);
  IFX_REQUIRE(K % 8 == 0, "wide_gemm: K=%d must be a multiple of 8", K);
  IFX_REQUIRE(out_dtype == DT_BF16 || out_dtype == DT_F32, "wide_gemm: unknown out dtype %d", out_dtype);
  IFX_REQUIRE(epi == 0 || (epi == 1 && N % 2 == 0 && !order && slices == 1), "wide_gemm: epilogue %d with N=%d, %d slices%s", epi, N,
              slices, order ? ", a tile order" : "");
  const int n_rounds = (K + WK - 1) / WK;
  IFX_REQUIRE(waves >= FEW_WAVES && waves <= MAX_WAVES && slices >= 1 && slices <= n_rounds, "wide_gemm: %d waves (%d-%d), %d slices of %d rounds",
              waves, FEW_WAVES, MAX_WAVES, slices, n_rounds);
  IFX_REQUIRE(M <= MANY_ROWS || waves == MIN_WAVES, "wide_gemm: %d rows take workgroups of %d waves, not %d", M, MIN_WAVES, waves);
  IFX_REQUIRE(slices == 1 || part, "wide_gemm: %d slices of K need a scratch buffer", slices);
  IFX_REQUIRE(!scale_pieces || (M <= 16 && n_scale_pieces > 0 && scale_width > 0.f),
              "wide_gemm: row factors take at most 16 rows (M=%d, %d pieces, width %g)", M, n_scale_pieces, (double)scale_width);
  const RowScale scale{scale_pieces, n_scale_pieces, scale_width, scale_eps};
  if (M == 0) return 0;
  const int rps = (n_rounds + slices - 1) / slices;
  IFX_REQUIRE((n_rounds + rps - 1) / rps == slices, "wide_gemm: %d rounds do not cut into %d slices (ask ifx_wide_gemm_plan)", n_rounds, slices);
  hipStream_t s = (hipStream_t)stream;
  switch ((M + 15) / 16) {
    case 1: return launch_wide<1>(x, Wt, out, out_dtype, part, M, N, K, waves, slices, rps, epi, order, out != nullptr, tile_rows, scale, s);
    case 2: return launch_wide<2>(x, Wt, out, out_dtype, part, M, N, K, waves, slices, rps, epi, order, out != nullptr, tile_rows, scale, s);
    case 3: return launch_wide<3>(x, Wt, out, out_dtype, part, M, N, K, waves, slices, rps, epi, order, out != nullptr, tile_rows, scale, s);
    case 4: return launch_wide<4>(x, Wt, out, out_dtype, part, M, N, K, waves, slices, rps, epi, order, out != nullptr, tile_rows, scale, s);
    case 5: return launch_wide<5>(x, Wt, out, out_dtype, part, M, N, K, waves, slices, rps, epi, order, out != nullptr, tile_rows, scale, s);
    case 6: return launch_wide<6>(x, Wt, out, out_dtype, part, M, N, K, waves, slices, rps, epi, order, out != nullptr, tile_rows, scale, s);
    case 7: return launch_wide<7>(x, Wt, out, out_dtype, part, M, N, K, waves, slices, rps, epi, order, out != nullptr, tile_rows, scale, s);
    default: return launch_wide<8>(x, Wt, out, out_dtype, part, M, N, K, waves, slices, rps, epi, order, out != nullptr, tile_rows, scale, s);
  }
}
