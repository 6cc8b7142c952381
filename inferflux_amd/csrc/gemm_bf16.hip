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
// The reference sends these products to cuBLAS (runtime/backends/cuda/native/cublas_gemm.cpp:
// 99-117) and measured 30-44 % of its roofline there (docs/benchmarks.md:180-183).
#include "common.h"

IFX_DEFINE_LAST_ERROR()

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

__device__ __forceinline__ bf16x8 zero8() {
  bf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = (__bf16)0.f;
  return z;
}

// EPI 0: out[m, n] = acc.  EPI 1: the rows of W alternate gate, up, gate, up ...; a lane holds two
// such pairs of one output row and writes silu(gate) * up to out[m, n / 2] (out is [M, N / 2]).
template <int MT, int NT, int U, typename TO, int EPI>
__global__ void skinny_gemm_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ W, TO* __restrict__ out,
                                   int M, int N, int K) {
  extern __shared__ float red[];  // [(waves - 1)][NT * MT][64 lanes][4]
  const int wid = threadIdx.x / WAVE, nw = blockDim.x / WAVE, lane = threadIdx.x % WAVE;
  const int col = lane & 15, g = lane >> 4;
  const int n_base = blockIdx.x * 16 * NT;
  floatx4 acc[NT][MT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[nt][mt] = floatx4{0.f, 0.f, 0.f, 0.f};

  const bf16_t* wrow[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) wrow[nt] = W + (size_t)min(n_base + 16 * nt + col, N - 1) * K;  // rows past N are read again, never stored
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
      const int k = (kb0 + u) * 64 + 16 * g;
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const bool kok = kb0 + u < nkb && k + 8 * h < K;
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) wa[u][nt][h] = kok ? *(const bf16x8*)(wrow[nt] + k + 8 * h) : zero8();
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) xa[u][mt][h] = (kok && xok[mt]) ? *(const bf16x8*)(xrow[mt] + k + 8 * h) : zero8();
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
    if (wid > 0) return;
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
  // acc[nt][mt][r] = out[m = 16 mt + col][n = n_base + 16 nt + 4 g + r]
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const int m = 16 * mt + col;
      if (m >= M) continue;
      if (EPI == 0) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int n = n_base + 16 * nt + 4 * g + r;
          if (n < N) out[(size_t)m * N + n] = from_f<TO>(acc[nt][mt][r]);
        }
      } else {
#pragma unroll
        for (int r = 0; r < 4; r += 2) {
          const int n = n_base + 16 * nt + 4 * g + r;  // even: gate at n, up at n + 1
          const float gt = acc[nt][mt][r], up = acc[nt][mt][r + 1];
          if (n + 1 < N) out[(size_t)m * (N / 2) + n / 2] = from_f<TO>(gt / (1.0f + expf(-gt)) * up);
        }
      }
    }
}

template <int MT, int NT, int U>
static int launch(const void* x, const void* W, void* out, int out_dtype, int M, int N, int K, int waves, int epi, hipStream_t s) {
  const int groups = (N + 16 * NT - 1) / (16 * NT);
  const size_t lds = (size_t)(waves - 1) * NT * MT * WAVE * 4 * sizeof(float);
  IFX_REQUIRE(lds <= 64 * 1024, "skinny_gemm: %d waves of %dx%d tiles need %zu bytes of LDS", waves, NT, MT, lds);
#define GO(TO_, EPI_)                                                                                              \
  hipLaunchKernelGGL((skinny_gemm_kernel<MT, NT, U, TO_, EPI_>), dim3(groups), dim3(waves * WAVE), lds, s,         \
                     (const bf16_t*)x, (const bf16_t*)W, (TO_*)out, M, N, K)
  if (out_dtype == DT_BF16 && epi == 0) GO(bf16_t, 0);
  else if (out_dtype == DT_BF16) GO(bf16_t, 1);
  else if (epi == 0) GO(float, 0);
  else GO(float, 1);
#undef GO
  IFX_LAUNCH_CHECK();
}

// nt, waves, unroll = 0: chosen here from the shape.
// epi 1: gate/up rows interleaved in W, out = silu(gate) * up, [M, N / 2].
extern "C" int ifx_skinny_gemm(const void* x, const void* W, void* out, int out_dtype, int M, int N, int K, int nt,
                               int waves, int unroll, int epi, void* stream) {
  IFX_REQUIRE(epi == 0 || (epi == 1 && N % 2 == 0), "skinny_gemm: epilogue %d with N=%d", epi, N);
  IFX_REQUIRE(M >= 0 && M <= 64 && N > 0 && K > 0, "skinny_gemm: M=%d must be at most 64 (N=%d K=%d)", M, N, K);
  IFX_REQUIRE(K % 8 == 0, "skinny_gemm: K=%d must be a multiple of 8", K);
  IFX_REQUIRE(out_dtype == DT_BF16 || out_dtype == DT_F32, "skinny_gemm: unknown out dtype %d", out_dtype);
  if (M == 0) return 0;
  const int mt = (M + 15) / 16;
  const int nkb = (K + 63) / 64;
  // Choices measured on the 7B shapes at 1-16 rows: two row tiles per wave pay off only for very tall
  // weights; deeper unrolling than 4 blocks spills; about 1500-2500 waves fill the chip.
  if (nt == 0) nt = (N >= 32768 && mt <= 2) ? 2 : 1;
  if (unroll == 0) unroll = (mt * nt >= 2) ? 2 : 4;
  if (waves == 0) {
    const int groups = (N + 16 * nt - 1) / (16 * nt);
    waves = 1;
    if (groups < 1024)
      while (waves < 16 && groups * waves < 1536 && nkb >= waves * 2) waves *= 2;
    while (waves > 1 && (size_t)(waves - 1) * nt * mt * WAVE * 16 > 64 * 1024) waves /= 2;
  }
  IFX_REQUIRE(waves >= 1 && waves <= 16, "skinny_gemm: waves=%d outside 1..16", waves);
  hipStream_t s = (hipStream_t)stream;
#define CASE(MT_, NT_, U_) if (mt == MT_ && nt == NT_ && unroll == U_) return launch<MT_, NT_, U_>(x, W, out, out_dtype, M, N, K, waves, epi, s)
  CASE(1, 1, 4); CASE(1, 2, 4); CASE(1, 1, 2); CASE(1, 2, 2); CASE(1, 1, 8); CASE(1, 2, 8);
  CASE(2, 1, 4); CASE(2, 2, 2); CASE(2, 1, 2); CASE(2, 2, 4);
  CASE(3, 1, 2); CASE(3, 2, 2); CASE(3, 1, 4);
  CASE(4, 1, 2); CASE(4, 2, 2); CASE(4, 1, 4);
#undef CASE
  IFX_FAIL("skinny_gemm: no kernel for m-tiles=%d n-tiles=%d unroll=%d", mt, nt, unroll);
}
