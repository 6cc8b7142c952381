// What this card's memory gives to a kernel that does nothing else: the yardstick beside the figures of the
// data sheet for kernels that are bound by reading weights or the cache.  Not part of any model's step.
//
//   stream_read : every wave reads contiguous kilobytes (16 bytes a lane, UNROLL loads on their way), the grid
//                 strides over the region; plain loads or streaming ("nontemporal") ones.  The sum of what was
//                 read is compared with a value it cannot have, so that no load is dropped.
//   stream_copy : the same with a store of every piece.
//
// The reference has no such tool: its figures come from whole runs through the HTTP server (docs/benchmarks.md:56-91).
#include "common.h"

IFX_DEFINE_LAST_ERROR()

typedef float f4 __attribute__((ext_vector_type(4)));
constexpr int UNROLL = 8;                      // 8 KB of a wave on their way
constexpr size_t PIECE = WAVE * sizeof(f4);    // one load of a wave: 1 KB

template <bool STREAMING>
__global__ __launch_bounds__(WAVE) void stream_read_kernel(const f4* __restrict__ src, size_t rounds, float* __restrict__ sink) {
  const int lane = threadIdx.x;
  f4 acc = {0.f, 0.f, 0.f, 0.f};
  for (size_t r = blockIdx.x; r < rounds; r += gridDim.x) {
    const f4* p = src + r * (UNROLL * WAVE) + lane;
    f4 v[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) v[u] = STREAMING ? __builtin_nontemporal_load(p + u * WAVE) : p[u * WAVE];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) acc += v[u];
  }
  if (acc.x + acc.y + acc.z + acc.w == 1.2345e38f) sink[0] = acc.x;      // never true for finite data that sums elsewhere
}

template <bool STREAMING>
__global__ __launch_bounds__(WAVE) void stream_copy_kernel(const f4* __restrict__ src, f4* __restrict__ dst, size_t rounds) {
  const int lane = threadIdx.x;
  for (size_t r = blockIdx.x; r < rounds; r += gridDim.x) {
    const size_t at = r * (UNROLL * WAVE) + lane;
    f4 v[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) v[u] = STREAMING ? __builtin_nontemporal_load(src + at + u * WAVE) : src[at + u * WAVE];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      if (STREAMING) __builtin_nontemporal_store(v[u], dst + at + u * WAVE);
      else dst[at + u * WAVE] = v[u];
    }
  }
}

static int check(const void* src, long long bytes, int waves) {
  IFX_REQUIRE(src != nullptr && bytes > 0 && bytes % (long long)(UNROLL * PIECE) == 0,
              "stream: %lld bytes is not a positive multiple of %zu", bytes, UNROLL * PIECE);
  IFX_REQUIRE(((uintptr_t)src & 15) == 0, "stream: the region does not start at a multiple of 16 bytes");
  IFX_REQUIRE(waves > 0 && waves <= (1 << 20), "stream: %d waves", waves);
  return 0;
}

// Reads ``bytes`` from src with ``waves`` one-wave workgroups.  sink: one float that is never written for finite data.
extern "C" int ifx_stream_read(const void* src, long long bytes, int waves, int streaming, float* sink, void* stream) {
  if (int rc = check(src, bytes, waves)) return rc;
  IFX_REQUIRE(sink != nullptr, "stream_read: no sink");
  const size_t rounds = (size_t)bytes / (UNROLL * PIECE);
  hipStream_t s = (hipStream_t)stream;
  if (streaming) hipLaunchKernelGGL(stream_read_kernel<true>, dim3(waves), dim3(WAVE), 0, s, (const f4*)src, rounds, sink);
  else hipLaunchKernelGGL(stream_read_kernel<false>, dim3(waves), dim3(WAVE), 0, s, (const f4*)src, rounds, sink);
  IFX_LAUNCH_CHECK();
}

// Copies ``bytes`` from src to dst (regions that do not overlap).
extern "C" int ifx_stream_copy(const void* src, void* dst, long long bytes, int waves, int streaming, void* stream) {
  if (int rc = check(src, bytes, waves)) return rc;
  IFX_REQUIRE(dst != nullptr && ((uintptr_t)dst & 15) == 0, "stream_copy: bad destination");
  const char *a = (const char*)src, *b = (const char*)dst;
  IFX_REQUIRE(a + bytes <= b || b + bytes <= a, "stream_copy: the regions overlap");
  const size_t rounds = (size_t)bytes / (UNROLL * PIECE);
  hipStream_t s = (hipStream_t)stream;
  if (streaming) hipLaunchKernelGGL(stream_copy_kernel<true>, dim3(waves), dim3(WAVE), 0, s, (const f4*)src, (f4*)dst, rounds);
  else hipLaunchKernelGGL(stream_copy_kernel<false>, dim3(waves), dim3(WAVE), 0, s, (const f4*)src, (f4*)dst, rounds);
  IFX_LAUNCH_CHECK();
}
