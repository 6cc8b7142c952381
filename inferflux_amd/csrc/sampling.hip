// Sampling from float logits [R, V]: argmax, penalties, logit bias, and temperature softmax
// with top-k / top-p / min-p filters followed by a walk along the cumulative distribution.
//
// Reference behaviour (runtime/backends/cuda/native/gpu_sampler.cu): greedy when temperature
// <= 0 (608-623); otherwise softmax(logits / temperature) (216-267), a top-p mask that keeps
// tokens in descending probability until the running sum reaches top_p, the crossing token
// included (273-330), then one uniform number and a walk along the cumulative sum in index
// order, falling back to the last index (374-401).  Penalties: 22-48.  The reference ignores
// top_k and min_p on this path (563-567); here they are honoured.  Its argmax keeps the lowest
// index only within one thread's stride (124-156); here the lowest index always wins a tie.
//
// The filters are expressed as thresholds on the unnormalised weight w_i = exp(l_i/T - max):
// a filter keeps every token whose weight is >= its threshold, found by bisection over the
// bit patterns of positive floats, so tokens of equal weight are kept or dropped together.
#include "common.h"
#include "sampling.h"

#include <mutex>

IFX_DEFINE_LAST_ERROR()

#define SAMPLE_THREADS 1024

// ---------------------------------------------------------------------------------------
__device__ __forceinline__ void argmax_merge(float& v, int& i, float ov, int oi) {
  if (ov > v || (ov == v && oi < i)) { v = ov; i = oi; }
}

// Lowest index among the maxima of row r.  NaN never wins.  Every thread returns the result.
__device__ int block_argmax(const float* __restrict__ row, int V, float* red_v, int* red_i) {
  float bv = -INFINITY;
  int bi = V;  // larger than any index: the first element with value -inf still wins below
  for (int i = threadIdx.x; i < V; i += blockDim.x) {
    const float x = row[i];
    if (x > bv || (x == bv && i < bi)) { bv = x; bi = i; }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_xor(bv, o, WAVE);
    const int oi = __shfl_xor(bi, o, WAVE);
    argmax_merge(bv, bi, ov, oi);
  }
  const int wid = threadIdx.x / WAVE, lane = threadIdx.x % WAVE, nw = blockDim.x / WAVE;
  __syncthreads();
  if (lane == 0) { red_v[wid] = bv; red_i[wid] = bi; }
  __syncthreads();
  bv = red_v[0]; bi = red_i[0];
  for (int w = 1; w < nw; ++w) argmax_merge(bv, bi, red_v[w], red_i[w]);
  return bi < V ? bi : 0;
}

__global__ __launch_bounds__(SAMPLE_THREADS) void argmax_kernel(const float* __restrict__ logits, int V,
                                                               int* __restrict__ out) {
  __shared__ float red_v[16];
  __shared__ int red_i[16];
  const int r = blockIdx.x;
  const int best = block_argmax(logits + (size_t)r * V, V, red_v, red_i);
  if (threadIdx.x == 0) out[r] = best;
}

// Two stages for wide rows, so that a handful of rows still fills the chip: stage 1 finds the best
// of each of ARGMAX_SLICES slices of a row, stage 2 the best of those (lowest index on ties in both).
#define ARGMAX_SLICES 32

__global__ __launch_bounds__(256) void argmax_slices_kernel(const float* __restrict__ logits, int V, float* __restrict__ pv,
                                                            int* __restrict__ pi) {
  __shared__ float red_v[16];
  __shared__ int red_i[16];
  const int r = blockIdx.y, sl = blockIdx.x;
  const int per = (V + ARGMAX_SLICES - 1) / ARGMAX_SLICES;
  const int lo = min(V, sl * per), hi = min(V, lo + per);
  const float* row = logits + (size_t)r * V;
  int best = hi > lo ? lo + block_argmax(row + lo, hi - lo, red_v, red_i) : V;
  if (threadIdx.x == 0) {
    pv[r * ARGMAX_SLICES + sl] = best < V ? row[best] : -INFINITY;
    pi[r * ARGMAX_SLICES + sl] = best;
  }
}

__global__ __launch_bounds__(WAVE) void argmax_final_kernel(const float* __restrict__ pv, const int* __restrict__ pi, int V,
                                                           int* __restrict__ out) {
  const int r = blockIdx.x, lane = threadIdx.x;
  float bv = lane < ARGMAX_SLICES ? pv[r * ARGMAX_SLICES + lane] : -INFINITY;
  int bi = lane < ARGMAX_SLICES ? pi[r * ARGMAX_SLICES + lane] : V;
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_xor(bv, o, WAVE);
    const int oi = __shfl_xor(bi, o, WAVE);
    argmax_merge(bv, bi, ov, oi);
  }
  if (lane == 0) out[r] = bi < V ? bi : 0;
}

// scratch: ARGMAX_SLICES floats and ints per row (used when V is large), or null.
extern "C" int ifx_argmax(const float* logits, int R, int V, int* out, float* scratch_v, int* scratch_i, void* stream) {
  IFX_REQUIRE(R >= 0 && V > 0, "argmax: bad sizes R=%d V=%d", R, V);
  if (R == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  if (V >= 16384 && scratch_v && scratch_i && R <= 65535) {
    hipLaunchKernelGGL(argmax_slices_kernel, dim3(ARGMAX_SLICES, R), dim3(256), 0, s, logits, V, scratch_v, scratch_i);
    hipLaunchKernelGGL(argmax_final_kernel, dim3(R), dim3(WAVE), 0, s, scratch_v, scratch_i, V, out);
  } else {
    hipLaunchKernelGGL(argmax_kernel, dim3(R), dim3(SAMPLE_THREADS), 0, s, logits, V, out);
  }
  IFX_LAUNCH_CHECK();
}

// The same two stages with their scratch in a file-scope device array instead of a workspace of the caller's: the entry
// point for callers that cannot allocate (see sampling.h).  In host code the array's name is only a stand-in for the
// symbol: the address the kernels are given is looked up per device with hipGetSymbolAddress, once, and kept.
#define ARGMAX_STATIC_BYTES (IFX_ARGMAX_STATIC_MAX_ROWS * ARGMAX_SLICES * (sizeof(float) + sizeof(int)))
static __device__ __align__(256) unsigned char scratch[ARGMAX_STATIC_BYTES];

#define ARGMAX_STATIC_MAX_DEVICES 64
static void* g_scratch_ptr[ARGMAX_STATIC_MAX_DEVICES];   // per device: that device's copy of `scratch`, or null before its first call
static std::mutex g_scratch_mutex;

// The address of the current device's `scratch` (each GPU holds its own copy at its own address).
static int argmax_static_scratch(void** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) IFX_FAIL("argmax_static: hipGetDevice failed: %s", hipGetErrorString(e));
  IFX_REQUIRE(dev >= 0 && dev < ARGMAX_STATIC_MAX_DEVICES, "argmax_static: device %d outside 0..%d", dev, ARGMAX_STATIC_MAX_DEVICES - 1);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || ptr == nullptr)
      IFX_FAIL("argmax_static: hipGetSymbolAddress(scratch) failed on device %d: %s", dev, hipGetErrorString(e));
    g_scratch_ptr[dev] = ptr;
  }
  *out = g_scratch_ptr[dev];
  return 0;
}

extern "C" int ifx_argmax_static(const float* logits, int R, int V, int* out, void* stream) {
  IFX_REQUIRE(R >= 0 && V > 0, "argmax_static: bad sizes R=%d V=%d", R, V);
  IFX_REQUIRE(R <= IFX_ARGMAX_STATIC_MAX_ROWS, "argmax_static: %d rows, the static scratch holds at most %d", R,
              IFX_ARGMAX_STATIC_MAX_ROWS);
  if (R == 0) return 0;
  IFX_REQUIRE(logits != nullptr && out != nullptr, "argmax_static: null logits or out");
  void* ptr = nullptr;
  if (const int rc = argmax_static_scratch(&ptr)) return rc;
  // the floats of all R rows first, then the ints (both 4 bytes wide, so both parts stay aligned)
  float* pv = (float*)ptr;
  int* pi = (int*)((unsigned char*)ptr + (size_t)IFX_ARGMAX_STATIC_MAX_ROWS * ARGMAX_SLICES * sizeof(float));
  return ifx_argmax(logits, R, V, out, pv, pi, stream);
}

// ---------------------------------------------------------------------------------------
// Entry e names (row, token id, count).  The logit of that token in that row becomes
//   l = l > 0 ? l / rep[row] : l * rep[row];  l -= freq[row] * count;  if count > 0: l -= pres[row]
// Each (row, id) pair appears at most once.
__global__ void penalties_kernel(float* __restrict__ logits, int V, const int* __restrict__ rows,
                                 const int* __restrict__ ids, const int* __restrict__ counts, int n,
                                 const float* __restrict__ rep, const float* __restrict__ freq,
                                 const float* __restrict__ pres) {
  const int e = blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= n) return;
  const int r = rows[e], id = ids[e];
  if (id < 0 || id >= V) return;
  float l = logits[(size_t)r * V + id];
  l = l > 0.f ? l / rep[r] : l * rep[r];
  const int c = counts[e];
  l -= freq[r] * (float)c;
  if (c > 0) l -= pres[r];
  logits[(size_t)r * V + id] = l;
}

extern "C" int ifx_apply_penalties(float* logits, int V, const int* rows, const int* ids, const int* counts,
                                   int n, const float* rep, const float* freq, const float* pres, void* stream) {
  IFX_REQUIRE(n >= 0 && V > 0, "penalties: bad sizes");
  if (n == 0) return 0;
  hipLaunchKernelGGL(penalties_kernel, dim3((n + 255) / 256), dim3(256), 0, (hipStream_t)stream, logits, V, rows,
                     ids, counts, n, rep, freq, pres);
  IFX_LAUNCH_CHECK();
}

// logits[rows[e], ids[e]] += bias[e]; each (row, id) pair appears at most once.
__global__ void logit_bias_kernel(float* __restrict__ logits, int V, const int* __restrict__ rows,
                                  const int* __restrict__ ids, const float* __restrict__ bias, int n) {
  const int e = blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= n) return;
  const int id = ids[e];
  if (id < 0 || id >= V) return;
  logits[(size_t)rows[e] * V + id] += bias[e];
}

extern "C" int ifx_add_logit_bias(float* logits, int V, const int* rows, const int* ids, const float* bias,
                                  int n, void* stream) {
  IFX_REQUIRE(n >= 0 && V > 0, "logit_bias: bad sizes");
  if (n == 0) return 0;
  hipLaunchKernelGGL(logit_bias_kernel, dim3((n + 255) / 256), dim3(256), 0, (hipStream_t)stream, logits, V, rows,
                     ids, bias, n);
  IFX_LAUNCH_CHECK();
}

// ---------------------------------------------------------------------------------------
struct SampleArgs {
  const float* logits;  // [R, V]
  float* weights;       // [R, V] scratch
  const float* temperature;
  const int* top_k;
  const float* top_p;
  const float* min_p;
  const float* uniform;  // one number in [0, 1) per row, or null:
  const unsigned* draws; // then [R, 4]: the row's seed and the number of its draw, 64 bits each, low word first
  int* out;
  int V;
};

// The top 24 bits of the first word of Philox4x32-10 (Salmon et al. 2011) keyed by the seed at counter (step, 0), as a
// number in [0, 1): it depends on the pair alone, so a request draws the same numbers whatever shares its batch.
__device__ float philox_uniform(unsigned seed_lo, unsigned seed_hi, unsigned step_lo, unsigned step_hi) {
  unsigned c0 = step_lo, c1 = step_hi, c2 = 0, c3 = 0, k0 = seed_lo, k1 = seed_hi;
  for (int round = 0; round < 10; ++round) {
    const unsigned long long p0 = 0xD2511F53ull * c0, p1 = 0xCD9E8D57ull * c2;
    const unsigned n0 = (unsigned)(p1 >> 32) ^ c1 ^ k0, n2 = (unsigned)(p0 >> 32) ^ c3 ^ k1;
    c0 = n0; c1 = (unsigned)p1; c2 = n2; c3 = (unsigned)p0;
    k0 += 0x9E3779B9u; k1 += 0xBB67AE85u;
  }
  return (float)(c0 >> 8) * (1.0f / 16777216.0f);
}

__device__ __forceinline__ int block_sum_int(int v, int* red) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, WAVE);
  const int wid = threadIdx.x / WAVE, lane = threadIdx.x % WAVE, nw = blockDim.x / WAVE;
  __syncthreads();
  if (lane == 0) red[wid] = v;
  __syncthreads();
  int t = 0;
  for (int i = 0; i < nw; ++i) t += red[i];
  return t;
}

// Calls f(i, p[i]) for every i < n, each index from exactly one thread of the block, with 16-byte loads where the
// row's address allows (a few of them in flight per thread: one workgroup has to keep a whole row moving).
template <typename F>
__device__ __forceinline__ void block_visit(const float* __restrict__ p, int n, F f) {
  const int head = min(n, (int)(((16 - ((size_t)p & 15)) & 15) >> 2));
  if ((int)threadIdx.x < head) f((int)threadIdx.x, p[threadIdx.x]);
  const float4* p4 = reinterpret_cast<const float4*>(p + head);
  const int n4 = (n - head) >> 2;
#pragma unroll 4
  for (int i = threadIdx.x; i < n4; i += blockDim.x) {
    const float4 v = p4[i];
    const int b = head + 4 * i;
    f(b, v.x); f(b + 1, v.y); f(b + 2, v.z); f(b + 3, v.w);
  }
  const int t = head + 4 * n4 + (int)threadIdx.x;
  if (t < n) f(t, p[t]);
}

// q[i] = f(p[i]) for every i < n; 16-byte loads and stores where both rows' addresses allow.
template <typename F>
__device__ __forceinline__ void block_map(const float* __restrict__ p, float* __restrict__ q, int n, F f) {
  if ((((size_t)p ^ (size_t)q) & 15) != 0) {
    for (int i = threadIdx.x; i < n; i += blockDim.x) q[i] = f(p[i]);
    return;
  }
  const int head = min(n, (int)(((16 - ((size_t)p & 15)) & 15) >> 2));
  if ((int)threadIdx.x < head) q[threadIdx.x] = f(p[threadIdx.x]);
  const float4* p4 = reinterpret_cast<const float4*>(p + head);
  float4* q4 = reinterpret_cast<float4*>(q + head);
  const int n4 = (n - head) >> 2;
#pragma unroll 4
  for (int i = threadIdx.x; i < n4; i += blockDim.x) {
    float4 v = p4[i];
    v.x = f(v.x); v.y = f(v.y); v.z = f(v.z); v.w = f(v.w);
    q4[i] = v;
  }
  const int t = head + 4 * n4 + (int)threadIdx.x;
  if (t < n) q[t] = f(p[t]);
}

// The thresholds of top-k and top-p are exact selections among the weights of one row.  A histogram over the upper
// bits of the weights' bit patterns (sign and exponent and the first HIST_MANTISSA bits of the mantissa: HIST_BINS
// bins, the largest weight 1.0 falls into bin 2032) says which bin each threshold lies in; the weights from the
// lower of these bins upwards (the candidates: usually a few hundred of the row) are gathered in LDS, and one
// wave bisects over the bit patterns within the bin there.  Counts are integers and sums are sums of the
// weights in fixed point (units of 2^-40, so a row of a million weights of 1.0 stays below 2^64): neither depends
// on the order in which the threads add, and the histogram's sums and the candidates' agree exactly.  A row whose
// candidates do not fit (more than SAMPLE_CANDIDATES: a wide nucleus) goes over the whole row twice more per threshold
// instead: the weights of the threshold's bin are counted by their next ten bits, then those of that sub-bin by
// their last nine (refine_threshold).
#define HIST_MANTISSA 4
#define HIST_SHIFT (23 - HIST_MANTISSA)
#define HIST_BINS 2048
#define SAMPLE_CANDIDATES 3072
typedef unsigned long long u64;

__device__ __forceinline__ u64 weight_fixed(float x) { return (u64)(x * 1099511627776.0f); }   // x * 2^40, x in [0, 1]

__device__ __forceinline__ u64 wave_sum_u64(u64 v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, WAVE);
  return v;
}
__device__ __forceinline__ int wave_sum_int(int v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, WAVE);
  return v;
}

struct SampleShared {
  float cand[SAMPLE_CANDIDATES];
  unsigned count[HIST_BINS];     // after the scan: the number of weights in this bin or a higher one
  u64 sum[HIST_BINS];            // after the scan: their sum in fixed point
  unsigned wave_count[16];
  u64 wave_sum[16];
  float seg_sum[16];
  int seg_last[16];
  float red_f[16];
  int red_i[16];
  unsigned n_cand;
  int bin_k, bin_p, bin_cand;
  unsigned thr_bits;
  int pick;
};

// count[b] and sum[b] (where SUMS) become the totals over the bins b and above.  Bin 0 (zero and the smallest
// denormals) is not counted by the threads: it is given what is left of the V weights.  All SAMPLE_THREADS threads, two
// bins each, the highest bins first.
template <bool SUMS>
__device__ void histogram_suffix_scan(unsigned* count, u64* sum, unsigned* wave_count, u64* wave_sum, int V) {
  const int tid = threadIdx.x, lane = tid % WAVE, wid = tid / WAVE;
  const int b0 = HIST_BINS - 1 - 2 * tid, b1 = b0 - 1;
  const unsigned c0 = count[b0], c1 = count[b1];
  const u64 s0 = SUMS ? sum[b0] : 0, s1 = SUMS ? sum[b1] : 0;
  unsigned ci = c0 + c1;
  u64 si = s0 + s1;
#pragma unroll
  for (int o = 1; o < WAVE; o <<= 1) {
    const unsigned oc = __shfl_up(ci, o, WAVE);
    if (lane >= o) ci += oc;
    if (SUMS) {
      const u64 os = __shfl_up(si, o, WAVE);
      if (lane >= o) si += os;
    }
  }
  if (lane == WAVE - 1) {
    wave_count[wid] = ci;
    if (SUMS) wave_sum[wid] = si;
  }
  __syncthreads();
  unsigned cb = 0;
  u64 sb = 0;
  for (int i = 0; i < wid; ++i) {
    cb += wave_count[i];
    if (SUMS) sb += wave_sum[i];
  }
  const unsigned ce = cb + ci - (c0 + c1);
  count[b0] = ce + c0;
  count[b1] = b1 == 0 ? (unsigned)V : ce + c0 + c1;
  if (SUMS) {
    const u64 se = sb + si - (s0 + s1);
    sum[b0] = se + s0;
    sum[b1] = se + s0 + s1;
  }
  __syncthreads();
}

// The largest bin in [lo, hi] whose entry of a non-increasing table is >= need; lo if none is (the caller knows that lo's is).
template <typename T>
__device__ __forceinline__ int last_bin_reaching(const T* table, T need, int lo, int hi) {
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (table[mid] >= need) lo = mid; else hi = mid - 1;
  }
  return lo;
}

// The exact threshold inside bin ``bin1`` of the histogram, over the whole row: the largest pattern t for which the
// weights >= t number at least ``need`` (BY_SUM false) or sum to at least ``need`` in fixed point (BY_SUM true), given
// what lies above the bin (``above_count`` weights that sum to ``above_sum``) and that the bin's lower edge satisfies
// it.  Two passes: the bin's weights by the next ten bits of their patterns, then the chosen sub-bin's by the last
// nine.  The histograms live in the memory of the candidates, which such a row does not use.  Every thread returns
// the pattern and the sum of the weights that reach it.
struct Refined { unsigned bits; u64 sum_from; };

template <bool BY_SUM>
__device__ Refined refine_threshold(const float* __restrict__ w, int V, unsigned bin1, unsigned above_count, u64 above_sum,
                                    u64 need, SampleShared& sh) {
  static_assert(SAMPLE_THREADS == 1024 && SAMPLE_CANDIDATES * sizeof(float) >= 1024 * (sizeof(unsigned) + sizeof(u64)),
                "one sub-bin per thread, in the candidates' memory");
  unsigned* c2 = reinterpret_cast<unsigned*>(sh.cand);
  u64* s2 = reinterpret_cast<u64*>(sh.cand + 1024);
  const int tid = threadIdx.x, lane = tid % WAVE, wid = tid / WAVE;
  unsigned prefix = bin1;      // the pattern's bits from ``shift`` upwards
  int shift = HIST_SHIFT;
  u64 reach_sum = 0;
  for (int level = 0; level < 2; ++level) {
    const int width = level == 0 ? 10 : shift;     // 10 bits, then the 9 that are left
    const int below = shift - width;
    const unsigned mask = (1u << width) - 1;
    __syncthreads();                               // (the last level's tables have been read)
    c2[tid] = 0;
    s2[tid] = 0;
    __syncthreads();
    block_visit(w, V, [&](int, float x) {
      const unsigned b = __float_as_uint(x);
      if ((b >> shift) == prefix) {
        const unsigned sub = (b >> below) & mask;
        atomicAdd(&c2[sub], 1u);
        atomicAdd(&s2[sub], weight_fixed(x));
      }
    });
    __syncthreads();
    // totals over the sub-bins from each one upwards: thread t has sub-bin 1023 - t
    unsigned ci = c2[1023 - tid];
    u64 si = s2[1023 - tid];
#pragma unroll
    for (int o = 1; o < WAVE; o <<= 1) {
      const unsigned oc = __shfl_up(ci, o, WAVE);
      const u64 os = __shfl_up(si, o, WAVE);
      if (lane >= o) { ci += oc; si += os; }
    }
    if (lane == WAVE - 1) { sh.wave_count[wid] = ci; sh.wave_sum[wid] = si; }
    __syncthreads();
    for (int i = 0; i < wid; ++i) { ci += sh.wave_count[i]; si += sh.wave_sum[i]; }
    c2[1023 - tid] = ci;
    s2[1023 - tid] = si;
    __syncthreads();
    int lo = 0, hi = (int)mask;                    // (every thread searches: the tables are in LDS)
    while (lo < hi) {
      const int mid = (lo + hi + 1) >> 1;
      const bool reached = BY_SUM ? above_sum + s2[mid] >= need : (u64)above_count + c2[mid] >= need;
      if (reached) lo = mid; else hi = mid - 1;
    }
    reach_sum = above_sum + s2[lo];
    if (lo < (int)mask) { above_count += c2[lo + 1]; above_sum += s2[lo + 1]; }
    prefix = (prefix << width) | (unsigned)lo;
    shift = below;
  }
  return Refined{prefix, reach_sum};
}

// The token at which the cumulative sum of the kept weights (those with bit pattern >= thr_bits), taken in index
// order, passes uniform * total.  Two rounds in which the 16 waves each sum a sixteenth of the range and the part
// that holds the target becomes the range, then one wave walks what is left, 64 weights at a time.  Every thread
// returns the token.  A target that rounding puts past the end of a range gives the range's last kept index.
__device__ int cumulative_pick(const float* __restrict__ w, int V, unsigned thr_bits, float uniform, SampleShared& sh) {
  const int tid = threadIdx.x, lane = tid % WAVE, wid = tid / WAVE, nw = blockDim.x / WAVE;
  int lo = 0, hi = V;
  float target = 0.f;
  for (int level = 0; level < 2; ++level) {
    const int seg = ((hi - lo + nw - 1) / nw + WAVE - 1) / WAVE * WAVE;
    const int s0 = min(hi, lo + wid * seg), s1 = min(hi, s0 + seg);
    float mine = 0.f;
    int last = -1;
#pragma unroll 4
    for (int i = s0 + lane; i < s1; i += WAVE) {
      const float x = w[i];
      if (__float_as_uint(x) >= thr_bits) { mine += x; last = i; }
    }
    mine = wave_sum(mine);
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) last = max(last, __shfl_xor(last, o, WAVE));
    __syncthreads();   // the arrays may still be read from the round before
    if (lane == 0) { sh.seg_sum[wid] = mine; sh.seg_last[wid] = last; }
    __syncthreads();
    if (level == 0) {
      float total = 0.f;
      for (int i = 0; i < nw; ++i) total += sh.seg_sum[i];
      target = uniform * total;
    }
    int sel = -1, last_any = -1;
    float before = 0.f;
    for (int i = 0; i < nw; ++i) {
      const float s = sh.seg_sum[i];
      last_any = max(last_any, sh.seg_last[i]);
      if (s > 0.f && target - before < s) { sel = i; break; }
      before += s;
    }
    if (sel < 0) return max(last_any, 0);
    target -= before;
    lo = min(hi, lo + sel * seg);
    hi = min(hi, lo + seg);
  }
  __syncthreads();
  if (wid == 0) {
    float run = 0.f;
    int pick = -1, last = -1;
    for (int g = lo; g < hi && pick < 0; g += WAVE) {
      const int i = g + lane;
      const float x = i < hi ? w[i] : 0.f;
      const bool kept = i < hi && __float_as_uint(x) >= thr_bits;
      float cum = kept ? x : 0.f;
#pragma unroll
      for (int o = 1; o < WAVE; o <<= 1) {
        const float up = __shfl_up(cum, o, WAVE);
        if (lane >= o) cum += up;
      }
      cum += run;
      const u64 hit = __ballot(kept && target < cum);
      const u64 any = __ballot(kept);
      if (hit) pick = g + __ffsll((long long)hit) - 1;
      if (any) last = g + 63 - __clzll((long long)any);
      run = __shfl(cum, WAVE - 1, WAVE);
    }
    if (lane == 0) sh.pick = pick >= 0 ? pick : max(last, 0);
  }
  __syncthreads();
  return sh.pick;
}

__global__ __launch_bounds__(SAMPLE_THREADS) void sample_kernel(SampleArgs a) {
  __shared__ SampleShared sh;
  const int r = blockIdx.x, V = a.V, tid = threadIdx.x, lane = tid % WAVE, wid = tid / WAVE;
  const float* row = a.logits + (size_t)r * V;
  const float temp = a.temperature[r];
  if (!(temp > 0.f)) {
    const int best = block_argmax(row, V, sh.red_f, sh.red_i);
    if (tid == 0) a.out[r] = best;
    return;
  }
  float* w = a.weights + (size_t)r * V;
  const float inv_t = 1.0f / temp;
  const int k = a.top_k[r];
  const float top_p = a.top_p[r];
  const bool k_on = k > 0 && k < V, p_on = top_p > 0.f && top_p < 1.f;

  float mx = -INFINITY;
  block_visit(row, V, [&](int, float l) { mx = fmaxf(mx, l * inv_t); });
  mx = block_max(mx, sh.red_f);

  // Thresholds as bit patterns: for non-negative floats the order of the values is the order
  // of their bits.  The largest weight is exp(0) = 1.
  const unsigned one_bits = __float_as_uint(1.0f);
  unsigned thr_bits = 0;  // keep everything
  if (!k_on && !p_on) {
    block_map(row, w, V, [&](float l) { return expf(l * inv_t - mx); });
    __syncthreads();
  } else {
    for (int b = tid; b < HIST_BINS; b += blockDim.x) { sh.count[b] = 0; sh.sum[b] = 0; }
    if (tid == 0) sh.n_cand = 0;
    __syncthreads();
    block_map(row, w, V, [&](float l) {
      const float x = expf(l * inv_t - mx);
      const unsigned b = __float_as_uint(x) >> HIST_SHIFT;
      if (b && b < HIST_BINS) {   // (a NaN's pattern lies beyond the last bin)
        atomicAdd(&sh.count[b], 1u);
        atomicAdd(&sh.sum[b], weight_fixed(x));
      }
      return x;
    });
    __syncthreads();
    histogram_suffix_scan<true>(sh.count, sh.sum, sh.wave_count, sh.wave_sum, V);
    if (tid == 0) {
      const int top_bin = one_bits >> HIST_SHIFT;
      int bk = 0, bp = 0, bc = top_bin;
      if (k_on) { bk = last_bin_reaching(sh.count, (unsigned)k, 0, top_bin); bc = min(bc, bk); }
      if (p_on) {
        // at least what the exact rule will ask for: top-k keeps no more than the bins from bk upwards hold
        const u64 need = (u64)((double)top_p * (double)sh.sum[bk]);
        bp = last_bin_reaching(sh.sum, need, 0, top_bin);
        bc = min(bc, bp);
      }
      sh.bin_k = bk; sh.bin_p = bp; sh.bin_cand = bc;
    }
    __syncthreads();
    const int bk = sh.bin_k, bc = sh.bin_cand;
    if (sh.count[bc] <= SAMPLE_CANDIDATES) {
      const unsigned first_bits = (unsigned)bc << HIST_SHIFT;
      block_visit(w, V, [&](int, float x) {
        if (__float_as_uint(x) >= first_bits) {
          const unsigned at = atomicAdd(&sh.n_cand, 1u);
          if (at < SAMPLE_CANDIDATES) sh.cand[at] = x;
        }
      });
      __syncthreads();
      if (wid == 0) {
        const int n = min(sh.n_cand, (unsigned)SAMPLE_CANDIDATES);
        if (k_on) {  // the largest pattern that at least k weights reach: it lies in bin bk
          unsigned lo = (unsigned)bk << HIST_SHIFT, hi = min(((unsigned)(bk + 1) << HIST_SHIFT) - 1, one_bits);
          while (lo < hi) {
            const unsigned mid = lo + (hi - lo + 1) / 2;
            int c = 0;
            for (int i = lane; i < n; i += WAVE) c += __float_as_uint(sh.cand[i]) >= mid ? 1 : 0;
            if (wave_sum_int(c) >= k) lo = mid; else hi = mid - 1;
          }
          thr_bits = lo;
        }
        if (p_on) {  // the largest pattern whose weights and all larger ones sum to top_p of what top-k kept
          u64 kept = 0;
          for (int i = lane; i < n; i += WAVE) {
            const float x = sh.cand[i];
            if (__float_as_uint(x) >= thr_bits) kept += weight_fixed(x);
          }
          const u64 kept_all = k_on ? wave_sum_u64(kept) : sh.sum[0];   // without top-k: the whole row, not the candidates
          const u64 need = (u64)((double)top_p * (double)kept_all);
          const int tb = thr_bits >> HIST_SHIFT;
          const int b = last_bin_reaching(sh.sum, need, tb, (int)(one_bits >> HIST_SHIFT));
          unsigned lo = max(thr_bits, (unsigned)b << HIST_SHIFT), hi = min(((unsigned)(b + 1) << HIST_SHIFT) - 1, one_bits);
          while (lo < hi) {
            const unsigned mid = lo + (hi - lo + 1) / 2;
            u64 s = 0;
            for (int i = lane; i < n; i += WAVE) {
              const float x = sh.cand[i];
              if (__float_as_uint(x) >= mid) s += weight_fixed(x);
            }
            if (wave_sum_u64(s) >= need) lo = mid; else hi = mid - 1;
          }
          thr_bits = lo;
        }
        if (lane == 0) sh.thr_bits = thr_bits;
      }
      __syncthreads();
      thr_bits = sh.thr_bits;
    } else {
      const int top_bin = one_bits >> HIST_SHIFT;
      u64 kept_all = sh.sum[0];
      if (k_on) {
        const Refined t = refine_threshold<false>(w, V, bk, sh.count[bk + 1], sh.sum[bk + 1], (u64)k, sh);
        thr_bits = t.bits;
        kept_all = t.sum_from;
      }
      if (p_on) {
        const u64 need = (u64)((double)top_p * (double)kept_all);
        const int b = last_bin_reaching(sh.sum, need, 0, top_bin);
        const Refined t = refine_threshold<true>(w, V, b, sh.count[b + 1], sh.sum[b + 1], need, sh);
        thr_bits = max(thr_bits, t.bits);   // (it is at least top-k's: the weights that reach that one sum to kept_all >= need)
      }
    }
  }
  const float min_p = a.min_p[r];
  if (min_p > 0.f) {
    const unsigned mb = __float_as_uint(fminf(min_p, 1.0f));
    if (mb > thr_bits) thr_bits = mb;
  }
  const float u = a.uniform ? a.uniform[r]
                            : philox_uniform(a.draws[4 * r], a.draws[4 * r + 1], a.draws[4 * r + 2], a.draws[4 * r + 3]);
  const int pick = cumulative_pick(w, V, thr_bits, u, sh);
  if (tid == 0) a.out[r] = pick;
}

extern "C" int ifx_sample(const float* logits, float* weights, const float* temperature, const int* top_k,
                          const float* top_p, const float* min_p, const float* uniform, const unsigned* draws, int* out,
                          int R, int V, void* stream) {
  IFX_REQUIRE(R >= 0 && V > 0, "sample: bad sizes R=%d V=%d", R, V);
  IFX_REQUIRE((uniform != nullptr) != (draws != nullptr), "sample: either the uniform numbers or the seeds and counters of the draws");
  if (R == 0) return 0;
  SampleArgs a{logits, weights, temperature, top_k, top_p, min_p, uniform, draws, out, V};
  hipLaunchKernelGGL(sample_kernel, dim3(R), dim3(SAMPLE_THREADS), 0, (hipStream_t)stream, a);
  IFX_LAUNCH_CHECK();
}


// ---------------------------------------------------------------------------------------
// Log-probabilities for reporting: lp[r] = logits[r, chosen[r]] - logsumexp(logits[r]) (the
// log-softmax the reference reports per sampled token, runtime/logprob.h:11-18), and the top_n
// most probable tokens of the row with theirs, in descending order (lowest index first among
// equals).  The k-th is found as the largest element that comes after the (k-1)-th in that
// order, so the logits are not modified.
#define MAX_TOP_LOGPROBS 20
#define LOGPROB_CANDIDATES 4096

struct LogprobShared {
  float cand_v[LOGPROB_CANDIDATES];
  int cand_i[LOGPROB_CANDIDATES];
  unsigned count[HIST_BINS];
  unsigned wave_count[16];
  float red_f[16];
  float red_v[16];
  int red_i[16];
  unsigned n_cand;
  int bin;
};

// The top_n are looked for among few candidates where that is possible: the pass that sums exp(l - max) also counts the
// terms by the upper bits of their patterns (the histogram of the sampling kernel), the logits whose terms reach the
// bin below the one that holds the top_n-th (a bin's width is far more than what rounding could do to the order of
// two terms) are gathered in LDS with their indices, and one wave picks from them.  A row whose candidates do not fit
// (its top_n-th logit among thousands of near-equal ones, or fewer than top_n finite logits) takes one pass over the
// whole row per rank instead.
__global__ __launch_bounds__(SAMPLE_THREADS) void logprobs_kernel(const float* __restrict__ logits, const int* __restrict__ chosen,
                                                                 int V, int top_n, float* __restrict__ lp,
                                                                 int* __restrict__ top_ids, float* __restrict__ top_lp) {
  __shared__ LogprobShared sh;
  const int r = blockIdx.x, tid = threadIdx.x, lane = tid % WAVE, wid = tid / WAVE, nw = blockDim.x / WAVE;
  const float* row = logits + (size_t)r * V;
  float mx = -INFINITY;
  block_visit(row, V, [&](int, float l) { mx = fmaxf(mx, l); });
  mx = block_max(mx, sh.red_f);
  if (top_n > 0) {
    for (int b = tid; b < HIST_BINS; b += blockDim.x) sh.count[b] = 0;
    if (tid == 0) sh.n_cand = 0;
    __syncthreads();
  }
  float sum = 0.f;
  block_visit(row, V, [&](int, float l) {
    const float x = expf(l - mx);
    sum += x;
    if (top_n > 0) {
      const unsigned b = __float_as_uint(x) >> HIST_SHIFT;
      if (b && b < HIST_BINS) atomicAdd(&sh.count[b], 1u);
    }
  });
  sum = block_sum(sum, sh.red_f);
  const float lse = mx + logf(sum);
  if (tid == 0) lp[r] = row[chosen[r]] - lse;
  if (top_n <= 0) return;
  histogram_suffix_scan<false>(sh.count, nullptr, sh.wave_count, nullptr, V);
  if (tid == 0) {
    const int bn = last_bin_reaching(sh.count, (unsigned)top_n, 0, (int)(__float_as_uint(1.0f) >> HIST_SHIFT));
    sh.bin = max(bn - 1, 0);
  }
  __syncthreads();
  const int bc = sh.bin;
  if (sh.count[bc] <= LOGPROB_CANDIDATES) {
    const unsigned first_bits = (unsigned)bc << HIST_SHIFT;
    block_visit(row, V, [&](int i, float l) {
      if (__float_as_uint(expf(l - mx)) >= first_bits) {
        const unsigned at = atomicAdd(&sh.n_cand, 1u);
        if (at < LOGPROB_CANDIDATES) { sh.cand_v[at] = l; sh.cand_i[at] = i; }
      }
    });
    __syncthreads();
    if (wid != 0) return;
    const int n = min(sh.n_cand, (unsigned)LOGPROB_CANDIDATES);
    float last_v = INFINITY;
    int last_i = -1;
    for (int k = 0; k < top_n; ++k) {
      float bv = -INFINITY;
      int bi = V;
      for (int j = lane; j < n; j += WAVE) {
        const float x = sh.cand_v[j];
        const int i = sh.cand_i[j];
        const bool after = x < last_v || (x == last_v && i > last_i);   // not yet reported
        if (after && (x > bv || (x == bv && i < bi))) { bv = x; bi = i; }
      }
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) {
        const float ov = __shfl_xor(bv, o, WAVE);
        const int oi = __shfl_xor(bi, o, WAVE);
        argmax_merge(bv, bi, ov, oi);
      }
      if (lane == 0) {
        top_ids[r * top_n + k] = bi < V ? bi : -1;
        top_lp[r * top_n + k] = bi < V ? bv - lse : -INFINITY;
      }
      last_v = bv; last_i = bi;
    }
    return;
  }
  float last_v = INFINITY;
  int last_i = -1;
  for (int k = 0; k < top_n; ++k) {
    float bv = -INFINITY;
    int bi = V;
    block_visit(row, V, [&](int i, float x) {
      const bool after = x < last_v || (x == last_v && i > last_i);   // not yet reported
      if (after && (x > bv || (x == bv && i < bi))) { bv = x; bi = i; }
    });
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ov = __shfl_xor(bv, o, WAVE);
      const int oi = __shfl_xor(bi, o, WAVE);
      argmax_merge(bv, bi, ov, oi);
    }
    __syncthreads();
    if (lane == 0) { sh.red_v[wid] = bv; sh.red_i[wid] = bi; }
    __syncthreads();
    bv = sh.red_v[0]; bi = sh.red_i[0];
    for (int w = 1; w < nw; ++w) argmax_merge(bv, bi, sh.red_v[w], sh.red_i[w]);
    if (tid == 0) {
      top_ids[r * top_n + k] = bi < V ? bi : -1;
      top_lp[r * top_n + k] = bi < V ? bv - lse : -INFINITY;
    }
    last_v = bv; last_i = bi;
  }
}

extern "C" int ifx_logprobs(const float* logits, const int* chosen, int R, int V, int top_n, float* lp, int* top_ids,
                            float* top_lp, void* stream) {
  IFX_REQUIRE(R >= 0 && V > 0 && top_n >= 0 && top_n <= MAX_TOP_LOGPROBS, "logprobs: bad sizes R=%d V=%d top_n=%d (at most %d)", R, V, top_n, MAX_TOP_LOGPROBS);
  if (R == 0) return 0;
  hipLaunchKernelGGL(logprobs_kernel, dim3(R), dim3(SAMPLE_THREADS), 0, (hipStream_t)stream, logits, chosen, V, top_n, lp,
                     top_ids, top_lp);
  IFX_LAUNCH_CHECK();
}
