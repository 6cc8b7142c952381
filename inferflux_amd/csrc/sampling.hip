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
// a filter keeps every token whose weight is >= its threshold, an exact selection on the bit
// patterns of the weights (a histogram of their upper bits, then the threshold's bin by its
// lower bits), so tokens of equal weight are kept or dropped together.
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
// lower of these bins upwards (the candidates: usually a few hundred of the row) are gathered in LDS, where the
// threshold's bin is counted by the next ten bits of the patterns and that sub-bin by the last nine.  Counts are integers and sums are sums of the
// weights in fixed point (units of 2^-40, so a row of a million weights of 1.0 stays below 2^64): neither depends
// on the order in which the threads add, and the histogram's sums and the candidates' agree exactly.  A row whose
// candidates do not fit (more than SAMPLE_CANDIDATES: a wide nucleus) makes the same two passes per threshold over
// the whole row instead (refine_threshold).
#define HIST_MANTISSA 4
#define HIST_SHIFT (23 - HIST_MANTISSA)
#define HIST_BINS 2048
#define SAMPLE_CANDIDATES 3072
typedef unsigned long long u64;

__device__ __forceinline__ u64 weight_fixed(float x) { return (u64)(x * 1099511627776.0f); }   // x * 2^40, x in [0, 1]

struct SampleShared {
  float cand[SAMPLE_CANDIDATES];
  unsigned count[HIST_BINS];     // after the scan: the number of weights in this bin or a higher one
  u64 sum[HIST_BINS];            // after the scan: their sum in fixed point
  unsigned sub_count[1024];      // the same for the sub-bins of one bin (refine_threshold)
  u64 sub_sum[1024];
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
// it.  Two passes over ``w`` [V] (the candidates in LDS, or in memory where they do not fit there): the bin's weights
// by the next ten bits of their patterns, then the chosen sub-bin's by the last nine.  Every thread returns the
// pattern and the sum of the weights that reach it.
struct Refined { unsigned bits; u64 sum_from; };

template <bool BY_SUM>
__device__ Refined refine_threshold(const float* __restrict__ w, int V, unsigned bin1, unsigned above_count, u64 above_sum,
                                    u64 need, SampleShared& sh) {
  static_assert(SAMPLE_THREADS == 1024, "one sub-bin per thread");
  unsigned* c2 = sh.sub_count;
  u64* s2 = sh.sub_sum;
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

// Thread 0 of the workgroup: the bins that hold the thresholds of top-k (sh.bin_k) and top-p (sh.bin_p, found with at
// least what the exact rule will ask for: top-k keeps no more than the bins from bin_k upwards hold) and the lower of
// them (sh.bin_cand: the weights from there upwards are the candidates), from the scanned histogram.
__device__ void choose_bins(SampleShared& sh, bool k_on, int k, bool p_on, float top_p) {
  const int top_bin = __float_as_uint(1.0f) >> HIST_SHIFT;
  int bk = 0, bp = 0, bc = top_bin;
  if (k_on) { bk = last_bin_reaching(sh.count, (unsigned)k, 0, top_bin); bc = min(bc, bk); }
  if (p_on) {
    const u64 need = (u64)((double)top_p * (double)sh.sum[bk]);
    bp = last_bin_reaching(sh.sum, need, 0, top_bin);
    bc = min(bc, bp);
  }
  sh.bin_k = bk; sh.bin_p = bp; sh.bin_cand = bc;
}

// The whole workgroup: the exact thresholds from ``w`` [n], which holds at least every weight from the candidates' bin
// upwards (the candidates in LDS; the list of them in memory, or the whole row, where they do not fit), by two passes
// per threshold.  Thresholds are bit patterns: for non-negative floats the order of the values is the order of their
// bits; the largest weight is 1.
__device__ unsigned thresholds_by_refinement(const float* __restrict__ w, int n, SampleShared& sh, bool k_on, int k, bool p_on,
                                             float top_p) {
  const int top_bin = __float_as_uint(1.0f) >> HIST_SHIFT, bk = sh.bin_k;
  unsigned thr_bits = 0;
  u64 kept_all = sh.sum[0];
  if (k_on) {
    const Refined t = refine_threshold<false>(w, n, bk, sh.count[bk + 1], sh.sum[bk + 1], (u64)k, sh);
    thr_bits = t.bits;
    kept_all = t.sum_from;
  }
  if (p_on) {
    const u64 need = (u64)((double)top_p * (double)kept_all);
    const int b = last_bin_reaching(sh.sum, need, 0, top_bin);
    const Refined t = refine_threshold<true>(w, n, b, sh.count[b + 1], sh.sum[b + 1], need, sh);
    thr_bits = max(thr_bits, t.bits);   // (it is at least top-k's: the weights that reach that one sum to kept_all >= need)
  }
  return thr_bits;
}

__device__ __forceinline__ unsigned with_min_p(unsigned thr_bits, float min_p) {
  if (min_p > 0.f) {
    const unsigned mb = __float_as_uint(fminf(min_p, 1.0f));
    if (mb > thr_bits) thr_bits = mb;
  }
  return thr_bits;
}

__device__ __forceinline__ float row_uniform(const SampleArgs& a, int r) {
  return a.uniform ? a.uniform[r] : philox_uniform(a.draws[4 * r], a.draws[4 * r + 1], a.draws[4 * r + 2], a.draws[4 * r + 3]);
}

// One workgroup takes a row whole: the form for vocabularies below SLICED_MIN_V tokens and for more than
// SLICED_MAX_ROWS rows (below).
__global__ __launch_bounds__(SAMPLE_THREADS) void sample_kernel(SampleArgs a) {
  __shared__ SampleShared sh;
  const int r = blockIdx.x, V = a.V, tid = threadIdx.x, wid = tid / WAVE;
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
    if (tid == 0) choose_bins(sh, k_on, k, p_on, top_p);
    __syncthreads();
    const int bc = sh.bin_cand;
    if (sh.count[bc] <= SAMPLE_CANDIDATES) {
      const unsigned first_bits = (unsigned)bc << HIST_SHIFT;
      block_visit(w, V, [&](int, float x) {
        if (__float_as_uint(x) >= first_bits) {
          const unsigned at = atomicAdd(&sh.n_cand, 1u);
          if (at < SAMPLE_CANDIDATES) sh.cand[at] = x;
        }
      });
      __syncthreads();
      thr_bits = thresholds_by_refinement(sh.cand, min(sh.n_cand, (unsigned)SAMPLE_CANDIDATES), sh, k_on, k, p_on, top_p);
    } else {
      thr_bits = thresholds_by_refinement(w, V, sh, k_on, k, p_on, top_p);
    }
  }
  thr_bits = with_min_p(thr_bits, a.min_p[r]);
  const int pick = cumulative_pick(w, V, thr_bits, row_uniform(a, r), sh);
  if (tid == 0) a.out[r] = pick;
}

// ---------------------------------------------------------------------------------------
// The same draw for large vocabularies with SAMPLE_SLICES workgroups to a row.  One workgroup pulls a row through one
// compute unit, 12 us a pass over 152,064 weights; here each pass is a launch of its own in which every wave of every
// workgroup takes one of the row's SAMPLE_SEGMENTS segments, and what the passes hand each other lies in scratch
// memory:
//   1. the largest logit of each slice;
//   2. the weights, and for rows with top-k or top-p the histogram (each workgroup's in LDS, added to the row's with
//      integer atomics: no order to depend on); rows without them get their segments' sums here already;
//   3. the candidates: every workgroup scans the row's histogram for itself, finds the candidates' bin and appends
//      its slice's candidates to the row's list (their order depends on timing, nothing computed from them does);
//   4. the thresholds, again by every workgroup for itself (in LDS from up to SAMPLE_CANDIDATES candidates, else by
//      refinement over the list), and the sum of the kept weights of each segment;
//   5. one wave per row finds the segment where the cumulative sum passes uniform * total and walks it.
// Rows with temperature <= 0 are left to an argmax launch.  The result depends on the row and its number alone.
// Measured on 152,064-token rows inside a replayed graph, us one workgroup a row / sliced: a temperature alone 35 / 17
// at one row, 36 / 21 at 8, 50 / 45 at 64; with top-k 50 and top-p 0.9: 73 / 49, 74 / 52, 96 / 162 (every workgroup scans
// the row's histogram and finds the thresholds for itself: with 64 rows that is 1,024 times), so up to 16 rows are sliced.
#define SAMPLE_SLICES 16
#define SAMPLE_SEGMENTS (SAMPLE_SLICES * (SAMPLE_THREADS / WAVE))
#define SLICED_MIN_V 32768        // smaller vocabularies, and
#define SLICED_MAX_ROWS 16        // more rows (which fill compute units enough by themselves): one workgroup a row, one launch;
#define SLICED_MAX_ROWS_PLAIN 64  // without top-k and top-p (three short launches) the sliced form pays up to this many

struct SlicedArgs {
  SampleArgs a;
  float* slice_max;       // [R, SAMPLE_SLICES]
  u64* hist_sum;          // [R, HIST_BINS]
  unsigned* hist_count;   // [R, HIST_BINS]
  float* cand;            // [R, V]
  unsigned* n_cand;       // [R]
  unsigned* thr_bits;     // [R]
  float* seg_sum;         // [R, SAMPLE_SEGMENTS]
  int* seg_last;          // [R, SAMPLE_SEGMENTS]
  int seg;                // elements of a segment (a multiple of 64)
  int any_filters;        // 0: top-k and top-p are taken as off in every row
};

struct RowFilters { bool k_on, p_on; int k; float top_p; };
__device__ __forceinline__ RowFilters row_filters(const SlicedArgs& g, int r) {
  const int k = g.a.top_k[r];
  const float top_p = g.a.top_p[r];
  return RowFilters{g.any_filters && k > 0 && k < g.a.V, g.any_filters && top_p > 0.f && top_p < 1.f, k, top_p};
}

// The sum of the weights of segment [a0, a1) that reach thr_bits, and the last index that does (-1: none): one wave.
__device__ __forceinline__ void segment_kept(const float* __restrict__ w, int a0, int a1, unsigned thr_bits, float& sum, int& last) {
  const int lane = threadIdx.x % WAVE;
  float mine = 0.f;
  last = -1;
  for (int i = a0 + lane; i < a1; i += WAVE) {
    const float x = w[i];
    if (__float_as_uint(x) >= thr_bits) { mine += x; last = i; }
  }
  sum = wave_sum(mine);
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) last = max(last, __shfl_xor(last, o, WAVE));
}

__global__ __launch_bounds__(SAMPLE_THREADS) void sliced_max_kernel(SlicedArgs g) {
  __shared__ float red[16];
  const int sl = blockIdx.x, r = blockIdx.y, V = g.a.V, tid = threadIdx.x, lane = tid % WAVE, wid = tid / WAVE;
  const float temp = g.a.temperature[r];
  if (!(temp > 0.f)) return;
  const float inv_t = 1.0f / temp;
  const float* row = g.a.logits + (size_t)r * V;
  const int j = sl * (SAMPLE_THREADS / WAVE) + wid, a0 = min(V, j * g.seg), a1 = min(V, a0 + g.seg);
  float mx = -INFINITY;
  for (int i = a0 + lane; i < a1; i += WAVE) mx = fmaxf(mx, row[i] * inv_t);
  mx = block_max(mx, red);
  if (tid == 0) g.slice_max[r * SAMPLE_SLICES + sl] = mx;
  // this workgroup's share of the row's histogram starts at zero, and the row's list of candidates empty
  constexpr int share = HIST_BINS / SAMPLE_SLICES;
  if (tid < share) {
    g.hist_count[(size_t)r * HIST_BINS + sl * share + tid] = 0;
    g.hist_sum[(size_t)r * HIST_BINS + sl * share + tid] = 0;
  }
  if (sl == 0 && tid == 0) g.n_cand[r] = 0;
}

__global__ __launch_bounds__(SAMPLE_THREADS) void sliced_weights_kernel(SlicedArgs g) {
  __shared__ unsigned count[HIST_BINS];
  __shared__ u64 sum[HIST_BINS];
  const int sl = blockIdx.x, r = blockIdx.y, V = g.a.V, tid = threadIdx.x, lane = tid % WAVE, wid = tid / WAVE;
  const float temp = g.a.temperature[r];
  if (!(temp > 0.f)) return;
  const float inv_t = 1.0f / temp;
  const float* row = g.a.logits + (size_t)r * V;
  float* w = g.a.weights + (size_t)r * V;
  float mx = -INFINITY;
#pragma unroll
  for (int i = 0; i < SAMPLE_SLICES; ++i) mx = fmaxf(mx, g.slice_max[r * SAMPLE_SLICES + i]);
  const RowFilters f = row_filters(g, r);
  const bool filters = f.k_on || f.p_on;
  if (filters) {
    for (int b = tid; b < HIST_BINS; b += blockDim.x) { count[b] = 0; sum[b] = 0; }
    __syncthreads();
  }
  const int j = sl * (SAMPLE_THREADS / WAVE) + wid, a0 = min(V, j * g.seg), a1 = min(V, a0 + g.seg);
  const unsigned thr_bits = with_min_p(0, g.a.min_p[r]);     // (without top-k and top-p the threshold is known here)
  float mine = 0.f;
  int last = -1;
  for (int i = a0 + lane; i < a1; i += WAVE) {
    const float x = expf(row[i] * inv_t - mx);
    w[i] = x;
    if (filters) {
      const unsigned b = __float_as_uint(x) >> HIST_SHIFT;
      if (b && b < HIST_BINS) {   // (a NaN's pattern lies beyond the last bin)
        atomicAdd(&count[b], 1u);
        atomicAdd(&sum[b], weight_fixed(x));
      }
    } else if (__float_as_uint(x) >= thr_bits) {
      mine += x;
      last = i;
    }
  }
  if (filters) {
    __syncthreads();
    for (int b = tid; b < HIST_BINS; b += blockDim.x) {
      const unsigned c = count[b];
      if (c) {
        atomicAdd(&g.hist_count[(size_t)r * HIST_BINS + b], c);
        atomicAdd(&g.hist_sum[(size_t)r * HIST_BINS + b], sum[b]);
      }
    }
    return;
  }
  mine = wave_sum(mine);
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) last = max(last, __shfl_xor(last, o, WAVE));
  if (lane == 0) {
    g.seg_sum[r * SAMPLE_SEGMENTS + j] = mine;
    g.seg_last[r * SAMPLE_SEGMENTS + j] = last;
  }
  if (sl == 0 && tid == 0) g.thr_bits[r] = thr_bits;
}

// The row's histogram from memory into sh, scanned, and the bins chosen (the same in every workgroup of the row).
__device__ void load_row_bins(const SlicedArgs& g, int r, const RowFilters& f, SampleShared& sh) {
  const int tid = threadIdx.x;
  for (int b = tid; b < HIST_BINS; b += blockDim.x) {
    sh.count[b] = g.hist_count[(size_t)r * HIST_BINS + b];
    sh.sum[b] = g.hist_sum[(size_t)r * HIST_BINS + b];
  }
  __syncthreads();
  histogram_suffix_scan<true>(sh.count, sh.sum, sh.wave_count, sh.wave_sum, g.a.V);
  if (tid == 0) choose_bins(sh, f.k_on, f.k, f.p_on, f.top_p);
  __syncthreads();
}

__global__ __launch_bounds__(SAMPLE_THREADS) void sliced_gather_kernel(SlicedArgs g) {
  __shared__ SampleShared sh;
  __shared__ unsigned wave_n[SAMPLE_THREADS / WAVE + 1];
  const int sl = blockIdx.x, r = blockIdx.y, V = g.a.V, tid = threadIdx.x, lane = tid % WAVE, wid = tid / WAVE;
  if (!(g.a.temperature[r] > 0.f)) return;
  const RowFilters f = row_filters(g, r);
  if (!f.k_on && !f.p_on) return;
  load_row_bins(g, r, f, sh);
  const unsigned first_bits = (unsigned)sh.bin_cand << HIST_SHIFT;
  const float* w = g.a.weights + (size_t)r * V;
  const int j = sl * (SAMPLE_THREADS / WAVE) + wid, a0 = min(V, j * g.seg), a1 = min(V, a0 + g.seg);
  unsigned mine = 0;
  for (int i0 = a0; i0 < a1; i0 += WAVE) {
    const int i = i0 + lane;
    mine += __popcll(__ballot(i < a1 && __float_as_uint(w[i]) >= first_bits));
  }
  if (lane == 0) wave_n[wid] = mine;
  __syncthreads();
  if (tid == 0) {   // one place in the row's list for the workgroup's candidates, wave after wave
    unsigned total = 0;
    for (int i = 0; i < SAMPLE_THREADS / WAVE; ++i) { const unsigned c = wave_n[i]; wave_n[i] = total; total += c; }
    wave_n[SAMPLE_THREADS / WAVE] = total ? atomicAdd(&g.n_cand[r], total) : 0;
  }
  __syncthreads();
  unsigned at = wave_n[SAMPLE_THREADS / WAVE] + wave_n[wid];
  float* cand = g.cand + (size_t)r * V;
  for (int i0 = a0; i0 < a1; i0 += WAVE) {
    const int i = i0 + lane;
    const float x = i < a1 ? w[i] : 0.f;
    const bool is = i < a1 && __float_as_uint(x) >= first_bits;
    const u64 m = __ballot(is);
    if (is) cand[at + __popcll(m & ((1ull << lane) - 1))] = x;
    at += __popcll(m);
  }
}

__global__ __launch_bounds__(SAMPLE_THREADS) void sliced_sums_kernel(SlicedArgs g) {
  __shared__ SampleShared sh;
  const int sl = blockIdx.x, r = blockIdx.y, V = g.a.V, tid = threadIdx.x, lane = tid % WAVE, wid = tid / WAVE;
  if (!(g.a.temperature[r] > 0.f)) return;
  const RowFilters f = row_filters(g, r);
  if (!f.k_on && !f.p_on) return;                  // (such a row's sums were made with its weights)
  load_row_bins(g, r, f, sh);
  const int n = (int)g.n_cand[r];
  const float* cand = g.cand + (size_t)r * V;
  unsigned thr_bits;
  if (n <= SAMPLE_CANDIDATES) {
    for (int i = tid; i < n; i += blockDim.x) sh.cand[i] = cand[i];
    __syncthreads();
    thr_bits = thresholds_by_refinement(sh.cand, n, sh, f.k_on, f.k, f.p_on, f.top_p);
  } else {
    thr_bits = thresholds_by_refinement(cand, n, sh, f.k_on, f.k, f.p_on, f.top_p);
  }
  thr_bits = with_min_p(thr_bits, g.a.min_p[r]);
  const int j = sl * (SAMPLE_THREADS / WAVE) + wid, a0 = min(V, j * g.seg), a1 = min(V, a0 + g.seg);
  float kept;
  int last;
  segment_kept(g.a.weights + (size_t)r * V, a0, a1, thr_bits, kept, last);
  if (lane == 0) {
    g.seg_sum[r * SAMPLE_SEGMENTS + j] = kept;
    g.seg_last[r * SAMPLE_SEGMENTS + j] = last;
  }
  if (sl == 0 && tid == 0) g.thr_bits[r] = thr_bits;
}

// One wave per row: lane l holds the segments 4 l ... 4 l + 3 (SAMPLE_SEGMENTS = 256), their sums are added in segment
// order, and the segment in which the cumulative sum passes uniform * total is walked 64 weights at a time.  A target
// that rounding puts past the end of the segment, or of the row, gives the last kept index there.
__global__ __launch_bounds__(WAVE) void sliced_pick_kernel(SlicedArgs g) {
  static_assert(SAMPLE_SEGMENTS == 4 * WAVE, "four segments to a lane");
  const int r = blockIdx.x, V = g.a.V, lane = threadIdx.x;
  if (!(g.a.temperature[r] > 0.f)) return;
  const float* w = g.a.weights + (size_t)r * V;
  const unsigned thr_bits = g.thr_bits[r];
  float s[4], mine = 0.f;
  int last_any = -1;
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    s[q] = g.seg_sum[r * SAMPLE_SEGMENTS + 4 * lane + q];
    mine += s[q];
    last_any = max(last_any, g.seg_last[r * SAMPLE_SEGMENTS + 4 * lane + q]);
  }
  float upto = mine;      // the sum of this lane's segments and all before them
#pragma unroll
  for (int o = 1; o < WAVE; o <<= 1) {
    const float up = __shfl_up(upto, o, WAVE);
    if (lane >= o) upto += up;
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) last_any = max(last_any, __shfl_xor(last_any, o, WAVE));
  const float total = __shfl(upto, WAVE - 1, WAVE);
  float target = row_uniform(g.a, r) * total;
  // the first segment with anything kept whose end the target lies before
  float before = upto - mine;
  int found = -1;
  float found_before = 0.f;
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    if (found < 0 && s[q] > 0.f && target - before < s[q]) { found = 4 * lane + q; found_before = before; }
    before += s[q];
  }
  const u64 any = __ballot(found >= 0);
  int pick = max(last_any, 0);
  if (any) {
    const int src = __ffsll((long long)any) - 1;
    const int j = __shfl(found, src, WAVE);
    target -= __shfl(found_before, src, WAVE);
    const int a0 = min(V, j * g.seg), a1 = min(V, a0 + g.seg);
    float run = 0.f;
    int hit_at = -1, last = -1;
    for (int i0 = a0; i0 < a1 && hit_at < 0; i0 += WAVE) {
      const int i = i0 + lane;
      const float x = i < a1 ? w[i] : 0.f;
      const bool kept = i < a1 && __float_as_uint(x) >= thr_bits;
      float cum = kept ? x : 0.f;
#pragma unroll
      for (int o = 1; o < WAVE; o <<= 1) {
        const float up = __shfl_up(cum, o, WAVE);
        if (lane >= o) cum += up;
      }
      cum += run;
      const u64 hit = __ballot(kept && target < cum);
      const u64 keeps = __ballot(kept);
      if (hit) hit_at = i0 + __ffsll((long long)hit) - 1;
      if (keeps) last = i0 + 63 - __clzll((long long)keeps);
      run = __shfl(cum, WAVE - 1, WAVE);
    }
    pick = hit_at >= 0 ? hit_at : max(last, 0);
  }
  if (lane == 0) g.a.out[r] = pick;
}

// Rows with temperature <= 0 of a launch whose other rows are drawn by the sliced kernels.
__global__ __launch_bounds__(SAMPLE_THREADS) void greedy_rows_kernel(SampleArgs a) {
  __shared__ float red_v[16];
  __shared__ int red_i[16];
  const int r = blockIdx.x;
  if (a.temperature[r] > 0.f) return;
  const int best = block_argmax(a.logits + (size_t)r * a.V, a.V, red_v, red_i);
  if (threadIdx.x == 0) a.out[r] = best;
}

static size_t align256(size_t n) { return (n + 255) / 256 * 256; }

// The scratch memory ifx_sample needs besides the weights [R, V], in blocks of 256 bytes (0: a launch of the
// one-workgroup form).
static bool sliced_form(int R, int V, int any_filters) {
  return V >= SLICED_MIN_V && R <= (any_filters ? SLICED_MAX_ROWS : SLICED_MAX_ROWS_PLAIN);
}

extern "C" int ifx_sample_scratch_blocks(int R, int V, int any_filters) {
  if (R <= 0 || !sliced_form(R, V, any_filters)) return 0;
  const size_t rows = (size_t)R;
  return (int)((align256(rows * SAMPLE_SLICES * sizeof(float)) + align256(rows * HIST_BINS * sizeof(u64)) +
                align256(rows * HIST_BINS * sizeof(unsigned)) + align256(rows * (size_t)V * sizeof(float)) +
                align256(rows * sizeof(unsigned)) * 2 + align256(rows * SAMPLE_SEGMENTS * sizeof(float)) * 2) / 256);
}

// ``scratch``: ifx_sample_scratch_blocks(R, V, any_filters) blocks of 256 bytes, aligned to 256 (or null when that is 0).  ``any_greedy`` 0: the
// caller knows that every row has a temperature above zero; ``any_filters`` 0: that no row has top-k or top-p (each
// saves the sliced form launches that would find nothing to do).
extern "C" int ifx_sample(const float* logits, float* weights, const float* temperature, const int* top_k,
                          const float* top_p, const float* min_p, const float* uniform, const unsigned* draws, int* out,
                          int R, int V, void* scratch, int any_greedy, int any_filters, void* stream) {
  IFX_REQUIRE(R >= 0 && V > 0, "sample: bad sizes R=%d V=%d", R, V);
  IFX_REQUIRE((uniform != nullptr) != (draws != nullptr), "sample: either the uniform numbers or the seeds and counters of the draws");
  if (R == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  SampleArgs a{logits, weights, temperature, top_k, top_p, min_p, uniform, draws, out, V};
  if (!sliced_form(R, V, any_filters)) {
    hipLaunchKernelGGL(sample_kernel, dim3(R), dim3(SAMPLE_THREADS), 0, s, a);
    IFX_LAUNCH_CHECK();
  }
  IFX_REQUIRE(scratch != nullptr && ((size_t)scratch & 255) == 0, "sample: needs ifx_sample_scratch_blocks() of scratch memory, aligned to 256");
  IFX_REQUIRE(R <= 65535, "sample: %d rows in one launch (at most 65,535)", R);
  unsigned char* at = (unsigned char*)scratch;
  auto take = [&](size_t bytes) { unsigned char* p = at; at += align256(bytes); return p; };
  const size_t rows = (size_t)R;
  SlicedArgs g;
  g.a = a;
  g.slice_max = (float*)take(rows * SAMPLE_SLICES * sizeof(float));
  g.hist_sum = (u64*)take(rows * HIST_BINS * sizeof(u64));
  g.hist_count = (unsigned*)take(rows * HIST_BINS * sizeof(unsigned));
  g.cand = (float*)take(rows * (size_t)V * sizeof(float));
  g.n_cand = (unsigned*)take(rows * sizeof(unsigned));
  g.thr_bits = (unsigned*)take(rows * sizeof(unsigned));
  g.seg_sum = (float*)take(rows * SAMPLE_SEGMENTS * sizeof(float));
  g.seg_last = (int*)take(rows * SAMPLE_SEGMENTS * sizeof(int));
  g.seg = ((V + SAMPLE_SEGMENTS - 1) / SAMPLE_SEGMENTS + WAVE - 1) / WAVE * WAVE;
  g.any_filters = any_filters;
  const dim3 slices(SAMPLE_SLICES, R);
  if (any_greedy) hipLaunchKernelGGL(greedy_rows_kernel, dim3(R), dim3(SAMPLE_THREADS), 0, s, a);
  hipLaunchKernelGGL(sliced_max_kernel, slices, dim3(SAMPLE_THREADS), 0, s, g);
  hipLaunchKernelGGL(sliced_weights_kernel, slices, dim3(SAMPLE_THREADS), 0, s, g);
  if (any_filters) {
    hipLaunchKernelGGL(sliced_gather_kernel, slices, dim3(SAMPLE_THREADS), 0, s, g);
    hipLaunchKernelGGL(sliced_sums_kernel, slices, dim3(SAMPLE_THREADS), 0, s, g);
  }
  hipLaunchKernelGGL(sliced_pick_kernel, dim3(R), dim3(WAVE), 0, s, g);
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
