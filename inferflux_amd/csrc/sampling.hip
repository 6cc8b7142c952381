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
  const float* uniform;  // one number in [0, 1) per row
  int* out;
  int V;
};

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

__device__ float kept_sum(const float* __restrict__ w, int V, float thr, float* red) {
  float s = 0.f;
  for (int i = threadIdx.x; i < V; i += blockDim.x) {
    const float x = w[i];
    if (x >= thr) s += x;
  }
  return block_sum(s, red);
}

__device__ int kept_count(const float* __restrict__ w, int V, float thr, int* red) {
  int c = 0;
  for (int i = threadIdx.x; i < V; i += blockDim.x) c += w[i] >= thr ? 1 : 0;
  return block_sum_int(c, red);
}

__global__ __launch_bounds__(SAMPLE_THREADS) void sample_kernel(SampleArgs a) {
  __shared__ float red_f[16];
  __shared__ int red_i[16];
  __shared__ float part[SAMPLE_THREADS];
  __shared__ int found;
  const int r = blockIdx.x, V = a.V;
  const float* row = a.logits + (size_t)r * V;
  const float temp = a.temperature[r];
  if (!(temp > 0.f)) {
    const int best = block_argmax(row, V, red_f, red_i);
    if (threadIdx.x == 0) a.out[r] = best;
    return;
  }
  float* w = a.weights + (size_t)r * V;
  const float inv_t = 1.0f / temp;
  float mx = -INFINITY;
  for (int i = threadIdx.x; i < V; i += blockDim.x) mx = fmaxf(mx, row[i] * inv_t);
  mx = block_max(mx, red_f);
  for (int i = threadIdx.x; i < V; i += blockDim.x) w[i] = expf(row[i] * inv_t - mx);
  __syncthreads();

  // Thresholds as bit patterns: for non-negative floats the order of the values is the order
  // of their bits.  The largest weight is exp(0) = 1.
  const unsigned one_bits = __float_as_uint(1.0f);
  unsigned thr_bits = 0;  // keep everything
  const int k = a.top_k[r];
  if (k > 0 && k < V) {
    unsigned lo = 0, hi = one_bits;  // count(w >= f(lo)) >= k holds for lo = 0
    while (lo < hi) {
      const unsigned mid = lo + (hi - lo + 1) / 2;
      if (kept_count(w, V, __uint_as_float(mid), red_i) >= k) lo = mid; else hi = mid - 1;
    }
    thr_bits = lo;
  }
  const float top_p = a.top_p[r];
  if (top_p > 0.f && top_p < 1.f) {
    const float need = top_p * kept_sum(w, V, __uint_as_float(thr_bits), red_f);
    unsigned lo = thr_bits, hi = one_bits;  // sum(w >= f(lo)) >= need holds for lo = thr_bits
    while (lo < hi) {
      const unsigned mid = lo + (hi - lo + 1) / 2;
      if (kept_sum(w, V, __uint_as_float(mid), red_f) >= need) lo = mid; else hi = mid - 1;
    }
    thr_bits = lo;
  }
  const float min_p = a.min_p[r];
  if (min_p > 0.f) {
    const unsigned mb = __float_as_uint(fminf(min_p, 1.0f));
    if (mb > thr_bits) thr_bits = mb;
  }
  const float thr = __uint_as_float(thr_bits);

  // Cumulative walk in index order: thread t owns the indices [t*chunk, (t+1)*chunk).
  const int chunk = (V + blockDim.x - 1) / blockDim.x;
  const int c0 = min(V, (int)threadIdx.x * chunk), c1 = min(V, c0 + chunk);
  float mine = 0.f;
  int last_kept = -1;
  for (int i = c0; i < c1; ++i)
    if (w[i] >= thr) { mine += w[i]; last_kept = i; }
  part[threadIdx.x] = mine;
  if (threadIdx.x == 0) found = -1;
  __syncthreads();
  if (threadIdx.x == 0) {  // exclusive prefix in place, sequential: one fixed order of additions
    float run = 0.f;
    for (int t = 0; t < (int)blockDim.x; ++t) { const float v = part[t]; part[t] = run; run += v; }
    red_f[0] = run;
  }
  __syncthreads();
  const float total = red_f[0];
  const float target = a.uniform[r] * total;
  const float before = part[threadIdx.x];
  const float after = threadIdx.x + 1 < blockDim.x ? part[threadIdx.x + 1] : total;
  if (mine > 0.f && before <= target && target < after) {
    float cum = before;
    int pick = last_kept;
    for (int i = c0; i < c1; ++i) {
      if (w[i] >= thr) {
        cum += w[i];
        if (target < cum) { pick = i; break; }
      }
    }
    found = pick;
  }
  // Fallback (target >= total through rounding): the last kept index.
  int lk = last_kept;
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) lk = max(lk, __shfl_xor(lk, o, WAVE));
  const int wid = threadIdx.x / WAVE, lane = threadIdx.x % WAVE, nw = blockDim.x / WAVE;
  __syncthreads();
  if (lane == 0) red_i[wid] = lk;
  __syncthreads();
  if (threadIdx.x == 0) {
    int best = found;
    if (best < 0) {
      best = red_i[0];
      for (int i = 1; i < nw; ++i) best = max(best, red_i[i]);
      if (best < 0) best = 0;
    }
    a.out[r] = best;
  }
}

extern "C" int ifx_sample(const float* logits, float* weights, const float* temperature, const int* top_k,
                          const float* top_p, const float* min_p, const float* uniform, int* out, int R, int V,
                          void* stream) {
  IFX_REQUIRE(R >= 0 && V > 0, "sample: bad sizes R=%d V=%d", R, V);
  if (R == 0) return 0;
  SampleArgs a{logits, weights, temperature, top_k, top_p, min_p, uniform, out, V};
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

__global__ __launch_bounds__(SAMPLE_THREADS) void logprobs_kernel(const float* __restrict__ logits, const int* __restrict__ chosen,
                                                                 int V, int top_n, float* __restrict__ lp,
                                                                 int* __restrict__ top_ids, float* __restrict__ top_lp) {
  __shared__ float red_f[16];
  __shared__ float red_v[16];
  __shared__ int red_i[16];
  const int r = blockIdx.x;
  const float* row = logits + (size_t)r * V;
  float mx = -INFINITY;
  for (int i = threadIdx.x; i < V; i += blockDim.x) mx = fmaxf(mx, row[i]);
  mx = block_max(mx, red_f);
  float sum = 0.f;
  for (int i = threadIdx.x; i < V; i += blockDim.x) sum += expf(row[i] - mx);
  sum = block_sum(sum, red_f);
  const float lse = mx + logf(sum);
  if (threadIdx.x == 0) lp[r] = row[chosen[r]] - lse;
  float last_v = INFINITY;
  int last_i = -1;
  for (int k = 0; k < top_n; ++k) {
    float bv = -INFINITY;
    int bi = V;
    for (int i = threadIdx.x; i < V; i += blockDim.x) {
      const float x = row[i];
      const bool after = x < last_v || (x == last_v && i > last_i);   // not yet reported
      if (after && (x > bv || (x == bv && i < bi))) { bv = x; bi = i; }
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
    if (threadIdx.x == 0) {
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
