// Row-wise kernels of the decoder: embedding gather, residual add + RMSNorm, bias + rotary
// position encoding + append to the paged cache, SwiGLU.  All math in float; the residual
// stream is float in every mode.
//
// Formulas follow the reference's dense path:
//   embedding  runtime/backends/cuda/native/cuda_kernels.cu:255-270, 674-689
//   RMSNorm    cuda_kernels.cu:15-48 (eps inside the square root, line 41)
//   residual add + norm  cuda_kernels.cu:193-249, 617-671
//   bias       cuda_kernels.cu:518-527
//   RoPE       cuda_kernels.cu:71-117 (split-half pairing 102-105), fused with the cache write
//              as in runtime/backends/cuda/native/kernels/fused_rope_kv_append.cuh:26-166
//   SwiGLU     cuda_kernels.cu:139-151
#include "common.h"

IFX_DEFINE_LAST_ERROR()

// ---------------------------------------------------------------------------------------
// out[t, :] = float(table[ids[t], :])
template <typename T>
__global__ void embedding_kernel(const int* __restrict__ ids, const T* __restrict__ table,
                                 float* __restrict__ out, int H) {
  // (a row is cut into runs of 4,096 columns, one workgroup each: rows as wide as a vocabulary then fill the chip too)
  const int t = blockIdx.x, i0 = blockIdx.y * 4096, i1 = min(H, i0 + 4096);
  const T* src = table + (size_t)ids[t] * H;
  float* dst = out + (size_t)t * H;
  for (int i = i0 + threadIdx.x; i < i1; i += blockDim.x) dst[i] = to_f(src[i]);
}

extern "C" int ifx_embedding(const int* ids, const void* table, int table_dtype, float* out, int T,
                             int H, void* stream) {
  IFX_REQUIRE(T >= 0 && H > 0, "embedding: bad sizes T=%d H=%d", T, H);
  if (T == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  if (table_dtype == DT_F32)
    hipLaunchKernelGGL(embedding_kernel<float>, dim3(T, (H + 4095) / 4096), dim3(256), 0, s, ids, (const float*)table, out, H);
  else if (table_dtype == DT_BF16)
    hipLaunchKernelGGL(embedding_kernel<bf16_t>, dim3(T, (H + 4095) / 4096), dim3(256), 0, s, ids, (const bf16_t*)table, out, H);
  else
    IFX_FAIL("embedding: unknown dtype %d", table_dtype);
  IFX_LAUNCH_CHECK();
}

// The same for up to 16 tokens, with what the RMS norm that reads the stream first needs written beside it, so that
// the norm takes no kernel of its own: rows[t, :] = bf16(out[t, :] * norm_w[:]) and pieces[run][t] = the sum of the
// squares of out[t, :] over run ``run`` of 4,096 columns (zero for t >= n_rows; ``pieces`` is [runs][16]).  The
// product that reads ``rows`` multiplies its sums by rsqrt(sum of the pieces / H + eps) (RowScale in gemm_bf16.hip).
template <typename T>
__global__ __launch_bounds__(256) void embedding_norm_kernel(const int* __restrict__ ids, const T* __restrict__ table,
                                                            const bf16_t* __restrict__ norm_w, float* __restrict__ out,
                                                            bf16_t* __restrict__ rows, float* __restrict__ pieces,
                                                            int n_rows, int H) {
  __shared__ float red[16];
  const int t = blockIdx.x, run = blockIdx.y, i0 = run * 4096, i1 = min(H, i0 + 4096);
  float ss = 0.f;
  if (t < n_rows) {
    const T* src = table + (size_t)ids[t] * H;
    for (int i = i0 + threadIdx.x; i < i1; i += blockDim.x) {
      const float x = to_f(src[i]);
      out[(size_t)t * H + i] = x;
      rows[(size_t)t * H + i] = (bf16_t)(x * to_f(norm_w[i]));
      ss += x * x;
    }
  }
  ss = block_sum(ss, red);
  if (threadIdx.x == 0) pieces[run * 16 + t] = ss;
}

extern "C" int ifx_embedding_norm(const int* ids, const void* table, int table_dtype, const void* norm_w, float* out,
                                  void* rows, float* pieces, int T, int H, void* stream) {
  IFX_REQUIRE(T >= 0 && T <= 16 && H > 0, "embedding_norm: T=%d must be at most 16 (H=%d)", T, H);
  IFX_REQUIRE(norm_w && out && rows && pieces, "embedding_norm: needs the norm's weight and three outputs");
  if (T == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid(16, (H + 4095) / 4096);
  if (table_dtype == DT_F32)
    hipLaunchKernelGGL(embedding_norm_kernel<float>, grid, dim3(256), 0, s, ids, (const float*)table, (const bf16_t*)norm_w, out, (bf16_t*)rows, pieces, T, H);
  else if (table_dtype == DT_BF16)
    hipLaunchKernelGGL(embedding_norm_kernel<bf16_t>, grid, dim3(256), 0, s, ids, (const bf16_t*)table, (const bf16_t*)norm_w, out, (bf16_t*)rows, pieces, T, H);
  else
    IFX_FAIL("embedding_norm: unknown dtype %d", table_dtype);
  IFX_LAUNCH_CHECK();
}

// ---------------------------------------------------------------------------------------
// x = residual[src] (+ delta[src]);  if write_back: residual[src] = x
// out[r, :] = x * rsqrt(mean(x^2) + eps) * weight         src = rows ? rows[r] : r
template <typename TD, typename TO>
__global__ void add_rmsnorm_kernel(float* __restrict__ residual, const TD* __restrict__ delta,
                                   const void* __restrict__ weight, int weight_dtype,
                                   TO* __restrict__ out, const int* __restrict__ rows, int H, float eps,
                                   int write_back, int n_slices, size_t slice_stride) {
  __shared__ float red[16];
  const int r = blockIdx.x;
  const size_t src = rows ? (size_t)rows[r] : (size_t)r;
  float* res = residual + src * H;
  const TD* dl = delta ? delta + src * H : nullptr;
  // the delta may come as partial sums: slice s lies slice_stride elements after slice s - 1
  auto delta_at = [&](int i) {
    float d = to_f(dl[i]);
    for (int s = 1; s < n_slices; ++s) d += to_f(dl[(size_t)s * slice_stride + i]);
    return d;
  };
  float ss = 0.f;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    float x = res[i];
    if (dl) {
      x += delta_at(i);
      if (write_back) res[i] = x;
    }
    ss += x * x;
  }
  ss = block_sum(ss, red);
  const float rms = rsqrtf(ss / (float)H + eps);
  TO* o = out + (size_t)r * H;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    float x = res[i];
    if (dl && !write_back) x += delta_at(i);
    o[i] = from_f<TO>(x * rms * load_dyn(weight, weight_dtype, i));
  }
}

// The same, for H a multiple of 4 up to 4 * 256 * NV: each thread keeps its elements in registers,
// so the row is read once, in 16-byte pieces.
template <typename T> struct Vec4;
template <> struct Vec4<float> { typedef float4 type; };
template <> struct Vec4<bf16_t> { typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 type; };

template <typename T> __device__ __forceinline__ void load4(const T* p, float* v);
template <> __device__ __forceinline__ void load4<float>(const float* p, float* v) {
  const float4 t = *(const float4*)p; v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
}
template <> __device__ __forceinline__ void load4<bf16_t>(const bf16_t* p, float* v) {
  const typename Vec4<bf16_t>::type t = *(const typename Vec4<bf16_t>::type*)p;
#pragma unroll
  for (int i = 0; i < 4; ++i) v[i] = (float)t[i];
}
template <typename T> __device__ __forceinline__ void store4(T* p, const float* v);
template <> __device__ __forceinline__ void store4<float>(float* p, const float* v) {
  *(float4*)p = make_float4(v[0], v[1], v[2], v[3]);
}
template <> __device__ __forceinline__ void store4<bf16_t>(bf16_t* p, const float* v) {
  typename Vec4<bf16_t>::type t;
#pragma unroll
  for (int i = 0; i < 4; ++i) t[i] = (__bf16)v[i];
  *(typename Vec4<bf16_t>::type*)p = t;
}

template <typename TD, typename TO, typename TW, int NV>
__global__ __launch_bounds__(256) void add_rmsnorm_vec_kernel(float* __restrict__ residual, const TD* __restrict__ delta,
                                                              const TW* __restrict__ weight, TO* __restrict__ out,
                                                              const int* __restrict__ rows, int H, float eps, int write_back) {
  __shared__ float red[16];
  const int r = blockIdx.x;
  const size_t src = rows ? (size_t)rows[r] : (size_t)r;
  float* res = residual + src * H;
  const TD* dl = delta ? delta + src * H : nullptr;
  float x[NV][4];
  float ss = 0.f;
#pragma unroll
  for (int v = 0; v < NV; ++v) {
    const int i = 4 * (threadIdx.x + 256 * v);
    if (i < H) {
      load4<float>(res + i, x[v]);
      if (dl) {
        float d4[4];
        load4<TD>(dl + i, d4);
#pragma unroll
        for (int e = 0; e < 4; ++e) x[v][e] += d4[e];
        if (write_back) store4<float>(res + i, x[v]);
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) ss += x[v][e] * x[v][e];
    }
  }
  ss = block_sum(ss, red);
  const float rms = rsqrtf(ss / (float)H + eps);
  TO* o = out + (size_t)r * H;
#pragma unroll
  for (int v = 0; v < NV; ++v) {
    const int i = 4 * (threadIdx.x + 256 * v);
    if (i < H) {
      float w4[4], y[4];
      load4<TW>(weight + i, w4);
#pragma unroll
      for (int e = 0; e < 4; ++e) y[e] = x[v][e] * rms * w4[e];
      store4<TO>(o + i, y);
    }
  }
}


// The same with the delta given as float partial sums (n_slices of them, slice_stride elements apart, added in slice
// order): the few rows of a decode step, where the kernel's time is its chain of trips to the L2.
template <typename TD, typename TO, typename TW, int NV>
__global__ __launch_bounds__(256) void add_rmsnorm_slices_kernel(float* __restrict__ residual, const TD* __restrict__ delta,
                                                              const TW* __restrict__ weight, TO* __restrict__ out,
                                                              const int* __restrict__ rows, int H, float eps, int write_back,
                                                              int n_slices, size_t slice_stride) {
  __shared__ float red[16];
  const int r = blockIdx.x;
  const size_t src = rows ? (size_t)rows[r] : (size_t)r;
  float* res = residual + src * H;
  const TD* dl = delta ? delta + src * H : nullptr;
  float x[NV][4];
  float ss = 0.f;
  // Every load that does not depend on another goes out before the first is used: the row and the delta (or
  // its first slice) for all of the thread's elements, then the further slices, up to seven at a time, for all elements.
  // With the elements outermost a row of 8 slices cost a dozen trips to the L2 one after the other.
#pragma unroll
  for (int v = 0; v < NV; ++v) {
    const int i = 4 * (threadIdx.x + 256 * v);
    if (i < H) load4<float>(res + i, x[v]);
    else x[v][0] = x[v][1] = x[v][2] = x[v][3] = 0.f;
  }
  if (dl) {
    float d4[NV][4];
#pragma unroll
    for (int v = 0; v < NV; ++v) {
      const int i = 4 * (threadIdx.x + 256 * v);
      if (i < H) load4<TD>(dl + i, d4[v]);
      else d4[v][0] = d4[v][1] = d4[v][2] = d4[v][3] = 0.f;
    }
    constexpr int AT_ONCE = NV <= 4 ? 7 : 4;   // (the products cut K into at most eight slices: one trip for all of them)
    for (int s0 = 1; s0 < n_slices; s0 += AT_ONCE) {   // partial sums, added in slice order
      float p4[AT_ONCE][NV][4];
#pragma unroll
      for (int u = 0; u < AT_ONCE; ++u)
#pragma unroll
        for (int v = 0; v < NV; ++v) {
          const int i = 4 * (threadIdx.x + 256 * v);
          if (s0 + u < n_slices && i < H) load4<TD>(dl + (size_t)(s0 + u) * slice_stride + i, p4[u][v]);
          else p4[u][v][0] = p4[u][v][1] = p4[u][v][2] = p4[u][v][3] = 0.f;
        }
#pragma unroll
      for (int u = 0; u < AT_ONCE; ++u)
#pragma unroll
        for (int v = 0; v < NV; ++v)
#pragma unroll
          for (int e = 0; e < 4; ++e) d4[v][e] += p4[u][v][e];
    }
#pragma unroll
    for (int v = 0; v < NV; ++v) {
      const int i = 4 * (threadIdx.x + 256 * v);
#pragma unroll
      for (int e = 0; e < 4; ++e) x[v][e] += d4[v][e];
      if (write_back && i < H) store4<float>(res + i, x[v]);
    }
  }
#pragma unroll
  for (int v = 0; v < NV; ++v)
#pragma unroll
    for (int e = 0; e < 4; ++e) ss += x[v][e] * x[v][e];
  ss = block_sum(ss, red);
  const float rms = rsqrtf(ss / (float)H + eps);
  TO* o = out + (size_t)r * H;
#pragma unroll
  for (int v = 0; v < NV; ++v) {
    const int i = 4 * (threadIdx.x + 256 * v);
    if (i < H) {
      float w4[4], y[4];
      load4<TW>(weight + i, w4);      // (asked for only now: held across the sum, it costs registers that many-row launches miss)
#pragma unroll
      for (int e = 0; e < 4; ++e) y[e] = x[v][e] * rms * w4[e];
      store4<TO>(o + i, y);
    }
  }
}

template <typename TD, typename TO, typename TW>
static void launch_rmsnorm_vec(float* residual, const void* delta, const void* weight, void* out, const int* rows,
                               int n_rows, int H, float eps, int write_back, int n_slices, size_t slice_stride, hipStream_t s) {
#define GO(NV_)                                                                                                              \
  do {                                                                                                                       \
    if (n_slices > 1)                                                                                                        \
      hipLaunchKernelGGL((add_rmsnorm_slices_kernel<TD, TO, TW, NV_>), dim3(n_rows), dim3(256), 0, s, residual, (const TD*)delta, \
                         (const TW*)weight, (TO*)out, rows, H, eps, write_back, n_slices, slice_stride);                      \
    else                                                                                                                     \
      hipLaunchKernelGGL((add_rmsnorm_vec_kernel<TD, TO, TW, NV_>), dim3(n_rows), dim3(256), 0, s, residual, (const TD*)delta, \
                         (const TW*)weight, (TO*)out, rows, H, eps, write_back);                                              \
  } while (0)
  if (H <= 4 * 256 * 2) GO(2);
  else if (H <= 4 * 256 * 4) GO(4);
  else GO(8);
#undef GO
}

// n_slices > 1: ``delta`` (float32) holds that many partial sums, slice_stride elements apart, added in order.
extern "C" int ifx_add_rmsnorm(float* residual, const void* delta, int delta_dtype, const void* weight,
                               int weight_dtype, void* out, int out_dtype, const int* rows, int n_rows,
                               int H, float eps, int write_back, int n_slices, long long slice_stride, void* stream) {
  IFX_REQUIRE(n_rows >= 0 && H > 0, "add_rmsnorm: bad sizes rows=%d H=%d", n_rows, H);
  IFX_REQUIRE(n_slices >= 1 && (n_slices == 1 || (delta && delta_dtype == DT_F32 && slice_stride > 0)),
              "add_rmsnorm: %d slices need a float32 delta and their distance", n_slices);
  IFX_REQUIRE(!(rows && write_back), "add_rmsnorm: a row gather cannot write the residual back");
  if (n_rows == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const int dd = delta ? delta_dtype : out_dtype;
  IFX_REQUIRE((dd == DT_F32 || dd == DT_BF16) && (out_dtype == DT_F32 || out_dtype == DT_BF16) &&
              (weight_dtype == DT_F32 || weight_dtype == DT_BF16),
              "add_rmsnorm: unknown dtypes delta=%d out=%d weight=%d", delta_dtype, out_dtype, weight_dtype);
  if (H % 4 == 0 && H <= 4 * 256 * 8) {
#define VEC(TD, TO)                                                                                                  \
  do {                                                                                                               \
    if (weight_dtype == DT_F32) launch_rmsnorm_vec<TD, TO, float>(residual, delta, weight, out, rows, n_rows, H, eps, write_back, n_slices, (size_t)slice_stride, s); \
    else launch_rmsnorm_vec<TD, TO, bf16_t>(residual, delta, weight, out, rows, n_rows, H, eps, write_back, n_slices, (size_t)slice_stride, s);      \
  } while (0)
    if (dd == DT_F32 && out_dtype == DT_F32) VEC(float, float);
    else if (dd == DT_BF16 && out_dtype == DT_BF16) VEC(bf16_t, bf16_t);
    else if (dd == DT_F32 && out_dtype == DT_BF16) VEC(float, bf16_t);
    else VEC(bf16_t, float);
#undef VEC
    IFX_LAUNCH_CHECK();
  }
  const int threads = H >= 2048 ? 512 : 256;
#define LAUNCH(TD, TO)                                                                              \
  hipLaunchKernelGGL((add_rmsnorm_kernel<TD, TO>), dim3(n_rows), dim3(threads), 0, s, residual,     \
                     (const TD*)delta, weight, weight_dtype, (TO*)out, rows, H, eps, write_back, n_slices, (size_t)slice_stride)
  if (dd == DT_F32 && out_dtype == DT_F32) LAUNCH(float, float);
  else if (dd == DT_BF16 && out_dtype == DT_BF16) LAUNCH(bf16_t, bf16_t);
  else if (dd == DT_F32 && out_dtype == DT_BF16) LAUNCH(float, bf16_t);
  else LAUNCH(bf16_t, float);
#undef LAUNCH
  IFX_LAUNCH_CHECK();
}

// ---------------------------------------------------------------------------------------
// cos[t, p], sin[t, p] of angle = float(positions[t]) * inv_freq[p]: the step's rotation table, made
// once per step and read by every layer.
__global__ void rope_table_kernel(const int* __restrict__ positions, const float* __restrict__ inv_freq,
                                  float* __restrict__ cs, float* __restrict__ sn, int n_pairs, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int t = i / n_pairs, p = i % n_pairs;
  sincosf((float)positions[t] * inv_freq[p], &sn[i], &cs[i]);
}

extern "C" int ifx_rope_table(const int* positions, const float* inv_freq, float* cs, float* sn, int T, int n_pairs,
                              void* stream) {
  IFX_REQUIRE(T >= 0 && n_pairs > 0, "rope_table: bad sizes T=%d pairs=%d", T, n_pairs);
  if (T == 0) return 0;
  const int n = T * n_pairs;
  hipLaunchKernelGGL(rope_table_kernel, dim3((n + 255) / 256), dim3(256), 0, (hipStream_t)stream, positions, inv_freq, cs, sn,
                     n_pairs, n);
  IFX_LAUNCH_CHECK();
}

// ---------------------------------------------------------------------------------------
// Per token t: qkv[t] = [q (nH*d) | k (nKV*d) | v (nKV*dv)].  Adds the bias, rotates q and k by
// the token's position, writes q to q_out[t] and k, v into the paged cache at slot[t]
// (slot = page * page_size + offset; slot < 0: nothing is written to the cache).
// Cache layouts: K [page][kv head][offset][d], V [page][kv head][dv][offset]; values may be
// narrower or wider than keys (dv != d).
// rope_style: 0 none, 1 split-half pairs (p, p + rot/2), 2 consecutive pairs (2p, 2p+1);
// cos/sin come from the step's table [T, rotary_dim / 2]; elements at or beyond rotary_dim are
// copied.  One block per (token, head): q heads, then k heads, then v heads.
struct RopeArgs {
  const void* qkv;       // [T, row width] of the activation type, or with n_slices > 1 float partial sums
  int n_slices;          // [n_slices][T, row width], slice_stride elements apart, added in order
  size_t slice_stride;
  const void* bias;
  int bias_dtype;
  const int* slots;
  const float* cs;
  const float* sn;
  int rope_style;
  int rotary_dim;
  int nH, nKV, d, page_size;
  void* q_out;
  void* k_cache;
  void* v_cache;
  int dv;                // width of a value head
};

template <typename T>
__global__ __launch_bounds__(64) void rope_append_kernel(RopeArgs a) {
  const int t = blockIdx.x, head = blockIdx.y;
  const int d = a.d, dv = a.dv, half = d / 2, rot_half = a.rope_style != 0 ? a.rotary_dim / 2 : 0;
  const int q_width = a.nH * d, kv_width = a.nKV * d, row_width = q_width + kv_width + a.nKV * dv;
  const T* row = (const T*)a.qkv + (size_t)t * row_width;
  const float* part = (const float*)a.qkv + (size_t)t * row_width;
  // Elements i0 and i1 of the row; partial sums are added in slice order, eight slices of both elements asked for
  // together (one after the other every slice would cost a trip to the L2).
  auto in2 = [&](int i0, int i1, float& x0, float& x1) {
    if (a.n_slices <= 1) { x0 = to_f(row[i0]); x1 = to_f(row[i1]); return; }
    for (int s0 = 0; s0 < a.n_slices; s0 += 8) {
      float p0[8], p1[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        p0[u] = s0 + u < a.n_slices ? part[(size_t)(s0 + u) * a.slice_stride + i0] : 0.f;
        p1[u] = s0 + u < a.n_slices ? part[(size_t)(s0 + u) * a.slice_stride + i1] : 0.f;
      }
      if (s0 == 0) { x0 = p0[0]; x1 = p1[0]; }
#pragma unroll
      for (int u = 0; u < 8; ++u)
        if (s0 + u > 0) { x0 += p0[u]; x1 += p1[u]; }
    }
  };
  const int slot = a.slots ? a.slots[t] : -1;
  const int page = slot >= 0 ? slot / a.page_size : 0, off = slot >= 0 ? slot % a.page_size : 0;
  const int col = head * d;  // q heads, k heads and v heads follow each other in the row
  if (head < a.nH + a.nKV) {
    const bool is_q = head < a.nH;
    if (!is_q && slot < 0) return;
    T* dst = is_q ? (T*)a.q_out + (size_t)t * q_width + col
                  : (T*)a.k_cache + (((size_t)page * a.nKV + (head - a.nH)) * a.page_size + off) * d;
    for (int p = threadIdx.x; p < half; p += blockDim.x) {
      int i0, i1;
      const bool rotate = p < rot_half;
      if (rotate) {
        if (a.rope_style == 1) { i0 = p; i1 = p + rot_half; }
        else { i0 = 2 * p; i1 = 2 * p + 1; }
      } else {
        i0 = 2 * p; i1 = 2 * p + 1;  // beyond the rotated part pairs are consecutive in both styles
      }
      float x0, x1;
      in2(col + i0, col + i1, x0, x1);
      if (a.bias) {
        x0 += load_dyn(a.bias, a.bias_dtype, col + i0);
        x1 += load_dyn(a.bias, a.bias_dtype, col + i1);
      }
      float y0 = x0, y1 = x1;
      if (rotate) {
        const float cs = a.cs[(size_t)t * rot_half + p], sn = a.sn[(size_t)t * rot_half + p];
        y0 = x0 * cs - x1 * sn;
        y1 = x0 * sn + x1 * cs;
      }
      dst[i0] = from_f<T>(y0);
      dst[i1] = from_f<T>(y1);
    }
  } else {
    if (slot < 0) return;
    const int kh = head - a.nH - a.nKV;
    const int vcol = q_width + kv_width + kh * dv;              // value heads are dv wide
    T* vc = (T*)a.v_cache + ((size_t)page * a.nKV + kh) * dv * a.page_size + off;
    for (int e = threadIdx.x; e < dv; e += 2 * blockDim.x) {    // two elements per thread and round: their loads go out together
      const int e1 = min(e + (int)blockDim.x, dv - 1);
      float x, x1;
      in2(vcol + e, vcol + e1, x, x1);
      if (a.bias) { x += load_dyn(a.bias, a.bias_dtype, vcol + e); x1 += load_dyn(a.bias, a.bias_dtype, vcol + e1); }
      vc[(size_t)e * a.page_size] = from_f<T>(x);
      if (e + (int)blockDim.x < dv) vc[(size_t)e1 * a.page_size] = from_f<T>(x1);
    }
  }
}

// The common case in 16-byte pieces: bfloat16, split-half pairs over the whole head, head size a
// multiple of 16, bias bfloat16 or none.  The first n_qk_blocks blocks rotate q and k: a thread takes 8
// consecutive dimensions of the first half of a head and their 8 partners in the second.  The other
// blocks append v: a thread takes one dimension of one kv head for 8 consecutive tokens and, when
// their slots are 8 consecutive offsets of one page starting at a multiple of 8, writes them as one
// piece of the transposed page; otherwise element by element.
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 rope_bf16x8;

__global__ __launch_bounds__(256) void rope_append_vec_kernel(RopeArgs a, int T, int n_qk_blocks) {
  const int d = a.d, half = d / 2;
  const int q_width = a.nH * d, kv_width = a.nKV * d, row_width = q_width + 2 * kv_width;
  const bf16_t* qkv = (const bf16_t*)a.qkv;
  const bf16_t* bias = (const bf16_t*)a.bias;
  if ((int)blockIdx.x < n_qk_blocks) {
    const int per_head = d / 16, heads = a.nH + (a.slots ? a.nKV : 0);
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (size_t)T * heads * per_head) return;
    const int j = (int)(idx % per_head), head = (int)(idx / per_head % heads), t = (int)(idx / per_head / heads);
    const int col = head * d + 8 * j;
    const bf16_t* row = qkv + (size_t)t * row_width + col;
    rope_bf16x8 x0 = *(const rope_bf16x8*)row, x1 = *(const rope_bf16x8*)(row + half);
    float f0[8], f1[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) { f0[e] = (float)x0[e]; f1[e] = (float)x1[e]; }
    if (bias) {
      const rope_bf16x8 b0 = *(const rope_bf16x8*)(bias + col), b1 = *(const rope_bf16x8*)(bias + col + half);
#pragma unroll
      for (int e = 0; e < 8; ++e) { f0[e] += (float)b0[e]; f1[e] += (float)b1[e]; }
    }
    const float* cs = a.cs + (size_t)t * half + 8 * j;
    const float* sn = a.sn + (size_t)t * half + 8 * j;
    rope_bf16x8 y0, y1;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      y0[e] = (__bf16)(f0[e] * cs[e] - f1[e] * sn[e]);
      y1[e] = (__bf16)(f0[e] * sn[e] + f1[e] * cs[e]);
    }
    bf16_t* dst;
    if (head < a.nH) {
      dst = (bf16_t*)a.q_out + (size_t)t * q_width + col;
    } else {
      const int slot = a.slots[t];
      if (slot < 0) return;
      const int page = slot / a.page_size, off = slot % a.page_size;
      dst = (bf16_t*)a.k_cache + (((size_t)page * a.nKV + (head - a.nH)) * a.page_size + off) * d + 8 * j;
    }
    *(rope_bf16x8*)dst = y0;
    *(rope_bf16x8*)(dst + half) = y1;
    return;
  }
  // v: (group of 8 tokens, kv head, dimension)
  const size_t idx = (size_t)(blockIdx.x - n_qk_blocks) * 256 + threadIdx.x;
  const int groups = (T + 7) / 8;
  if (idx >= (size_t)groups * a.nKV * d) return;
  const int e = (int)(idx % d), kh = (int)(idx / d % a.nKV), t0 = (int)(idx / d / a.nKV) * 8;
  const int col = q_width + kv_width + kh * d + e;
  const float b = bias ? (float)bias[col] : 0.f;
  int slot[8];
  float x[8];
#pragma unroll
  for (int k = 0; k < 8; ++k) {   // all loads of the group are independent: they go out together
    slot[k] = t0 + k < T ? a.slots[t0 + k] : -1;
    x[k] = t0 + k < T ? (float)qkv[(size_t)(t0 + k) * row_width + col] + b : 0.f;
  }
  bool run = slot[0] >= 0 && slot[0] % 8 == 0;
#pragma unroll
  for (int k = 1; k < 8; ++k) run = run && slot[k] == slot[0] + k;
  bf16_t* vc = (bf16_t*)a.v_cache;
  if (run) {
    rope_bf16x8 v;
#pragma unroll
    for (int k = 0; k < 8; ++k) v[k] = (__bf16)x[k];
    const int page = slot[0] / a.page_size, off = slot[0] % a.page_size;
    *(rope_bf16x8*)(vc + (((size_t)page * a.nKV + kh) * d + e) * a.page_size + off) = v;
  } else {
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      if (slot[k] < 0) continue;
      const int page = slot[k] / a.page_size, off = slot[k] % a.page_size;
      vc[(((size_t)page * a.nKV + kh) * d + e) * a.page_size + off] = (__bf16)x[k];
    }
  }
}

// dtype: the type of q_out and the cache, and of qkv unless n_slices > 1 (then qkv holds float partial sums,
// slice_stride elements apart).
extern "C" int ifx_rope_append(const void* qkv, int dtype, const void* bias, int bias_dtype, const int* slots,
                               const float* cs, const float* sn, int rope_style, int rotary_dim, int T, int nH,
                               int nKV, int d, int page_size, void* q_out, void* k_cache, void* v_cache, int n_slices,
                               long long slice_stride, int dv, void* stream) {
  IFX_REQUIRE(n_slices >= 1 && (n_slices == 1 || slice_stride > 0), "rope_append: %d slices, %lld apart", n_slices, slice_stride);
  IFX_REQUIRE(T >= 0 && nH > 0 && nKV >= 0 && d > 0 && d % 2 == 0 && dv > 0, "rope_append: bad sizes T=%d nH=%d nKV=%d d=%d dv=%d", T, nH, nKV, d, dv);
  IFX_REQUIRE(rope_style >= 0 && rope_style <= 2, "rope_append: unknown rope style %d", rope_style);
  IFX_REQUIRE(rope_style == 0 || (rotary_dim > 0 && rotary_dim <= d && rotary_dim % 2 == 0 && cs && sn),
              "rope_append: rotary_dim %d must be even, within head_dim %d, with a rotation table", rotary_dim, d);
  IFX_REQUIRE(!slots || (page_size > 0 && k_cache && v_cache), "rope_append: cache write without cache");
  IFX_REQUIRE(nH + 2 * nKV <= 65535, "rope_append: too many heads for one launch");
  if (T == 0) return 0;
  RopeArgs a{qkv, n_slices, (size_t)slice_stride, bias, bias_dtype, slots, cs, sn, rope_style, rotary_dim, nH, nKV, d, page_size,
             q_out, k_cache, v_cache, dv};
  hipStream_t s = (hipStream_t)stream;
  // (a few tokens are quicker with one small block per token and head: nothing waits on a loop over tokens)
  if (dv == d && T >= 128 && n_slices == 1 && dtype == DT_BF16 && rope_style == 1 && rotary_dim == d && d % 16 == 0 && (!bias || bias_dtype == DT_BF16) &&
      (!slots || page_size % 8 == 0)) {
    const size_t qk_threads = (size_t)T * (nH + (slots ? nKV : 0)) * (d / 16);
    const size_t v_threads = slots ? (size_t)((T + 7) / 8) * nKV * d : 0;
    const unsigned qk_blocks = (unsigned)((qk_threads + 255) / 256), v_blocks = (unsigned)((v_threads + 255) / 256);
    hipLaunchKernelGGL(rope_append_vec_kernel, dim3(qk_blocks + v_blocks), dim3(256), 0, s, a, T, (int)qk_blocks);
    IFX_LAUNCH_CHECK();
  }
  const dim3 grid(T, nH + 2 * nKV);
  if (dtype == DT_F32) hipLaunchKernelGGL(rope_append_kernel<float>, grid, dim3(64), 0, s, a);
  else if (dtype == DT_BF16) hipLaunchKernelGGL(rope_append_kernel<bf16_t>, grid, dim3(64), 0, s, a);
  else IFX_FAIL("rope_append: unknown dtype %d", dtype);
  IFX_LAUNCH_CHECK();
}

// ---------------------------------------------------------------------------------------
// out[t, i] = gate / (1 + exp(-gate)) * up, with gu[t] = [gate (I) | up (I)] or, interleaved,
// gu[t] = [gate_0, up_0, gate_1, up_1, ...].
template <typename T>
__global__ void swiglu_kernel(const T* __restrict__ gu, T* __restrict__ out, int I, size_t n, int interleaved) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= n) return;
  const size_t t = idx / I;
  const int i = (int)(idx % I);
  const float g = to_f(gu[t * 2 * I + (interleaved ? 2 * i : i)]);
  const float u = to_f(gu[t * 2 * I + (interleaved ? 2 * i + 1 : I + i)]);
  out[idx] = from_f<T>(g / (1.0f + expf(-g)) * u);
}

// The interleaved bf16 case in 32-byte pieces: 8 gate/up pairs in, 8 results out (I a multiple of 8).
__global__ void swiglu_pairs_bf16_kernel(const bf16_t* __restrict__ gu, bf16_t* __restrict__ out, size_t n8) {
  typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n8) return;
  const bf16x8 a = *(const bf16x8*)(gu + 16 * i), b = *(const bf16x8*)(gu + 16 * i + 8);
  bf16x8 o;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const float g0 = (float)a[2 * e], u0 = (float)a[2 * e + 1], g1 = (float)b[2 * e], u1 = (float)b[2 * e + 1];
    o[e] = (__bf16)(g0 / (1.0f + expf(-g0)) * u0);
    o[e + 4] = (__bf16)(g1 / (1.0f + expf(-g1)) * u1);
  }
  *(bf16x8*)(out + 8 * i) = o;
}

extern "C" int ifx_swiglu(const void* gu, void* out, int dtype, int T, int I, int interleaved, void* stream) {
  IFX_REQUIRE(T >= 0 && I > 0, "swiglu: bad sizes T=%d I=%d", T, I);
  if (T == 0) return 0;
  const size_t n = (size_t)T * I;
  if (interleaved && dtype == DT_BF16 && I % 8 == 0) {
    const size_t n8 = n / 8;
    hipLaunchKernelGGL(swiglu_pairs_bf16_kernel, dim3((unsigned)((n8 + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                       (const bf16_t*)gu, (bf16_t*)out, n8);
    IFX_LAUNCH_CHECK();
  }
  const unsigned blocks = (unsigned)((n + 255) / 256);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == DT_F32) hipLaunchKernelGGL(swiglu_kernel<float>, dim3(blocks), dim3(256), 0, s, (const float*)gu, (float*)out, I, n, interleaved);
  else if (dtype == DT_BF16) hipLaunchKernelGGL(swiglu_kernel<bf16_t>, dim3(blocks), dim3(256), 0, s, (const bf16_t*)gu, (bf16_t*)out, I, n, interleaved);
  else IFX_FAIL("swiglu: unknown dtype %d", dtype);
  IFX_LAUNCH_CHECK();
}

