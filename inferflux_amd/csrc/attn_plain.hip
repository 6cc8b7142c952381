// Plain attention over the paged cache: any head size up to 256, float or bf16 storage, float
// math.  One wave per (query row, query head): each lane scores one key of a 64-key tile, the
// wave takes the tile's maximum and sum, then every lane accumulates its output elements over
// the tile's keys in ascending order.  Tiles are aligned to absolute key positions (multiples of
// 64), so the sequence of operations for a (position, head) is the same however the request was
// cut into steps: results are bit-equal across cuttings.  This is the attention of the 32-bit
// path and the reference beside the matrix-core kernels.
//
// Formula (runtime/backends/cuda/kernels/flash_attention.cu:71-72 GQA map, 86 causal limit, 144
// scale after the dot product, 152-173 online softmax): head h reads kv head h / (nH / nKV);
// the query at position p sees keys j with max(0, p - window + 1) <= j <= p; s_j = (q . k_j) *
// scale; o = sum_j softmax(s)_j v_j.
//
// Cache layouts: K [page][kv head][offset][d], V [page][kv head][dv][offset].  Values may have another width
// than keys (dv != d): the output row of a head then has dv elements.
#include "common.h"

IFX_DEFINE_LAST_ERROR()

#define MAX_D 256
#define DC (MAX_D / WAVE)
#define WAVES_PER_BLOCK 4

struct AttnArgs {
  const void* q;
  const void* k_cache;
  const void* v_cache;
  void* out;
  const int* row_req;
  const int* positions;
  const int* block_table;
  int max_blocks;
  int T, nH, nKV, d, dv, page_size, window;
  float scale;
};

template <typename T>
__global__ __launch_bounds__(WAVE * WAVES_PER_BLOCK) void attn_plain_kernel(AttnArgs a) {
  __shared__ float q_s[WAVES_PER_BLOCK][MAX_D];
  const int wid = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const long long item = (long long)blockIdx.x * WAVES_PER_BLOCK + wid;
  // All lanes of a wave share `item`, so the whole wave leaves together; no block-wide
  // barrier follows.
  if (item >= (long long)a.T * a.nH) return;
  const int row = (int)(item / a.nH), head = (int)(item % a.nH);
  const int d = a.d, dv = a.dv, P = a.page_size;
  const int kvh = head / (a.nH / a.nKV);
  const int pos = a.positions[row];
  const int* table = a.block_table + (size_t)a.row_req[row] * a.max_blocks;
  const int lo = a.window > 0 ? max(0, pos - a.window + 1) : 0;

  const T* qrow = (const T*)a.q + ((size_t)row * a.nH + head) * d;
  for (int e = lane; e < d; e += WAVE) q_s[wid][e] = to_f(qrow[e]);
  // q_s[wid] is written and read by this wave only.
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_s_waitcnt(0);

  float m = -INFINITY, l = 0.f;
  float acc[DC];
#pragma unroll
  for (int c = 0; c < DC; ++c) acc[c] = 0.f;

  const T* Kc = (const T*)a.k_cache;
  const T* Vc = (const T*)a.v_cache;
  for (int t0 = (lo / WAVE) * WAVE; t0 <= pos; t0 += WAVE) {
    const int j = t0 + lane;
    const bool valid = j >= lo && j <= pos;
    int page = 0, off = 0;
    float s = -INFINITY;
    if (valid) {
      page = table[j / P];
      off = j % P;
      const T* kr = Kc + (((size_t)page * a.nKV + kvh) * P + off) * d;
      float dot = 0.f;
      for (int e = 0; e < d; ++e) dot = fmaf(q_s[wid][e], to_f(kr[e]), dot);
      s = dot * a.scale;
    }
    const float m_new = fmaxf(m, wave_max(s));  // finite: the tile holds key `lo` or later, up to pos
    const float p = valid ? expf(s - m_new) : 0.f;
    const float alpha = expf(m - m_new);  // 0 on the first tile (m = -inf)
    l = l * alpha + wave_sum(p);
#pragma unroll
    for (int c = 0; c < DC; ++c) acc[c] *= alpha;
    for (int jj = 0; jj < WAVE; ++jj) {
      const float pj = __shfl(p, jj, WAVE);
      const int pg = __shfl(page, jj, WAVE), of = __shfl(off, jj, WAVE);
      if (pj == 0.f) continue;  // uniform over the wave; keys outside the range are never read
      const T* vb = Vc + ((size_t)pg * a.nKV + kvh) * dv * P + of;
#pragma unroll
      for (int c = 0; c < DC; ++c) {
        const int e = lane + c * WAVE;
        if (e < dv) acc[c] = fmaf(pj, to_f(vb[(size_t)e * P]), acc[c]);
      }
    }
    m = m_new;
  }
  T* orow = (T*)a.out + ((size_t)row * a.nH + head) * dv;
  const float inv = l > 0.f ? 1.f / l : 0.f;
#pragma unroll
  for (int c = 0; c < DC; ++c) {
    const int e = lane + c * WAVE;
    if (e < dv) orow[e] = from_f<T>(acc[c] * inv);
  }
}

extern "C" int ifx_attn_plain(const void* q, const void* k_cache, const void* v_cache, void* out, int dtype,
                              const int* row_req, const int* positions, const int* block_table,
                              int max_blocks, int T, int nH, int nKV, int d, int dv, int page_size, int window,
                              float scale, void* stream) {
  IFX_REQUIRE(T >= 0 && nH > 0 && nKV > 0 && nH % nKV == 0, "attn_plain: bad head counts nH=%d nKV=%d", nH, nKV);
  IFX_REQUIRE(d > 0 && d <= MAX_D, "attn_plain: head_dim %d outside 1..%d", d, MAX_D);
  IFX_REQUIRE(dv > 0 && dv <= MAX_D, "attn_plain: value head_dim %d outside 1..%d", dv, MAX_D);
  IFX_REQUIRE(page_size > 0 && max_blocks > 0 && window >= 0, "attn_plain: bad page_size/max_blocks/window");
  if (T == 0) return 0;
  AttnArgs a{q, k_cache, v_cache, out, row_req, positions, block_table, max_blocks, T, nH, nKV, d, dv, page_size, window, scale};
  const long long items = (long long)T * nH;
  const unsigned blocks = (unsigned)((items + WAVES_PER_BLOCK - 1) / WAVES_PER_BLOCK);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == DT_F32) hipLaunchKernelGGL(attn_plain_kernel<float>, dim3(blocks), dim3(WAVE * WAVES_PER_BLOCK), 0, s, a);
  else if (dtype == DT_BF16) hipLaunchKernelGGL(attn_plain_kernel<bf16_t>, dim3(blocks), dim3(WAVE * WAVES_PER_BLOCK), 0, s, a);
  else IFX_FAIL("attn_plain: unknown dtype %d", dtype);
  IFX_LAUNCH_CHECK();
}
