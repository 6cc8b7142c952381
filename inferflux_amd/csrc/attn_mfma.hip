// Attention over the paged cache on the matrix cores (bf16 in, float accumulate), for one head
// size fixed at compile time (-DHEAD_DIM=..., a multiple of 16 up to 256).
//
// Two kernels compute the same function as attn_plain.hip (causal, optionally windowed,
// grouped-query attention; reference formula runtime/backends/cuda/kernels/flash_attention.cu:
// 71-72, 86, 144, 152-173; split merge 944-991):
//
//   rows   one wave per (row, kv head, split of the key range): the query heads that share the
//          kv head are the 16 columns of the matrix tile, so keys and values are read once for
//          all of them (any group size; more than 16 heads take several passes).  Partial
//          results (max, sum, unnormalised output) go to scratch and a second kernel merges
//          the splits.  For decode tokens and short portions.  Where the (row, kv head) pairs of a launch fill the
//          chip by themselves, one workgroup of several waves takes a pair whole instead: its waves share the
//          keys, meet in LDS and write the output (no scratch, no second kernel).
//   tiles  one workgroup of 4 waves per (64 or 128 consecutive rows of one request, query head;
//          -DTILE_QT=1 or 2 tiles of 16 rows per wave): key and value tiles of 64 positions are
//          staged in LDS and shared by the 4 waves.  For long portions of prompts.  The keys can
//          be cut into splits that run as workgroups of their own and are merged like the row
//          kernel's (portions late in a long context: few tiles, many keys).
//
// Both work on transposed tiles so that no register shuffle is needed between the two matrix
// products: S^T[key, q] = K Q^T leaves each lane holding four consecutive keys of one query
// column, which is exactly the operand layout of O^T[dim, q] += V^T[dim, key] P^T[key, q].
// The cache layouts make both A operands contiguous: K [page][kv head][offset][d] and
// V [page][kv head][d][offset].
//
// Softmax runs in float on the accumulators (base-2 exponent with the scale folded in); P is
// rounded to bf16 for the second product, the row sum is kept in float.
#include "common.h"

IFX_DEFINE_LAST_ERROR()

#ifndef HEAD_DIM
#error "compile with -DHEAD_DIM=<multiple of 16>"
#endif
static_assert(HEAD_DIM % 16 == 0 && HEAD_DIM >= 16 && HEAD_DIM <= 256, "HEAD_DIM must be a multiple of 16 in 16..256");

#include "attn_shared.h"

extern "C" int ifx_attn_head_dim() { return D; }

// =======================================================================================
// rows
// =======================================================================================
// The operands of one block of 32 keys (two pages' worth of 16): loaded together, K and V at once,
// so that a block costs one trip to memory, and one block ahead of the arithmetic.  The page numbers come
// from a register: lane i of ``pages`` holds entry ``page_base + i`` of the request's block table, read once
// for 64 pages, so that no block waits for a table entry before it can ask for its keys.
//
// STREAM: the keys and values are asked for with streaming loads.  A launch of many rows reads each of them once and
// gains from it (64 rows over 3,072 keys: 82 -> 76 us); a single row is faster with plain loads (a decode step of one
// request loses 1.6 % with streaming ones), so the launch chooses by its number of rows.  Pages of more than 16 tokens
// are read with plain loads always: a tile of 16 keys takes 32 bytes of each 2 P-byte row of V, and the lines must stay
// in the L2 for the tiles that want the rest (64 rows over 3,100 keys in pages of 64: 141 us streaming, 108 plain).
constexpr int ROW_STREAM_MIN_ROWS = 8;

template <bool STREAM, typename T>
__device__ __forceinline__ T row_load(const T* p) {
  if constexpr (STREAM) return __builtin_nontemporal_load(p);
  else return *p;
}

struct RowBlock {
  bf16x8 k[2][KS];
  bf16x4 v[DT][2];
  bool live[2];
};

template <bool STREAM>
__device__ __forceinline__ void load_row_block(RowBlock& b, const RowArgs& a, int pages, int page_base, int kvh, int j0,
                                               int ka, int kb, int col, int g4) {
  const int P = a.P;
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    const int k0 = j0 + 16 * t;  // 16 keys k0..k0+15, all in one page
    bool live = k0 < kb && k0 + 16 > ka;
    const int page = live ? __builtin_amdgcn_readlane(pages, k0 / P - page_base) : -1;
    live = live && page >= 0;
    b.live[t] = live;
    const int off = k0 % P;
    const bf16_t* kp = a.k_cache + (((size_t)(live ? page : 0) * a.nKV + kvh) * P + off + col) * D + 8 * g4;
    const bf16_t* vp = a.v_cache + (((size_t)(live ? page : 0) * a.nKV + kvh) * D + col) * P + off + 4 * g4;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
      b.k[t][ks] = (live && 32 * ks + 8 * g4 < D) ? row_load<STREAM>((const bf16x8*)(kp + 32 * ks)) : zero8();
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
      b.v[dt][t] = live ? row_load<STREAM>((const bf16x4*)(vp + (size_t)16 * dt * P)) : zero4();
  }
}

__device__ __forceinline__ void use_row_block(const RowBlock& b, const RowArgs& a, const bf16x8* qop, floatx4* o, float& m,
                                              float& l, int j0, int ka, int kb, int g4) {
  floatx4 s[2];
  float mb = -INFINITY;
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    s[t] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) s[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(b.k[t][ks], qop[ks], s[t], 0, 0, 0);
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int key = j0 + 16 * t + 4 * g4 + r;
      const bool vis = b.live[t] && key >= ka && key < kb;
      s[t][r] = vis ? s[t][r] * a.scale_log2e : -INFINITY;
      mb = fmaxf(mb, s[t][r]);
    }
  }
  const float m_new = fmaxf(m, col_max(mb));
  const float m_safe = m_new == -INFINITY ? 0.f : m_new;
  const float alpha = fast_exp2(m - m_safe);
  float psum = 0.f;
  bf16x4 pb[2];
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const float p = fast_exp2(s[t][r] - m_safe);
      psum += p;
      pb[t][r] = (__bf16)p;
    }
  l = l * alpha + psum;
  m = m_new;
  const bf16x8 pop = join4(pb[0], pb[1]);
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) {
#pragma unroll
    for (int r = 0; r < 4; ++r) o[dt][r] *= alpha;
    o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(join4(b.v[dt][0], b.v[dt][1]), pop, o[dt], 0, 0, 0);
  }
}

template <bool STREAM>
__global__ __launch_bounds__(WAVE) __attribute__((amdgpu_waves_per_eu(2, 2))) void attn_rows_kernel(RowArgs a) {
  const int split = blockIdx.x, kvh = blockIdx.y, ri = blockIdx.z;
  const int lane = threadIdx.x, col = lane & 15, g4 = lane >> 4;
  const int row = a.rows ? a.rows[ri] : ri;
  // A step in which every request brings one row (a decode step) says so: the row's request is the row itself, and
  // without a window a split's first key does not depend on the row's position, so the split's block-table entries
  // are asked for together with the position instead of after it (one trip to memory fewer before the first keys).
  const bool early = a.req_is_row && a.window <= 0;
  const int* early_table = a.block_table + (size_t)row * a.max_blocks;
  const int early_base = split * a.chunk / a.P;
  const int early_pages = (early && early_base + lane < a.max_blocks) ? early_table[early_base + lane] : -1;
  const int pos = a.positions[row];
  const int lo = a.window > 0 ? max(0, pos - a.window + 1) : 0;
  const int ka = max(lo, split * a.chunk), kb = min(pos + 1, (split + 1) * a.chunk);  // keys [ka, kb)
  const int ratio = a.nH / a.nKV;
  const int* table = early ? early_table : a.block_table + (size_t)a.row_req[row] * a.max_blocks;

  for (int qt = 0; qt < ratio; qt += 16) {
    const int head = kvh * ratio + qt + col;
    const bool head_ok = qt + col < ratio;
    float* po = a.part_o + (((size_t)ri * a.nH + head) * a.max_splits + split) * D;
    float* pml = a.part_ml + (((size_t)ri * a.nH + head) * a.max_splits + split) * 2;
    if (ka >= kb) {  // nothing of this split is visible: the merge skips it
      if (head_ok && g4 == 0) { pml[0] = -INFINITY; pml[1] = 0.f; }
      continue;
    }
    bf16x8 qop[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int c = 32 * ks + 8 * g4;
      qop[ks] = (head_ok && c < D) ? *(const bf16x8*)(a.q + ((size_t)row * a.nH + head) * D + c) : zero8();
    }
    floatx4 o[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) o[dt] = floatx4{0.f, 0.f, 0.f, 0.f};
    float m = -INFINITY, l = 0.f;

    RowBlock b0, b1;
    int j0 = (ka / 32) * 32;
    int page_base = early_base, pages = early_pages;
    bool have_pages = early;
    // the table entries of the block of 32 keys from j: in ``pages`` already, or read now (64 entries from j's)
    auto table_for = [&](int j) {
      if (have_pages && (j + 31) / a.P - page_base < WAVE) return;
      have_pages = true;
      page_base = j / a.P;
      pages = page_base + lane < a.max_blocks ? table[page_base + lane] : -1;
    };
    table_for(j0);
    load_row_block<STREAM>(b0, a, pages, page_base, kvh, j0, ka, kb, col, g4);
    for (; j0 < kb; j0 += 64) {
      const bool more1 = j0 + 32 < kb, more2 = j0 + 64 < kb;
      if (more1) {
        table_for(j0 + 32);
        load_row_block<STREAM>(b1, a, pages, page_base, kvh, j0 + 32, ka, kb, col, g4);
      }
      use_row_block(b0, a, qop, o, m, l, j0, ka, kb, g4);
      if (more1) {
        if (more2) {
          table_for(j0 + 64);
          load_row_block<STREAM>(b0, a, pages, page_base, kvh, j0 + 64, ka, kb, col, g4);
        }
        use_row_block(b1, a, qop, o, m, l, j0 + 32, ka, kb, g4);
      }
    }
    l = col_sum(l);
    if (head_ok) {
      if (g4 == 0) { pml[0] = m; pml[1] = l; }
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) *(floatx4*)(po + 16 * dt + 4 * g4) = o[dt];
    }
  }
}

// The same walk by a workgroup of ``a.waves`` waves per (row, kv head), for launches whose (row, kv head) pairs fill
// the chip by themselves: the row's visible keys are dealt evenly to the waves in runs of 32, every wave walks its
// share exactly as above, and the waves' (max, sum, unnormalised output) meet in LDS, are combined in wave order and
// written to ``out``.  No partial results in memory and no second launch (64 rows x 4 kv heads over 3,100 keys:
// 67 us against 88 in splits with the merge launch).
//
// Fewer pairs than compute units need a pair's keys on several units, hence a merge across workgroups.  Measured
// for that, and not kept: the workgroup that finishes a row last merges it inside the launch (partial results,
// a release fence at device scope, a counter per pair).  The fence (a write-back of the unit's L2) takes about
// 45-60 ns per workgroup and the chip serves them one after the other: 8 rows over 3,100 keys in 224 workgroups
// 36 us against 21 with the merge launch, 64 rows in 8,192 workgroups 518 us against 104; without the fence (wrong,
// for timing) 21 and 154 us, the counters' atomics costing about 10 ns apiece on top.
//
// Dynamic LDS: waves x nc x (D + 4) floats of outputs and waves x nc x 2 of (max, sum); nc = heads per pass.
constexpr int OPAD = D + 4;       // floats per output row in LDS (the padding spreads the 16 columns over the banks)

template <bool STREAM>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2))) void attn_rows_whole_kernel(RowArgs a) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  const int kvh = blockIdx.x, ri = blockIdx.y;
  const int tid = threadIdx.x, wid = tid / WAVE, lane = tid % WAVE, col = lane & 15, g4 = lane >> 4;
  const int W = a.waves, n_threads = W * WAVE;
  const int row = a.rows ? a.rows[ri] : ri;
  const int pos = a.positions[row];
  const int lo = a.window > 0 ? max(0, pos - a.window + 1) : 0;
  // this wave's keys: the visible ones from the first visible run of 32 on, in W equal shares of whole runs
  const int first = lo / 32 * 32;
  const int chunk = ((pos + 1 - first + W - 1) / W + 31) / 32 * 32;
  const int ka = max(lo, first + wid * chunk), kb = min(pos + 1, first + (wid + 1) * chunk);
  const int ratio = a.nH / a.nKV;
  const int nc_max = min(16, ratio);
  const int* table = a.block_table + (size_t)a.row_req[row] * a.max_blocks;
  float* o_s = lds;                                        // [W][nc_max][OPAD]
  float* ml_s = lds + W * nc_max * OPAD;                   // [W][nc_max][2]
  constexpr int D4 = D / 4;

  for (int qt = 0; qt < ratio; qt += 16) {
    const int nc = min(16, ratio - qt);
    const int head = kvh * ratio + qt + col;
    const bool head_ok = col < nc;
    floatx4 o[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) o[dt] = floatx4{0.f, 0.f, 0.f, 0.f};
    float m = -INFINITY, l = 0.f;
    if (ka < kb) {
      bf16x8 qop[KS];
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const int c = 32 * ks + 8 * g4;
        qop[ks] = (head_ok && c < D) ? *(const bf16x8*)(a.q + ((size_t)row * a.nH + head) * D + c) : zero8();
      }
      RowBlock b0, b1;
      int j0 = (ka / 32) * 32;
      int page_base = 0, pages = -1;
      bool have_pages = false;
      auto table_for = [&](int j) {
        if (have_pages && (j + 31) / a.P - page_base < WAVE) return;
        have_pages = true;
        page_base = j / a.P;
        pages = page_base + lane < a.max_blocks ? table[page_base + lane] : -1;
      };
      table_for(j0);
      load_row_block<STREAM>(b0, a, pages, page_base, kvh, j0, ka, kb, col, g4);
      for (; j0 < kb; j0 += 64) {
        const bool more1 = j0 + 32 < kb, more2 = j0 + 64 < kb;
        if (more1) {
          table_for(j0 + 32);
          load_row_block<STREAM>(b1, a, pages, page_base, kvh, j0 + 32, ka, kb, col, g4);
        }
        use_row_block(b0, a, qop, o, m, l, j0, ka, kb, g4);
        if (more1) {
          if (more2) {
            table_for(j0 + 64);
            load_row_block<STREAM>(b0, a, pages, page_base, kvh, j0 + 64, ka, kb, col, g4);
          }
          use_row_block(b1, a, qop, o, m, l, j0 + 32, ka, kb, g4);
        }
      }
      l = col_sum(l);
    }
    // the waves' results meet in LDS (a wave without visible keys brings weight zero)
    if (qt > 0) __syncthreads();                           // everyone is done with the last pass's LDS
    if (head_ok) {
      float* os = o_s + (wid * nc_max + col) * OPAD;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) *(floatx4*)(os + 16 * dt + 4 * g4) = o[dt];
      if (g4 == 0) { ml_s[(wid * nc_max + col) * 2] = m; ml_s[(wid * nc_max + col) * 2 + 1] = l; }
    }
    __syncthreads();
    for (int i = tid; i < nc * D4; i += n_threads) {
      const int c = i / D4, e = 4 * (i % D4);
      float M = -INFINITY;
      for (int w = 0; w < W; ++w) M = fmaxf(M, ml_s[(w * nc_max + c) * 2]);
      floatx4 acc{0.f, 0.f, 0.f, 0.f};
      float L = 0.f;
      for (int w = 0; w < W; ++w) {
        const float mw = ml_s[(w * nc_max + c) * 2];
        if (mw == -INFINITY) continue;
        const float wgt = fast_exp2(mw - M);
        L = fmaf(wgt, ml_s[(w * nc_max + c) * 2 + 1], L);
        const floatx4 v = *(const floatx4*)(o_s + (w * nc_max + c) * OPAD + e);
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[r] = fmaf(wgt, v[r], acc[r]);
      }
      const float inv = L > 0.f ? 1.f / L : 0.f;
      bf16x4 w4;
#pragma unroll
      for (int r = 0; r < 4; ++r) w4[r] = (__bf16)(acc[r] * inv);
      *(bf16x4*)(a.out + ((size_t)row * a.nH + kvh * ratio + qt + c) * D + e) = w4;
    }
  }
}

// ``waves`` 0: one wave per (row, kv head, split of ``chunk`` keys) and a second launch that merges the splits
// (``max_splits`` * chunk must reach past every row's position; part_o / part_ml are the partial results).
// ``waves`` 1-8: one workgroup of that many waves per (row, kv head), which shares the row's keys evenly and writes
// the output itself; chunk, max_splits and the scratch are not used.
// ``req_is_row``: the caller knows that row_req[r] == r for every row of the step (each request brings one row).
extern "C" int ifx_attn_rows(const void* q, const void* k_cache, const void* v_cache, void* out, const int* rows,
                             const int* row_req, const int* positions, const int* block_table, int max_blocks,
                             int n_rows, int nH, int nKV, int d, int page_size, int window, int chunk,
                             int max_splits, float scale, float* part_o, float* part_ml, int waves, int req_is_row,
                             void* stream) {
  IFX_REQUIRE(d == D, "attn_rows: built for head_dim %d, called with %d", D, d);
  IFX_REQUIRE(n_rows >= 0 && nH > 0 && nKV > 0 && nH % nKV == 0, "attn_rows: bad head counts nH=%d nKV=%d", nH, nKV);
  IFX_REQUIRE(page_size > 0 && page_size % 16 == 0, "attn_rows: page_size %d must be a multiple of 16", page_size);
  IFX_REQUIRE(nKV <= 65535 && n_rows <= 65535, "attn_rows: too many kv heads or rows for one launch");
  IFX_REQUIRE(waves >= 0 && waves <= 8, "attn_rows: %d waves per workgroup (0-8)", waves);
  if (n_rows == 0) return 0;
  RowArgs a{(const bf16_t*)q, (const bf16_t*)k_cache, (const bf16_t*)v_cache, rows, row_req, positions, block_table,
            part_o, part_ml, (bf16_t*)out, max_blocks, n_rows, nH, nKV, page_size, window, chunk, max_splits,
            scale * 1.4426950408889634f, 0, waves, req_is_row};
  hipStream_t s = (hipStream_t)stream;
  const bool streaming = n_rows >= ROW_STREAM_MIN_ROWS && page_size == 16;
  if (waves > 0) {
    const int nc = nH / nKV < 16 ? nH / nKV : 16;
    const size_t lds = (size_t)waves * nc * (OPAD + 2) * sizeof(float);
    IFX_REQUIRE(lds <= 65536, "attn_rows: %d waves of %d heads need %zu bytes of LDS", waves, nc, lds);
    if (streaming)
      hipLaunchKernelGGL(attn_rows_whole_kernel<true>, dim3(nKV, n_rows), dim3(WAVE * waves), lds, s, a);
    else
      hipLaunchKernelGGL(attn_rows_whole_kernel<false>, dim3(nKV, n_rows), dim3(WAVE * waves), lds, s, a);
    IFX_LAUNCH_CHECK();
  }
  IFX_REQUIRE(chunk > 0 && chunk % 32 == 0 && max_splits > 0 && max_splits <= 65535, "attn_rows: bad chunk %d / splits %d", chunk, max_splits);
  IFX_REQUIRE(part_o && part_ml, "attn_rows: splits need scratch for their partial results");
  if (streaming) hipLaunchKernelGGL(attn_rows_kernel<true>, dim3(max_splits, nKV, n_rows), dim3(WAVE), 0, s, a);
  else hipLaunchKernelGGL(attn_rows_kernel<false>, dim3(max_splits, nKV, n_rows), dim3(WAVE), 0, s, a);
  hipLaunchKernelGGL(attn_rows_merge_kernel, dim3(n_rows, nH), dim3(WAVE * merge_waves(max_splits)), 0, s, a);
  IFX_LAUNCH_CHECK();
}

// =======================================================================================
// tiles
// =======================================================================================
#ifndef TILE_QT
#define TILE_QT 2
#endif
constexpr int QT = TILE_QT;       // 16-row query tiles per wave: each K and V operand read from LDS feeds QT products
constexpr int TQ = 64 * QT;       // query rows per workgroup (4 waves)
extern "C" int ifx_attn_tile_rows() { return TQ; }
constexpr int TK = 64;            // keys per staged tile
// Rows in LDS are padded by 16 elements: with the 16-byte reads of the operands (16 rows at a time, one
// per lane) the LDS bank-conflict counter shows half as many conflict cycles as with 8 or 24, and none
// of 32, 40, 48 or 80 does better.
constexpr int KPAD = D + 16;      // bf16 elements per K row in LDS
constexpr int VPAD = TK + 16;     // bf16 elements per V^T row in LDS

struct TileArgs {
  const bf16_t* q;
  const bf16_t* k_cache;
  const bf16_t* v_cache;
  bf16_t* out;
  const int* tile_req;    // [n_tiles] request of each tile
  const int* tile_q0;     // [n_tiles] first row of the tile within its request's rows
  const int* q_start;     // [R] first batch row of each request
  const int* q_len;       // [R]
  const int* kv_len;      // [R] length after this step
  const int* block_table;
  int max_blocks, nH, nKV, P, window;
  float scale_log2e;
  int page_shift;         // log2(P): the tile kernel takes power-of-two pages and splits positions by shift and mask
  int n_tiles, per_xcd;   // work items are (tile, head, split); per_xcd = ceil(n_tiles * nH * max_splits / n_xcd)
  int n_xcd;              // the chip's dies, which a launch deals its workgroups to in turn
  // With max_splits > 1 a workgroup takes only the keys [split * chunk, (split + 1) * chunk) (chunk a multiple of
  // 64) and writes unnormalised partial results in the row kernel's format, at the batch row's number; the
  // row kernel's merge finishes them.  For portions of prompts with a long past: few tiles, many keys.
  int chunk, max_splits;
  float* part_o;          // [T, nH, max_splits, D]
  float* part_ml;         // [T, nH, max_splits, 2]
  // [n_xcd * per_xcd] or nullptr: the work item of each place in the launch (-1: none), place x * per_xcd + i being
  // the i-th workgroup that XCD x is given.  The caller orders the items so that the workgroups that come to
  // share a compute unit have about the same number of key tiles between them on every unit.
  const int* order;
};

constexpr int N_PIECES = TK * (D / 8);                // 16-byte pieces of a K tile, and as many of a V^T tile
constexpr int K_PIECES = (N_PIECES + 255) / 256;      // ... per thread (256 threads)
constexpr int V_PIECES = K_PIECES;

// A thread's share of one K tile and one V^T tile, fetched into registers one tile ahead of the
// arithmetic and stored to LDS when the previous tile has been consumed.
struct TileRegs {
  bf16x8 k[K_PIECES];
  bf16x8 v[V_PIECES];
};

// The pages of a tile's four runs of 16 keys (-1: none), the same for every thread and held in scalar
// registers.  They are looked up one tile before the data is fetched, so that fetching costs one trip
// to memory, not two.
static_assert(TK == 64, "a tile is four runs of 16 keys");
struct TilePages { int p0, p1, p2, p3; };

__device__ __forceinline__ TilePages tile_pages(const TileArgs& a, const int* table, int j0, int pos_last) {
  auto look = [&](int i) {
    const int j = j0 + 16 * i, blk = j >> a.page_shift;
    return __builtin_amdgcn_readfirstlane((j <= pos_last && blk < a.max_blocks) ? table[blk] : -1);
  };
  return TilePages{look(0), look(1), look(2), look(3)};
}

__device__ __forceinline__ int pick_page(const TilePages& pg, int sub) {
  return sub == 0 ? pg.p0 : sub == 1 ? pg.p1 : sub == 2 ? pg.p2 : pg.p3;
}

// Pieces are numbered run by run (a run = 16 keys = one page or part of one): piece c of a tile belongs
// to run c / (2 D); a run's K pieces are (key in run, 8 dims), its V^T pieces (dim, half of the run).
// With 2 D a multiple of 256 (head sizes 128 and 256) a thread's i-th piece lies in a run known at
// compile time, so the run's page and base address stay in scalar registers and a piece costs two or
// three vector instructions of address arithmetic; smaller heads select per lane.
constexpr int RUN_PIECES = 2 * D;
constexpr bool STATIC_RUN = RUN_PIECES % 256 == 0;

struct PieceAt { int run, within; bool live; };
__device__ __forceinline__ PieceAt piece_at(int i, int tid) {
  const int c = tid + 256 * i;
  if (STATIC_RUN) return PieceAt{(256 * i) / RUN_PIECES, tid + (256 * i) % RUN_PIECES, true};
  return PieceAt{c / RUN_PIECES, c % RUN_PIECES, c < N_PIECES};
}

typedef unsigned int uintx4 __attribute__((ext_vector_type(4)));

// A buffer descriptor over ``bytes`` at ``p``: loads through it return zeros beyond its end, so a run
// without a page gets a descriptor of no bytes instead of a branch around its loads.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t run_buffer(const bf16_t* p, int bytes) {
  return __builtin_amdgcn_make_buffer_rsrc((void*)p, 0, bytes, 0x00020000);   // raw 32-bit data format of gfx9
}
__device__ __forceinline__ bf16x8 buffer_load8(__amdgpu_buffer_rsrc_t rs, int byte_offset) {
  const uintx4 v = __builtin_amdgcn_raw_buffer_load_b128(rs, byte_offset, 0, 0);
  return *(const bf16x8*)&v;
}

__device__ __forceinline__ void fetch_tile(TileRegs& r, const TileArgs& a, const TilePages& pg, int kvh, int j0, int tid) {
  const int P = a.P;
  if (STATIC_RUN) {
    // Every piece's run is known here: one descriptor per run for K (the run's 16 rows are contiguous) and
    // one for V^T (D rows of P, of which the run takes 16 keys), built from scalars; a piece is one load
    // at an offset that depends on the thread alone.
#pragma unroll
    for (int i = 0; i < K_PIECES; ++i) {
      const PieceAt at = piece_at(i, tid);
      const int page = pick_page(pg, at.run), pos0 = (j0 + 16 * at.run) & (P - 1);
      const bf16_t* base = a.k_cache + (((size_t)max(page, 0) * a.nKV + kvh) * P + pos0) * D;
      r.k[i] = buffer_load8(run_buffer(base, page >= 0 ? 16 * D * 2 : 0), at.within * 16);
    }
#pragma unroll
    for (int i = 0; i < V_PIECES; ++i) {
      const PieceAt at = piece_at(i, tid);
      const int page = pick_page(pg, at.run), pos0 = (j0 + 16 * at.run) & (P - 1);
      const bf16_t* base = a.v_cache + ((size_t)max(page, 0) * a.nKV + kvh) * D * P + pos0;
      r.v[i] = buffer_load8(run_buffer(base, page >= 0 ? ((D - 1) * P + 16) * 2 : 0), ((at.within / 2) * P + 8 * (at.within % 2)) * 2);
    }
    return;
  }
#pragma unroll
  for (int i = 0; i < K_PIECES; ++i) {
    const PieceAt at = piece_at(i, tid);
    const int key = at.within / (D / 8), c8 = at.within % (D / 8);
    const int page = at.live ? pick_page(pg, at.run) : -1;
    const bf16_t* base = a.k_cache + ((size_t)max(page, 0) * a.nKV + kvh) * P * D;
    r.k[i] = page >= 0 ? *(const bf16x8*)(base + ((j0 + 16 * at.run + key) & (P - 1)) * D + 8 * c8) : zero8();
  }
#pragma unroll
  for (int i = 0; i < V_PIECES; ++i) {
    const PieceAt at = piece_at(i, tid);
    const int dim = at.within / 2, half = at.within % 2;   // 8 keys never straddle a page
    const int page = at.live ? pick_page(pg, at.run) : -1;
    const bf16_t* base = a.v_cache + ((size_t)max(page, 0) * a.nKV + kvh) * D * P;
    r.v[i] = page >= 0 ? *(const bf16x8*)(base + dim * P + ((j0 + 16 * at.run + 8 * half) & (P - 1))) : zero8();
  }
}

__device__ __forceinline__ void stage_tile(const TileRegs& r, bf16_t* k_s, bf16_t* v_s, int tid) {
#pragma unroll
  for (int i = 0; i < K_PIECES; ++i) {
    const PieceAt at = piece_at(i, tid);
    if (at.live) *(bf16x8*)(k_s + (16 * at.run + at.within / (D / 8)) * KPAD + 8 * (at.within % (D / 8))) = r.k[i];
  }
#pragma unroll
  for (int i = 0; i < V_PIECES; ++i) {
    const PieceAt at = piece_at(i, tid);
    if (at.live) {
      // Keys are stored in the order the second product consumes them: within each run of 32 keys,
      // position 8 g + 4 h + r holds key 16 h + 4 g + r, so that one 16-byte read gives a lane its
      // four keys of both 16-key score tiles.  A piece of 8 consecutive keys (half a run of 16: keys
      // 16 run + 8 half ...) lands as two halves.
      const int dim = at.within / 2, half = at.within % 2;
      bf16_t* dst = v_s + dim * VPAD + 32 * (at.run / 2) + 16 * half + 4 * (at.run % 2);
      bf16x4 lo, hi;
#pragma unroll
      for (int e = 0; e < 4; ++e) { lo[e] = r.v[i][e]; hi[e] = r.v[i][e + 4]; }
      *(bf16x4*)dst = lo;
      *(bf16x4*)(dst + 8) = hi;
    }
  }
}

// One staged tile of 64 keys against a wave's QT tiles of 16 query rows: scores, running softmax,
// output.  Scores stay unscaled; the scale (with log2 e) enters the exponent through one fused
// multiply-add.  MASKED adds the causal / window / row-validity test per score.
struct QueryTile {
  bf16x8 qop[KS];
  floatx4 o[DT];
  float m, l;
  int pos, lo;     // this lane's query: its position and the first position it sees
  bool ok;
};

template <bool MASKED>
__device__ __forceinline__ void tile_math(const bf16_t* k_s, const bf16_t* v_s, QueryTile* q, float c_log2e, int j0, int col,
                                          int g4) {
  floatx4 s[QT][4];
#pragma unroll
  for (int t = 0; t < 4; ++t) {
#pragma unroll
    for (int qt = 0; qt < QT; ++qt) s[qt][t] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int c = 32 * ks + 8 * g4;
      const bf16x8 kop = c < D ? *(const bf16x8*)(k_s + (16 * t + col) * KPAD + c) : zero8();
#pragma unroll
      for (int qt = 0; qt < QT; ++qt) s[qt][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kop, q[qt].qop[ks], s[qt][t], 0, 0, 0);
    }
  }
  bf16x8 pop[QT][2];
  float alpha[QT];
  bool rescale = false;
#pragma unroll
  for (int qt = 0; qt < QT; ++qt) {
    float mb = -INFINITY;
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        if (MASKED) {
          const int key = j0 + 16 * t + 4 * g4 + r;
          const bool vis = q[qt].ok && key <= q[qt].pos && key >= q[qt].lo;
          s[qt][t][r] = vis ? s[qt][t][r] : -INFINITY;
        }
        mb = fmaxf(mb, s[qt][t][r]);
      }
    const float m_new = fmaxf(q[qt].m, col_max(mb));
    const float m_safe = m_new == -INFINITY ? 0.f : m_new;
    alpha[qt] = fast_exp2((q[qt].m - m_safe) * c_log2e);
    const float ms = m_safe * c_log2e;
    float psum = 0.f;
    bf16x4 pb[4];
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float p = fast_exp2(fmaf(s[qt][t][r], c_log2e, -ms));
        psum += p;
        pb[t][r] = (__bf16)p;
      }
    q[qt].l = q[qt].l * alpha[qt] + psum;
    q[qt].m = m_new;
    pop[qt][0] = join4(pb[0], pb[1]);
    pop[qt][1] = join4(pb[2], pb[3]);
    rescale = rescale || __any(alpha[qt] != 1.0f);   // once the running maxima have settled nothing is rescaled
  }
  if (rescale) {
    // The empty statement keeps this a branch the whole wave takes or skips: as straight-line code
    // (multiply and select per element) it would be nearly half of the tile's vector instructions.
    asm volatile("");
#pragma unroll
    for (int qt = 0; qt < QT; ++qt)
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r = 0; r < 4; ++r) q[qt].o[dt][r] *= alpha[qt];
  }
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) {
    const bf16_t* vr = v_s + (16 * dt + col) * VPAD + 8 * g4;
    const bf16x8 vop0 = *(const bf16x8*)(vr), vop1 = *(const bf16x8*)(vr + 32);
#pragma unroll
    for (int qt = 0; qt < QT; ++qt) {
      q[qt].o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vop0, pop[qt][0], q[qt].o[dt], 0, 0, 0);
      q[qt].o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vop1, pop[qt][1], q[qt].o[dt], 0, 0, 0);
    }
  }
}

// The kernel waits on LDS and on the matrix pipe, so waves to switch to are worth more than the
// registers they cost: 3 waves per SIMD with one query tile per wave (162 registers, no spill), 2 with two.
#ifndef TILE_WAVES_PER_SIMD
#if TILE_QT == 1
#define TILE_WAVES_PER_SIMD 3
#else
#define TILE_WAVES_PER_SIMD 2
#endif
#endif
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(TILE_WAVES_PER_SIMD, TILE_WAVES_PER_SIMD)))
void attn_tiles_kernel(TileArgs a) {
  __shared__ __attribute__((aligned(16))) bf16_t k_s[TK * KPAD];
  __shared__ __attribute__((aligned(16))) bf16_t v_s[D * VPAD];
  const int tid = threadIdx.x, wid = tid / WAVE, lane = tid % WAVE, col = lane & 15, g4 = lane >> 4;
  // Workgroups go to the 8 XCDs round-robin by their number, and every XCD has an L2 of its own.
  // Work items are ordered kv head first and dealt to the XCDs in contiguous runs, so that the
  // workgroups that read one kv head's keys and values share an L2 instead of filling all eight with
  // everything; within a run the tiles with the most keys (the latest rows) come first.
  const int ratio = a.nH / a.nKV;
  const int place = (blockIdx.x % a.n_xcd) * a.per_xcd + blockIdx.x / a.n_xcd;
  if (blockIdx.x / a.n_xcd >= a.per_xcd) return;                                              // the whole workgroup leaves together
  const int work = a.order ? a.order[place] : place;
  if (work < 0 || work >= a.n_tiles * a.nH * a.max_splits) return;
  const int item = work / a.max_splits, split = work % a.max_splits;
  const int per_kv = ratio * a.n_tiles;
  const int kvh = item / per_kv, rem = item % per_kv;
  const int head = kvh * ratio + rem / a.n_tiles, ti = a.n_tiles - 1 - rem % a.n_tiles;
  const int req = a.tile_req[ti], q0 = a.tile_q0[ti];
  const int qlen = a.q_len[req], kvlen = a.kv_len[req];
  const int start = kvlen - qlen;                       // position of the request's first row in this step
  const int* table = a.block_table + (size_t)req * a.max_blocks;
  const int rows_here = min(TQ, qlen - q0);
  const int pos_first = start + q0, row_last = pos_first + rows_here - 1;
  // the keys of this workgroup: what its rows can see, cut to its split
  const int lo_wg = max(a.window > 0 ? max(0, pos_first - a.window + 1) : 0, a.max_splits > 1 ? split * a.chunk : 0);
  const int pos_last = a.max_splits > 1 ? min(row_last, (split + 1) * a.chunk - 1) : row_last;

  // this wave's rows: QT tiles of 16, lane `col` of tile qt holds row 16 * QT * wid + 16 * qt + col of the tile
  const int wave_q = q0 + 16 * QT * wid;
  const size_t row0 = (size_t)a.q_start[req];
  QueryTile q[QT];
#pragma unroll
  for (int qt = 0; qt < QT; ++qt) {
    const int my_q = wave_q + 16 * qt + col;
    q[qt].ok = my_q < qlen;
    q[qt].pos = start + my_q;
    q[qt].lo = a.window > 0 ? max(0, q[qt].pos - a.window + 1) : 0;
    q[qt].m = -INFINITY;
    q[qt].l = 0.f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int c = 32 * ks + 8 * g4;
      q[qt].qop[ks] = (q[qt].ok && c < D) ? *(const bf16x8*)(a.q + ((row0 + my_q) * a.nH + head) * D + c) : zero8();
    }
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) q[qt].o[dt] = floatx4{0.f, 0.f, 0.f, 0.f};
  }
  // the keys this wave's rows can see at all: tiles outside are skipped by the whole wave
  const int wave_first = start + wave_q;
  const int wave_hi = min(row_last, wave_first + 16 * QT - 1);
  const int wave_lo = a.window > 0 ? max(0, wave_first - a.window + 1) : 0;

  TileRegs regs;
  int j0 = (lo_wg / TK) * TK;
  TilePages pg = tile_pages(a, table, j0, pos_last);
  fetch_tile(regs, a, pg, kvh, j0, tid);
  pg = tile_pages(a, table, j0 + TK, pos_last);
  for (; j0 <= pos_last; j0 += TK) {
    __syncthreads();  // everyone is done with the previous tile
    stage_tile(regs, k_s, v_s, tid);
    __syncthreads();
    if (j0 + TK <= pos_last) {  // the next tile's data and the one after's pages: in flight during the arithmetic
      fetch_tile(regs, a, pg, kvh, j0 + TK, tid);
      pg = tile_pages(a, table, j0 + 2 * TK, pos_last);
    }
    if (j0 > wave_hi || j0 + TK <= wave_lo) continue;   // uniform over the wave; barriers are at the loop's top

    // A tile every key of which every row of this wave sees needs no mask: the common case.
    const bool full = j0 + TK - 1 <= wave_first && (a.window <= 0 || j0 >= wave_hi - a.window + 1);
    if (full) tile_math<false>(k_s, v_s, q, a.scale_log2e, j0, col, g4);
    else tile_math<true>(k_s, v_s, q, a.scale_log2e, j0, col, g4);
  }
#pragma unroll
  for (int qt = 0; qt < QT; ++qt) {
    const float l = col_sum(q[qt].l);
    if (!q[qt].ok) continue;
    const size_t row = row0 + wave_q + 16 * qt + col;
    if (a.max_splits > 1) {
      float* po = a.part_o + ((row * a.nH + head) * a.max_splits + split) * D;
      float* pml = a.part_ml + ((row * a.nH + head) * a.max_splits + split) * 2;
      if (g4 == 0) { pml[0] = q[qt].m * a.scale_log2e; pml[1] = l; }   // -inf stays -inf: nothing of this split was visible
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) *(floatx4*)(po + 16 * dt + 4 * g4) = q[qt].o[dt];
    } else {
      const float inv = l > 0.f ? 1.f / l : 0.f;
      bf16_t* orow = a.out + (row * a.nH + head) * D;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        bf16x4 w;
#pragma unroll
        for (int r = 0; r < 4; ++r) w[r] = (__bf16)(q[qt].o[dt][r] * inv);
        *(bf16x4*)(orow + 16 * dt + 4 * g4) = w;
      }
    }
  }
}

// chunk / max_splits / part_o / part_ml / rows / n_rows / positions: with max_splits > 1 the keys are cut into
// splits of ``chunk`` (a multiple of 64; max_splits * chunk reaches past the largest position), the partial
// results go to part_o [T, nH, max_splits, D] and part_ml [T, nH, max_splits, 2], and the rows named by ``rows``
// (every row of every tiled request, n_rows of them) are merged into ``out`` at the end.
extern "C" int ifx_attn_tiles(const void* q, const void* k_cache, const void* v_cache, void* out,
                              const int* tile_req, const int* tile_q0, int n_tiles, const int* q_start,
                              const int* q_len, const int* kv_len, const int* block_table, int max_blocks,
                              int nH, int nKV, int d, int page_size, int window, float scale, int chunk, int max_splits,
                              float* part_o, float* part_ml, const int* rows, int n_rows, const int* row_req,
                              const int* positions, const int* order, int order_per_xcd, int n_xcd, void* stream) {
  IFX_REQUIRE(d == D, "attn_tiles: built for head_dim %d, called with %d", D, d);
  IFX_REQUIRE(n_tiles >= 0 && nH > 0 && nKV > 0 && nH % nKV == 0, "attn_tiles: bad head counts nH=%d nKV=%d", nH, nKV);
  IFX_REQUIRE(page_size > 0 && page_size % 16 == 0, "attn_tiles: page_size %d must be a multiple of 16", page_size);
  IFX_REQUIRE(nH <= 65535, "attn_tiles: too many heads for one launch");
  IFX_REQUIRE((page_size & (page_size - 1)) == 0, "attn_tiles: page_size %d must be a power of two", page_size);
  IFX_REQUIRE(max_splits >= 1 && max_splits <= 65535, "attn_tiles: bad number of splits %d", max_splits);
  IFX_REQUIRE(max_splits == 1 || (chunk > 0 && chunk % TK == 0 && part_o && part_ml && rows && positions && row_req && n_rows > 0),
              "attn_tiles: %d splits need a chunk that is a multiple of %d (got %d), scratch, and the rows to merge", max_splits,
              TK, chunk);
  int page_shift = 0;
  while ((1 << page_shift) < page_size) ++page_shift;
  if (n_tiles == 0) return 0;
  TileArgs a{(const bf16_t*)q, (const bf16_t*)k_cache, (const bf16_t*)v_cache, (bf16_t*)out, tile_req, tile_q0, q_start,
             q_len, kv_len, block_table, max_blocks, nH, nKV, page_size, window, scale * 1.4426950408889634f, page_shift,
             n_tiles, 0, n_xcd, chunk, max_splits, part_o, part_ml, order};
  const long long items = (long long)n_tiles * nH * max_splits;
  IFX_REQUIRE(items <= (1LL << 30), "attn_tiles: too many tiles for one launch");
  IFX_REQUIRE(!order || (order_per_xcd > 0 && (long long)n_xcd * order_per_xcd >= items && order_per_xcd <= items),
              "attn_tiles: an order of %d x %d places cannot hold %lld work items", n_xcd, order_per_xcd, items);
  IFX_REQUIRE(n_xcd >= 1 && n_xcd <= 64, "%s: %d dies", "attn_tiles", n_xcd);
  a.n_xcd = n_xcd;
  a.per_xcd = order ? order_per_xcd : (int)((items + n_xcd - 1) / n_xcd);
  hipStream_t s = (hipStream_t)stream;
  hipLaunchKernelGGL(attn_tiles_kernel, dim3(n_xcd * a.per_xcd), dim3(256), 0, s, a);
  if (max_splits > 1) {
    RowArgs m{(const bf16_t*)q, (const bf16_t*)k_cache, (const bf16_t*)v_cache, rows, row_req, positions, block_table,
              part_o, part_ml, (bf16_t*)out, max_blocks, n_rows, nH, nKV, page_size, window, chunk, max_splits,
              scale * 1.4426950408889634f, 1};
    hipLaunchKernelGGL(attn_rows_merge_kernel, dim3(n_rows, nH), dim3(WAVE * merge_waves(max_splits)), 0, s, m);
  }
  IFX_LAUNCH_CHECK();
}
