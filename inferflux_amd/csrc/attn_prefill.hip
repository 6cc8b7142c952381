// Attention of prompt portions over the paged cache on the matrix cores, head size 128: the tile kernel of
// attn_mfma.hip rebuilt around what limited it.  There, a tile of 64 keys goes global memory -> registers -> LDS
// between two barriers, which costs every thread 32 registers, eight LDS stores and their addresses per tile, and
// a workgroup of four waves with its own copy of every tile.  Here:
//
//   * tiles go from global memory straight into LDS (buffer_load ... lds: the data never passes through
//     registers), one tile ahead of the arithmetic, into one of two LDS stages;
//   * one barrier per tile: "my loads of this tile have landed" and "I am done with the last tile" in one;
//   * eight waves of 16 query rows share a stage, so a tile is fetched once for 128 rows, and without the
//     staging registers a wave fits in 107 registers: four waves per SIMD (two workgroups per compute unit)
//     instead of two or three, which is what hides the waits between a tile's products and its softmax;
//   * rows in LDS are not padded (the direct loads write 1 KB runs in lane order); bank conflicts are avoided by
//     which 16-byte piece a lane fetches: piece p of K row r lies at slot p ^ g(r), of V^T in 16-key sub-tiles
//     with the two halves of a row swapped for every other group of 8 rows.
//
// Measured (28 query heads on 4 kv heads, causal, workgroups in attention.tile_order): 55 / 142 / 495 us at 2,048 /
// 4,096 / 8,192 rows against the other kernel's 75 / 178 / 606.  A version with three stages (one workgroup per
// compute unit) that also overlapped the scores of one tile with the softmax of the one before inside a wave took
// 66 / 201 / 700: the second workgroup on the unit is worth more than the deeper pipeline.
//
// The function computed is attn_mfma.hip's tile kernel's (causal, optionally windowed, grouped-query attention;
// reference formula runtime/backends/cuda/kernels/flash_attention.cu:71-72, 86, 144, 152-173), with the same
// transposed products S^T = K Q^T and O^T += V^T P^T, the same softmax in float and the same split format.
//
// Key order inside a tile.  The second product's B operand holds, per lane, 8 k-values: the lane's four scores
// of two 16-key score tiles.  Which key a score tile's row j stands for is free (it is the K row a lane reads
// for the first product), so rows are dealt such that a lane's 8 scores are 8 consecutive keys:
// row j of score tile t is key 32 (t / 2) + 8 (j / 4) + 4 (t % 2) + j % 4 of the 64.  V^T is then read in
// plain 16-byte pieces of 8 consecutive keys, as the cache holds them.
#include "common.h"

IFX_DEFINE_LAST_ERROR()

#ifndef HEAD_DIM
#define HEAD_DIM 128
#endif
static_assert(HEAD_DIM == 128, "the direct-to-LDS tile kernel is written for head size 128");

#include "attn_shared.h"

#ifndef TILE_QT
#define TILE_QT 1
#endif
#ifndef TILE_WAVES
#define TILE_WAVES 8
#endif
constexpr int QT = TILE_QT;            // 16-row query tiles per wave
constexpr int NW = TILE_WAVES;         // waves per workgroup
constexpr int NS = 2;                  // LDS stages: a tile is asked for one tile before it is used
constexpr int TQ = 16 * QT * NW;       // query rows per workgroup
constexpr int TK = 64;                 // keys per stage
constexpr int K_BYTES = TK * D * 2;    // a stage's K tile: 64 rows of 256 bytes
constexpr int V_BYTES = D * TK * 2;    // a stage's V^T tile: four sub-tiles (16 keys each) of 128 rows of 32 bytes
constexpr int STAGE_BYTES = K_BYTES + V_BYTES;
constexpr int CHUNKS = K_BYTES / 1024; // 1 KB runs (one direct load of a wave) per operand and stage: 16
static_assert(CHUNKS % NW == 0 && CHUNKS == 16 && V_BYTES == K_BYTES, "a stage is 16 + 16 runs of 1 KB dealt to the waves");
constexpr int CH = CHUNKS / NW;        // runs per wave, operand and stage
static_assert(CH == 1 || CH == 2 || CH == 4, "4, 8 or 16 waves");

extern "C" int ifx_attn_prefill_tile_rows() { return TQ; }
extern "C" int ifx_attn_prefill_lds_bytes() { return NS * STAGE_BYTES; }

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
  int page_shift;         // log2(P)
  int n_tiles, per_xcd;   // work items are (tile, head, split); per_xcd = ceil(n_tiles * nH * max_splits / n_xcd)
  int n_xcd;              // the chip's dies, which a launch deals its workgroups to in turn
  int chunk, max_splits;  // as in attn_mfma.hip's tile kernel: keys [split * chunk, (split + 1) * chunk) per workgroup
  float* part_o;          // [T, nH, max_splits, D]
  float* part_ml;         // [T, nH, max_splits, 2]
  const int* order;       // as in attn_mfma.hip's tile kernel
};

typedef unsigned int uintx4 __attribute__((ext_vector_type(4)));

// One direct load: lane l's 16 bytes at ``base + voffset[l]`` go to LDS address ``lds_addr + 16 l``; lanes whose
// offset lies at or beyond ``bytes`` deliver zeros.  Written in assembly so that the compiler does not know that
// LDS is written: it would otherwise wait for every such load before the next LDS read (it cannot tell the
// stages apart), which is the wait this kernel exists to avoid.  The ordering that matters is kept by hand: see
// the loop in the kernel.
__device__ __forceinline__ void direct_load(unsigned long long base, int bytes, int voffset, unsigned lds_addr) {
  uintx4 rsrc;
  rsrc[0] = (unsigned)base;
  rsrc[1] = (unsigned)(base >> 32) & 0xffffu;
  rsrc[2] = (unsigned)bytes;
  rsrc[3] = 0x00020000u;                       // raw 32-bit data format of gfx9
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
               :
               : "s"(lds_addr), "v"(voffset), "s"(rsrc)
               : "memory", "m0");
}

// Wait until at most N of this wave's vector memory loads are still in flight and none of its LDS reads is, then
// meet the other waves.  The barrier says two things at once: "my loads of this tile have landed" (vmcnt) and "I
// have read everything I will of the tile before" (lgkmcnt: right behind the barrier other waves start loads into
// that tile's stage, so every LDS read of it must have returned, not merely have been issued; a tile's operands have
// all been consumed by matrix instructions by then, so this wait costs nothing).
template <int N>
__device__ __forceinline__ void wait_loads_and_barrier() {
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
  asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" : : "n"(N) : "memory");
}

struct QueryTile {
  bf16x8 qop[KS];
  floatx4 o[DT];
  float m, l;
  int pos, lo;     // this lane's query: its position and the first position it sees
  bool ok;
};
struct Scores { floatx4 s[QT][4]; };     // S^T of one tile of 64 keys: four score tiles of 16 keys per query tile
struct Weights { bf16x8 p[QT][2]; };     // P^T of one tile as the second product's operands: two blocks of 32 keys

// S^T = K Q^T of one staged tile.  ``k_rd[ks]``: this lane's byte offset into the K tile for score tile 0, k-step ks.
__device__ __forceinline__ void scores_of(const unsigned char* k_tile, const int* k_rd, const QueryTile* q, Scores& S) {
  // k-step outermost: the four score tiles are four chains of products that do not wait for each other
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      // rows of score tile t: 32 (t / 2) + 4 (t % 2) + (this lane's row of tile 0)
      const bf16x8 kop = *(const bf16x8*)(k_tile + k_rd[ks] + (32 * (t / 2) + 4 * (t % 2)) * D * 2);
#pragma unroll
      for (int qt = 0; qt < QT; ++qt)
        S.s[qt][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kop, q[qt].qop[ks], ks == 0 ? floatx4{0.f, 0.f, 0.f, 0.f} : S.s[qt][t], 0, 0, 0);
    }
  }
}

// Running softmax over one tile's scores: new maxima and sums, the weights as bf16 operands, and the factor the
// output so far has to be multiplied by (``alpha``; ``rescale``: whether any lane's differs from 1).  Scores stay
// unscaled; the scale (with log2 e) enters the exponent through one fused multiply-add.  MASKED adds the causal /
// window / row-validity test per score.
template <bool MASKED>
__device__ __forceinline__ void weights_of(Scores& S, QueryTile* q, float c_log2e, int j0, int g4, Weights& W, float* alpha,
                                           bool& rescale) {
  rescale = false;
#pragma unroll
  for (int qt = 0; qt < QT; ++qt) {
    float mb = -INFINITY;
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        if (MASKED) {
          const int key = j0 + 32 * (t / 2) + 8 * g4 + 4 * (t % 2) + r;
          const bool vis = q[qt].ok && key <= q[qt].pos && key >= q[qt].lo;
          S.s[qt][t][r] = vis ? S.s[qt][t][r] : -INFINITY;
        }
        mb = fmaxf(mb, S.s[qt][t][r]);
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
        const float p = fast_exp2(fmaf(S.s[qt][t][r], c_log2e, -ms));
        psum += p;
        pb[t][r] = (__bf16)p;
      }
    q[qt].l = q[qt].l * alpha[qt] + psum;
    q[qt].m = m_new;
    W.p[qt][0] = join4(pb[0], pb[1]);     // keys 8 g4 .. 8 g4 + 7 of the tile's first 32
    W.p[qt][1] = join4(pb[2], pb[3]);     // ... of its second 32
    rescale = rescale || __any(alpha[qt] != 1.0f);   // once the running maxima have settled nothing is rescaled
  }
}

// O^T += V^T P^T of one staged tile.  ``v_rd``: this lane's byte offset into the V^T tile for output tile 0, key block 0.
__device__ __forceinline__ void add_values(const unsigned char* v_tile, int v_rd, QueryTile* q, const Weights& W) {
  // key block outermost: the eight output tiles are eight chains of products that do not wait for each other
#pragma unroll
  for (int blk = 0; blk < 2; ++blk) {
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      // output tile dt: dims 16 dt + col: 16 rows of 32 bytes further in every sub-tile; key block 1: two sub-tiles on
      const bf16x8 vop = *(const bf16x8*)(v_tile + v_rd + dt * 16 * 32 + blk * 2 * 4096);
#pragma unroll
      for (int qt = 0; qt < QT; ++qt)
        q[qt].o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vop, W.p[qt][blk], q[qt].o[dt], 0, 0, 0);
    }
  }
}

// registers: 107 with one query tile per wave, about 200 with two
#ifndef TILE_WAVES_PER_SIMD
#if TILE_QT == 1
#define TILE_WAVES_PER_SIMD 4
#else
#define TILE_WAVES_PER_SIMD 2
#endif
#endif
__global__ __launch_bounds__(64 * NW) __attribute__((amdgpu_waves_per_eu(TILE_WAVES_PER_SIMD, TILE_WAVES_PER_SIMD)))
void attn_prefill_kernel(TileArgs a) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];
  const int tid = threadIdx.x, wid = __builtin_amdgcn_readfirstlane(tid / WAVE), lane = tid % WAVE, col = lane & 15, g4 = lane >> 4;
  // Work items as in attn_mfma.hip's tile kernel: kv head first, dealt to the 8 XCDs in contiguous runs (an L2
  // then holds a few kv heads' keys and values, not all of them), tiles with the most keys first within a run.
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
  // The table is read through the constant address space, which makes the reads scalar loads: they must not count
  // among the vector memory operations, whose number in flight the pipeline below waits on.
  const __attribute__((address_space(4))) int* table =
      (const __attribute__((address_space(4))) int*)(a.block_table + (size_t)req * a.max_blocks);
  const int rows_here = min(TQ, qlen - q0);
  const int pos_first = start + q0, row_last = pos_first + rows_here - 1;
  // the keys of this workgroup: what its rows can see, cut to its split
  const int lo_wg = max(a.window > 0 ? max(0, pos_first - a.window + 1) : 0, a.max_splits > 1 ? split * a.chunk : 0);
  const int pos_last = a.max_splits > 1 ? min(row_last, (split + 1) * a.chunk - 1) : row_last;
  const int P = a.P;

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
    for (int ks = 0; ks < KS; ++ks)
      q[qt].qop[ks] = q[qt].ok ? *(const bf16x8*)(a.q + ((row0 + my_q) * a.nH + head) * D + 32 * ks + 8 * g4) : zero8();
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) q[qt].o[dt] = floatx4{0.f, 0.f, 0.f, 0.f};
  }
  const int wave_first = start + wave_q;
  const int wave_hi = min(row_last, wave_first + 16 * QT - 1);
  const int wave_lo = a.window > 0 ? max(0, wave_first - a.window + 1) : 0;

  // What this wave fetches of every tile: runs c = CH wid + i (i < CH) of 1 KB of K and of V^T, which all lie in
  // one run of 16 keys of the tile (``my_run``), so one page number serves them all.  K: rows 4 c .. 4 c + 3 of the
  // tile, 16 slots of 16 bytes each; lane l -> row 4 c + l / 16, slot l % 16, which holds piece slot ^ g(row).
  // V^T: sub-tile c / 4, dims 32 (c % 4) + l / 2; half l % 2 of the row's 32 bytes holds the row's half (l % 2) ^ (dim / 8 % 2).
  static_assert(CH <= 4, "a wave's runs lie in one run of 16 keys");
  const int my_run = (CH * wid) / 4;
  int k_off[CH], v_off[CH];
#pragma unroll
  for (int i = 0; i < CH; ++i) {
    const int c = CH * wid + i;
    const int row = 4 * c + lane / 16;
    const int g = (row & 3) | (((row >> 3) & 3) << 2);
    k_off[i] = (row % 16) * D * 2 + (((lane % 16) ^ g) * 16);           // within the run's 16 rows of the cache page
    const int dim = 32 * (c % 4) + lane / 2;
    v_off[i] = dim * P * 2 + (((lane % 2) ^ ((dim >> 3) & 1)) * 16);    // within the page's [D][P]
  }
  // What this lane reads of a staged tile: K row 8 (col / 4) + col % 4 of score tile 0 (slot = piece ^ g(row) = piece ^ col),
  // V^T row col of output tile 0 (sub-tile g4 / 2 of key block 0, half (g4 % 2) ^ (col / 8)).
  int k_rd[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) k_rd[ks] = (8 * (col / 4) + col % 4) * D * 2 + (((4 * ks + g4) ^ col) * 16);
  const int v_rd = (g4 / 2) * 4096 + col * 32 + (((g4 % 2) ^ (col >> 3)) * 16);

  const int j_first = (lo_wg / TK) * TK;
  const int n_tiles_k = pos_last >= j_first ? (pos_last - j_first) / TK + 1 : 0;      // key tiles of this workgroup
  // The page of this wave's run of key tile t (-1: none, also for tiles before the first and after the last).
  auto page_of = [&](int t) {
    const int j = j_first + TK * t + 16 * my_run, blk = j >> a.page_shift;
    return (t >= 0 && j <= pos_last && blk < a.max_blocks) ? table[blk] : -1;
  };
  const unsigned lds_base = (unsigned)(size_t)(__attribute__((address_space(3))) unsigned char*)lds;
  const unsigned long long k_head = (unsigned long long)(a.k_cache + (size_t)kvh * P * D);
  const unsigned long long v_head = (unsigned long long)(a.v_cache + (size_t)kvh * D * P);
  const unsigned long long page_bytes = (unsigned long long)a.nKV * P * D * 2;
  // where this wave's run of key tile t starts inside its page (tiles start at multiples of 64 keys: with pages of
  // up to 64 tokens that is the same for every tile, with larger pages it is not)
  auto run_at_of = [&](int t) { return (j_first + TK * t + 16 * my_run) & (P - 1); };
  // Ask for this wave's part of key tile t (its run's page ``kpage`` = ``vpage``) into K slot ``k_slot`` and V slot ``v_slot``.
  auto issue = [&](int t, int k_slot, int kpage, int v_slot, int vpage) {
    const int run_at = run_at_of(t);
    const unsigned long long kb = k_head + (unsigned long long)max(kpage, 0) * page_bytes + (unsigned)(run_at * D * 2);
    const unsigned long long vb = v_head + (unsigned long long)max(vpage, 0) * page_bytes + (unsigned)(run_at * 2);
    const int kbytes = kpage >= 0 ? 16 * D * 2 : 0, vbytes = vpage >= 0 ? ((D - 1) * P + 16) * 2 : 0;
#pragma unroll
    for (int i = 0; i < CH; ++i) {
      const int c = CH * wid + i;
      direct_load(kb, kbytes, k_off[i], lds_base + k_slot * K_BYTES + c * 1024);
      direct_load(vb, vbytes, v_off[i], lds_base + NS * K_BYTES + v_slot * V_BYTES + c * 1024);
    }
  };

  // Every load the compiler knows of (the queries) is waited for here, once: it cannot see the direct loads, and
  // left to itself it waits for "everything in flight" at the queries' first use inside the loop, every iteration.
  __builtin_amdgcn_s_waitcnt(0);

  // Step s waits for this wave's loads of tile s (everything it has in flight), meets the other waves (tile s is
  // whole, and everyone is done with tile s - 1), asks for tile s + 1 into the stage that tile s - 1 has left, and
  // computes tile s while those loads are on their way.  Loads are asked for in every step, also for tiles that do
  // not exist (no page: they deliver zeros).  The other workgroup on the compute unit fills the waits.
  issue(0, 0, page_of(0), 0, page_of(0));
  int next_page = page_of(1);
  for (int s = 0; s < n_tiles_k; ++s) {
    wait_loads_and_barrier<0>();
    const int slot = s & 1;
    issue(s + 1, slot ^ 1, next_page, slot ^ 1, next_page);
    next_page = page_of(s + 2);
    const int j0 = j_first + TK * s;
    if (wave_q >= qlen || j0 > wave_hi || j0 + TK <= wave_lo) continue;   // (a wave without rows only fetches) uniform over the wave; the barrier is at the loop's top
    const unsigned char* k_tile = lds + slot * K_BYTES;
    const unsigned char* v_tile = lds + NS * K_BYTES + slot * V_BYTES;
    // A tile every key of which every row of this wave sees needs no mask: the common case.
    const bool full = j0 + TK - 1 <= wave_first && (a.window <= 0 || j0 >= wave_hi - a.window + 1);
    Scores S;
    Weights W;
    float alpha[QT];
    bool rescale = false;
    scores_of(k_tile, k_rd, q, S);
    if (full) weights_of<false>(S, q, a.scale_log2e, j0, g4, W, alpha, rescale);
    else weights_of<true>(S, q, a.scale_log2e, j0, g4, W, alpha, rescale);
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
    add_values(v_tile, v_rd, q, W);
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");     // no load may still be writing LDS when the workgroup gives it back
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

// Arguments as ifx_attn_tiles of attn_mfma.hip (tiles of ifx_attn_prefill_tile_rows() rows here).
extern "C" int ifx_attn_prefill(const void* q, const void* k_cache, const void* v_cache, void* out,
                                const int* tile_req, const int* tile_q0, int n_tiles, const int* q_start,
                                const int* q_len, const int* kv_len, const int* block_table, int max_blocks,
                                int nH, int nKV, int d, int page_size, int window, float scale, int chunk, int max_splits,
                                float* part_o, float* part_ml, const int* rows, int n_rows, const int* row_req,
                                const int* positions, const int* order, int order_per_xcd, int n_xcd, void* stream) {
  IFX_REQUIRE(d == D, "attn_prefill: built for head_dim %d, called with %d", D, d);
  IFX_REQUIRE(n_tiles >= 0 && nH > 0 && nKV > 0 && nH % nKV == 0, "attn_prefill: bad head counts nH=%d nKV=%d", nH, nKV);
  IFX_REQUIRE(page_size >= 16 && (page_size & (page_size - 1)) == 0, "attn_prefill: page_size %d must be a power of two from 16", page_size);
  IFX_REQUIRE(nH <= 65535, "attn_prefill: too many heads for one launch");
  IFX_REQUIRE(max_splits >= 1 && max_splits <= 65535, "attn_prefill: bad number of splits %d", max_splits);
  IFX_REQUIRE(max_splits == 1 || (chunk > 0 && chunk % TK == 0 && part_o && part_ml && rows && positions && row_req && n_rows > 0),
              "attn_prefill: %d splits need a chunk that is a multiple of %d (got %d), scratch, and the rows to merge", max_splits,
              TK, chunk);
  int page_shift = 0;
  while ((1 << page_shift) < page_size) ++page_shift;
  if (n_tiles == 0) return 0;
  static bool lds_allowed = false;      // more than 64 KB of LDS per workgroup has to be asked for once
  if (!lds_allowed) {
    const hipError_t e = hipFuncSetAttribute((const void*)attn_prefill_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, NS * STAGE_BYTES);
    if (e != hipSuccess) IFX_FAIL("attn_prefill: %d bytes of LDS per workgroup refused: %s", NS * STAGE_BYTES, hipGetErrorString(e));
    lds_allowed = true;
  }
  TileArgs a{(const bf16_t*)q, (const bf16_t*)k_cache, (const bf16_t*)v_cache, (bf16_t*)out, tile_req, tile_q0, q_start,
             q_len, kv_len, block_table, max_blocks, nH, nKV, page_size, window, scale * 1.4426950408889634f, page_shift,
             n_tiles, 0, n_xcd, chunk, max_splits, part_o, part_ml, order};
  const long long items = (long long)n_tiles * nH * max_splits;
  IFX_REQUIRE(items <= (1LL << 30), "attn_prefill: too many tiles for one launch");
  IFX_REQUIRE(!order || (order_per_xcd > 0 && (long long)n_xcd * order_per_xcd >= items && order_per_xcd <= items),
              "attn_prefill: an order of %d x %d places cannot hold %lld work items", n_xcd, order_per_xcd, items);
  IFX_REQUIRE(n_xcd >= 1 && n_xcd <= 64, "%s: %d dies", "attn_prefill", n_xcd);
  a.n_xcd = n_xcd;
  a.per_xcd = order ? order_per_xcd : (int)((items + n_xcd - 1) / n_xcd);
  hipStream_t s = (hipStream_t)stream;
  hipLaunchKernelGGL(attn_prefill_kernel, dim3(n_xcd * a.per_xcd), dim3(64 * NW), NS * STAGE_BYTES, s, a);
  if (max_splits > 1) {
    RowArgs m{(const bf16_t*)q, (const bf16_t*)k_cache, (const bf16_t*)v_cache, rows, row_req, positions, block_table,
              part_o, part_ml, (bf16_t*)out, max_blocks, n_rows, nH, nKV, page_size, window, chunk, max_splits,
              scale * 1.4426950408889634f, 1};
    hipLaunchKernelGGL(attn_rows_merge_kernel, dim3(n_rows, nH), dim3(WAVE * merge_waves(max_splits)), 0, s, m);
  }
  IFX_LAUNCH_CHECK();
}
