// Linear layer on bfloat16 operands with MFMA and 32-bit accumulation:
//   out[m, n] = epilogue( sum_k A[m, k] * W[n, k] + bias[n] )
// A is [M, K] activations, W is [N, K] (the [out, in] layout of a linear
// layer), both contiguous along k, which is what both MFMA operands want.
// Epilogues: plain, tanh-GELU, or accumulate into a 32-bit residual stream.
// Replaces nn.Linear calls of the reference (mlx_lm/models/gpt2.py:41-42,52,
// 68,76-80) and the tied head (mlx_lm/models/gpt2.py:167).
//
// Two kernels:
//  * gemm_bf16_tile: 128x128x64 block tile, 4 waves in 2x2, each wave a 64x64
//    tile of four v_mfma_f32_32x32x16_bf16 accumulators (or 256x256x64 with 8
//    waves); two k-blocks in LDS, two more in registers; each die gets a run
//    of neighbouring tiles that share their operands in its L2; K may be
//    split over blocks where rows are few.  Any M, N; K % 8 == 0.
//  * gemm_bf16_skinny: M <= 64 rows (decode).  A block of four waves owns 16
//    output features and splits K among its waves; W streams from HBM once
//    as the MFMA A-operand, the activations are the B-operand.
#include "common.h"

#include <algorithm>
#include <type_traits>

#define FLAG_GELU 1
#define FLAG_ACCUMULATE 2
#define FLAG_OUT_F32 4
#define FLAG_KV 8  // columns from q_width on are keys, then values: they go to their cache pages, not to out
#define FLAG_THROUGH 16  // (set here) out and ws are below 4 GB: the tile kernels' stores go through to memory

// Out-of-range loads read a clamped address and are zeroed afterwards with this
// constant: selecting between an address and a zero kept in a variable turns
// the load into a flat load through scratch memory.
#define ZERO4 make_uint4(0u, 0u, 0u, 0u)

struct GemmArgs {
  const uint16_t* A;
  const uint16_t* W;
  const float* bias;
  void* out;
  int M, N, K;
  int lda, ldw, ldo;
  int flags;
  // K split over blockIdx.y (tile kernel, 128 x 128): partial sums [n_splits][M][N] go to ws
  float* ws;
  int n_splits, blocks_per_split;
  // key/value scatter (FLAG_KV): row m is token m of the step, at positions[m] of request token_req[m]
  uint16_t* k_pages;
  uint16_t* v_pages;
  size_t page_stride;
  const int* block_table;
  const int* token_req;
  const int* positions;
  int max_blocks, q_width, kv_width, head_dim, page_size;
  // W in the decode kernels' packed order instead of row-major (ldw == 0 at the entry point):
  // tiles of 16 features x 64 k (1024 elements), zero padded, w_kblocks of them a feature block;
  // in a tile the 8 values k = 16 g + 8 h + 0..7 of feature f lie at ((4 h + g) * 16 + f) * 8.
  int w_packed, w_kblocks;
};

// Element offset of the 16-byte piece `piece` (k = 8 piece ..) of feature row n in k-block 0.
__device__ __forceinline__ int packed_piece(int n, int piece, int w_kblocks) {
  return (n >> 4) * w_kblocks * 1024 + ((((piece & 1) << 2) + (piece >> 1)) * 16 + (n & 15)) * 8;
}

// Where column n (a key's or a value's: n >= q_width) of token m lies in the cache pages.
__device__ __forceinline__ uint16_t* kv_place(const GemmArgs& p, int m, int n) {
  const int c = n - p.q_width;
  const bool is_v = c >= p.kv_width;
  const int cc = is_v ? c - p.kv_width : c;
  const int head = cc / p.head_dim, d = cc - head * p.head_dim;
  const int pos = p.positions[m];
  const int page = p.block_table[(size_t)p.token_req[m] * p.max_blocks + pos / p.page_size];
  return (is_v ? p.v_pages : p.k_pages) + (size_t)page * p.page_stride +
         ((size_t)head * p.page_size + pos % p.page_size) * p.head_dim + d;
}

__device__ __forceinline__ void store_out(const GemmArgs& p, int m, int n, float v) {
  if (p.bias) v += p.bias[n];
  if (p.flags & FLAG_GELU) v = gelu_tanh_fast(v);
  if ((p.flags & FLAG_KV) && n >= p.q_width) {
    *kv_place(p, m, n) = f32_to_bf16_bits(v);
    return;
  }
  const size_t idx = (size_t)m * p.ldo + n;
  if (p.flags & FLAG_ACCUMULATE) {
    float* o = (float*)p.out;
    o[idx] += v;
  } else if (p.flags & FLAG_OUT_F32) {
    ((float*)p.out)[idx] = v;
  } else {
    ((uint16_t*)p.out)[idx] = f32_to_bf16_bits(v);
  }
}

// ---------------------------------------------------------------------------

// Rows of a tile beyond the matrix read some row inside it (what they give is
// never stored), and not all the same one: a tile of which only a few rows
// exist would read that one row from hundreds of lanes at once, as would every
// block of that row of tiles, and the cache channel that holds it serves them
// one after another (a step of 2,056 rows took half as long again as one of 2,048).
__device__ __forceinline__ int row_inside(int r, int n) { return r < n ? r : r % n; }

#define BK 64
#define LDS_STRIDE (BK + 8)  // 144 bytes a row: 16-byte reads of 16 rows hit distinct banks

// Which tile a block works on.  Blocks go to the eight dies (each with an L2 of
// its own) in turn, so block b runs on die b % 8.  The tiles are put in an
// order in which neighbours share operands (panels of PANEL rows of tiles; in
// a panel column after column) and that sequence is cut into eight runs of
// equal length, one a die.  So every die gets the same number of tiles to
// within one (dealing whole groups of tiles left a die with 40 tiles and
// another with 4 at 2,056 rows), and the blocks at work on a die at one time
// are a few columns of one panel: what one brings into the L2 the others find
// there.  Returns false for the padding blocks of the grid.
template <int PANEL>
__device__ __forceinline__ bool tile_of_block(int tiles_m, int tiles_n, int& tm, int& tn) {
  const int total = tiles_m * tiles_n, run = (total + 7) / 8;
  const int die = blockIdx.x & 7, local = blockIdx.x >> 3;
  const int idx = die * run + local;
  if (local >= run || idx >= total) return false;
  const int panel = min(idx / (PANEL * tiles_n), (tiles_m + PANEL - 1) / PANEL - 1);  // (only the last is short)
  const int rem = idx - panel * PANEL * tiles_n;
  const int h = min(PANEL, tiles_m - panel * PANEL);
  tn = rem / h;
  tm = panel * PANEL + rem % h;
  return true;
}

// The shape of a block: WAVES_M x WAVES_N waves, each with TM x TN MFMA tiles of
// 32 x 32.  What bounds this kernel is how fast a CU is fed from the L2s, so
// the larger the block's tile, the fewer bytes per product: 128 x 128 (two
// blocks a CU) where the matrix gives few tiles, 256 x 256 (one block a CU,
// half the bytes) where it gives enough of them.
template <int WAVES_M_, int WAVES_N_, int TM_, int TN_, int PANEL_, int BLOCKS_PER_CU_>
struct TileShape {
  static constexpr int WAVES_M = WAVES_M_, WAVES_N = WAVES_N_, TM = TM_, TN = TN_;
  static constexpr int PANEL = PANEL_, BLOCKS_PER_CU = BLOCKS_PER_CU_;  // PANEL: rows of tiles that share a die's L2
  static constexpr int THREADS = 64 * WAVES_M * WAVES_N;
  static constexpr int BM = WAVES_M * TM * 32, BN = WAVES_N * TN * 32;
  static constexpr int PA = BM * 8 / THREADS, PB = BN * 8 / THREADS;  // 16-byte pieces a thread moves per k-block
  static constexpr int ROW_STEP = THREADS / 8;                          // rows between a thread's pieces
};
using Tile128 = TileShape<2, 2, 2, 2, 8, 2>;
using Tile256 = TileShape<2, 4, 4, 2, 4, 1>;
using Tile256x192 = TileShape<4, 2, 2, 3, 4, 1>;
using Tile64x128 = TileShape<1, 4, 2, 1, 8, 2>;
using Tile32x128 = TileShape<1, 4, 1, 1, 8, 2>;
using Tile128x8 = TileShape<2, 4, 2, 1, 8, 1>;  // the same tile with eight waves, for a block that has its CU alone

// Pipeline: LDS holds two k-blocks; registers hold two more on their way.  In
// iteration i the loads of k-block i+2 are issued and k-block i is multiplied
// out of LDS; between the MFMAs of its four steps k-block i+1 (loaded an
// iteration ago) goes from registers to the other half of LDS, a quarter at a
// time (all at the end, the LDS writes of all waves came in one burst with the
// MFMA units idle: 8 % slower); one barrier an iteration.
// SPLIT: K is shared out over blockIdx.y and the partial sums go to the workspace (a kernel of
// its own, so that the unsplit one carries none of it).
// PACKED: W lies in the decode kernels' packed order.  A wave's load is then half a tile of 16
// features x 64 k, 1 KB of consecutive bytes: lane l gets the 8 values k = 16 (l / 16) + 8 h + 0..7
// of feature l % 16, and load g of the block's BN / 8 covers feature block g / 2, half h = g % 2.
// (Reading the packed order with the row-major kernel's lanes, eight pieces of one row to eight
// neighbouring lanes, touched eight lines with every eight lanes: 14 % slower.)
template <typename S, bool SPLIT, bool PACKED>
__global__ __launch_bounds__(S::THREADS, S::BLOCKS_PER_CU) void gemm_bf16_tile_kernel(GemmArgs p) {
  constexpr int BM = S::BM, BN = S::BN, TM = S::TM, TN = S::TN, PA = S::PA, PB = S::PB;
  // (one buffer: the epilogue uses it again for the output tiles)
  __shared__ __attribute__((aligned(16))) uint16_t smem[2 * (BM + BN) * LDS_STRIDE];
  uint16_t* const As[2] = {smem, smem + BM * LDS_STRIDE};
  uint16_t* const Bs[2] = {smem + 2 * BM * LDS_STRIDE, smem + (2 * BM + BN) * LDS_STRIDE};

  int tm, tn;
  if (!tile_of_block<S::PANEL>((p.M + BM - 1) / BM, (p.N + BN - 1) / BN, tm, tn)) return;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave / S::WAVES_N, wn = wave % S::WAVES_N;
  const int m0 = tm * BM;
  const int n0 = tn * BN;

  f32x16_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // each thread moves PA 16-byte pieces of A and PB of W per k-block: piece c
  // is row c / 8, columns (c % 8) * 8 ..; rows beyond the matrix read rows
  // inside it (their products land in rows or columns that are never stored)
  // (32-bit element offsets and one LDS offset: registers are scarce here)
  constexpr int ROW_STEP = S::ROW_STEP;
  int a_off[PA], b_off[PB];
  const int lds_off0 = (tid >> 3) * LDS_STRIDE + (tid & 7) * 8;  // piece i lies ROW_STEP rows further down
#pragma unroll
  for (int i = 0; i < PA; ++i) a_off[i] = row_inside(m0 + (tid >> 3) + ROW_STEP * i, p.M) * p.lda + (tid & 7) * 8;
  // (packed weights: a k-block further on is 1024 elements further on, not 64)
  constexpr int wmul = PACKED ? 16 : 1;
  int lds_b[PB];  // where the thread's pieces of W go in a stage of LDS
#pragma unroll
  for (int i = 0; i < PB; ++i) {
    if constexpr (PACKED) {
      const int g = wave * PB + i, fb = g >> 1, h = g & 1;
      const int nb = min(n0 / 16 + fb, (p.N + 15) / 16 - 1);  // (blocks beyond the matrix read its last one)
      b_off[i] = nb * p.w_kblocks * 1024 + h * 512 + lane * 8;
      lds_b[i] = (fb * 16 + (lane & 15)) * LDS_STRIDE + (2 * (lane >> 4) + h) * 8;
    } else {
      b_off[i] = row_inside(n0 + (tid >> 3) + ROW_STEP * i, p.N) * p.ldw + (tid & 7) * 8;
      lds_b[i] = lds_off0 + i * ROW_STEP * LDS_STRIDE;
    }
  }
  const int kc_mine = (tid & 7) * 8;
  // this split's k-blocks (all of them without a split); the offsets start at its first column
  const int kb_lo = SPLIT ? blockIdx.y * p.blocks_per_split : 0;
  const int n_blocks = SPLIT ? min((p.K + BK - 1) / BK, kb_lo + p.blocks_per_split) - kb_lo : (p.K + BK - 1) / BK;
  const int k_lo = kb_lo * BK;
  if constexpr (SPLIT) {
#pragma unroll
    for (int i = 0; i < PA; ++i) a_off[i] += k_lo;
#pragma unroll
    for (int i = 0; i < PB; ++i) b_off[i] += k_lo * wmul;
  }

  uint4 ra[2][PA], rb[2][PB];
  auto load_global = [&](uint4 (&xa)[PA], uint4 (&xb)[PB], int k0) {
    // a piece beyond K is read from the row's last eight columns instead (K may be
    // smaller than a k-block, so no earlier k-block is sure to hold this piece's
    // columns) and zeroed when it goes to LDS: zeroing it here would make the
    // loads wait at once
    const int kk = (k_lo + k0 + kc_mine < p.K) ? k0 : p.K - 8 - kc_mine - k_lo;
    const int kw = PACKED ? k0 * 16 : kk;  // (packed weights are padded with zeros to whole k-blocks)
#pragma unroll
    for (int i = 0; i < PA; ++i) xa[i] = *(const uint4*)(p.A + a_off[i] + kk);
#pragma unroll
    for (int i = 0; i < PB; ++i) xb[i] = *(const uint4*)(p.W + b_off[i] + kw);
  };
  auto store_lds = [&](int stage, const uint4 (&xa)[PA], const uint4 (&xb)[PB], int k0) {
    const bool in = k_lo + k0 + kc_mine < p.K;
#pragma unroll
    for (int i = 0; i < PA; ++i) *(uint4*)(As[stage] + lds_off0 + i * ROW_STEP * LDS_STRIDE) = in ? xa[i] : ZERO4;
#pragma unroll
    for (int i = 0; i < PB; ++i) *(uint4*)(Bs[stage] + lds_b[i]) = (PACKED || in) ? xb[i] : ZERO4;
  };

  load_global(ra[0], rb[0], 0);
  if (n_blocks > 1) load_global(ra[1], rb[1], BK);
  store_lds(0, ra[0], rb[0], 0);
  __syncthreads();

  const int frag_row = lane & 31;
  const int frag_k = (lane >> 5) * 8;
  const uint16_t* a_frag = As[0] + (wm * TM * 32 + frag_row) * LDS_STRIDE + frag_k;
  const uint16_t* b_frag = Bs[0] + (wn * TN * 32 + frag_row) * LDS_STRIDE + frag_k;

  // Without a split the tiles are accumulated transposed (the weights' rows as the MFMA's rows):
  // a lane then holds four neighbouring columns of one output row, which the epilogue wants.
  auto mfma_tile = [](const bf16x8_t& a, const bf16x8_t& b, const f32x16_t& c) __attribute__((always_inline)) {
    if constexpr (SPLIT)
      return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    else
      return __builtin_amdgcn_mfma_f32_32x32x16_bf16(b, a, c, 0, 0, 0);
  };
  auto multiply = [&](int stage) {
    const uint16_t* af = a_frag + stage * (BM * LDS_STRIDE);
    const uint16_t* bf = b_frag + stage * (BN * LDS_STRIDE);
#pragma unroll
    for (int ks = 0; ks < BK; ks += 16) {
      bf16x8_t a[TM], b[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i) a[i] = *(const bf16x8_t*)(af + i * 32 * LDS_STRIDE + ks);
#pragma unroll
      for (int j = 0; j < TN; ++j) b[j] = *(const bf16x8_t*)(bf + j * 32 * LDS_STRIDE + ks);
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = mfma_tile(a[i], b[j], acc[i][j]);
    }
  };

  // Two k-blocks an iteration, so that the register sets are named statically.
  // The steady part has no branch and no select inside: only then does the
  // compiler count exactly how many loads may stay in flight at each wait
  // (a conditional load makes it wait for all of them).
  auto load_whole = [&](uint4 (&xa)[PA], uint4 (&xb)[PB], int k0) {  // a k-block that lies inside K
#pragma unroll
    for (int i = 0; i < PA; ++i) xa[i] = *(const uint4*)(p.A + a_off[i] + k0);
#pragma unroll
    for (int i = 0; i < PB; ++i) xb[i] = *(const uint4*)(p.W + b_off[i] + k0 * wmul);
  };
  // multiply out of `stage` and, a quarter with each 16 columns, move the next k-block (in
  // registers since the iteration before) into the other stage, which nobody reads any more
  auto multiply_store = [&](int stage, const uint4 (&xa)[PA], const uint4 (&xb)[PB]) {
    const uint16_t* af = a_frag + stage * (BM * LDS_STRIDE);
    const uint16_t* bf = b_frag + stage * (BN * LDS_STRIDE);
    uint16_t* an = As[stage ^ 1] + lds_off0;
    uint16_t* bn = Bs[stage ^ 1];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int ks = q * 16;
      bf16x8_t a[TM], b[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i) a[i] = *(const bf16x8_t*)(af + i * 32 * LDS_STRIDE + ks);
#pragma unroll
      for (int j = 0; j < TN; ++j) b[j] = *(const bf16x8_t*)(bf + j * 32 * LDS_STRIDE + ks);
#pragma unroll
      for (int i = q * PA / 4; i < (q + 1) * PA / 4; ++i) *(uint4*)(an + i * ROW_STEP * LDS_STRIDE) = xa[i];
#pragma unroll
      for (int i = q * PB / 4; i < (q + 1) * PB / 4; ++i) *(uint4*)(bn + lds_b[i]) = xb[i];
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = mfma_tile(a[i], b[j], acc[i][j]);
    }
  };
  int kb = 0;
  const int whole_blocks = SPLIT ? min(n_blocks, p.K / BK - kb_lo) : p.K / BK;  // k-blocks that need no masking
  for (; kb + 4 <= whole_blocks; kb += 2) {
    load_whole(ra[0], rb[0], (kb + 2) * BK);
    __builtin_amdgcn_sched_barrier(0);  // the loads go out before the arithmetic, not after it
    multiply_store(0, ra[1], rb[1]);
    __syncthreads();
    load_whole(ra[1], rb[1], (kb + 3) * BK);
    __builtin_amdgcn_sched_barrier(0);
    multiply_store(1, ra[0], rb[0]);
    __syncthreads();
  }
  // the last few k-blocks, with every guard
  for (; kb < n_blocks; kb += 2) {
    if (kb + 2 < n_blocks) load_global(ra[0], rb[0], (kb + 2) * BK);
    multiply(0);
    if (kb + 1 < n_blocks) store_lds(1, ra[1], rb[1], (kb + 1) * BK);
    __syncthreads();
    if (kb + 1 >= n_blocks) break;
    if (kb + 3 < n_blocks) load_global(ra[1], rb[1], (kb + 3) * BK);
    multiply(1);
    if (kb + 2 < n_blocks) store_lds(0, ra[0], rb[0], (kb + 2) * BK);
    __syncthreads();
  }

  if constexpr (SPLIT) {  // the partial sums as they are; sum_partials adds them and runs the epilogue
    float* ws = p.ws + (size_t)blockIdx.y * p.M * p.N;
    const bool through = p.flags & FLAG_THROUGH;
    const __amdgpu_buffer_rsrc_t ws_buf = through_buffer(ws, (size_t)p.M * p.N * 4);
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int n = n0 + wn * TN * 32 + j * 32 + (lane & 31);
      if (n >= p.N) continue;
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        const int mb = m0 + wm * TM * 32 + i * 32 + 4 * (lane >> 5);
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int m = mb + 8 * (r >> 2) + (r & 3);
          if (m >= p.M) continue;
          if (through)
            store_through(ws_buf, (uint32_t)(((size_t)m * p.N + n) * 4), acc[i][j][r]);
          else
            ws[(size_t)m * p.N + n] = acc[i][j][r];
        }
      }
    }
    return;
  }

  // Epilogue.  Accumulator r of a transposed 32x32 tile: output row lane % 32, column
  // 8*(r/4) + 4*(lane/32) + r%4.  Stored like that, every lane of a store would be in
  // another row (and with the tiles not transposed, a store would be 64 bytes of 2-byte
  // pieces): the epilogue took 13 to 24 us of a product's 43 to 62 at 2,048 rows.  So each
  // wave passes its tile through LDS, 32 rows at a time, and takes it out again with eight
  // neighbouring columns a lane: stores of 16 or 32 bytes a lane that cover whole rows of
  // the wave's tile.  The region of a wave is its own; a wave's LDS accesses keep their order.
  constexpr int NW = S::THREADS / 64;
  constexpr int WCOLS = TN * 32;   // columns of a wave's tile
  constexpr int EST = WCOLS + 4;   // floats a row in LDS: sixteen-byte pieces of neighbouring rows on other banks
  static_assert(NW * 32 * EST * 4 <= (int)sizeof(smem), "the waves' output tiles fit the k-blocks' LDS");
  __syncthreads();  // nobody reads a k-block any more
  float* const tile = (float*)smem + wave * 32 * EST;
  // (read and written through two names: an element is read and then written by the same lane,
  // and no load has to wait for stores to other elements)
  const float* __restrict__ res = (const float*)p.out;
  float* __restrict__ out_f = (float*)p.out;
  uint16_t* __restrict__ out_h = (uint16_t*)p.out;
  const bool f32_out = p.flags & (FLAG_ACCUMULATE | FLAG_OUT_F32);
  const bool through = p.flags & FLAG_THROUGH;
  const __amdgpu_buffer_rsrc_t out_buf = through_buffer(p.out, ((size_t)(p.M - 1) * p.ldo + p.N) * (f32_out ? 4 : 2));
  // CPL columns a lane on the way out, 16 bytes of the output: eight bfloat16 or four floats, so
  // that a store covers whole 128-byte lines of a few rows
  auto emit = [&](auto cpl) __attribute__((always_inline)) {
    constexpr int CPL = decltype(cpl)::value;
    constexpr int LPR = WCOLS / CPL;  // lanes a row
    constexpr int RPP = 64 / LPR;     // rows a pass
    constexpr int PASSES = (32 + RPP - 1) / RPP;
    constexpr int GROUP = PASSES < 32 / CPL ? PASSES : 32 / CPL;  // passes whose values are in registers at a time
    const int erow = lane / LPR, ecol = (lane % LPR) * CPL;
    const bool elane = erow < RPP;
    const int n = n0 + wn * WCOLS + ecol;  // this lane's columns, in every row it takes out
    float bias[CPL];
#pragma unroll
    for (int c = 0; c < CPL; ++c) bias[c] = p.bias ? p.bias[min(n + c, p.N - 1)] : 0.f;
    // whole pieces of 16 bytes: the row stride and the base keep them aligned, and all the columns exist
    const bool vec = n + CPL <= p.N && p.ldo % CPL == 0 && ((uintptr_t)p.out & 15) == 0;
    // this lane's columns are a key's or a value's: its pieces go to the token's place in the
    // cache pages (the host has seen to it that a piece of eight columns stays inside a head)
    const bool kv_lane = CPL == 8 && (p.flags & FLAG_KV) && n >= p.q_width;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int mt = m0 + wm * TM * 32 + i * 32;  // first row of this 32-row tile
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();  // every lane has read the tile before
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int g = 0; g < 4; ++g)
          *(float4*)(tile + (lane & 31) * EST + j * 32 + 8 * g + 4 * (lane >> 5)) =
              make_float4(acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]);
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
      for (int s0 = 0; s0 < PASSES; s0 += GROUP) {
        // what is added to goes out first, all of the group's at once (left to itself the
        // compiler puts each load next to its use: one trip after another)
        float o[GROUP][CPL];
        if (p.flags & FLAG_ACCUMULATE) {
#pragma unroll
          for (int s = 0; s < GROUP; ++s) {
            const float* orow = res + (size_t)min(mt + (s0 + s) * RPP + erow, p.M - 1) * p.ldo;
            if (vec) {
              const float4 t = *(const float4*)(orow + n);  // (CPL is 4 with 32-bit outputs)
              o[s][0] = t.x, o[s][1] = t.y, o[s][2] = t.z, o[s][3] = t.w;
            } else {
#pragma unroll
              for (int c = 0; c < CPL; ++c) o[s][c] = orow[min(n + c, p.N - 1)];
            }
          }
        }
        uint16_t* place[GROUP];
        if (kv_lane) {
#pragma unroll
          for (int s = 0; s < GROUP; ++s) place[s] = kv_place(p, min(mt + (s0 + s) * RPP + erow, p.M - 1), n);
        }
        __builtin_amdgcn_sched_barrier(0);
        float v[GROUP][CPL];
#pragma unroll
        for (int s = 0; s < GROUP; ++s) {
          const int row = min((s0 + s) * RPP + erow, 31);
#pragma unroll
          for (int c = 0; c < CPL; c += 4) {
            const float4 t = *(const float4*)(tile + row * EST + ecol + c);
            v[s][c] = t.x + bias[c], v[s][c + 1] = t.y + bias[c + 1], v[s][c + 2] = t.z + bias[c + 2], v[s][c + 3] = t.w + bias[c + 3];
          }
        }
        if (p.flags & FLAG_ACCUMULATE) {
#pragma unroll
          for (int s = 0; s < GROUP; ++s)
#pragma unroll
            for (int c = 0; c < CPL; ++c) v[s][c] += o[s][c];
        } else if (p.flags & FLAG_GELU) {
#pragma unroll
          for (int s = 0; s < GROUP; ++s)
#pragma unroll
            for (int c = 0; c < CPL; ++c) v[s][c] = gelu_tanh_fast(v[s][c]);
        }
#pragma unroll
        for (int s = 0; s < GROUP; ++s) {
          const int row = (s0 + s) * RPP + erow, m = mt + row;
          if (!elane || row >= 32 || m >= p.M || n >= p.N) continue;
          const size_t at = (size_t)m * p.ldo + n;
          if (vec) {
            u32x4_t t;
            if constexpr (CPL == 4)
              t = u32x4_t{__float_as_uint(v[s][0]), __float_as_uint(v[s][1]), __float_as_uint(v[s][2]), __float_as_uint(v[s][3])};
            else
              t = u32x4_t{pack_bf16x2(v[s][0], v[s][1]), pack_bf16x2(v[s][2], v[s][3]),
                          pack_bf16x2(v[s][4], v[s][5]), pack_bf16x2(v[s][6], v[s][7])};
            if (kv_lane)
              *(u32x4_t*)place[s] = t;  // (attention reads it next: it may stay in the L2)
            else if (through)
              store_through(out_buf, (uint32_t)(at * (CPL == 4 ? 4 : 2)), t);
            else
              *(u32x4_t*)(CPL == 4 ? (void*)(out_f + at) : (void*)(out_h + at)) = t;
          } else if (kv_lane) {
#pragma unroll
            for (int c = 0; c < CPL; ++c)
              if (n + c < p.N) place[s][c] = f32_to_bf16_bits(v[s][c]);
          } else {
#pragma unroll
            for (int c = 0; c < CPL; ++c) {
              if (n + c >= p.N) break;
              if constexpr (CPL == 4)
                out_f[at + c] = v[s][c];
              else
                out_h[at + c] = f32_to_bf16_bits(v[s][c]);
            }
          }
        }
      }
    }
  };
  if (f32_out)
    emit(std::integral_constant<int, 4>{});
  else
    emit(std::integral_constant<int, 8>{});
}

// ---------------------------------------------------------------------------
// Skinny kernel: out^T tile = W[16 features, K] x A^T[K, up to 64 rows].
// Lane l of a wave reads 32 contiguous bytes of W row (l % 16) per 64-wide
// k-block, at k offset (l / 16) * 16, and feeds them to two 16x16x32 MFMAs;
// the activation fragment uses the same k offsets, so the products pair up.

#define SK_WAVES 4
#define SK_MAXM 64
// From 17 rows on this file's kernels take the product: tiles of 32 x 128 up to 32 rows and of
// 64 x 128 up to 64 (and beyond where 128 x 128 tiles would be few), with K split over blocks
// where the tiles alone do not fill the GPU.  (A kernel that streamed the weights once for 17 to
// 64 rows, 64 features a block, was 3 to 17 % slower than these at GPT-2 XL's projections and
// twice as slow at the vocabulary's head.)
#define TILE_MIN_ROWS 17

template <int MT>  // number of 16-row groups of activations (1..4)
__global__ __launch_bounds__(256) void gemm_bf16_skinny_kernel(GemmArgs p) {
  __shared__ float red[SK_WAVES][MT][64 * 4];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int n0 = blockIdx.x * 16;
  const int wrow = n0 + (lane & 15);
  const int koff = (lane >> 4) * 16;
  const bool wvalid = wrow < p.N;
  const uint16_t* wrow_p = p.W + (size_t)(wvalid ? wrow : 0) * p.ldw;
  // packed weights: the lane's two pieces of a k-block are pieces 2 g and 2 g + 1 of its feature
  const uint16_t* wpack0 = p.W + packed_piece(wvalid ? wrow : 0, 2 * (lane >> 4), p.w_kblocks);
  const uint16_t* wpack1 = p.W + packed_piece(wvalid ? wrow : 0, 2 * (lane >> 4) + 1, p.w_kblocks);

  f32x4_t acc[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) acc[t] = (f32x4_t){0.f, 0.f, 0.f, 0.f};

  union Frag {
    uint4 u;
    bf16x8_t v;
  };

  for (int k0 = wave * 64; k0 < p.K; k0 += SK_WAVES * 64) {
    const int k = k0 + koff;  // this lane covers k .. k+15
    Frag w0, w1;
    const uint4 t0 = *(const uint4*)(p.w_packed ? wpack0 + (size_t)k0 * 16 : wrow_p + min(k, p.K - 8));
    const uint4 t1 = *(const uint4*)(p.w_packed ? wpack1 + (size_t)k0 * 16 : wrow_p + min(k + 8, p.K - 8));
    w0.u = (wvalid && k < p.K) ? t0 : ZERO4;
    w1.u = (wvalid && k + 8 < p.K) ? t1 : ZERO4;
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      const int m = t * 16 + (lane & 15);
      const bool av = m < p.M;
      const uint16_t* arow = p.A + (size_t)(av ? m : 0) * p.lda;
      Frag a0, a1;
      const uint4 u0 = *(const uint4*)(arow + min(k, p.K - 8));
      const uint4 u1 = *(const uint4*)(arow + min(k + 8, p.K - 8));
      a0.u = (av && k < p.K) ? u0 : ZERO4;
      a1.u = (av && k + 8 < p.K) ? u1 : ZERO4;
      acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w0.v, a0.v, acc[t], 0, 0, 0);
      acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w1.v, a1.v, acc[t], 0, 0, 0);
    }
  }

  // sum the waves' partial tiles in a fixed order
#pragma unroll
  for (int t = 0; t < MT; ++t)
#pragma unroll
    for (int r = 0; r < 4; ++r) red[wave][t][lane * 4 + r] = acc[t][r];
  __syncthreads();
  if (wave == 0) {
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      // accumulator r: feature row 4*(lane/16) + r, activation column lane%16
      const int m = t * 16 + (lane & 15);
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        float v = 0.f;
#pragma unroll
        for (int w = 0; w < SK_WAVES; ++w) v += red[w][t][lane * 4 + r];
        const int n = n0 + 4 * (lane >> 4) + r;
        if (m < p.M && n < p.N) store_out(p, m, n, v);
      }
    }
  }
}

// ---------------------------------------------------------------------------

DEFINE_LAST_ERROR(mlxlm_last_error)

static int check_args(const GemmArgs& p) {
  if (p.M < 0 || p.N <= 0 || p.K <= 0) FAIL("gemm_bf16: bad sizes M=%d N=%d K=%d", p.M, p.N, p.K);
  if (p.K % 8 != 0) FAIL("gemm_bf16: K=%d must be a multiple of 8", p.K);
  if (p.lda % 8 != 0 || p.ldw % 8 != 0)
    FAIL("gemm_bf16: row strides lda=%d ldw=%d must be multiples of 8", p.lda, p.ldw);
  if (p.lda < p.K || (!p.w_packed && p.ldw < p.K) || p.ldo < p.N)
    FAIL("gemm_bf16: row strides smaller than the rows (lda=%d ldw=%d ldo=%d)", p.lda, p.ldw, p.ldo);
  if (!p.A || !p.W || !p.out) FAIL("gemm_bf16: null pointer");
  if (((uintptr_t)p.A | (uintptr_t)p.W) & 15) FAIL("gemm_bf16: A and W must be 16-byte aligned");
  const size_t w_elements = p.w_packed ? (size_t)((p.N + 15) / 16) * p.w_kblocks * 1024 : (size_t)p.N * p.ldw;
  if ((size_t)p.M * p.lda >= (1u << 31) || w_elements >= (1u << 31))
    FAIL("gemm_bf16: operands of 2^31 elements or more are not supported");
  if ((p.flags & FLAG_ACCUMULATE) && (p.flags & FLAG_GELU))
    FAIL("gemm_bf16: GELU and accumulate cannot be combined");
  return 0;
}

template <typename S>
static void launch_tiles(const GemmArgs& p, hipStream_t stream) {
  const long tiles = (long)((p.M + S::BM - 1) / S::BM) * ((p.N + S::BN - 1) / S::BN);
  dim3 grid((unsigned)((tiles + 7) / 8 * 8), p.n_splits), block(S::THREADS);  // a run of tiles for each die
  if (p.n_splits > 1) {
    if (p.w_packed)
      hipLaunchKernelGGL((gemm_bf16_tile_kernel<S, true, true>), grid, block, 0, stream, p);
    else
      hipLaunchKernelGGL((gemm_bf16_tile_kernel<S, true, false>), grid, block, 0, stream, p);
  } else {
    if (p.w_packed)
      hipLaunchKernelGGL((gemm_bf16_tile_kernel<S, false, true>), grid, block, 0, stream, p);
    else
      hipLaunchKernelGGL((gemm_bf16_tile_kernel<S, false, false>), grid, block, 0, stream, p);
  }
}

// How many tiles a die gets (tile_of_block shares them out evenly).
template <typename S>
static int busiest_die(int M, int N) {
  const long tiles = (long)((M + S::BM - 1) / S::BM) * ((N + S::BN - 1) / S::BN);
  return (int)((tiles + 7) / 8);
}

// Microseconds per k-block of the busiest die, from what was measured at GPT-2 XL
// sizes: two 128 x 128 blocks on a CU finish a k-block each in 1.15 us, one
// alone in 1.3 us (its fetching and its arithmetic take turns; two blocks
// overlap each other's), a 256 x 256 block (four times the work) in 2.0 us.  A
// die has 32 CUs.
static double cost_128(int M, int N) {
  const int per_die = n_compute_units() / N_DIES;  // CUs of a die: two of these blocks fit each
  const int tiles = busiest_die<Tile128>(M, N);
  const int rest = tiles % (2 * per_die);
  // (a last round of few blocks finds the L2 idle: 1.0)
  return (double)(tiles / (2 * per_die)) * 1.15 +
         (rest == 0 ? 0.0 : rest <= per_die / 2 ? 1.0 : rest <= per_die ? 1.3 : 1.15);
}
static double cost_256(int M, int N) {
  const int per_die = n_compute_units() / N_DIES;
  return (double)((busiest_die<Tile256>(M, N) + per_die - 1) / per_die) * 2.0;
}
// (256 x 192: three quarters of the arithmetic, seven eighths of the bytes; its tiles fit N = 4800)
static double cost_256x192(int M, int N) {
  const int per_die = n_compute_units() / N_DIES;
  return (double)((busiest_die<Tile256x192>(M, N) + per_die - 1) / per_die) * 1.6;
}

// Tiles of 64 x 128 instead of 128 x 128 where the latter would be few (up to 128): twice the
// blocks, each with half the arithmetic and three quarters of the bytes.  Measured at widths
// from 768 to 2,048: ahead by up to a quarter while the 128 x 128 tiles leave half the CUs idle,
// level at 144 tiles, behind from 160 on (2,048 rows of a projection to 1,280 features with
// K = 5,120: 59 us against 51), where what the tiles fetch from the L2s counts for more.
static bool small_tiles(int M, int N) { return (long)((M + 127) / 128) * ((N + 127) / 128) <= 128; }

// Microseconds a CU takes per k-block when it holds `n` blocks of tiles `rows` x 128 (measured at
// widths 768 to 2,048): a block alone waits for its fetches most of the time, so a second block
// on the CU costs little; from the third on they take turns.
static double kblock_us(int rows, int n) {
  const double alone = rows <= 32 ? 0.37 : rows <= 64 ? 0.52 : 0.62;
  const double pair = rows <= 32 ? 0.56 : rows <= 64 ? 0.80 : 1.14;
  return (n / 2) * pair + (n % 2) * alone;
}

// Into how many parts the kernels with tiles 128 wide should split K (1: no split).  Few rows
// give few tiles (up to 128 rows of GPT-2 XL's projections are 13 to 50 tiles for 256 CUs), and a
// tile's walk through K takes the same time whether 50 or 500 of them run; a split shortens the
// walk and costs a second kernel that reads the partial sums ([parts][M][N] floats).  Both sides
// are priced from what was measured (65 to 768 rows, widths 768 to 2,048, K up to 8,192): the walk
// as k-blocks times the time per k-block of the busiest CU, the second kernel as a launch plus
// its bytes at 3 TB/s.  `fused`: the second kernel stands in for one that would run anyway (the
// norm that follows a sum into the residual stream, the write of keys and values into their
// pages), so it costs only the extra bytes.  A part keeps three k-blocks or more.
// `force` > 0 asks for that many parts wherever K has them (for tests of small sizes).
extern "C" int gemm_bf16_splits(int M, int N, int K, int fused, int force) {
  if (M < TILE_MIN_ROWS) return 1;
  const long cols = (N + 127) / 128;
  const int rows = M <= 32 ? 32 : small_tiles(M, N) ? 64 : 128;
  const long tiles = (long)((M + rows - 1) / rows) * cols;
  const int n_blocks = (K + BK - 1) / BK;
  int best = 1;
  if (force > 0) {
    best = force < n_blocks ? force : n_blocks;
  } else {
    double best_us = 0.0, whole_us = 0.0;
    for (int s = 1; s <= 16 && s <= (n_blocks >= 3 ? n_blocks / 3 : 1); ++s) {
      const int per = (n_blocks + s - 1) / s;
      const int on_cu = (int)((tiles * s + n_compute_units() - 1) / n_compute_units());
      double us = kblock_us(rows, on_cu) * per;
      if (s > 1) us += (fused ? 1.0 : 2.5) + 8.0 * (fused ? s - 1 : s) * (double)M * N / 3e6;
      if (s == 1) whole_us = us;
      if (s == 1 || us < best_us) best = s, best_us = us;
    }
    if (best_us > 0.9 * whole_us) best = 1;  // (the prices are good to a tenth)
  }
  if (best <= 1) return 1;
  const int per = (n_blocks + best - 1) / best;
  return (n_blocks + per - 1) / per;  // no empty part
}

// variant: 0 = choose, 1 = 128 x 128 tiles, 2 = skinny kernel, 3 = 256 x 256 tiles, 4 = 256 x 192
// tiles, 5 = 64 x 128 tiles, 6 = 32 x 128 tiles.  n_splits > 1 (variants 1, 5 and 6 only): no
// epilogue, the partial sums go to ws.  ldw == 0: W is in the decode kernels' packed order
// (tiles of 16 features x 64 k, zero padded), which all kernels here read as well as rows.
extern "C" int gemm_bf16_scatter(void* out, const void* A, const void* W, const float* bias, int M, int N,
                                 int K, int lda, int ldw, int ldo, int flags, int variant, int n_splits,
                                 float* ws, size_t ws_floats, void* k_pages, void* v_pages, size_t page_stride,
                                 const int* block_table, int max_blocks, const int* token_req,
                                 const int* positions, int q_width, int kv_width, int head_dim, int page_size,
                                 hipStream_t stream);

extern "C" int gemm_bf16(void* out, const void* A, const void* W, const float* bias, int M, int N,
                         int K, int lda, int ldw, int ldo, int flags, int variant, int n_splits,
                         float* ws, size_t ws_floats, hipStream_t stream) {
  return gemm_bf16_scatter(out, A, W, bias, M, N, K, lda, ldw, ldo, flags, variant, n_splits, ws, ws_floats,
                           nullptr, nullptr, 0, nullptr, 0, nullptr, nullptr, 0, 0, 0, 0, stream);
}

// The same with the cache scatter of a fused q/k/v projection (k_pages != null, no split of K, a
// bfloat16 output): the columns from q_width on (kv_width of keys, then kv_width of values) of
// row m go to position positions[m] of request token_req[m] in the pages, through the block
// table, and are not written to out.
extern "C" int gemm_bf16_scatter(void* out, const void* A, const void* W, const float* bias, int M, int N,
                                 int K, int lda, int ldw, int ldo, int flags, int variant, int n_splits,
                                 float* ws, size_t ws_floats, void* k_pages, void* v_pages, size_t page_stride,
                                 const int* block_table, int max_blocks, const int* token_req,
                                 const int* positions, int q_width, int kv_width, int head_dim, int page_size,
                                 hipStream_t stream) {
  GemmArgs p;
  p.A = (const uint16_t*)A;
  p.W = (const uint16_t*)W;
  p.bias = bias;
  p.out = out;
  p.M = M, p.N = N, p.K = K;
  p.lda = lda, p.ldw = ldw, p.ldo = ldo;
  p.flags = flags & (FLAG_GELU | FLAG_ACCUMULATE | FLAG_OUT_F32);
  p.w_packed = ldw == 0 ? 1 : 0, p.w_kblocks = (K + BK - 1) / BK;
  if (check_args(p)) return 1;
  if (M == 0) return 0;
  p.k_pages = (uint16_t*)k_pages, p.v_pages = (uint16_t*)v_pages, p.page_stride = page_stride;
  p.block_table = block_table, p.token_req = token_req, p.positions = positions;
  p.max_blocks = max_blocks, p.q_width = q_width, p.kv_width = kv_width, p.head_dim = head_dim, p.page_size = page_size;
  if (k_pages) {
    if (flags & (FLAG_GELU | FLAG_ACCUMULATE | FLAG_OUT_F32)) FAIL("gemm_bf16: the cache scatter goes with a plain bfloat16 output");
    if (n_splits > 1) FAIL("gemm_bf16: with K split, sum_partials scatters keys and values");
    if (!v_pages || !block_table || !token_req || !positions)
      FAIL("gemm_bf16: the cache scatter needs pages, block table, token_req and positions");
    if (head_dim <= 0 || page_size <= 0 || head_dim % 8 != 0 || q_width % 8 != 0 || kv_width % head_dim != 0 ||
        q_width + 2 * kv_width != N)
      FAIL("gemm_bf16: q_width %d + 2 * kv_width %d must be N=%d, widths multiples of 8, kv_width of head_dim %d",
           q_width, kv_width, N, head_dim);
    if (page_stride % 8 != 0 || (((uintptr_t)k_pages | (uintptr_t)v_pages) & 15))
      FAIL("gemm_bf16: cache pages must be 16-byte aligned");
    if (ldo < q_width) FAIL("gemm_bf16: ldo=%d smaller than q_width=%d", ldo, q_width);
    p.flags |= FLAG_KV;
  }
  const int n_blocks = (K + BK - 1) / BK;
  if (n_splits < 1 || n_splits > n_blocks) FAIL("gemm_bf16: %d splits of K=%d", n_splits, K);
  p.ws = ws, p.n_splits = n_splits, p.blocks_per_split = (n_blocks + n_splits - 1) / n_splits;
  if (fits_through_buffer((size_t)M * ldo * 4) && fits_through_buffer((size_t)M * N * 4)) p.flags |= FLAG_THROUGH;
  if (n_splits > 1) {
    if (variant == 0) variant = M <= 32 ? 6 : small_tiles(M, N) ? 5 : 1;
    if (variant != 1 && variant != 5 && variant != 6) FAIL("gemm_bf16: only the tiles of 128, 64 and 32 rows by 128 split K");
    if (p.blocks_per_split * (n_splits - 1) >= n_blocks) FAIL("gemm_bf16: %d splits of K=%d leave one empty", n_splits, K);
    if (!ws || ((uintptr_t)ws & 15) || ws_floats < (size_t)n_splits * M * N)
      FAIL("gemm_bf16: %d splits of %d x %d need an aligned workspace of that many floats", n_splits, M, N);
  }
  if (variant == 0) {
    if (M < TILE_MIN_ROWS)
      variant = 2;
    else if (M <= 32)
      variant = 6;
    else if (M <= 64 || small_tiles(M, N))
      variant = 5;
    else {
      const double c1 = cost_128(M, N), c3 = cost_256(M, N), c4 = cost_256x192(M, N);
      variant = c4 < c3 && c4 < c1 ? 4 : c3 < c1 ? 3 : 1;
      // No more tiles of 128 x 128 than CUs: a block alone on its CU hides more of its waits with eight
      // waves of 64 x 32 than with four of 64 x 64 (2,048 rows to 1,600 features: 24.0 us against 26.4 at
      // K = 1,600, 65.1 against 67.6 at 6,400; with two blocks a CU the four waves are level or ahead).
      if (variant == 1 && n_splits == 1 && busiest_die<Tile128>(M, N) <= n_compute_units() / N_DIES) variant = 7;
    }
  }
  if (variant == 2) {
    if (M > SK_MAXM) FAIL("gemm_bf16: the skinny kernel takes at most %d rows, got %d", SK_MAXM, M);
    dim3 grid((N + 15) / 16), block(256);
    const int mt = (M + 15) / 16;
    if (mt == 1)
      hipLaunchKernelGGL(gemm_bf16_skinny_kernel<1>, grid, block, 0, stream, p);
    else if (mt == 2)
      hipLaunchKernelGGL(gemm_bf16_skinny_kernel<2>, grid, block, 0, stream, p);
    else if (mt == 3)
      hipLaunchKernelGGL(gemm_bf16_skinny_kernel<3>, grid, block, 0, stream, p);
    else
      hipLaunchKernelGGL(gemm_bf16_skinny_kernel<4>, grid, block, 0, stream, p);
  } else if (variant == 7) {
    launch_tiles<Tile128x8>(p, stream);

  } else if (variant == 1 || variant == 3 || variant == 4 || variant == 5 || variant == 6) {
    if (variant == 1)
      launch_tiles<Tile128>(p, stream);
    else if (variant == 3)
      launch_tiles<Tile256>(p, stream);
    else if (variant == 4)
      launch_tiles<Tile256x192>(p, stream);
    else if (variant == 5)
      launch_tiles<Tile64x128>(p, stream);
    else
      launch_tiles<Tile32x128>(p, stream);
  } else {
    FAIL("gemm_bf16: unknown variant %d", variant);
  }
  CHECK_LAUNCH("gemm_bf16");
  return 0;
}
