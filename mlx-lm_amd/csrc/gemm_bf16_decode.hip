// Linear layer for decode steps: at most 16 rows of activations against a
// bfloat16 weight matrix that streams from HBM exactly once.
//   out[m, n] = epilogue( sum_k A[m, k] * W[n, k] + bias[n] )
// with fusions that save launches and round trips through memory:
//  * prologue: A may be given as the float32 residual stream plus LayerNorm
//    parameters; every block then norms the (few) rows itself into LDS
//    (mlx_lm/models/gpt2.py:104,106: ln_1 / ln_2 before c_attn / c_fc);
//  * epilogue: output columns from `q_width` on may be scattered straight
//    into the pages of the key/value cache (mlx_lm/models/cache.py:352-354)
//    instead of the output matrix.
// Otherwise the epilogues of gemm_bf16.hip: plain, tanh-GELU, accumulate into
// the float32 residual stream, float32 out.
//
// Weights come row-major [N, K] or packed (ldw == 0): tiles of 16 features x
// 64 k stored in the order the lanes read them, so that a wave's load is 1 KB
// of consecutive bytes; packed weights stream about twice as fast, because a
// row-major tile is sixteen 64-byte pieces per load.
//
// A block of eight waves owns 16 output features.  The
// activations (normed or copied) sit in LDS whole as the MFMA B-operand; each
// wave takes every eighth 64-wide k-block of the 16 weight rows as the
// A-operand of two v_mfma_f32_16x16x32_bf16 (lane l reads 32 contiguous bytes
// of row l % 16 at k offset (l / 16) * 16).  Weight loads run two passes ahead
// of the MFMAs; the eight partial tiles are summed in a fixed order.  Where
// the matrix has few features and K is not split, a block owns only eight of
// them (lanes 8..15 of a group repeat the eighth): twice as many blocks.
// (17 to 48 rows have a kernel of their own further down, gemm_bf16_rows; more
// are the tile kernels' of gemm_bf16.hip.  Both leave their partial sums to the
// second kernels of this file in the same way.)
//
// A CU keeps only so many loads in flight, so a launch that does not occupy
// every CU cannot reach the memory's bandwidth.  Where the feature blocks alone
// are too few, K is split over blockIdx.y: each split then writes its partial
// sums [split][m][n] in float32 to a workspace instead of running the
// epilogue, and a second, small kernel adds them in the order of the splits
// and runs the epilogue (sum_partials), or, for the residual stream, adds them
// to it and norms the new rows in the same pass (sum_partials_norm): the
// LayerNorm that follows a block's last projection costs no launch of its own
// and the next projection needs no norm prologue.  (A hand-over inside one
// kernel, last block to arrive sums, was tried: the release/acquire pair it
// needs writes back and invalidates an L2 per block on this multi-die GPU and
// took 120 us where the whole product takes 8.)
#include "common.h"
#include "no_alloc.h"

#include <mutex>

#define FLAG_GELU 1
#define FLAG_ACCUMULATE 2
#define FLAG_OUT_F32 4
#define FLAG_KV 8
#define FLAG_OUT_PACKED 16  // a bfloat16 out in tiles of 16 rows x 64 columns, in the weights' packed order

#define NW 8        // waves per block
#define U 4         // k-blocks per pass and wave
#define LN_MAX_V 8  // float4 per lane a normed row may take (K <= 2048)
#define ZERO4 make_uint4(0u, 0u, 0u, 0u)  // a constant, not a variable: see load_pass

struct DecodeGemmArgs {
  const uint16_t* W;
  const float* bias;
  void* out;
  const uint16_t* A;   // [M, K] activations, or null when X is given
  const float* X;      // [M, K] residual stream to be normed
  const float* gamma;
  const float* beta;
  float eps;
  int M, N, K, lda, ldx, ldw, ldo, flags;
  int a_stride;        // LDS row stride in elements
  // key/value scatter
  uint16_t* k_pages;
  uint16_t* v_pages;
  size_t page_stride;
  const int* block_table;
  const int* token_req;
  const int* positions;
  int max_blocks, q_width, kv_width, head_dim, page_size;
  // split of K over blockIdx.y
  int n_splits, chunks_per_split;
  int rows;            // output features a block of the 16-row kernel owns (16, or 8 where features are few)
  float* ws;           // [n_splits][M][N] partial sums, when n_splits > 1
  int vec4;            // four outputs at a time: N, ldo and the scatter widths are multiples of 4, pointers aligned
  int a_packed;        // rows kernel: A lies in tiles of 16 rows x 64 k in the weights' packed order (packed_at)
  int row_groups;      // rows kernel: the rows go in this many groups of R_TILES tiles, a block each
  int out_kblocks;     // FLAG_OUT_PACKED: tiles a tile row of out, (N + 63) / 64
};

__device__ __forceinline__ uint32_t pack2(float a, float b) { return pack_bf16x2(a, b); }


union Frag {
  uint4 u;
  bf16x8_t v;
};

// bias, activation and where one output goes: the matrix, the residual stream or a cache page.
// What that takes from memory the caller has read already: `bias`, `old` (the stream's value,
// where the product is added into it), and for a key or value the row's position and the page
// that position lies in.
struct FinishLoads {
  float bias, old;
  int pos, page;
};
__device__ __forceinline__ void finish_with(const DecodeGemmArgs& p, int m, int n, float v, const FinishLoads& l) {
  if (p.bias) v += l.bias;
  if (p.flags & FLAG_GELU) v = gelu_tanh_fast(v);
  if ((p.flags & FLAG_KV) && n >= p.q_width) {
    const int c = n - p.q_width;
    const bool is_v = c >= p.kv_width;
    const int cc = is_v ? c - p.kv_width : c;
    const int head = cc / p.head_dim, d = cc - head * p.head_dim;
    const size_t dst = (size_t)l.page * p.page_stride +
                       ((size_t)head * p.page_size + l.pos % p.page_size) * p.head_dim + d;
    (is_v ? p.v_pages : p.k_pages)[dst] = f32_to_bf16_bits(v);
  } else {
    const size_t idx = (size_t)m * p.ldo + n;
    if (p.flags & FLAG_OUT_PACKED)
      ((uint16_t*)p.out)[packed_at(m, n, p.out_kblocks)] = f32_to_bf16_bits(v);
    else if (p.flags & FLAG_ACCUMULATE)
      ((float*)p.out)[idx] = l.old + v;
    else if (p.flags & FLAG_OUT_F32)
      ((float*)p.out)[idx] = v;
    else
      ((uint16_t*)p.out)[idx] = f32_to_bf16_bits(v);
  }
}
__device__ __forceinline__ void finish(const DecodeGemmArgs& p, int m, int n, float v) {
  const bool kv = (p.flags & FLAG_KV) && n >= p.q_width;
  const bool adds = (p.flags & FLAG_ACCUMULATE) && !kv && !(p.flags & FLAG_OUT_PACKED);
  FinishLoads l;
  l.bias = p.bias ? p.bias[n] : 0.f;
  l.old = adds ? ((const float*)p.out)[(size_t)m * p.ldo + n] : 0.f;
  l.pos = kv ? p.positions[m] : 0;
  l.page = kv ? p.block_table[(size_t)p.token_req[m] * p.max_blocks + l.pos / p.page_size] : 0;
  finish_with(p, m, n, v, l);
}

// The same for outputs n .. n + 3 of row m (n % 4 == 0, p.vec4 holds); bias, position and page read by the caller.
__device__ __forceinline__ void finish4_with(const DecodeGemmArgs& p, int m, int n, float4 v, const float4& b, int pos,
                                             int page) {
  if (p.bias) v.x += b.x, v.y += b.y, v.z += b.z, v.w += b.w;
  if (p.flags & FLAG_GELU) v.x = gelu_tanh_fast(v.x), v.y = gelu_tanh_fast(v.y), v.z = gelu_tanh_fast(v.z), v.w = gelu_tanh_fast(v.w);
  uint2 packed;
  packed.x = pack2(v.x, v.y), packed.y = pack2(v.z, v.w);
  if ((p.flags & FLAG_KV) && n >= p.q_width) {
    const int c = n - p.q_width;
    const bool is_v = c >= p.kv_width;
    const int cc = is_v ? c - p.kv_width : c;
    const int head = cc / p.head_dim, d = cc - head * p.head_dim;
    const size_t dst = (size_t)page * p.page_stride +
                       ((size_t)head * p.page_size + pos % p.page_size) * p.head_dim + d;
    *(uint2*)((is_v ? p.v_pages : p.k_pages) + dst) = packed;
  } else {
    const size_t idx = (size_t)m * p.ldo + n;
    if (p.flags & FLAG_OUT_PACKED) {  // (four neighbouring columns from a multiple of four on stay together)
      *(uint2*)((uint16_t*)p.out + packed_at(m, n, p.out_kblocks)) = packed;
    } else if (p.flags & FLAG_ACCUMULATE) {
      float4* o = (float4*)((float*)p.out + idx);
      const float4 h = *o;
      *o = make_float4(h.x + v.x, h.y + v.y, h.z + v.z, h.w + v.w);
    } else if (p.flags & FLAG_OUT_F32) {
      *(float4*)((float*)p.out + idx) = v;
    } else {
      *(uint2*)((uint16_t*)p.out + idx) = packed;
    }
  }
}
__device__ __forceinline__ void finish4(const DecodeGemmArgs& p, int m, int n, float4 v) {
  const bool kv = (p.flags & FLAG_KV) && n >= p.q_width;
  const float4 b = p.bias ? *(const float4*)(p.bias + n) : make_float4(0.f, 0.f, 0.f, 0.f);
  const int pos = kv ? p.positions[m] : 0;
  const int page = kv ? p.block_table[(size_t)p.token_req[m] * p.max_blocks + pos / p.page_size] : 0;
  finish4_with(p, m, n, v, b, pos, page);
}

// LN: norm the rows of X in the prologue (K <= 2048: a lane holds its share of
// a row in NV float4).  MULTI: K is longer than one pass of NW * U k-blocks
// (2048); only then is the second set of weight registers needed.
template <bool LN, bool MULTI>
__global__ __launch_bounds__(NW * 64) void gemm_bf16_decode_kernel(DecodeGemmArgs p) {
  constexpr int NV = LN_MAX_V;
  constexpr int UU = MULTI ? 2 * U : U;  // k-blocks per pass and wave: long rows keep more in flight
  extern __shared__ __attribute__((aligned(16))) uint16_t As[];  // [M][a_stride]
  __shared__ float red[NW][256];
  __shared__ __attribute__((aligned(16))) float gb[LN ? 2 * LN_MAX_V * 256 : 4];  // norm scale, shift

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n0 = blockIdx.x * p.rows;
  const int koff = (lane >> 4) * 16;
  // lanes beyond the block's features (or the matrix) repeat its last row; their results are dropped
  const uint16_t* wrow = p.W + (size_t)min(n0 + min(lane & 15, p.rows - 1), p.N - 1) * p.ldw;
  // packed weights (ldw == 0): the 16 x 64 tile of block b and k-block c lies at
  // (b * n_chunks_all + c) * 1024 elements, first halves of the lanes' 16 values, then second halves
  const bool packed = p.ldw == 0;
  const int fpk = n0 + min(lane & 15, p.rows - 1);  // this lane's feature (inside the padded matrix)
  const uint16_t* wtile = p.W + (size_t)(fpk >> 4) * ((p.K + 63) / 64) * 1024 + ((lane & 48) | (fpk & 15)) * 8;
  const int n_chunks_all = (p.K + 63) / 64;
  const int c_begin = blockIdx.y * p.chunks_per_split;  // this split's k-blocks
  const int n_chunks = min(n_chunks_all, c_begin + p.chunks_per_split) - c_begin;
  const int kb = c_begin * 64;  // LDS holds the activations' columns from here on

  // Loads are never predicated on their address (a select between an address
  // and a dummy makes them flat loads, which also count as LDS traffic) and
  // weight fragments are not even zeroed when they lie outside the matrix:
  // every address is pulled into range, and what such a fragment meets is a
  // zero activation (k >= K) or an output that is never stored (n >= N).  So
  // nothing has to wait for a weight before the MFMA that uses it.  (Whole
  // k-blocks beyond the last are another matter: a wave skips them.)
  auto load_pass = [&](Frag (&w)[UU][2], int pass) {
    if (wave + NW * pass * UU >= n_chunks) return;  // the whole pass lies beyond K (uniform)
#pragma unroll
    for (int u = 0; u < UU; ++u) {
      // a wave's k-blocks beyond the last are not asked for: clamped to the last, seven of eight waves
      // asked for that one at once where K is 25 k-blocks (a decode step 0.5 to 1 % longer)
      if (wave + NW * (pass * UU + u) >= n_chunks) continue;
      const int c = c_begin + wave + NW * (pass * UU + u);
      const int k = c * 64 + koff;
      if (packed) {
        w[u][0].u = *(const uint4*)(wtile + (size_t)c * 1024);
        w[u][1].u = *(const uint4*)(wtile + (size_t)c * 1024 + 512);
      } else {
        w[u][0].u = *(const uint4*)(wrow + min(k, p.K - 8));
        w[u][1].u = *(const uint4*)(wrow + min(k + 8, p.K - 8));
      }
    }
  };

  Frag w0[UU][2], w1[MULTI ? UU : 1][2];

  // ---- activations into LDS ------------------------------------------------
  if constexpr (LN) {
    // Wave w norms rows w and w + 8.  Order of the loads: the first row and
    // this thread's share of scale and shift, then the weights, so that
    // waiting for the former leaves the weights in flight.
    float* gs = gb;
    float* bs = gb + LN_MAX_V * 256;
    for (int r = wave, first = 1; first || r < p.M; r += NW, first = 0) {
      const bool row_live = r < p.M;
      const float* x = p.X + (size_t)min(r, p.M - 1) * p.ldx;
      float4 v[NV];
      if (row_live) {  // (uniform over the wave; a wave without a row still shares in scale and shift below)
#pragma unroll
        for (int i = 0; i < NV; ++i) v[i] = *(const float4*)(x + min((lane + 64 * i) * 4, p.K - 4));
      } else {
#pragma unroll
        for (int i = 0; i < NV; ++i) v[i] = make_float4(0.f, 0.f, 0.f, 0.f);
      }
      float4 g4, b4;
      const int gk = min(tid * 4, p.K - 4);  // K / 4 <= 512 pieces: one a thread, surplus threads repeat the last
      if (first) {
        g4 = *(const float4*)(p.gamma + gk);
        b4 = *(const float4*)(p.beta + gk);
        asm volatile("" ::: "memory");  // keep the weights' loads behind these
        __builtin_amdgcn_sched_barrier(0);
        load_pass(w0, 0);
      }
      float s = 0.f;
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        if ((lane + 64 * i) * 4 >= p.K) v[i] = make_float4(0.f, 0.f, 0.f, 0.f);
        s += (v[i].x + v[i].y) + (v[i].z + v[i].w);
      }
      const float mean = wave_sum(s) / (float)p.K;
      float q = 0.f;
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        const bool in = (lane + 64 * i) * 4 < p.K;
        const float a = v[i].x - mean, b = v[i].y - mean, c = v[i].z - mean, d = v[i].w - mean;
        q += in ? (a * a + b * b) + (c * c + d * d) : 0.f;
      }
      const float rstd = 1.0f / sqrtf(wave_sum(q) / (float)p.K + p.eps);
      if (first) {  // every wave runs the first round
        *(float4*)(gs + gk) = g4, *(float4*)(bs + gk) = b4;
        __syncthreads();
      }
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        const int k = (lane + 64 * i) * 4;
        if (row_live && k < p.K) {
          const float4 g = *(const float4*)(gs + k), b = *(const float4*)(bs + k);
          uint2 o;
          o.x = pack2((v[i].x - mean) * rstd * g.x + b.x, (v[i].y - mean) * rstd * g.y + b.y);
          o.y = pack2((v[i].z - mean) * rstd * g.z + b.z, (v[i].w - mean) * rstd * g.w + b.w);
          *(uint2*)(As + r * p.a_stride + k) = o;
        }
      }
    }
  } else {
    load_pass(w0, 0);  // in flight while the activations are copied
    // four independent loads a thread and round: one trip to L2 instead of four in a row
    const int per_row = (min(p.K, kb + n_chunks * 64) - kb) / 8;
    const int total = p.M * per_row;
    for (int c0 = tid; c0 < total; c0 += 4 * NW * 64) {
      uint4 t[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int c = min(c0 + j * NW * 64, total - 1);
        const int r = c / per_row, k = (c - r * per_row) * 8;
        t[j] = *(const uint4*)(p.A + (size_t)r * p.lda + kb + k);
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int c = c0 + j * NW * 64;
        const int r = c / per_row, k = (c - r * per_row) * 8;
        if (c < total) *(uint4*)(As + r * p.a_stride + k) = t[j];
      }
    }
  }
  // What the epilogue takes from memory (the bias, and the stream's old value where the product
  // goes into the stream) is asked for now, without a condition: after the sum of the waves it
  // was one more trip to memory at the kernel's end (a decode step of twelve layers at batch 1 /
  // 8 / 16: 0.520 / 0.590 / 0.743 ms before, 0.504 / 0.581 / 0.730 after).  (Element t = 4 L + r of
  // the tile: feature 4 (L / 16) + r, row L % 16; indices beyond the matrix are pulled inside, a
  // pointer that is not there points at the weights.)  A key's or value's position and page are
  // still looked up at the end: asked for here, by every block of the fused q/k/v product, they
  // cost that product 1 % more than they saved.
  const int e_t = tid & 255, e_l = e_t >> 2;
  const int e_n = min(n0 + 4 * (e_l >> 4) + (e_t & 3), p.N - 1), e_m = min(e_l & 15, p.M - 1);
  const bool e_adds = (p.flags & FLAG_ACCUMULATE) && p.n_splits == 1 && !(p.flags & FLAG_OUT_PACKED);
  FinishLoads early;
  early.bias = *(p.bias ? p.bias + e_n : (const float*)p.W);
  early.old = *(e_adds ? (const float*)p.out + (size_t)e_m * p.ldo + e_n : (const float*)p.W);
  early.pos = early.page = 0;
  __syncthreads();

  // ---- main loop: two passes of loads ahead of the MFMAs --------------------
  f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
  const bool avalid = (lane & 15) < p.M;
  const uint16_t* arow = As + min(lane & 15, p.M - 1) * p.a_stride;

  auto compute_pass = [&](Frag (&w)[UU][2], int pass) {
#pragma unroll
    for (int u = 0; u < UU; ++u) {
      const int c = wave + NW * (pass * UU + u);
      if (c < n_chunks) {  // uniform over the wave
        const int k = kb + c * 64 + koff;
        Frag a0, a1;
        const uint4 t0 = *(const uint4*)(arow + min(k, p.K - 8) - kb);
        const uint4 t1 = *(const uint4*)(arow + min(k + 8, p.K - 8) - kb);
        a0.u = (avalid && k < p.K) ? t0 : ZERO4;
        a1.u = (avalid && k + 8 < p.K) ? t1 : ZERO4;
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[u][0].v, a0.v, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[u][1].v, a1.v, acc, 0, 0, 0);
      }
    }
  };

  if constexpr (MULTI) {
    const int n_pass = (n_chunks + NW * UU - 1) / (NW * UU);
    for (int pass = 0; pass < n_pass; pass += 2) {
      load_pass(w1, pass + 1);
      compute_pass(w0, pass);
      load_pass(w0, pass + 2);
      compute_pass(w1, pass + 1);
    }
  } else {
    compute_pass(w0, 0);
  }

  // ---- sum the waves' tiles in a fixed order, then the epilogue ---------------
#pragma unroll
  for (int r = 0; r < 4; ++r) red[wave][lane * 4 + r] = acc[r];
  __syncthreads();
  float v = 0.f;
  if (tid < 256) {
#pragma unroll
    for (int w = 0; w < NW; ++w) v += red[w][tid];
  }
  if (tid < 256) {
    // element tid = 4 * L + r of the MFMA tile: feature 4 * (L / 16) + r, row L % 16
    const int L = tid >> 2, r = tid & 3;
    const int f = 4 * (L >> 4) + r;
    const int n = n0 + f;
    const int m = L & 15;
    if (m < p.M && f < p.rows && n < p.N) {
      if (p.n_splits > 1)
        p.ws[((size_t)blockIdx.y * p.M + m) * p.N + n] = v;  // summed, and finished, by sum_partials
      else if ((p.flags & FLAG_KV) && n >= p.q_width)
        finish(p, m, n, v);
      else
        finish_with(p, m, n, v, early);  // (m, n are e_m, e_n here)
    }
  }
}

// ---------------------------------------------------------------------------
// 17 to 64 rows.  The weights still stream exactly once and all of a block's are in flight from
// its first instruction on: a block of four waves owns 32 output features (two packed chunks)
// and a slice of K of at most 28 k-blocks; wave w takes the slice's k-blocks w, w + 4, ... and
// holds their weights in registers (seven k-blocks of two chunks: 112 registers a lane).  The
// activations are the MFMA's other operand, two or three tiles of 16 rows, read straight from
// memory (the L2s: every block reads the same rows) a k-block ahead; no LDS on the way.  They
// come row-major or, much faster, in the packed order (packed_at: a wave's load is then 1 KB of
// consecutive bytes instead of sixteen pieces of 64: GPT-2 XL's four products at 48 rows took
// 15.8 / 17.3 / 12.8 / 17.0 us from rows and 10.8 / 12.4 / 8.0 / 11.8 packed), which the kernels
// that make these rows write where the host asks them to (the sum-and-norm, decode attention,
// this kernel's own epilogue).  The four waves' tiles are summed in their order through LDS and
// finished as in the kernel above.  The tile kernels of gemm_bf16.hip need K split over some 220
// blocks at these sizes and a second kernel for the sum; here the wide products are one launch of
// 150 or 200 blocks, and the narrow ones split K in two or four.  49 to 64 rows go as two groups
// of two tiles, a block each, eight block ids apart: both on one die, so that the second finds
// the weights in that die's L2 (the fetch counter shows them read from memory once).
// (Other shapes measured at 64 rows of GPT-2 XL's sizes, packed rows, a decode step of twelve
// layers: four tiles a block with 32 features and four or eight waves 1.34 and 1.29 ms, with 16
// features 1.58, sixteen waves that hold everything after one trip to memory 1.65; two groups
// 1.28; the tile kernels with K split and their second kernels 1.33.)
#define RW 4          // waves a block
#define R_FEATURES 32 // output features a block
#define R_HELD 7      // k-blocks whose weights a wave holds
#define ROWS_MAX_M 64
#define ROWS_GROUP_FROM 49    // from this many rows on: groups of 32 rows, a block each
#define ROWS_WANT_BLOCKS 100  // a split of K where the features give fewer blocks than this
// R_TILES: tiles of 16 rows; FT: chunks of 16 features a block; WAVES: waves a block; HELD: k-blocks a wave holds
template <int R_TILES, int FT, int WAVES, int HELD>
__global__ __launch_bounds__(WAVES * 64) void gemm_bf16_rows_kernel(DecodeGemmArgs p) {
  __shared__ float red[WAVES][R_TILES * FT][256];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  // Blocks go to the dies in turn (block b to die b % 8).  The groups of rows that meet the same
  // weights are eight block ids apart: on one die, one after the other, so that only the first
  // fetches the weights from memory and the others find them in the die's L2.
  const int within = blockIdx.x % (8 * p.row_groups);
  const int group = within >> 3;
  const int n0 = ((blockIdx.x / (8 * p.row_groups)) * 8 + (within & 7)) * (16 * FT);
  const int t0 = group * R_TILES;  // this block's first tile of rows
  if (n0 >= p.N) return;           // (the grid is padded to whole eights of feature blocks)
  const int n_chunks_all = (p.K + 63) / 64;
  const int c_begin = blockIdx.y * p.chunks_per_split;
  const int n_chunks = min(n_chunks_all, c_begin + p.chunks_per_split) - c_begin;
  const int n_fb = (p.N + 15) / 16;
  const int koff = (lane >> 4) * 16;

  // the weights, all at once (k-blocks beyond the slice repeat its last one and are not used)
  Frag w[HELD][FT][2];
#pragma unroll
  for (int i = 0; i < HELD; ++i) {
    const int c = c_begin + min(wave + WAVES * i, n_chunks - 1);
#pragma unroll
    for (int ft = 0; ft < FT; ++ft) {
      const int fb = min((n0 >> 4) + ft, n_fb - 1);  // (a second chunk beyond the matrix repeats the first)
      const uint16_t* t = p.W + ((size_t)fb * n_chunks_all + c) * 1024 + lane * 8;
      w[i][ft][0].u = *(const uint4*)t;
      w[i][ft][1].u = *(const uint4*)(t + 512);
    }
  }
  // the activations of a k-block: lane l holds row l % 16 of each tile, 16 columns from
  // (l / 16) * 16 on (rows beyond M repeat the last; what they give is not stored)
  const uint16_t* arow[R_TILES];
#pragma unroll
  for (int rt = 0; rt < R_TILES; ++rt) arow[rt] = p.A + (size_t)min((t0 + rt) * 16 + (lane & 15), p.M - 1) * p.lda;
  const int m_tiles = (p.M + 15) / 16;
  auto load_a = [&](Frag (&a)[R_TILES][2], int i) {
    const int c = c_begin + min(wave + WAVES * i, n_chunks - 1);
    const int k = c * 64 + koff;
    if (p.a_packed) {
#pragma unroll
      for (int rt = 0; rt < R_TILES; ++rt) {
        const uint16_t* t = p.A + ((size_t)min(t0 + rt, m_tiles - 1) * n_chunks_all + c) * 1024 + lane * 8;
        a[rt][0].u = *(const uint4*)t;
        a[rt][1].u = *(const uint4*)(t + 512);
      }
    } else {
#pragma unroll
      for (int rt = 0; rt < R_TILES; ++rt) {
        a[rt][0].u = *(const uint4*)(arow[rt] + min(k, p.K - 8));
        a[rt][1].u = *(const uint4*)(arow[rt] + min(k + 8, p.K - 8));
      }
    }
  };
  f32x4_t acc[R_TILES][FT];
#pragma unroll
  for (int rt = 0; rt < R_TILES; ++rt)
#pragma unroll
    for (int ft = 0; ft < FT; ++ft) acc[rt][ft] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  auto multiply = [&](Frag (&a)[R_TILES][2], int i) {
    if (wave + WAVES * i >= n_chunks) return;  // (uniform over the wave)
    const int k = (c_begin + wave + WAVES * i) * 64 + koff;
    // columns beyond K meet zero weights (the packed order pads them), but must not be NaN
    const bool in0 = k < p.K, in1 = k + 8 < p.K;
#pragma unroll
    for (int rt = 0; rt < R_TILES; ++rt) {
      Frag a0, a1;
      a0.u = in0 ? a[rt][0].u : ZERO4, a1.u = in1 ? a[rt][1].u : ZERO4;
#pragma unroll
      for (int ft = 0; ft < FT; ++ft) {
        acc[rt][ft] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[i][ft][0].v, a0.v, acc[rt][ft], 0, 0, 0);
        acc[rt][ft] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[i][ft][1].v, a1.v, acc[rt][ft], 0, 0, 0);
      }
    }
  };
  // What the epilogue takes from memory for the tiles that this wave will finish (the bias; a
  // key's or value's position and page) is asked for now, without a condition: after the sum
  // of the waves these were two more trips to memory at the kernel's end (a decode step of
  // twelve layers at batch 32: 0.902 ms with the lookups at the end, 0.893 with them here).
  constexpr int MY_TILES = (R_TILES * FT + WAVES - 1) / WAVES;
  float4 e_bias[MY_TILES];
  int e_pos[MY_TILES], e_page[MY_TILES];
  {
    const bool vec = p.vec4 && p.n_splits == 1, kv = (p.flags & FLAG_KV) && vec;
    const int* const some_ints = (const int*)p.W;
#pragma unroll
    for (int k = 0; k < MY_TILES; ++k) {
      const int t = min(wave + k * WAVES, R_TILES * FT - 1);
      const int rt = t / FT, ft = t - rt * FT;
      const int n = min(n0 + ft * 16 + 4 * (lane >> 4), max(p.N - 4, 0));
      const int m = min((t0 + rt) * 16 + (lane & 15), p.M - 1);
      e_bias[k] = *(const float4*)(vec && p.bias ? p.bias + n : (const float*)p.W);
      e_pos[k] = (kv ? p.positions : some_ints)[kv ? m : 0];
      const int req = (kv ? p.token_req : some_ints)[kv ? m : 0];
      e_page[k] = (kv ? p.block_table : some_ints)[kv ? (size_t)req * p.max_blocks + e_pos[k] / p.page_size : 0];
    }
  }
  Frag a0[R_TILES][2], a1[R_TILES][2];
  load_a(a0, 0);
#pragma unroll
  for (int i = 0; i < HELD; i += 2) {
    if (i + 1 < HELD) load_a(a1, i + 1);
    multiply(a0, i);
    if (i + 2 < HELD) load_a(a0, i + 2);
    if (i + 1 < HELD) multiply(a1, i + 1);
  }

  // ---- sum the waves' tiles in their order, then the epilogue -----------------
#pragma unroll
  for (int rt = 0; rt < R_TILES; ++rt)
#pragma unroll
    for (int ft = 0; ft < FT; ++ft)
#pragma unroll
      for (int r = 0; r < 4; ++r) red[wave][rt * FT + ft][lane * 4 + r] = acc[rt][ft][r];
  __syncthreads();
  // elements 4 * L .. 4 * L + 3 of a tile: features 4 * (L / 16) + 0..3 of row L % 16; a wave a tile
  const int L = lane;
#pragma unroll
  for (int k = 0; k < MY_TILES; ++k) {
    const int t = wave + k * WAVES;
    if (t >= R_TILES * FT) break;
    const int rt = t / FT, ft = t - rt * FT;
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int wv = 0; wv < WAVES; ++wv) {
      const float4 x = *(const float4*)&red[wv][t][4 * L];
      v.x += x.x, v.y += x.y, v.z += x.z, v.w += x.w;
    }
    const int n = n0 + ft * 16 + 4 * (L >> 4);
    const int m = (t0 + rt) * 16 + (L & 15);
    if (m >= p.M || n >= p.N) continue;
    const float vs[4] = {v.x, v.y, v.z, v.w};
    if (p.n_splits > 1) {  // summed, and finished, by sum_partials
      float* dst = p.ws + ((size_t)blockIdx.y * p.M + m) * p.N + n;
      if ((p.N & 3) == 0) {
        *(float4*)dst = v;
      } else {
        for (int j = 0; j < 4 && n + j < p.N; ++j) dst[j] = vs[j];
      }
    } else if (p.vec4) {
      finish4_with(p, m, n, v, e_bias[k], e_pos[k], e_page[k]);  // (read for this m and n above)
    } else {
      for (int j = 0; j < 4 && n + j < p.N; ++j) finish(p, m, n + j, vs[j]);
    }
  }
}

// ---------------------------------------------------------------------------
// The second step of a split product: out = epilogue(sum over splits, in their order).
__global__ __launch_bounds__(256) void sum_partials_kernel(DecodeGemmArgs p) {
  const int n4 = (p.N + 3) / 4;
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= p.M * n4) return;
  const int m = i / n4, n = (i - m * n4) * 4;
  const float* src = p.ws + (size_t)m * p.N + n;
  const size_t step = (size_t)p.M * p.N;
  if (p.vec4) {
    // four splits' loads at a time, none waiting for another (surplus ones repeat the last and are dropped)
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int s0 = 0; s0 < p.n_splits; s0 += 4) {
      float4 t[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) t[j] = *(const float4*)(src + min(s0 + j, p.n_splits - 1) * step);
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (s0 + j < p.n_splits) v.x += t[j].x, v.y += t[j].y, v.z += t[j].z, v.w += t[j].w;
    }
    finish4(p, m, n, v);
  } else {
    for (int j = 0; j < 4 && n + j < p.N; ++j) {
      float v = src[j];
      for (int s = 1; s < p.n_splits; ++s) v += src[s * step + j];
      finish(p, m, n + j, v);
    }
  }
}

// The second step for the residual stream, with the norm that follows it:
//   h[m] += bias + sum over splits;  out[m] = LayerNorm(h[m]) * gamma + beta
// One block a row, the row in registers (NV4 float4 a thread); N % 4 == 0.
struct SumNormArgs {
  float* h;
  const float* ws;
  const float* bias;
  const float* gamma;
  const float* beta;
  void* out;
  float eps;
  int M, N, ldh, n_splits, out_dtype;
  int out_packed;  // out (bfloat16) in the packed order of packed_at, for a product that takes its rows so
  // Blocks beyond the M rows read `ahead` (16-byte pieces) and drop it: the weights of the
  // product that comes next, which then finds them in the caches.  A row a block leaves nearly
  // every CU idle, and so does the memory.
  const uint4* ahead;
  size_t ahead_pieces;  // in a chunk
  int ahead_chunks;
};

template <int NV4>
__global__ __launch_bounds__(256) void sum_partials_norm_kernel(SumNormArgs q) {
  __shared__ float red[32];
  const int m = blockIdx.x, tid = threadIdx.x;
  if (m >= q.M) {  // (uniform over the block)
    // Block b of a launch runs on die b % 8, and so will block j of the product that comes next,
    // which reads chunk j of `ahead` (`ahead_pieces` pieces each): this block reads chunks of its
    // own die, so that they lie in the L2 where they will be asked for.
    const int die = blockIdx.x & 7, rank = (m - q.M) >> 3, per_die = max(1, (int)(gridDim.x - q.M) >> 3);
    // the die's chunks (die, die + 8, ...) laid end to end and cut into equal shares, one a block
    const size_t mine = die < q.ahead_chunks ? (size_t)((q.ahead_chunks - die + 7) / 8) * q.ahead_pieces : 0;
    const size_t share = (mine + per_die - 1) / per_die;
    const size_t lo = (size_t)rank * share, hi = min(lo + share, mine);
    unsigned int seen = 0u;
    // (sixteen loads a thread in flight: a share of some 60 KB in one trip)
    for (size_t i0 = lo + tid; i0 < hi; i0 += 16 * 256) {
      uint4 v[16];
#pragma unroll
      for (int u = 0; u < 16; ++u) {
        const size_t t = min(i0 + u * 256, hi - 1);
        const size_t c = t / q.ahead_pieces;
        v[u] = q.ahead[((size_t)die + 8 * c) * q.ahead_pieces + (t - c * q.ahead_pieces)];
      }
#pragma unroll
      for (int u = 0; u < 16; ++u) seen |= v[u].x;
    }
    asm volatile("" ::"v"(seen));  // the loads stay although nobody wants the values
    return;
  }
  float* hrow = q.h + (size_t)m * q.ldh;
  const size_t step = (size_t)q.M * q.N;
  const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f), one = make_float4(1.f, 1.f, 1.f, 1.f);
  // Few blocks, little data: what counts is how many trips to memory follow
  // one another.  Everything the row needs is asked for at once.
  float4 v[NV4], bias[NV4], g[NV4], b[NV4];
#pragma unroll
  for (int i = 0; i < NV4; ++i) {
    const int k = min((tid + 256 * i) * 4, q.N - 4);
    v[i] = *(const float4*)(hrow + k);
    bias[i] = q.bias ? *(const float4*)(q.bias + k) : zero;
    g[i] = q.gamma ? *(const float4*)(q.gamma + k) : one;
    b[i] = q.beta ? *(const float4*)(q.beta + k) : zero;
  }
  float4 part[NV4];
#pragma unroll
  for (int i = 0; i < NV4; ++i) part[i] = zero;
  for (int s0 = 0; s0 < q.n_splits; s0 += 4) {
    float4 t[NV4][4];
#pragma unroll
    for (int i = 0; i < NV4; ++i) {
      const float* src = q.ws + (size_t)m * q.N + min((tid + 256 * i) * 4, q.N - 4);
#pragma unroll
      for (int j = 0; j < 4; ++j) t[i][j] = *(const float4*)(src + min(s0 + j, q.n_splits - 1) * step);
    }
#pragma unroll
    for (int i = 0; i < NV4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (s0 + j < q.n_splits)
          part[i].x += t[i][j].x, part[i].y += t[i][j].y, part[i].z += t[i][j].z, part[i].w += t[i][j].w;
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < NV4; ++i) {
    const int k = (tid + 256 * i) * 4;
    v[i].x += bias[i].x + part[i].x, v[i].y += bias[i].y + part[i].y;
    v[i].z += bias[i].z + part[i].z, v[i].w += bias[i].w + part[i].w;
    if (k < q.N) {
      *(float4*)(hrow + k) = v[i];
      s += (v[i].x + v[i].y) + (v[i].z + v[i].w);
    }
  }
  const float mean = block_sum(s, red) / (float)q.N;
  float qq = 0.f;
#pragma unroll
  for (int i = 0; i < NV4; ++i) {
    if ((tid + 256 * i) * 4 < q.N) {
      const float a = v[i].x - mean, bb = v[i].y - mean, c = v[i].z - mean, d = v[i].w - mean;
      qq += (a * a + bb * bb) + (c * c + d * d);
    }
  }
  const float rstd = 1.0f / sqrtf(block_sum(qq, red) / (float)q.N + q.eps);
#pragma unroll
  for (int i = 0; i < NV4; ++i) {
    const int k = (tid + 256 * i) * 4;
    if (k >= q.N) continue;
    const float y0 = (v[i].x - mean) * rstd * g[i].x + b[i].x, y1 = (v[i].y - mean) * rstd * g[i].y + b[i].y;
    const float y2 = (v[i].z - mean) * rstd * g[i].z + b[i].z, y3 = (v[i].w - mean) * rstd * g[i].w + b[i].w;
    if (q.out_dtype == DT_F32) {
      *(float4*)((float*)q.out + (size_t)m * q.N + k) = make_float4(y0, y1, y2, y3);
    } else {
      uint2 o;
      o.x = pack2(y0, y1), o.y = pack2(y2, y3);
      *(uint2*)((uint16_t*)q.out + (q.out_packed ? packed_at(m, k, (q.N + 63) / 64) : (size_t)m * q.N + k)) = o;
    }
  }
}

DEFINE_LAST_ERROR(mlxlm_last_error)

#define MAX_LDS_BYTES (120 * 1024)
// Fewer blocks of 16 features than this leave many CUs idle: 75/128 of the device's CUs
// (150 of 256).  The thresholds below are fractions of the CU count and a time, not sizes: they
// were measured at widths 768 to 2,048 on 256 CUs and move with the device, not with one model.
static int few_blocks() { return n_compute_units() * 75 / 128; }
extern "C" int gemm_bf16_decode_few_blocks(void) { return few_blocks(); }
// A CU draws some 30 GB/s of a matrix that comes from memory; a second kernel costs some 5 us.
#define CU_STREAM_BYTES_PER_US 30000.0
#define SECOND_KERNEL_US 1.3  // a matrix that streams in less than this gains nothing from a split

// LDS row stride: rows of 16-byte reads from 16 lanes must fall on distinct
// banks, which holds when the stride in 32-bit words is 4 mod 32.
static int a_stride_for(int K) { return K + ((8 - K % 64) + 64) % 64; }

static int chunks_per_split(int K, int n_splits) { return ((K + 63) / 64 + n_splits - 1) / n_splits; }

// 1 if gemm_bf16_decode takes these sizes (the caller falls back otherwise)
extern "C" int gemm_bf16_decode_takes(int M, int K, int with_norm, int n_splits) {
  if (M < 1 || M > 16 || K < 8 || K % 8 != 0 || n_splits < 1 || n_splits > (K + 63) / 64) return 0;
  if (with_norm && (n_splits != 1 || K > LN_MAX_V * 256 || K > NW * U * 64 || K % 4 != 0)) return 0;
  const int range = K < chunks_per_split(K, n_splits) * 64 ? K : chunks_per_split(K, n_splits) * 64;
  return (size_t)M * a_stride_for(range) * 2 <= MAX_LDS_BYTES;
}

// Into how many parts to split K so that the launch fills the GPU (1: no
// split, the product's kernel runs the epilogue itself).  `force` > 0 asks for
// that many wherever a split is possible at all (for tests of small sizes).
extern "C" int gemm_bf16_decode_splits(int M, int N, int K, int with_norm, int force) {
  const int n_chunks = (K + 63) / 64;
  if (with_norm || M < 1 || M > 16) return 1;
  int want;
  if (force > 0) {
    want = force;
  } else {
    const int n_blocks = (N + 15) / 16;
    // enough blocks as it is (four fifths of the CUs; 200 of 256), or one to three rows: the next
    // projection's norm prologue is cheaper than a second kernel
    if (n_blocks >= n_compute_units() * 4 / 5 || M < 4) return 1;
    // a small matrix streams in less time than the second kernel costs (measured at N = 1600:
    // K = 1600, 5 MB, loses 2 us by the split; K = 6400, 20 MB, gains 4)
    if (2.0 * N * K / (CU_STREAM_BYTES_PER_US * n_compute_units()) < SECOND_KERNEL_US) return 1;
    // one and a half blocks a CU (N = 1600, K = 6400: four parts; with six, two blocks a CU, a decode step of
    // GPT-2 XL's sizes at batch 8 took 2.25 ms instead of 2.22, the parts' sum being read by the next kernel;
    // three parts are more k-blocks than a wave holds at once, 2.41 ms)
    want = (3 * n_compute_units() / 2 + n_blocks - 1) / n_blocks;
    if (want > n_chunks / 4) want = n_chunks / 4;  // at least four k-blocks a split
  }
  if (want < 1) want = 1;
  if (want > n_chunks) want = n_chunks;
  const int cps = (n_chunks + want - 1) / want;
  return (n_chunks + cps - 1) / cps;  // no empty split
}

static bool aligned16(const void* q) { return ((uintptr_t)q & 15) == 0; }

// Checks and fields that the product and sum_partials share.  Returns 0 or -1.
static int fill_epilogue(DecodeGemmArgs& p, const char* who, void* out, const float* bias, int M, int N,
                         int ldo, int flags, void* k_pages, void* v_pages, size_t page_stride,
                         const int* block_table, int max_blocks, const int* token_req,
                         const int* positions, int q_width, int kv_width, int head_dim, int page_size) {
  if (N <= 0) FAIL("%s: bad N=%d", who, N);
  if (!out) FAIL("%s: null pointer", who);
  if ((flags & FLAG_ACCUMULATE) && (flags & (FLAG_GELU | FLAG_KV)))
    FAIL("%s: accumulate cannot be combined with GELU or the cache scatter", who);
  if ((flags & FLAG_OUT_PACKED) && (flags & (FLAG_ACCUMULATE | FLAG_OUT_F32 | FLAG_KV)))
    FAIL("%s: the packed order is for a bfloat16 out that is neither added to nor scattered", who);
  if (flags & FLAG_KV) {
    if (!k_pages || !v_pages || !block_table || !token_req || !positions)
      FAIL("%s: the cache scatter needs pages, block table, token_req and positions", who);
    if (head_dim <= 0 || page_size <= 0 || kv_width % head_dim != 0 || q_width + 2 * kv_width != N)
      FAIL("%s: q_width %d + 2 * kv_width %d must be N=%d, kv_width a multiple of head_dim %d", who,
           q_width, kv_width, N, head_dim);
    if (flags & (FLAG_OUT_F32 | FLAG_GELU)) FAIL("%s: the cache scatter writes bfloat16, no GELU", who);
    if (ldo < q_width) FAIL("%s: ldo=%d smaller than q_width=%d", who, ldo, q_width);
  } else if (ldo < N && !(flags & FLAG_OUT_PACKED)) {
    FAIL("%s: ldo=%d smaller than N=%d", who, ldo, N);
  }
  p.bias = bias, p.out = out, p.M = M, p.N = N, p.ldo = ldo, p.flags = flags;
  p.k_pages = (uint16_t*)k_pages, p.v_pages = (uint16_t*)v_pages, p.page_stride = page_stride;
  p.block_table = block_table, p.token_req = token_req, p.positions = positions;
  p.max_blocks = max_blocks, p.q_width = q_width, p.kv_width = kv_width;
  p.head_dim = head_dim, p.page_size = page_size;
  p.out_kblocks = (N + 63) / 64;
  p.vec4 = N % 4 == 0 && ldo % 4 == 0 && aligned16(out) && aligned16(bias);
  if (flags & FLAG_KV)
    p.vec4 = p.vec4 && q_width % 4 == 0 && kv_width % 4 == 0 && head_dim % 4 == 0 && page_stride % 4 == 0 &&
             aligned16(k_pages) && aligned16(v_pages);
  return 0;
}

// With n_splits > 1 the epilogue does not run: the partial sums go to `ws`
// ([n_splits][M][N] floats) and sum_partials or sum_partials_norm finishes.
extern "C" int gemm_bf16_decode(
    void* out, const void* A, int lda, const float* X, int ldx, const float* gamma,
    const float* beta, float eps, const void* W, const float* bias, int M, int N, int K, int ldw,
    int ldo, int flags, void* k_pages, void* v_pages, size_t page_stride, const int* block_table,
    int max_blocks, const int* token_req, const int* positions, int q_width, int kv_width,
    int head_dim, int page_size, int n_splits, float* ws, size_t ws_floats, hipStream_t stream) {
  if (M == 0) return 0;
  const bool ln = X != nullptr;
  if (!gemm_bf16_decode_takes(M, K, ln, n_splits))
    FAIL("gemm_bf16_decode: M=%d K=%d%s in %d splits is outside what this kernel takes", M, K,
         ln ? " with norm" : "", n_splits);
  if ((A == nullptr) == (X == nullptr)) FAIL("gemm_bf16_decode: give activations or a residual stream to norm");
  if (!W) FAIL("gemm_bf16_decode: null pointer");
  // ldw == 0: W is packed (tiles of 16 features x 64 k, zero padded)
  if (ldw != 0 && (ldw % 8 != 0 || ldw < K)) FAIL("gemm_bf16_decode: W rows must be 16-byte aligned");
  if (!aligned16(W)) FAIL("gemm_bf16_decode: W must be 16-byte aligned");
  if (A && (lda % 8 != 0 || lda < K || !aligned16(A))) FAIL("gemm_bf16_decode: A rows must be 16-byte aligned");
  if (X && (ldx % 4 != 0 || ldx < K || !aligned16(X))) FAIL("gemm_bf16_decode: X rows must be 16-byte aligned");
  if (X && (!gamma || !beta || !aligned16(gamma) || !aligned16(beta)))
    FAIL("gemm_bf16_decode: the norm needs scale and shift, 16-byte aligned");
  DecodeGemmArgs p;
  if (fill_epilogue(p, "gemm_bf16_decode", out, bias, M, N, ldo, flags, k_pages, v_pages, page_stride,
                    block_table, max_blocks, token_req, positions, q_width, kv_width, head_dim, page_size))
    return -1;
  p.W = (const uint16_t*)W, p.A = (const uint16_t*)A, p.X = X;
  p.gamma = gamma, p.beta = beta, p.eps = eps;
  p.K = K, p.lda = lda, p.ldx = ldx, p.ldw = ldw;
  // Few features and no split of K: blocks of eight features (half of each MFMA
  // tile is idle, which costs nothing here) put twice as many CUs to work.
  p.rows = (n_splits == 1 && (N + 15) / 16 < few_blocks()) ? 8 : 16;
  p.n_splits = n_splits, p.chunks_per_split = chunks_per_split(K, n_splits);
  p.ws = ws;
  if (n_splits > 1) {
    if (!ws || !aligned16(ws)) FAIL("gemm_bf16_decode: a split of K needs a 16-byte aligned workspace");
    if (ws_floats < (size_t)n_splits * M * N)
      FAIL("gemm_bf16_decode: workspace of %zu floats is too small for %d splits of %d x %d", ws_floats,
           n_splits, M, N);
    if ((p.chunks_per_split * (n_splits - 1)) >= (K + 63) / 64)
      FAIL("gemm_bf16_decode: %d splits of K=%d leave one empty", n_splits, K);
  }
  const int n_blocks = (N + p.rows - 1) / p.rows;
  const int range = K < p.chunks_per_split * 64 ? K : p.chunks_per_split * 64;
  p.a_stride = a_stride_for(range);
  const size_t lds = (size_t)M * p.a_stride * 2;
  const bool multi = p.chunks_per_split > NW * U;
  const int which = ln ? 2 : (multi ? 1 : 0);
  void (*kernels[3])(DecodeGemmArgs) = {gemm_bf16_decode_kernel<false, false>,
                                        gemm_bf16_decode_kernel<false, true>,
                                        gemm_bf16_decode_kernel<true, false>};
  static size_t granted[3] = {0, 0, 0};
  const size_t fixed = sizeof(float) * (NW * 256 + (ln ? 2 * LN_MAX_V * 256 : 4));
  if (lds + fixed > 64 * 1024 && granted[which] < lds) {
    hipError_t e = hipFuncSetAttribute((const void*)kernels[which],
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) FAIL("gemm_bf16_decode: cannot get %zu bytes of LDS: %s", lds, hipGetErrorString(e));
    granted[which] = lds;
  }
  hipLaunchKernelGGL(kernels[which], dim3(n_blocks, n_splits), dim3(NW * 64), lds, stream, p);
  CHECK_LAUNCH("gemm_bf16_decode");
  return 0;
}

// 1 if gemm_bf16_rows takes these sizes
extern "C" int gemm_bf16_rows_takes(int M, int K, int n_splits) {
  if (M < 17 || M > ROWS_MAX_M || K < 8 || K % 8 != 0 || n_splits < 1 || n_splits > (K + 63) / 64) return 0;
  const int cps = chunks_per_split(K, n_splits);
  return cps <= RW * R_HELD && cps * (n_splits - 1) < (K + 63) / 64;
}

// Into how many parts gemm_bf16_rows splits K: as few as give some ROWS_WANT_BLOCKS blocks of 32 features and
// slices of at most 28 k-blocks (0: the sizes do not fit, for the workspace's room or otherwise).
// `force` > 0 asks for that many wherever K has them (for tests of small sizes).
extern "C" int gemm_bf16_rows_splits(int M, int N, int K, int force) {
  const int n_chunks = (K + 63) / 64;
  if (M < 17 || M > ROWS_MAX_M || K % 8 != 0) return 0;
  const int blocks = (N + R_FEATURES - 1) / R_FEATURES;
  int want = force > 0 ? force : (ROWS_WANT_BLOCKS + blocks - 1) / blocks;
  const int least = (n_chunks + RW * R_HELD - 1) / (RW * R_HELD);
  if (want < least) want = least;
  if (want > n_chunks) want = n_chunks;
  if (force <= 0 && want > least && n_chunks / want < 4) want = n_chunks / 4 > least ? n_chunks / 4 : least;  // four k-blocks a part
  const int cps = (n_chunks + want - 1) / want;
  const int n = (n_chunks + cps - 1) / cps;  // no empty part
  return gemm_bf16_rows_takes(M, K, n) ? n : 0;
}

// The product for 17 to 64 rows (see gemm_bf16_rows_kernel): W in the packed order only; A
// row-major, or with lda == 0 in the packed order of packed_at ([M, K] in tiles of 16 rows x 64
// columns; what lies beyond row M or column K is never used and need not be written).  Flag 16
// (with a bfloat16 out, no accumulate, no scatter) writes out in that order too, for the product
// that reads it next; ldo is not used then.  With n_splits > 1 the partial sums go to `ws` and
// sum_partials or sum_partials_norm finishes.
extern "C" int gemm_bf16_rows(void* out, const void* A, int lda, const void* W, const float* bias, int M,
                              int N, int K, int ldo, int flags, void* k_pages, void* v_pages,
                              size_t page_stride, const int* block_table, int max_blocks,
                              const int* token_req, const int* positions, int q_width, int kv_width,
                              int head_dim, int page_size, int n_splits, float* ws, size_t ws_floats,
                              hipStream_t stream) {
  if (M == 0) return 0;
  if (!gemm_bf16_rows_takes(M, K, n_splits))
    FAIL("gemm_bf16_rows: M=%d K=%d in %d splits is outside what this kernel takes", M, K, n_splits);
  if (!A || !W) FAIL("gemm_bf16_rows: null pointer");
  if (!aligned16(W)) FAIL("gemm_bf16_rows: W must be 16-byte aligned");
  if (lda != 0 && (lda % 8 != 0 || lda < K)) FAIL("gemm_bf16_rows: A rows must be 16-byte aligned");
  if (!aligned16(A)) FAIL("gemm_bf16_rows: A must be 16-byte aligned");
  DecodeGemmArgs p = {};
  if (fill_epilogue(p, "gemm_bf16_rows", out, bias, M, N, ldo, flags, k_pages, v_pages, page_stride,
                    block_table, max_blocks, token_req, positions, q_width, kv_width, head_dim, page_size))
    return -1;
  p.W = (const uint16_t*)W, p.A = (const uint16_t*)A;
  p.K = K, p.lda = lda, p.ldw = 0;
  p.a_packed = lda == 0;
  p.n_splits = n_splits, p.chunks_per_split = chunks_per_split(K, n_splits);
  p.ws = ws;
  if (n_splits > 1) {
    if (!ws || !aligned16(ws)) FAIL("gemm_bf16_rows: a split of K needs a 16-byte aligned workspace");
    if (ws_floats < (size_t)n_splits * M * N)
      FAIL("gemm_bf16_rows: workspace of %zu floats is too small for %d splits of %d x %d", ws_floats, n_splits, M, N);
  }
  p.row_groups = M >= ROWS_GROUP_FROM ? (M + 31) / 32 : 1;
  // (the grid holds whole eights of feature blocks, so that a group's blocks and the next group's
  // are on the same dies; the surplus blocks return at once)
  const int fbs = ((N + R_FEATURES - 1) / R_FEATURES + 7) / 8 * 8;
  const dim3 grid(fbs * p.row_groups, n_splits), block(RW * 64);
  // (eight waves of four k-blocks each where a block takes all the rows: a wave's trips to the L2s for
  // its rows follow one another, and four are fewer than seven; a decode step of GPT-2 XL's sizes
  // at 32 and at 48 rows 2 and 4 % shorter, with the groups of 49 to 64 rows 3 % longer)
  if (p.row_groups > 1)
    hipLaunchKernelGGL((gemm_bf16_rows_kernel<2, 2, RW, R_HELD>), grid, block, 0, stream, p);
  else if (M <= 32)
    hipLaunchKernelGGL((gemm_bf16_rows_kernel<2, 2, 2 * RW, 4>), grid, dim3(2 * RW * 64), 0, stream, p);
  else
    hipLaunchKernelGGL((gemm_bf16_rows_kernel<3, 2, 2 * RW, 4>), grid, dim3(2 * RW * 64), 0, stream, p);
  CHECK_LAUNCH("gemm_bf16_rows");
  return 0;
}

// out = epilogue(sum of the n_splits partial products in ws): what gemm_bf16_decode left out.
extern "C" int sum_partials(void* out, const float* ws, int n_splits, const float* bias, int M, int N,
                            int ldo, int flags, void* k_pages, void* v_pages, size_t page_stride,
                            const int* block_table, int max_blocks, const int* token_req,
                            const int* positions, int q_width, int kv_width, int head_dim,
                            int page_size, hipStream_t stream) {
  if (M == 0) return 0;
  if (M < 0 || n_splits < 1 || !ws) FAIL("sum_partials: bad M=%d, splits=%d or workspace", M, n_splits);
  DecodeGemmArgs p = {};
  if (fill_epilogue(p, "sum_partials", out, bias, M, N, ldo, flags, k_pages, v_pages, page_stride,
                    block_table, max_blocks, token_req, positions, q_width, kv_width, head_dim, page_size))
    return -1;
  p.ws = (float*)ws, p.n_splits = n_splits;
  p.vec4 = p.vec4 && aligned16(ws);
  const long total = (long)M * ((N + 3) / 4);
  hipLaunchKernelGGL(sum_partials_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, p);
  CHECK_LAUNCH("sum_partials");
  return 0;
}

// 1 if sum_partials_norm takes this width
extern "C" int sum_partials_norm_takes(int N, int ldh) { return N > 0 && N % 4 == 0 && N <= 8192 && ldh % 4 == 0; }

// h[m] += bias + sum of the partial products;  out[m] = LayerNorm(h[m]) (float32 or bfloat16, [M][N];
// with out_packed a bfloat16 out in the packed order that gemm_bf16_rows reads fastest)
extern "C" int sum_partials_norm(float* h, int ldh, const float* ws, int n_splits, const float* bias,
                                 const float* gamma, const float* beta, float eps, void* out,
                                 int out_dtype, int out_packed, int M, int N, const void* ahead,
                                 size_t ahead_chunk_bytes, int ahead_chunks, hipStream_t stream) {
  if (M == 0) return 0;
  if (ahead && (!aligned16(ahead) || ahead_chunk_bytes % 16 != 0 || ahead_chunks < 0))
    FAIL("sum_partials_norm: what is read ahead must be chunks of 16-byte pieces");
  if (M < 0 || n_splits < 1 || !ws || !h || !out) FAIL("sum_partials_norm: bad M=%d, splits=%d or null pointer", M, n_splits);
  if (!sum_partials_norm_takes(N, ldh) || ldh < N)
    FAIL("sum_partials_norm: width %d (row stride %d) must be a multiple of 4, at most 8192", N, ldh);
  if (!aligned16(h) || !aligned16(ws) || !aligned16(bias) || !aligned16(gamma) || !aligned16(beta) || !aligned16(out))
    FAIL("sum_partials_norm: pointers must be 16-byte aligned");
  if (out_dtype != DT_F32 && out_dtype != DT_BF16) FAIL("sum_partials_norm: unknown dtype code %d", out_dtype);
  if (out_packed && out_dtype != DT_BF16) FAIL("sum_partials_norm: the packed order is for a bfloat16 out");
  SumNormArgs q;
  q.out_packed = out_packed ? 1 : 0;
  q.h = h, q.ws = ws, q.bias = bias, q.gamma = gamma, q.beta = beta, q.out = out, q.eps = eps;
  q.M = M, q.N = N, q.ldh = ldh, q.n_splits = n_splits, q.out_dtype = out_dtype;
  q.ahead = (const uint4*)ahead, q.ahead_pieces = ahead ? ahead_chunk_bytes / 16 : 0;
  q.ahead_chunks = ahead ? ahead_chunks : 0;
  // as many reading blocks as leave a CU each to the rows' blocks (few rows only: with many, the
  // CUs are busy and the memory too)
  const int readers = q.ahead_pieces > 0 && q.ahead_chunks > 0 && M <= 16 ? (n_compute_units() - M) / N_DIES * N_DIES : 0;
  if (N <= 2048)
    hipLaunchKernelGGL(sum_partials_norm_kernel<2>, dim3(M + readers), dim3(256), 0, stream, q);
  else
    hipLaunchKernelGGL(sum_partials_norm_kernel<8>, dim3(M + readers), dim3(256), 0, stream, q);
  CHECK_LAUNCH("sum_partials_norm");
  return 0;
}

// ---------------------------------------------------------------------------
// The split product for callers that cannot allocate (no_alloc.h).  The partial sums lie in
// an array of the library's own, one copy on every GPU.  In host code the array's name is only
// a handle for hipGetSymbolAddress: what kernels, copies and fills get is the address looked
// up there, once per device, with that device current.

static __device__ __align__(256) float scratch[GEMM_BF16_DECODE_STATIC_FLOATS];

#define STATIC_MAX_DEVICES 64
static float* g_scratch_ptr[STATIC_MAX_DEVICES];  // per device: where its copy of `scratch` lies
static std::mutex g_scratch_lock;

// The current device's copy of the array (looked up at the first call on that device).
static int scratch_of_current_device(float** ptr) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) FAIL("gemm_bf16_decode_split_static: no current device: %s", hipGetErrorString(e));
  if (dev < 0 || dev >= STATIC_MAX_DEVICES)
    FAIL("gemm_bf16_decode_split_static: device %d is beyond the %d this library keeps an array for", dev,
         STATIC_MAX_DEVICES);
  std::lock_guard<std::mutex> guard(g_scratch_lock);
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p)
      FAIL("gemm_bf16_decode_split_static: the array's address on device %d: %s", dev, hipGetErrorString(e));
    g_scratch_ptr[dev] = (float*)p;
  }
  *ptr = g_scratch_ptr[dev];
  return 0;
}

extern "C" int gemm_bf16_decode_static_init(void) {
  float* ptr = nullptr;
  return scratch_of_current_device(&ptr);
}

extern "C" int gemm_bf16_decode_split_static(void* out, const void* A, int lda, const void* W,
                                             const float* bias, int M, int N, int K, int ldw, int ldo,
                                             int flags, int n_splits, hipStream_t stream) {
  if (M == 0) return 0;
  if (flags & ~(FLAG_GELU | FLAG_ACCUMULATE | FLAG_OUT_F32))
    FAIL("gemm_bf16_decode_split_static: flags %d: only GELU (1), accumulate (2) and float32 out (4)", flags);
  if (M < 0 || N <= 0 || n_splits < 1) FAIL("gemm_bf16_decode_split_static: bad M=%d, N=%d or splits=%d", M, N, n_splits);
  if ((size_t)n_splits * (size_t)M * (size_t)N > (size_t)GEMM_BF16_DECODE_STATIC_FLOATS)
    FAIL("gemm_bf16_decode_split_static: %d splits of %d x %d are %zu partial sums, the library's array holds %u",
         n_splits, M, N, (size_t)n_splits * M * N, GEMM_BF16_DECODE_STATIC_FLOATS);
  float* ws = nullptr;
  if (scratch_of_current_device(&ws)) return 1;
  // (with one part the product's own kernel runs the epilogue and the array is not touched)
  int rc = gemm_bf16_decode(out, A, lda, nullptr, 0, nullptr, nullptr, 0.f, W, bias, M, N, K, ldw, ldo, flags,
                            nullptr, nullptr, 0, nullptr, 0, nullptr, nullptr, 0, 0, 0, 0, n_splits, ws,
                            GEMM_BF16_DECODE_STATIC_FLOATS, stream);
  if (rc != 0 || n_splits == 1) return rc != 0;
  // Every partial sum read below was written by the launch above: each of the n_splits parts
  // holds k-blocks (an empty part is refused) and its blocks write all M x N sums of the part.
  rc = sum_partials(out, ws, n_splits, bias, M, N, ldo, flags, nullptr, nullptr, 0, nullptr, 0, nullptr,
                    nullptr, 0, 0, 0, 0, stream);
  return rc != 0;
}
