// Linear layer for decode steps: at most 64 rows of activations (the main
// kernel: up to 16; a wide variant: 17 to 64) against a bfloat16 weight matrix
// that streams from HBM exactly once.
//   out[m, n] = epilogue( sum_k A[m, k] * W[n, k] + bias[n] )
// with two fusions that save a launch and a round trip through memory each:
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
// A block of eight waves owns 16 output features (8 or 4 where N is narrow:
// a CU can only keep so many loads in flight, so a launch that does not
// occupy every CU cannot reach the memory's bandwidth).  The activations (normed or
// copied) sit in LDS as the MFMA B-operand; each wave takes every eighth
// 64-wide k-block of the 16 weight rows as the A-operand of two
// v_mfma_f32_16x16x32_bf16 (lane l reads 32 contiguous bytes of row l % 16 at
// k offset (l / 16) * 16).  Weight loads run two passes of four k-blocks ahead
// of the MFMAs; the eight partial tiles are summed in a fixed order.
//
// Where 16-feature blocks alone are too few to fill the GPU (N = 1600), K is
// also split over blockIdx.y.  Each split writes its partial tile to a
// workspace and bumps a counter; the block that arrives last adds the partial
// tiles in the order of the splits (so the sum does not depend on who was
// last), runs the epilogue and sets the counter back to zero.  The workspace
// and the counters belong to the caller; launches that share them must not
// overlap.
#include "common.h"

#define FLAG_GELU 1
#define FLAG_ACCUMULATE 2
#define FLAG_OUT_F32 4
#define FLAG_KV 8

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
  // split of K over blockIdx.y: partial tiles and one arrival counter per 16 features
  int n_splits, chunks_per_split;
  int rows;            // output features a block owns: 16, 8 or 4 (fewer = more blocks for a narrow N)
  float* ws;           // [n_blocks][n_splits][256]
  unsigned int* counters;  // [n_blocks], zero between launches
};

__device__ __forceinline__ float gelu_tanh(float x) {
  const float c = 0.7978845608028654f;
  const float u = c * (x + 0.044715f * x * x * x);
  return 0.5f * x * (1.0f + tanhf(u));
}

__device__ __forceinline__ uint32_t pack2(float a, float b) {
  return (uint32_t)f32_to_bf16_bits(a) | ((uint32_t)f32_to_bf16_bits(b) << 16);
}

union Frag {
  uint4 u;
  bf16x8_t v;
};

// bias, activation and where one output goes: the matrix, the residual stream or a cache page
__device__ __forceinline__ void finish(const DecodeGemmArgs& p, int m, int n, float v) {
  if (p.bias) v += p.bias[n];
  if (p.flags & FLAG_GELU) v = gelu_tanh(v);
  if ((p.flags & FLAG_KV) && n >= p.q_width) {
    const int c = n - p.q_width;
    const bool is_v = c >= p.kv_width;
    const int cc = is_v ? c - p.kv_width : c;
    const int head = cc / p.head_dim, d = cc - head * p.head_dim;
    const int pos = p.positions[m];
    const int page = p.block_table[(size_t)p.token_req[m] * p.max_blocks + pos / p.page_size];
    const size_t dst = (size_t)page * p.page_stride +
                       ((size_t)head * p.page_size + pos % p.page_size) * p.head_dim + d;
    (is_v ? p.v_pages : p.k_pages)[dst] = f32_to_bf16_bits(v);
  } else {
    const size_t idx = (size_t)m * p.ldo + n;
    if (p.flags & FLAG_ACCUMULATE)
      ((float*)p.out)[idx] += v;
    else if (p.flags & FLAG_OUT_F32)
      ((float*)p.out)[idx] = v;
    else
      ((uint16_t*)p.out)[idx] = f32_to_bf16_bits(v);
  }
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
  const uint16_t* wtile = p.W + (size_t)blockIdx.x * ((p.K + 63) / 64) * 1024 + lane * 8;
  const int n_chunks_all = (p.K + 63) / 64;
  const int c_begin = blockIdx.y * p.chunks_per_split;  // this split's k-blocks
  const int n_chunks = min(n_chunks_all, c_begin + p.chunks_per_split) - c_begin;
  const int kb = c_begin * 64;  // LDS holds the activations' columns from here on

  // Loads are never predicated on their address (a select between an address
  // and a dummy makes them flat loads, which also count as LDS traffic) and
  // weight fragments are not even zeroed when they lie outside the matrix:
  // every address is pulled into range, and what such a fragment meets is a
  // zero activation (k >= K) or an output that is never stored (n >= N).  So
  // nothing has to wait for a weight before the MFMA that uses it.
  auto load_pass = [&](Frag (&w)[UU][2], int pass) {
    if (wave + NW * pass * UU >= n_chunks) return;  // the whole pass lies beyond K (uniform)
#pragma unroll
    for (int u = 0; u < UU; ++u) {
      const int c = c_begin + min(wave + NW * (pass * UU + u), n_chunks - 1);
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
#pragma unroll
      for (int i = 0; i < NV; ++i) v[i] = *(const float4*)(x + min((lane + 64 * i) * 4, p.K - 4));
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
    const int per_row = (min(p.K, kb + n_chunks * 64) - kb) / 8;
    for (int c = tid; c < p.M * per_row; c += NW * 64) {
      const int r = c / per_row, k = (c - r * per_row) * 8;
      *(uint4*)(As + r * p.a_stride + k) = *(const uint4*)(p.A + (size_t)r * p.lda + kb + k);
    }
  }
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
  if (p.n_splits > 1) {
    // leave the partial tile, count the arrival; the last block goes on alone
    __shared__ unsigned int arrived;
    float* mine = p.ws + ((size_t)blockIdx.x * p.n_splits + blockIdx.y) * 256;
    if (tid < 256) mine[tid] = v;
    __threadfence();
    __syncthreads();
    if (tid == 0) arrived = atomicAdd(p.counters + blockIdx.x, 1u);
    __syncthreads();
    if (arrived != (unsigned int)(p.n_splits - 1)) return;
    __threadfence();
    if (tid == 0) p.counters[blockIdx.x] = 0u;  // ready for the next launch
    if (tid < 256) {
      const float* all = p.ws + (size_t)blockIdx.x * p.n_splits * 256;
      v = 0.f;
      for (int sp = 0; sp < p.n_splits; ++sp)
        v += __uint_as_float(__hip_atomic_load((const unsigned int*)(all + sp * 256 + tid), __ATOMIC_RELAXED,
                                               __HIP_MEMORY_SCOPE_AGENT));  // from L2, where the others wrote
    }
  }
  if (tid < 256) {
    // element tid = 4 * L + r of the MFMA tile: feature 4 * (L / 16) + r, row L % 16
    const int L = tid >> 2, r = tid & 3;
    const int f = 4 * (L >> 4) + r;
    const int n = n0 + f;
    const int m = L & 15;
    if (m < p.M && f < p.rows && n < p.N) finish(p, m, n, v);
  }
}

// ---------------------------------------------------------------------------
// 17 to 64 rows of activations (MT groups of 16): they no longer fit in LDS
// whole, so they pass through it in chunks of 512 columns, one k-block a wave.
// Weights: packed or row-major as above, two chunks ahead in registers.
#define WIDE_CHUNK (NW * 64)          // columns staged at a time
#define WIDE_STRIDE (WIDE_CHUNK + 8)  // LDS row stride: 16-byte reads of 16 rows on distinct banks

template <int MT>
__global__ __launch_bounds__(NW * 64, 2) void gemm_bf16_decode_wide_kernel(DecodeGemmArgs p) {
  extern __shared__ __attribute__((aligned(16))) uint16_t As[];  // [MT * 16][WIDE_STRIDE]
  __shared__ float red[NW][MT][256];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n0 = blockIdx.x * 16;
  const int koff = (lane >> 4) * 16;
  const int n_chunks = (p.K + 63) / 64;               // k-blocks
  const int n_stages = (n_chunks + NW - 1) / NW;      // chunks of NW k-blocks
  const bool packed = p.ldw == 0;
  const uint16_t* wrow = p.W + (size_t)min(n0 + (lane & 15), p.N - 1) * p.ldw;
  const uint16_t* wtile = p.W + (size_t)blockIdx.x * n_chunks * 1024 + lane * 8;

  auto load_w = [&](Frag (&w)[2], int stage) {
    const int c = min(stage * NW + wave, n_chunks - 1);
    if (packed) {
      w[0].u = *(const uint4*)(wtile + (size_t)c * 1024);
      w[1].u = *(const uint4*)(wtile + (size_t)c * 1024 + 512);
    } else {
      const int k = c * 64 + koff;
      w[0].u = *(const uint4*)(wrow + min(k, p.K - 8));
      w[1].u = *(const uint4*)(wrow + min(k + 8, p.K - 8));
    }
  };

  f32x4_t acc[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) acc[t] = (f32x4_t){0.f, 0.f, 0.f, 0.f};

  Frag w[3][2];  // this stage's fragments and the next two
  load_w(w[0], 0);
  load_w(w[1], 1);

  const int rows = min(p.M, MT * 16);
  const uint16_t* arow[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) arow[t] = As + min(t * 16 + (lane & 15), rows - 1) * WIDE_STRIDE + koff;

  // three stages an iteration, so that the register sets are named statically
  auto one_stage = [&](int stage, Frag (&cur)[2], Frag (&next2)[2]) {
    if (stage >= n_stages) return;
    load_w(next2, stage + 2);
    __syncthreads();  // the previous chunk is no longer read
    const int k0 = stage * WIDE_CHUNK;
    const int width = min(WIDE_CHUNK, p.K - k0);  // a multiple of 8
    const int per_row = width / 8;
    for (int c = tid; c < rows * per_row; c += NW * 64) {
      const int r = c / per_row, k = (c - r * per_row) * 8;
      *(uint4*)(As + r * WIDE_STRIDE + k) = *(const uint4*)(p.A + (size_t)r * p.lda + k0 + k);
    }
    __syncthreads();
    if (stage * NW + wave < n_chunks) {  // uniform over the wave
      const int kl = wave * 64 + koff;   // this lane's columns within the chunk
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        const bool live = t * 16 + (lane & 15) < p.M;
        Frag a0, a1;
        // (columns beyond `width` are stale LDS of an earlier chunk: read, then dropped)
        const uint4 t0 = *(const uint4*)(arow[t] + wave * 64);
        const uint4 t1 = *(const uint4*)(arow[t] + wave * 64 + 8);
        a0.u = (live && kl < width) ? t0 : ZERO4;
        a1.u = (live && kl + 8 < width) ? t1 : ZERO4;
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(cur[0].v, a0.v, acc[t], 0, 0, 0);
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(cur[1].v, a1.v, acc[t], 0, 0, 0);
      }
    }
  };
  for (int stage = 0; stage < n_stages; stage += 3) {
    one_stage(stage, w[0], w[2]);
    one_stage(stage + 1, w[1], w[0]);
    one_stage(stage + 2, w[2], w[1]);
  }

#pragma unroll
  for (int t = 0; t < MT; ++t)
#pragma unroll
    for (int r = 0; r < 4; ++r) red[wave][t][lane * 4 + r] = acc[t][r];
  __syncthreads();
  for (int e = tid; e < MT * 256; e += NW * 64) {
    const int t = e >> 8, i = e & 255;
    float v = 0.f;
#pragma unroll
    for (int wv = 0; wv < NW; ++wv) v += red[wv][t][i];
    const int L = i >> 2, r = i & 3;
    const int n = n0 + 4 * (L >> 4) + r;
    const int m = t * 16 + (L & 15);
    if (m < p.M && n < p.N) finish(p, m, n, v);
  }
}

DEFINE_LAST_ERROR(mlxlm_last_error)

#define MAX_LDS_BYTES (120 * 1024)

// LDS row stride: rows of 16-byte reads from 16 lanes must fall on distinct
// banks, which holds when the stride in 32-bit words is 4 mod 32.
static int a_stride_for(int K) { return K + ((8 - K % 64) + 64) % 64; }

// Features per block.
static int rows_per_block(int N) {
  // 16 always, for now: with fewer, the lanes of the unused rows repeat a load, which costs the
  // same address and cache bandwidth as a useful one (measured: no gain at N = 1600, K = 6400)
  (void)N;
  return 16;
}

static int chunks_per_split(int K, int n_splits) { return ((K + 63) / 64 + n_splits - 1) / n_splits; }

// 1 if gemm_bf16_decode takes these sizes (the caller falls back otherwise)
extern "C" int gemm_bf16_decode_takes(int M, int K, int with_norm, int n_splits) {
  if (M > 16 && M <= 64) return !with_norm && n_splits == 1 && K % 8 == 0;  // the wide kernel
  if (M < 1 || M > 16 || K % 8 != 0 || n_splits < 1 || n_splits > (K + 63) / 64) return 0;
  if (with_norm && (n_splits != 1 || K > LN_MAX_V * 256 || K > NW * U * 64 || K % 4 != 0)) return 0;
  const int range = K < chunks_per_split(K, n_splits) * 64 ? K : chunks_per_split(K, n_splits) * 64;
  return (size_t)M * a_stride_for(range) * 2 <= MAX_LDS_BYTES;
}

// How many ways to split K by default.
extern "C" int gemm_bf16_decode_splits(int N, int K, int with_norm) {
  // One, for now: the release/acquire pair that the hand-over between blocks
  // needs writes back and invalidates an L2 per block on this multi-die GPU,
  // which costs far more than the parallelism gains (measured: 8 us -> 120 us).
  (void)N, (void)K, (void)with_norm;
  return 1;
}

extern "C" int gemm_bf16_decode(
    void* out, const void* A, int lda, const float* X, int ldx, const float* gamma,
    const float* beta, float eps, const void* W, const float* bias, int M, int N, int K, int ldw,
    int ldo, int flags, void* k_pages, void* v_pages, size_t page_stride, const int* block_table,
    int max_blocks, const int* token_req, const int* positions, int q_width, int kv_width,
    int head_dim, int page_size, int n_splits, float* ws, size_t ws_floats, unsigned int* counters,
    size_t n_counters, hipStream_t stream) {
  if (M == 0) return 0;
  const bool ln = X != nullptr;
  if (!gemm_bf16_decode_takes(M, K, ln, n_splits))
    FAIL("gemm_bf16_decode: M=%d K=%d%s is outside what this kernel takes", M, K, ln ? " with norm" : "");
  if (N <= 0) FAIL("gemm_bf16_decode: bad N=%d", N);
  if ((A == nullptr) == (X == nullptr)) FAIL("gemm_bf16_decode: give activations or a residual stream to norm");
  if (!W || !out) FAIL("gemm_bf16_decode: null pointer");
  // ldw == 0: W is packed by pack_weight_for_decode (tiles of 16 features x 64 k, zero padded)
  if (ldw != 0 && (ldw % 8 != 0 || ldw < K)) FAIL("gemm_bf16_decode: W rows must be 16-byte aligned");
  if ((uintptr_t)W & 15) FAIL("gemm_bf16_decode: W must be 16-byte aligned");
  if (A && (lda % 8 != 0 || lda < K || ((uintptr_t)A & 15))) FAIL("gemm_bf16_decode: A rows must be 16-byte aligned");
  if (X && (ldx % 4 != 0 || ldx < K || ((uintptr_t)X & 15))) FAIL("gemm_bf16_decode: X rows must be 16-byte aligned");
  if (X && (!gamma || !beta || ((uintptr_t)gamma & 15) || ((uintptr_t)beta & 15)))
    FAIL("gemm_bf16_decode: the norm needs scale and shift, 16-byte aligned");
  if ((flags & FLAG_ACCUMULATE) && (flags & (FLAG_GELU | FLAG_KV)))
    FAIL("gemm_bf16_decode: accumulate cannot be combined with GELU or the cache scatter");
  if (flags & FLAG_KV) {
    if (!k_pages || !v_pages || !block_table || !token_req || !positions)
      FAIL("gemm_bf16_decode: the cache scatter needs pages, block table, token_req and positions");
    if (head_dim <= 0 || page_size <= 0 || kv_width % head_dim != 0 || q_width + 2 * kv_width != N)
      FAIL("gemm_bf16_decode: q_width %d + 2 * kv_width %d must be N=%d, kv_width a multiple of head_dim %d",
           q_width, kv_width, N, head_dim);
    if (flags & (FLAG_OUT_F32 | FLAG_GELU)) FAIL("gemm_bf16_decode: the cache scatter writes bfloat16, no GELU");
    if (ldo < q_width) FAIL("gemm_bf16_decode: ldo=%d smaller than q_width=%d", ldo, q_width);
  } else if (ldo < N) {
    FAIL("gemm_bf16_decode: ldo=%d smaller than N=%d", ldo, N);
  }
  DecodeGemmArgs p;
  p.W = (const uint16_t*)W, p.bias = bias, p.out = out, p.A = (const uint16_t*)A, p.X = X;
  p.gamma = gamma, p.beta = beta, p.eps = eps;
  p.M = M, p.N = N, p.K = K, p.lda = lda, p.ldx = ldx, p.ldw = ldw, p.ldo = ldo, p.flags = flags;
  p.k_pages = (uint16_t*)k_pages, p.v_pages = (uint16_t*)v_pages, p.page_stride = page_stride;
  p.block_table = block_table, p.token_req = token_req, p.positions = positions;
  p.max_blocks = max_blocks, p.q_width = q_width, p.kv_width = kv_width;
  p.head_dim = head_dim, p.page_size = page_size;
  if (M > 16) {
    p.rows = 16, p.n_splits = 1, p.chunks_per_split = 0, p.ws = nullptr, p.counters = nullptr, p.a_stride = 0;
    const int mt = (M + 15) / 16;
    const size_t lds = (size_t)mt * 16 * WIDE_STRIDE * 2;
    void (*wide[3])(DecodeGemmArgs) = {gemm_bf16_decode_wide_kernel<2>, gemm_bf16_decode_wide_kernel<3>,
                                       gemm_bf16_decode_wide_kernel<4>};
    static size_t granted_wide[3] = {0, 0, 0};
    const size_t fixed = sizeof(float) * NW * mt * 256;
    if (lds + fixed > 64 * 1024 && granted_wide[mt - 2] < lds) {
      hipError_t e = hipFuncSetAttribute((const void*)wide[mt - 2], hipFuncAttributeMaxDynamicSharedMemorySize,
                                         (int)lds);
      if (e != hipSuccess) FAIL("gemm_bf16_decode: cannot get %zu bytes of LDS: %s", lds, hipGetErrorString(e));
      granted_wide[mt - 2] = lds;
    }
    hipLaunchKernelGGL(wide[mt - 2], dim3((N + 15) / 16), dim3(NW * 64), lds, stream, p);
    CHECK_LAUNCH("gemm_bf16_decode");
    return 0;
  }
  p.rows = rows_per_block(N);
  const int n_blocks = (N + p.rows - 1) / p.rows;
  p.n_splits = n_splits, p.chunks_per_split = chunks_per_split(K, n_splits);
  p.ws = ws, p.counters = counters;
  if (n_splits > 1) {
    if (!ws || !counters) FAIL("gemm_bf16_decode: a split of K needs the workspace and the counters");
    if (ws_floats < (size_t)n_blocks * n_splits * 256 || n_counters < (size_t)n_blocks)
      FAIL("gemm_bf16_decode: workspace of %zu floats / %zu counters is too small for %d blocks x %d splits",
           ws_floats, n_counters, n_blocks, n_splits);
  }
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
