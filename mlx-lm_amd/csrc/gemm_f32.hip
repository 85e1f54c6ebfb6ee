// Linear layer in true 32-bit: float operands, float products and sums
// (v_mfma_f32_16x16x4_f32; no reduced-precision matrix mode, no float cut
// into shorter pieces).
//   out[m, n] = epilogue( sum_k A[m, k] * W[n, k] + bias[n] )
// A is [M, K], W is [N, K], both contiguous along k.  Epilogues: plain,
// tanh-GELU, or accumulate into the residual stream.  Any M, N; K % 4 == 0.
// The 32-bit twin of gemm_bf16.hip; replaces the same nn.Linear calls
// (mlx_lm/models/gpt2.py:41-42,52,68,76-80,167).
//
// Up to 64 rows (decode steps) take a kernel of their own, which streams W
// once through v_mfma_f32_16x16x4_f32, 16 features a block: a 64 x 64 tile
// would spend its time on rows that are not there and leave most compute units
// without a block.  Where 16 features a block still give fewer blocks than
// units, K goes in parts and a second kernel (the caller's) adds them up.
#include "common.h"

#define FLAG_GELU 1
#define FLAG_ACCUMULATE 2

struct GemmArgs {
  const float* A;
  const float* W;
  const float* bias;
  float* out;
  int M, N, K;
  int lda, ldw, ldo;
  int flags;
  // the kernel for few rows: blockIdx.y takes part y of K's chunks and leaves its sums in
  // ws[y][M][N], without bias or epilogue
  int n_splits;
  float* ws;
};

// Rows of a tile beyond the matrix read a row inside it (their products are
// never stored): the row one tile back where there is one, so that they do not
// all read the matrix's last row at once, which one cache channel would have
// to serve to every block of that row of tiles.
__device__ __forceinline__ int row_inside(int r, int n, int tile) {
  return r < n ? r : (r - tile >= 0 && r - tile < n ? r - tile : n - 1);
}

// Many rows: 2 x 2 waves a block, each with RT x RT tiles of 16 x 16 outputs (a block tile of
// 128 x 128 or 64 x 64).  v_mfma_f32_16x16x4_f32 computes D = A B for A 16 x 4 and B 4 x 16: lane
// l brings A[l % 16][l / 16] and B[l / 16][l % 16] and gets D[4 * (l / 16) + r][l % 16] in
// accumulator r.  Which column of k an instruction's four slots stand for is free as long as both
// operands agree, so a lane loads 16 bytes, columns 4 * (l / 16) .. + 3 of each 16, of row l % 16
// of a tile of A and of feature l % 16 of a tile of W, and the four floats go to four
// instructions.  The operands come straight from memory (the L2s, mostly) in that layout: no LDS
// and no barrier; the next 32 columns are asked for before this step's products begin.  At 32-bit
// speed of the matrix cores (a sixteenth of bfloat16's) the L1 carries that easily.
template <int RT>
__global__ __launch_bounds__(256) void gemm_f32_kernel(GemmArgs p) {
  constexpr int WT = 16 * RT;  // a wave's tile
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int x = lane & 15, g = lane >> 4;
  const int m0 = blockIdx.y * (2 * WT) + (wave >> 1) * WT;
  const int n0 = blockIdx.x * (2 * WT) + (wave & 1) * WT;
  // rows and features beyond the matrix read one inside it; their products are never stored
  const float* arow[RT];
  const float* wrow[RT];
#pragma unroll
  for (int i = 0; i < RT; ++i) {
    arow[i] = p.A + (size_t)row_inside(m0 + 16 * i + x, p.M, 2 * WT) * p.lda + 4 * g;
    wrow[i] = p.W + (size_t)row_inside(n0 + 16 * i + x, p.N, 2 * WT) * p.ldw + 4 * g;
  }
  f32x4_t acc[RT][RT];
#pragma unroll
  for (int i = 0; i < RT; ++i)
#pragma unroll
    for (int j = 0; j < RT; ++j) acc[i][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  // a step: 32 columns, two 16-byte pieces a lane of each row and feature (a whole 128-byte line
  // of each by the lane's group of four).  The rows' values beyond K count as zero.
  f32x4_t a0[2][RT], w0[2][RT], a1[2][RT], w1[2][RT];
  auto ask = [&](int k0, f32x4_t (&ad)[2][RT], f32x4_t (&wd)[2][RT]) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int col = min(k0 + 16 * h, p.K - 4 - 4 * g);  // (+ 4 * g is in the pointers)
#pragma unroll
      for (int i = 0; i < RT; ++i) {
        ad[h][i] = *(const f32x4_t*)(arow[i] + col);
        wd[h][i] = *(const f32x4_t*)(wrow[i] + col);
      }
    }
  };
  auto multiply = [&](int k0, const f32x4_t (&as)[2][RT], const f32x4_t (&ws)[2][RT]) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const float live = k0 + 16 * h + 4 * g < p.K ? 1.f : 0.f;
#pragma unroll
      for (int i = 0; i < RT; ++i) {
        const f32x4_t av = as[h][i] * live;
#pragma unroll
        for (int j = 0; j < RT; ++j) {
          acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(av.x, ws[h][j].x, acc[i][j], 0, 0, 0);
          acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(av.y, ws[h][j].y, acc[i][j], 0, 0, 0);
          acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(av.z, ws[h][j].z, acc[i][j], 0, 0, 0);
          acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(av.w, ws[h][j].w, acc[i][j], 0, 0, 0);
        }
      }
    }
  };
  // Two steps a round, their operands in two sets of registers by turns.  A step's loads are
  // issued on one path whether its columns exist or not (beyond K they read inside the matrix),
  // and stay ahead of the products before them: the wait is then for the older set only.
  ask(0, a0, w0);
  for (int k0 = 0; k0 < p.K; k0 += 64) {
    ask(k0 + 32, a1, w1);
    __builtin_amdgcn_sched_barrier(0);
    multiply(k0, a0, w0);
    __builtin_amdgcn_sched_barrier(0);
    ask(k0 + 64, a0, w0);
    __builtin_amdgcn_sched_barrier(0);
    if (k0 + 32 < p.K) multiply(k0 + 32, a1, w1);  // (uniform)
    __builtin_amdgcn_sched_barrier(0);
  }

  // Epilogue.  Accumulator r of tile (i, j): row 16 * i + 4 * g + r, feature 16 * j + x.  What is
  // read (bias, the residual stream to add to) is read for a row of tiles before anything of it is
  // stored: a load that comes after a store to memory it might alias waits for it.
#pragma unroll
  for (int i = 0; i < RT; ++i) {
    const int mb = m0 + 16 * i + 4 * g;
    f32x4_t v[RT];
#pragma unroll
    for (int j = 0; j < RT; ++j) {
      const int n = n0 + 16 * j + x;
      const int nc = min(n, p.N - 1);
      const float bias = p.bias ? p.bias[nc] : 0.f;
      if (p.flags & FLAG_ACCUMULATE) {
#pragma unroll
        for (int r = 0; r < 4; ++r) v[j][r] = p.out[(size_t)min(mb + r, p.M - 1) * p.ldo + nc];
#pragma unroll
        for (int r = 0; r < 4; ++r) v[j][r] += acc[i][j][r] + bias;
      } else {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          v[j][r] = acc[i][j][r] + bias;
          if (p.flags & FLAG_GELU) v[j][r] = gelu_tanh(v[j][r]);
        }
      }
    }
#pragma unroll
    for (int j = 0; j < RT; ++j) {
      const int n = n0 + 16 * j + x;
      if (n >= p.N) continue;
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (mb + r < p.M) p.out[(size_t)(mb + r) * p.ldo + n] = v[j][r];
    }
  }
}

#define SKF_WAVES_FEW 8   // waves a block where the blocks are fewer than the compute units
#define SKF_WAVES_MANY 4  // and where every unit has a block or more (8: 12.1 us instead of 10.6 for 4,800 features of 1,600)
#define SKF_MAX_WAVES 8
#define SKF_MAX_ROWS 64
#define SKF_SPLIT_FROM 5000000L  // elements of a matrix from which a split of K pays
#define SKF_CHUNK 64                    // columns of a chunk
#define SKF_STRIDE (SKF_CHUNK + 4)      // floats between a chunk's rows in LDS: no two of a load's lanes share a bank

// Up to 64 rows, in RB blocks of 16.  A block owns 16 features and, where K is split over
// blockIdx.y, a run of chunks of 64 columns; its waves take the run's chunks in turn, each wave on
// its own (no barrier inside the loop).  A chunk of the weights comes from memory as 256
// contiguous bytes a feature, four features a load, goes through the wave's own piece of LDS and
// comes back in the layout of v_mfma_f32_16x16x4_f32: lane l holds columns 4 * (l / 16) .. + 3 of
// each 16 of feature l % 16.  The rows are the other operand, read in that layout from the L2,
// where they stay.  The next chunk is asked for before this one is multiplied; other waves cover
// the rest of the wait (a deeper queue was slower: 82 us against 72 for the vocabulary's matrix
// at 8 rows).  The same instructions run for every number of rows that fills the same blocks of
// 16, and a block of rows is multiplied on its own, so a row's result does not depend on the
// others.  With four blocks of rows the instructions bound the stream at some 4.8 TB/s.
template <int RB>
__global__ __launch_bounds__(64 * SKF_MAX_WAVES) void gemm_f32_skinny_kernel(GemmArgs p) {
  // (native vectors: a struct copied to LDS keeps what was loaded out of registers)
  __shared__ f32x4_t stage[SKF_MAX_WAVES][16 * SKF_STRIDE / 4];
  static_assert(sizeof(float) * SKF_MAX_WAVES * RB * 256 <= sizeof(f32x4_t) * SKF_MAX_WAVES * (16 * SKF_STRIDE / 4),
                "the waves' sums fit where the chunks were");
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, n_waves = blockDim.x >> 6;
  const int n0 = blockIdx.x * 16;
  const int l16 = lane & 15, kq = lane >> 4;
  // features and rows that are not there read the last one that is; nothing of theirs is stored
  const float* wsrc[4];  // load i: feature 4 * i + l / 16, columns 4 * (l % 16) .. + 3 of the chunk
#pragma unroll
  for (int i = 0; i < 4; ++i) wsrc[i] = p.W + (size_t)min(n0 + 4 * i + kq, p.N - 1) * p.ldw;
  const float* arow[RB];
#pragma unroll
  for (int b = 0; b < RB; ++b) arow[b] = p.A + (size_t)min(16 * b + l16, p.M - 1) * p.lda;
  f32x4_t* mine = stage[wave];
  const int n_chunks = (p.K + SKF_CHUNK - 1) / SKF_CHUNK;
  const int per_split = (n_chunks + p.n_splits - 1) / p.n_splits;
  const int c_end = min(n_chunks, (blockIdx.y + 1) * per_split);

  f32x4_t wv[4], av[RB][4];
  // columns beyond K (in the last chunk) and chunks beyond the run (asked for ahead by the wave's
  // last round) are read from inside the matrix; the rows' values beyond K count as zero
  auto ask = [&](int c) {
#pragma unroll
    for (int i = 0; i < 4; ++i) wv[i] = *(const f32x4_t*)(wsrc[i] + min(c * SKF_CHUNK + 4 * l16, p.K - 4));
#pragma unroll
    for (int b = 0; b < RB; ++b)
#pragma unroll
      for (int t = 0; t < 4; ++t)
        av[b][t] = *(const f32x4_t*)(arow[b] + min(c * SKF_CHUNK + 16 * t + 4 * kq, p.K - 4));
  };
  f32x4_t acc[RB];
#pragma unroll
  for (int b = 0; b < RB; ++b) acc[b] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  int c = blockIdx.y * per_split + wave;
  ask(c);
  for (; c < c_end; c += n_waves) {
    f32x4_t a[RB][4];
#pragma unroll
    for (int i = 0; i < 4; ++i) mine[(4 * i + kq) * (SKF_STRIDE / 4) + l16] = wv[i];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const float live = c * SKF_CHUNK + 16 * t + 4 * kq < p.K ? 1.f : 0.f;
#pragma unroll
      for (int b = 0; b < RB; ++b) a[b][t] = av[b][t] * live;
    }
    ask(c + n_waves);
    __builtin_amdgcn_wave_barrier();  // (orders the compiler; a wave's LDS accesses run in order)
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const f32x4_t w = mine[l16 * (SKF_STRIDE / 4) + 4 * t + kq];
#pragma unroll
      for (int b = 0; b < RB; ++b) {
        acc[b] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[b][t].x, w.x, acc[b], 0, 0, 0);
        acc[b] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[b][t].y, w.y, acc[b], 0, 0, 0);
        acc[b] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[b][t].z, w.z, acc[b], 0, 0, 0);
        acc[b] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[b][t].w, w.w, acc[b], 0, 0, 0);
      }
    }
    __builtin_amdgcn_wave_barrier();
  }
  // accumulator r of lane l: row 4 * (l / 16) + r of its block of rows, feature l % 16.  The
  // waves' sums are added in the order of the waves, one thread an output and block of rows.
  __syncthreads();  // the pieces of LDS are no longer read
  float* parts = (float*)&stage[0][0];  // [wave][block of rows][row][feature]
#pragma unroll
  for (int b = 0; b < RB; ++b)
#pragma unroll
    for (int r = 0; r < 4; ++r) parts[((wave * RB + b) * 16 + 4 * kq + r) * 16 + l16] = acc[b][r];
  __syncthreads();
  if (tid < 256) {
    const int n = n0 + (tid & 15);
#pragma unroll
    for (int b = 0; b < RB; ++b) {
      const int m = 16 * b + (tid >> 4);
      if (m >= p.M || n >= p.N) continue;
      float v = parts[b * 256 + tid];
      for (int w = 1; w < n_waves; ++w) v += parts[(w * RB + b) * 256 + tid];
      if (p.n_splits > 1) {
        p.ws[((size_t)blockIdx.y * p.M + m) * p.N + n] = v;  // added up, and finished, by the caller's second kernel
        continue;
      }
      if (p.bias) v += p.bias[n];
      const size_t idx = (size_t)m * p.ldo + n;
      if (p.flags & FLAG_ACCUMULATE)
        p.out[idx] += v;
      else
        p.out[idx] = (p.flags & FLAG_GELU) ? gelu_tanh(v) : v;
    }
  }
}

DEFINE_LAST_ERROR(mlxlm_last_error)

// In how many parts the kernel for few rows should take K so that its blocks fill the GPU: one
// and a half blocks a compute unit, eight chunks of 64 columns a part at least.  1 where the
// matrix gives a block to every unit anyway, or is so small that a second kernel costs more
// than the split gains.
extern "C" int gemm_f32_splits(int M, int N, int K, int force) {
  const int n_chunks = (K + SKF_CHUNK - 1) / SKF_CHUNK;
  if (M < 1 || M > SKF_MAX_ROWS) return 1;
  int want;
  if (force > 0) {
    want = force;
  } else {
    const int n_blocks = (N + 15) / 16;
    if (n_blocks >= n_compute_units() || (long)N * K < SKF_SPLIT_FROM) return 1;
    want = (3 * n_compute_units() / 2 + n_blocks - 1) / n_blocks;
    if (want > n_chunks / 8) want = n_chunks / 8;
  }
  if (want < 1) want = 1;
  if (want > n_chunks) want = n_chunks;
  const int per = (n_chunks + want - 1) / want;
  return (n_chunks + per - 1) / per;  // no empty part
}

// variant: 0 = choose, 1 = 128x128 block tile, 2 = 64x64 block tile, 3 = the kernel for up to 64 rows.
// n_splits > 1 (the kernel for few rows only): K in that many parts, whose sums go to
// ws[part][M][N] (ws_floats floats at least) for sum_partials of gemm_bf16_decode.hip to add up
// and finish; out is not written then.
extern "C" int gemm_f32(void* out, const void* A, const void* W, const float* bias, int M, int N,
                        int K, int lda, int ldw, int ldo, int flags, int variant, int n_splits, float* ws,
                        size_t ws_floats, hipStream_t stream) {
  GemmArgs p;
  p.A = (const float*)A;
  p.W = (const float*)W;
  p.bias = bias;
  p.out = (float*)out;
  p.M = M, p.N = N, p.K = K;
  p.lda = lda, p.ldw = ldw, p.ldo = ldo;
  p.flags = flags;
  p.n_splits = 1, p.ws = nullptr;
  if (M < 0 || N <= 0 || K <= 0) FAIL("gemm_f32: bad sizes M=%d N=%d K=%d", M, N, K);
  if (K % 4 != 0) FAIL("gemm_f32: K=%d must be a multiple of 4", K);
  if (lda % 4 != 0 || ldw % 4 != 0)
    FAIL("gemm_f32: row strides lda=%d ldw=%d must be multiples of 4", lda, ldw);
  if (lda < K || ldw < K || ldo < N)
    FAIL("gemm_f32: row strides smaller than the rows (lda=%d ldw=%d ldo=%d)", lda, ldw, ldo);
  if (!A || !W || !out) FAIL("gemm_f32: null pointer");
  if (((uintptr_t)A | (uintptr_t)W) & 15) FAIL("gemm_f32: A and W must be 16-byte aligned");
  if ((flags & FLAG_ACCUMULATE) && (flags & FLAG_GELU))
    FAIL("gemm_f32: GELU and accumulate cannot be combined");
  if (M == 0) return 0;
  if (n_splits < 1) FAIL("gemm_f32: n_splits=%d", n_splits);
  if (n_splits > 1) {
    if (variant == 0 && M <= SKF_MAX_ROWS) variant = 3;
    if (variant != 3) FAIL("gemm_f32: only the kernel for up to %d rows takes K in parts", SKF_MAX_ROWS);
    if (n_splits > (K + SKF_CHUNK - 1) / SKF_CHUNK) FAIL("gemm_f32: %d parts of K=%d", n_splits, K);
    if (!ws || ws_floats < (size_t)n_splits * M * N) FAIL("gemm_f32: the parts' workspace is too small");
    p.n_splits = n_splits, p.ws = ws;
  }
  if (variant == 0) variant = M <= SKF_MAX_ROWS ? 3 : (size_t)M * N < (size_t)128 * 128 * 128 ? 2 : 1;
  if (variant == 1) {
    dim3 grid((N + 127) / 128, (M + 127) / 128), block(256);
    hipLaunchKernelGGL(gemm_f32_kernel<4>, grid, block, 0, stream, p);
  } else if (variant == 2) {
    dim3 grid((N + 63) / 64, (M + 63) / 64), block(256);
    hipLaunchKernelGGL(gemm_f32_kernel<2>, grid, block, 0, stream, p);
  } else if (variant == 3) {
    if (M > SKF_MAX_ROWS) FAIL("gemm_f32: the kernel for few rows takes at most %d, got %d", SKF_MAX_ROWS, M);
    // where the blocks are fewer than the compute units, more waves each
    const int blocks = (N + 15) / 16;
    const int waves = blocks * p.n_splits < n_compute_units() ? SKF_WAVES_FEW : SKF_WAVES_MANY;
    const dim3 grid(blocks, p.n_splits), block(64 * waves);
    if (M <= 16)
      hipLaunchKernelGGL(gemm_f32_skinny_kernel<1>, grid, block, 0, stream, p);
    else if (M <= 32)
      hipLaunchKernelGGL(gemm_f32_skinny_kernel<2>, grid, block, 0, stream, p);
    else if (M <= 48)
      hipLaunchKernelGGL(gemm_f32_skinny_kernel<3>, grid, block, 0, stream, p);
    else
      hipLaunchKernelGGL(gemm_f32_skinny_kernel<4>, grid, block, 0, stream, p);
  } else {
    FAIL("gemm_f32: unknown variant %d", variant);
  }
  CHECK_LAUNCH("gemm_f32");
  return 0;
}
