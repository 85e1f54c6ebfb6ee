// Linear layer in true 32-bit: float operands, float products and sums
// (v_mfma_f32_32x32x2_f32; no reduced-precision matrix mode, no splitting).
//   out[m, n] = epilogue( sum_k A[m, k] * W[n, k] + bias[n] )
// A is [M, K], W is [N, K], both contiguous along k.  Epilogues: plain,
// tanh-GELU, or accumulate into the residual stream.  Any M, N; K % 4 == 0.
// The 32-bit twin of gemm_bf16.hip; replaces the same nn.Linear calls
// (mlx_lm/models/gpt2.py:41-42,52,68,76-80,167).
//
// Up to 16 rows (decode steps) take a kernel of their own, which streams W
// once with plain float FMAs: a 64 x 64 MFMA tile would spend its time on rows
// that are not there.  A wave owns four features; its lanes stride along k in
// float4 pieces, the rows sit in LDS in stretches of 512 columns; a lane sums
// its share in the order of k and the 64 shares are added by a fixed tree, so
// an output does not depend on the other rows of the step.
#include "common.h"

#define FLAG_GELU 1
#define FLAG_ACCUMULATE 2

// Out-of-range loads read a clamped address and are zeroed afterwards with this
// constant: selecting between an address and a zero kept in a variable turns
// the load into a flat load through scratch memory.
#define ZERO4 make_float4(0.f, 0.f, 0.f, 0.f)

struct GemmArgs {
  const float* A;
  const float* W;
  const float* bias;
  float* out;
  int M, N, K;
  int lda, ldw, ldo;
  int flags;
};

#define BK 16
#define LDS_STRIDE (BK + 1)

// Rows of a tile beyond the matrix read a row inside it (their products are
// never stored): the row one tile back where there is one, so that they do not
// all read the matrix's last row at once, which one cache channel would have
// to serve to every block of that row of tiles.
__device__ __forceinline__ int row_inside(int r, int n, int tile) {
  return r < n ? r : (r - tile >= 0 && r - tile < n ? r - tile : n - 1);
}

// WM x WN waves of 64x64 (BIG) or 32x32 (small) wave tiles
template <int TM, int TN>  // 32x32 MFMA tiles per wave along m and n
__global__ __launch_bounds__(256) void gemm_f32_kernel(GemmArgs p) {
  constexpr int BM_ = 2 * TM * 32;
  constexpr int BN_ = 2 * TN * 32;
  __shared__ float As[BM_ * LDS_STRIDE];
  __shared__ float Bs[BN_ * LDS_STRIDE];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int m0 = blockIdx.y * BM_;
  const int n0 = blockIdx.x * BN_;

  f32x16_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // a k-block of a tile is BM_ x 16 floats = BM_*4 pieces of 16 bytes
  constexpr int PA = (BM_ * 4) / 256;
  constexpr int PB = (BN_ * 4) / 256;
  float4 ra[PA], rb[PB];

  auto load_global = [&](int k0) {
#pragma unroll
    for (int i = 0; i < PA; ++i) {
      const int c = tid + 256 * i;
      const int row = c >> 2, gk = k0 + (c & 3) * 4, gm = m0 + row;
      const float4 t = *(const float4*)(p.A + (size_t)row_inside(gm, p.M, BM_) * p.lda + min(gk, p.K - 4));
      ra[i] = (gm < p.M && gk < p.K) ? t : ZERO4;
    }
#pragma unroll
    for (int i = 0; i < PB; ++i) {
      const int c = tid + 256 * i;
      const int row = c >> 2, gk = k0 + (c & 3) * 4, gn = n0 + row;
      const float4 t = *(const float4*)(p.W + (size_t)row_inside(gn, p.N, BN_) * p.ldw + min(gk, p.K - 4));
      rb[i] = (gn < p.N && gk < p.K) ? t : ZERO4;
    }
  };
  auto store_lds = [&]() {
#pragma unroll
    for (int i = 0; i < PA; ++i) {
      const int c = tid + 256 * i;
      float* d = As + (c >> 2) * LDS_STRIDE + (c & 3) * 4;
      d[0] = ra[i].x, d[1] = ra[i].y, d[2] = ra[i].z, d[3] = ra[i].w;
    }
#pragma unroll
    for (int i = 0; i < PB; ++i) {
      const int c = tid + 256 * i;
      float* d = Bs + (c >> 2) * LDS_STRIDE + (c & 3) * 4;
      d[0] = rb[i].x, d[1] = rb[i].y, d[2] = rb[i].z, d[3] = rb[i].w;
    }
  };

  load_global(0);
  store_lds();
  __syncthreads();

  const int frag_row = lane & 31;
  const int frag_k = lane >> 5;

  for (int k0 = 0; k0 < p.K; k0 += BK) {
    const bool more = (k0 + BK) < p.K;
    if (more) load_global(k0 + BK);
#pragma unroll
    for (int ks = 0; ks < BK; ks += 2) {
      float a[TM], b[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i)
        a[i] = As[(wm * TM * 32 + i * 32 + frag_row) * LDS_STRIDE + ks + frag_k];
#pragma unroll
      for (int j = 0; j < TN; ++j)
        b[j] = Bs[(wn * TN * 32 + j * 32 + frag_row) * LDS_STRIDE + ks + frag_k];
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[j], acc[i][j], 0, 0, 0);
    }
    __syncthreads();
    if (more) {
      store_lds();
      __syncthreads();
    }
  }

  // Epilogue.  Accumulator r of a 32x32 tile: row 8*(r/4) + 4*(lane/32) + r%4,
  // column lane%32.  What is read (bias, the residual stream to add to) is
  // read for a whole 32x32 tile before anything is stored: a load that comes
  // after a store to memory it might alias waits for it, sixteen times over.
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int n = n0 + wn * TN * 32 + j * 32 + (lane & 31);
    const int nc = min(n, p.N - 1);
    const float bias = p.bias ? p.bias[nc] : 0.f;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int mb = m0 + wm * TM * 32 + i * 32 + 4 * (lane >> 5);
      float v[16];
      if (p.flags & FLAG_ACCUMULATE) {
#pragma unroll
        for (int r = 0; r < 16; ++r)
          v[r] = p.out[(size_t)min(mb + 8 * (r >> 2) + (r & 3), p.M - 1) * p.ldo + nc];
#pragma unroll
        for (int r = 0; r < 16; ++r) v[r] += acc[i][j][r] + bias;
      } else {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          v[r] = acc[i][j][r] + bias;
          if (p.flags & FLAG_GELU) v[r] = gelu_tanh(v[r]);
        }
      }
      if (n >= p.N) continue;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = mb + 8 * (r >> 2) + (r & 3);
        if (m < p.M) p.out[(size_t)m * p.ldo + n] = v[r];
      }
    }
  }
}

#define SKF_FW 4     // features a wave
#define SKF_KC 512   // columns of the rows held in LDS at a time

template <int MR>  // rows, rounded up to a power of two (rows that are not there are zero)
__global__ __launch_bounds__(256) void gemm_f32_skinny_kernel(GemmArgs p) {
  __shared__ float4 As[MR][SKF_KC / 4];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n_base = blockIdx.x * (4 * SKF_FW) + wave * SKF_FW;
  const float* wrow[SKF_FW];
#pragma unroll
  for (int f = 0; f < SKF_FW; ++f) wrow[f] = p.W + (size_t)min(n_base + f, p.N - 1) * p.ldw;

  float acc[SKF_FW][MR];
#pragma unroll
  for (int f = 0; f < SKF_FW; ++f)
#pragma unroll
    for (int m = 0; m < MR; ++m) acc[f][m] = 0.f;

  for (int k0 = 0; k0 < p.K; k0 += SKF_KC) {
    const int width = min(SKF_KC, p.K - k0);  // a multiple of 4
    // the weights first: they are on their way while the rows are copied into LDS
    // (columns beyond the stretch are read from inside it; they meet zeros in LDS)
    float4 w[SKF_KC / 256][SKF_FW];
#pragma unroll
    for (int j = 0; j < SKF_KC / 256; ++j)
#pragma unroll
      for (int f = 0; f < SKF_FW; ++f) w[j][f] = *(const float4*)(wrow[f] + k0 + min((lane + 64 * j) * 4, width - 4));
    __syncthreads();  // the stretch before is no longer read
    for (int i = tid; i < MR * (SKF_KC / 4); i += 256) {
      const int r = i / (SKF_KC / 4), c = i - r * (SKF_KC / 4);
      const float4 t = *(const float4*)(p.A + (size_t)min(r, p.M - 1) * p.lda + k0 + min(c * 4, width - 4));
      As[r][c] = (r < p.M && c * 4 < width) ? t : ZERO4;
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < SKF_KC / 256; ++j) {
      const int c = lane + 64 * j;
#pragma unroll
      for (int m = 0; m < MR; ++m) {
        const float4 a = As[m][c];
#pragma unroll
        for (int f = 0; f < SKF_FW; ++f) {
          acc[f][m] = fmaf(w[j][f].x, a.x, acc[f][m]);
          acc[f][m] = fmaf(w[j][f].y, a.y, acc[f][m]);
          acc[f][m] = fmaf(w[j][f].z, a.z, acc[f][m]);
          acc[f][m] = fmaf(w[j][f].w, a.w, acc[f][m]);
        }
      }
    }
  }
#pragma unroll
  for (int f = 0; f < SKF_FW; ++f) {
    const int n = n_base + f;
#pragma unroll
    for (int m = 0; m < MR; ++m) {
      float v = wave_sum(acc[f][m]);
      if (lane == 0 && n < p.N && m < p.M) {
        if (p.bias) v += p.bias[n];
        const size_t idx = (size_t)m * p.ldo + n;
        if (p.flags & FLAG_ACCUMULATE)
          p.out[idx] += v;
        else
          p.out[idx] = (p.flags & FLAG_GELU) ? gelu_tanh(v) : v;
      }
    }
  }
}

DEFINE_LAST_ERROR(mlxlm_last_error)

// variant: 0 = choose, 1 = 128x128 block tile, 2 = 64x64 block tile, 3 = the kernel for up to 16 rows
extern "C" int gemm_f32(void* out, const void* A, const void* W, const float* bias, int M, int N,
                        int K, int lda, int ldw, int ldo, int flags, int variant,
                        hipStream_t stream) {
  GemmArgs p;
  p.A = (const float*)A;
  p.W = (const float*)W;
  p.bias = bias;
  p.out = (float*)out;
  p.M = M, p.N = N, p.K = K;
  p.lda = lda, p.ldw = ldw, p.ldo = ldo;
  p.flags = flags;
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
  if (variant == 0) variant = M <= 16 ? 3 : (M <= 64 || (size_t)M * N < (size_t)128 * 128 * 128) ? 2 : 1;
  if (variant == 1) {
    dim3 grid((N + 127) / 128, (M + 127) / 128), block(256);
    hipLaunchKernelGGL((gemm_f32_kernel<2, 2>), grid, block, 0, stream, p);
  } else if (variant == 2) {
    dim3 grid((N + 63) / 64, (M + 63) / 64), block(256);
    hipLaunchKernelGGL((gemm_f32_kernel<1, 1>), grid, block, 0, stream, p);
  } else if (variant == 3) {
    if (M > 16) FAIL("gemm_f32: the kernel for few rows takes at most 16, got %d", M);
    dim3 grid((N + 4 * SKF_FW - 1) / (4 * SKF_FW)), block(256);
    if (M <= 1)
      hipLaunchKernelGGL(gemm_f32_skinny_kernel<1>, grid, block, 0, stream, p);
    else if (M <= 2)
      hipLaunchKernelGGL(gemm_f32_skinny_kernel<2>, grid, block, 0, stream, p);
    else if (M <= 4)
      hipLaunchKernelGGL(gemm_f32_skinny_kernel<4>, grid, block, 0, stream, p);
    else if (M <= 8)
      hipLaunchKernelGGL(gemm_f32_skinny_kernel<8>, grid, block, 0, stream, p);
    else
      hipLaunchKernelGGL(gemm_f32_skinny_kernel<16>, grid, block, 0, stream, p);
  } else {
    FAIL("gemm_f32: unknown variant %d", variant);
  }
  CHECK_LAUNCH("gemm_f32");
  return 0;
}
