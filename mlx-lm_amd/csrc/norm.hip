// LayerNorm over the last axis of the 32-bit residual stream:
//   y = (x - mean) / sqrt(var + eps) * gamma + beta      (biased variance)
// Statistics, scale and shift are computed in 32-bit; the output is float or
// bfloat16.  With `rows` given, output row r is made from input row rows[r]
// (used to norm only the rows whose logits are wanted).
// The reference's blocks call nn.LayerNorm(n_embd, eps=layer_norm_epsilon)
// (mlx_lm/models/gpt2.py:92-96,123,151).
#include "common.h"

template <typename T>
__global__ __launch_bounds__(256) void layernorm_kernel(T* __restrict__ out,
                                                        const float* __restrict__ x,
                                                        const int* __restrict__ rows,
                                                        const float* __restrict__ gamma,
                                                        const float* __restrict__ beta, float eps,
                                                        int width) {
  __shared__ float red[32];
  const int r = blockIdx.x;
  const float* xr = x + (size_t)(rows ? rows[r] : r) * width;
  T* o = out + (size_t)r * width;

  float s = 0.f;
  for (int d = threadIdx.x; d < width; d += blockDim.x) s += xr[d];
  const float mean = block_sum(s, red) / (float)width;

  float q = 0.f;
  for (int d = threadIdx.x; d < width; d += blockDim.x) {
    const float c = xr[d] - mean;
    q += c * c;
  }
  const float var = block_sum(q, red) / (float)width;
  const float rstd = 1.0f / sqrtf(var + eps);

  for (int d = threadIdx.x; d < width; d += blockDim.x) {
    float y = (xr[d] - mean) * rstd;
    if (gamma) y *= gamma[d];
    if (beta) y += beta[d];
    o[d] = from_f32<T>(y);
  }
}

// One wave a row, the row held in registers (NV float4 a lane): the input is
// read once, the statistics need no barrier.  width % 4 == 0, width <= 256 * NV.
template <typename T, int NV>
__global__ __launch_bounds__(256) void layernorm_wave_kernel(T* __restrict__ out,
                                                             const float* __restrict__ x,
                                                             const int* __restrict__ rows,
                                                             const float* __restrict__ gamma,
                                                             const float* __restrict__ beta,
                                                             float eps, int n_rows, int width, bool through) {
  const int lane = threadIdx.x & 63;
  const int r = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (r >= n_rows) return;  // whole waves leave; no barrier follows
  const float* xr = x + (size_t)(rows ? rows[r] : r) * width;
  float4 v[NV], g[NV], b[NV];
#pragma unroll
  for (int i = 0; i < NV; ++i) v[i] = *(const float4*)(xr + min((lane + 64 * i) * 4, width - 4));
  // scale and shift come in beside the row, not after its statistics
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int k = min((lane + 64 * i) * 4, width - 4);
    g[i] = gamma ? *(const float4*)(gamma + k) : make_float4(1.f, 1.f, 1.f, 1.f);
    b[i] = beta ? *(const float4*)(beta + k) : make_float4(0.f, 0.f, 0.f, 0.f);
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    if ((lane + 64 * i) * 4 >= width) v[i] = make_float4(0.f, 0.f, 0.f, 0.f);
    s += (v[i].x + v[i].y) + (v[i].z + v[i].w);
  }
  const float mean = wave_sum(s) / (float)width;
  float q = 0.f;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const float a = v[i].x - mean, b = v[i].y - mean, c = v[i].z - mean, d = v[i].w - mean;
    q += (lane + 64 * i) * 4 < width ? (a * a + b * b) + (c * c + d * d) : 0.f;
  }
  const float rstd = 1.0f / sqrtf(wave_sum(q) / (float)width + eps);
  T* o = out + (size_t)r * width;
  // (the next kernel reads the rows, this one does not: the stores go through to memory)
  const __amdgpu_buffer_rsrc_t out_buf = through_buffer(out, (size_t)n_rows * width * sizeof(T));
  const uint32_t o_at = (uint32_t)((size_t)r * width * sizeof(T));
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int k = (lane + 64 * i) * 4;
    if (k >= width) continue;
    const float y[4] = {(v[i].x - mean) * rstd * g[i].x + b[i].x, (v[i].y - mean) * rstd * g[i].y + b[i].y,
                        (v[i].z - mean) * rstd * g[i].z + b[i].z, (v[i].w - mean) * rstd * g[i].w + b[i].w};
    if constexpr (sizeof(T) == 4) {
      const u32x4_t t = {__float_as_uint(y[0]), __float_as_uint(y[1]), __float_as_uint(y[2]), __float_as_uint(y[3])};
      if (through)
        store_through(out_buf, o_at + k * 4, t);
      else
        *(u32x4_t*)((float*)o + k) = t;
    } else {
      const u32x2_t pk = {pack_bf16x2(y[0], y[1]), pack_bf16x2(y[2], y[3])};
      if (through)
        store_through(out_buf, o_at + k * 2, pk);
      else
        *(u32x2_t*)((uint16_t*)o + k) = pk;
    }
  }
}

template <typename T>
static void launch_wave(int nv, dim3 grid, hipStream_t stream, T* out, const float* x, const int* rows,
                        const float* gamma, const float* beta, float eps, int n_rows, int width) {
  dim3 block(256);
  const bool through = fits_through_buffer((size_t)n_rows * width * sizeof(T));
  if (nv <= 2)
    hipLaunchKernelGGL((layernorm_wave_kernel<T, 2>), grid, block, 0, stream, out, x, rows, gamma, beta, eps, n_rows, width, through);
  else if (nv <= 4)
    hipLaunchKernelGGL((layernorm_wave_kernel<T, 4>), grid, block, 0, stream, out, x, rows, gamma, beta, eps, n_rows, width, through);
  else if (nv <= 8)
    hipLaunchKernelGGL((layernorm_wave_kernel<T, 8>), grid, block, 0, stream, out, x, rows, gamma, beta, eps, n_rows, width, through);
  else
    hipLaunchKernelGGL((layernorm_wave_kernel<T, 16>), grid, block, 0, stream, out, x, rows, gamma, beta, eps, n_rows, width, through);
}

DEFINE_LAST_ERROR(mlxlm_last_error)

extern "C" int layernorm(void* out, const float* x, const int* rows, const float* gamma,
                         const float* beta, float eps, int n_rows, int width, int out_dtype,
                         hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (width <= 0) FAIL("layernorm: width %d must be positive", width);
  if (!out || !x) FAIL("layernorm: null pointer");
  if (out_dtype != DT_F32 && out_dtype != DT_BF16) FAIL("layernorm: unknown dtype code %d", out_dtype);
  const bool aligned = !(((uintptr_t)x | (uintptr_t)out | (uintptr_t)gamma | (uintptr_t)beta) & 15);
  if (width % 4 == 0 && width <= 4096 && aligned) {  // a wave a row
    const int nv = (width / 4 + 63) / 64;
    dim3 grid((n_rows + 3) / 4);
    if (out_dtype == DT_F32)
      launch_wave<float>(nv, grid, stream, (float*)out, x, rows, gamma, beta, eps, n_rows, width);
    else
      launch_wave<bf16>(nv, grid, stream, (bf16*)out, x, rows, gamma, beta, eps, n_rows, width);
  } else {
    dim3 grid(n_rows), block(256);
    if (out_dtype == DT_F32)
      hipLaunchKernelGGL(layernorm_kernel<float>, grid, block, 0, stream, (float*)out, x, rows, gamma,
                         beta, eps, width);
    else
      hipLaunchKernelGGL(layernorm_kernel<bf16>, grid, block, 0, stream, (bf16*)out, x, rows, gamma,
                         beta, eps, width);
  }
  CHECK_LAUNCH("layernorm");
  return 0;
}
