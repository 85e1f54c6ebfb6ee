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

DEFINE_LAST_ERROR(mlxlm_last_error)

extern "C" int layernorm(void* out, const float* x, const int* rows, const float* gamma,
                         const float* beta, float eps, int n_rows, int width, int out_dtype,
                         hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (width <= 0) FAIL("layernorm: width %d must be positive", width);
  if (!out || !x) FAIL("layernorm: null pointer");
  dim3 grid(n_rows), block(256);
  if (out_dtype == DT_F32)
    hipLaunchKernelGGL(layernorm_kernel<float>, grid, block, 0, stream, (float*)out, x, rows, gamma,
                       beta, eps, width);
  else if (out_dtype == DT_BF16)
    hipLaunchKernelGGL(layernorm_kernel<bf16>, grid, block, 0, stream, (bf16*)out, x, rows, gamma,
                       beta, eps, width);
  else
    FAIL("layernorm: unknown dtype code %d", out_dtype);
  CHECK_LAUNCH("layernorm");
  return 0;
}
