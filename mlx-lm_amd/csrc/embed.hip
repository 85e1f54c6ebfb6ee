// Embedding gather with an optional second table added row by row:
//   out[t, :] = table[ids[t], :] (+ add_table[add_ids[t], :])
// The output is the 32-bit residual stream; tables are float or bfloat16.
// The reference does the two lookups and the sum as three array ops
// (mlx_lm/models/gpt2.py:132,137-144).
#include "common.h"

template <typename T>
__global__ __launch_bounds__(256) void embed_gather_add_kernel(
    float* __restrict__ out, const T* __restrict__ table, const int* __restrict__ ids,
    const T* __restrict__ add_table, const int* __restrict__ add_ids, int width) {
  const int t = blockIdx.x;
  const T* row = table + (size_t)ids[t] * width;
  const T* add = add_table ? add_table + (size_t)add_ids[t] * width : nullptr;
  float* o = out + (size_t)t * width;
  for (int d = threadIdx.x; d < width; d += blockDim.x) {
    float v = to_f32(row[d]);
    if (add) v += to_f32(add[d]);
    o[d] = v;
  }
}

// Tokens that a sampling kernel left on the device take their place among the
// step's token ids without a trip through the host: ids[t] = src[index[t]]
// where index[t] >= 0 (clamped into the vocabulary: nothing on the host has
// seen these values).  This is what lets the next decode step be launched
// before the host has read the tokens of this one, the job of mx.async_eval in
// the reference's loops (mlx_lm/generate.py:446-451,1449-1456).
__global__ void feed_tokens_kernel(int* __restrict__ ids, const int* __restrict__ src,
                                   const int* __restrict__ index, int n, int vocab) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= n) return;
  const int i = index[t];
  if (i >= 0) ids[t] = min(max(src[i], 0), vocab - 1);
}

DEFINE_LAST_ERROR(mlxlm_last_error)

extern "C" int feed_tokens(int* ids, const int* src, const int* index, int n, int vocab, hipStream_t stream) {
  if (n <= 0) return 0;
  if (!ids || !src || !index || vocab <= 0) FAIL("feed_tokens: null pointer or bad vocabulary %d", vocab);
  hipLaunchKernelGGL(feed_tokens_kernel, dim3((n + 255) / 256), dim3(256), 0, stream, ids, src, index, n, vocab);
  CHECK_LAUNCH("feed_tokens");
  return 0;
}

extern "C" int embed_gather_add(void* out, const void* table, const int* ids, const void* add_table,
                                const int* add_ids, int n_tokens, int width, int dtype,
                                hipStream_t stream) {
  if (n_tokens <= 0) return 0;
  if (width <= 0) FAIL("embed_gather_add: width %d must be positive", width);
  if (!out || !table || !ids) FAIL("embed_gather_add: null pointer");
  if (add_table && !add_ids) FAIL("embed_gather_add: add_table without add_ids");
  dim3 grid(n_tokens), block(256);
  if (dtype == DT_F32)
    hipLaunchKernelGGL(embed_gather_add_kernel<float>, grid, block, 0, stream, (float*)out,
                       (const float*)table, ids, (const float*)add_table, add_ids, width);
  else if (dtype == DT_BF16)
    hipLaunchKernelGGL(embed_gather_add_kernel<bf16>, grid, block, 0, stream, (float*)out,
                       (const bf16*)table, ids, (const bf16*)add_table, add_ids, width);
  else
    FAIL("embed_gather_add: unknown dtype code %d", dtype);
  CHECK_LAUNCH("embed_gather_add");
  return 0;
}
