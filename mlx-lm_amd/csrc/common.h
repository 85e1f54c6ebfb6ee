// Shared device helpers for the gfx950 kernels: element types, 64-lane wave
// reductions, block reductions through LDS and the error channel that every
// extern "C" entry point uses.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#define WAVE 64

// element type codes shared with the Python side
#define DT_F32 0
#define DT_BF16 1

struct bf16 {
  uint16_t bits;
};

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;

__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(bf16 v) {
  return __uint_as_float(((uint32_t)v.bits) << 16);
}
__device__ __forceinline__ float bits_to_f32(uint16_t b) {
  return __uint_as_float(((uint32_t)b) << 16);
}

// Round to nearest even, NaN kept quiet: gfx950 has an instruction for it
// (v_cvt_pk_bf16_f32, two values at a time), which the compiler picks for the
// conversion of a float vector to __bf16.
typedef __bf16 hw_bf16x2_t __attribute__((ext_vector_type(2)));
typedef float hw_f32x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  const hw_f32x2_t v = {lo, hi};
  const hw_bf16x2_t b = __builtin_convertvector(v, hw_bf16x2_t);
  return __builtin_bit_cast(uint32_t, b);
}
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
  return (uint16_t)(pack_bf16x2(f, 0.f) & 0xffffu);
}

template <typename T>
__device__ __forceinline__ T from_f32(float v);
template <>
__device__ __forceinline__ float from_f32<float>(float v) {
  return v;
}
template <>
__device__ __forceinline__ bf16 from_f32<bf16>(float v) {
  bf16 r;
  r.bits = f32_to_bf16_bits(v);
  return r;
}

// Reductions over a wave.  Inside a row of 16 lanes the values move through the
// data-parallel primitives of the vector unit (swaps within quads, a mirror of
// 8 lanes, a mirror of 16), which cost an instruction each; a shuffle through
// __shfl_xor goes through the LDS crossbar and takes some 60 ns, six of them in
// a row for a sum.  The four rows' results are read as scalars and joined in a
// fixed order.  Every lane gets the result.
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
#define DPP_QUAD_SWAP1 0xB1     // quad_perm [1, 0, 3, 2]
#define DPP_QUAD_SWAP2 0x4E     // quad_perm [2, 3, 0, 1]
#define DPP_HALF_MIRROR 0x141   // lane i of each 8 reads lane 7 - i
#define DPP_ROW_MIRROR 0x140    // lane i of each 16 reads lane 15 - i
__device__ __forceinline__ float lane_value(float v, int lane) {
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}
// sum (max) over each group of 4, 8 or 16 neighbouring lanes, in every lane of the group
template <int GROUP>
__device__ __forceinline__ float group_sum(float v) {
  v += dpp_move<DPP_QUAD_SWAP1>(v);
  v += dpp_move<DPP_QUAD_SWAP2>(v);
  if (GROUP >= 8) v += dpp_move<DPP_HALF_MIRROR>(v);
  if (GROUP >= 16) v += dpp_move<DPP_ROW_MIRROR>(v);
  return v;
}
template <int GROUP>
__device__ __forceinline__ float group_max(float v) {
  v = fmaxf(v, dpp_move<DPP_QUAD_SWAP1>(v));
  v = fmaxf(v, dpp_move<DPP_QUAD_SWAP2>(v));
  if (GROUP >= 8) v = fmaxf(v, dpp_move<DPP_HALF_MIRROR>(v));
  if (GROUP >= 16) v = fmaxf(v, dpp_move<DPP_ROW_MIRROR>(v));
  return v;
}
__device__ __forceinline__ float wave_sum(float v) {
  v = group_sum<16>(v);
  return (lane_value(v, 0) + lane_value(v, 16)) + (lane_value(v, 32) + lane_value(v, 48));
}
__device__ __forceinline__ float wave_max(float v) {
  v = group_max<16>(v);
  return fmaxf(fmaxf(lane_value(v, 0), lane_value(v, 16)), fmaxf(lane_value(v, 32), lane_value(v, 48)));
}

// tanh-GELU: 0.5 x (1 + tanh(u)) with u = sqrt(2/pi) (x + 0.044715 x^3), written
// as x / (1 + exp(-2u)): one exponential and one division instead of a tanh.
// `gelu_tanh` keeps float accuracy; `gelu_tanh_fast` is eight instructions on the hardware's
// exponential and reciprocal (an ulp or two each; written with `__expf` and `__fdividef` it
// was nineteen, the division alone eleven), for results that are rounded to bfloat16 anyway.
// Large |x| gives x or -0 without special cases.
__device__ __forceinline__ float gelu_tanh(float x) {
  const float u = 0.7978845608028654f * (x + 0.044715f * x * x * x);
  return x / (1.0f + expf(-2.0f * u));
}
__device__ __forceinline__ float gelu_tanh_fast(float x) {
  // exp(-2u) = 2^(x (c1 + c2 x^2)) with c1 = -2 sqrt(2/pi) log2(e), c2 = 0.044715 c1
  constexpr float c1 = -2.0f * 0.7978845608028654f * 1.4426950408889634f, c2 = c1 * 0.044715f;
  const float e = __builtin_amdgcn_exp2f(x * __builtin_fmaf(x * x, c2, c1));
  return x * __builtin_amdgcn_rcpf(1.0f + e);
}

// Sum over a block of up to 1024 threads; `red` is LDS of at least 17 floats.
// Every thread gets the result.  Safe to call repeatedly with the same `red`.
__device__ __forceinline__ float block_sum(float v, float* red) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int nw = (blockDim.x + 63) >> 6;
  v = wave_sum(v);
  __syncthreads();
  if (lane == 0) red[wave] = v;
  __syncthreads();
  float t = 0.f;
  for (int i = 0; i < nw; ++i) t += red[i];
  return t;
}
__device__ __forceinline__ float block_max(float v, float* red) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int nw = (blockDim.x + 63) >> 6;
  v = wave_max(v);
  __syncthreads();
  if (lane == 0) red[wave] = v;
  __syncthreads();
  float t = red[0];
  for (int i = 1; i < nw; ++i) t = fmaxf(t, red[i]);
  return t;
}

// Stores that go through to memory as they are issued (system scope: sc0 sc1).  When a kernel
// ends, what its stores left dirty in the eight L2s is written back before the next kernel may
// start: 9 us after a product that wrote 26 MB, 3 us when the stores had gone through at once,
// spread over the kernel's last microseconds.  For outputs of megabytes that the same kernel does
// not read again.  The compiler takes a cache policy only on buffer stores, so the output is
// described as a buffer: offsets are 32-bit byte offsets from its base, and the hardware drops a
// store at or beyond `bytes` (which must be below 4 GB; `fits_through_buffer` on the host).
typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
#define BUFFER_WORD3 0x00020000  // untyped 32-bit data, no swizzle
#define POLICY_THROUGH 0x11      // sc0 | sc1
__device__ __forceinline__ __amdgpu_buffer_rsrc_t through_buffer(void* base, size_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(base, 0, (int)(uint32_t)bytes, BUFFER_WORD3);
}
__device__ __forceinline__ void store_through(__amdgpu_buffer_rsrc_t r, uint32_t byte_offset, u32x4_t v) {
  __builtin_amdgcn_raw_buffer_store_b128(v, r, (int)byte_offset, 0, POLICY_THROUGH);
}
typedef unsigned int u32x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ void store_through(__amdgpu_buffer_rsrc_t r, uint32_t byte_offset, u32x2_t v) {
  __builtin_amdgcn_raw_buffer_store_b64(v, r, (int)byte_offset, 0, POLICY_THROUGH);
}
__device__ __forceinline__ void store_through(__amdgpu_buffer_rsrc_t r, uint32_t byte_offset, float v) {
  __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned int, v), r, (int)byte_offset, 0, POLICY_THROUGH);
}
static inline bool fits_through_buffer(size_t bytes) { return bytes < ((size_t)1 << 32); }

// ---------------------------------------------------------------------------
// host side: the device's size; one error string per thread, returned codes are 0 (ok) or 1.

// Dies (XCDs) of the GPU: consecutive blocks of a launch go to the dies in turn, and each die has
// an L2 of its own.  (Kernels that deal tiles or chunks to dies index with it too.)
#define N_DIES 8

// Compute units of the current device, asked of the device once (256 on an MI355X).
static inline int n_compute_units() {
  static int n = 0;
  if (n == 0) {
    int dev = 0, v = 0;
    if (hipGetDevice(&dev) == hipSuccess &&
        hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0)
      n = v;
    else
      n = 256;
  }
  return n;
}

static thread_local char g_err[512];

#define FAIL(...)                               \
  do {                                          \
    snprintf(g_err, sizeof(g_err), __VA_ARGS__); \
    return 1;                                   \
  } while (0)

#define CHECK_LAUNCH(name)                                                    \
  do {                                                                        \
    hipError_t e_ = hipGetLastError();                                        \
    if (e_ != hipSuccess) FAIL("%s: launch failed: %s", name, hipGetErrorString(e_)); \
  } while (0)

#define DEFINE_LAST_ERROR(fn) \
  extern "C" const char* fn() { return g_err; }

// Where element (m, n) of an activation matrix lies in the packed order: tiles of 16 rows x 64
// columns, `kblocks` of them a tile row ((N + 63) / 64); in a tile the 8 values n = 16 g + 8 h + 0..7
// of row f lie at ((4 h + g) * 16 + f) * 8, so that lane l of a wave (row l % 16, g = l / 16) reads
// 16 bytes at l * 8 (h = 0) and at 512 + l * 8 (h = 1): a wave's load is 1 KB of consecutive bytes,
// as with the packed weights.  Rows as an MFMA operand straight from a row-major matrix are
// sixteen pieces of 64 bytes a load, which a CU fetches at a third of the speed.  Kernels that
// make the rows of a product of 17 to 64 rows (the sum-and-norm, decode attention, that product's
// own epilogue) write this order where the host asks for it.
__device__ __forceinline__ size_t packed_at(int m, int n, int kblocks) {
  const int kk = n & 63;
  return ((size_t)(m >> 4) * kblocks + (n >> 6)) * 1024 + ((((kk >> 3) & 1) * 4 + (kk >> 4)) * 16 + (m & 15)) * 8 + (kk & 7);
}
