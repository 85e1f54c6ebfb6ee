// Causal attention over a paged key/value cache, float or bfloat16 storage,
// all arithmetic (scores, softmax, weighted sum) in 32-bit.
//
// A step's tokens lie in one flat list; token t belongs to request
// token_req[t] and sits at absolute position positions[t].  Its keys are
// positions max(0, pos - window + 1) .. pos of the same request (window 0 =
// all of them), found through the request's row of the block table:
// position p lives in page block_table[req][p / page_size], row p % page_size.
// A page of one cache slot holds [n_kv_heads][page_size][head_dim] keys and
// the same for values.  Query head h reads key head h / (n_heads/n_kv_heads).
//
// Replaces cache.update_and_fetch + scaled_dot_product_attention of the
// reference (mlx_lm/models/gpt2.py:60-65, mlx_lm/models/base.py:132-139,
// mlx_lm/models/cache.py:333-355) and its causal/window masks
// (mlx_lm/models/base.py:24-35).
//
// Kernels:
//  * kv_write: scatter this step's keys and values into their pages.
//  * attn_tile: 16 consecutive queries of one request per block, key tiles
//    of 64 staged in LDS; any head_dim that is a multiple of 16 up to 256.
//    Float caches with head_dim 64 or 128 in pages of whole 16 keys take
//    attn_tile_mfma instead: a wave a tile, v_mfma_f32_16x16x4_f32, no LDS.
//  * attn_row: one query per block, its keys split over the block's four
//    waves and over `n_splits` blocks; attn_merge joins the splits.
#include "common.h"
#include "attention_tiles.h"

struct AttnArgs {
  void* out;          // [n_tokens, n_heads*head_dim]
  const void* q;      // first query element; row stride ldq
  const void* k_pages;
  const void* v_pages;
  const int* block_table;  // [n_requests, max_blocks]
  const int* token_req;    // [n_tokens]
  const int* positions;    // [n_tokens]
  const int* items;        // tiles: (first row, n rows) pairs; rows: flat row indices
  float* part_o;           // [n_items, n_heads, n_splits, head_dim]
  float* part_ml;          // [n_items, n_heads, n_splits, 2]
  size_t page_stride;      // elements between pages
  int ldq, ldo;
  int max_blocks;
  int n_heads, n_kv_heads, head_dim, page_size;
  int window;
  int n_splits;
  float scale;
};

#define KT 64   // keys per tile
#define QT ATTN_TILE_QUERIES  // queries per block in attn_tile

template <typename T>
struct Vec;
template <>
struct Vec<float> {
  static constexpr int N = 4;
  typedef float4 type;
  static __device__ __forceinline__ void unpack(const type& v, float* f) {
    f[0] = v.x, f[1] = v.y, f[2] = v.z, f[3] = v.w;
  }
};
template <>
struct Vec<bf16> {
  static constexpr int N = 8;
  typedef uint4 type;
  static __device__ __forceinline__ void unpack(const type& v, float* f) {
    f[0] = __uint_as_float(v.x << 16), f[1] = __uint_as_float(v.x & 0xffff0000u);
    f[2] = __uint_as_float(v.y << 16), f[3] = __uint_as_float(v.y & 0xffff0000u);
    f[4] = __uint_as_float(v.z << 16), f[5] = __uint_as_float(v.z & 0xffff0000u);
    f[6] = __uint_as_float(v.w << 16), f[7] = __uint_as_float(v.w & 0xffff0000u);
  }
};

// Copy keys (or values) kt .. kt+KT-1 of one request and key head into LDS as
// floats, `n_threads` threads taking part; rows outside [lo, hi) become zero.
template <typename T>
__device__ __forceinline__ void stage_tile(float* dst, int dst_stride, const T* pages,
                                           const int* table, const AttnArgs& p, int kv_head, int kt,
                                           int lo, int hi, int tid, int n_threads) {
  constexpr int VN = Vec<T>::N;
  const int chunks = p.head_dim / VN;
  const int total = KT * chunks;
  for (int c = tid; c < total; c += n_threads) {
    const int key = c / chunks, part = c - key * chunks;
    const int pos = kt + key;
    float f[VN];
    if (pos >= lo && pos < hi) {
      const int page = table[pos / p.page_size];
      const T* src = pages + (size_t)page * p.page_stride +
                     ((size_t)kv_head * p.page_size + (pos % p.page_size)) * p.head_dim +
                     part * VN;
      const typename Vec<T>::type v = *(const typename Vec<T>::type*)src;
      Vec<T>::unpack(v, f);
    } else {
#pragma unroll
      for (int i = 0; i < VN; ++i) f[i] = 0.f;
    }
    float* d = dst + key * dst_stride + part * VN;
#pragma unroll
    for (int i = 0; i < VN; ++i) d[i] = f[i];
  }
}

// ---------------------------------------------------------------------------

template <typename T>
__global__ __launch_bounds__(256) void kv_write_kernel(const T* __restrict__ k_src,
                                                       const T* __restrict__ v_src, int ld_src,
                                                       T* __restrict__ k_pages,
                                                       T* __restrict__ v_pages, size_t page_stride,
                                                       const int* __restrict__ block_table,
                                                       int max_blocks,
                                                       const int* __restrict__ token_req,
                                                       const int* __restrict__ positions,
                                                       int n_kv_heads, int head_dim,
                                                       int page_size) {
  const int t = blockIdx.x;
  const int pos = positions[t];
  const int page = block_table[(size_t)token_req[t] * max_blocks + pos / page_size];
  const int row = pos % page_size;
  const int width = n_kv_heads * head_dim;
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    const int h = c / head_dim, d = c - h * head_dim;
    const size_t dst = (size_t)page * page_stride + ((size_t)h * page_size + row) * head_dim + d;
    k_pages[dst] = k_src[(size_t)t * ld_src + c];
    v_pages[dst] = v_src[(size_t)t * ld_src + c];
  }
}

// The same, 16 bytes a thread (head_dim a multiple of the vector, rows and pages aligned).
template <typename T>
__global__ __launch_bounds__(256) void kv_write_vec_kernel(const T* __restrict__ k_src,
                                                           const T* __restrict__ v_src, int ld_src,
                                                           T* __restrict__ k_pages,
                                                           T* __restrict__ v_pages, size_t page_stride,
                                                           const int* __restrict__ block_table,
                                                           int max_blocks,
                                                           const int* __restrict__ token_req,
                                                           const int* __restrict__ positions,
                                                           int n_kv_heads, int head_dim,
                                                           int page_size) {
  constexpr int VN = 16 / sizeof(T);
  const int t = blockIdx.x;
  const int pos = positions[t];
  const int page = block_table[(size_t)token_req[t] * max_blocks + pos / page_size];
  const int row = pos % page_size;
  const int chunks = n_kv_heads * head_dim / VN;
  for (int c = threadIdx.x; c < chunks; c += blockDim.x) {
    const int col = c * VN;
    const int h = col / head_dim, d = col - h * head_dim;
    const size_t dst = (size_t)page * page_stride + ((size_t)h * page_size + row) * head_dim + d;
    const uint4 kk = *(const uint4*)(k_src + (size_t)t * ld_src + col);
    const uint4 vv = *(const uint4*)(v_src + (size_t)t * ld_src + col);
    *(uint4*)(k_pages + dst) = kk;
    *(uint4*)(v_pages + dst) = vv;
  }
}

// ---------------------------------------------------------------------------
// attn_tile: grid (n_tiles, n_heads), 256 threads.  Wave w owns queries
// 4w .. 4w+3 of the tile.  In the score phase a lane is a key, in the
// weighted-sum phase a lane is a set of head_dim columns (lane, lane+64, ...).

template <typename T>
__global__ __launch_bounds__(256) void attn_tile_kernel(AttnArgs p) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  const int hd = p.head_dim;
  const int kv_stride = hd + 1;
  float* Qs = lds;                    // [QT][hd], scaled
  float* KVs = Qs + QT * hd;          // [KT][hd+1]
  float* Ps = KVs + KT * kv_stride;   // [QT][KT]

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int row0 = p.items[2 * blockIdx.x];
  const int nq = p.items[2 * blockIdx.x + 1];
  const int h = blockIdx.y;
  const int kv_head = h / (p.n_heads / p.n_kv_heads);
  const int req = p.token_req[row0];
  const int pos0 = p.positions[row0];
  const int* table = p.block_table + (size_t)req * p.max_blocks;
  const T* q = (const T*)p.q;
  const T* k_pages = (const T*)p.k_pages;
  const T* v_pages = (const T*)p.v_pages;

  for (int c = tid; c < QT * hd; c += 256) {
    const int qi = c / hd, d = c - qi * hd;
    Qs[c] = qi < nq ? to_f32(q[(size_t)(row0 + qi) * p.ldq + h * hd + d]) * p.scale : 0.f;
  }

  const int k_hi = pos0 + nq;  // one past the last key any query of the tile sees
  const int k_lo = p.window > 0 ? max(0, pos0 - p.window + 1) : 0;
  const int kt0 = (k_lo / KT) * KT;

  float m[4], l[4], o[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    m[i] = -INFINITY, l[i] = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) o[i][j] = 0.f;
  }

  for (int kt = kt0; kt < k_hi; kt += KT) {
    __syncthreads();  // previous tile's values are no longer read; Qs is written
    stage_tile<T>(KVs, kv_stride, k_pages, table, p, kv_head, kt, k_lo, k_hi, tid, 256);
    __syncthreads();
    const int kpos = kt + lane;
    const float* krow = KVs + lane * kv_stride;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int qi = wave * 4 + i;
      const int qpos = pos0 + qi;
      const float* qrow = Qs + qi * hd;
      float s = 0.f;
      for (int d = 0; d < hd; d += 4) {
        const float4 qv = *(const float4*)(qrow + d);
        s += qv.x * krow[d] + qv.y * krow[d + 1] + qv.z * krow[d + 2] + qv.w * krow[d + 3];
      }
      bool ok = qi < nq && kpos <= qpos && kpos >= k_lo;
      if (p.window > 0) ok = ok && kpos > qpos - p.window;
      s = ok ? s : -INFINITY;
      const float m_new = fmaxf(m[i], wave_max(s));
      float pr = 0.f, alpha = 1.f;
      if (m_new != -INFINITY) {
        pr = ok ? expf(s - m_new) : 0.f;
        alpha = expf(m[i] - m_new);
      }
      l[i] = l[i] * alpha + wave_sum(pr);
#pragma unroll
      for (int j = 0; j < 4; ++j) o[i][j] *= alpha;
      m[i] = m_new;
      Ps[qi * KT + lane] = pr;
    }
    __syncthreads();  // keys are no longer read
    stage_tile<T>(KVs, kv_stride, v_pages, table, p, kv_head, kt, k_lo, k_hi, tid, 256);
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float* prow = Ps + (wave * 4 + i) * KT;
      for (int key = 0; key < KT; ++key) {
        const float pv = prow[key];
        const float* vrow = KVs + key * kv_stride;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int d = lane + 64 * j;
          if (d < hd) o[i][j] += pv * vrow[d];
        }
      }
    }
  }

  T* out = (T*)p.out;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int qi = wave * 4 + i;
    if (qi >= nq) continue;
    const float inv = 1.0f / l[i];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int d = lane + 64 * j;
      if (d < hd) out[(size_t)(row0 + qi) * p.ldo + h * hd + d] = from_f32<T>(o[i][j] * inv);
    }
  }
}

// ---------------------------------------------------------------------------
// attn_tile_mfma: float storage, head_dim = 64 * NV, page_size a multiple of 16.  Grid
// (ceil(n_tiles / 4), n_heads), 256 threads; every wave takes a tile of its own and walks its
// keys 16 at a time (no LDS, no barrier).  v_mfma_f32_16x16x4_f32 computes D = A B for A 16 x 4
// and B 4 x 16: lane l brings A[l % 16][l / 16] and B[l / 16][l % 16] and gets
// D[4 * (l / 16) + r][l % 16] in accumulator r.
//   scores, transposed: S^T[key][query] = sum_d K[key][d] Q[query][d].  The four floats of one
//     16-byte load go to four instructions; which d an instruction's four slots stand for is
//     free as long as both operands agree: lane (x = l % 16, g = l / 16) loads columns
//     16 * t + 4 * g .. + 3 of key x and of query x.  Accumulator r is key 4 * g + r, query x.
//   softmax runs per query, which is one lane column: the four keys of a lane, then the four
//     lane groups by two shuffles.
//   output, transposed: O^T[column][query] = sum_key V[key][column] P[key][query].  The scores'
//     accumulator r is the second operand as it stands, with slot g standing for key 4 * g + r;
//     the first is V[key 4 * g + r][columns 4 * x .. + 3], one 16-byte load of a row that the 16
//     lanes read whole, its four floats going to four accumulators: accumulator r' of the c-th
//     is column 16 * g + 4 * r' + c, so a lane ends with 16 consecutive columns of its query.
// Keys of a tile beyond the last one written are read from that one instead (their scores are
// masked; a page's unwritten rows may hold anything, and 0 x NaN is NaN).

template <int NV>
__global__ __launch_bounds__(256) void attn_tile_mfma_kernel(AttnArgs p, int n_tiles) {
  constexpr int HD = 64 * NV;
  constexpr int NT = 4 * NV;  // 16-byte loads that cover a row of HD floats, per lane group
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int tile = blockIdx.x * 4 + wave;
  if (tile >= n_tiles) return;
  const int x = lane & 15, g = lane >> 4;
  // (the same in every lane: said so, the page numbers below come through scalar loads)
  const int row0 = __builtin_amdgcn_readfirstlane(p.items[2 * tile]);
  const int nq = __builtin_amdgcn_readfirstlane(p.items[2 * tile + 1]);
  const int h = blockIdx.y;
  const int kv_head = h / (p.n_heads / p.n_kv_heads);
  const int req = __builtin_amdgcn_readfirstlane(p.token_req[row0]);
  const int pos0 = __builtin_amdgcn_readfirstlane(p.positions[row0]);
  const int* table = p.block_table + (size_t)req * p.max_blocks;
  const float* k_pages = (const float*)p.k_pages;
  const float* v_pages = (const float*)p.v_pages;

  f32x4_t qv[NT];
  {
    const float* qrow = (const float*)p.q + (size_t)(row0 + min(x, nq - 1)) * p.ldq + h * HD + 4 * g;
#pragma unroll
    for (int t = 0; t < NT; ++t) qv[t] = *(const f32x4_t*)(qrow + 16 * t) * p.scale;
  }
  const int qpos = pos0 + x;
  const int k_hi = pos0 + nq;  // one past the last key any query of the tile sees
  const int k_lo = p.window > 0 ? max(0, pos0 - p.window + 1) : 0;
  const size_t head_off = (size_t)kv_head * p.page_size * HD;

  f32x4_t kf[NT], vf[NV][4];
  auto ask = [&](int kt, int page) {
    const size_t base = (size_t)page * p.page_stride + head_off;
    const int in_page = kt % p.page_size;
    const float* krow = k_pages + base + (size_t)(in_page + min(x, k_hi - 1 - kt)) * HD + 4 * g;
#pragma unroll
    for (int t = 0; t < NT; ++t) kf[t] = *(const f32x4_t*)(krow + 16 * t);
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const float* vrow = v_pages + base + (size_t)(in_page + min(4 * g + r, k_hi - 1 - kt)) * HD + 4 * x;
#pragma unroll
      for (int v = 0; v < NV; ++v) vf[v][r] = *(const f32x4_t*)(vrow + 64 * v);
    }
  };

  float m = -INFINITY, l = 0.f;
  f32x4_t o[NT];
#pragma unroll
  for (int i = 0; i < NT; ++i) o[i] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  // the page of the tile after next is looked up while the next tile's keys are on their way
  int kt = (k_lo / 16) * 16;
  const int last_block = (k_hi - 1) / p.page_size;
  ask(kt, table[kt / p.page_size]);
  int page_next = table[min((kt + 16) / p.page_size, last_block)];
  for (; kt < k_hi; kt += 16) {
    f32x4_t s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      s = __builtin_amdgcn_mfma_f32_16x16x4f32(kf[t].x, qv[t].x, s, 0, 0, 0);
      s = __builtin_amdgcn_mfma_f32_16x16x4f32(kf[t].y, qv[t].y, s, 0, 0, 0);
      s = __builtin_amdgcn_mfma_f32_16x16x4f32(kf[t].z, qv[t].z, s, 0, 0, 0);
      s = __builtin_amdgcn_mfma_f32_16x16x4f32(kf[t].w, qv[t].w, s, 0, 0, 0);
    }
    f32x4_t vc[NV][4];
#pragma unroll
    for (int v = 0; v < NV; ++v)
#pragma unroll
      for (int r = 0; r < 4; ++r) vc[v][r] = vf[v][r];
    ask(min(kt + 16, ((k_hi - 1) / 16) * 16), page_next);  // the next tile (after the last: the last again)
    page_next = table[min((kt + 32) / p.page_size, last_block)];
    __builtin_amdgcn_sched_barrier(0);  // (the loads stay here, ahead of the softmax and the second products)

    bool ok[4];
    float tmax = -INFINITY;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int key = kt + 4 * g + r;
      ok[r] = x < nq && key <= qpos && key >= k_lo && (p.window == 0 || key > qpos - p.window);
      tmax = fmaxf(tmax, ok[r] ? s[r] : -INFINITY);
    }
    tmax = fmaxf(tmax, __shfl_xor(tmax, 16, WAVE));
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, WAVE));
    const float m_new = fmaxf(m, tmax);
    float alpha = 1.f, sum = 0.f;
    f32x4_t pr = {0.f, 0.f, 0.f, 0.f};
    if (m_new != -INFINITY) {
      alpha = expf(m - m_new);
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        pr[r] = ok[r] ? expf(s[r] - m_new) : 0.f;
        sum += pr[r];
      }
    }
    sum += __shfl_xor(sum, 16, WAVE);
    sum += __shfl_xor(sum, 32, WAVE);
    l = l * alpha + sum;
    m = m_new;
#pragma unroll
    for (int i = 0; i < NT; ++i) o[i] *= alpha;
#pragma unroll
    for (int v = 0; v < NV; ++v)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        o[4 * v + 0] = __builtin_amdgcn_mfma_f32_16x16x4f32(vc[v][r].x, pr[r], o[4 * v + 0], 0, 0, 0);
        o[4 * v + 1] = __builtin_amdgcn_mfma_f32_16x16x4f32(vc[v][r].y, pr[r], o[4 * v + 1], 0, 0, 0);
        o[4 * v + 2] = __builtin_amdgcn_mfma_f32_16x16x4f32(vc[v][r].z, pr[r], o[4 * v + 2], 0, 0, 0);
        o[4 * v + 3] = __builtin_amdgcn_mfma_f32_16x16x4f32(vc[v][r].w, pr[r], o[4 * v + 3], 0, 0, 0);
      }
  }

  if (x < nq) {
    const float inv = 1.0f / l;
    float* orow = (float*)p.out + (size_t)(row0 + x) * p.ldo + h * HD + 16 * g;
#pragma unroll
    for (int v = 0; v < NV; ++v)
#pragma unroll
      for (int r = 0; r < 4; ++r)
        *(f32x4_t*)(orow + 64 * v + 4 * r) =
            f32x4_t{o[4 * v][r], o[4 * v + 1][r], o[4 * v + 2][r], o[4 * v + 3][r]} * inv;
  }
}

// ---------------------------------------------------------------------------
// attn_row: grid (n_rows, n_heads, n_splits), 256 threads.  The row's keys
// are cut into n_splits runs of whole tiles; inside a block wave w takes the
// tiles w, w+4, ... of its run.  Each wave stages its tile in its own LDS
// region.  The four waves' states are merged at the end; with n_splits == 1
// the result is final, otherwise the split's (max, sum, unnormalised output)
// goes to the partial buffers for attn_merge.

template <typename T>
__global__ __launch_bounds__(256) void attn_row_kernel(AttnArgs p) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  const int hd = p.head_dim;
  const int kv_stride = hd + 1;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  float* Qs = lds;                                      // [hd]
  float* KVs = Qs + hd + wave * (KT * kv_stride);       // this wave's [KT][hd+1]
  float* Ps = lds + hd + 4 * (KT * kv_stride) + wave * KT;  // this wave's [KT]
  float* Ms = lds + hd + 4 * (KT * kv_stride) + 4 * KT;     // [4] max, [4] sum, [4][hd] out
  float* Ls = Ms + 4;
  float* Os = Ls + 4;

  const int item = blockIdx.x;
  const int row = p.items[item];
  const int h = blockIdx.y;
  const int split = blockIdx.z;
  const int kv_head = h / (p.n_heads / p.n_kv_heads);
  const int req = p.token_req[row];
  const int pos = p.positions[row];
  const int* table = p.block_table + (size_t)req * p.max_blocks;
  const T* q = (const T*)p.q;
  const T* k_pages = (const T*)p.k_pages;
  const T* v_pages = (const T*)p.v_pages;

  for (int d = tid; d < hd; d += 256) Qs[d] = to_f32(q[(size_t)row * p.ldq + h * hd + d]) * p.scale;

  const int k_hi = pos + 1;
  const int k_lo = p.window > 0 ? max(0, pos - p.window + 1) : 0;
  const int kt0 = (k_lo / KT) * KT;
  const int n_tiles = (k_hi - kt0 + KT - 1) / KT;
  const int tiles_per_split = (n_tiles + p.n_splits - 1) / p.n_splits;
  const int t_begin = split * tiles_per_split;
  const int t_end = min(n_tiles, t_begin + tiles_per_split);
  const int rounds = (max(0, t_end - t_begin) + 3) / 4;

  float m = -INFINITY, l = 0.f, o[4] = {0.f, 0.f, 0.f, 0.f};
  __syncthreads();

  for (int r = 0; r < rounds; ++r) {
    const int tile = t_begin + r * 4 + wave;
    const bool active = tile < t_end;
    const int kt = kt0 + tile * KT;
    if (active) stage_tile<T>(KVs, kv_stride, k_pages, table, p, kv_head, kt, k_lo, k_hi, lane, 64);
    __syncthreads();
    if (active) {
      const int kpos = kt + lane;
      const float* krow = KVs + lane * kv_stride;
      float s = 0.f;
      for (int d = 0; d < hd; d += 4) {
        const float4 qv = *(const float4*)(Qs + d);
        s += qv.x * krow[d] + qv.y * krow[d + 1] + qv.z * krow[d + 2] + qv.w * krow[d + 3];
      }
      const bool ok = kpos >= k_lo && kpos < k_hi;
      s = ok ? s : -INFINITY;
      const float m_new = fmaxf(m, wave_max(s));
      float pr = 0.f, alpha = 1.f;
      if (m_new != -INFINITY) {
        pr = ok ? expf(s - m_new) : 0.f;
        alpha = expf(m - m_new);
      }
      l = l * alpha + wave_sum(pr);
#pragma unroll
      for (int j = 0; j < 4; ++j) o[j] *= alpha;
      m = m_new;
      Ps[lane] = pr;
    }
    __syncthreads();
    if (active) stage_tile<T>(KVs, kv_stride, v_pages, table, p, kv_head, kt, k_lo, k_hi, lane, 64);
    __syncthreads();
    if (active) {
      for (int key = 0; key < KT; ++key) {
        const float pv = Ps[key];
        const float* vrow = KVs + key * kv_stride;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int d = lane + 64 * j;
          if (d < hd) o[j] += pv * vrow[d];
        }
      }
    }
    __syncthreads();
  }

  if (lane == 0) Ms[wave] = m, Ls[wave] = l;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int d = lane + 64 * j;
    if (d < hd) Os[wave * hd + d] = o[j];
  }
  __syncthreads();

  const float M = fmaxf(fmaxf(Ms[0], Ms[1]), fmaxf(Ms[2], Ms[3]));
  float w[4], L = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    w[i] = (Ms[i] == -INFINITY) ? 0.f : expf(Ms[i] - M);
    L += Ls[i] * w[i];
  }
  for (int d = tid; d < hd; d += 256) {
    float acc = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) acc += Os[i * hd + d] * w[i];
    if (p.n_splits == 1) {
      ((T*)p.out)[(size_t)row * p.ldo + h * hd + d] = from_f32<T>(acc / L);
    } else {
      const size_t base = ((size_t)item * p.n_heads + h) * p.n_splits + split;
      p.part_o[base * hd + d] = acc;
      if (d == 0) p.part_ml[base * 2] = M, p.part_ml[base * 2 + 1] = L;
    }
  }
}

// grid (n_rows, n_heads), 64 threads
template <typename T>
__global__ __launch_bounds__(64) void attn_merge_kernel(AttnArgs p) {
  const int item = blockIdx.x, h = blockIdx.y;
  const int row = p.items[item];
  const int hd = p.head_dim;
  const size_t base = ((size_t)item * p.n_heads + h) * p.n_splits;
  float M = -INFINITY;
  for (int s = 0; s < p.n_splits; ++s) M = fmaxf(M, p.part_ml[(base + s) * 2]);
  float L = 0.f;
  for (int s = 0; s < p.n_splits; ++s) {
    const float ms = p.part_ml[(base + s) * 2];
    if (ms != -INFINITY) L += p.part_ml[(base + s) * 2 + 1] * expf(ms - M);
  }
  for (int d = threadIdx.x; d < hd; d += 64) {
    float acc = 0.f;
    for (int s = 0; s < p.n_splits; ++s) {
      const float ms = p.part_ml[(base + s) * 2];
      if (ms != -INFINITY) acc += p.part_o[(base + s) * hd + d] * expf(ms - M);
    }
    ((T*)p.out)[(size_t)row * p.ldo + h * hd + d] = from_f32<T>(acc / L);
  }
}

// ---------------------------------------------------------------------------

DEFINE_LAST_ERROR(mlxlm_last_error)

static int check_geometry(const char* who, int n_heads, int n_kv_heads, int head_dim,
                          int page_size, int dtype) {
  if (dtype != DT_F32 && dtype != DT_BF16) FAIL("%s: unknown dtype code %d", who, dtype);
  if (n_heads <= 0 || n_kv_heads <= 0 || n_heads % n_kv_heads != 0)
    FAIL("%s: %d query heads cannot be grouped over %d key heads", who, n_heads, n_kv_heads);
  if (head_dim < 16 || head_dim > 256 || head_dim % 16 != 0)
    FAIL("%s: head_dim %d must be a multiple of 16 between 16 and 256", who, head_dim);
  if (page_size <= 0) FAIL("%s: page_size %d must be positive", who, page_size);
  return 0;
}

extern "C" int kv_write(const void* k_src, const void* v_src, int ld_src, void* k_pages,
                        void* v_pages, size_t page_stride, const int* block_table, int max_blocks,
                        const int* token_req, const int* positions, int n_tokens, int n_kv_heads,
                        int head_dim, int page_size, int dtype, hipStream_t stream) {
  if (n_tokens <= 0) return 0;
  if (check_geometry("kv_write", n_kv_heads, n_kv_heads, head_dim, page_size, dtype)) return 1;
  if (!k_src || !v_src || !k_pages || !v_pages || !block_table || !token_req || !positions)
    FAIL("kv_write: null pointer");
  if (page_stride < (size_t)n_kv_heads * page_size * head_dim)
    FAIL("kv_write: page stride smaller than a page");
  dim3 grid(n_tokens), block(256);
  const int vn = dtype == DT_F32 ? 4 : 8;
  const uintptr_t all = (uintptr_t)k_src | (uintptr_t)v_src | (uintptr_t)k_pages | (uintptr_t)v_pages;
  if (head_dim % vn == 0 && ld_src % vn == 0 && page_stride % vn == 0 && (all & 15) == 0) {
    if (dtype == DT_F32)
      hipLaunchKernelGGL(kv_write_vec_kernel<float>, grid, block, 0, stream, (const float*)k_src,
                         (const float*)v_src, ld_src, (float*)k_pages, (float*)v_pages, page_stride,
                         block_table, max_blocks, token_req, positions, n_kv_heads, head_dim,
                         page_size);
    else
      hipLaunchKernelGGL(kv_write_vec_kernel<bf16>, grid, block, 0, stream, (const bf16*)k_src,
                         (const bf16*)v_src, ld_src, (bf16*)k_pages, (bf16*)v_pages, page_stride,
                         block_table, max_blocks, token_req, positions, n_kv_heads, head_dim,
                         page_size);
    CHECK_LAUNCH("kv_write");
    return 0;
  }
  if (dtype == DT_F32)
    hipLaunchKernelGGL(kv_write_kernel<float>, grid, block, 0, stream, (const float*)k_src,
                       (const float*)v_src, ld_src, (float*)k_pages, (float*)v_pages, page_stride,
                       block_table, max_blocks, token_req, positions, n_kv_heads, head_dim,
                       page_size);
  else
    hipLaunchKernelGGL(kv_write_kernel<bf16>, grid, block, 0, stream, (const bf16*)k_src,
                       (const bf16*)v_src, ld_src, (bf16*)k_pages, (bf16*)v_pages, page_stride,
                       block_table, max_blocks, token_req, positions, n_kv_heads, head_dim,
                       page_size);
  CHECK_LAUNCH("kv_write");
  return 0;
}

static int fill_args(AttnArgs& p, const char* who, void* out, const void* q, int ldq, int ldo,
                     const void* k_pages, const void* v_pages, size_t page_stride,
                     const int* block_table, int max_blocks, const int* token_req,
                     const int* positions, const int* items, int n_heads, int n_kv_heads,
                     int head_dim, int page_size, int window, float scale, int dtype) {
  if (check_geometry(who, n_heads, n_kv_heads, head_dim, page_size, dtype)) return 1;
  if (!out || !q || !k_pages || !v_pages || !block_table || !token_req || !positions || !items)
    FAIL("%s: null pointer", who);
  const int vec = dtype == DT_F32 ? 4 : 8;
  if (page_stride % vec != 0) FAIL("%s: page stride %zu must be a multiple of %d", who, page_stride, vec);
  if (((uintptr_t)k_pages | (uintptr_t)v_pages) & 15) FAIL("%s: pages must be 16-byte aligned", who);
  if (window < 0) FAIL("%s: window %d must not be negative", who, window);
  p.out = out, p.q = q, p.k_pages = k_pages, p.v_pages = v_pages;
  p.block_table = block_table, p.token_req = token_req, p.positions = positions, p.items = items;
  p.part_o = nullptr, p.part_ml = nullptr;
  p.page_stride = page_stride, p.ldq = ldq, p.ldo = ldo, p.max_blocks = max_blocks;
  p.n_heads = n_heads, p.n_kv_heads = n_kv_heads, p.head_dim = head_dim, p.page_size = page_size;
  p.window = window, p.n_splits = 1, p.scale = scale;
  return 0;
}

// Kernels that want more than 64 KB of LDS have to be told so once per size.
static int allow_lds(const char* who, const void* kernel, size_t bytes) {
  static const void* seen[8];
  static size_t granted[8];
  static int n_seen = 0;
  if (bytes > 160 * 1024) FAIL("%s: needs %zu bytes of LDS, more than a CU has", who, bytes);
  if (bytes <= 64 * 1024) return 0;
  int i = 0;
  while (i < n_seen && seen[i] != kernel) ++i;
  if (i < n_seen && granted[i] >= bytes) return 0;
  hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
  if (e != hipSuccess) FAIL("%s: cannot get %zu bytes of LDS: %s", who, bytes, hipGetErrorString(e));
  if (i == n_seen && n_seen < 8) seen[n_seen++] = kernel;
  if (i < 8) granted[i] = bytes;
  return 0;
}

// items: n_tiles pairs (first flat row, number of rows 1..16); the rows of a
// tile are consecutive tokens of one request at consecutive positions.
extern "C" int attn_tile(void* out, const void* q, int ldq, int ldo, const void* k_pages,
                         const void* v_pages, size_t page_stride, const int* block_table,
                         int max_blocks, const int* token_req, const int* positions,
                         const int* tiles, int n_tiles, int n_heads, int n_kv_heads, int head_dim,
                         int page_size, int window, float scale, int dtype, hipStream_t stream) {
  if (n_tiles <= 0) return 0;
  AttnArgs p;
  if (fill_args(p, "attn_tile", out, q, ldq, ldo, k_pages, v_pages, page_stride, block_table,
                max_blocks, token_req, positions, tiles, n_heads, n_kv_heads, head_dim, page_size,
                window, scale, dtype))
    return 1;
  if (dtype == DT_F32 && (head_dim == 64 || head_dim == 128) && page_size % 16 == 0 && ldq % 4 == 0 &&
      ldo % 4 == 0 && (((uintptr_t)q | (uintptr_t)out) & 15) == 0) {
    dim3 grid((n_tiles + 3) / 4, n_heads), block(256);
    if (head_dim == 64)
      hipLaunchKernelGGL(attn_tile_mfma_kernel<1>, grid, block, 0, stream, p, n_tiles);
    else
      hipLaunchKernelGGL(attn_tile_mfma_kernel<2>, grid, block, 0, stream, p, n_tiles);
    CHECK_LAUNCH("attn_tile");
    return 0;
  }
  const size_t lds = sizeof(float) * ((size_t)QT * head_dim + (size_t)KT * (head_dim + 1) + QT * KT);
  dim3 grid(n_tiles, n_heads), block(256);
  if (dtype == DT_F32) {
    if (allow_lds("attn_tile", (const void*)attn_tile_kernel<float>, lds)) return 1;
    hipLaunchKernelGGL(attn_tile_kernel<float>, grid, block, lds, stream, p);
  } else {
    if (allow_lds("attn_tile", (const void*)attn_tile_kernel<bf16>, lds)) return 1;
    hipLaunchKernelGGL(attn_tile_kernel<bf16>, grid, block, lds, stream, p);
  }
  CHECK_LAUNCH("attn_tile");
  return 0;
}

// rows: n_rows flat row indices, each handled as a single query.  With
// n_splits > 1 the caller gives part_o [n_rows*n_heads*n_splits*head_dim] and
// part_ml [n_rows*n_heads*n_splits*2] floats.
extern "C" int attn_row(void* out, const void* q, int ldq, int ldo, const void* k_pages,
                        const void* v_pages, size_t page_stride, const int* block_table,
                        int max_blocks, const int* token_req, const int* positions,
                        const int* rows, int n_rows, int n_heads, int n_kv_heads, int head_dim,
                        int page_size, int window, float scale, int n_splits, float* part_o,
                        float* part_ml, int dtype, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  AttnArgs p;
  if (fill_args(p, "attn_row", out, q, ldq, ldo, k_pages, v_pages, page_stride, block_table,
                max_blocks, token_req, positions, rows, n_heads, n_kv_heads, head_dim, page_size,
                window, scale, dtype))
    return 1;
  if (n_splits < 1 || n_splits > 65535) FAIL("attn_row: n_splits %d out of range", n_splits);
  if (n_splits > 1 && (!part_o || !part_ml)) FAIL("attn_row: splits need the partial buffers");
  p.n_splits = n_splits, p.part_o = part_o, p.part_ml = part_ml;
  const size_t lds =
      sizeof(float) * ((size_t)head_dim + 4 * (size_t)KT * (head_dim + 1) + 4 * KT + 8 + 4 * (size_t)head_dim);
  dim3 grid(n_rows, n_heads, n_splits), block(256);
  if (dtype == DT_F32) {
    if (allow_lds("attn_row", (const void*)attn_row_kernel<float>, lds)) return 1;
    hipLaunchKernelGGL(attn_row_kernel<float>, grid, block, lds, stream, p);
    if (n_splits > 1)
      hipLaunchKernelGGL(attn_merge_kernel<float>, dim3(n_rows, n_heads), dim3(64), 0, stream, p);
  } else {
    if (allow_lds("attn_row", (const void*)attn_row_kernel<bf16>, lds)) return 1;
    hipLaunchKernelGGL(attn_row_kernel<bf16>, grid, block, lds, stream, p);
    if (n_splits > 1)
      hipLaunchKernelGGL(attn_merge_kernel<bf16>, dim3(n_rows, n_heads), dim3(64), 0, stream, p);
  }
  CHECK_LAUNCH("attn_row");
  return 0;
}
