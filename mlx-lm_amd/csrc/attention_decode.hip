// Decode attention: one query row per block, keys streamed from the pages
// straight into registers (no LDS staging).  bfloat16 caches with head sizes
// 32, 64 and 128, float caches with 16, 32 and 64 (a lane holds 16 bytes of a
// key, and 4 to 16 lanes a key).  Same contract as attn_row in attention.hip
// (same arguments, same partial buffers, same merge); this is the kernel that
// serving uses, attn_row stays as the general one (any head size).
//
// Replaces scaled_dot_product_attention with one query per sequence
// (mlx_lm/models/base.py:132-139 with mask=None, mlx_lm/generate.py:1414).
//
// Work split: grid (rows, heads, n_splits), 1 to 16 waves a block.  The row's
// keys [k_lo, k_hi) are cut into tiles of 32 or 64; the tiles are dealt to the splits
// in runs and, inside a block, to the waves in turn.  With few rows in a step
// it is the many waves of a block, joined through LDS, that give the GPU
// enough to do; the parts of splits are joined by the block of a (row, head) that
// finishes last, or by a second kernel.  A wave reads a tile as
// CPK-lane groups: lane l holds 16 bytes (EPL = 8 bfloat16 or 4 float columns)
// l % CPK of key l / CPK of each load, where CPK = head_dim / EPL lanes cover
// one key.  One load instruction therefore reads 64 / CPK whole keys that lie
// back to back in a page.  Scores: EPL products per lane, summed over the CPK
// lanes of the key by xor shuffles.  The weighted sum keeps, per lane, the EPL
// columns of *its* keys and is only joined over the lane groups (and then the
// waves) at the end.
#include "common.h"

struct DecodeArgs {
  void* out;  // out, q and the pages hold the kernel's element type
  const void* q;
  const void* k_pages;
  const void* v_pages;
  const int* block_table;
  const int* token_req;
  const int* positions;
  const int* rows;
  float* part_o;
  float* part_ml;
  size_t page_stride;
  int ldq, ldo, max_blocks;
  int n_heads, n_kv_heads, page_size, window, n_splits;
  float scale;
  // Blocks with blockIdx.y >= n_heads have no row: they read `ahead` (chunks of `ahead_pieces`
  // 16-byte pieces: the weights of a product that comes soon) and drop it, each the chunks that
  // a block on its own die will ask for.  Few rows leave most CUs idle, and the memory with them.
  const uint4* ahead;
  size_t ahead_pieces;
  int ahead_chunks;
  // rows_are_requests: item i of `rows` is row i and belongs to request i (a step in which every
  // request brings one token), so neither `rows` nor `token_req` has to be read.
  // table_in_lds: the request's page numbers are copied to LDS once (max_blocks of them fit).
  int rows_are_requests, table_in_lds;
  int out_head_dim;
  // 1 or 2: the blocks that share a row's keys join their sums themselves: the one that arrives
  // last at the (row, head)'s counter adds them in the order of the parts (no second kernel);
  // 2: n_splits is the most a row takes, and a row takes as many as its own length calls for
  int join_here;
};

#define MAX_WAVES 16

// ldo == 0: out is in the packed order, tiles of 16 rows x 64 columns
__device__ __forceinline__ size_t out_at(const DecodeArgs& p, int row, int col) {
  return p.ldo != 0 ? (size_t)row * p.ldo + col : packed_at(row, col, (p.n_heads * p.out_head_dim + 63) / 64);
}

// Keys a wave takes at a time: 32 or 64, the caller's choice.  With 64, a context of 530 gave nine
// of a block's waves a tile and the others none: 9.3 us for 8 rows of 25 heads against 7.3 with 32.
// Where rows x heads are several blocks a CU and the walk is long, the larger tile's sixteen
// loads a lane in flight are ahead (32 rows at contexts of 512 to 1,022: 2 % of the step).

// 16 bytes of a row as floats, and a float back as an element
__device__ __forceinline__ void unpack(const uint4& v, float (&f)[8], const uint16_t*) {
  f[0] = __uint_as_float(v.x << 16), f[1] = __uint_as_float(v.x & 0xffff0000u);
  f[2] = __uint_as_float(v.y << 16), f[3] = __uint_as_float(v.y & 0xffff0000u);
  f[4] = __uint_as_float(v.z << 16), f[5] = __uint_as_float(v.z & 0xffff0000u);
  f[6] = __uint_as_float(v.w << 16), f[7] = __uint_as_float(v.w & 0xffff0000u);
}
__device__ __forceinline__ void unpack(const uint4& v, float (&f)[4], const float*) {
  f[0] = __uint_as_float(v.x), f[1] = __uint_as_float(v.y);
  f[2] = __uint_as_float(v.z), f[3] = __uint_as_float(v.w);
}
__device__ __forceinline__ void put(uint16_t* at, float v) { *at = f32_to_bf16_bits(v); }
__device__ __forceinline__ void put(float* at, float v) { *at = v; }

// Joining a row's parts inside the kernel.  The parts' sums pass between blocks on different
// dies, whose L2s do not see each other's lines: they are written and read at agent scope (past
// the die's L2), and a counter a (row, head) says when all are there.  The counters are zero
// between launches (the block that arrives last puts its counter back); all launches on a GPU
// share them, so launches that overlap on one GPU race.
#define JOIN_MAX_ITEMS 65536
static __device__ unsigned join_counters[JOIN_MAX_ITEMS];
__device__ __forceinline__ void put_shared(float* at, float v) {
  __hip_atomic_store(at, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float get_shared(const float* at) {
  return __hip_atomic_load(at, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// Called by every thread of the block after its put_shared calls; true in all threads of the
// block that arrives last of `n_parts` at `counter`.  No block waits for another.
__device__ __forceinline__ bool last_to_arrive(unsigned* counter, unsigned n_parts, int* s_last) {
  __builtin_amdgcn_s_waitcnt(0);  // this thread's sums have been taken
  __syncthreads();
  if (threadIdx.x == 0) {
    const unsigned before = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    *s_last = before == n_parts - 1;
    if (*s_last) __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  __syncthreads();
  return *s_last != 0;
}

// T: uint16_t (bfloat16 bits) or float.  CPK lanes per key: head_dim = EPL * CPK.  TILE: keys a wave at a time.
template <typename T, int CPK, int TILE>
__global__ __launch_bounds__(64 * (CPK >= 16 ? MAX_WAVES / 2 : MAX_WAVES)) void attn_decode_kernel(DecodeArgs p) {
  constexpr int EPL = 16 / sizeof(T);  // elements a lane holds of a key
  constexpr int HD = EPL * CPK;
  constexpr int KPL = 64 / CPK;    // keys per load instruction
  constexpr int NL = TILE / KPL;   // loads per tile (= CPK)
  __shared__ float Ms[MAX_WAVES], Ls[MAX_WAVES];
  __shared__ float Os[MAX_WAVES][HD];
  __shared__ int s_last;
  extern __shared__ int page_of[];  // [max_blocks] with table_in_lds

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n_waves = blockDim.x >> 6;
  if (blockIdx.y >= p.n_heads) {  // a reading block (uniform)
    if (blockIdx.z != 0) return;
    // blocks go to the dies in turn, in the order x, y, z: this one is on die `lin % 8`, and
    // block j of the product to come, which reads chunk j, on die j % 8
    const int r = blockIdx.x + gridDim.x * (blockIdx.y - p.n_heads);
    const int readers = gridDim.x * (gridDim.y - p.n_heads);
    const int lin = gridDim.x * p.n_heads + r;
    const int die = lin & 7, rank = r >> 3, per_die = (readers + 7) >> 3;
    // the die's chunks (die, die + 8, ...) laid end to end and cut into equal shares, one a block
    const size_t mine = die < p.ahead_chunks ? (size_t)((p.ahead_chunks - die + 7) / 8) * p.ahead_pieces : 0;
    const size_t share = (mine + per_die - 1) / per_die;
    const size_t lo = (size_t)rank * share, hi = min(lo + share, mine);
    unsigned int seen = 0u;
    for (size_t i0 = lo + tid; i0 < hi; i0 += 8 * (size_t)blockDim.x) {
      uint4 v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const size_t t = min(i0 + u * (size_t)blockDim.x, hi - 1);
        const size_t c = t / p.ahead_pieces;
        v[u] = p.ahead[((size_t)die + 8 * c) * p.ahead_pieces + (t - c * p.ahead_pieces)];
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) seen |= v[u].x;
    }
    asm volatile("" ::"v"(seen));  // the loads stay although nobody wants the values
    return;
  }
  const int item = blockIdx.x, h = blockIdx.y, split = blockIdx.z;
  // Which row, whose pages, at which position: looked up one after the other these are three
  // trips to memory before the first key can be asked for, in a kernel that otherwise makes one
  // or two.  In a decode step item i is row i of request i, and the request's page numbers go to
  // LDS beside the position and the query: one trip, then the keys.
  const int row = p.rows_are_requests ? item : p.rows[item];
  const int req = p.rows_are_requests ? item : p.token_req[row];
  const int kv_head = h / (p.n_heads / p.n_kv_heads);
  const int* table = p.block_table + (size_t)req * p.max_blocks;
  if (p.table_in_lds) {
    for (int i = tid; i < p.max_blocks; i += blockDim.x) page_of[i] = table[i];
  }
  const int pos = p.positions[row];
  const int sub = lane % CPK;  // which EPL columns of the key
  const int kin = lane / CPK;  // which key of a load
  const T* k_pages = (const T*)p.k_pages;
  const T* v_pages = (const T*)p.v_pages;

  float qf[EPL];
  {
    const uint4 qv = *(const uint4*)((const T*)p.q + (size_t)row * p.ldq + h * HD + sub * EPL);
    unpack(qv, qf, (const T*)nullptr);
#pragma unroll
    for (int i = 0; i < EPL; ++i) qf[i] *= p.scale;
  }

  const int k_hi = pos + 1;
  const int k_lo = p.window > 0 ? max(0, pos - p.window + 1) : 0;
  const int kt0 = (k_lo / TILE) * TILE;
  const int n_tiles = (k_hi - kt0 + TILE - 1) / TILE;
  // Joined here, a row may take fewer splits than the launch has: as many as leave a wave a tile
  // of 32 keys, and one if a wave has fewer than 96 keys anyway (joining costs about a tile's
  // time).  Blocks of the splits it does not take have nothing to do.
  int n_splits = p.n_splits;
  if (p.join_here == 2) {
    const int keys_a_wave = (k_hi - kt0) / n_waves;
    n_splits = keys_a_wave >= 96 ? min(n_splits, keys_a_wave / 32) : 1;
    if (split >= n_splits) return;  // (the whole block)
  }
  const int per_split = (n_tiles + n_splits - 1) / n_splits;
  const int t_begin = split * per_split;
  const int t_end = min(n_tiles, t_begin + per_split);

  float m = -INFINITY, l = 0.f, o[EPL];
#pragma unroll
  for (int i = 0; i < EPL; ++i) o[i] = 0.f;

  const size_t head_off = (size_t)kv_head * p.page_size * HD;
  if (p.table_in_lds) __syncthreads();  // (uniform over the block)

  for (int t = t_begin + wave; t < t_end; t += n_waves) {
    const int kt = kt0 + t * TILE;
    uint4 kv[NL], vv[NL];
    // all loads of the tile first; addresses of keys outside [k_lo, k_hi) are
    // pulled inside (their scores are masked below)
#pragma unroll
    for (int j = 0; j < NL; ++j) {
      int key = kt + j * KPL + kin;
      key = min(max(key, k_lo), k_hi - 1);
      const int page = p.table_in_lds ? page_of[key / p.page_size] : table[key / p.page_size];
      const size_t off = (size_t)page * p.page_stride + head_off +
                         (size_t)(key % p.page_size) * HD + sub * EPL;
      kv[j] = *(const uint4*)(k_pages + off);
      vv[j] = *(const uint4*)(v_pages + off);
    }
    float s[NL];
    float tmax = -INFINITY;
#pragma unroll
    for (int j = 0; j < NL; ++j) {
      float kf[EPL];
      unpack(kv[j], kf, (const T*)nullptr);
      float d = 0.f;
#pragma unroll
      for (int i = 0; i < EPL; ++i) d += qf[i] * kf[i];
      d = group_sum<CPK>(d);  // over the key's lanes
      const int key = kt + j * KPL + kin;
      s[j] = (key >= k_lo && key < k_hi) ? d : -INFINITY;
      tmax = fmaxf(tmax, s[j]);
    }
    tmax = wave_max(tmax);
    const float m_new = fmaxf(m, tmax);  // finite: every tile holds at least one live key
    const float alpha = __expf(m - m_new);
    l *= alpha;
#pragma unroll
    for (int i = 0; i < EPL; ++i) o[i] *= alpha;
#pragma unroll
    for (int j = 0; j < NL; ++j) {
      const float pj = __expf(s[j] - m_new);  // exp(-inf) = 0 for masked keys
      float vf[EPL];
      unpack(vv[j], vf, (const T*)nullptr);
      if (sub == 0) l += pj;  // one lane of the key's group counts it
#pragma unroll
      for (int i = 0; i < EPL; ++i) o[i] += pj * vf[i];
    }
    m = m_new;
  }

  // join the lane groups: lanes with the same `sub` hold the same columns
  // (rotations of the row of 16 by 4 and by 8 through DPP moves; rows and halves of the wave
  // through shuffles)
  auto over_groups = [](float v) {
    if (CPK <= 4) v += dpp_move<0x124>(v);  // row_ror:4
    if (CPK <= 8) v += dpp_move<0x128>(v);  // row_ror:8
    v += __shfl_xor(v, 16, WAVE);
    return v + __shfl_xor(v, 32, WAVE);
  };
  l = over_groups(l);
#pragma unroll
  for (int i = 0; i < EPL; ++i) o[i] = over_groups(o[i]);
  l = group_sum<CPK>(l);

  if (lane == 0) Ms[wave] = m, Ls[wave] = l;
  if (lane < CPK) {
#pragma unroll
    for (int i = 0; i < EPL; ++i) Os[wave][lane * EPL + i] = o[i];
  }
  __syncthreads();

  // every thread joins the waves' results the same way, in the order of the waves
  float M = -INFINITY;
  for (int i = 0; i < n_waves; ++i) M = fmaxf(M, Ms[i]);
  float L = 0.f, acc = 0.f;
  for (int i = 0; i < n_waves; ++i) {
    const float w = (Ms[i] == -INFINITY) ? 0.f : __expf(Ms[i] - M);
    L += Ls[i] * w;
    if (tid < HD) acc += Os[i][tid] * w;
  }
  if (n_splits > 1 && p.join_here) {  // (uniform over the block)
    const size_t first = ((size_t)item * p.n_heads + h) * p.n_splits;
    if (tid < HD) put_shared(p.part_o + (first + split) * HD + tid, acc);
    if (tid == 0) put_shared(p.part_ml + (first + split) * 2, M), put_shared(p.part_ml + (first + split) * 2 + 1, L);
    if (!last_to_arrive(join_counters + (size_t)item * p.n_heads + h, (unsigned)n_splits, &s_last)) return;
    if (tid < HD) {  // the parts in their order, whoever arrived when
      float Mj = -INFINITY, Lj = 0.f, aj = 0.f;
      for (int s0 = 0; s0 < n_splits; s0 += 4) {
        float ms[4], ls[4], os[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {  // four parts' values on their way at a time
          const size_t at = first + min(s0 + j, n_splits - 1);
          ms[j] = get_shared(p.part_ml + at * 2), ls[j] = get_shared(p.part_ml + at * 2 + 1);
          os[j] = get_shared(p.part_o + at * HD + tid);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          if (s0 + j >= n_splits || ms[j] == -INFINITY) continue;  // (a part without a tile)
          const float M2 = fmaxf(Mj, ms[j]);
          const float wa = __expf(Mj - M2), wb = __expf(ms[j] - M2);
          Lj = Lj * wa + ls[j] * wb;
          aj = aj * wa + os[j] * wb;
          Mj = M2;
        }
      }
      put((T*)p.out + out_at(p, row, h * HD + tid), aj / Lj);
    }
    return;
  }
  if (tid < HD) {
    if (n_splits == 1) {
      put((T*)p.out + out_at(p, row, h * HD + tid), acc / L);
    } else {
      const size_t base = ((size_t)item * p.n_heads + h) * p.n_splits + split;
      p.part_o[base * HD + tid] = acc;
      if (tid == 0) p.part_ml[base * 2] = M, p.part_ml[base * 2 + 1] = L;
    }
  }
}

// grid (rows, heads), HD threads: join the splits
template <typename T, int CPK>
__global__ void attn_decode_merge_kernel(DecodeArgs p) {
  constexpr int HD = 16 / sizeof(T) * CPK;
  const int item = blockIdx.x, h = blockIdx.y, d = threadIdx.x;
  const int row = p.rows_are_requests ? item : p.rows[item];
  const size_t base = ((size_t)item * p.n_heads + h) * p.n_splits;
  float M = -INFINITY;
  for (int s = 0; s < p.n_splits; ++s) M = fmaxf(M, p.part_ml[(base + s) * 2]);
  float L = 0.f, acc = 0.f;
  for (int s = 0; s < p.n_splits; ++s) {
    const float ms = p.part_ml[(base + s) * 2];
    if (ms == -INFINITY) continue;
    const float w = __expf(ms - M);
    L += p.part_ml[(base + s) * 2 + 1] * w;
    acc += p.part_o[(base + s) * HD + d] * w;
  }
  put((T*)p.out + out_at(p, row, h * HD + d), acc / L);
}

DEFINE_LAST_ERROR(mlxlm_last_error)

template <typename T, int CPK>
static void launch(const DecodeArgs& p, int n_rows, int n_waves, int key_tile, hipStream_t stream) {
  // reading blocks for the CUs that the rows leave idle, if there are eight or more
  int extra_y = 0;
  if (p.ahead && p.ahead_chunks > 0) {
    extra_y = (n_compute_units() - n_rows * p.n_heads * p.n_splits) / n_rows;
    if (extra_y * n_rows < 8) extra_y = 0;
  }
  const size_t lds = p.table_in_lds ? (size_t)p.max_blocks * sizeof(int) : 0;
  const dim3 grid(n_rows, p.n_heads + extra_y, p.n_splits), block(64 * n_waves);
  if (key_tile == 64)
    hipLaunchKernelGGL((attn_decode_kernel<T, CPK, 64>), grid, block, lds, stream, p);
  else
    hipLaunchKernelGGL((attn_decode_kernel<T, CPK, 32>), grid, block, lds, stream, p);
  if (p.n_splits > 1 && !p.join_here)
    hipLaunchKernelGGL((attn_decode_merge_kernel<T, CPK>), dim3(n_rows, p.n_heads), dim3(16 / sizeof(T) * CPK), 0, stream, p);
}

// Same arguments as attn_row, with what is read ahead and rows_are_requests between: 1 says that
// item i of `rows` is row i and belongs to request i (every request of the step brings one token),
// which saves the kernel two trips to memory.  dtype DT_BF16 with head_dim 32, 64 or 128, DT_F32
// with 16, 32 or 64, and pages that hold whole loads (page_size a multiple of the keys in 1 KB).
// key_tile: 32 or 64 keys a wave at a time (0: 32).  join_in_kernel: 0, a second kernel joins the
// n_splits parts of a (row, head); 1, the block that finishes a (row, head) last does (up to
// 65,536 (row, head)s; part_o and part_ml are still where the parts pass through); 2, the same,
// and n_splits is only the most a row takes: a short row takes fewer, by its own length.
// Launches that join in the kernel and overlap on one GPU race (they share the counters).
extern "C" int attn_decode_rows(void* out, const void* q, int ldq, int ldo, const void* k_pages,
                                const void* v_pages, size_t page_stride, const int* block_table,
                                int max_blocks, const int* token_req, const int* positions,
                                const int* rows, int n_rows, int n_heads, int n_kv_heads, int head_dim,
                                int page_size, int window, float scale, int n_splits, float* part_o,
                                float* part_ml, int n_waves, const void* ahead, size_t ahead_chunk_bytes,
                                int ahead_chunks, int rows_are_requests, int dtype, int key_tile,
                                int join_in_kernel, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (key_tile == 0) key_tile = 32;
  if (key_tile != 32 && key_tile != 64) FAIL("attn_decode: a wave takes 32 or 64 keys at a time, not %d", key_tile);
  if (dtype != DT_F32 && dtype != DT_BF16) FAIL("attn_decode: unknown dtype code %d", dtype);
  const int epl = dtype == DT_F32 ? 4 : 8;  // elements in a lane's 16 bytes
  if (n_waves < 1 || n_waves > MAX_WAVES) FAIL("attn_decode: %d waves a block, must be 1 to %d", n_waves, MAX_WAVES);
  if (head_dim != 4 * epl && head_dim != 8 * epl && head_dim != 16 * epl)
    FAIL("attn_decode: head_dim %d is not %d, %d or %d (attn_row takes the others)", head_dim, 4 * epl, 8 * epl,
         16 * epl);
  const int cpk = head_dim / epl;
  if (head_dim > 64 * n_waves) FAIL("attn_decode: head_dim %d needs at least %d waves", head_dim, (head_dim + 63) / 64);
  if (cpk == 16 && n_waves > MAX_WAVES / 2) n_waves = MAX_WAVES / 2;  // (that kernel's registers allow eight)
  const int kpl = 64 / cpk;
  if (page_size <= 0 || page_size % kpl != 0)
    FAIL("attn_decode: page_size %d must be a multiple of %d for head_dim %d", page_size, kpl, head_dim);
  if (n_heads <= 0 || n_kv_heads <= 0 || n_heads % n_kv_heads != 0)
    FAIL("attn_decode: %d query heads cannot be grouped over %d key heads", n_heads, n_kv_heads);
  if (!out || !q || !k_pages || !v_pages || !block_table || !token_req || !positions || !rows)
    FAIL("attn_decode: null pointer");
  if (ldq % epl != 0 || ((uintptr_t)q & 15)) FAIL("attn_decode: queries must be 16-byte aligned rows");
  if (page_stride % epl != 0 || (((uintptr_t)k_pages | (uintptr_t)v_pages) & 15))
    FAIL("attn_decode: pages must be 16-byte aligned");
  if (window < 0) FAIL("attn_decode: window %d must not be negative", window);
  if (n_splits < 1 || n_splits > 65535) FAIL("attn_decode: n_splits %d out of range", n_splits);
  if (n_splits > 1 && (!part_o || !part_ml)) FAIL("attn_decode: splits need the partial buffers");
  DecodeArgs p;
  p.out = out, p.q = q, p.k_pages = k_pages, p.v_pages = v_pages;
  p.block_table = block_table, p.token_req = token_req, p.positions = positions, p.rows = rows;
  p.part_o = part_o, p.part_ml = part_ml, p.page_stride = page_stride;
  p.ldq = ldq, p.ldo = ldo, p.max_blocks = max_blocks;
  p.n_heads = n_heads, p.n_kv_heads = n_kv_heads, p.page_size = page_size;
  p.window = window, p.n_splits = n_splits, p.scale = scale;
  if (ahead && (((uintptr_t)ahead & 15) || ahead_chunk_bytes % 16 != 0 || ahead_chunks < 0))
    FAIL("attn_decode: what is read ahead must be chunks of 16-byte pieces");
  p.ahead = (const uint4*)ahead, p.ahead_pieces = ahead ? ahead_chunk_bytes / 16 : 0;
  p.ahead_chunks = ahead ? ahead_chunks : 0;
  p.out_head_dim = head_dim;
  if (ldo == 0 && dtype != DT_BF16) FAIL("attn_decode: the packed order (ldo == 0) is for a bfloat16 out");
  p.rows_are_requests = rows_are_requests ? 1 : 0;
  // (more (row, head)s than counters: the second kernel joins the parts)
  if (join_in_kernel < 0 || join_in_kernel > 2) FAIL("attn_decode: join_in_kernel %d is not 0, 1 or 2", join_in_kernel);
  p.join_here = n_splits > 1 && (long)n_rows * n_heads <= JOIN_MAX_ITEMS ? join_in_kernel : 0;
  p.table_in_lds = max_blocks > 0 && max_blocks <= 8192;  // (32 KB of LDS at most)
  if (dtype == DT_BF16) {
    if (cpk == 4)
      launch<uint16_t, 4>(p, n_rows, n_waves, key_tile, stream);
    else if (cpk == 8)
      launch<uint16_t, 8>(p, n_rows, n_waves, key_tile, stream);
    else
      launch<uint16_t, 16>(p, n_rows, n_waves, key_tile, stream);
  } else {
    if (cpk == 4)
      launch<float, 4>(p, n_rows, n_waves, key_tile, stream);
    else if (cpk == 8)
      launch<float, 8>(p, n_rows, n_waves, key_tile, stream);
    else
      launch<float, 16>(p, n_rows, n_waves, key_tile, stream);
  }
  CHECK_LAUNCH("attn_decode");
  return 0;
}
