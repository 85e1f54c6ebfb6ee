// Prefill attention for bfloat16 caches on the matrix cores: portions of
// prompts, 128 consecutive queries of one request per block, keys and values
// read from the pages in tiles of 64.  Same contract as attn_tile in
// attention.hip (same tile list, with up to 128 rows a tile); this is the
// kernel that serving uses for head sizes 32, 64 and 128, attn_tile stays as
// the general one (any head size, float caches).
//
// Replaces scaled_dot_product_attention with the "causal" mask and a cache
// offset (mlx_lm/models/base.py:24-35,132-139, mlx_lm/models/gpt2.py:60-65).
//
// Data flow, chosen so that a lane only ever deals with one query:
//  * Each of the four waves owns 32 queries.  Scores are computed transposed,
//    S^T = K Q^T, with v_mfma_f32_32x32x16_bf16: keys are the rows (A-operand,
//    from LDS), the wave's queries the columns (B-operand, kept in registers).
//    A lane then holds 16 scores of query (lane % 32) per 32-key subtile, so
//    the row maximum and sum need a single cross-lane step.
//  * The rows of a subtile are fed in a permuted key order such that the 8
//    scores a lane holds per 16-key chunk are 8 *consecutive* keys.  They are
//    exactly the B-operand fragment of O^T = V^T P^T; no shuffle, no LDS.
//  * V^T is needed with keys contiguous.  Values sit in the pages with head
//    columns contiguous, so the value tile is transposed on its way into LDS:
//    a thread reads the same 8 columns of two neighbouring keys and writes
//    eight 32-bit words (two keys each).
//  * Online softmax in 32-bit per lane; outputs leave as O^T accumulators.
#include "common.h"
#include "attention_tiles.h"
#include <type_traits>

struct PrefillArgs {
  uint16_t* out;
  const uint16_t* q;
  const uint16_t* k_pages;
  const uint16_t* v_pages;
  const int* block_table;
  const int* token_req;
  const int* positions;
  const int* tiles;  // (first row, n rows <= 128) pairs
  size_t page_stride;
  int ldq, ldo, max_blocks;
  int n_heads, n_kv_heads, page_size, window;
  int page_shift;  // log2(page_size), or -1 if that is no power of two
  float scale;
};

#define BQ ATTN_PREFILL_TILE_QUERIES  // queries per block
#define KT 64   // keys per tile
#define VT_STRIDE (KT + 8)  // 144 bytes a row: 16-byte reads of 32 rows fall on distinct banks

union Frag8 {
  uint4 u;
  bf16x8_t v;
};

// S^T row rho of a 32-key subtile holds this key of the subtile (see above)
__device__ __forceinline__ int key_of_row(int rho) {
  const int j = rho >> 3, g = (rho >> 2) & 1, i = rho & 3;
  return 16 * (j >> 1) + 8 * g + 4 * (j & 1) + i;
}

// POW2: the page size is a power of two (a key's page and row are a shift and a mask)
template <int HD, bool POW2>
__global__ __launch_bounds__(256, HD <= 64 ? 2 : 1) void attn_prefill_kernel(PrefillArgs p) {
  constexpr int KS_STRIDE = HD + 8;
  constexpr int DC = HD / 16;           // 16-column chunks of a head (QK contraction steps)
  constexpr int DT = HD / 32;           // 32-row tiles of O^T
  constexpr int K_CHUNKS = KT * HD / 8; // 16-byte pieces of a key tile
  constexpr int K_PER_T = (K_CHUNKS + 255) / 256;
  constexpr int V_ITEMS = (KT / 2) * (HD / 8);  // (key pair, 8-column chunk) items of a value tile
  constexpr int V_PER_T = (V_ITEMS + 255) / 256;
  __shared__ __attribute__((aligned(16))) uint16_t Ks[KT * KS_STRIDE];
  __shared__ __attribute__((aligned(16))) uint16_t Vt[HD * VT_STRIDE];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  // Which tile and head.  The tiles come with the most keys first, and a tile's heads are
  // neighbours in the launch, so the blocks with the longest walks start first and the short
  // ones fill in behind them (with the tiles as the fast index, a CU's two blocks were two
  // equally long ones, which took turns on its SIMDs to the end: 32 us a layer instead of 26
  // for 2 x 1,024 tokens of GPT-2 XL).
  const int h = blockIdx.x, tile = blockIdx.y;
  const int row0 = p.tiles[2 * tile];
  const int nq = p.tiles[2 * tile + 1];
  const int kv_head = h / (p.n_heads / p.n_kv_heads);
  const int pos0 = p.positions[row0];
  const int* table = p.block_table + (size_t)p.token_req[row0] * p.max_blocks;
  const uint32_t head_off = (uint32_t)(kv_head * p.page_size * HD);  // (within a page: below its stride)

  const int ql = lane & 31, g = lane >> 5;
  const int qi = wave * 32 + ql;         // this lane's query within the tile
  const bool q_live = qi < nq;
  const int qpos = pos0 + qi;
  const int q_lo = p.window > 0 ? max(0, qpos - p.window + 1) : 0;

  // the wave's queries as B-operand fragments: column = query, k = head columns
  Frag8 qf[DC];
  {
    const uint16_t* qrow = p.q + (size_t)(row0 + min(qi, nq - 1)) * p.ldq + h * HD + 8 * g;
#pragma unroll
    for (int dc = 0; dc < DC; ++dc) {
      const uint4 t = *(const uint4*)(qrow + dc * 16);
      qf[dc].u = q_live ? t : make_uint4(0u, 0u, 0u, 0u);
    }
  }

  const int k_hi = pos0 + nq;  // one past the last key any query of the tile sees
  const int k_lo = p.window > 0 ? max(0, pos0 - p.window + 1) : 0;
  const int kt0 = (k_lo / KT) * KT;
  // keys this wave's queries can see end here; later tiles it only helps to load
  const int wave_hi = min(k_hi, pos0 + wave * 32 + 32);
  const int wave_q0 = pos0 + wave * 32;            // position of the wave's first query
  const float c2 = p.scale * 1.4426950408889634f;  // scores to units of log 2

  float m = -INFINITY, l = 0.f;
  f32x16_t ot[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int r = 0; r < 16; ++r) ot[dt][r] = 0.f;

  // two tiles on their way (the keys' two sets as arrays of their own: as one array
  // indexed by the set they stayed in scratch memory)
  uint4 kreg0[K_PER_T], kreg1[K_PER_T], vreg[2][V_PER_T][2];

  // The request's page numbers go to LDS once: a load of keys or values then
  // depends on no other load from memory, and two tiles can be on their way
  // while one is multiplied.  (Looked up from memory per load, every load
  // waited for its page number first: eight trips to memory in a row per tile.)
  extern __shared__ int page_of[];  // [max_blocks]
  const int pg0 = k_lo / p.page_size;
  const int n_pg = (k_hi - 1) / p.page_size - pg0 + 1;
  for (int i = tid; i < n_pg; i += 256) page_of[i] = table[pg0 + i];
  __syncthreads();

  // Loads are never predicated and never zeroed: a key outside [k_lo, k_hi) is
  // read from the nearest key inside (a valid address with finite numbers);
  // its score is masked below, so its probability is zero.
  // An address is a dozen integer instructions, four times a thread and tile, in a kernel whose
  // time is its vector instructions: a division by a run-time page size alone costs thirty, and
  // choosing between it and a shift at run time put a branch around every address.  So the
  // choice is the kernel's template argument, and everything but the page's start is 32-bit.
  const uint32_t stride32 = (uint32_t)p.page_stride;
  const int shift = p.page_shift, row_mask = p.page_size - 1;
  auto address = [&](int key, int col) __attribute__((always_inline)) -> size_t {
    const int kk = min(max(key, k_lo), k_hi - 1);
    int idx, row;
    if constexpr (POW2) {
      idx = kk >> shift, row = kk & row_mask;
    } else {
      idx = kk / p.page_size, row = kk - idx * p.page_size;
    }
    const uint32_t within = head_off + (uint32_t)(row * HD + col);
    return (size_t)(uint32_t)page_of[idx - pg0] * stride32 + within;
  };
  auto fetch = [&](int kt, const int set) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < K_PER_T; ++i) {
      const int c = min(tid + 256 * i, K_CHUNKS - 1);  // surplus threads repeat the last piece
      const uint4 t = *(const uint4*)(p.k_pages + address(kt + c / (HD / 8), (c % (HD / 8)) * 8));
      if (set == 0) kreg0[i] = t; else kreg1[i] = t;
    }
#pragma unroll
    for (int i = 0; i < V_PER_T; ++i) {
      const int it = min(tid + 256 * i, V_ITEMS - 1);
      const int jp = it % (KT / 2), col = (it / (KT / 2)) * 8;
#pragma unroll
      for (int e = 0; e < 2; ++e) vreg[set][i][e] = *(const uint4*)(p.v_pages + address(kt + 2 * jp + e, col));
    }
  };
  auto stage = [&](const int set) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < K_PER_T; ++i) {
      const int c = tid + 256 * i;
      if (K_CHUNKS % 256 == 0 || c < K_CHUNKS)
        *(uint4*)(Ks + (c / (HD / 8)) * KS_STRIDE + (c % (HD / 8)) * 8) = set == 0 ? kreg0[i] : kreg1[i];
    }
#pragma unroll
    for (int i = 0; i < V_PER_T; ++i) {
      const int it = tid + 256 * i;
      if (V_ITEMS % 256 == 0 || it < V_ITEMS) {
        const int jp = it % (KT / 2), col = (it / (KT / 2)) * 8;
        const uint32_t a[4] = {vreg[set][i][0].x, vreg[set][i][0].y, vreg[set][i][0].z, vreg[set][i][0].w};
        const uint32_t b[4] = {vreg[set][i][1].x, vreg[set][i][1].y, vreg[set][i][1].z, vreg[set][i][1].w};
        uint32_t* dst = (uint32_t*)(Vt + col * VT_STRIDE + 2 * jp);
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          // columns col+2w and col+2w+1 of keys 2jp (low half) and 2jp+1 (high half)
          dst[(2 * w) * (VT_STRIDE / 2)] = (a[w] & 0xffffu) | (b[w] << 16);
          dst[(2 * w + 1) * (VT_STRIDE / 2)] = (a[w] >> 16) | (b[w] & 0xffff0000u);
        }
      }
    }
  };

  // One tile: its keys and values go from registers to LDS, the registers take
  // the tile after the next, then the arithmetic.
  // `steady` (a compile-time flag): the tile lies below every query of the block
  // and there is no window, so no wave is idle and nothing is masked; a loop of
  // such tiles has no branch inside, and the compiler lets the loads of the
  // other register set stay in flight while this one is staged.
  auto one_tile = [&](int kt, const int set, auto steady) __attribute__((always_inline)) {
    constexpr bool STEADY = decltype(steady)::value;
    __syncthreads();  // the previous tile is no longer read
    stage(set);
    __syncthreads();
    fetch(kt + 2 * KT, set);  // (beyond the last tile: harmless reads of the last key)
    if constexpr (!STEADY) {
      if (kt >= wave_hi || wave * 32 >= nq) return;  // nothing here for this wave (uniform)
    }

    // ---- S^T = K Q^T for the two 32-key subtiles --------------------------------
    f32x16_t st[2];
#pragma unroll
    for (int s = 0; s < 2; ++s) {
#pragma unroll
      for (int r = 0; r < 16; ++r) st[s][r] = 0.f;
      const uint16_t* krow = Ks + (32 * s + key_of_row(ql)) * KS_STRIDE + 8 * g;
#pragma unroll
      for (int dc = 0; dc < DC; ++dc) {
        Frag8 a;
        a.u = *(const uint4*)(krow + dc * 16);
        st[s] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.v, qf[dc].v, st[s], 0, 0, 0);
      }
    }
    // element r of subtile s: key kt + 32 s + 16 (r / 8) + 8 g + r % 8.
    // Scores are kept in units of log 2 (scale * log2(e) folded into one
    // factor), so that a probability is one fused multiply-add and one
    // v_exp_f32.  Tiles that every query of the wave sees whole (below the
    // diagonal, inside the window) skip the masks: this arithmetic, not the
    // MFMAs, is what the kernel's time goes to.
    const bool whole = STEADY || (kt + KT - 1 <= wave_q0 && (p.window <= 0 || kt >= wave_q0 + 31 - p.window + 1));
    float tmax = -INFINITY;
    if (whole) {
#pragma unroll
      for (int s = 0; s < 2; ++s)
#pragma unroll
        for (int r = 0; r < 16; ++r) tmax = fmaxf(tmax, st[s][r]);
      tmax *= c2;  // c2 > 0: the largest score stays the largest
    } else {
#pragma unroll
      for (int s = 0; s < 2; ++s)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int key = kt + 32 * s + 16 * (r >> 3) + 8 * g + (r & 7);
          const bool ok = q_live && key <= qpos && key >= q_lo;
          st[s][r] = ok ? st[s][r] : -INFINITY;
          tmax = fmaxf(tmax, st[s][r] * c2);
        }
    }
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, WAVE));
    const float m_new = fmaxf(m, tmax);
    const float m_use = (m_new == -INFINITY) ? 0.f : m_new;  // a row with no key yet
    const float alpha = exp2f(m - m_use);
    float lsum = 0.f;
    Frag8 pf[2][2];
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
      for (int c = 0; c < 2; ++c) {
        float e[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          e[i] = __builtin_amdgcn_exp2f(fmaf(st[s][8 * c + i], c2, -m_use));
          lsum += e[i];
        }
        pf[s][c].u.x = pack_bf16x2(e[0], e[1]);
        pf[s][c].u.y = pack_bf16x2(e[2], e[3]);
        pf[s][c].u.z = pack_bf16x2(e[4], e[5]);
        pf[s][c].u.w = pack_bf16x2(e[6], e[7]);
      }
    l = l * alpha + lsum;
    m = m_new;
    // ---- O^T = O^T * alpha + V^T P^T ---------------------------------------------
    const bool rescale = __any(alpha != 1.0f);  // no row's maximum moved: nothing to scale
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      if (rescale) {
#pragma unroll
        for (int r = 0; r < 16; ++r) ot[dt][r] *= alpha;
      }
      const uint16_t* vrow = Vt + (dt * 32 + ql) * VT_STRIDE + 8 * g;
#pragma unroll
      for (int s = 0; s < 2; ++s)
#pragma unroll
        for (int c = 0; c < 2; ++c) {
          Frag8 a;
          a.u = *(const uint4*)(vrow + 32 * s + 16 * c);
          ot[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.v, pf[s][c].v, ot[dt], 0, 0, 0);
        }
    }
  };

  fetch(kt0, 0);
  fetch(kt0 + KT, 1);
  int kt = kt0;
  if (p.window <= 0) {
    for (; kt + 2 * KT - 1 <= pos0; kt += 2 * KT) {
      one_tile(kt, 0, std::true_type{});
      one_tile(kt + KT, 1, std::true_type{});
    }
  }
  for (; kt < k_hi; kt += 2 * KT) {  // the tiles around the diagonal, or all of them under a window
    one_tile(kt, 0, std::false_type{});
    if (kt + KT >= k_hi) break;  // uniform
    one_tile(kt + KT, 1, std::false_type{});
  }

  // the two halves of the wave hold different keys of the same query
  l += __shfl_xor(l, 32, WAVE);
  if (q_live) {
    const float inv = 1.0f / l;
    uint16_t* orow = p.out + (size_t)(row0 + qi) * p.ldo + h * HD;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        // accumulators 4j .. 4j+3: head columns dt*32 + 8j + 4g + (0..3)
        uint2 o;
        o.x = pack_bf16x2(ot[dt][4 * j] * inv, ot[dt][4 * j + 1] * inv);
        o.y = pack_bf16x2(ot[dt][4 * j + 2] * inv, ot[dt][4 * j + 3] * inv);
        *(uint2*)(orow + dt * 32 + 8 * j + 4 * g) = o;
      }
  }
}

DEFINE_LAST_ERROR(mlxlm_last_error)

// tiles: n_tiles pairs (first flat row, number of rows 1..128); the rows of a
// tile are consecutive tokens of one request at consecutive positions.
// bfloat16 only, head_dim 32, 64 or 128.
extern "C" int attn_prefill(void* out, const void* q, int ldq, int ldo, const void* k_pages,
                            const void* v_pages, size_t page_stride, const int* block_table,
                            int max_blocks, const int* token_req, const int* positions,
                            const int* tiles, int n_tiles, int n_heads, int n_kv_heads,
                            int head_dim, int page_size, int window, float scale,
                            hipStream_t stream) {
  if (n_tiles <= 0) return 0;
  if (head_dim != 32 && head_dim != 64 && head_dim != 128)
    FAIL("attn_prefill: head_dim %d is not 32, 64 or 128 (attn_tile takes the others)", head_dim);
  if (n_heads <= 0 || n_kv_heads <= 0 || n_heads % n_kv_heads != 0)
    FAIL("attn_prefill: %d query heads cannot be grouped over %d key heads", n_heads, n_kv_heads);
  if (page_size <= 0) FAIL("attn_prefill: page_size %d must be positive", page_size);
  if (!out || !q || !k_pages || !v_pages || !block_table || !token_req || !positions || !tiles)
    FAIL("attn_prefill: null pointer");
  if (ldq % 8 != 0 || ((uintptr_t)q & 15)) FAIL("attn_prefill: query rows must be 16-byte aligned");
  if (ldo % 4 != 0 || ((uintptr_t)out & 7)) FAIL("attn_prefill: output rows must be 8-byte aligned");
  if (page_stride % 8 != 0 || (((uintptr_t)k_pages | (uintptr_t)v_pages) & 15))
    FAIL("attn_prefill: pages must be 16-byte aligned");
  if (window < 0) FAIL("attn_prefill: window %d must not be negative", window);
  if (page_stride >= ((size_t)1 << 32)) FAIL("attn_prefill: a page of %zu elements is too large", page_stride);
  PrefillArgs p;
  p.out = (uint16_t*)out, p.q = (const uint16_t*)q;
  p.k_pages = (const uint16_t*)k_pages, p.v_pages = (const uint16_t*)v_pages;
  p.block_table = block_table, p.token_req = token_req, p.positions = positions, p.tiles = tiles;
  p.page_stride = page_stride, p.ldq = ldq, p.ldo = ldo, p.max_blocks = max_blocks;
  p.page_shift = -1;
  for (int sh = 0; sh < 31; ++sh)
    if ((1 << sh) == page_size) p.page_shift = sh;
  p.n_heads = n_heads, p.n_kv_heads = n_kv_heads, p.page_size = page_size, p.window = window;
  p.scale = scale;
  if (n_tiles > 65535) FAIL("attn_prefill: %d tiles in a launch, at most 65535", n_tiles);
  dim3 grid(n_heads, n_tiles), block(256);
  // a request's page numbers lie in LDS beside the tiles
  if (max_blocks > 7168)
    FAIL("attn_prefill: block tables of %d pages a request do not fit beside the tiles (at most 7168)", max_blocks);
  const size_t lds = (size_t)max_blocks * sizeof(int);
  const bool pow2 = p.page_shift >= 0;
#define LAUNCH_PREFILL(HD)                                                                    \
  if (pow2) hipLaunchKernelGGL((attn_prefill_kernel<HD, true>), grid, block, lds, stream, p); \
  else hipLaunchKernelGGL((attn_prefill_kernel<HD, false>), grid, block, lds, stream, p)
  if (head_dim == 32) {
    LAUNCH_PREFILL(32);
  } else if (head_dim == 64) {
    LAUNCH_PREFILL(64);
  } else {
    LAUNCH_PREFILL(128);
  }
#undef LAUNCH_PREFILL
  CHECK_LAUNCH("attn_prefill");
  return 0;
}
