// The native host of a step.  A model is a tree of parts; eng_model_forward walks it and
// issues every launch of the step from this one call: which product kernel takes which
// rows, where K is split and who adds the partial sums, which norm is fused into which
// product, which attention kernel takes which rows of the batch.  The kernels themselves
// live in their own libraries (one per source file) and are looked up by name at first
// use through a resolver that the Python side sets, so a run compiles only what it calls.
//
// The order of a forward pass follows mlx_lm/models/gpt2.py:125-151,161-168 (embeddings,
// blocks, final norm, head) and :98-108 (a block), :44-68 (attention), :71-80 (the MLP);
// it has no counterpart there as code: the reference's array library schedules its own
// launches.
#include "common.h"
#include "engine.h"
#include "engine_parts.h"
#include "attention_tiles.h"

#include <stdarg.h>
#include <string.h>

#include <memory>
#include <vector>

DEFINE_LAST_ERROR(mlxlm_last_error)

#define GEMM_GELU 1
#define GEMM_ACCUMULATE 2
#define GEMM_OUT_F32 4
#define GEMM_KV 8
#define DECODE_MAX_ROWS 16
#define F32_FEW_ROWS 64  // rows that the 32-bit product's streaming kernel takes
#define GEMM_OUT_PACKED 16
#define ROWS_MAX_ROWS 64  // up to here the kernel for 17 to 64 rows
#define ATTN_ROW_MAX_HEAD_DIM 144
#define READ_AHEAD_BYTES_PER_CU (160 * 1024)  // what an idle CU reads while decode attention runs

// ---------------------------------------------------------------------------
// the kernels' entry points, looked up at first use

static eng_resolver_t g_resolver = nullptr;
static eng_callback_t g_callback = nullptr;

extern "C" void eng_set_hooks(eng_resolver_t resolver, eng_callback_t callback) {
  g_resolver = resolver;
  g_callback = callback;
}

extern "C" int eng_compute_units(void) { return n_compute_units(); }

// The decode kernel's waves a block where rows are few, and the keys a wave from which a row's keys
// are split over blocks (the kernel narrows a launch's splits row by row with the same number).
#define ROW_WAVES 8
#define ROW_SPLIT_KEYS_A_WAVE 96

// The context length from which a decode step may split a row's keys over blocks (what a recorded
// step's planning length is chosen by: below it no step launches splits).
extern "C" int eng_rows_split_from(void) { return ROW_WAVES * ROW_SPLIT_KEYS_A_WAVE; }

extern "C" void eng_attn_tile_sizes(int* tile, int* prefill_tile) {
  *tile = ATTN_TILE_QUERIES, *prefill_tile = ATTN_PREFILL_TILE_QUERIES;
}

template <typename F>
struct Entry {
  const char* lib;
  const char* name;
  F fn = nullptr;
  const char* (*err)() = nullptr;
  Entry(const char* l, const char* n) : lib(l), name(n) {}
  F get() {
    if (!fn && g_resolver) {
      fn = (F)g_resolver(lib, name);
      err = (const char* (*)())g_resolver(lib, "mlxlm_last_error");
    }
    return fn;
  }
};

typedef int (*fn_embed)(void*, const void*, const int*, const void*, const int*, int, int, int, hipStream_t);
typedef int (*fn_layernorm)(void*, const float*, const int*, const float*, const float*, float, int, int, int,
                            hipStream_t);
typedef int (*fn_gemm_f32)(void*, const void*, const void*, const float*, int, int, int, int, int, int, int,
                           int, int, float*, size_t, hipStream_t);
typedef int (*fn_gemm_bf16)(void*, const void*, const void*, const float*, int, int, int, int, int, int, int,
                            int, int, float*, size_t, void*, void*, size_t, const int*, int, const int*,
                            const int*, int, int, int, int, hipStream_t);
typedef int (*fn_int5)(int, int, int, int, int);
typedef int (*fn_int4)(int, int, int, int);
typedef int (*fn_int3)(int, int, int);
typedef int (*fn_int2)(int, int);
typedef int (*fn_gemm_decode)(void*, const void*, int, const float*, int, const float*, const float*, float,
                              const void*, const float*, int, int, int, int, int, int, void*, void*, size_t,
                              const int*, int, const int*, const int*, int, int, int, int, int, float*,
                              size_t, hipStream_t);
typedef int (*fn_gemm_rows)(void*, const void*, int, const void*, const float*, int, int, int, int, int, void*,
                            void*, size_t, const int*, int, const int*, const int*, int, int, int, int, int,
                            float*, size_t, hipStream_t);
typedef int (*fn_sum_partials)(void*, const float*, int, const float*, int, int, int, int, void*, void*,
                               size_t, const int*, int, const int*, const int*, int, int, int, int,
                               hipStream_t);
typedef int (*fn_sum_partials_norm)(float*, int, const float*, int, const float*, const float*, const float*,
                                    float, void*, int, int, int, int, const void*, size_t, int, hipStream_t);
typedef int (*fn_kv_write)(const void*, const void*, int, void*, void*, size_t, const int*, int, const int*,
                           const int*, int, int, int, int, int, hipStream_t);
typedef int (*fn_attn_tile)(void*, const void*, int, int, const void*, const void*, size_t, const int*, int,
                            const int*, const int*, const int*, int, int, int, int, int, int, float, int,
                            hipStream_t);
typedef int (*fn_attn_row)(void*, const void*, int, int, const void*, const void*, size_t, const int*, int,
                           const int*, const int*, const int*, int, int, int, int, int, int, float, int,
                           float*, float*, int, hipStream_t);
typedef int (*fn_attn_decode)(void*, const void*, int, int, const void*, const void*, size_t, const int*, int,
                              const int*, const int*, const int*, int, int, int, int, int, int, float, int,
                              float*, float*, int, const void*, size_t, int, int, int, int, int, hipStream_t);
typedef int (*fn_attn_prefill)(void*, const void*, int, int, const void*, const void*, size_t, const int*,
                               int, const int*, const int*, const int*, int, int, int, int, int, int, float,
                               hipStream_t);

static Entry<fn_embed> k_embed("embed", "embed_gather_add");
static Entry<fn_layernorm> k_layernorm("norm", "layernorm");
static Entry<fn_gemm_f32> k_gemm_f32("gemm_f32", "gemm_f32");
static Entry<fn_int4> k_gemm_f32_splits("gemm_f32", "gemm_f32_splits");
static Entry<fn_gemm_bf16> k_gemm_bf16("gemm_bf16", "gemm_bf16_scatter");
static Entry<fn_int5> k_gemm_bf16_splits("gemm_bf16", "gemm_bf16_splits");
static Entry<fn_gemm_decode> k_gemm_decode("gemm_bf16_decode", "gemm_bf16_decode");
static Entry<fn_int4> k_decode_takes("gemm_bf16_decode", "gemm_bf16_decode_takes");
static Entry<int (*)()> k_decode_few_blocks("gemm_bf16_decode", "gemm_bf16_decode_few_blocks");
static Entry<fn_int5> k_decode_splits("gemm_bf16_decode", "gemm_bf16_decode_splits");
static Entry<fn_gemm_rows> k_gemm_rows("gemm_bf16_decode", "gemm_bf16_rows");
static Entry<fn_int4> k_rows_splits("gemm_bf16_decode", "gemm_bf16_rows_splits");
static Entry<fn_int3> k_rows_takes("gemm_bf16_decode", "gemm_bf16_rows_takes");
static Entry<fn_sum_partials> k_sum_partials("gemm_bf16_decode", "sum_partials");
static Entry<fn_sum_partials_norm> k_sum_partials_norm("gemm_bf16_decode", "sum_partials_norm");
static Entry<fn_int2> k_sum_partials_norm_takes("gemm_bf16_decode", "sum_partials_norm_takes");
static Entry<fn_kv_write> k_kv_write("attention", "kv_write");
static Entry<fn_attn_tile> k_attn_tile("attention", "attn_tile");
static Entry<fn_attn_row> k_attn_row("attention", "attn_row");
static Entry<fn_attn_decode> k_attn_decode("attention_decode", "attn_decode_rows");
static Entry<fn_attn_prefill> k_attn_prefill("attention_prefill", "attn_prefill");

// Launch through an entry: a missing library or a refused call becomes this library's error.
#define KERNEL(entry, ctx, ...)                                                                  \
  do {                                                                                           \
    auto f_ = (entry).get();                                                                     \
    if (!f_) FAIL("the '%s' kernels are not loaded (%s)", (entry).lib, (entry).name);            \
    if (f_(__VA_ARGS__) != 0) FAIL("%s", (entry).err ? (entry).err() : (entry).name);            \
    if ((ctx)->stats) (ctx)->stats->launches++;                                                  \
  } while (0)

#define QUERY(entry, into, ...)                                                        \
  do {                                                                                 \
    auto f_ = (entry).get();                                                           \
    if (!f_) FAIL("the '%s' kernels are not loaded (%s)", (entry).lib, (entry).name);  \
    into = f_(__VA_ARGS__);                                                            \
  } while (0)

#define TRY(expr)            \
  do {                       \
    int rc_ = (expr);        \
    if (rc_ != 0) return rc_; \
  } while (0)

// ---------------------------------------------------------------------------
// scratch memory, matrices

static inline size_t elem_size(int dtype) { return dtype == DT_BF16 ? 2 : 4; }

static int take(EngCtx* ctx, int rows, int cols, int dtype, EngMat* out) {
  EngScratch* s = ctx->scratch;
  if (!s) FAIL("this call needs scratch memory, and its context has none");
  const size_t nbytes = (size_t)rows * cols * elem_size(dtype);
  const size_t start = (s->offset + 255) / 256 * 256, end = start + nbytes;
  if (end > s->size) {
    if (s->frozen) FAIL("scratch memory would have to grow while a step is being recorded");
    if (!g_callback) FAIL("scratch memory of %zu bytes is too small and nobody can grow it", s->size);
    EngCall call = {};
    call.nbytes = end;
    if (g_callback(0, ENG_CB_GROW, ctx, &call) != 0) return 2;
    if (end > s->size) FAIL("scratch memory did not grow to %zu bytes", end);
  }
  s->offset = end;
  if (end > s->peak) s->peak = end;
  out->p = s->base + start, out->rows = rows, out->cols = cols, out->ld = cols, out->dtype = dtype;
  return 0;
}

static inline EngMat columns(const EngMat& m, int from, int n) {
  EngMat v = m;
  v.p = (char*)m.p + (size_t)from * elem_size(m.dtype);
  v.cols = n;
  return v;
}

// ---------------------------------------------------------------------------
// pending sums

static inline bool waits_on(const EngPending& p, const EngMat& x) {
  return p.target != nullptr && (void*)p.target == x.p && p.rows == x.rows && p.cols == x.cols;
}

static int sum_partials(EngCtx* ctx, const EngMat& out, const float* ws, int n_splits, const float* bias,
                        bool gelu, bool accumulate, const EngScatter* sc, bool out_packed = false) {
  int flags = (gelu ? GEMM_GELU : 0) | (accumulate ? GEMM_ACCUMULATE : 0) | (out_packed ? GEMM_OUT_PACKED : 0);
  if (out.dtype == DT_F32) {
    if (!accumulate) flags |= GEMM_OUT_F32;
  } else if (accumulate) {
    FAIL("sum_partials: adding into the output needs a float32 output");
  }
  if (sc) flags |= GEMM_KV;
  KERNEL(k_sum_partials, ctx, out.p, ws, n_splits, bias, out.rows, out.cols, out.ld, flags, sc ? sc->k : nullptr,
         sc ? sc->v : nullptr, sc ? sc->page_stride : (size_t)0, sc ? sc->block_table : nullptr,
         sc ? sc->max_blocks : 0, sc ? sc->token_req : nullptr, sc ? sc->positions : nullptr,
         sc ? sc->q_width : 0, sc ? sc->kv_width : 0, sc ? sc->head_dim : 0, sc ? sc->page_size : 0, ctx->stream);
  return 0;
}

// Add what is pending (if anything) into its target.
static int settle(EngCtx* ctx, EngPending* p) {
  if (!p || !p->target) return 0;
  EngMat target = {p->target, p->rows, p->cols, p->ld, DT_F32};
  p->target = nullptr;
  if (ctx->stats) ctx->stats->settle_plain++;
  return sum_partials(ctx, target, p->ws, p->n_splits, p->bias, false, true, nullptr);
}

extern "C" int eng_settle(EngCtx* ctx) { return settle(ctx, &ctx->pending); }

static int can_norm(const EngPending& p, const EngMat& x, bool* yes) {
  *yes = false;
  if (!waits_on(p, x)) return 0;
  int takes = 0;
  QUERY(k_sum_partials_norm_takes, takes, x.cols, x.ld);
  *yes = takes != 0;
  return 0;
}

// Add what is pending into its target and write the LayerNorm of the new rows to `out`.
static int settle_normed(EngCtx* ctx, EngPending* p, const EngMat& out, const float* gamma, const float* beta,
                         float eps, const EngWeight* ahead, bool out_packed = false) {
  if (!p->target) FAIL("settle_normed: nothing is pending");
  float* h = p->target;
  p->target = nullptr;
  if (out.rows != p->rows || out.cols != p->cols || (!out_packed && out.ld != out.cols)) FAIL("settle_normed: out's shape");
  if (ctx->stats) ctx->stats->settle_normed++;
  KERNEL(k_sum_partials_norm, ctx, h, p->ld, p->ws, p->n_splits, p->bias, gamma, beta, eps, out.p, out.dtype,
         out_packed ? 1 : 0, p->rows, p->cols, ahead ? ahead->packed : nullptr,
         ahead ? ahead->chunk_bytes : (size_t)0, ahead ? ahead->n_chunks : 0, ctx->stream);
  return 0;
}

// Memory for `rows` x `cols` bfloat16 values in the packed order: whole tiles of 16 rows x 64 columns.
static int take_packed(EngCtx* ctx, int rows, int cols, EngMat* out) {
  TRY(take(ctx, (rows + 15) / 16 * 16, (cols + 63) / 64 * 64, DT_BF16, out));
  out->rows = rows, out->cols = cols, out->ld = 0;
  return 0;
}

// Whether the rows' next product should have `w` read ahead by the kernel before it: packed
// weights that the decode kernel takes whole, 16 features a block (then block j reads chunk j,
// on die j % 8), for few enough rows that most CUs have none.
static int read_ahead_pays(const EngCtx* ctx, const EngWeight* w, int n_rows, bool with_norm, bool* yes) {
  *yes = false;
  // (a matrix of few chunks is read by blocks of eight features, whose chunks are not the reading
  // blocks': the decode kernels' library says from how many on it is sixteen)
  int few = 0;
  QUERY(k_decode_few_blocks, few);
  if (!w || !w->packed || n_rows <= 0 || n_rows > DECODE_MAX_ROWS || w->n_chunks < few) return 0;
  int takes = 0, splits = 0;
  QUERY(k_decode_takes, takes, n_rows, w->K, with_norm ? 1 : 0, 1);
  if (!takes) return 0;
  QUERY(k_decode_splits, splits, n_rows, w->N, w->K, with_norm ? 1 : 0, ctx->force_splits);
  *yes = splits == 1;
  return 0;
}

// ---------------------------------------------------------------------------
// norms and products

static int layernorm(EngCtx* ctx, const EngMat& out, const float* x, const float* gamma, const float* beta,
                     float eps, const int* rows) {
  KERNEL(k_layernorm, ctx, out.p, x, rows, gamma, beta, eps, out.rows, out.cols, out.dtype, ctx->stream);
  return 0;
}

static int materialize(EngCtx* ctx, const EngValue& v, EngMat* out) {
  if (v.packed) FAIL("rows in the packed order were handed to a part that did not ask for them");
  if (!v.lazy) {
    *out = v.m;
    return 0;
  }
  if (v.ldx != v.m.cols) FAIL("a lazy norm's rows must be contiguous");
  TRY(take(ctx, v.m.rows, v.m.cols, v.m.dtype, out));
  return layernorm(ctx, *out, v.x, v.gamma, v.beta, v.eps, nullptr);
}

static int ceil_div(int a, int b) { return (a + b - 1) / b; }

static int split_count(int n_blocks, int want) {
  const int per = ceil_div(n_blocks, want < 1 ? 1 : (want > n_blocks ? n_blocks : want));
  return ceil_div(n_blocks, per);  // no empty part
}

static int kv_write(EngCtx* ctx, const EngMat& k, const EngMat& v, const EngScatter& sc) {
  if (k.ld != v.ld) FAIL("kv_write: k and v row strides differ");
  KERNEL(k_kv_write, ctx, k.p, v.p, k.ld, sc.k, sc.v, sc.page_stride, sc.block_table, sc.max_blocks,
         sc.token_req, sc.positions, k.rows, sc.n_kv_heads, sc.head_dim, sc.page_size, k.dtype, ctx->stream);
  return 0;
}

extern "C" int eng_linear_norms_itself(const EngCtx* ctx, int M, int N, int K, int dtype, int splits) {
  if (dtype != DT_BF16 || M <= 0 || M > DECODE_MAX_ROWS) return 0;
  auto takes = k_decode_takes.get();
  auto auto_splits = k_decode_splits.get();
  if (!takes || !auto_splits) return 0;
  const int n_splits = splits == 0 ? auto_splits(M, N, K, 1, ctx ? ctx->force_splits : 0)
                                   : split_count((K + 63) / 64, splits);
  return takes(M, K, 1, n_splits) != 0;
}

// What follows a product that left K in parts in the workspace: the sum stays pending where it
// goes into the residual stream and the caller allows that (the next norm adds it), otherwise
// the second kernel adds the parts and runs the epilogue.
static int finish_parts(EngCtx* ctx, const EngMat& out, float* ws, int n_splits, const float* bias, bool gelu,
                        bool accumulate, const EngScatter* sc, EngPending* pending, bool out_packed = false) {
  if (accumulate && pending && pending->allowed) {
    pending->target = (float*)out.p, pending->rows = out.rows, pending->cols = out.cols, pending->ld = out.ld;
    pending->ws = ws, pending->n_splits = n_splits, pending->bias = bias;
    return 0;
  }
  return sum_partials(ctx, out, ws, n_splits, bias, gelu, accumulate, sc, out_packed);
}

// Whether the kernel for 17 to 64 rows takes the product of M rows with w, and with K in how many
// parts (*n_splits; 0: it does not).
// (A matrix of more blocks than two a CU, the vocabulary's, would take that kernel several rounds,
// each with its own wait for memory: the tiles stream it 6 us faster.  Beyond 32 rows it wins
// only where K is long enough for the tiles to split it: at widths 768 and 1,024 a decode
// step of 48 rows is 4 to 5 % slower through it, at 1,280 the same, at 1,600 4 % faster.)
static int rows_parts(const EngCtx* ctx, int M, const EngWeight& w, int variant, int splits, int* n_splits) {
  *n_splits = 0;
  const int N = w.N, K = w.K;
  if (!(w.dtype == DT_BF16 && variant == 0 && M > DECODE_MAX_ROWS && M <= ROWS_MAX_ROWS && w.packed &&
        (M <= 32 || K >= 1536) && (N + 31) / 32 <= 2 * ctx->n_compute_units))
    return 0;
  int n = 0;
  if (splits == 0)
    QUERY(k_rows_splits, n, M, N, K, ctx->force_splits);
  else
    n = split_count((K + 63) / 64, splits);
  if (n > 1 && (!ctx->split_ws || (size_t)n > ctx->split_ws_floats / ((size_t)M * N))) n = 0;  // (the tiles then)
  if (n >= 1) {
    int takes = 0;
    QUERY(k_rows_takes, takes, M, K, n);
    if (!takes) n = 0;
  }
  *n_splits = n;
  return 0;
}

// That product reads its rows fastest in the packed order: who makes the rows may write them so.
static bool wants_packed(const EngCtx* ctx, int M, const EngWeight* w) {
  int n = 0;
  return w && rows_parts(ctx, M, *w, 0, 0, &n) == 0 && n >= 1;
}

extern "C" int eng_wants_packed_rows(const EngCtx* ctx, const EngWeight* w, int n_rows) {
  return wants_packed(ctx, n_rows, w) ? 1 : 0;
}

static int linear(EngCtx* ctx, const EngMat& out, const EngValue& a, const EngWeight& w, const float* bias,
                  bool gelu, bool accumulate, int variant, const EngScatter* sc, int splits,
                  EngPending* pending, bool out_packed = false) {
  const int M = a.m.rows, K = a.m.cols, N = w.N;
  if (a.packed && a.lazy) FAIL("linear: a norm not computed yet has no packed rows");
  if (out_packed && (accumulate || sc || out.dtype != DT_BF16)) FAIL("linear: only a plain bfloat16 out can be packed");
  if (w.K != K) FAIL("linear: a is [%d,%d] but w is [%d,%d]", M, K, w.N, w.K);
  if (out.rows != M || out.cols != N) FAIL("linear: out is [%d,%d], want [%d,%d]", out.rows, out.cols, M, N);
  if (a.m.dtype != w.dtype || (w.dtype != DT_F32 && w.dtype != DT_BF16))
    FAIL("linear: a and w must share float32 or bfloat16");
  if (!w.w && !(w.packed && w.dtype == DT_BF16)) FAIL("linear: the weights have no memory");
  if (M == 0) return 0;
  int flags = gelu ? GEMM_GELU : 0;
  if (accumulate) {
    if (out.dtype != DT_F32) FAIL("linear: accumulate needs a float32 out");
    flags |= GEMM_ACCUMULATE;
    if (pending && waits_on(*pending, out)) TRY(settle(ctx, pending));  // an earlier sum into the same rows goes first
  }
  if (sc) {
    if (accumulate || gelu || out.dtype != w.dtype) FAIL("linear: scatter goes with a plain epilogue");
    if (sc->q_width + 2 * sc->kv_width != N) FAIL("linear: scatter widths do not add up to N");
    if (sc->dtype != w.dtype) FAIL("linear: cache dtype differs from the projection's");
  }
  if (w.dtype == DT_F32) {
    if (out.dtype != DT_F32) FAIL("linear: float32 operands give a float32 out");
  } else if (out.dtype == DT_F32) {
    flags |= GEMM_OUT_F32;
  } else if (out.dtype != DT_BF16) {
    FAIL("linear: out must be float32 or bfloat16");
  }
  float* ws = ctx->split_ws;
  const size_t ws_floats = ctx->split_ws_floats;
  if (a.packed || out_packed) {
    int n = 0;
    if (M > 0) TRY(rows_parts(ctx, M, w, variant, splits, &n));
    if (n < 1) FAIL("linear: rows in the packed order are for the product of 17 to 64 rows only");
  }

  if (w.dtype == DT_BF16 && variant == 0 && M <= DECODE_MAX_ROWS) {
    const int with_norm = a.lazy ? 1 : 0;
    int n_splits = 1;
    if (splits == 0)
      QUERY(k_decode_splits, n_splits, M, N, K, with_norm, ctx->force_splits);
    else
      n_splits = split_count((K + 63) / 64, splits);
    if (n_splits > 1) {
      const size_t most = ws ? ws_floats / ((size_t)M * N) : 0;
      if ((size_t)n_splits > most) n_splits = (int)most;
      if (n_splits > 1) n_splits = split_count((K + 63) / 64, n_splits);  // (no part left empty by the cut)
      if (n_splits < 1) n_splits = 1;
    }
    int takes = 0;
    QUERY(k_decode_takes, takes, M, K, with_norm, n_splits);
    if (takes) {
      if (n_splits > 1 && pending) TRY(settle(ctx, pending));  // the workspace is about to be written again
      KERNEL(k_gemm_decode, ctx, out.p, a.lazy ? nullptr : a.m.p, a.lazy ? 0 : a.m.ld, a.lazy ? a.x : nullptr,
             a.lazy ? a.ldx : 0, a.lazy ? a.gamma : nullptr, a.lazy ? a.beta : nullptr, a.lazy ? a.eps : 0.f,
             w.packed ? w.packed : w.w, bias, M, N, K, w.packed ? 0 : w.ldw, out.ld, flags | (sc ? GEMM_KV : 0),
             sc ? sc->k : nullptr, sc ? sc->v : nullptr, sc ? sc->page_stride : (size_t)0,
             sc ? sc->block_table : nullptr, sc ? sc->max_blocks : 0, sc ? sc->token_req : nullptr,
             sc ? sc->positions : nullptr, sc ? sc->q_width : 0, sc ? sc->kv_width : 0, sc ? sc->head_dim : 0,
             sc ? sc->page_size : 0, n_splits, n_splits > 1 ? ws : nullptr, n_splits > 1 ? ws_floats : (size_t)0,
             ctx->stream);
      return n_splits > 1 ? finish_parts(ctx, out, ws, n_splits, bias, gelu, accumulate, sc, pending) : 0;
    }
  }

  EngMat A;
  if (a.packed)
    A = a.m;
  else
    TRY(materialize(ctx, a, &A));
  {
    // 17 to 64 rows: the kernel that holds a block's weights in registers, if the sizes fit it
    int n_splits = 0;
    TRY(rows_parts(ctx, M, w, variant, splits, &n_splits));
    if (n_splits >= 1) {
      if (n_splits > 1 && pending) TRY(settle(ctx, pending));  // the workspace is about to be written again
      KERNEL(k_gemm_rows, ctx, out.p, A.p, a.packed ? 0 : A.ld, w.packed, bias, M, N, K, out_packed ? 0 : out.ld,
             flags | (sc ? GEMM_KV : 0) | (out_packed ? GEMM_OUT_PACKED : 0),
             sc ? sc->k : nullptr, sc ? sc->v : nullptr, sc ? sc->page_stride : (size_t)0,
             sc ? sc->block_table : nullptr, sc ? sc->max_blocks : 0, sc ? sc->token_req : nullptr,
             sc ? sc->positions : nullptr, sc ? sc->q_width : 0, sc ? sc->kv_width : 0, sc ? sc->head_dim : 0,
             sc ? sc->page_size : 0, n_splits, n_splits > 1 ? ws : nullptr, n_splits > 1 ? ws_floats : (size_t)0,
             ctx->stream);
      return n_splits > 1 ? finish_parts(ctx, out, ws, n_splits, bias, gelu, accumulate, sc, pending, out_packed) : 0;
    }
  }
  if (w.dtype == DT_F32) {
    // Few rows of a narrow matrix give the kernel for them fewer blocks than there are compute
    // units: K goes in parts then, and the same second kernels add them up as for bfloat16.
    int n_splits = 1;
    if ((variant == 0 || variant == 3) && M <= F32_FEW_ROWS) {
      if (splits == 0)
        QUERY(k_gemm_f32_splits, n_splits, M, N, K, ctx->force_splits);
      else
        n_splits = split_count((K + 63) / 64, splits);
      if (n_splits > 1) {
        const size_t most = ws ? ws_floats / ((size_t)M * N) : 0;
        if ((size_t)n_splits > most) n_splits = (int)most;
        if (n_splits > 1) n_splits = split_count((K + 63) / 64, n_splits);
      }
      if (n_splits < 1) n_splits = 1;
      if (n_splits > 1 && pending) TRY(settle(ctx, pending));  // the workspace is about to be written again
    }
    KERNEL(k_gemm_f32, ctx, out.p, A.p, w.w, bias, M, N, K, A.ld, w.ldw, out.ld, flags, variant, n_splits,
           n_splits > 1 ? ws : nullptr, n_splits > 1 ? ws_floats : (size_t)0, ctx->stream);
    // (keys and values go to their pages from the finished rows, below)
    if (n_splits > 1) TRY(finish_parts(ctx, out, ws, n_splits, bias, gelu, accumulate, nullptr, pending));
  } else {
    // Few rows give the tile kernel few tiles: K is split then as for the decode kernels,
    // and the same second kernels add the parts and run the epilogue.
    int n_splits = 1;
    if ((variant == 0 || variant == 1 || variant == 5 || variant == 6) && M > DECODE_MAX_ROWS) {
      const int n_blocks = (K + 63) / 64;
      if (splits == 0) {
        // (the second kernel stands in for one that would run anyway: the next norm, or the cache write)
        const int fused = (accumulate && pending && pending->allowed) || sc != nullptr;
        QUERY(k_gemm_bf16_splits, n_splits, M, N, K, fused, ctx->force_splits);
      } else {
        n_splits = split_count(n_blocks, splits);
      }
      if (n_splits > 1) {
        const size_t most = ws ? ws_floats / ((size_t)M * N) : 0;
        if ((size_t)n_splits > most) n_splits = (int)most;
        if (n_splits > 1) n_splits = split_count(n_blocks, n_splits);
      }
      if (n_splits > 1 && pending) TRY(settle(ctx, pending));  // the workspace is about to be written again
    }
    if (n_splits < 1) n_splits = 1;
    // (weights kept only in the packed order are read in that order: row stride 0 says so; without a
    // split of K the product's own epilogue puts keys and values into their pages)
    const EngScatter* own = n_splits == 1 ? sc : nullptr;
    KERNEL(k_gemm_bf16, ctx, out.p, A.p, w.w ? w.w : w.packed, bias, M, N, K, A.ld, w.w ? w.ldw : 0, out.ld, flags,
           variant, n_splits, n_splits > 1 ? ws : nullptr, n_splits > 1 ? ws_floats : (size_t)0,
           own ? own->k : nullptr, own ? own->v : nullptr, own ? own->page_stride : (size_t)0,
           own ? own->block_table : nullptr, own ? own->max_blocks : 0, own ? own->token_req : nullptr,
           own ? own->positions : nullptr, own ? own->q_width : 0, own ? own->kv_width : 0,
           own ? own->head_dim : 0, own ? own->page_size : 0, ctx->stream);
    if (own) return 0;
    if (n_splits > 1) return finish_parts(ctx, out, ws, n_splits, bias, gelu, accumulate, sc, pending);
  }
  if (sc) {
    const EngMat k = columns(out, sc->q_width, sc->kv_width);
    const EngMat v = columns(out, sc->q_width + sc->kv_width, sc->kv_width);
    TRY(kv_write(ctx, k, v, *sc));
  }
  return 0;
}

extern "C" int eng_linear(EngCtx* ctx, const EngLinear* c, EngPending* pending) {
  return linear(ctx, c->out, c->a, c->w, c->bias, c->gelu != 0, c->accumulate != 0, c->variant, c->scatter,
                c->splits, pending, c->out_packed != 0);
}

// ---------------------------------------------------------------------------
// parts

static int call_python(int part_id, int method, EngCtx* ctx, EngCall* call) {
  if (!g_callback) FAIL("a part that lives in Python was called, and no callback is set");
  if (ctx->stats) ctx->stats->callbacks++;
  return g_callback(part_id, method, ctx, call) != 0 ? 2 : 0;
}

// -- parts that live in Python ------------------------------------------------

struct PyNorm : Norm {
  int id;
  PyNorm(int i, int flags) : id(i) {
    settles_pending = flags & ENG_SETTLES_PENDING, reads_ahead = false;
  }
  int forward(EngCtx* ctx, const EngMat& x, const int* rows, int n_rows, bool, const EngWeight*, bool,
              EngValue* out) override {
    EngCall c = {};
    c.x = x, c.rows = rows, c.n_rows = n_rows;
    TRY(call_python(id, ENG_CB_NORM, ctx, &c));
    if (!c.result.p) FAIL("a norm that lives in Python returned nothing");
    *out = EngValue{};
    out->m = c.result;
    return 0;
  }
};

struct PyPosition : Position {
  int id;
  bool has_rotate;
  PyPosition(int i, int flags) : id(i), has_rotate(true) { (void)flags; }
  int embedding_term(EngCtx* ctx, EngMat* table, const int** index) override {
    EngCall c = {};
    TRY(call_python(id, ENG_CB_EMBEDDING_TERM, ctx, &c));
    *table = c.result, *index = c.index;
    return 0;
  }
  int rotate(EngCtx* ctx, const EngMat& q, const EngMat& k) override {
    EngCall c = {};
    c.q = q, c.k = k;
    return call_python(id, ENG_CB_ROTATE, ctx, &c);
  }
  bool rotates() const override { return true; }
};

struct PyMixer : Mixer {
  int id;
  PyMixer(int i, int flags) : id(i) { accepts_lazy = false, (void)flags; }
  int forward(EngCtx* ctx, const EngValue& x, const EngMat& residual, int slot, bool writes) override {
    EngCall c = {};
    TRY(materialize(ctx, x, &c.x));
    c.residual = residual, c.cache_slot = slot, c.writes_cache = writes;
    return call_python(id, ENG_CB_MIXER, ctx, &c);
  }
};

struct PyFeedForward : FeedForward {
  int id;
  PyFeedForward(int i, int flags) : id(i) { accepts_lazy = false, (void)flags; }
  int forward(EngCtx* ctx, const EngValue& x, const EngMat& residual) override {
    EngCall c = {};
    TRY(materialize(ctx, x, &c.x));
    c.residual = residual;
    return call_python(id, ENG_CB_FFN, ctx, &c);
  }
};

struct PyBlock : Block {
  int id;
  PyBlock(int i, int flags) : id(i) { handles_pending = false, (void)flags; }
  int forward(EngCtx* ctx, const EngMat& h, int slot, bool writes) override {
    EngCall c = {};
    c.residual = h, c.cache_slot = slot, c.writes_cache = writes;
    return call_python(id, ENG_CB_BLOCK, ctx, &c);
  }
};

struct PyEmbedding : Embedding {
  int id;
  explicit PyEmbedding(int i) : id(i) {}
  int forward(EngCtx* ctx, const EngMat& out, const EngMat& add_table, const int* add_index) override {
    EngCall c = {};
    c.out = out, c.result = add_table, c.index = add_index;
    return call_python(id, ENG_CB_EMBEDDING, ctx, &c);
  }
};

struct PyHead : Head {
  int id;
  explicit PyHead(int i) : id(i) {}
  int forward(EngCtx* ctx, const EngValue& x, const EngMat& out) override {
    EngCall c = {};
    TRY(materialize(ctx, x, &c.x));
    c.out = out;
    return call_python(id, ENG_CB_HEAD, ctx, &c);
  }
};

// -- LayerNorm ------------------------------------------------------------------

struct LayerNorm : Norm {
  int width;
  float eps;
  const float* gamma;
  const float* beta;
  LayerNorm(int w, float e, const float* g, const float* b) : width(w), eps(e), gamma(g), beta(b) {
    settles_pending = true;  // adds a sum that is pending on x before (or while) it norms the rows
    reads_ahead = true;      // takes the weights that its result meets first
  }
  int forward(EngCtx* ctx, const EngMat& x, const int* rows, int n_rows, bool lazy, const EngWeight* ahead,
              bool may_pack, EngValue* out) override {
    if (x.cols != width || x.dtype != DT_F32) FAIL("layernorm: float32 rows of width %d", width);
    *out = EngValue{};
    EngPending* pending = &ctx->pending;
    if (waits_on(*pending, x)) {
      bool fused = false;
      if (!rows) TRY(can_norm(*pending, x, &fused));
      if (fused) {
        // the last projection split its sum: add the parts and norm the new rows in one kernel
        // (in the packed order, where the product that takes them reads that faster)
        const bool pack = may_pack && ctx->dtype == DT_BF16 && wants_packed(ctx, x.rows, ahead);
        if (pack)
          TRY(take_packed(ctx, x.rows, width, &out->m));
        else
          TRY(take(ctx, x.rows, width, ctx->dtype, &out->m));
        out->packed = pack ? 1 : 0;
        bool pays = false;
        if (ahead) TRY(read_ahead_pays(ctx, ahead, x.rows, false, &pays));
        return settle_normed(ctx, pending, out->m, gamma, beta, eps, pays ? ahead : nullptr, pack);
      }
      TRY(settle(ctx, pending));
    }
    if (lazy && !rows) {
      // the consumer's first matrix product may norm the rows itself
      out->lazy = 1, out->x = (const float*)x.p, out->ldx = x.ld, out->gamma = gamma, out->beta = beta;
      out->eps = eps;
      out->m = EngMat{nullptr, x.rows, width, width, ctx->dtype};
      return 0;
    }
    if (!rows && x.ld != width) FAIL("layernorm: the stream's rows must be contiguous");
    TRY(take(ctx, rows ? n_rows : x.rows, width, ctx->dtype, &out->m));
    return layernorm(ctx, out->m, (const float*)x.p, gamma, beta, eps, rows);
  }
};

// -- attention ------------------------------------------------------------------

// ids of the arrays that the attention part asks the packer for, from `array_base` on
enum { ARR_TILES = 0, ARR_ROWS, ARR_ALL_TILES, ARR_BIG_TILES, ARR_MAX_ROW_CONTEXT, ARR_ROWS_ARE_REQUESTS };

struct Attention : Mixer {
  int width, n_heads, n_kv_heads, head_dim, window, q_width, kv_width, array_base;
  float scale;
  EngWeight qkv_w, out_w;
  const float* qkv_b;
  const float* out_b;
  Position* position;

  Attention() { accepts_lazy = true, accepts_packed = true; }

  int scatter_for(EngCtx* ctx, int slot, EngScatter* sc) const;

  // (n_splits, n_waves, keys a wave at a time) for the decode kernel.  Eight waves a block (four
  // where the rows' blocks alone are more than the CUs, or the keys no more than four waves'
  // tiles): measured at 1 to 64 rows and contexts of 100 to 7,000, eight were level with or ahead
  // of sixteen everywhere.  Tiles of 32 keys, so that every wave has some at a context of a few
  // hundred; of 64 where the blocks are more than three a CU and the context is 640 or more (the
  // larger tile keeps more loads in flight; a recorded step plans for the model's positions: at
  // 1,024 of them, 12 to 30 rows were 1 to 3 % faster with 32 over contexts of 512 to 1,022, 32
  // rows 2 % faster with 64).  The block that finishes a (row, head) last joins its splits, which
  // costs about as much as a tile of keys: splits only where a wave would walk 96 keys or more, as
  // many as leave it a tile, and no more than give every block a compute unit at once (one row at
  // 1,000 keys: 9.4 us unsplit, 7.3 in four; at 7,000: 44 unsplit, 13.6 in eight, 15.9 in twelve).
  // This is the most a row takes; the kernel gives a shorter row fewer by the same rule, so a
  // recorded step, planned for the model's positions, splits only the rows that are long.
  void row_work(const EngCtx* ctx, int n_rows, long max_row_context, int* n_splits, int* n_waves,
                int* key_tile) const {
    const long c = window <= 0 ? max_row_context : (max_row_context < window + 31 ? max_row_context : window + 31);
    const long tiles = c + 31 < 32 ? 1 : (c + 31) / 32;
    const long blocks = n_rows * n_heads < 1 ? 1 : (long)n_rows * n_heads;
    int nw = blocks > ctx->n_compute_units ? 4 : ROW_WAVES;
    const int fewest = head_dim > 128 ? 4 : 2;  // (the block's threads write a column of the head each)
    while (nw > fewest && nw / 2 >= tiles) nw /= 2;
    const long keys_a_wave = c / nw;
    long ns = 1;
    if (keys_a_wave >= ROW_SPLIT_KEYS_A_WAVE) {
      ns = keys_a_wave / 32;
      if (ctx->n_compute_units / blocks < ns) ns = ctx->n_compute_units / blocks;
      if (ns > 64) ns = 64;
      if (ns < 1) ns = 1;
    }
    *n_splits = (int)ns, *n_waves = nw, *key_tile = 32;
    if (blocks > 3 * ctx->n_compute_units && c >= 640) {
      // many rows and a long walk: tiles of 64 keys, and as many waves a block as make eight a CU
      // (32 rows: four; 64 rows: two.  With four at 64 rows the step took 5.92 ms instead of 5.76.)
      const long want = (8L * ctx->n_compute_units + blocks - 1) / blocks;
      nw = fewest;
      while (nw < 8 && nw < want) nw *= 2;
      *n_waves = nw, *key_tile = 64;
    }
  }

  // How many ways to split a row's keys so that the general row kernel's launch fills the GPU.
  int row_splits(const EngCtx* ctx, int n_rows, long max_row_context) const {
    const long c = window <= 0 ? max_row_context : (max_row_context < window + 63 ? max_row_context : window + 63);
    long most = (c + 255) / 256;
    if (most < 1) most = 1;
    const long blocks = n_rows * n_heads < 1 ? 1 : (long)n_rows * n_heads;
    long want = (2L * ctx->n_compute_units + blocks - 1) / blocks;
    if (want > most) want = most;
    if (want > 64) want = 64;
    return want < 1 ? 1 : (int)want;
  }

  // Whether the step's rows all go to the decode kernel, which can write its output in the
  // packed order (the output projection of 17 to 64 rows reads that faster).
  bool rows_only_fast(const EngCtx* ctx, const EngMat& q, const EngScatter& kv) const {
    const int n_tiles = (int)ctx->counts[array_base + ARR_TILES] / 2;
    const int n_rows = (int)ctx->counts[array_base + ARR_ROWS];
    const int key_bytes = head_dim * (q.dtype == DT_BF16 ? 2 : 4);
    return n_tiles == 0 && n_rows == q.rows && head_dim <= ATTN_ROW_MAX_HEAD_DIM &&
           (key_bytes == 64 || key_bytes == 128 || key_bytes == 256) && kv.page_size % (1024 / key_bytes) == 0;
  }

  int attend(EngCtx* ctx, const EngMat& out, const EngMat& q, const EngScatter& kv, bool out_packed) const {
    const int* tiles = ctx->arrays[array_base + ARR_TILES];
    const int* rows = ctx->arrays[array_base + ARR_ROWS];
    const int* all_tiles = ctx->arrays[array_base + ARR_ALL_TILES];
    const int* big_tiles = ctx->arrays[array_base + ARR_BIG_TILES];
    const int n_tiles = (int)ctx->counts[array_base + ARR_TILES] / 2;
    const int n_rows = (int)ctx->counts[array_base + ARR_ROWS];
    const int n_all_tiles = (int)ctx->counts[array_base + ARR_ALL_TILES] / 2;
    const int n_big_tiles = (int)ctx->counts[array_base + ARR_BIG_TILES] / 2;
    const long max_row_context = ctx->counts[array_base + ARR_MAX_ROW_CONTEXT];
    const int rows_are_requests = ctx->counts[array_base + ARR_ROWS_ARE_REQUESTS] != 0;
    if (n_tiles == 0 && n_rows == 0 && q.rows > 0)
      FAIL("attention: the step carries no work lists for its %d rows", q.rows);
    const bool bf16 = q.dtype == DT_BF16;
    if (head_dim > ATTN_ROW_MAX_HEAD_DIM) {
      KERNEL(k_attn_tile, ctx, out.p, q.p, q.ld, out.ld, kv.k, kv.v, kv.page_stride, kv.block_table, kv.max_blocks,
             kv.token_req, kv.positions, all_tiles, n_all_tiles, n_heads, n_kv_heads, head_dim, kv.page_size,
             window, scale, q.dtype, ctx->stream);
      return 0;
    }
    const bool mfma_sizes = bf16 && (head_dim == 32 || head_dim == 64 || head_dim == 128);
    if (n_tiles) {
      if (mfma_sizes)
        KERNEL(k_attn_prefill, ctx, out.p, q.p, q.ld, out.ld, kv.k, kv.v, kv.page_stride, kv.block_table,
               kv.max_blocks, kv.token_req, kv.positions, big_tiles, n_big_tiles, n_heads, n_kv_heads, head_dim,
               kv.page_size, window, scale, ctx->stream);
      else
        KERNEL(k_attn_tile, ctx, out.p, q.p, q.ld, out.ld, kv.k, kv.v, kv.page_stride, kv.block_table,
               kv.max_blocks, kv.token_req, kv.positions, tiles, n_tiles, n_heads, n_kv_heads, head_dim,
               kv.page_size, window, scale, q.dtype, ctx->stream);
    }
    if (n_rows) {
      // the kernel that streams keys into registers: a key in 4, 8 or 16 lanes of 16 bytes
      const int key_bytes = head_dim * (bf16 ? 2 : 4);
      const bool fast = (key_bytes == 64 || key_bytes == 128 || key_bytes == 256) &&
                        kv.page_size % (1024 / key_bytes) == 0;
      int n_splits = 1, n_waves = 4, key_tile = 32;
      if (fast)
        row_work(ctx, n_rows, max_row_context, &n_splits, &n_waves, &key_tile);
      else
        n_splits = row_splits(ctx, n_rows, max_row_context);
      if (ctx->stats && n_splits > ctx->stats->key_splits_most) ctx->stats->key_splits_most = n_splits;
      EngMat part_o = {}, part_ml = {};
      if (n_splits > 1) {
        const long n = (long)n_rows * n_heads * n_splits;
        TRY(take(ctx, 1, (int)(n * head_dim), DT_F32, &part_o));
        TRY(take(ctx, 1, (int)(n * 2), DT_F32, &part_ml));
      }
      if (fast) {
        // CUs without a row read the weights that come after this mixer's own (the block says
        // which), as many chunks as they manage while the rows' blocks run; where fewer than half
        // the CUs are idle the reading slows the rows' blocks by more than it gains
        const EngWeight* ahead = ctx->read_ahead;
        int chunks = 0;
        const long idle = ctx->n_compute_units - (long)n_rows * n_heads * n_splits;
        bool pays = false;
        if (ahead && idle >= ctx->n_compute_units / 2 && n_tiles == 0 && n_rows == q.rows)
          TRY(read_ahead_pays(ctx, ahead, n_rows, true, &pays));
        if (pays) {
          chunks = (int)(idle * READ_AHEAD_BYTES_PER_CU / (long)ahead->chunk_bytes);
          if (chunks > ahead->n_chunks) chunks = ahead->n_chunks;
        } else {
          ahead = nullptr;
        }
        KERNEL(k_attn_decode, ctx, out.p, q.p, q.ld, out_packed ? 0 : out.ld, kv.k, kv.v, kv.page_stride, kv.block_table,
               kv.max_blocks, kv.token_req, kv.positions, rows, n_rows, n_heads, n_kv_heads, head_dim,
               kv.page_size, window, scale, n_splits, (float*)part_o.p, (float*)part_ml.p, n_waves,
               ahead ? ahead->packed : nullptr, ahead ? ahead->chunk_bytes : (size_t)0, chunks, rows_are_requests,
               q.dtype, key_tile, 2, ctx->stream);
      } else {
        KERNEL(k_attn_row, ctx, out.p, q.p, q.ld, out.ld, kv.k, kv.v, kv.page_stride, kv.block_table,
               kv.max_blocks, kv.token_req, kv.positions, rows, n_rows, n_heads, n_kv_heads, head_dim,
               kv.page_size, window, scale, n_splits, (float*)part_o.p, (float*)part_ml.p, q.dtype, ctx->stream);
      }
    }
    return 0;
  }

  int forward(EngCtx* ctx, const EngValue& x, const EngMat& residual, int slot, bool writes) override {
    const int T = x.m.rows;
    EngScatter kv;
    TRY(scatter_for(ctx, slot, &kv));
    EngMat qkv;
    TRY(take(ctx, T, q_width + 2 * kv_width, ctx->dtype, &qkv));
    const EngMat q = columns(qkv, 0, q_width);
    if (!position || !position->rotates()) {
      // keys and values go to their pages from the projection's epilogue
      TRY(linear(ctx, qkv, x, qkv_w, qkv_b, false, false, 0, writes ? &kv : nullptr, 0, &ctx->pending));
    } else {
      TRY(linear(ctx, qkv, x, qkv_w, qkv_b, false, false, 0, nullptr, 0, &ctx->pending));
      const EngMat k = columns(qkv, q_width, kv_width), v = columns(qkv, q_width + kv_width, kv_width);
      TRY(position->rotate(ctx, q, k));
      if (writes) TRY(kv_write(ctx, k, v, kv));
    }
    EngMat out;
    const bool pack = ctx->dtype == DT_BF16 && wants_packed(ctx, T, &out_w) && rows_only_fast(ctx, q, kv);
    if (pack)
      TRY(take_packed(ctx, T, q_width, &out));
    else
      TRY(take(ctx, T, q_width, ctx->dtype, &out));
    TRY(attend(ctx, out, q, kv, pack));
    EngValue o = {};
    o.m = out, o.packed = pack ? 1 : 0;
    return linear(ctx, residual, o, out_w, out_b, false, true, 0, nullptr, 0, &ctx->pending);
  }
};

static int host_slot_pages(EngCtx* ctx, int slot, int q_width, int kv_width, EngScatter* sc);

int Attention::scatter_for(EngCtx* ctx, int slot, EngScatter* sc) const {
  TRY(host_slot_pages(ctx, slot, q_width, kv_width, sc));
  if (sc->n_kv_heads != n_kv_heads || sc->head_dim != head_dim)
    FAIL("attention: cache slot %d holds %d heads of %d, the mixer has %d of %d", slot, sc->n_kv_heads,
         sc->head_dim, n_kv_heads, head_dim);
  return 0;
}

// -- feed-forward ---------------------------------------------------------------

struct GeluMlp : FeedForward {
  int width, inner;
  EngWeight fc_w, proj_w;
  const float* fc_b;
  const float* proj_b;
  GeluMlp() { accepts_lazy = true, accepts_packed = true; }
  int forward(EngCtx* ctx, const EngValue& x, const EngMat& residual) override {
    EngMat act;
    // (both products through the kernel for 17 to 64 rows: the first writes what the second reads
    // in the packed order)
    const int M = x.m.rows;
    const bool pack = ctx->dtype == DT_BF16 && wants_packed(ctx, M, &fc_w) && wants_packed(ctx, M, &proj_w);
    if (pack)
      TRY(take_packed(ctx, M, inner, &act));
    else
      TRY(take(ctx, M, inner, ctx->dtype, &act));
    TRY(linear(ctx, act, x, fc_w, fc_b, true, false, 0, nullptr, 0, &ctx->pending, pack));
    EngValue a = {};
    a.m = act, a.packed = pack ? 1 : 0;
    return linear(ctx, residual, a, proj_w, proj_b, false, true, 0, nullptr, 0, &ctx->pending);
  }
};

// -- block ----------------------------------------------------------------------

// h += mixer(norm1(h)); h += ffn(norm2(h)).  The two sums happen inside the mixer's and the
// feed-forward's last product; such a product may leave its sum pending, and the norm that
// reads h next adds it.
struct PreNormBlock : Block {
  Norm* mixer_norm;
  Mixer* mixer;
  Norm* ffn_norm;
  FeedForward* ffn;
  PreNormBlock() { handles_pending = true; }

  static int normed(EngCtx* ctx, Norm* norm, const EngMat& h, bool lazy, bool may_pack, const EngWeight* first,
                    EngValue* x) {
    if (!norm->settles_pending) TRY(settle(ctx, &ctx->pending));
    return norm->forward(ctx, h, nullptr, 0, lazy, norm->reads_ahead ? first : nullptr, may_pack, x);
  }

  int forward(EngCtx* ctx, const EngMat& h, int slot, bool writes) override {
    const size_t mark = ctx->scratch->offset;
    EngValue x;
    TRY(normed(ctx, mixer_norm, h, mixer->accepts_lazy, mixer->accepts_packed, mixer->first_weight, &x));
    // (a mixer whose kernels leave CUs idle may have them read the weights that come after its own)
    ctx->read_ahead = ffn->first_weight;
    int rc = mixer->forward(ctx, x, h, slot, writes);
    ctx->read_ahead = nullptr;
    if (rc) return rc;
    TRY(normed(ctx, ffn_norm, h, ffn->accepts_lazy, ffn->accepts_packed, ffn->first_weight, &x));
    TRY(ffn->forward(ctx, x, h));
    ctx->scratch->offset = mark;
    return 0;
  }
};

// -- embedding, positions, head ---------------------------------------------------

struct TokenEmbedding : Embedding {
  const void* table;
  int vocab, width, dtype;
  int forward(EngCtx* ctx, const EngMat& out, const EngMat& add_table, const int* add_index) override {
    if (out.cols != width || out.dtype != DT_F32 || out.ld != width) FAIL("embedding: out must be float32 [tokens, %d]", width);
    if (add_table.p && (add_table.cols != width || add_table.dtype != dtype))
      FAIL("embedding: the position table must share the token table's width and dtype");
    KERNEL(k_embed, ctx, out.p, table, ctx->token_ids, add_table.p, add_table.p ? add_index : nullptr, out.rows,
           width, dtype, ctx->stream);
    return 0;
  }
};

struct LearnedPositions : Position {
  const void* table;
  int max_positions, width, dtype;
  int embedding_term(EngCtx* ctx, EngMat* t, const int** index) override {
    *t = EngMat{(void*)table, max_positions, width, width, dtype};
    *index = ctx->positions;
    return 0;
  }
};

struct LinearHead : Head {
  EngWeight w;
  int forward(EngCtx* ctx, const EngValue& x, const EngMat& out) override {
    return linear(ctx, out, x, w, nullptr, false, false, 0, nullptr, 0, &ctx->pending);
  }
};

// -- the model ---------------------------------------------------------------------

struct Run {
  int layer, cache, writes;
};

struct Model : EngPart {
  int width, vocab;
  Embedding* embedding;
  Position* positions;
  std::vector<Block*> layers;
  std::vector<Run> schedule;
  Norm* final_norm;
  Head* head;
  Model() : EngPart(KIND_MODEL) {}

  int forward(EngCtx* ctx) {
    if (ctx->stats) ctx->stats->steps++;
    EngMat h;
    TRY(take(ctx, ctx->n_tokens, width, DT_F32, &h));
    EngMat add = {};
    const int* add_index = nullptr;
    if (positions) TRY(positions->embedding_term(ctx, &add, &add_index));
    TRY(embedding->forward(ctx, h, add, add_index));
    EngPending* pending = &ctx->pending;
    for (const Run& run : schedule) {
      Block* block = layers[run.layer];
      // a block that does not know of pending sums gets the stream with everything added
      pending->allowed = block->handles_pending;
      if (!pending->allowed) TRY(settle(ctx, pending));
      TRY(block->forward(ctx, h, run.cache, run.writes != 0));
    }
    pending->allowed = 0;
    if (ctx->n_wanted == 0 || !final_norm->settles_pending) TRY(settle(ctx, pending));
    if (ctx->n_wanted == 0) return 0;
    EngValue x;
    if (ctx->wants_every_row)
      TRY(final_norm->forward(ctx, h, nullptr, 0, false, nullptr, false, &x));
    else
      TRY(final_norm->forward(ctx, h, ctx->wanted_rows, ctx->n_wanted, false, nullptr, false, &x));
    if (!ctx->logits || ctx->logits_rows < ctx->n_wanted) FAIL("the step's logits buffer is too small");
    const EngMat logits = {ctx->logits, ctx->n_wanted, vocab, vocab, DT_F32};
    return head->forward(ctx, x, logits);
  }
};

// ---------------------------------------------------------------------------
// the host's routines for parts in libraries of their own

static int host_materialize(EngCtx* ctx, const EngValue* v, EngMat* out) { return materialize(ctx, *v, out); }

static int host_slot_pages(EngCtx* ctx, int slot, int q_width, int kv_width, EngScatter* sc) {
  if (slot < 0 || slot >= ctx->n_slots) FAIL("cache slot %d of %d", slot, ctx->n_slots);
  const EngSlot& s = ctx->slots[slot];
  if (s.group < 0 || !s.k) FAIL("cache slot %d holds no pages", slot);
  if (s.v_head_dim != s.head_dim || s.v_page_stride != s.page_stride)
    FAIL("cache slot %d holds values of width %d beside keys of %d: no one description fits both", slot,
         s.v_head_dim, s.head_dim);
  sc->k = s.k, sc->v = s.v, sc->page_stride = s.page_stride;
  sc->n_kv_heads = s.n_kv_heads, sc->head_dim = s.head_dim, sc->page_size = s.page_size, sc->dtype = s.dtype;
  sc->block_table = ctx->block_tables[s.group], sc->max_blocks = ctx->table_width[s.group];
  sc->token_req = ctx->token_req, sc->positions = ctx->positions;
  sc->q_width = q_width, sc->kv_width = kv_width;
  return 0;
}

static int host_kv_write(EngCtx* ctx, const EngMat* k, const EngMat* v, const EngScatter* sc) {
  return kv_write(ctx, *k, *v, *sc);
}

static void* host_kernel(const char* library, const char* symbol) {
  return g_resolver ? g_resolver(library, symbol) : nullptr;
}

static void host_launched(EngCtx* ctx) {
  if (ctx->stats) ctx->stats->launches++;
}

static int host_fail(const char* format, ...) {
  va_list args;
  va_start(args, format);
  vsnprintf(g_err, sizeof(g_err), format, args);
  va_end(args);
  return 1;
}

extern "C" int eng_linear(EngCtx* ctx, const EngLinear* c, EngPending* pending);

extern "C" const EngHost* eng_host(void) {
  static const EngHost host = {take, host_materialize, eng_linear, settle, host_slot_pages, host_kv_write,
                               host_kernel, host_launched, host_fail};
  return &host;
}

// ---------------------------------------------------------------------------
// C entry points

template <typename T>
static T* as(EngPart* p, int kind, const char* what) {
  if (!p || p->kind != kind) {
    snprintf(g_err, sizeof(g_err), "%s: not a part of that kind", what);
    return nullptr;
  }
  return static_cast<T*>(p);
}

extern "C" EngPart* eng_make_callback(int kind, int part_id, int flags) {
  switch (kind) {
    case KIND_NORM: return new PyNorm(part_id, flags);
    case KIND_MIXER: return new PyMixer(part_id, flags);
    case KIND_FFN: return new PyFeedForward(part_id, flags);
    case KIND_BLOCK: return new PyBlock(part_id, flags);
    case KIND_POSITION: return new PyPosition(part_id, flags);
    case KIND_EMBEDDING: return new PyEmbedding(part_id);
    case KIND_HEAD: return new PyHead(part_id);
  }
  snprintf(g_err, sizeof(g_err), "eng_make_callback: unknown kind %d", kind);
  return nullptr;
}

extern "C" EngPart* eng_make_layernorm(int width, float eps, const float* gamma, const float* beta) {
  return new LayerNorm(width, eps, gamma, beta);
}

extern "C" EngPart* eng_make_attention(int width, int n_heads, int n_kv_heads, int head_dim, float scale,
                                       int window, const EngWeight* qkv_w, const float* qkv_b,
                                       const EngWeight* out_w, const float* out_b, EngPart* position,
                                       int array_base) {
  Position* pos = nullptr;
  if (position && !(pos = as<Position>(position, KIND_POSITION, "eng_make_attention"))) return nullptr;
  if (array_base < 0 || array_base + ARR_ROWS_ARE_REQUESTS >= ENG_MAX_ARRAYS) {
    snprintf(g_err, sizeof(g_err), "eng_make_attention: array ids from %d do not fit", array_base);
    return nullptr;
  }
  Attention* a = new Attention();
  a->width = width, a->n_heads = n_heads, a->n_kv_heads = n_kv_heads, a->head_dim = head_dim;
  a->scale = scale, a->window = window, a->q_width = n_heads * head_dim, a->kv_width = n_kv_heads * head_dim;
  a->qkv_w = *qkv_w, a->out_w = *out_w, a->qkv_b = qkv_b, a->out_b = out_b;
  a->position = pos, a->array_base = array_base;
  a->first_weight = &a->qkv_w;
  return a;
}

extern "C" EngPart* eng_make_gelu_mlp(int width, int inner_padded, const EngWeight* fc_w, const float* fc_b,
                                      const EngWeight* proj_w, const float* proj_b) {
  GeluMlp* m = new GeluMlp();
  m->width = width, m->inner = inner_padded;
  m->fc_w = *fc_w, m->proj_w = *proj_w, m->fc_b = fc_b, m->proj_b = proj_b;
  m->first_weight = &m->fc_w;
  return m;
}

extern "C" EngPart* eng_make_pre_norm_block(EngPart* mixer_norm, EngPart* mixer, EngPart* ffn_norm,
                                            EngPart* ffn) {
  PreNormBlock* b = new PreNormBlock();
  b->mixer_norm = as<Norm>(mixer_norm, KIND_NORM, "eng_make_pre_norm_block");
  b->mixer = as<Mixer>(mixer, KIND_MIXER, "eng_make_pre_norm_block");
  b->ffn_norm = as<Norm>(ffn_norm, KIND_NORM, "eng_make_pre_norm_block");
  b->ffn = as<FeedForward>(ffn, KIND_FFN, "eng_make_pre_norm_block");
  if (!b->mixer_norm || !b->mixer || !b->ffn_norm || !b->ffn) {
    delete b;
    return nullptr;
  }
  return b;
}

extern "C" EngPart* eng_make_token_embedding(const void* table, int vocab, int width, int dtype) {
  TokenEmbedding* e = new TokenEmbedding();
  e->table = table, e->vocab = vocab, e->width = width, e->dtype = dtype;
  return e;
}

extern "C" EngPart* eng_make_learned_positions(const void* table, int max_positions, int width, int dtype) {
  LearnedPositions* p = new LearnedPositions();
  p->table = table, p->max_positions = max_positions, p->width = width, p->dtype = dtype;
  return p;
}

extern "C" EngPart* eng_make_linear_head(const EngWeight* w) {
  LinearHead* h = new LinearHead();
  h->w = *w;
  return h;
}

extern "C" EngPart* eng_make_model(int width, int vocab, EngPart* embedding, EngPart* positions, int n_layers,
                                   EngPart** layers, int n_runs, const int* run_layer, const int* run_cache,
                                   const int* run_writes, EngPart* final_norm, EngPart* head) {
  std::unique_ptr<Model> m(new Model());
  m->width = width, m->vocab = vocab;
  if (!(m->embedding = as<Embedding>(embedding, KIND_EMBEDDING, "eng_make_model"))) return nullptr;
  m->positions = nullptr;
  if (positions && !(m->positions = as<Position>(positions, KIND_POSITION, "eng_make_model"))) return nullptr;
  for (int i = 0; i < n_layers; ++i) {
    Block* b = as<Block>(layers[i], KIND_BLOCK, "eng_make_model");
    if (!b) return nullptr;
    m->layers.push_back(b);
  }
  for (int i = 0; i < n_runs; ++i) {
    if (run_layer[i] < 0 || run_layer[i] >= n_layers) {
      snprintf(g_err, sizeof(g_err), "eng_make_model: run %d names layer %d of %d", i, run_layer[i], n_layers);
      return nullptr;
    }
    m->schedule.push_back(Run{run_layer[i], run_cache[i], run_writes[i]});
  }
  if (!(m->final_norm = as<Norm>(final_norm, KIND_NORM, "eng_make_model"))) return nullptr;
  if (!(m->head = as<Head>(head, KIND_HEAD, "eng_make_model"))) return nullptr;
  return m.release();
}

extern "C" void eng_free(EngPart* part) { delete part; }

extern "C" int eng_model_forward(EngPart* model, EngCtx* ctx) {
  Model* m = as<Model>(model, KIND_MODEL, "eng_model_forward");
  return m ? m->forward(ctx) : 1;
}

extern "C" int eng_block_forward(EngPart* block, EngCtx* ctx, const EngMat* h, int cache_slot,
                                 int writes_cache) {
  Block* b = as<Block>(block, KIND_BLOCK, "eng_block_forward");
  return b ? b->forward(ctx, *h, cache_slot, writes_cache != 0) : 1;
}

extern "C" int eng_norm_forward(EngPart* norm, EngCtx* ctx, const EngMat* x, const int* rows, int n_rows,
                                int lazy, const EngWeight* ahead, EngValue* out) {
  Norm* n = as<Norm>(norm, KIND_NORM, "eng_norm_forward");
  return n ? n->forward(ctx, *x, rows, n_rows, lazy != 0, ahead, false, out) : 1;
}

extern "C" int eng_mixer_forward(EngPart* mixer, EngCtx* ctx, const EngValue* x, const EngMat* residual,
                                 int cache_slot, int writes_cache) {
  Mixer* m = as<Mixer>(mixer, KIND_MIXER, "eng_mixer_forward");
  return m ? m->forward(ctx, *x, *residual, cache_slot, writes_cache != 0) : 1;
}

extern "C" int eng_ffn_forward(EngPart* ffn, EngCtx* ctx, const EngValue* x, const EngMat* residual) {
  FeedForward* f = as<FeedForward>(ffn, KIND_FFN, "eng_ffn_forward");
  return f ? f->forward(ctx, *x, *residual) : 1;
}

extern "C" int eng_embedding_forward(EngPart* embedding, EngCtx* ctx, const EngMat* out, EngPart* positions) {
  Embedding* e = as<Embedding>(embedding, KIND_EMBEDDING, "eng_embedding_forward");
  if (!e) return 1;
  EngMat add = {};
  const int* index = nullptr;
  if (positions) {
    Position* p = as<Position>(positions, KIND_POSITION, "eng_embedding_forward");
    if (!p) return 1;
    TRY(p->embedding_term(ctx, &add, &index));
  }
  return e->forward(ctx, *out, add, index);
}

extern "C" int eng_head_forward(EngPart* head, EngCtx* ctx, const EngValue* x, const EngMat* out) {
  Head* h = as<Head>(head, KIND_HEAD, "eng_head_forward");
  return h ? h->forward(ctx, *x, *out) : 1;
}

// A pending sum outside a step's own (ops.kernels.PendingSum): the same three operations.
extern "C" int eng_pending_settle(EngCtx* ctx, EngPending* pending) { return settle(ctx, pending); }

extern "C" int eng_pending_can_norm(const EngPending* pending, const EngMat* x) {
  bool yes = false;
  if (can_norm(*pending, *x, &yes) != 0) return 0;
  return yes ? 1 : 0;
}

extern "C" int eng_pending_settle_normed(EngCtx* ctx, EngPending* pending, const EngMat* out, const float* gamma,
                                         const float* beta, float eps, const EngWeight* ahead, int out_packed) {
  return settle_normed(ctx, pending, *out, gamma, beta, eps, ahead, out_packed != 0);
}

extern "C" int eng_read_ahead_pays(const EngCtx* ctx, const EngWeight* w, int n_rows, int with_norm) {
  bool yes = false;
  if (read_ahead_pays(ctx, w, n_rows, with_norm != 0, &yes) != 0) return 0;
  return yes ? 1 : 0;
}

// Sizes of the structs that the Python side mirrors, in the order of ops/native.py's check.
extern "C" int eng_struct_sizes(long* out, int n) {
  const long sizes[] = {sizeof(EngMat),     sizeof(EngWeight), sizeof(EngValue), sizeof(EngPending),
                        sizeof(EngSlot),    sizeof(EngScratch), sizeof(EngStats), sizeof(EngCtx),
                        sizeof(EngCall),    sizeof(EngScatter), sizeof(EngLinear),
                        (long)offsetof(EngCtx, pending), (long)offsetof(EngCall, nbytes)};
  const int have = (int)(sizeof(sizes) / sizeof(sizes[0]));
  for (int i = 0; i < n && i < have; ++i) out[i] = sizes[i];
  return have;
}
