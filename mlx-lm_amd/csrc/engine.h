// The native host of a step: the structs that the Python side fills (layouts
// are mirrored with ctypes in ops/native.py) and the entry points of
// engine.hip.  A model is a tree of parts (norms, mixers, feed-forwards,
// blocks, embedding, head), each made by an eng_make_* call from its sizes,
// constants and device pointers; eng_model_forward runs a whole step's launches
// from one call.  A part that exists only in Python takes its place in the tree
// as a callback part.
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ENG_MAX_ARRAYS 32  // named integer arrays (and scalars) that parts ask the packer for
#define ENG_MAX_GROUPS 8   // cache groups (block tables) a step can carry

// A matrix with contiguous rows on the device.  dtype: 0 float32, 1 bfloat16, 2 int32.
typedef struct {
  void* p;
  int rows, cols, ld, dtype;
} EngMat;

// A weight matrix [N, K]: row-major, and for bfloat16 also in the order the
// decode kernel's lanes read it (packed == null where there is no such copy).
typedef struct {
  const void* w;
  const void* packed;
  int N, K, ldw, dtype;
  size_t chunk_bytes;
  int n_chunks, pad_;
} EngWeight;

// The input of a mixer or feed-forward: a matrix, or the LayerNorm of float32
// rows that is not computed yet (lazy != 0; m then gives shape and dtype only).
typedef struct {
  EngMat m;
  int lazy, ldx;
  const float* x;
  const float* gamma;
  const float* beta;
  float eps;
  // packed != 0: m.p holds the bfloat16 rows in tiles of 16 rows x 64 columns, each tile in the
  // order of the packed weights' tiles (what the product of 17 to 64 rows reads fastest); m.ld is
  // not used then.  Only a part that asked for it (eng_wants_packed_rows) is handed such a value.
  int packed;
} EngValue;

// Partial products that still have to be added into the residual stream.
typedef struct {
  float* target;
  int rows, cols, ld, n_splits;
  float* ws;
  const float* bias;
  int allowed, pad_;
} EngPending;

// One cache slot: pages of keys and values, or a state tensor, or nothing.  A slot of per-request
// state (group == -2) has the tensor [max_requests, ...] at k, the elements a request's row holds
// in page_stride and the element type in dtype; a request's row is EngCtx.slot_ids[request].
typedef struct {
  void* k;
  void* v;
  size_t page_stride;    // elements from a page's keys to the next page's
  size_t v_page_stride;  // the same for values (the built-in attention asks for equal strides and widths)
  int n_kv_heads, head_dim, page_size, dtype;
  int group, v_head_dim;  // group: index of the slot's block table in a step; -1: nothing; -2: a state tensor
} EngSlot;

// Scratch memory of a step: a bump allocator over one device buffer.  The
// struct is shared by both sides, so a Python part's allocations and a native
// part's follow each other in one sequence.
typedef struct {
  char* base;
  size_t size, offset, peak;
  int frozen, pad_;
} EngScratch;

typedef struct {
  long launches, settle_normed, settle_plain, callbacks, steps;
  long key_splits_most;  // the most parts that a row kernel split a row's keys into
} EngStats;

// One step's batch as the parts see it.
typedef struct {
  hipStream_t stream;
  int dtype;  // compute dtype: 0 float32, 1 bfloat16
  int n_tokens, n_requests, n_wanted, wants_every_row;
  int force_splits;  // tests: split K wherever the kernels can
  const int* token_ids;
  const int* positions;
  const int* token_req;
  const int* wanted_rows;
  const int* slot_ids;
  const int* arrays[ENG_MAX_ARRAYS];  // parts' own arrays, by the id the packer gave their names
  long counts[ENG_MAX_ARRAYS];        // their lengths (or, for a scalar, its value)
  const int* block_tables[ENG_MAX_GROUPS];
  int table_width[ENG_MAX_GROUPS];
  const EngSlot* slots;
  int n_slots, n_compute_units;
  EngScratch* scratch;
  float* split_ws;
  size_t split_ws_floats;
  float* logits;  // [>= n_wanted, vocab] float32
  long logits_rows;
  EngPending pending;
  const EngWeight* read_ahead;
  EngStats* stats;
  void* py;  // the Python side's own handle of this step (opaque here)
} EngCtx;

// What a callback part's method gets and gives.
typedef struct {
  EngMat x, residual, out, q, k;
  const int* rows;
  int n_rows, cache_slot, writes_cache, lazy;
  // results: a norm's output; an embedding term's table and index
  EngMat result;
  const int* index;
  size_t nbytes;  // ENG_CB_GROW: what the scratch buffer has to hold
} EngCall;

enum {
  ENG_CB_NORM = 1, ENG_CB_MIXER, ENG_CB_FFN, ENG_CB_BLOCK, ENG_CB_ROTATE, ENG_CB_EMBEDDING_TERM,
  ENG_CB_EMBEDDING, ENG_CB_HEAD, ENG_CB_GROW
};

// int callback(part_id, method, ctx, call): 0, or 1 after keeping the Python exception
typedef int (*eng_callback_t)(int, int, EngCtx*, EngCall*);
// void* resolver(library, symbol): loads (builds, if need be) csrc/<library>.hip's library
typedef void* (*eng_resolver_t)(const char*, const char*);

void eng_set_hooks(eng_resolver_t resolver, eng_callback_t callback);
int eng_struct_sizes(long* out, int n);  // for the Python side's check of its mirrored layouts
int eng_compute_units(void);
// queries a tile of attn_tile's and of attn_prefill's work lists holds (attention_tiles.h)
void eng_attn_tile_sizes(int* tile, int* prefill_tile);
// The context length from which a decode step may split a row's keys over blocks.
int eng_rows_split_from(void);

// flags of a callback part
#define ENG_ACCEPTS_LAZY 1
#define ENG_SETTLES_PENDING 2
#define ENG_HANDLES_PENDING 4
#define ENG_READS_AHEAD 8

typedef struct EngPart EngPart;

// kinds of part (eng_make_callback's first argument)
enum {
  ENG_NORM = 1, ENG_MIXER, ENG_FFN, ENG_BLOCK, ENG_POSITION, ENG_EMBEDDING, ENG_HEAD, ENG_MODEL
};

EngPart* eng_make_callback(int kind, int part_id, int flags);
EngPart* eng_make_layernorm(int width, float eps, const float* gamma, const float* beta);
EngPart* eng_make_attention(int width, int n_heads, int n_kv_heads, int head_dim, float scale, int window,
                            const EngWeight* qkv_w, const float* qkv_b, const EngWeight* out_w,
                            const float* out_b, EngPart* position, int array_base);
EngPart* eng_make_gelu_mlp(int width, int inner_padded, const EngWeight* fc_w, const float* fc_b,
                           const EngWeight* proj_w, const float* proj_b);
EngPart* eng_make_pre_norm_block(EngPart* mixer_norm, EngPart* mixer, EngPart* ffn_norm, EngPart* ffn);
EngPart* eng_make_token_embedding(const void* table, int vocab, int width, int dtype);
EngPart* eng_make_learned_positions(const void* table, int max_positions, int width, int dtype);
EngPart* eng_make_linear_head(const EngWeight* w);
EngPart* eng_make_model(int width, int vocab, EngPart* embedding, EngPart* positions, int n_layers,
                        EngPart** layers, int n_runs, const int* run_layer, const int* run_cache,
                        const int* run_writes, EngPart* final_norm, EngPart* head);
void eng_free(EngPart* part);

// Each returns 0, or 1 with the text in mlxlm_last_error() (2: a callback kept a Python exception).
int eng_model_forward(EngPart* model, EngCtx* ctx);
int eng_block_forward(EngPart* block, EngCtx* ctx, const EngMat* h, int cache_slot, int writes_cache);
int eng_norm_forward(EngPart* norm, EngCtx* ctx, const EngMat* x, const int* rows, int n_rows, int lazy,
                     const EngWeight* ahead, EngValue* out);
int eng_mixer_forward(EngPart* mixer, EngCtx* ctx, const EngValue* x, const EngMat* residual, int cache_slot,
                      int writes_cache);
int eng_ffn_forward(EngPart* ffn, EngCtx* ctx, const EngValue* x, const EngMat* residual);
int eng_embedding_forward(EngPart* embedding, EngCtx* ctx, const EngMat* out, EngPart* positions);
int eng_head_forward(EngPart* head, EngCtx* ctx, const EngValue* x, const EngMat* out);
int eng_settle(EngCtx* ctx);

// out = epilogue(a @ w^T + bias): the choice among the product kernels, the split of K and its
// second kernel, the norm prologue and the cache scatter; what ops.kernels.linear calls too.
typedef struct {
  void* k;
  void* v;
  size_t page_stride;
  int n_kv_heads, head_dim, page_size, dtype;
  const int* block_table;
  const int* token_req;
  const int* positions;
  int max_blocks, q_width, kv_width, pad_;
} EngScatter;  // where the key and value columns of a fused q/k/v projection go
typedef struct {
  EngMat out;
  EngValue a;
  EngWeight w;
  const float* bias;
  const EngScatter* scatter;
  int gelu, accumulate, variant, splits;  // splits: 0 = the library chooses
  int out_packed, pad_;  // out (bfloat16, [rows padded to 16][cols padded to 64]) in the packed order
} EngLinear;
int eng_linear(EngCtx* ctx, const EngLinear* call, EngPending* pending);
// A pending sum outside a step's own: add it; whether the fused sum-and-norm takes it; add and norm.
int eng_pending_settle(EngCtx* ctx, EngPending* pending);
int eng_pending_can_norm(const EngPending* pending, const EngMat* x);
int eng_pending_settle_normed(EngCtx* ctx, EngPending* pending, const EngMat* out, const float* gamma,
                              const float* beta, float eps, const EngWeight* ahead, int out_packed);
int eng_read_ahead_pays(const EngCtx* ctx, const EngWeight* w, int n_rows, int with_norm);
// 1 if the product of these sizes would norm a lazy input in its own prologue
int eng_linear_norms_itself(const EngCtx* ctx, int M, int N, int K, int dtype, int splits);
// 1 if the product of n_rows rows with w reads its rows fastest in the packed order (EngValue.packed)
int eng_wants_packed_rows(const EngCtx* ctx, const EngWeight* w, int n_rows);

// The host's own routines, for a native part that lives in a library of its own (engine_parts.h).
// Each returns 0, or non-zero with the text kept where mlxlm_last_error() of the host finds it.
typedef struct EngHost {
  // rows x cols values of dtype in the step's scratch memory (freed when the block is done)
  int (*take)(EngCtx* ctx, int rows, int cols, int dtype, EngMat* out);
  // a value as a matrix: a norm not computed yet is computed now
  int (*materialize)(EngCtx* ctx, const EngValue* v, EngMat* out);
  // out = epilogue(a @ w^T + bias): eng_linear
  int (*linear)(EngCtx* ctx, const EngLinear* call, EngPending* pending);
  // add a pending sum into its target (eng_pending_settle); the step's own is &ctx->pending
  int (*settle)(EngCtx* ctx, EngPending* pending);
  // where the keys and values of cache slot `slot` go and come from in this step
  int (*slot_pages)(EngCtx* ctx, int slot, int q_width, int kv_width, EngScatter* out);
  // keys and values of this step's tokens into their pages
  int (*kv_write)(EngCtx* ctx, const EngMat* k, const EngMat* v, const EngScatter* sc);
  // an entry point of csrc/<library>.hip's library (built at first use), or null
  void* (*kernel)(const char* library, const char* symbol);
  // a launch was made (the step's counters)
  void (*launched)(EngCtx* ctx);
  // keep a message as the error of the call under way; returns 1
  int (*fail)(const char* format, ...);
} EngHost;
const EngHost* eng_host(void);

#ifdef __cplusplus
}
#endif
