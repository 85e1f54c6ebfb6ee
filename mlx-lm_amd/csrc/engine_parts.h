// What a native part is made of: the base classes that the native walk of a step calls
// (norm, position encoding, mixer, feed-forward, block, embedding, head) and the host's own
// routines that a part needs (EngHost: scratch memory, the product routine with its choice of
// kernels and splits, pending sums, cache slots, kernel look-up, errors).
//
// A part with a native twin is one .hip file: a class here derived from the base of its
// family, its kernels, and an extern "C" maker that takes the host's table and the part's
// sizes, constants and device pointers and returns the EngPart*; the part's Python class
// calls that maker from make_native().  The walk (csrc/engine.hip) needs no change for it: it
// knows a part by its family's interface only, and a library of its own is loaded beside the
// others.  The built-in parts (LayerNorm, Attention, GeluMlp, PreNormBlock, ...) are written
// the same way, inside engine.hip.
//
// No counterpart in the reference, whose parts are Python modules over an array library
// (mlx_lm/models/gpt2.py:28-108).
#pragma once

#include "engine.h"

#ifdef __cplusplus

enum { KIND_NORM = ENG_NORM, KIND_MIXER = ENG_MIXER, KIND_FFN = ENG_FFN, KIND_BLOCK = ENG_BLOCK, KIND_POSITION = ENG_POSITION,
       KIND_EMBEDDING = ENG_EMBEDDING, KIND_HEAD = ENG_HEAD, KIND_MODEL = ENG_MODEL };

struct EngPart {
  int kind;
  explicit EngPart(int k) : kind(k) {}
  virtual ~EngPart() {}
};

struct Norm : EngPart {
  bool settles_pending = false, reads_ahead = false;
  Norm() : EngPart(KIND_NORM) {}
  // The norm of rows of the float32 stream `x` (all, or those listed in `rows`).
  // `ahead`: the weights that the result meets first, if the caller knows them; `may_pack`: whoever
  // takes the result takes it in the packed order too (EngValue.packed), where those weights'
  // product reads it faster so.
  virtual int forward(EngCtx* ctx, const EngMat& x, const int* rows, int n_rows, bool lazy,
                      const EngWeight* ahead, bool may_pack, EngValue* out) = 0;
};

struct Position : EngPart {
  Position() : EngPart(KIND_POSITION) {}
  virtual int embedding_term(EngCtx* ctx, EngMat* table, const int** index) {
    table->p = nullptr, *index = nullptr;
    return 0;
  }
  virtual int rotate(EngCtx*, const EngMat&, const EngMat&) { return 0; }
  virtual bool rotates() const { return false; }
};

// forward adds the mixer's output into `residual` (float32 rows of the stream); `slot` is its
// cache slot (EngCtx.slots[slot]: pages of keys and values, or a state tensor), `writes` whether
// this run puts the step's tokens there.  accepts_lazy: x may be a norm not computed yet
// (EngHost.materialize computes it); accepts_packed: x may come in the packed order;
// first_weight: the weights that x meets first, for kernels before it that read ahead.
struct Mixer : EngPart {
  bool accepts_lazy = false, accepts_packed = false;
  const EngWeight* first_weight = nullptr;
  Mixer() : EngPart(KIND_MIXER) {}
  virtual int forward(EngCtx* ctx, const EngValue& x, const EngMat& residual, int slot, bool writes) = 0;
};

struct FeedForward : EngPart {
  bool accepts_lazy = false, accepts_packed = false;
  const EngWeight* first_weight = nullptr;
  FeedForward() : EngPart(KIND_FFN) {}
  virtual int forward(EngCtx* ctx, const EngValue& x, const EngMat& residual) = 0;
};

struct Block : EngPart {
  bool handles_pending = false;
  Block() : EngPart(KIND_BLOCK) {}
  virtual int forward(EngCtx* ctx, const EngMat& h, int slot, bool writes) = 0;
};

struct Embedding : EngPart {
  Embedding() : EngPart(KIND_EMBEDDING) {}
  virtual int forward(EngCtx* ctx, const EngMat& out, const EngMat& add_table, const int* add_index) = 0;
};

struct Head : EngPart {
  Head() : EngPart(KIND_HEAD) {}
  virtual int forward(EngCtx* ctx, const EngValue& x, const EngMat& out) = 0;
};

#endif  // __cplusplus
