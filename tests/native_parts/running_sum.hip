// A mixer with per-request state as a native part in a library of its own: nothing of the
// framework's files knows it.  s[request] += sum of the portion's rows; every row of the
// portion adds the new s to the residual stream.  (A toy for the tests, no model's layer.)
#include "engine_parts.h"

static const EngHost* host = nullptr;

// one block a request of the step: its rows are consecutive, q_start .. q_start + n
__global__ void running_sum_kernel(float* state, size_t state_stride, const int* slot_ids, const int* token_req,
                                   const void* x, int ldx, int x_is_bf16, float* residual, int ldr, int n_tokens,
                                   int width) {
  const int req = blockIdx.x;
  // the request's rows: found by scanning token_req (tiny steps; a toy)
  int first = -1, n = 0;
  for (int t = 0; t < n_tokens; ++t)
    if (token_req[t] == req) {
      if (first < 0) first = t;
      ++n;
    }
  if (n == 0) return;
  float* s = state + (size_t)slot_ids[req] * state_stride;
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    float add = 0.f;
    for (int t = first; t < first + n; ++t) {
      if (x_is_bf16) {
        const unsigned int bits = ((const unsigned short*)x)[(size_t)t * ldx + c];
        add += __uint_as_float(bits << 16);
      } else {
        add += ((const float*)x)[(size_t)t * ldx + c];
      }
    }
    const float now = s[c] + add;
    s[c] = now;
    for (int t = first; t < first + n; ++t) residual[(size_t)t * ldr + c] += now;
  }
}

struct RunningSum : Mixer {
  int width;
  explicit RunningSum(int w) : width(w) {}
  int forward(EngCtx* ctx, const EngValue& x, const EngMat& residual, int slot, bool) override {
    EngMat xm;
    if (host->materialize(ctx, &x, &xm)) return 1;
    if (slot < 0 || slot >= ctx->n_slots) return host->fail("running sum: cache slot %d of %d", slot, ctx->n_slots);
    const EngSlot& s = ctx->slots[slot];
    if (s.group != -2 || !s.k || s.dtype != 0 || (int)s.page_stride != width)
      return host->fail("running sum: cache slot %d is not a float32 state of width %d", slot, width);
    if (xm.cols != width || residual.cols != width || residual.dtype != 0)
      return host->fail("running sum: rows of width %d, a float32 stream", width);
    hipLaunchKernelGGL(running_sum_kernel, dim3(ctx->n_requests), dim3(64), 0, ctx->stream, (float*)s.k, s.page_stride,
                       ctx->slot_ids, ctx->token_req, xm.p, xm.ld, xm.dtype == 1 ? 1 : 0, (float*)residual.p,
                       residual.ld, ctx->n_tokens, width);
    if (hipGetLastError() != hipSuccess) return host->fail("running sum: the launch failed");
    host->launched(ctx);
    return 0;
  }
};

extern "C" EngPart* make_running_sum(const EngHost* h, int width) {
  host = h;
  return new RunningSum(width);
}
