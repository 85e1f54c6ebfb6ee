// Sampling from rows of 32-bit logits, one block per row, everything in 32-bit.
//
// sample_rows does, in the reference's order (mlx_lm/sample_utils.py:46-67 and
// mlx_lm/generate.py:411-412):
//   logprobs = logits - logsumexp(logits)
//   temp == 0: token = argmax(logprobs)
//   else: top_p -> min_p -> xtc -> top_k filters, then a draw from
//         softmax(filtered / temp).
// Every filter of the reference keeps the tokens whose log-probability lies
// on one side of a threshold, so the kept set is always
//   { lo <= lp <= hi } plus the xtc special tokens above hi,
// and each filter only moves lo or hi.  Thresholds that the reference finds by
// sorting (top_p: sample_utils.py:204-237, top_k: 129-151, the min_p floor:
// 154-201) are found here by bisection over the ordered bit patterns of the
// floats, each probe being one block-wide sum or count.  Tokens that tie with
// a threshold are all kept.  The draw is Gumbel-max with uniforms hashed from
// (seed, counter, token id), so a row's result does not depend on the rows
// beside it (the reference draws with mx.random.categorical,
// sample_utils.py:279-281).
//
// apply_logit_bias and apply_penalties are the logits processors of
// mlx_lm/sample_utils.py:72-126,284-369, run before sample_rows.
#include "common.h"

#define SAMPLE_THREADS 1024
#define CAND_CAP 4608  // tokens in the list of candidates: three arrays of 18 KB in LDS

struct SampleArgs {
  int* tokens;            // [R]
  float* token_logprob;   // [R]
  float* logprobs;        // [R, ld_logprobs] or null
  const float* logits;    // [R, ld]
  const float* temp;      // [R]
  const float* top_p;     // [R]
  const float* min_p;     // [R]
  const int* min_keep;    // [R]
  const int* top_k;       // [R]
  const float* xtc_prob;  // [R]
  const float* xtc_thr;   // [R]
  const unsigned long long* seed;  // [R]
  const int* counter;     // [R]
  const int* xtc_special; // [n_special]
  int n_special;
  int vocab, ld, ld_logprobs;
};

__device__ __forceinline__ unsigned int ordered_key(float f) {
  const unsigned int b = __float_as_uint(f);
  return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}
__device__ __forceinline__ float key_to_float(unsigned int k) {
  const unsigned int b = (k & 0x80000000u) ? (k & 0x7fffffffu) : ~k;
  return __uint_as_float(b);
}

__device__ __forceinline__ unsigned long long mix64(unsigned long long x) {
  x ^= x >> 30;
  x *= 0xBF58476D1CE4E5B9ull;
  x ^= x >> 27;
  x *= 0x94D049BB133111EBull;
  x ^= x >> 31;
  return x;
}
// The key of a row's draws: 64 bits mixed from (seed, counter), once per thread.
__device__ __forceinline__ unsigned long long draw_key(unsigned long long seed, unsigned int counter) {
  return mix64(seed + 0x9E3779B97F4A7C15ull * (unsigned long long)(counter + 1u));
}
// uniform in (0, 1), 24 bits, from a key and an index: two rounds of a 32-bit finalizer
// (multiply, shift, xor), each keyed with half the key.  32-bit multiplies only: 64-bit
// ones are several instructions each at a quarter of the rate, and this runs once per
// vocabulary entry on the one CU that has the row.
__device__ __forceinline__ unsigned int fmix32(unsigned int x) {
  x ^= x >> 16;
  x *= 0x85EBCA6Bu;
  x ^= x >> 13;
  x *= 0xC2B2AE35u;
  x ^= x >> 16;
  return x;
}
__device__ __forceinline__ float uniform01(unsigned long long key, unsigned int index) {
  unsigned int x = fmix32((index + 1u) * 0x9E3779B1u ^ (unsigned int)key);
  x = fmix32(x + (unsigned int)(key >> 32));
  return ((float)(x >> 8) + 0.5f) * (1.0f / 16777216.0f);
}

struct Kept {
  float lo, hi;
  const int* special;
  int n_special;
  __device__ __forceinline__ bool operator()(int i, float lp) const {
    if (!(lp >= lo)) return false;
    if (lp <= hi) return true;
    for (int s = 0; s < n_special; ++s)
      if (special[s] == i) return true;
    return false;
  }
};

// (value, index) argmax over the block; ties go to the lowest index
__device__ __forceinline__ void block_argmax(float& v, int& idx, float* redv, int* redi) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int nw = (blockDim.x + 63) >> 6;
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_xor(v, o, WAVE);
    const int oi = __shfl_xor(idx, o, WAVE);
    if (ov > v || (ov == v && oi < idx)) v = ov, idx = oi;
  }
  __syncthreads();
  if (lane == 0) redv[wave] = v, redi[wave] = idx;
  __syncthreads();
  v = redv[0], idx = redi[0];
  for (int w = 1; w < nw; ++w)
    if (redv[w] > v || (redv[w] == v && redi[w] < idx)) v = redv[w], idx = redi[w];
}

// f(i, x[i]) for this thread's elements of a row, i = tid, tid + nt, ... in that order, eight
// loads at a time: a loop that loads one value and then branches on it waits for memory once an
// element (49 trips in a row for a vocabulary of 50,257 and 1,024 threads: 24 us a row).
template <typename F>
__device__ __forceinline__ void for_row(const float* x, int V, int tid, int nt, F f) {
  constexpr int UN = 8;
  int i0 = tid;
  for (; i0 + (UN - 1) * nt < V; i0 += UN * nt) {
    float v[UN];
#pragma unroll
    for (int u = 0; u < UN; ++u) v[u] = x[i0 + u * nt];
    __builtin_amdgcn_sched_barrier(0);  // all eight go out before the first is used
#pragma unroll
    for (int u = 0; u < UN; ++u) f(i0 + u * nt, v[u]);
  }
  for (; i0 < V; i0 += nt) f(i0, x[i0]);
}

__global__ __launch_bounds__(SAMPLE_THREADS) void sample_rows_kernel(SampleArgs a) {
  __shared__ float red[32];
  __shared__ int redi[32];
  const int r = blockIdx.x;
  const int V = a.vocab;
  const float* x = a.logits + (size_t)r * a.ld;
  const int tid = threadIdx.x, nt = blockDim.x;

  // One pass over the row: running maximum, sum of exponentials relative to it
  // (rescaled whenever the maximum moves) and the first index of the maximum.
  float mx = -INFINITY, se = 0.f;
  int bi = 0x7fffffff;
  // Eight values at a time: their maximum first, then one rescale of the sum and eight
  // exponentials that do not wait for one another.
  {
    constexpr int UN = 8;
    int i0 = tid;
    for (; i0 + (UN - 1) * nt < V; i0 += UN * nt) {
      float v[UN];
#pragma unroll
      for (int u = 0; u < UN; ++u) v[u] = x[i0 + u * nt];
      __builtin_amdgcn_sched_barrier(0);
      float cm = v[0];
#pragma unroll
      for (int u = 1; u < UN; ++u) cm = fmaxf(cm, v[u]);
      if (cm > mx) {
        int first = UN - 1;
#pragma unroll
        for (int u = UN - 2; u >= 0; --u) first = v[u] == cm ? u : first;
        se *= expf(mx - cm);  // (exp(-inf) = 0 the first time)
        mx = cm, bi = i0 + first * nt;
      }
      const float base = mx == -INFINITY ? 0.f : mx;  // (nothing but -inf so far: every term is 0)
      float part = 0.f;
#pragma unroll
      for (int u = 0; u < UN; ++u) part += expf(v[u] - base);
      se += part;
    }
    for (; i0 < V; i0 += nt) {
      const float v = x[i0];
      if (v > mx) {
        se = se * expf(mx - v) + 1.f;
        mx = v, bi = i0;
      } else {
        se += expf(v - mx);
      }
    }
  }
  const float row_max = block_max(mx, red);
  se = block_sum(mx == -INFINITY ? 0.f : se * expf(mx - row_max), red);
  const float lse = row_max + logf(se);
  float bv = mx;
  block_argmax(bv, bi, red, redi);  // ties go to the lowest index
  mx = row_max;

  if (a.logprobs) {
    float* lp = a.logprobs + (size_t)r * a.ld_logprobs;
    for (int i = tid; i < V; i += nt) lp[i] = x[i] - lse;
  }

  const float temp = a.temp[r];
  if (temp == 0.f) {
    if (tid == 0) a.tokens[r] = bi, a.token_logprob[r] = bv - lse;
    return;
  }

  Kept kept;
  kept.lo = -INFINITY, kept.hi = INFINITY;
  kept.special = a.xtc_special, kept.n_special = 0;
  const float lp_max = mx - lse;
  const float top_p = a.top_p[r], min_p = a.min_p[r], xtc_prob = a.xtc_prob[r];
  const int top_k = a.top_k[r], min_keep = a.min_keep[r];
  const int lane = tid & 63, wave = tid >> 6;

  // ---- candidates ------------------------------------------------------------
  // The thresholds of top_p, top_k and min_tokens_to_keep lie among the most likely tokens.
  // Where some filter needs a bisection (32 probes, each a pass over the row: 170 us a filter at
  // GPT-2's vocabulary), the tokens nearest the maximum are first put into a list in LDS, as
  // many as fit: the bins of a histogram over lp_max - lp in quarters of a nat say how far down
  // the list can go.  One wave then bisects over the list (a fraction of a microsecond a probe),
  // and the draw runs over the list as well if every kept token is in it.  The list's order is
  // fixed (by thread, then by index), so sums over it are repeatable.  Whatever the list cannot
  // decide (a flat row, a nucleus of thousands of tokens, xtc) takes the passes over the row.
  __shared__ float c_lp[CAND_CAP], c_p[CAND_CAP];
  __shared__ int c_idx[CAND_CAP];
  __shared__ int hist[64];
  __shared__ int wave_tot[SAMPLE_THREADS / 64];
  __shared__ float bcast[2];
  auto bin_of = [&](float lp) {
    const float d = (lp_max - lp) * 4.f;
    return d < 63.f ? (int)d : 63;  // (lp = -inf: the last bin)
  };
  const bool bisects = (top_p > 0.f && top_p < 1.f) || top_k > 0 || (min_p != 0.f && min_keep > 1);
  bool cand = false;
  int n_cand = 0;
  float m_low = 0.f, noncand_max = -INFINITY;
  if (bisects && !(xtc_prob > 0.f) && V < (1 << 24)) {
    if (tid < 64) hist[tid] = 0;
    __syncthreads();
    // (the first and the last bin are counted in registers: on a flat row, or on a peaked one,
    // nearly every token falls into one of them, and adds to one LDS word take turns)
    float in_first = 0.f;
    for_row(x, V, tid, nt, [&](int, float v) {
      const int b = bin_of(v - lse);
      if (b == 0)
        in_first += 1.f;
      else if (b < 63)
        atomicAdd(&hist[b], 1);
    });
    in_first = block_sum(in_first, red);  // (exact: at most V < 2^24)
    int cum = 0, b_last = -1;
    for (int b = 0; b < 64; ++b) {
      cum = b == 63 ? V : cum + (b == 0 ? (int)in_first : hist[b]);
      if (cum <= CAND_CAP) b_last = b, n_cand = cum;
    }
    if (b_last >= 0) {
      cand = true;
      int cnt = 0;
      float low = 0.f, ncmax = -INFINITY;
      for_row(x, V, tid, nt, [&](int, float v) {
        const float lp = v - lse;
        if (bin_of(lp) <= b_last) {
          ++cnt;
        } else {
          low += expf(lp);
          ncmax = fmaxf(ncmax, lp);
        }
      });
      m_low = block_sum(low, red);
      noncand_max = block_max(ncmax, red);
      // where this thread's candidates start: the counts of the threads before it
      int incl = cnt;
#pragma unroll
      for (int o = 1; o < 64; o <<= 1) {
        const int up = __shfl_up(incl, o, WAVE);
        if (lane >= o) incl += up;
      }
      __syncthreads();
      if (lane == 63) wave_tot[wave] = incl;
      __syncthreads();
      int pos = incl - cnt;
      for (int w = 0; w < wave; ++w) pos += wave_tot[w];
      for_row(x, V, tid, nt, [&](int i, float v) {
        const float lp = v - lse;
        if (bin_of(lp) <= b_last) {
          c_lp[pos] = lp, c_p[pos] = expf(lp), c_idx[pos] = i;
          ++pos;
        }
      });
      __syncthreads();
    }
  }

  // top_p: keep lp >= v*, v* the smallest value whose ascending cumulative
  // probability H(v) = sum_{lp_j <= v} p_j exceeds 1 - top_p.
  if (top_p > 0.f && top_p < 1.f) {
    const float need = 1.f - top_p;
    if (cand && m_low <= need) {
      // v* is in the list: H(v) = what lies below the list + the list's part
      if (wave == 0) {
        unsigned int lo = 0u, hi = ordered_key(lp_max);
        while (lo < hi) {
          const unsigned int mid = lo + ((hi - lo) >> 1);
          const float c = key_to_float(mid);
          float s = 0.f;
          for (int j = lane; j < n_cand; j += 64)
            if (c_lp[j] <= c) s += c_p[j];
          s = m_low + wave_sum(s);
          if (s > need)
            hi = mid;
          else
            lo = mid + 1u;
        }
        if (lane == 0) bcast[0] = key_to_float(lo);
      }
      __syncthreads();
      kept.lo = fmaxf(kept.lo, bcast[0]);
      __syncthreads();
    } else {
      unsigned int lo = 0u, hi = ordered_key(lp_max);  // H(hi) = 1 > need
      while (lo < hi) {
        const unsigned int mid = lo + ((hi - lo) >> 1);
        const float c = key_to_float(mid);
        float s = 0.f;
        for_row(x, V, tid, nt, [&](int, float v) {
          const float lp = v - lse;
          if (lp <= c) s += expf(lp);
        });
        s = block_sum(s, red);
        if (s > need)
          hi = mid;
        else
          lo = mid + 1u;
      }
      kept.lo = fmaxf(kept.lo, key_to_float(lo));
    }
  }

  // k-th largest value among the kept tokens, -inf if fewer than k are kept
  auto kth_largest = [&](int k) -> float {
    if (cand) {  // (no xtc here: kept is lp >= kept.lo)
      if (wave == 0) {
        float n = 0.f;
        for (int j = lane; j < n_cand; j += 64) n += c_lp[j] >= kept.lo ? 1.f : 0.f;
        n = wave_sum(n);
        float found = NAN;  // the list holds fewer than k kept tokens: the row decides
        if (n >= (float)k) {
          unsigned int lo = 0u, hi = ordered_key(lp_max);  // largest c with count(lp >= c) >= k
          while (lo < hi) {
            const unsigned int mid = lo + ((hi - lo + 1u) >> 1);
            const float c = key_to_float(mid);
            float cnt = 0.f;
            for (int j = lane; j < n_cand; j += 64) cnt += (c_lp[j] >= c && c_lp[j] >= kept.lo) ? 1.f : 0.f;
            cnt = wave_sum(cnt);
            if (cnt >= (float)k)
              lo = mid;
            else
              hi = mid - 1u;
          }
          found = key_to_float(lo);
        }
        if (lane == 0) bcast[1] = found;
      }
      __syncthreads();
      const float found = bcast[1];
      __syncthreads();
      if (found == found) return found;
    }
    float cnt_all = 0.f;
    for_row(x, V, tid, nt, [&](int i, float v) { cnt_all += kept(i, v - lse) ? 1.f : 0.f; });
    cnt_all = block_sum(cnt_all, red);
    if (cnt_all < (float)k) return -INFINITY;
    unsigned int lo = 0u, hi = ordered_key(lp_max);  // largest c with count(lp >= c) >= k
    while (lo < hi) {
      const unsigned int mid = lo + ((hi - lo + 1u) >> 1);
      const float c = key_to_float(mid);
      float cnt = 0.f;
      for_row(x, V, tid, nt, [&](int i, float v) {
        const float lp = v - lse;
        cnt += (lp >= c && kept(i, lp)) ? 1.f : 0.f;
      });
      cnt = block_sum(cnt, red);
      if (cnt >= (float)k)
        lo = mid;
      else
        hi = mid - 1u;
    }
    return key_to_float(lo);
  };

  // min_p: drop lp < max + log(min_p), but never one of the min_keep best
  if (min_p != 0.f) {
    float floor_lp = lp_max + logf(min_p);
    const int mk = min_keep;
    if (mk > 1) floor_lp = fminf(floor_lp, kth_largest(mk));
    kept.lo = fmaxf(kept.lo, floor_lp);
  }

  // xtc: with probability xtc_prob drop every token whose (renormalised)
  // probability is above the threshold, except the least likely of them and
  // the special tokens
  if (xtc_prob > 0.f) {
    const float u = uniform01(draw_key(a.seed[r], (unsigned int)a.counter[r]), 0xfffffffeu);
    if (!(u > xtc_prob)) {
      float z = 0.f;
      for (int i = tid; i < V; i += nt) {
        const float lp = x[i] - lse;
        if (kept(i, lp)) z += expf(lp);
      }
      z = block_sum(z, red);
      const float thr = a.xtc_thr[r];
      float least = INFINITY;
      for (int i = tid; i < V; i += nt) {
        const float lp = x[i] - lse;
        if (kept(i, lp) && expf(lp) / z > thr) least = fminf(least, lp);
      }
      least = -block_max(-least, red);
      kept.hi = least;
      kept.n_special = a.n_special;
    }
  }

  if (top_k > 0) kept.lo = fmaxf(kept.lo, kth_largest(top_k));

  // Gumbel-max draw from softmax(lp / temp) over the kept tokens
  const float inv_temp = 1.f / temp;
  const unsigned long long key = draw_key(a.seed[r], (unsigned int)a.counter[r]);
  bv = -INFINITY, bi = 0x7fffffff;
  auto consider = [&](int i, float lp) {
    // Gumbel noise -log(-log u) through the hardware's log2 (u has 24 bits; v_log_f32 is good to
    // an ulp of its result)
    const float u = uniform01(key, (unsigned int)i);
    const float g = -0.69314718f * __log2f(-0.69314718f * __log2f(u));
    const float v = lp * inv_temp + g;
    if (v > bv || (v == bv && i < bi)) bv = v, bi = i;
  };
  if (cand && (n_cand == V || kept.lo > noncand_max)) {
    // every kept token is in the list (xtc is off: kept is lp >= kept.lo)
    for (int j = tid; j < n_cand; j += nt)
      if (c_lp[j] >= kept.lo) consider(c_idx[j], c_lp[j]);
  } else {
    for_row(x, V, tid, nt, [&](int i, float xi) {
      const float lp = xi - lse;
      if (kept(i, lp)) consider(i, lp);
    });
  }
  block_argmax(bv, bi, red, redi);
  if (tid == 0) {
    a.tokens[r] = bi;
    a.token_logprob[r] = x[bi] - lse;
  }
}

// ---------------------------------------------------------------------------

// logits[row, idx[j]] += val[j] for j in [offsets[row], offsets[row+1])
__global__ __launch_bounds__(256) void logit_bias_kernel(float* logits, int ld,
                                                         const int* offsets, const int* idx,
                                                         const float* val) {
  const int r = blockIdx.x;
  float* x = logits + (size_t)r * ld;
  // duplicates in one row are applied one after the other by one thread
  for (int j = offsets[r] + threadIdx.x; j < offsets[r + 1]; j += blockDim.x) {
    bool first = true;
    for (int k = offsets[r]; k < j; ++k)
      if (idx[k] == idx[j]) first = false;
    if (!first) continue;
    float v = x[idx[j]];
    for (int k = j; k < offsets[r + 1]; ++k)
      if (idx[k] == idx[j]) v += val[k];
    x[idx[j]] = v;
  }
}

// Repetition, presence and frequency penalties over the tail of each row's
// token history; hist[offsets[row] .. offsets[row+1]) is that history, oldest
// first, and each penalty looks at its own last `*_ctx` tokens of it.
__global__ __launch_bounds__(256) void penalties_kernel(float* logits, int ld, const int* offsets,
                                                        const int* hist, const float* rep,
                                                        const int* rep_ctx, const float* pres,
                                                        const int* pres_ctx, const float* freq,
                                                        const int* freq_ctx, int vocab) {
  const int r = blockIdx.x;
  float* x = logits + (size_t)r * ld;
  const int b = offsets[r], e = offsets[r + 1];
  const int rep_b = max(b, e - rep_ctx[r]);
  const int pres_b = max(b, e - pres_ctx[r]);
  const int freq_b = max(b, e - freq_ctx[r]);
  for (int j = b + threadIdx.x; j < e; j += blockDim.x) {
    const int t = hist[j];
    if (t < 0 || t >= vocab) continue;  // (the host refuses such a history; this keeps the write inside the row)
    bool first = true;
    for (int k = b; k < j; ++k)
      if (hist[k] == t) first = false;
    if (!first) continue;
    bool in_rep = false, in_pres = false;
    int n_freq = 0;
    for (int k = j; k < e; ++k) {
      if (hist[k] != t) continue;
      if (k >= rep_b) in_rep = true;
      if (k >= pres_b) in_pres = true;
      if (k >= freq_b) ++n_freq;
    }
    float v = x[t];
    const float rp = rep[r];
    if (in_rep && rp != 0.f && rp != 1.f) v = v < 0.f ? v * rp : v / rp;
    if (in_pres) v -= pres[r];
    v -= freq[r] * (float)n_freq;
    x[t] = v;
  }
}

DEFINE_LAST_ERROR(mlxlm_last_error)

extern "C" int sample_rows(int* tokens, float* token_logprob, float* logprobs, int ld_logprobs,
                           const float* logits, int ld, int n_rows, int vocab, const float* temp,
                           const float* top_p, const float* min_p, const int* min_keep,
                           const int* top_k, const float* xtc_prob, const float* xtc_thr,
                           const unsigned long long* seed, const int* counter,
                           const int* xtc_special, int n_special, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (vocab <= 0 || ld < vocab) FAIL("sample_rows: bad vocab %d / row stride %d", vocab, ld);
  if (!tokens || !token_logprob || !logits || !temp || !top_p || !min_p || !min_keep || !top_k ||
      !xtc_prob || !xtc_thr || !seed || !counter)
    FAIL("sample_rows: null pointer");
  if (logprobs && ld_logprobs < vocab) FAIL("sample_rows: logprobs row stride %d too small", ld_logprobs);
  if (n_special > 0 && !xtc_special) FAIL("sample_rows: special tokens missing");
  SampleArgs a;
  a.tokens = tokens, a.token_logprob = token_logprob, a.logprobs = logprobs, a.logits = logits;
  a.temp = temp, a.top_p = top_p, a.min_p = min_p, a.min_keep = min_keep, a.top_k = top_k;
  a.xtc_prob = xtc_prob, a.xtc_thr = xtc_thr, a.seed = seed, a.counter = counter;
  a.xtc_special = xtc_special, a.n_special = n_special;
  a.vocab = vocab, a.ld = ld, a.ld_logprobs = ld_logprobs;
  hipLaunchKernelGGL(sample_rows_kernel, dim3(n_rows), dim3(SAMPLE_THREADS), 0, stream, a);
  CHECK_LAUNCH("sample_rows");
  return 0;
}

extern "C" int apply_logit_bias(float* logits, int ld, int n_rows, const int* offsets,
                                const int* idx, const float* val, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (!logits || !offsets || !idx || !val) FAIL("apply_logit_bias: null pointer");
  hipLaunchKernelGGL(logit_bias_kernel, dim3(n_rows), dim3(256), 0, stream, logits, ld, offsets, idx,
                     val);
  CHECK_LAUNCH("apply_logit_bias");
  return 0;
}

extern "C" int apply_penalties(float* logits, int ld, int n_rows, const int* offsets,
                               const int* hist, const float* rep, const int* rep_ctx,
                               const float* pres, const int* pres_ctx, const float* freq,
                               const int* freq_ctx, int vocab, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (vocab <= 0) FAIL("apply_penalties: vocabulary of %d", vocab);
  if (!logits || !offsets || !hist || !rep || !rep_ctx || !pres || !pres_ctx || !freq || !freq_ctx)
    FAIL("apply_penalties: null pointer");
  hipLaunchKernelGGL(penalties_kernel, dim3(n_rows), dim3(256), 0, stream, logits, ld, offsets, hist,
                     rep, rep_ctx, pres, pres_ctx, freq, freq_ctx, vocab);
  CHECK_LAUNCH("apply_penalties");
  return 0;
}
