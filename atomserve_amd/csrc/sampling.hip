// Choosing the next token from fp32 logits [B, V], one workgroup of 1024 threads per row.
//
//   penalty -> top-k on the raw logits -> / temperature -> softmax -> top-p -> draw
//
// The draw is an exponential race, argmax(p_i / E_i) with E_i ~ Exp(1), which picks
// token i with probability p_i / sum(p) and needs no renormalisation after masking.
// The noise comes from a counter-based generator keyed by (the request's seed, how many
// tokens it has sampled before, the candidate), so a request's stream does not depend
// on which other requests share the batch.
// Plain reference: reference atomserve/sampler.py:82-129, atomserve/kernels.py:362-435.
#include "common.h"

#define SAMPLE_THREADS 1024
#define SAMPLE_KMAX 1024

// (value, index) as one 64-bit key: a larger key is a larger value, or the same value at
// a lower index.  NaN maps to key 0 and is never chosen.
__device__ __forceinline__ unsigned long long make_key(float v, int idx) {
  if (v != v) return 0ull;
  uint32_t u = __float_as_uint(v);
  u = (u & 0x80000000u) ? ~u : (u | 0x80000000u);
  return ((unsigned long long)u << 32) | (uint32_t)(~(uint32_t)idx);
}
__device__ __forceinline__ int key_index(unsigned long long k) { return (int)(~(uint32_t)(k & 0xffffffffull)); }
__device__ __forceinline__ float key_value(unsigned long long k) {
  uint32_t u = (uint32_t)(k >> 32);
  u = (u & 0x80000000u) ? (u & 0x7fffffffu) : ~u;
  return __uint_as_float(u);
}

__device__ __forceinline__ unsigned long long wave_max_u64(unsigned long long v) {
#pragma unroll
  for (int off = WAVE / 2; off > 0; off >>= 1) {
    const unsigned long long o = __shfl_xor(v, off, WAVE);
    v = o > v ? o : v;
  }
  return v;
}

// Maximum over the block; every thread gets it.  `red` is __shared__ u64[17].
__device__ __forceinline__ unsigned long long block_max_u64(unsigned long long v, unsigned long long* red) {
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6, nw = blockDim.x >> 6;
  v = wave_max_u64(v);
  __syncthreads();
  if (lane == 0) red[wid] = v;
  __syncthreads();
  if (threadIdx.x == 0) {
    unsigned long long m = 0ull;
    for (int i = 0; i < nw; ++i) m = red[i] > m ? red[i] : m;
    red[16] = m;
  }
  __syncthreads();
  return red[16];
}

__device__ __forceinline__ float block_max_f32(float v, float* red) {
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6, nw = blockDim.x >> 6;
  v = wave_max(v);
  __syncthreads();
  if (lane == 0) red[wid] = v;
  __syncthreads();
  if (threadIdx.x == 0) {
    float m = red[0];
    for (int i = 1; i < nw; ++i) m = fmaxf(m, red[i]);
    red[16] = m;
  }
  __syncthreads();
  return red[16];
}

// Philox 4x32 with 10 rounds: a counter-based generator.
__device__ __forceinline__ uint32_t philox_first(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3, uint32_t k0,
                                                 uint32_t k1) {
#pragma unroll
  for (int r = 0; r < 10; ++r) {
    const uint32_t hi0 = __umulhi(0xD2511F53u, c0), lo0 = 0xD2511F53u * c0;
    const uint32_t hi1 = __umulhi(0xCD9E8D57u, c2), lo1 = 0xCD9E8D57u * c2;
    const uint32_t n0 = hi1 ^ c1 ^ k0, n1 = lo1, n2 = hi0 ^ c3 ^ k1, n3 = lo0;
    c0 = n0; c1 = n1; c2 = n2; c3 = n3;
    k0 += 0x9E3779B9u; k1 += 0xBB67AE85u;
  }
  return c0;
}

// E ~ Exp(1) for (seed, counter, candidate), never below 1e-10 (reference atomserve/sampler.py:128).
__device__ __forceinline__ float exp1_noise(long long seed, int counter, int candidate) {
  const uint32_t r = philox_first((uint32_t)candidate, (uint32_t)counter, 0x5A3Cu, 0u, (uint32_t)seed,
                                  (uint32_t)((unsigned long long)seed >> 32));
  const float u = ((float)(r >> 8) + 0.5f) * (1.0f / 16777216.0f);  // (0, 1)
  return fmaxf(-logf(u), 1e-10f);
}

// ---- greedy -----------------------------------------------------------------------
__global__ __launch_bounds__(SAMPLE_THREADS) void argmax_kernel(const float* __restrict__ logits,
                                                                int* __restrict__ out, int V) {
  __shared__ unsigned long long red[17];
  const float* x = logits + (size_t)blockIdx.x * V;
  unsigned long long best = 0ull;
  for (int i = threadIdx.x; i < V; i += blockDim.x) {
    const unsigned long long k = make_key(x[i], i);
    best = k > best ? k : best;
  }
  best = block_max_u64(best, red);
  if (threadIdx.x == 0) out[blockIdx.x] = best ? key_index(best) : 0;
}

extern "C" int as_argmax(const float* logits, int* out, int B, int V, hipStream_t stream) {
  if (B <= 0) return AS_OK;
  if (V <= 0) return AS_BAD_SHAPE;
  argmax_kernel<<<B, SAMPLE_THREADS, 0, stream>>>(logits, out, V);
  return launch_status();
}

// ---- penalties ----------------------------------------------------------------------
// logits[rows[i], cols[i]] -= amounts[i]; the (row, col) pairs are distinct.
__global__ void penalty_kernel(float* __restrict__ logits, const int* __restrict__ rows,
                               const int* __restrict__ cols, const float* __restrict__ amounts, int n, int V) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) logits[(size_t)rows[i] * V + cols[i]] -= amounts[i];
}

extern "C" int as_apply_penalty(float* logits, const int* rows, const int* cols, const float* amounts, int n,
                                int V, hipStream_t stream) {
  if (n <= 0) return AS_OK;
  penalty_kernel<<<(n + 255) / 256, 256, 0, stream>>>(logits, rows, cols, amounts, n, V);
  return launch_status();
}

// ---- the full pipeline ------------------------------------------------------------
__global__ __launch_bounds__(SAMPLE_THREADS) void sample_kernel(
    const float* __restrict__ logits, int V, const float* __restrict__ temperature, const int* __restrict__ top_k,
    const float* __restrict__ top_p, const long long* __restrict__ seeds, const int* __restrict__ counters,
    int* __restrict__ out) {
  __shared__ unsigned long long red[17];
  __shared__ float fred[17];
  __shared__ unsigned long long sel[SAMPLE_KMAX];
  __shared__ float ework[SAMPLE_KMAX];
  const int row = blockIdx.x, tid = threadIdx.x;
  const float* x = logits + (size_t)row * V;
  float T = temperature[row];
  int k = top_k[row];
  const float p_keep = top_p[row];
  const long long seed = seeds[row];
  const int counter = counters[row];
  if (T <= 0.f || p_keep <= 0.f) { k = 1; T = 1.f; }  // greedy: the best token alone
  const bool all = (k <= 0 || k >= V);

  if (!all) {
    // The k largest in order, by repeated block-wide maximum; after each pick only the
    // thread that owned it looks for its next candidate.
    if (k > SAMPLE_KMAX) k = SAMPLE_KMAX;  // refused on the host; never index outside
    unsigned long long cand = 0ull;
    for (int i = tid; i < V; i += SAMPLE_THREADS) {
      const unsigned long long key = make_key(x[i], i);
      cand = key > cand ? key : cand;
    }
    int found = 0;
    for (int r = 0; r < k; ++r) {
      const unsigned long long best = block_max_u64(cand, red);
      if (best == 0ull) break;  // fewer than k usable entries
      if (tid == 0) sel[r] = best;
      found = r + 1;
      if (key_index(best) % SAMPLE_THREADS == tid) {
        unsigned long long next = 0ull;
        for (int i = tid; i < V; i += SAMPLE_THREADS) {
          const unsigned long long key = make_key(x[i], i);
          if (key < best && key > next) next = key;
        }
        cand = next;
      }
    }
    __syncthreads();
    if (tid == 0) {
      int choice = 0;
      if (found > 1) {
        const float v0 = key_value(sel[0]);
        float sum = 0.f;
        for (int i = 0; i < found; ++i) {
          const float e = expf((key_value(sel[i]) - v0) / T);
          ework[i] = e;
          sum += e;
        }
        float mass = 0.f, best_score = -1.f;
        for (int i = 0; i < found; ++i) {
          const float p = ework[i] / sum;
          if (mass >= p_keep) break;  // the mass ranked above already reaches top_p
          mass += p;
          const float score = p / exp1_noise(seed, counter, i);
          if (score > best_score) { best_score = score; choice = i; }
        }
      }
      out[row] = found ? key_index(sel[choice]) : 0;
    }
    return;
  }

  // Every token is a candidate.  With p_i = softmax(x / T)_i, argmax p_i / E_i equals
  // argmax x_i / T - log E_i, so no normalisation is needed for the draw itself.
  float keep_from = -1.f;  // tokens with p_i >= keep_from stay
  float mx = -__builtin_inff();
  for (int i = tid; i < V; i += SAMPLE_THREADS) { const float v = x[i]; if (v == v) mx = fmaxf(mx, v); }
  mx = block_max_f32(mx, fred);
  float z = 0.f;
  if (p_keep < 1.f) {
    for (int i = tid; i < V; i += SAMPLE_THREADS) { const float v = x[i]; if (v == v) z += expf((v - mx) / T); }
    z = block_sum(z, fred);
    // Bisection for the smallest probability that is still kept: a token stays iff the mass
    // of the tokens above it is below top_p.  f(t) = mass of tokens with p > t falls with t;
    // f(lo) >= top_p and f(hi) < top_p throughout.  Tokens of equal probability stay or go together.
    float lo = -1.f, hi = 1.f;  // p_max <= 1, and f(1) = 0 < top_p
    for (int it = 0; it < 48; ++it) {
      const float mid = 0.5f * (lo + hi);
      if (mid <= lo || mid >= hi) break;
      float mass = 0.f;
      for (int i = tid; i < V; i += SAMPLE_THREADS) {
        const float v = x[i];
        if (v == v) { const float p = expf((v - mx) / T) / z; if (p > mid) mass += p; }
      }
      mass = block_sum(mass, fred);
      if (mass >= p_keep) lo = mid; else hi = mid;
    }
    keep_from = hi;
  }
  unsigned long long best = 0ull;
  for (int i = tid; i < V; i += SAMPLE_THREADS) {
    const float v = x[i];
    if (v != v) continue;
    if (keep_from > 0.f && expf((v - mx) / T) / z < keep_from && v < mx) continue;  // the best always stays
    const unsigned long long key = make_key(v / T - logf(exp1_noise(seed, counter, i)), i);
    best = key > best ? key : best;
  }
  best = block_max_u64(best, red);
  if (tid == 0) out[row] = best ? key_index(best) : 0;
}

extern "C" int as_sample(const float* logits, int B, int V, const float* temperature, const int* top_k,
                         const float* top_p, const long long* seeds, const int* counters, int* out,
                         hipStream_t stream) {
  if (B <= 0) return AS_OK;
  if (V <= 0) return AS_BAD_SHAPE;
  sample_kernel<<<B, SAMPLE_THREADS, 0, stream>>>(logits, V, temperature, top_k, top_p, seeds, counters, out);
  return launch_status();
}

// Sorted top-k of each row (values and indices), k <= SAMPLE_KMAX; exposed for tests and tools.
__global__ __launch_bounds__(SAMPLE_THREADS) void topk_kernel(const float* __restrict__ logits, int V, int k,
                                                              float* __restrict__ values, int* __restrict__ indices) {
  __shared__ unsigned long long red[17];
  const int row = blockIdx.x, tid = threadIdx.x;
  const float* x = logits + (size_t)row * V;
  unsigned long long cand = 0ull;
  for (int i = tid; i < V; i += SAMPLE_THREADS) {
    const unsigned long long key = make_key(x[i], i);
    cand = key > cand ? key : cand;
  }
  for (int r = 0; r < k; ++r) {
    const unsigned long long best = block_max_u64(cand, red);
    if (tid == 0) {
      values[(size_t)row * k + r] = best ? key_value(best) : -__builtin_inff();
      indices[(size_t)row * k + r] = best ? key_index(best) : -1;
    }
    if (best != 0ull && key_index(best) % SAMPLE_THREADS == tid) {
      unsigned long long next = 0ull;
      for (int i = tid; i < V; i += SAMPLE_THREADS) {
        const unsigned long long key = make_key(x[i], i);
        if (key < best && key > next) next = key;
      }
      cand = next;
    }
  }
}

extern "C" int as_topk(const float* logits, int B, int V, int k, float* values, int* indices, hipStream_t stream) {
  if (B <= 0) return AS_OK;
  if (V <= 0 || k <= 0 || k > SAMPLE_KMAX || k > V) return AS_BAD_SHAPE;
  topk_kernel<<<B, SAMPLE_THREADS, 0, stream>>>(logits, V, k, values, indices);
  return launch_status();
}
