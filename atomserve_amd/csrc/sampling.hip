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

// The largest key among a thread's elements i = tid, tid + T, ...; four independent chains
// keep several loads in flight.
__device__ __forceinline__ unsigned long long thread_max_key(const float* __restrict__ x, int V) {
  unsigned long long b0 = 0ull, b1 = 0ull, b2 = 0ull, b3 = 0ull;
  const int T = blockDim.x;
  int i = threadIdx.x;
  for (; i + 3 * T < V; i += 4 * T) {
    const float v0 = x[i], v1 = x[i + T], v2 = x[i + 2 * T], v3 = x[i + 3 * T];
    const unsigned long long k0 = make_key(v0, i), k1 = make_key(v1, i + T), k2 = make_key(v2, i + 2 * T),
                             k3 = make_key(v3, i + 3 * T);
    b0 = k0 > b0 ? k0 : b0; b1 = k1 > b1 ? k1 : b1; b2 = k2 > b2 ? k2 : b2; b3 = k3 > b3 ? k3 : b3;
  }
  for (; i < V; i += T) { const unsigned long long k = make_key(x[i], i); b0 = k > b0 ? k : b0; }
  b0 = b1 > b0 ? b1 : b0;
  b2 = b3 > b2 ? b3 : b2;
  return b2 > b0 ? b2 : b0;
}

// The k largest keys of a row in order, into sel[0..k-1]; returns how many were found (fewer
// than k only if the row has fewer usable entries).  Block-wide; k <= SAMPLE_KMAX.
//
// 1. every thread finds the maximum of its own elements;
// 2. t = the k-th largest of those 1024 maxima, by radix selection on the value bits: at
//    least k elements are >= t, and usually few more;
// 3. a second pass collects every element >= t into LDS;
// 4. each candidate's rank is the number of candidates with a larger key.
// If more candidates turn up than LDS holds (long runs of equal values), the slower
// selection by repeated block-wide maximum takes over.
#define SAMPLE_CAND 2048
struct TopKShared {
  unsigned long long red[17];
  unsigned long long cand[SAMPLE_CAND];
  unsigned int hist[256];
  int wave_total[4];
  unsigned int count;
  unsigned int prefix;
  unsigned int remaining;
};

__device__ int block_topk(const float* __restrict__ x, int V, int k, unsigned long long* sel, TopKShared& sh) {
  const int tid = threadIdx.x;
  const unsigned long long mine = thread_max_key(x, V);
  // radix selection of the k-th largest value (upper 32 bits of the key) among the thread maxima
  const unsigned int myval = (unsigned int)(mine >> 32);
  unsigned int prefix = 0, mask = 0;
  int want = k;  // the want-th largest among the values matching the prefix
  const int have = __syncthreads_count(mine != 0ull);
  if (have < k) want = have;  // fewer than k usable maxima: take them all (t becomes the smallest)
  if (want > 0) {
    for (int shift = 24; shift >= 0; shift -= 8) {
      if (tid < 256) sh.hist[tid] = 0;
      __syncthreads();
      if (mine != 0ull && (myval & mask) == prefix) atomicAdd(&sh.hist[(myval >> shift) & 255], 1u);
      __syncthreads();
      // The digit of the want-th largest: the bin b with (values in bins > b) < want <= (values
      // in bins >= b).  Thread b holds bin b; the counts from a bin upwards come from a scan
      // over the four waves that hold the 256 bins (a walk by one thread costs an LDS round
      // trip per bin).
      int above_incl = 0, own = 0;
      if (tid < 256) {
        own = (int)sh.hist[tid];
        above_incl = own;
        const int lane = tid & 63;
#pragma unroll
        for (int off = 1; off < WAVE; off <<= 1) {
          const int o = __shfl_down(above_incl, off, WAVE);
          if (lane + off < WAVE) above_incl += o;
        }
        if (lane == 0) sh.wave_total[tid >> 6] = above_incl;
      }
      __syncthreads();
      if (tid < 256) {
        for (int w = (tid >> 6) + 1; w < 4; ++w) above_incl += sh.wave_total[w];
        const int above = above_incl - own;  // values in higher bins
        if (above < want && above_incl >= want) {  // exactly one bin
          sh.prefix = prefix | ((unsigned int)tid << shift);
          sh.remaining = want - above;
        }
      }
      __syncthreads();
      prefix = sh.prefix;
      want = sh.remaining;
      mask |= 255u << shift;
    }
  }
  const unsigned int threshold = prefix;
  if (tid == 0) sh.count = 0;
  __syncthreads();
  if (have > 0) {
    const int T = blockDim.x;
    for (int i0 = tid; i0 < V; i0 += 4 * T) {
      float v[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) v[u] = (i0 + u * T < V) ? x[i0 + u * T] : __builtin_nanf("");
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const unsigned long long key = make_key(v[u], i0 + u * T);
        if (key != 0ull && (unsigned int)(key >> 32) >= threshold) {
          const unsigned int at = atomicAdd(&sh.count, 1u);
          if (at < SAMPLE_CAND) sh.cand[at] = key;
        }
      }
    }
  }
  __syncthreads();
  const int count = sh.count;
  if (count <= SAMPLE_CAND) {
    for (int c = tid; c < count; c += blockDim.x) {
      const unsigned long long key = sh.cand[c];
      int rank = 0;
      for (int j = 0; j < count; ++j) rank += sh.cand[j] > key;
      if (rank < k) sel[rank] = key;
    }
    __syncthreads();
    return count < k ? count : k;
  }
  // fallback: repeated block-wide maximum; after each pick only its owner looks for its next
  unsigned long long cand = mine;
  int found = 0;
  for (int r = 0; r < k; ++r) {
    const unsigned long long best = block_max_u64(cand, sh.red);
    if (best == 0ull) break;
    if (tid == 0) sel[r] = best;
    found = r + 1;
    if (key_index(best) % (int)blockDim.x == tid) {
      unsigned long long next = 0ull;
      for (int i = tid; i < V; i += blockDim.x) {
        const unsigned long long key = make_key(x[i], i);
        if (key < best && key > next) next = key;
      }
      cand = next;
    }
  }
  __syncthreads();
  return found;
}

// The order-preserving bits of the k-th largest value of a row (1 <= k <= number of usable
// entries, else of the smallest usable one), by radix selection over ALL entries: four passes,
// eight bits each.  For a k beyond what block_topk holds; the caller keeps every entry whose bits
// are at least the result, so entries equal to the k-th stay together.  0 if nothing is usable.
__device__ unsigned int block_kth_value_bits(const float* __restrict__ x, int V, int k, TopKShared& sh) {
  const int tid = threadIdx.x, T = blockDim.x;
  int usable = 0;
  for (int i = tid; i < V; i += T) usable += x[i] == x[i];
  __syncthreads();
  if (tid == 0) sh.count = 0;
  __syncthreads();
  if (usable) atomicAdd(&sh.count, (unsigned int)usable);
  __syncthreads();
  const int have = (int)sh.count;
  if (have == 0) return 0u;
  unsigned int prefix = 0, mask = 0;
  int want = k < have ? k : have;
  for (int shift = 24; shift >= 0; shift -= 8) {
    if (tid < 256) sh.hist[tid] = 0;
    __syncthreads();
    for (int i = tid; i < V; i += T) {
      const unsigned long long key = make_key(x[i], i);
      const unsigned int bits = (unsigned int)(key >> 32);
      if (key != 0ull && (bits & mask) == prefix) atomicAdd(&sh.hist[(bits >> shift) & 255], 1u);
    }
    __syncthreads();
    // the bin with (entries in higher bins) < want <= (entries in this bin and higher): as in block_topk
    int above_incl = 0, own = 0;
    if (tid < 256) {
      own = (int)sh.hist[tid];
      above_incl = own;
      const int lane = tid & 63;
#pragma unroll
      for (int off = 1; off < WAVE; off <<= 1) {
        const int o = __shfl_down(above_incl, off, WAVE);
        if (lane + off < WAVE) above_incl += o;
      }
      if (lane == 0) sh.wave_total[tid >> 6] = above_incl;
    }
    __syncthreads();
    if (tid < 256) {
      for (int w = (tid >> 6) + 1; w < 4; ++w) above_incl += sh.wave_total[w];
      const int above = above_incl - own;
      if (above < want && above_incl >= want) {
        sh.prefix = prefix | ((unsigned int)tid << shift);
        sh.remaining = want - above;
      }
    }
    __syncthreads();
    prefix = sh.prefix;
    want = sh.remaining;
    mask |= 255u << shift;
  }
  return prefix;
}

// ---- greedy -----------------------------------------------------------------------
__global__ __launch_bounds__(SAMPLE_THREADS) void argmax_kernel(const float* __restrict__ logits,
                                                                int* __restrict__ out, int V) {
  __shared__ unsigned long long red[17];
  const float* x = logits + (size_t)blockIdx.x * V;
  const unsigned long long best = block_max_u64(thread_max_key(x, V), red);
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
// The draw among a row's candidates, ranked best first in sel[0..found-1] (found <= blockDim.x): softmax at
// temperature T over them, the best ones kept while the mass ranked above is below p_keep, and the
// exponential race among those.  Block-wide, every thread calls it; thread 0 returns the choice's place in
// `sel` (0 for fewer than two candidates), the others nothing of use.  The exponentials, the noise and the
// quotients are one candidate per thread; the two sums run over them in order in one thread, so the
// result is that of the plain loop over the candidates, whatever the block's size.
// work: __shared__ float[3 * (most candidates) + 1].
__device__ __forceinline__ int draw_among_ranked(const unsigned long long* sel, int found, float T, float p_keep,
                                                 long long seed, int counter, float* work) {
  if (found <= 1) return 0;  // uniform over the block
  const int tid = threadIdx.x;
  float* e = work;
  float* noise = work + found;
  float* score = work + 2 * found;
  float* total = work + 3 * found;
  const float v0 = key_value(sel[0]);
  if (tid < found) {
    e[tid] = expf((key_value(sel[tid]) - v0) / T);
    noise[tid] = exp1_noise(seed, counter, tid);
  }
  __syncthreads();
  if (tid == 0) {
    float sum = 0.f;
    for (int i = 0; i < found; ++i) sum += e[i];
    *total = sum;
  }
  __syncthreads();
  if (tid < found) {
    const float p = e[tid] / *total;
    e[tid] = p;
    score[tid] = p / noise[tid];
  }
  __syncthreads();
  int choice = 0;
  if (tid == 0) {
    float mass = 0.f, best_score = -1.f;
    for (int i = 0; i < found; ++i) {
      if (mass >= p_keep) break;  // the mass ranked above already reaches top_p
      mass += e[i];
      if (score[i] > best_score) { best_score = score[i]; choice = i; }
    }
  }
  return choice;
}

__global__ __launch_bounds__(SAMPLE_THREADS) void sample_kernel(
    const float* __restrict__ logits, int V, const float* __restrict__ temperature, const int* __restrict__ top_k,
    const float* __restrict__ top_p, const long long* __restrict__ seeds, const int* __restrict__ counters,
    int* __restrict__ out) {
  __shared__ TopKShared topk_shared;
  unsigned long long* red = topk_shared.red;
  __shared__ float fred[17];
  __shared__ unsigned long long sel[SAMPLE_KMAX];
  __shared__ float ework[3 * SAMPLE_KMAX + 1];
  const int row = blockIdx.x, tid = threadIdx.x;
  const float* x = logits + (size_t)row * V;
  float T = temperature[row];
  int k = top_k[row];
  const float p_keep = top_p[row];
  const long long seed = seeds[row];
  const int counter = counters[row];
  if (T <= 0.f || p_keep <= 0.f) { k = 1; T = 1.f; }  // greedy: the best token alone
  const bool all = (k <= 0 || k >= V);
  const bool wide = !all && k > SAMPLE_KMAX;  // more candidates than LDS ranks: a floor on the value instead

  if (!all && !wide) {
    const int found = block_topk(x, V, k, sel, topk_shared);
    __syncthreads();
    const int choice = draw_among_ranked(sel, found, T, p_keep, seed, counter, ework);
    if (tid == 0) out[row] = found ? key_index(sel[choice]) : 0;
    return;
  }

  // Every token is a candidate (or, with a top-k beyond SAMPLE_KMAX, every token whose logit is at
  // least the k-th largest: equal ones stay together).  With p_i = softmax(x / T)_i, argmax p_i / E_i
  // equals argmax x_i / T - log E_i, so no normalisation is needed for the draw itself.
  const unsigned int floor_bits = wide ? block_kth_value_bits(x, V, k, topk_shared) : 0u;
  auto usable = [&](float v, int i) { return v == v && (!wide || (unsigned int)(make_key(v, i) >> 32) >= floor_bits); };
  float keep_from = -1.f;  // tokens with p_i >= keep_from stay
  float mx = -__builtin_inff();
  for (int i = tid; i < V; i += SAMPLE_THREADS) { const float v = x[i]; if (v == v) mx = fmaxf(mx, v); }
  mx = block_max_f32(mx, fred);
  float z = 0.f;
  if (p_keep < 1.f) {
    for (int i = tid; i < V; i += SAMPLE_THREADS) { const float v = x[i]; if (usable(v, i)) z += expf((v - mx) / T); }
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
        if (usable(v, i)) { const float p = expf((v - mx) / T) / z; if (p > mid) mass += p; }
      }
      mass = block_sum(mass, fred);
      if (mass >= p_keep) lo = mid; else hi = mid;
    }
    keep_from = hi;
  }
  unsigned long long best = 0ull;
  for (int i = tid; i < V; i += SAMPLE_THREADS) {
    const float v = x[i];
    if (!usable(v, i)) continue;
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

// ---- the same draw for small top-k, spread over the GPU ---------------------------------
// One workgroup per row reads a vocabulary of 150 thousand logits alone, which takes longer
// than everything else a decode step does after its last matrix product.  When every row
// keeps at most SPLIT_KMAX candidates, the row is cut into SPLIT_SLICES slices instead:
// a first kernel finds each slice's k best (keys carry the index within the whole row), a
// second one ranks the slices' candidates, of which the row's k best are a subset, and
// draws exactly as sample_kernel does: same candidates, same order, same noise.
#define SPLIT_SLICES 32
#define SPLIT_KMAX 64
#define SPLIT_THREADS 256

__device__ __forceinline__ int effective_top_k(float T, int k, float p_keep) {
  return (T <= 0.f || p_keep <= 0.f) ? 1 : k;  // greedy: the best token alone
}

__global__ __launch_bounds__(SPLIT_THREADS) void topk_slices_kernel(
    const float* __restrict__ logits, int V, const float* __restrict__ temperature, const int* __restrict__ top_k,
    const float* __restrict__ top_p, unsigned long long* __restrict__ cand, int* __restrict__ counts) {
  __shared__ TopKShared topk_shared;
  __shared__ unsigned long long sel[SPLIT_KMAX];
  const int row = blockIdx.x, slice = blockIdx.y;
  int k = effective_top_k(temperature[row], top_k[row], top_p[row]);
  k = k < 1 ? 1 : (k > SPLIT_KMAX ? SPLIT_KMAX : k);  // refused on the host; never index outside
  const int len = (V + SPLIT_SLICES - 1) / SPLIT_SLICES, off = slice * len;
  const int n = min(len, V - off);
  int found = 0;
  if (n > 0) found = block_topk(logits + (size_t)row * V + off, n, min(k, n), sel, topk_shared);
  unsigned long long* dst = cand + ((size_t)row * SPLIT_SLICES + slice) * SPLIT_KMAX;
  for (int r = threadIdx.x; r < found; r += SPLIT_THREADS) dst[r] = make_key(key_value(sel[r]), key_index(sel[r]) + off);
  if (threadIdx.x == 0) counts[row * SPLIT_SLICES + slice] = found;
}

__global__ __launch_bounds__(SAMPLE_THREADS) void sample_candidates_kernel(
    const unsigned long long* __restrict__ cand, const int* __restrict__ counts,
    const float* __restrict__ temperature, const int* __restrict__ top_k, const float* __restrict__ top_p,
    const long long* __restrict__ seeds, const int* __restrict__ counters, int* __restrict__ out) {
  __shared__ unsigned long long pool[SPLIT_SLICES * SPLIT_KMAX];
  __shared__ int first[SPLIT_SLICES + 1];
  __shared__ unsigned long long sel[SPLIT_KMAX];
  __shared__ float ework[3 * SPLIT_KMAX + 1];
  const int row = blockIdx.x, tid = threadIdx.x;
  float T = temperature[row];
  const float p_keep = top_p[row];
  int k = effective_top_k(T, top_k[row], p_keep);
  if (T <= 0.f || p_keep <= 0.f) T = 1.f;
  k = k < 1 ? 1 : (k > SPLIT_KMAX ? SPLIT_KMAX : k);
  __shared__ int found_in[SPLIT_SLICES];
  if (tid < SPLIT_SLICES) found_in[tid] = counts[row * SPLIT_SLICES + tid];  // all loads at once
  __syncthreads();
  if (tid == 0) {
    int at = 0;
    for (int sl = 0; sl < SPLIT_SLICES; ++sl) { first[sl] = at; at += found_in[sl]; }
    first[SPLIT_SLICES] = at;
  }
  __syncthreads();
  const int total = first[SPLIT_SLICES];
  for (int sl = tid / SPLIT_KMAX; sl < SPLIT_SLICES; sl += SAMPLE_THREADS / SPLIT_KMAX) {
    const int r = tid % SPLIT_KMAX, n = first[sl + 1] - first[sl];
    if (r < n) pool[first[sl] + r] = cand[((size_t)row * SPLIT_SLICES + sl) * SPLIT_KMAX + r];
  }
  __syncthreads();
  for (int c = tid; c < total; c += SAMPLE_THREADS) {
    const unsigned long long key = pool[c];
    int rank = 0;
    for (int j = 0; j < total; ++j) rank += pool[j] > key;
    if (rank < k) sel[rank] = key;
  }
  __syncthreads();
  const int found = total < k ? total : k;
  const int choice = draw_among_ranked(sel, found, T, p_keep, seeds[row], counters[row], ework);
  if (tid == 0) out[row] = found ? key_index(sel[choice]) : 0;
}

// As as_sample, for batches whose every row keeps between 1 and 64 candidates (greedy rows
// count as 1).  cand: [B, 32, 64] 64-bit scratch, counts: [B, 32] int32 scratch.
extern "C" int as_sample_split(const float* logits, int B, int V, const float* temperature, const int* top_k,
                               const float* top_p, const long long* seeds, const int* counters, void* cand,
                               int* counts, int* out, hipStream_t stream) {
  if (B <= 0) return AS_OK;
  if (V <= 0 || !cand || !counts) return AS_BAD_SHAPE;
  topk_slices_kernel<<<dim3(B, SPLIT_SLICES), SPLIT_THREADS, 0, stream>>>(logits, V, temperature, top_k, top_p,
                                                                         (unsigned long long*)cand, counts);
  if (hipGetLastError() != hipSuccess) return AS_LAUNCH_FAILED;
  sample_candidates_kernel<<<B, SAMPLE_THREADS, 0, stream>>>((const unsigned long long*)cand, counts, temperature,
                                                            top_k, top_p, seeds, counters, out);
  return launch_status();
}

// Sorted top-k of each row (values and indices), k <= SAMPLE_KMAX; exposed for tests and tools.
__global__ __launch_bounds__(SAMPLE_THREADS) void topk_kernel(const float* __restrict__ logits, int V, int k,
                                                              float* __restrict__ values, int* __restrict__ indices) {
  __shared__ TopKShared topk_shared;
  __shared__ unsigned long long sel[SAMPLE_KMAX];
  const int row = blockIdx.x;
  const int found = block_topk(logits + (size_t)row * V, V, k, sel, topk_shared);
  for (int r = threadIdx.x; r < k; r += blockDim.x) {
    values[(size_t)row * k + r] = r < found ? key_value(sel[r]) : -__builtin_inff();
    indices[(size_t)row * k + r] = r < found ? key_index(sel[r]) : -1;
  }
}

extern "C" int as_topk(const float* logits, int B, int V, int k, float* values, int* indices, hipStream_t stream) {
  if (B <= 0) return AS_OK;
  if (V <= 0 || k <= 0 || k > SAMPLE_KMAX || k > V) return AS_BAD_SHAPE;
  topk_kernel<<<B, SAMPLE_THREADS, 0, stream>>>(logits, V, k, values, indices);
  return launch_status();
}
