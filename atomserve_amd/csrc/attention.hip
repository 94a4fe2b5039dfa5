// Attention over the paged cache.
//
// Cache pages of one layer: k_pages [num_pages, KV, block_size, D] and v_pages
// [num_pages, KV, D, block_size] (values transposed within a page); a token at position p
// of a request lives in page table[p / block_size] at offset p % block_size.  A query at position p sees the keys at positions lo..p, with
// lo = max(0, p - window + 1) if window > 0, else 0.  Query head h reads kv head
// h / (H / KV).  Scores, softmax and the weighted sum are fp32.
//
// attn_single_query: one work item per query token.  A workgroup (4 waves) takes one
// token, one kv head, up to GT query heads of its group, and one partition of
// `part_size` keys.  Inside a wave, LPK lanes share a key (each holds 16 bytes of
// the head) and 64 / LPK keys are in flight at once, each such lane group keeping an
// online-softmax stream (m, l, acc) of its own; streams are merged by shuffles, waves
// through LDS, partitions by attn_reduce.  Serves fp32 (every row) and bf16 (decode).
// Plain reference: reference atomserve/kernels.py:167-334, atomserve/model.py:269-289.
#include "common.h"
#include "no_alloc.h"
#include <type_traits>

#define NEG_INF (-__builtin_inff())

// exp of the fp32 path is the precise one; bf16 serving uses the hardware approximation.
template <typename T> __device__ __forceinline__ float fexp(float x);
template <> __device__ __forceinline__ float fexp<float>(float x) { return expf(x); }
template <> __device__ __forceinline__ float fexp<bf16>(float x) { return __expf(x); }

template <typename T> struct Chunk;  // 16 bytes of a head
template <> struct Chunk<float> {
  static constexpr int N = 4;
  static __device__ __forceinline__ void load(const float* p, float* v) {
    const float4 r = *reinterpret_cast<const float4*>(p);
    v[0] = r.x; v[1] = r.y; v[2] = r.z; v[3] = r.w;
  }
};
template <> struct Chunk<bf16> {
  static constexpr int N = 8;
  static __device__ __forceinline__ void load(const bf16* p, float* v) {
    const uint4 r = *reinterpret_cast<const uint4*>(p);
    const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      v[2 * i] = __uint_as_float(w[i] << 16);
      v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
  }
};

template <typename T, int GT>
__global__ __launch_bounds__(256) void attn_single_query_kernel(
    const T* __restrict__ q, const T* __restrict__ k_pages, const T* __restrict__ v_pages,
    const int* __restrict__ items, const int* __restrict__ positions, const int* __restrict__ tok_row,
    const int* __restrict__ block_tables, int table_width, T* __restrict__ out,
    float* __restrict__ part_m, float* __restrict__ part_l, float* __restrict__ part_acc, int H, int KV,
    int D, int bs, float scale, int window, int part_size, int P, int lpk) {
  constexpr int CH = Chunk<T>::N;
  extern __shared__ float smem[];  // [4][GT] m, [4][GT] l, [4][GT][D] acc
  const int G = H / KV;
  const int HC = (G + GT - 1) / GT;
  const int item = blockIdx.x, kvh = blockIdx.y / HC, hc = blockIdx.y % HC, part = blockIdx.z;
  const int t = items ? items[item] : item;  // null: every token, in order
  const int pos = positions[t];
  const int ctx = pos + 1;
  const int lo = window > 0 ? max(0, ctx - window) : 0;
  const int k0 = max(lo, part * part_size), k1 = min(ctx, (part + 1) * part_size);
  const int h0 = kvh * G + hc * GT;       // first query head of this workgroup
  const int ng = min(GT, G - hc * GT);    // valid heads among the GT
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;

  if (k0 >= k1) {  // an empty partition (P > 1 only): mark it so for the reduce
    if (tid < ng) {
      const size_t o = ((size_t)item * H + h0 + tid) * P + part;
      part_m[o] = NEG_INF;
      part_l[o] = 0.f;
    }
    for (int idx = tid; idx < ng * D; idx += 256)
      part_acc[(((size_t)item * H + h0 + idx / D) * P + part) * D + idx % D] = 0.f;
    return;
  }

  const int nsub = 64 / lpk;  // keys in flight per wave
  const int sub = lane / lpk, j = lane % lpk;
  const bool active = j * CH < D;
  const int* table = block_tables + (size_t)(tok_row ? tok_row[t] : t) * table_width;  // null: token t is row t

  float qr[GT][CH];
#pragma unroll
  for (int g = 0; g < GT; ++g) {
    if (active && g < ng) {
      Chunk<T>::load(q + ((size_t)t * H + h0 + g) * D + j * CH, qr[g]);
#pragma unroll
      for (int c = 0; c < CH; ++c) qr[g][c] *= scale;
    } else {
#pragma unroll
      for (int c = 0; c < CH; ++c) qr[g][c] = 0.f;
    }
  }

  float m[GT], l[GT], acc[GT][CH];
#pragma unroll
  for (int g = 0; g < GT; ++g) {
    m[g] = NEG_INF;
    l[g] = 0.f;
#pragma unroll
    for (int c = 0; c < CH; ++c) acc[g][c] = 0.f;
  }

  const int stride = 4 * nsub;
  const int iters = (k1 - k0 + stride - 1) / stride;  // uniform over the workgroup
  for (int it = 0; it < iters; ++it) {
    const int key = k0 + it * stride + wave * nsub + sub;
    const bool valid = key < k1;
    float kv[CH], vv[CH];
    if (valid && active) {
      const int page = table[key / bs];
      const size_t head = ((size_t)page * KV + kvh) * bs * D;
      Chunk<T>::load(k_pages + head + (size_t)(key % bs) * D + j * CH, kv);
      const T* vt = v_pages + head + (size_t)(j * CH) * bs + key % bs;
#pragma unroll
      for (int c = 0; c < CH; ++c) vv[c] = to_f32(vt[(size_t)c * bs]);
    } else {
#pragma unroll
      for (int c = 0; c < CH; ++c) { kv[c] = 0.f; vv[c] = 0.f; }
    }
    float s[GT];
#pragma unroll
    for (int g = 0; g < GT; ++g) {
      float d = 0.f;
#pragma unroll
      for (int c = 0; c < CH; ++c) d += qr[g][c] * kv[c];
      for (int off = 1; off < lpk; off <<= 1) d += __shfl_xor(d, off, WAVE);
      s[g] = d;
    }
    if (valid) {
#pragma unroll
      for (int g = 0; g < GT; ++g) {
        const float mn = fmaxf(m[g], s[g]);
        const float a = fexp<T>(m[g] - mn);  // m = -inf gives 0
        const float p = fexp<T>(s[g] - mn);
        l[g] = l[g] * a + p;
#pragma unroll
        for (int c = 0; c < CH; ++c) acc[g][c] = acc[g][c] * a + p * vv[c];
        m[g] = mn;
      }
    }
  }

  // merge the streams of a wave
  for (int off = lpk; off < 64; off <<= 1) {
#pragma unroll
    for (int g = 0; g < GT; ++g) {
      const float mo = __shfl_xor(m[g], off, WAVE), lo_ = __shfl_xor(l[g], off, WAVE);
      const float mn = fmaxf(m[g], mo);
      const float a = (m[g] == NEG_INF) ? 0.f : fexp<T>(m[g] - mn);
      const float b = (mo == NEG_INF) ? 0.f : fexp<T>(mo - mn);
      l[g] = l[g] * a + lo_ * b;
#pragma unroll
      for (int c = 0; c < CH; ++c) {
        const float ao = __shfl_xor(acc[g][c], off, WAVE);
        acc[g][c] = acc[g][c] * a + ao * b;
      }
      m[g] = mn;
    }
  }

  float* sm = smem;
  float* sl = smem + 4 * GT;
  float* sacc = smem + 8 * GT;
  if (lane < lpk) {
#pragma unroll
    for (int g = 0; g < GT; ++g) {
      if (j == 0) { sm[wave * GT + g] = m[g]; sl[wave * GT + g] = l[g]; }
      if (active) {
#pragma unroll
        for (int c = 0; c < CH; ++c) sacc[((size_t)wave * GT + g) * D + j * CH + c] = acc[g][c];
      }
    }
  }
  __syncthreads();

  for (int idx = tid; idx < ng * D; idx += 256) {
    const int g = idx / D, d = idx % D;
    float mx = NEG_INF;
#pragma unroll
    for (int w = 0; w < 4; ++w) mx = fmaxf(mx, sm[w * GT + g]);
    float num = 0.f, den = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const float mw = sm[w * GT + g];
      const float e = (mw == NEG_INF) ? 0.f : fexp<T>(mw - mx);
      num += sacc[((size_t)w * GT + g) * D + d] * e;
      den += sl[w * GT + g] * e;
    }
    const int h = h0 + g;
    if (P == 1) {
      out[((size_t)t * H + h) * D + d] = from_f32<T>(num / den);
    } else {
      const size_t o = ((size_t)item * H + h) * P + part;
      part_acc[o * D + d] = num;
      if (d == 0) { part_m[o] = mx; part_l[o] = den; }
    }
  }
}

// Merge the partitions of each (item, head): out = sum_p acc_p e^(m_p - M) / sum_p l_p e^(m_p - M).
// One workgroup per (item, head), one thread per output coordinate; every thread derives the
// weights itself (P small values, all loads independent), so there is one round of loads for
// the weights and one for the sums.  Empty partitions carry m = -inf, l = 0 and acc = 0.
#define REDUCE_MAX_P 64
template <typename T>
__global__ __launch_bounds__(256) void attn_reduce_kernel(const int* __restrict__ items,
                                                          const float* __restrict__ part_m,
                                                          const float* __restrict__ part_l,
                                                          const float* __restrict__ part_acc, T* __restrict__ out,
                                                          int H, int D, int P) {
  const int item = blockIdx.x, h = blockIdx.y;
  const size_t base = ((size_t)item * H + h) * P;
  float mx = NEG_INF;
  for (int p = 0; p < P; ++p) mx = fmaxf(mx, part_m[base + p]);
  float den = 0.f;
  for (int p = 0; p < P; ++p) {
    const float mp = part_m[base + p];
    den += (mp == NEG_INF) ? 0.f : part_l[base + p] * fexp<T>(mp - mx);
  }
  const float inv = 1.0f / den;
  const int t = items ? items[item] : item;  // null: every token, in order
  for (int d = threadIdx.x; d < D; d += blockDim.x) {
    float num = 0.f;
#pragma unroll 4
    for (int p = 0; p < P; ++p) {
      const float mp = part_m[base + p];
      const float wgt = (mp == NEG_INF) ? 0.f : fexp<T>(mp - mx);
      num += part_acc[(base + p) * D + d] * wgt;
    }
    out[((size_t)t * H + h) * D + d] = from_f32<T>(num * inv);
  }
}

// ---- bf16 decode through the matrix cores ---------------------------------------------
//
// One workgroup (4 waves) per (query token, kv head, partition).  All G <= 16 query heads
// of the group ride in the 16 columns of one MFMA tile, so every key and value is read
// once for the whole group.  Per step a wave takes 32 keys (two tiles of 16):
//
//   S^T[key][head] = K[key][:] . Q[head][:]     A = keys, straight from the page (16 bytes
//                                               per lane), B = queries, kept in registers
//   online softmax per head on the accumulator layout (lane = head column)
//   O^T[d][head]  += V^T[d][key] P^T[key][head] A = the transposed value page, straight from
//                                               memory, B = P, which the lane already holds
//
// The softmax weights are rounded to bf16 for the second product; maxima, sums and the
// output accumulate in fp32.  Needs D % 32 == 0, D <= 256, block_size % 16 == 0.
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

// Which of a step's 32 keys row `row` of its score tile `tile` (0, 1) stands for.  Rows 4g..4g+3
// of both tiles are what lane group g holds after the score product, and they are keys
// 8g .. 8g+7: eight neighbours, whose values are one 16-byte piece of a transposed page.
#define KEY_OF_ROW(tile, row) (8 * ((row) >> 2) + ((row) & 3) + 4 * (tile))

// Sums and maxima over the four lanes that share `lane % 16` (lane ^ 16, lane ^ 32) without a
// trip through LDS: v_permlane16_swap / v_permlane32_swap exchange rows of 16 lanes between
// two registers.  With both operands equal to x, the results hold (rows 0 0 2 2, rows 1 1 3 3)
// and (rows 0 1 0 1, rows 2 3 2 3) of x.
__device__ __forceinline__ float quad_rows_max(float v) {
  auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  v = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
  auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
__device__ __forceinline__ float quad_rows_sum(float v) {
  auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  v = __uint_as_float(a[0]) + __uint_as_float(a[1]);
  auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

// The keys and values of one step (32 keys, two 16-key pieces of pages) of one kv head, as the
// MFMA operands of this lane: keys as rows of A (16 bytes of the head of key KEY_OF_ROW(tile,
// lane % 16)), values as the transposed page gives them (the lane group's 8 keys of one
// coordinate: 16 bytes).  A piece that starts at or beyond `end` is not read and counts as zeros.
// Loading the next step before computing the current one keeps memory busy while the matrix
// cores work.
template <int DC>
struct KVStep {
  bf16x8_t k[2][DC];
  bf16x8_t v[2 * DC];
};

template <int DC>
__device__ __forceinline__ void load_kv_step(KVStep<DC>& st, const bf16* __restrict__ k_pages,
                                             const bf16* __restrict__ v_pages, const int* __restrict__ table,
                                             int kb, int end, int KV, int kvh, int bs, int col, int grp) {
  constexpr int D = DC * 32, DT = DC * 2;
  const bf16x8_t zero = {0, 0, 0, 0, 0, 0, 0, 0};
  size_t head[2];
  int off0[2];
#pragma unroll
  for (int pc = 0; pc < 2; ++pc) {  // uniform over the wave
    const int key0 = kb + 16 * pc;
    const int page = key0 < end ? table[key0 / bs] : 0;
    head[pc] = ((size_t)page * KV + kvh) * bs * D;
    off0[pc] = key0 % bs;
  }
  {  // keys: rows 0-7 of both tiles lie in the first piece, rows 8-15 in the second
    const int pc = col >> 3;
    const bool live = kb + 16 * pc < end;
    const bf16* krow = k_pages + (pc ? head[1] : head[0]) + (size_t)((pc ? off0[1] : off0[0]) + (KEY_OF_ROW(0, col) & 15)) * D + grp * 8;
#pragma unroll
    for (int tt = 0; tt < 2; ++tt)
#pragma unroll
      for (int c = 0; c < DC; ++c)
        st.k[tt][c] = live ? *reinterpret_cast<const bf16x8_t*>(krow + (size_t)tt * 4 * D + c * 32) : zero;
  }
  {  // values: keys 8 grp .. 8 grp + 7 of coordinates col, col + 16, ...  One instruction of the wave reads two runs of
     // 512 bytes, every 128-byte line whole, and a decode step reads a value once: marked as not to be kept (batch 64
     // of Qwen3-8B sizes 8,542 -> 8,872 tokens/s).  With pages of more than 32 tokens a step's 32 keys are part of a line,
     // which the next step needs again: no mark there.  The keys' loads share their lines in pairs and stay as they are.
    const int pc = grp >> 1;
    const bool live = kb + 16 * pc < end;
    const bf16* vcol = v_pages + (pc ? head[1] : head[0]) + (pc ? off0[1] : off0[0]) + 8 * (grp & 1) + (size_t)col * bs;
    if (bs <= 32) {  // uniform over the grid: two loops, so that neither holds a choice per load
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
        st.v[dt] = live ? __builtin_nontemporal_load(reinterpret_cast<const bf16x8_t*>(vcol + (size_t)dt * 16 * bs)) : zero;
    } else {
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
        st.v[dt] = live ? *reinterpret_cast<const bf16x8_t*>(vcol + (size_t)dt * 16 * bs) : zero;
    }
  }
}

// FRESH: the kernel takes the projection's output qkv [T, H + 2 KV, D] instead of finished queries
// and does what the norm-rotate-store kernel does before a decode step, for a step whose tokens
// are their own rows: each workgroup norms and rotates the queries of its group in registers (the
// partner i + D/2 of coordinate i lies in the same lane when D % 64 == 0), and the workgroup whose
// partition holds the token's own position makes the token's key and value, writes them to the
// pages and attends them from LDS, so nothing waits for those writes.  Same arithmetic as
// qk_norm_rope_store_bf16x8_kernel; the squares are summed in another order.
struct FreshQKV {
  const bf16* qkv;
  const void* qw;      // gains of the per-head norms, D values each, bf16 or fp32
  const void* kw;
  const float2* cs;    // [T, D/2] cos, sin of the whole head's rotation
  const int* slots;    // [T] page * block_size + offset of the new token, -1: keep it out of the pages
  bf16* k_store;       // the pages again, to write through
  bf16* v_store;
  float eps;
  int store;           // 0: queries only, the pages already hold the token's key and value
};

__device__ __forceinline__ void load_gains8(const float* w, float* g) {
  const float4 a = *reinterpret_cast<const float4*>(w), b = *reinterpret_cast<const float4*>(w + 4);
  g[0] = a.x; g[1] = a.y; g[2] = a.z; g[3] = a.w; g[4] = b.x; g[5] = b.y; g[6] = b.z; g[7] = b.w;
}
__device__ __forceinline__ void load_gains8(const bf16* w, float* g) {
  const bf16x8_t v = *reinterpret_cast<const bf16x8_t*>(w);
#pragma unroll
  for (int j = 0; j < 8; ++j) g[j] = (float)v[j];
}

template <int DC, int FRESH>  // D / 32; FRESH 0: finished queries, 1: qkv with bf16 gains, 2: with fp32 gains
__global__ __launch_bounds__(256) void attn_decode_mfma_kernel(
    const bf16* __restrict__ q, const bf16* __restrict__ k_pages, const bf16* __restrict__ v_pages,
    const int* __restrict__ items, const int* __restrict__ positions, const int* __restrict__ tok_row,
    const int* __restrict__ block_tables, int table_width, bf16* __restrict__ out, float* __restrict__ part_m,
    float* __restrict__ part_l, float* __restrict__ part_acc, int H, int KV, int bs, float scale, int window,
    int part_size, int P, int cus, FreshQKV fresh) {
  constexpr int D = DC * 32, DT = DC * 2;  // DT: tiles of 16 output coordinates
  extern __shared__ float smem[];          // [4][16] m, [4][16] l, [4][D][G] acc
  __shared__ __align__(16) bf16 fresh_kv[2][256];  // FRESH: the new token's key and value
  const int G = H / KV;
  int item = blockIdx.x, kvh = blockIdx.y;
  const int part = blockIdx.z;
  if (P == 1) {
    // Whole contexts, one workgroup each, of unequal length: two workgroups share a compute unit, and
    // the first two rounds of `cus` workgroups are placed at once, the second on top of the first.
    // Work is taken eight items at a time, their kv heads one after the other (so neighbours in this
    // order read different pages at the same time), with the second round backwards: with `items`
    // sorted longest first a compute unit's first two are a long and a short one, and what follows
    // goes to whichever compute unit is free, longest first.
    int s = blockIdx.x + gridDim.x * blockIdx.y;
    const int total = gridDim.x * gridDim.y;
    if (s >= cus && s < 2 * cus) s = cus + (min(2 * cus, total) - 1 - s);
    const int N = gridDim.x, first = s / (8 * KV) * 8, r = s % (8 * KV), here = min(8, N - first);
    item = first + r % here;
    kvh = r / here;
  }
  const int t = items ? items[item] : item;  // null: every token, in order
  const int pos = positions[t];
  const int ctx = pos + 1;
  const int lo = window > 0 ? max(0, ctx - window) : 0;
  const int k0 = max(lo, part * part_size), k1 = min(ctx, (part + 1) * part_size);
  const int h0 = kvh * G;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int col = lane & 15, grp = lane >> 4;  // col: head within the group (and key row of A)

  if (k0 >= k1) {  // an empty partition (P > 1 only): mark it so for the reduce
    if (tid < G) {
      const size_t o = ((size_t)item * H + h0 + tid) * P + part;
      part_m[o] = NEG_INF;
      part_l[o] = 0.f;
    }
    for (int idx = tid; idx < G * D; idx += 256)
      part_acc[(((size_t)item * H + h0 + idx / D) * P + part) * D + idx % D] = 0.f;
    return;
  }
  const int* table = block_tables + (size_t)(tok_row ? tok_row[t] : t) * table_width;  // null: token t is row t

  // Everything is asked for before anything is waited for: the queries (FRESH: as the projection
  // left them, with the gains and angles of this lane's coordinates; in the workgroup that holds the
  // token's own position, wave 0 the new key and wave 1 the new value), then the first keys and values.
  constexpr int HC = DC / 2, HALF = D / 2, PAIRS = (HALF + WAVE - 1) / WAVE;
  using W = typename std::conditional<FRESH == 2, float, bf16>::type;  // the gains' type
  bf16x8_t qop[DC];
  const bf16x8_t zero = {0, 0, 0, 0, 0, 0, 0, 0};
  const size_t row = (size_t)t * (H + 2 * KV);  // FRESH: the token's heads in qkv
  {
    const bf16* qrow = FRESH ? fresh.qkv + (row + h0 + min(col, G - 1)) * D + grp * 8
                             : q + ((size_t)t * H + h0 + min(col, G - 1)) * D + grp * 8;
#pragma unroll
    for (int c = 0; c < DC; ++c) qop[c] = col < G ? *reinterpret_cast<const bf16x8_t*>(qrow + c * 32) : zero;
  }
  [[maybe_unused]] float gain[FRESH ? DC * 8 : 1];
  [[maybe_unused]] float4 angle[FRESH ? HC * 4 : 1];  // (cos, sin) of two pairs each
  [[maybe_unused]] bool fresh_here = false;           // this workgroup's keys include the token's own
  [[maybe_unused]] int slot = -1;
  [[maybe_unused]] bf16 ka[PAIRS], kb2[PAIRS], vv[2 * PAIRS];
  [[maybe_unused]] float gka[PAIRS], gkb[PAIRS];
  [[maybe_unused]] float2 kcs[PAIRS];
  if constexpr (FRESH != 0) {
#pragma unroll
    for (int c = 0; c < HC; ++c) {
      const int i0 = c * 32 + grp * 8;
      load_gains8((const W*)fresh.qw + i0, &gain[c * 8]);
      load_gains8((const W*)fresh.qw + i0 + HALF, &gain[(c + HC) * 8]);
      const float4* cs4 = reinterpret_cast<const float4*>(fresh.cs + (size_t)t * HALF + i0);
#pragma unroll
      for (int j = 0; j < 4; ++j) angle[c * 4 + j] = cs4[j];
    }
    fresh_here = fresh.store && pos >= k0 && pos < k1;  // the same for the whole workgroup
    if (fresh_here && wave == 0) {
      slot = fresh.slots[t];
      const bf16* src = fresh.qkv + (row + H + kvh) * D;
#pragma unroll
      for (int p = 0; p < PAIRS; ++p) {
        const int i = min(lane + p * WAVE, HALF - 1);
        ka[p] = src[i];
        kb2[p] = src[i + HALF];
        gka[p] = (float)((const W*)fresh.kw)[i];
        gkb[p] = (float)((const W*)fresh.kw)[i + HALF];
        kcs[p] = fresh.cs[(size_t)t * HALF + i];
      }
    } else if (fresh_here && wave == 1) {
      slot = fresh.slots[t];
      const bf16* src = fresh.qkv + (row + H + KV + kvh) * D;
#pragma unroll
      for (int p = 0; p < 2 * PAIRS; ++p) vv[p] = src[min(lane + p * WAVE, D - 1)];
    }
  }
  const int first = (k0 / 32) * 32;
  KVStep<DC> cur, nxt;
  int kb = first + 32 * wave;
  if (kb < k1) load_kv_step<DC>(cur, k_pages, v_pages, table, kb, k1, KV, kvh, bs, col, grp);

  if constexpr (FRESH != 0) {
    // the queries of this lane's head: norm over the head (its D values lie in four lanes), rotation
    float ss = 0.f;
#pragma unroll
    for (int c = 0; c < DC; ++c)
#pragma unroll
      for (int j = 0; j < 8; ++j) ss += (float)qop[c][j] * (float)qop[c][j];
    ss += __shfl_xor(ss, 16, WAVE);
    ss += __shfl_xor(ss, 32, WAVE);
    const float inv = 1.0f / sqrtf(ss / (float)D + fresh.eps);
#pragma unroll
    for (int c = 0; c < HC; ++c)
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float a = (float)qop[c][j] * inv * gain[c * 8 + j];
        const float b = (float)qop[c + HC][j] * inv * gain[(c + HC) * 8 + j];
        const float4 cs2 = angle[c * 4 + j / 2];
        const float cc = (j & 1) ? cs2.z : cs2.x, sn = (j & 1) ? cs2.w : cs2.y;
        qop[c][j] = (bf16)(a * cc - b * sn);
        qop[c + HC][j] = (bf16)(b * cc + a * sn);
      }
    if (col >= G) {
#pragma unroll
      for (int c = 0; c < DC; ++c) qop[c] = zero;
    }
    if (fresh_here) {
      const size_t head = slot >= 0 ? ((size_t)(slot / bs) * KV + kvh) * bs * D : 0;
      if (wave == 0) {  // the key: norm and rotation as for the queries, one wave over the pairs
        float ks = 0.f;
#pragma unroll
        for (int p = 0; p < PAIRS; ++p)
          if (lane + p * WAVE < HALF) ks += (float)ka[p] * (float)ka[p] + (float)kb2[p] * (float)kb2[p];
        ks = wave_sum(ks);
        const float kinv = 1.0f / sqrtf(ks / (float)D + fresh.eps);
        bf16* dst = fresh.k_store + head + (size_t)(slot % bs) * D;
#pragma unroll
        for (int p = 0; p < PAIRS; ++p) {
          const int i = lane + p * WAVE;
          if (i < HALF) {
            const float a = (float)ka[p] * kinv * gka[p], b = (float)kb2[p] * kinv * gkb[p];
            const bf16 ra = finite_or_zero((bf16)(a * kcs[p].x - b * kcs[p].y));
            const bf16 rb = finite_or_zero((bf16)(b * kcs[p].x + a * kcs[p].y));
            fresh_kv[0][i] = ra;
            fresh_kv[0][i + HALF] = rb;
            if (slot >= 0) { dst[i] = ra; dst[i + HALF] = rb; }
          }
        }
      } else if (wave == 1) {  // the value, as it is; its page is stored transposed
        bf16* vt = fresh.v_store + head + slot % bs;
#pragma unroll
        for (int p = 0; p < 2 * PAIRS; ++p) {
          const int i = lane + p * WAVE;
          if (i < D) {
            const bf16 rv = finite_or_zero((bf16)vv[p]);
            fresh_kv[1][i] = rv;
            if (slot >= 0) vt[(size_t)i * bs] = rv;
          }
        }
      }
      __syncthreads();
    }
  }
  f32x4_t o[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) o[dt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  float m = NEG_INF, l = 0.f;

  for (; kb < k1; kb += 128) {
    const bool more = kb + 128 < k1;
    if (more) load_kv_step<DC>(nxt, k_pages, v_pages, table, kb + 128, k1, KV, kvh, bs, col, grp);
    if constexpr (FRESH != 0) {
      if (fresh_here && pos >= kb && pos < kb + 32) {  // this wave's step holds the token itself: take it from LDS
        const int at = pos - kb;  // = KEY_OF_ROW(tile, row) for
        const int tile = (at >> 2) & 1, row = 4 * (at >> 3) + (at & 3);
        if (col == row) {
#pragma unroll
          for (int tt = 0; tt < 2; ++tt)
            if (tt == tile) {
#pragma unroll
              for (int c = 0; c < DC; ++c) cur.k[tt][c] = *reinterpret_cast<const bf16x8_t*>(&fresh_kv[0][c * 32 + grp * 8]);
            }
        }
        if (grp == (at >> 3)) {
#pragma unroll
          for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int j = 0; j < 8; ++j)
              if (j == (at & 7)) cur.v[dt][j] = fresh_kv[1][dt * 16 + col];
        }
      }
    }
    // ---- scores of 32 keys
    f32x4_t s[2];
#pragma unroll
    for (int tt = 0; tt < 2; ++tt) {
      s[tt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int c = 0; c < DC; ++c) s[tt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(cur.k[tt][c], qop[c], s[tt], 0, 0, 0);
    }
    // ---- online softmax for this lane's head column
    float mx = NEG_INF;
#pragma unroll
    for (int tt = 0; tt < 2; ++tt)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int key = kb + KEY_OF_ROW(tt, 4 * grp + r);
        const bool seen = key >= k0 && key < k1;
        s[tt][r] = seen ? s[tt][r] * scale : NEG_INF;
        mx = fmaxf(mx, s[tt][r]);
      }
    mx = quad_rows_max(mx);
    const float mn = fmaxf(m, mx);
    float alpha = 1.f, rs = 0.f;
    bf16x8_t pop;
    if (mn == NEG_INF) {  // nothing seen yet (a window may hide whole steps)
#pragma unroll
      for (int j = 0; j < 8; ++j) pop[j] = (bf16)0.f;
    } else {
      alpha = (m == NEG_INF) ? 0.f : __expf(m - mn);
#pragma unroll
      for (int tt = 0; tt < 2; ++tt)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float pv = __expf(s[tt][r] - mn);  // exp(-inf) = 0 for hidden keys
          rs += pv;
          pop[tt * 4 + r] = (bf16)pv;
        }
      m = mn;
    }
    l = l * alpha + quad_rows_sum(rs);
    // ---- weighted values
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      o[dt] *= alpha;
      o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(cur.v[dt], pop, o[dt], 0, 0, 0);
    }
    if (more) cur = nxt;
  }

  // ---- merge the four waves
  float* sm = smem;
  float* sl = smem + 64;
  float* so = smem + 128;  // [4][D][G]
  if (grp == 0 && col < G) { sm[wave * 16 + col] = m; sl[wave * 16 + col] = l; }
  if (col < G) {
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int r = 0; r < 4; ++r) so[((size_t)wave * D + dt * 16 + 4 * grp + r) * G + col] = o[dt][r];
  }
  __syncthreads();
  for (int idx = tid; idx < G * D; idx += 256) {
    const int g = idx / D, d = idx % D;
    float mxw = NEG_INF;
#pragma unroll
    for (int w = 0; w < 4; ++w) mxw = fmaxf(mxw, sm[w * 16 + g]);
    float num = 0.f, den = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const float mw = sm[w * 16 + g];
      const float e = (mw == NEG_INF) ? 0.f : __expf(mw - mxw);
      num += so[((size_t)w * D + d) * G + g] * e;
      den += sl[w * 16 + g] * e;
    }
    const int h = h0 + g;
    if (P == 1) {
      out[((size_t)t * H + h) * D + d] = (bf16)(num / den);
    } else {
      const size_t ob = ((size_t)item * H + h) * P + part;
      part_acc[ob * D + d] = num;
      if (d == 0) { part_m[ob] = mxw; part_l[ob] = den; }
    }
  }
}

// ---- bf16 prefill through the matrix cores ----------------------------------------------
//
// Work item: up to 64 consecutive query tokens of one request (`tiles` rows: first flat
// token, count, block-table row, position of the first) for one kv head.  A wave owns 32
// of those queries for one query head, as two MFMA column tiles of 16; the four waves of a
// workgroup take heads of the same group (or the other half of the queries), so they all
// need the same keys and values.  Those come into LDS once per workgroup by loads that write
// LDS directly (global_load_lds_dwordx4: no staging registers), into a ring of four stages
// of 32 keys.  A round of the main loop computes 64 keys (two stages) while the copies of the
// next 64 are in flight into the other two, and costs one barrier; 64 keys give a wave 64
// independent MFMAs between its softmax reductions, which is what hides their latency.
// Two waves copy a stage's keys, two its values (a 16-key piece of a page is contiguous in
// memory both for keys and, thanks to the transposed value pages, for values).
//
// LDS layout of a stage, in 16-byte slots:
//   keys:   slot (chunk * 32 + t) holds coordinates 8 chunk .. + 7 of the key behind row t % 16
//           of score tile t / 16, so the 64 lanes of an MFMA operand (row = lane % 16,
//           chunk = 4 step + lane / 16) read four runs of 16 consecutive slots: no bank
//           conflicts, no padding, any head width;
//   values: per 16-key piece, slot (h * D + d) holds keys 8h .. 8h+7 of coordinate d: the eight
//           keys whose weights a lane holds are one slot, and 16 lanes read 256 consecutive bytes.
// A load instruction fills 64 consecutive slots (slot = first + lane); which 16 bytes of
// memory a lane fetches is free, which is how the key layout comes about.
// A query at position p sees keys lo..p by absolute position, wherever the row starts.
// max(a, b, c) as the one instruction it is; NaN operands lose, as with fmaxf.
__device__ __forceinline__ float max3(float a, float b, float c) {
  float r;
  asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
}

#define PF_STAGES 4
// s_waitcnt that only constrains the vector-memory counter (vmcnt: bits 3:0 and 15:14)
#define PF_WAIT_VM(N) __builtin_amdgcn_s_waitcnt(((N) & 15) | (((N) >> 4) << 14) | (7 << 4) | (15 << 8))

// A step of few work items takes as long as its longest one (a portion of a prompt behind thousands of cached
// tokens: a hundred workgroups of hundreds of rounds each, on a GPU with room for five hundred).  With `pieces` > 1
// every work item comes as that many workgroups: an item of more than `piece_rounds` rounds of 64 keys is cut
// along its keys into pieces of that many rounds (the last one, with the causal diagonal, may be shorter), each
// piece leaves the maxima, sums and unnormalised outputs of its queries, and `attn_prefill_merge_kernel` puts them
// together; a shorter item is its first workgroup's alone, as without the cut, and the others leave at once.
struct PrefillSplit {
  int pieces;        // workgroups per item; 1: no item is cut
  int piece_rounds;  // rounds of a piece
  int* cut;          // [items]: the pieces the item was cut into (1: not cut), for the merge
  float* ml;         // [T, H, pieces, 2]: maximum (base 2, scaled) and sum
  float* acc;        // [T, H, pieces, D]: unnormalised output
};
constexpr int PREFILL_MIN_PIECE_ROUNDS = 2;  // an item's last two rounds hold its own tokens: one piece

template <int DC, int QT>  // D / 32; column tiles of 16 queries that a wave owns: 2, or 1 (see the launcher)
__global__ __launch_bounds__(256, 2) void attn_prefill_mfma_kernel(
    const bf16* __restrict__ q, const bf16* __restrict__ k_pages, const bf16* __restrict__ v_pages,
    const int* __restrict__ tiles, const int* __restrict__ block_tables, int table_width,
    bf16* __restrict__ out, int H, int KV, int bs, float scale, int window, int units_z, int pass, PrefillSplit split) {
  constexpr int D = DC * 32, DT = DC * 2;
  constexpr int PIECE = 64 * DC;  // 16-byte slots of a 16-key piece: 16 * D / 8
  typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
  typedef __attribute__((address_space(3))) void* lds_ptr_t;
  typedef const __attribute__((address_space(1))) void* global_ptr_t;
  __shared__ __attribute__((aligned(16))) u32x4_t lds[PF_STAGES][4][PIECE];  // [stage][K0 K1 V0 V1][slot]

  const int G = H / KV;
  // Work items (tile, kv head, group of four waves) in the order of `tiles`, which the caller
  // sorts by the number of keys seen, most first; blocks of `pass` items alternate direction.
  // With one pass per round of workgroups that the GPU places (its compute units), a compute
  // unit that received one of the longest items in one round receives one of the shortest of
  // the next, so that causal prompts, whose items range from one step to hundreds, finish
  // together.
  const int per_tile = KV * units_z;
  int item = blockIdx.x;
  {
    const int block = item / pass, first = block * pass;
    const int size = min(pass, (int)gridDim.x - first);
    if (block & 1) item = first + size - 1 - (item - first);
  }
  int piece = 0;  // which of an item's workgroups this is
  if (split.pieces > 1) {
    piece = item % split.pieces;
    item /= split.pieces;
  }
  const int tile = item / per_tile, kvh = (item % per_tile) / units_z, bz = item % units_z;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int col = lane & 15, grp = lane >> 4;
  const int tok0 = tiles[4 * tile], count = tiles[4 * tile + 1], row = tiles[4 * tile + 2];
  const int pos0 = tiles[4 * tile + 3];
  const int* table = block_tables + (size_t)row * table_width;

  // the keys this workgroup walks: from the first key any of its waves sees to the last
  int wg_lo = 0x7fffffff, wg_last = -1;
  constexpr int WQ = 16 * QT, PARTS = 64 / WQ;  // queries of a wave; waves that share a head's 64 queries
  for (int u = bz * 4; u < bz * 4 + 4 && u < PARTS * G; ++u) {
    const int uq0 = (u / G) * WQ;
    if (uq0 >= count) continue;
    wg_last = max(wg_last, pos0 + min(count, uq0 + WQ) - 1);
    wg_lo = min(wg_lo, window > 0 ? max(0, pos0 + uq0 - window + 1) : 0);
  }
  if (wg_last < 0) {  // uniform over the workgroup
    if (split.pieces > 1 && piece == 0 && threadIdx.x == 0) split.cut[item] = 1;
    return;
  }
  bool partial = false;  // this workgroup leaves its share of a cut item for the merge
  if (split.pieces > 1) {
    const int kb_first = (wg_lo / 32) * 32, all_rounds = ((wg_last - kb_first) / 32 + 2) / 2;
    const int mine = min(split.pieces, (all_rounds + split.piece_rounds - 1) / split.piece_rounds);  // pieces of this item
    if (piece == 0 && threadIdx.x == 0) split.cut[item] = mine;
    if (piece >= mine) return;
    if (mine > 1) {
      partial = true;
      const int from = kb_first + 64 * split.piece_rounds * piece;  // the piece's first key
      if (piece + 1 < mine) wg_last = from + 64 * split.piece_rounds - 1;
      if (piece > 0) wg_lo = from;
    }
  }

  // this wave's queries
  const int unit = bz * 4 + wave;
  const int head = kvh * G + unit % G;
  const int q0 = (unit / G) * WQ;
  const bool working = unit < PARTS * G && q0 < count;
  const int nq = working ? min(WQ, count - q0) : 1;
  const int my_last = working ? pos0 + q0 + nq - 1 : -1;
  const int my_first_q = pos0 + q0;                  // position of this wave's first query
  const float scale2 = scale * 1.4426950408889634f;  // scores are kept in base 2
  const int my_lo = working ? (window > 0 ? max(0, pos0 + q0 - window + 1) : 0) : 0x7fffffff;

  bf16x8_t qop[QT][DC];
  int qpos[QT];
  bool qok[QT];
#pragma unroll
  for (int qt = 0; qt < QT; ++qt) {
    const int qi = qt * 16 + col;
    qok[qt] = working && qi < nq;
    const int qc = min(qi, nq - 1);  // columns past the end repeat the last query and are not stored
    qpos[qt] = pos0 + q0 + qc;
    if (working) {
      const bf16* qrow = q + ((size_t)(tok0 + q0 + qc) * H + head) * D + grp * 8;
#pragma unroll
      for (int c = 0; c < DC; ++c) qop[qt][c] = *reinterpret_cast<const bf16x8_t*>(qrow + c * 32);
    } else {
#pragma unroll
      for (int c = 0; c < DC; ++c) qop[qt][c] = bf16x8_t{0, 0, 0, 0, 0, 0, 0, 0};
    }
  }
  f32x4_t o[QT][DT];
  float m[QT], l[QT];
#pragma unroll
  for (int qt = 0; qt < QT; ++qt) {
    m[qt] = NEG_INF;
    l[qt] = 0.f;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) o[qt][dt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  }

  // ---- this wave's share of the copies: of every 32-key step, waves 0 and 1 bring the keys
  // (half of the 16-byte chunks of all 32 rows each), waves 2 and 3 the values of keys 0-15 and
  // 16-31.
  const int kb0 = (wg_lo / 32) * 32;
  const int nsteps = (wg_last - kb0) / 32 + 1;
  const int last_piece = (wg_last / 16) * 16;
  // Where the 16-key pieces lie in memory is worked out 64 pieces at a time, one piece per lane
  // (its page from the block table, asked for one batch of 64 ahead), and a step reads the two
  // it copies out of those lanes.  Done by the scalar unit for every step instead, the divisions
  // by the page size and the 64-bit products took a fifth of the kernel's time: that unit is
  // shared by all waves of the compute unit.  A piece that would start beyond the last key
  // repeats the last one (finite numbers; its scores are masked).
  unsigned long long k_at = 0, v_at = 0;  // byte offsets of this lane's piece in k_pages and v_pages
  auto entry_of = [&](int piece) { return min(kb0 + 16 * piece, last_piece) / bs; };
  int page_ahead = table[entry_of(lane)];
  auto locate = [&](int batch) {  // pieces 64 batch .. 64 batch + 63
    const int piece = 64 * batch + lane, key = min(kb0 + 16 * piece, last_piece);
    const unsigned long long row = (unsigned long long)((unsigned)page_ahead * KV + kvh) * bs;
    k_at = (row + key % bs) * (D * 2);
    v_at = (row * D + key % bs) * 2;
    page_ahead = table[entry_of(piece + 64)];
  };
  auto at = [&](unsigned long long offsets, int piece) {
    const unsigned lo = __builtin_amdgcn_readlane((unsigned)offsets, piece & 63);
    const unsigned hi = __builtin_amdgcn_readlane((unsigned)(offsets >> 32), piece & 63);
    return ((unsigned long long)hi << 32) | lo;
  };
  // what of a copy's address belongs to the lane, in bytes
  int lane_at[DC];
  if (wave >= 2) {
#pragma unroll
    for (int i = 0; i < DC; ++i) {  // values: slot = h * D + d holds keys 8h .. 8h+7 of coordinate d
      const int slot = i * 64 + lane, h = slot / D, d = slot % D;
      lane_at[i] = (d * bs + h * 8) * 2;
    }
  } else {
    // keys: slot = chunk * 32 + t holds coordinates 8 chunk .. + 7 of the key that row t of the
    // step's two score tiles stands for (see KEY_OF_ROW)
    const int t = lane & 31, key = KEY_OF_ROW(t >> 4, t & 15);
    lane_at[0] = ((key & 15) * D + (wave * (2 * DC) + (lane >> 5)) * 8) * 2;  // the further chunks: + 32 bytes each
  }
  const bool second_piece = KEY_OF_ROW((lane & 31) >> 4, lane & 15) >> 4;
  auto issue = [&](int step) {
    if ((step & 31) == 0) locate(step >> 5);
    if (wave >= 2) {
      const char* src = reinterpret_cast<const char*>(v_pages) + at(v_at, 2 * step + wave - 2);
      u32x4_t* dst = &lds[step % PF_STAGES][wave][0];
#pragma unroll
      for (int i = 0; i < DC; ++i)
        __builtin_amdgcn_global_load_lds((global_ptr_t)(src + lane_at[i]), (lds_ptr_t)(dst + i * 64), 16, 0, 0);
    } else {
      const unsigned long long first = at(k_at, 2 * step), second = at(k_at, 2 * step + 1);
      const char* src = reinterpret_cast<const char*>(k_pages) + (second_piece ? second : first) + lane_at[0];
      u32x4_t* dst = &lds[step % PF_STAGES][0][0] + wave * (DC * 64);
#pragma unroll
      for (int i = 0; i < DC; ++i)
        __builtin_amdgcn_global_load_lds((global_ptr_t)(src + i * 32), (lds_ptr_t)(dst + i * 64), 16, 0, 0);
    }
  };
  // The same copies one instruction at a time, for a round's two steps: `aim` works out where they read
  // and write, `copy(k)` issues the k-th of their 2 DC instructions (between the round's matrix products,
  // whose issue otherwise leaves the wave idle, instead of in one block that the wave waits through).
  const char* from[2];
  u32x4_t* to[2];
  auto aim = [&](int step0) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int step = step0 + j;
      if ((step & 31) == 0) locate(step >> 5);
      if (wave >= 2) {
        from[j] = reinterpret_cast<const char*>(v_pages) + at(v_at, 2 * step + wave - 2);
        to[j] = &lds[step % PF_STAGES][wave][0];
      } else {
        const unsigned long long first = at(k_at, 2 * step), second = at(k_at, 2 * step + 1);
        from[j] = reinterpret_cast<const char*>(k_pages) + (second_piece ? second : first) + lane_at[0];
        to[j] = &lds[step % PF_STAGES][0][0] + wave * (DC * 64);
      }
    }
  };
  auto copy = [&](int k) {
    const int j = k / DC, i = k % DC;
    if (wave >= 2) __builtin_amdgcn_global_load_lds((global_ptr_t)(from[j] + lane_at[i]), (lds_ptr_t)(to[j] + i * 64), 16, 0, 0);
    else __builtin_amdgcn_global_load_lds((global_ptr_t)(from[j] + i * 32), (lds_ptr_t)(to[j] + i * 64), 16, 0, 0);
  };
  const int nrounds = (nsteps + 1) / 2;
  issue(0);
  issue(1);  // beyond the last key it repeats the last piece
  for (int rd = 0; rd < nrounds; ++rd) {
    PF_WAIT_VM(0);    // this wave's copies for the round have landed
    __syncthreads();  // ... and everyone's; and everyone is done with the round before
    const bool more = rd + 1 < nrounds;  // copies into the two stages the round before used
    const int kb = kb0 + 64 * rd;
    const bool active = working && kb <= my_last && kb + 63 >= my_lo;
    if (more) {
      aim(2 * rd + 2);
      if (!active) {
#pragma unroll
        for (int k = 0; k < 2 * DC; ++k) copy(k);
      }
    }
    if (active) {
      // raw scores of 64 keys x 16 QT queries; a key operand is read from LDS once for all of a wave's query tiles
      f32x4_t sc[QT][4];
#pragma unroll
      for (int qt = 0; qt < QT; ++qt)
#pragma unroll
        for (int tt = 0; tt < 4; ++tt) sc[qt][tt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
      // The operands of a whole tile are asked from LDS before its products start, and the next
      // tile's while they run: a product must not wait for a read issued just before it.
      u32x4_t kraw[2][DC];
      auto read_keys = [&](int tt, u32x4_t (&into)[DC]) {
        // score tile tt: rows KEY_OF_ROW(tt & 1, .) of step tt >> 1
        const u32x4_t* keys = &lds[(2 * rd + (tt >> 1)) % PF_STAGES][0][0] + (tt & 1) * 16 + col;
#pragma unroll
        for (int c = 0; c < DC; ++c) into[c] = keys[(c * 4 + grp) * 32];
      };
      read_keys(0, kraw[0]);
#pragma unroll
      for (int tt = 0; tt < 4; ++tt) {
        if (tt + 1 < 4) read_keys(tt + 1, kraw[(tt + 1) & 1]);
        __builtin_amdgcn_sched_barrier(0);  // or the compiler moves every read down to its product
#pragma unroll
        for (int c = 0; c < DC; ++c) {
          const bf16x8_t kop = __builtin_bit_cast(bf16x8_t, kraw[tt & 1][c]);
#pragma unroll
          for (int qt = 0; qt < QT; ++qt)
            sc[qt][tt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kop, qop[qt][c], sc[qt][tt], 0, 0, 0);
        }
        if (more) {  // a quarter of the round's copies behind each tile's products
#pragma unroll
          for (int k = tt * (2 * DC) / 4; k < (tt + 1) * (2 * DC) / 4; ++k) copy(k);
        }
      }
      // Only rounds that touch the causal diagonal, the window's edge or the end of the context
      // need a mask; the others see all 64 keys (uniform over the wave).
      const bool masked = kb + 63 > my_first_q || (window > 0 && kb < my_last - window + 1);
      bf16x8_t pop[QT][2];
      float alpha[QT];
      bool rescale = false;
#pragma unroll
      for (int qt = 0; qt < QT; ++qt) {
        if (masked) {
#pragma unroll
          for (int tt = 0; tt < 4; ++tt)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              const int key = kb + 32 * (tt >> 1) + KEY_OF_ROW(tt & 1, 4 * grp + r);
              const bool seen = key <= qpos[qt] && (window <= 0 || key > qpos[qt] - window);
              sc[qt][tt][r] = seen ? sc[qt][tt][r] : NEG_INF;
            }
        }
        // sixteen scores to one in eight three-way maxima (fmaxf would first quiet every operand)
        const float m0 = max3(sc[qt][0][0], sc[qt][0][1], sc[qt][0][2]), m1 = max3(sc[qt][0][3], sc[qt][1][0], sc[qt][1][1]);
        const float m2 = max3(sc[qt][1][2], sc[qt][1][3], sc[qt][2][0]), m3 = max3(sc[qt][2][1], sc[qt][2][2], sc[qt][2][3]);
        const float m4 = max3(sc[qt][3][0], sc[qt][3][1], sc[qt][3][2]);
        const float mx = quad_rows_max(max3(max3(m0, m1, m2), max3(m3, m4, sc[qt][3][3]), NEG_INF));
        // base-2 softmax: scale and log2(e) are folded into one factor (positive, so maxima agree)
        const float mn = fmaxf(m[qt], mx * scale2);
        // Without a branch, so that the two query tiles' arithmetic can be interleaved: while a row
        // has seen no key, every score and mn are -inf, and 2^(-inf - 0) = 0 is what each weight and
        // the factor of the (empty) past should be.
        const float base = mn == NEG_INF ? 0.f : mn;
        alpha[qt] = __builtin_amdgcn_exp2f(m[qt] - base);
        float part[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int tt = 0; tt < 4; ++tt)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const float pv = __builtin_amdgcn_exp2f(fmaf(sc[qt][tt][r], scale2, -base));
            part[r] += pv;
            pop[qt][tt >> 1][(tt & 1) * 4 + r] = (bf16)pv;
          }
        const float rs = (part[0] + part[1]) + (part[2] + part[3]);
        m[qt] = mn;
        l[qt] = l[qt] * alpha[qt] + quad_rows_sum(rs);
        rescale = rescale || alpha[qt] != 1.f;
      }
      // the accumulated output is rescaled only when some query's maximum moved (rare once the
      // first keys have been seen)
      if (__any(rescale)) {
#pragma unroll
        for (int qt = 0; qt < QT; ++qt)
#pragma unroll
          for (int dt = 0; dt < DT; ++dt) o[qt][dt] *= alpha[qt];
      }
      u32x4_t vraw[2][DT];
      auto read_values = [&](int j, u32x4_t (&into)[DT]) {
        // this lane's eight weights of step j belong to keys 8 grp .. 8 grp + 7: one 16-byte slot
        const u32x4_t* values = &lds[(2 * rd + j) % PF_STAGES][2 + (grp >> 1)][(grp & 1) * D + col];
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) into[dt] = values[dt * 16];
      };
      read_values(0, vraw[0]);
      read_values(1, vraw[1]);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int j = 0; j < 2; ++j) {
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
          const bf16x8_t vop = __builtin_bit_cast(bf16x8_t, vraw[j][dt]);
#pragma unroll
          for (int qt = 0; qt < QT; ++qt) o[qt][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vop, pop[qt][j], o[qt][dt], 0, 0, 0);
        }
      }
    }
  }

  if (partial) {
#pragma unroll
    for (int qt = 0; qt < QT; ++qt) {
      if (!qok[qt]) continue;
      const size_t at = ((size_t)(tok0 + q0 + qt * 16 + col) * H + head) * split.pieces + piece;
      if (grp == 0) *reinterpret_cast<float2*>(split.ml + at * 2) = make_float2(m[qt], l[qt]);
      float* arow = split.acc + at * D + 4 * grp;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) *reinterpret_cast<f32x4_t*>(arow + dt * 16) = o[qt][dt];
    }
    return;
  }
#pragma unroll
  for (int qt = 0; qt < QT; ++qt) {
    if (!qok[qt]) continue;
    const float inv = 1.0f / l[qt];
    bf16* orow = out + ((size_t)(tok0 + q0 + qt * 16 + col) * H + head) * D + 4 * grp;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      const bf16x4_t r4 = {(bf16)(o[qt][dt][0] * inv), (bf16)(o[qt][dt][1] * inv), (bf16)(o[qt][dt][2] * inv),
                           (bf16)(o[qt][dt][3] * inv)};
      *reinterpret_cast<bf16x4_t*>(orow + dt * 16) = r4;
    }
  }
}

// The pieces of every cut item, put together: one workgroup per item, its waves and lanes holding the queries and
// coordinates they hold in the kernel above.  out = sum_j acc_j 2^(m_j - m) / sum_j l_j 2^(m_j - m) with m the
// largest maximum; a piece that saw no key has m = -inf and l = 0.
template <int DC, int QT>
__global__ __launch_bounds__(256) void attn_prefill_merge_kernel(const int* __restrict__ tiles, bf16* __restrict__ out,
                                                                  int H, int KV, int units_z, PrefillSplit split) {
  constexpr int D = DC * 32, DT = DC * 2, WQ = 16 * QT, PARTS = 64 / WQ;
  const int item = blockIdx.x;
  const int n = split.cut[item];
  if (n <= 1) return;
  const int G = H / KV, per_tile = KV * units_z;
  const int tile = item / per_tile, kvh = (item % per_tile) / units_z, bz = item % units_z;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, col = lane & 15, grp = lane >> 4;
  const int tok0 = tiles[4 * tile], count = tiles[4 * tile + 1];
  const int unit = bz * 4 + wave, head = kvh * G + unit % G, q0 = (unit / G) * WQ;
  if (unit >= PARTS * G || q0 >= count) return;
#pragma unroll
  for (int qt = 0; qt < QT; ++qt) {
    const int qi = q0 + qt * 16 + col;
    if (qi >= count) continue;
    const size_t at = ((size_t)(tok0 + qi) * H + head) * split.pieces;
    const float2* ml = reinterpret_cast<const float2*>(split.ml) + at;  // (m, l) of the pieces
    float m = NEG_INF;
    for (int j = 0; j < n; ++j) m = fmaxf(m, ml[j].x);
    f32x4_t sum[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) sum[dt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    float den = 0.f;
    for (int j = 0; j < n; ++j) {
      const float2 p = ml[j];
      const float w = p.x == NEG_INF ? 0.f : __builtin_amdgcn_exp2f(p.x - m);
      den += p.y * w;
      const float* a = split.acc + (at + j) * D + 4 * grp;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) sum[dt] += *reinterpret_cast<const f32x4_t*>(a + dt * 16) * w;
    }
    const float inv = 1.0f / den;
    bf16* orow = out + ((size_t)(tok0 + qi) * H + head) * D + 4 * grp;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      const bf16x4_t r4 = {(bf16)(sum[dt][0] * inv), (bf16)(sum[dt][1] * inv), (bf16)(sum[dt][2] * inv), (bf16)(sum[dt][3] * inv)};
      *reinterpret_cast<bf16x4_t*>(orow + dt * 16) = r4;
    }
  }
}

// tiles: [num_tiles, 4] int32 (first flat token, count <= 64, block-table row, first position);
// fastest when sorted by first position + count, largest first.
// query_tiles: 2, a wave owns 32 queries of a head and a workgroup two heads' 64; or 1, a wave owns 16 and a
// workgroup one head's 64: twice the workgroups, each with half the arithmetic for the same keys and values
// brought into LDS, so that a round of 64 keys is shorter.  That pays where few work items decide the time
// (a lone prompt of a few thousand tokens: its last tile's rounds are a chain that nothing shortens).
// pieces > 1: every work item comes as that many workgroups, and items of more than piece_rounds rounds of 64 keys are
// cut along their keys into pieces of that many rounds and merged by a second kernel (see PrefillSplit); the caller
// then brings cut [num_tiles * KV * units] int32 with units = ceil(64 / (16 query_tiles) * (H / KV) / 4), part_ml
// [T, H, pieces, 2] and part_acc [T, H, pieces, D] fp32, T being one more than the largest flat token of a tile, and
// piece_rounds * pieces covers the longest item.  pieces <= 1: none is cut, the three may be null.
extern "C" int as_attn_prefill_mfma(const void* q, const void* k_pages, const void* v_pages, const int* tiles,
                                    int num_tiles, const int* block_tables, int table_width, void* out, int H,
                                    int KV, int D, int bs, float scale, int window, int query_tiles,
                                    int pieces, int piece_rounds, int* cut, float* part_ml, float* part_acc,
                                    hipStream_t stream) {
  if (num_tiles <= 0) return AS_OK;
  if (H <= 0 || KV <= 0 || H % KV || bs <= 0 || table_width <= 0) return AS_BAD_SHAPE;
  const int G = H / KV;
  if (D % 32 || D <= 0 || D > 256 || bs % 16) return AS_BAD_SHAPE;
  if (query_tiles != 1 && query_tiles != 2) return AS_BAD_SHAPE;
  if (pieces < 1) pieces = 1;
  if (pieces > 1 && (piece_rounds < PREFILL_MIN_PIECE_ROUNDS || !cut || !part_ml || !part_acc)) return AS_BAD_SHAPE;
  const int units_z = (64 / (16 * query_tiles) * G + 3) / 4;
  const long items = (long)num_tiles * KV * units_z;
  const long blocks = items * pieces;
  if (blocks > 0x7fffffffL) return AS_BAD_SHAPE;
  const int pass = compute_units();
  const PrefillSplit split{pieces, piece_rounds, cut, part_ml, part_acc};
#define LAUNCH(DCV)                                                                                   \
  if (query_tiles == 1) {                                                                             \
    attn_prefill_mfma_kernel<DCV, 1><<<(int)blocks, 256, 0, stream>>>(                                \
        (const bf16*)q, (const bf16*)k_pages, (const bf16*)v_pages, tiles, block_tables, table_width, \
        (bf16*)out, H, KV, bs, scale, window, units_z, pass, split);                                  \
    if (pieces > 1)                                                                                   \
      attn_prefill_merge_kernel<DCV, 1><<<(int)items, 256, 0, stream>>>(tiles, (bf16*)out, H, KV, units_z, split); \
  } else {                                                                                            \
    attn_prefill_mfma_kernel<DCV, 2><<<(int)blocks, 256, 0, stream>>>(                                \
        (const bf16*)q, (const bf16*)k_pages, (const bf16*)v_pages, tiles, block_tables, table_width, \
        (bf16*)out, H, KV, bs, scale, window, units_z, pass, split);                                  \
    if (pieces > 1)                                                                                   \
      attn_prefill_merge_kernel<DCV, 2><<<(int)items, 256, 0, stream>>>(tiles, (bf16*)out, H, KV, units_z, split); \
  }
  switch (D / 32) {
    case 1: LAUNCH(1); break;
    case 2: LAUNCH(2); break;
    case 3: LAUNCH(3); break;
    case 4: LAUNCH(4); break;
    case 5: LAUNCH(5); break;
    case 6: LAUNCH(6); break;
    case 7: LAUNCH(7); break;
    default: LAUNCH(8); break;
  }
#undef LAUNCH
  return launch_status();
}

static int launch_decode_mfma(const void* q, const void* k_pages, const void* v_pages, const int* items,
                              int num_items, const int* positions, const int* tok_row, const int* block_tables,
                              int table_width, void* out, float* part_m, float* part_l, float* part_acc, int H,
                              int KV, int D, int bs, float scale, int window, int part_size, int P,
                              const FreshQKV* fresh, int gains_dtype, hipStream_t stream) {
  const int G = H / KV;
  if (D % 32 || D > 256 || G > 16 || bs % 16 || part_size % 32) return AS_BAD_SHAPE;
  if (fresh && D % 64) return AS_BAD_SHAPE;
  dim3 grid(num_items, KV, P);
  const size_t shmem = sizeof(float) * (size_t)(128 + 4 * D * G);
  if (shmem + 1024 > (64u << 10)) return AS_BAD_SHAPE;  // wide heads in large groups: the general kernel's
  const FreshQKV none = {};
#define LAUNCH(DCV, FRESHV)                                                                               \
  attn_decode_mfma_kernel<DCV, FRESHV><<<grid, 256, shmem, stream>>>(                                     \
      (const bf16*)q, (const bf16*)k_pages, (const bf16*)v_pages, items, positions, tok_row, block_tables, \
      table_width, (bf16*)out, part_m, part_l, part_acc, H, KV, bs, scale, window, part_size, P,          \
      compute_units(), FRESHV ? *fresh : none)
#define LAUNCH_FRESH(FRESHV)            \
  switch (D / 64) {                     \
    case 1: LAUNCH(2, FRESHV); break;   \
    case 2: LAUNCH(4, FRESHV); break;   \
    case 3: LAUNCH(6, FRESHV); break;   \
    default: LAUNCH(8, FRESHV); break;  \
  }
  if (fresh && gains_dtype == DT_F32) {
    LAUNCH_FRESH(2)
  } else if (fresh) {
    LAUNCH_FRESH(1)
  } else {
    switch (D / 32) {
      case 1: LAUNCH(1, 0); break;
      case 2: LAUNCH(2, 0); break;
      case 3: LAUNCH(3, 0); break;
      case 4: LAUNCH(4, 0); break;
      case 5: LAUNCH(5, 0); break;
      case 6: LAUNCH(6, 0); break;
      case 7: LAUNCH(7, 0); break;
      default: LAUNCH(8, 0); break;
    }
  }
#undef LAUNCH_FRESH
#undef LAUNCH
  if (hipGetLastError() != hipSuccess) return AS_LAUNCH_FAILED;
  if (P > 1) {
    attn_reduce_kernel<bf16><<<dim3(num_items, H), D <= 64 ? 64 : (D <= 128 ? 128 : 256), 0, stream>>>(
        items, part_m, part_l, part_acc, (bf16*)out, H, D, P);
  }
  return launch_status();
}

// Same contract as as_attn_single_query, bf16 only, through the matrix cores.
extern "C" int as_attn_decode_mfma(const void* q, const void* k_pages, const void* v_pages, const int* items,
                                   int num_items, const int* positions, const int* tok_row,
                                   const int* block_tables, int table_width, void* out, float* part_m,
                                   float* part_l, float* part_acc, int H, int KV, int D, int bs, float scale,
                                   int window, int part_size, int P, hipStream_t stream) {
  if (num_items <= 0) return AS_OK;
  if (H <= 0 || KV <= 0 || H % KV || D <= 0 || bs <= 0 || part_size <= 0 || P <= 0 || table_width <= 0)
    return AS_BAD_SHAPE;
  if (P > 1 && (!part_m || !part_l || !part_acc)) return AS_BAD_SHAPE;
  return launch_decode_mfma(q, k_pages, v_pages, items, num_items, positions, tok_row, block_tables, table_width,
                            out, part_m, part_l, part_acc, H, KV, D, bs, scale, window, part_size, P, nullptr,
                            DT_BF16, stream);
}

// A decode step (token t is row t of the block tables) from the projection's output: per-head norm,
// rotation of the whole head, the new token's key and value written to its slot (store 0: queries
// only, the pages already hold them), and attention, in one kernel.  qkv [T, H + 2 KV, D] bf16;
// qw, kw [D] bf16 or fp32; cs [T, D/2] float2; slots [T]; items [T]: the order in which the tokens are
// taken (null: as they come), best the longest contexts first.  Needs D % 64 == 0.
extern "C" int as_attn_decode_fresh(const void* qkv, const void* qw, const void* kw, int gains_dtype,
                                    const float* cs, const int* slots, float eps, int store, void* k_pages,
                                    void* v_pages, const int* items, int num_tokens, const int* positions,
                                    const int* block_tables, int table_width, void* out, float* part_m,
                                    float* part_l, float* part_acc, int H, int KV, int D, int bs, float scale,
                                    int window, int part_size, int P, hipStream_t stream) {
  if (num_tokens <= 0) return AS_OK;
  if (H <= 0 || KV <= 0 || H % KV || D <= 0 || bs <= 0 || part_size <= 0 || P <= 0 || table_width <= 0)
    return AS_BAD_SHAPE;
  if (P > 1 && (!part_m || !part_l || !part_acc)) return AS_BAD_SHAPE;
  if (!qkv || !qw || !kw || !cs || (store && !slots)) return AS_BAD_SHAPE;
  if (gains_dtype != DT_BF16 && gains_dtype != DT_F32) return AS_BAD_DTYPE;
  const FreshQKV fresh = {(const bf16*)qkv, qw, kw, (const float2*)cs, slots, (bf16*)k_pages, (bf16*)v_pages,
                          eps, store};
  return launch_decode_mfma(nullptr, k_pages, v_pages, items, num_tokens, positions, nullptr, block_tables,
                            table_width, out, part_m, part_l, part_acc, H, KV, D, bs, scale, window, part_size,
                            P, &fresh, gains_dtype, stream);
}

static int pow2ceil(int v) { int p = 1; while (p < v) p <<= 1; return p; }

template <typename T>
static int launch_single_query(const void* q, const void* k_pages, const void* v_pages, const int* items,
                               int num_items, const int* positions, const int* tok_row,
                               const int* block_tables, int table_width, void* out, float* part_m,
                               float* part_l, float* part_acc, int H, int KV, int D, int bs, float scale,
                               int window, int part_size, int P, hipStream_t stream) {
  constexpr int CH = Chunk<T>::N;
  if (D % CH != 0 || D > 64 * CH || D > 256) return AS_BAD_SHAPE;
  const int G = H / KV;
  const int lpk = pow2ceil(D / CH);
  const int GT = G >= 8 ? 8 : (G > 2 ? 4 : (G == 2 ? 2 : 1));
  const int HC = (G + GT - 1) / GT;
  dim3 grid(num_items, KV * HC, P);
  const size_t shmem = sizeof(float) * (size_t)(8 * GT + 4 * GT * D);
#define LAUNCH(GTV)                                                                                      \
  attn_single_query_kernel<T, GTV><<<grid, 256, shmem, stream>>>(                                        \
      (const T*)q, (const T*)k_pages, (const T*)v_pages, items, positions, tok_row, block_tables,       \
      table_width, (T*)out, part_m, part_l, part_acc, H, KV, D, bs, scale, window, part_size, P, lpk)
  switch (GT) {
    case 1: LAUNCH(1); break;
    case 2: LAUNCH(2); break;
    case 4: LAUNCH(4); break;
    default: LAUNCH(8); break;
  }
#undef LAUNCH
  if (hipGetLastError() != hipSuccess) return AS_LAUNCH_FAILED;
  if (P > 1) {
    attn_reduce_kernel<T><<<dim3(num_items, H), D <= 64 ? 64 : (D <= 128 ? 128 : 256), 0, stream>>>(
        items, part_m, part_l, part_acc, (T*)out, H, D, P);
  }
  return launch_status();
}

// part_m, part_l: [num_items, H, P] fp32; part_acc: [num_items, H, P, D] fp32 (unused when P == 1).
// P must be >= ceil(max context of the items / part_size).
extern "C" int as_attn_single_query(const void* q, const void* k_pages, const void* v_pages, int dtype,
                                    const int* items, int num_items, const int* positions,
                                    const int* tok_row, const int* block_tables, int table_width, void* out,
                                    float* part_m, float* part_l, float* part_acc, int H, int KV, int D,
                                    int bs, float scale, int window, int part_size, int P,
                                    hipStream_t stream) {
  if (num_items <= 0) return AS_OK;
  if (H <= 0 || KV <= 0 || H % KV || D <= 0 || bs <= 0 || part_size <= 0 || P <= 0 || table_width <= 0)
    return AS_BAD_SHAPE;
  if (P > 1 && (!part_m || !part_l || !part_acc)) return AS_BAD_SHAPE;
  if (dtype == DT_F32)
    return launch_single_query<float>(q, k_pages, v_pages, items, num_items, positions, tok_row, block_tables,
                                      table_width, out, part_m, part_l, part_acc, H, KV, D, bs, scale,
                                      window, part_size, P, stream);
  if (dtype == DT_BF16)
    return launch_single_query<bf16>(q, k_pages, v_pages, items, num_items, positions, tok_row, block_tables,
                                     table_width, out, part_m, part_l, part_acc, H, KV, D, bs, scale, window,
                                     part_size, P, stream);
  return AS_BAD_DTYPE;
}

// ---- the same without scratch buffers from the caller ----------------------------------
//
// The partial results of a split context live in an array of the library's own; see no_alloc.h.
// In host code `scratch` is only a stand-in for the symbol: the address that kernels and copies
// use is the one hipGetSymbolAddress returns, and every GPU has its own.
static __device__ __align__(256) float scratch[AS_STATIC_SCRATCH_FLOATS];
static float* scratch_on_device[64] = {nullptr};

static int scratch_of_current_device(float** ptr) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return AS_LAUNCH_FAILED;
  if (scratch_on_device[dev] == nullptr) {
    void* found = nullptr;
    if (hipGetSymbolAddress(&found, HIP_SYMBOL(scratch)) != hipSuccess || found == nullptr) return AS_LAUNCH_FAILED;
    scratch_on_device[dev] = (float*)found;
  }
  *ptr = scratch_on_device[dev];
  return AS_OK;
}

extern "C" int as_attn_single_query_static(const void* q, const void* k_pages, const void* v_pages, int dtype,
                                           const int* items, int num_items, const int* positions,
                                           const int* tok_row, const int* block_tables, int table_width,
                                           void* out, int H, int KV, int D, int bs, float scale, int window,
                                           int part_size, int P, hipStream_t stream) {
  if (num_items <= 0) return AS_OK;
  if (H <= 0 || KV <= 0 || H % KV || D <= 0 || bs <= 0 || part_size <= 0 || P <= 0 || table_width <= 0)
    return AS_BAD_SHAPE;
  float *part_m = nullptr, *part_l = nullptr, *part_acc = nullptr;
  if (P > 1) {
    const unsigned long long rows = (unsigned long long)num_items * (unsigned long long)H * (unsigned long long)P;
    if (rows > AS_STATIC_SCRATCH_FLOATS || rows * (unsigned long long)(D + 2) > AS_STATIC_SCRATCH_FLOATS)
      return AS_TOO_LARGE;
    float* base = nullptr;
    const int status = scratch_of_current_device(&base);
    if (status != AS_OK) return status;
    part_acc = base;  // [rows, D]: first, so that it keeps the array's alignment
    part_m = base + rows * D;
    part_l = part_m + rows;
  }
  return as_attn_single_query(q, k_pages, v_pages, dtype, items, num_items, positions, tok_row, block_tables,
                              table_width, out, part_m, part_l, part_acc, H, KV, D, bs, scale, window,
                              part_size, P, stream);
}
