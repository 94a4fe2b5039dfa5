// Row-wise kernels of the decoder: embedding lookup, RMSNorm with the residual sum
// fused in, the rotary table, per-head q/k norm + rotation + cache store, and the
// gated activation.  All arithmetic is fp32; storage is fp32 or bf16.
#include "common.h"

// ---- embedding --------------------------------------------------------------------
// out[t, :] = scale * table[ids[t], :] as fp32 (the residual stream is always fp32; the scale is 1
// for models that do not multiply their embeddings).
// Plain reference: reference atomserve/model.py:373.
template <typename T>
__global__ void embed_gather_kernel(const T* __restrict__ table, const int* __restrict__ ids,
                                    float* __restrict__ out, int width, int vocab, float scale) {
  const int t = blockIdx.x;
  int id = ids[t];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);  // ids are validated on the host; never read outside
  const T* src = table + (size_t)id * width;
  float* dst = out + (size_t)t * width;
  for (int i = threadIdx.x; i < width; i += blockDim.x) dst[i] = to_f32(src[i]) * scale;
}

extern "C" int as_embed_gather(const void* table, int table_dtype, const int* ids, float* out,
                               int num_tokens, int width, int vocab, float scale, hipStream_t stream) {
  if (num_tokens <= 0) return AS_OK;
  if (width <= 0 || vocab <= 0) return AS_BAD_SHAPE;
  const int threads = width >= 1024 ? 256 : 64;
  if (table_dtype == DT_F32)
    embed_gather_kernel<float><<<num_tokens, threads, 0, stream>>>((const float*)table, ids, out, width, vocab, scale);
  else if (table_dtype == DT_BF16)
    embed_gather_kernel<bf16><<<num_tokens, threads, 0, stream>>>((const bf16*)table, ids, out, width, vocab, scale);
  else
    return AS_BAD_DTYPE;
  return launch_status();
}

// ---- what a head may still do to its logits ------------------------------------------
// logits = cap * tanh(scale * logits / cap) (cap 0: only the scale), in place, fp32.  Qwen3 does
// neither (reference atomserve/model.py:405-415); the decoder launches this only for a plan that
// names a scale or a cap.
__global__ void logits_finish_kernel(float* __restrict__ logits, size_t count, float scale, float cap) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += stride) {
    const float v = logits[i] * scale;
    logits[i] = cap > 0.f ? cap * tanhf(v / cap) : v;
  }
}

extern "C" int as_logits_finish(float* logits, long long count, float scale, float cap, hipStream_t stream) {
  if (count <= 0) return AS_OK;
  if (cap < 0.f) return AS_BAD_SHAPE;
  const long long blocks = (count + 255) / 256;
  logits_finish_kernel<<<(int)(blocks < 2048 ? blocks : 2048), 256, 0, stream>>>(logits, (size_t)count, scale, cap);
  return launch_status();
}

// ---- RMSNorm with fused residual sum and row selection --------------------------
// For output row r (source row s = rows ? rows[r] : r):
//   v = x[s] + (delta ? delta[s] : 0)          in fp32; written back to x[s] if update_x
//   out[r] = v / sqrt(mean(v^2) + eps) * w     rounded once
// Plain reference: reference atomserve/model.py:125-139 (weight multiplies directly).
//
// The pending sum may also arrive as the partial sums of a matrix product whose K was cut into
// `splits` ranges (SplitDelta: fp32 [splits, rows, n]): they are added in the order of the ranges
// and rounded to O once, which is what the product alone would have stored.
struct SplitDelta {
  const float* sums;  // null: none
  int splits;
  size_t stride;  // elements from one range's sums to the next: rows * n
};

template <typename O>
__device__ __forceinline__ float split_delta(const SplitDelta& sd, size_t at) {
  float d = sd.sums[at];
  for (int k = 1; k < sd.splits; ++k) d += sd.sums[(size_t)k * sd.stride + at];
  return to_f32(from_f32<O>(d));
}

template <typename O, typename W>
__global__ void rmsnorm_kernel(float* __restrict__ x, const O* __restrict__ delta,
                               const int* __restrict__ rows, const W* __restrict__ w, float eps,
                               O* __restrict__ out, int n, int update_x, SplitDelta sd) {
  __shared__ float red[17];
  const int r = blockIdx.x;
  const size_t s = rows ? (size_t)rows[r] : (size_t)r;
  float* xr = x + s * n;
  const O* dr = delta ? delta + s * n : nullptr;
  const bool pending = dr || sd.sums;
  float ss = 0.f;
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    float v = xr[i];
    if (pending) {
      v += dr ? to_f32(dr[i]) : split_delta<O>(sd, s * n + i);
      if (update_x) xr[i] = v;
    }
    ss += v * v;
  }
  ss = block_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)n + eps);
  O* o = out + (size_t)r * n;
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    float v = xr[i];  // the thread's own earlier store, if any, is what it reads back
    if (pending && !update_x) v += dr ? to_f32(dr[i]) : split_delta<O>(sd, s * n + i);
    o[i] = from_f32<O>(v * inv * to_f32(w[i]));
  }
}

// The same with 16-byte accesses and the row kept in registers between the two passes:
// every load of a row is in flight at once, which is what a decode step (few rows) needs.
// Requires n % 4 == 0 and n <= 4 * blockDim.x * RN_CHUNKS.
#define RN_CHUNKS 4
template <typename T> struct Vec4;
template <> struct Vec4<float> {
  static __device__ __forceinline__ float4 load(const float* p) { return *reinterpret_cast<const float4*>(p); }
  static __device__ __forceinline__ void store(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
};
template <> struct Vec4<bf16> {
  typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
  static __device__ __forceinline__ float4 load(const bf16* p) {
    const bf16x4 r = *reinterpret_cast<const bf16x4*>(p);
    return make_float4((float)r[0], (float)r[1], (float)r[2], (float)r[3]);
  }
  static __device__ __forceinline__ void store(bf16* p, float4 v) {
    const bf16x4 r = {(bf16)v.x, (bf16)v.y, (bf16)v.z, (bf16)v.w};
    *reinterpret_cast<bf16x4*>(p) = r;
  }
};

template <typename O, typename W>
__global__ __launch_bounds__(1024) void rmsnorm_vec_kernel(float* __restrict__ x, const O* __restrict__ delta,
                                                           const int* __restrict__ rows,
                                                           const W* __restrict__ w, float eps,
                                                           O* __restrict__ out, int n, int update_x,
                                                           SplitDelta sd) {
  __shared__ float red[17];
  const int r = blockIdx.x;
  const size_t s = rows ? (size_t)rows[r] : (size_t)r;
  float* xr = x + s * n;
  const O* dr = delta ? delta + s * n : nullptr;
  const int chunks = n >> 2;
  float4 v[RN_CHUNKS];
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < RN_CHUNKS; ++j) {
    const int c = threadIdx.x + j * blockDim.x;
    if (c < chunks) {
      v[j] = Vec4<float>::load(xr + 4 * c);
      if (dr || sd.sums) {
        float4 d;
        if (dr) {
          d = Vec4<O>::load(dr + 4 * c);
        } else {
          const float* p = sd.sums + s * n + 4 * c;
          d = Vec4<float>::load(p);
          for (int k = 1; k < sd.splits; ++k) {
            const float4 e = Vec4<float>::load(p + (size_t)k * sd.stride);
            d.x += e.x; d.y += e.y; d.z += e.z; d.w += e.w;
          }
          d = make_float4(to_f32(from_f32<O>(d.x)), to_f32(from_f32<O>(d.y)), to_f32(from_f32<O>(d.z)),
                          to_f32(from_f32<O>(d.w)));
        }
        v[j].x += d.x; v[j].y += d.y; v[j].z += d.z; v[j].w += d.w;
        if (update_x) Vec4<float>::store(xr + 4 * c, v[j]);
      }
      ss += v[j].x * v[j].x + v[j].y * v[j].y + v[j].z * v[j].z + v[j].w * v[j].w;
    }
  }
  ss = block_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)n + eps);
  O* o = out + (size_t)r * n;
#pragma unroll
  for (int j = 0; j < RN_CHUNKS; ++j) {
    const int c = threadIdx.x + j * blockDim.x;
    if (c < chunks) {
      const float4 g = Vec4<W>::load(w + 4 * c);
      Vec4<O>::store(o + 4 * c, make_float4(v[j].x * inv * g.x, v[j].y * inv * g.y, v[j].z * inv * g.z, v[j].w * inv * g.w));
    }
  }
}

static int launch_rmsnorm(float* x, const void* delta, const SplitDelta& sd, const int* rows, const void* w,
                          int w_dtype, float eps, void* out, int out_dtype, int num_out_rows, int n, int update_x,
                          hipStream_t stream) {
  if (num_out_rows <= 0) return AS_OK;
  if (n <= 0) return AS_BAD_SHAPE;
  const bool vec = (n & 3) == 0 && n <= 4 * 1024 * RN_CHUNKS;
  int threads = n >= 2048 ? 256 : (n >= 512 ? 128 : 64);
  if (vec) {
    // few rows: one chunk per thread, all loads in flight; many rows: fewer, fuller threads
    const int chunks = n >> 2, per_thread = num_out_rows >= 512 ? RN_CHUNKS : 1;
    threads = (chunks + per_thread - 1) / per_thread;
    threads = ((threads + 63) / 64) * 64;
    if (threads > 1024) threads = 1024;
  }
#define LAUNCH(O, W)                                                                               \
  do {                                                                                             \
    if (vec)                                                                                       \
      rmsnorm_vec_kernel<O, W><<<num_out_rows, threads, 0, stream>>>(x, (const O*)delta, rows, (const W*)w, eps, \
                                                                     (O*)out, n, update_x, sd);    \
    else                                                                                           \
      rmsnorm_kernel<O, W><<<num_out_rows, threads, 0, stream>>>(x, (const O*)delta, rows, (const W*)w, eps,     \
                                                                 (O*)out, n, update_x, sd);        \
  } while (0)
  if (out_dtype == DT_F32 && w_dtype == DT_F32) LAUNCH(float, float);
  else if (out_dtype == DT_BF16 && w_dtype == DT_BF16) LAUNCH(bf16, bf16);
  else if (out_dtype == DT_BF16 && w_dtype == DT_F32) LAUNCH(bf16, float);
  else return AS_BAD_DTYPE;
#undef LAUNCH
  return launch_status();
}

extern "C" int as_rmsnorm(float* x, const void* delta, const int* rows, const void* w, int w_dtype,
                          float eps, void* out, int out_dtype, int num_out_rows, int n, int update_x,
                          hipStream_t stream) {
  return launch_rmsnorm(x, delta, SplitDelta{nullptr, 0, 0}, rows, w, w_dtype, eps, out, out_dtype, num_out_rows, n,
                        update_x, stream);
}

// The same with the pending sum given as the partial sums [splits, num_rows, n] (fp32) of a product
// whose K was cut into ranges; num_rows counts the rows of x.
extern "C" int as_rmsnorm_split(float* x, const float* sums, int splits, int num_rows, const int* rows, const void* w,
                                int w_dtype, float eps, void* out, int out_dtype, int num_out_rows, int n,
                                int update_x, hipStream_t stream) {
  if (!sums || splits <= 0 || num_rows <= 0) return AS_BAD_SHAPE;
  return launch_rmsnorm(x, nullptr, SplitDelta{sums, splits, (size_t)num_rows * n}, rows, w, w_dtype, eps, out,
                        out_dtype, num_out_rows, n, update_x, stream);
}

// ---- rotary table -------------------------------------------------------------------
// cs[t, i] = (cos, sin)(positions[t] * inv_freq[i]), i < half.  The product and the
// range reduction are done in fp64 so that large positions keep fp32-exact angles;
// the rotation itself is fp32.  Plain reference: reference atomserve/model.py:142-169.
__global__ void rope_table_kernel(const int* __restrict__ positions, const double* __restrict__ inv_freq,
                                  float2* __restrict__ cs, int num_tokens, int half) {
  const int idx = blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= num_tokens * half) return;
  const int t = idx / half, i = idx % half;
  const double a = (double)positions[t] * inv_freq[i];
  double s, c;
  sincos(a, &s, &c);
  cs[idx] = make_float2((float)c, (float)s);
}

extern "C" int as_rope_table(const int* positions, const double* inv_freq, float* cs, int num_tokens,
                             int half, hipStream_t stream) {
  if (num_tokens <= 0) return AS_OK;
  if (half <= 0) return AS_BAD_SHAPE;
  const int total = num_tokens * half;
  rope_table_kernel<<<(total + 255) / 256, 256, 0, stream>>>(positions, inv_freq, (float2*)cs, num_tokens, half);
  return launch_status();
}

// ---- per-head q/k norm + rotation + cache store -----------------------------------
// One wave per (token, head slot) of qkv [T, H + 2 KV, D].  q and k heads: optional
// RMSNorm over the head's D values with gains qw / kw, then rotation of the pairs
// (i, i + R/2), i < R/2, by the token's angle; coordinates >= R pass unrotated.
// q goes to q_out [T, H, D]; k goes to k_pages [num_pages, KV, bs, D] and v, copied as it
// is, to v_pages [num_pages, KV, D, bs] (each page of values is stored transposed, so that
// the keys of one coordinate are contiguous), at slot = page * bs + offset.
// store_kv = 0 computes q only.
// Plain reference: reference atomserve/kernels.py:74-145, atomserve/model.py:326-333.
template <typename O, typename W>
__global__ void qk_norm_rope_store_kernel(const O* __restrict__ qkv, const W* __restrict__ qw,
                                          const W* __restrict__ kw, const float2* __restrict__ cs,
                                          const int* __restrict__ slots, O* __restrict__ q_out,
                                          O* __restrict__ k_pages, O* __restrict__ v_pages, int H, int KV,
                                          int D, int R, float eps, int block_size) {
  const int t = blockIdx.x, hs = blockIdx.y, lane = threadIdx.x;
  const O* src = qkv + ((size_t)t * (H + 2 * KV) + hs) * D;
  const bool is_q = hs < H, is_k = !is_q && hs < H + KV;
  O* dst;
  if (is_q) {
    dst = q_out + ((size_t)t * H + hs) * D;
  } else {
    const int slot = slots[t];
    if (slot < 0) return;  // this token's keys are not stored (whole wave returns)
    const int kvh = is_k ? hs - H : hs - H - KV;
    const size_t head = (size_t)(slot / block_size) * KV + kvh;
    if (!is_k) {  // values: transposed within the page
      O* vt = v_pages + head * block_size * D + slot % block_size;
      for (int i = lane; i < D; i += WAVE) vt[(size_t)i * block_size] = finite_or_zero(src[i]);
      return;
    }
    dst = k_pages + (head * block_size + slot % block_size) * D;
  }
  const W* w = is_q ? qw : kw;
  float inv = 1.0f;
  if (w) {
    float ss = 0.f;
    for (int i = lane; i < D; i += WAVE) { const float v = to_f32(src[i]); ss += v * v; }
    ss = wave_sum(ss);
    inv = 1.0f / sqrtf(ss / (float)D + eps);
  }
  const int half = R / 2;
  for (int i = lane; i < half; i += WAVE) {
    float a = to_f32(src[i]) * inv, b = to_f32(src[i + half]) * inv;
    if (w) { a *= to_f32(w[i]); b *= to_f32(w[i + half]); }
    float c = 1.f, s = 0.f;
    if (cs) { const float2 v = cs[(size_t)t * half + i]; c = v.x; s = v.y; }
    const O ra = from_f32<O>(a * c - b * s), rb = from_f32<O>(b * c + a * s);
    dst[i] = is_k ? finite_or_zero(ra) : ra;
    dst[i + half] = is_k ? finite_or_zero(rb) : rb;
  }
  for (int i = R + lane; i < D; i += WAVE) {
    float a = to_f32(src[i]) * inv;
    if (w) a *= to_f32(w[i]);
    const O ra = from_f32<O>(a);
    dst[i] = is_k ? finite_or_zero(ra) : ra;
  }
}

// The same for bf16 heads that are rotated whole (R == D) and whose width is 16 times a power
// of two: a group of D / 16 lanes owns one (token, head) and every lane moves 16-byte pieces
// (coordinates 8l .. 8l+7 and their partners in the other half), so a wave serves several
// heads at once and a prompt's rows move at memory speed.  Same arithmetic, same order.
template <typename W> struct Gain8;
template <> struct Gain8<bf16> {
  static __device__ __forceinline__ void load(const bf16* p, float* g) {
    typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
    const bf16x8 v = *reinterpret_cast<const bf16x8*>(p);
#pragma unroll
    for (int j = 0; j < 8; ++j) g[j] = (float)v[j];
  }
};
template <> struct Gain8<float> {
  static __device__ __forceinline__ void load(const float* p, float* g) {
    const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
    g[0] = a.x; g[1] = a.y; g[2] = a.z; g[3] = a.w; g[4] = b.x; g[5] = b.y; g[6] = b.z; g[7] = b.w;
  }
};

template <typename W>
__global__ __launch_bounds__(256) void qk_norm_rope_store_bf16x8_kernel(
    const bf16* __restrict__ qkv, const W* __restrict__ qw, const W* __restrict__ kw,
    const float2* __restrict__ cs, const int* __restrict__ slots, bf16* __restrict__ q_out,
    bf16* __restrict__ k_pages, bf16* __restrict__ v_pages, int H, int KV, int D, float eps, int block_size,
    int heads, size_t units) {
  typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
  const int lpu = D >> 4, half = D >> 1;  // lanes per (token, head)
  const size_t unit = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) / lpu;
  const int l = threadIdx.x & (lpu - 1);
  if (unit >= units) return;  // whole groups leave: the shuffles below stay inside a group
  const size_t t = unit / heads;
  const int hs = (int)(unit % heads);
  const bf16* src = qkv + (t * (H + 2 * KV) + hs) * D;
  const bool is_q = hs < H, is_k = !is_q && hs < H + KV;
  bf16* dst;
  if (!is_q && !is_k) {  // values: transposed within the page
    const int slot = slots[t];
    if (slot < 0) return;  // uniform over the group
    const size_t head = (size_t)(slot / block_size) * KV + (hs - H - KV);
    // A prompt's tokens fill a page slot after slot.  Where eight tokens in a row go to eight
    // slots in a row that start at a multiple of eight, a coordinate's eight values are 16
    // contiguous bytes of the transposed page, where token by token they would be eight stores
    // of two bytes, 2 * block_size bytes apart.  The eight tokens' lane groups share that work:
    // each takes an eighth of the coordinates, two per lane, reads them from all eight tokens'
    // rows and stores two 16-byte pieces.
    const int nth = slot & 7;
    const long lead = (long)t - nth;
    bool run = (block_size & 7) == 0 && lead >= 0 && lead + 8 <= (long)(units / heads);
    if (run) {
#pragma unroll
      for (int i = 0; i < 8; ++i) run = run && slots[lead + i] == slot - nth + i;
    }
    if (run) {  // uniform over the lanes of this (token, head), and the same for all eight tokens
      typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
      const int d0 = nth * (D >> 3) + 2 * l;
      const bf16* first = qkv + ((size_t)lead * (H + 2 * KV) + hs) * D + d0;
      bf16x2 pair[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) pair[i] = *reinterpret_cast<const bf16x2*>(first + (size_t)i * (H + 2 * KV) * D);
      bf16x8 oa, ob;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        oa[i] = finite_or_zero((bf16)pair[i][0]);
        ob[i] = finite_or_zero((bf16)pair[i][1]);
      }
      bf16* vt = v_pages + head * block_size * D + (slot - nth) % block_size;
      *reinterpret_cast<bf16x8*>(vt + (size_t)d0 * block_size) = oa;
      *reinterpret_cast<bf16x8*>(vt + (size_t)(d0 + 1) * block_size) = ob;
      return;
    }
    const bf16x8 a8 = *reinterpret_cast<const bf16x8*>(src + 8 * l);
    const bf16x8 b8 = *reinterpret_cast<const bf16x8*>(src + half + 8 * l);
    bf16* vt = v_pages + head * block_size * D + slot % block_size;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      vt[(size_t)(8 * l + j) * block_size] = finite_or_zero((bf16)a8[j]);
      vt[(size_t)(half + 8 * l + j) * block_size] = finite_or_zero((bf16)b8[j]);
    }
    return;
  }
  const bf16x8 a8 = *reinterpret_cast<const bf16x8*>(src + 8 * l);
  const bf16x8 b8 = *reinterpret_cast<const bf16x8*>(src + half + 8 * l);
  if (is_q) {
    dst = q_out + (t * H + hs) * D;
  } else {
    const int slot = slots[t];
    if (slot < 0) return;  // uniform over the group
    const size_t head = (size_t)(slot / block_size) * KV + (hs - H);
    dst = k_pages + (head * block_size + slot % block_size) * D;
  }
  const W* w = is_q ? qw : kw;
  float inv = 1.0f;
  if (w) {
    float ss = 0.f;
    // the generic kernel's order within a lane differs; the sum over D squares is the same up to rounding
#pragma unroll
    for (int j = 0; j < 8; ++j) ss += (float)a8[j] * (float)a8[j];
#pragma unroll
    for (int j = 0; j < 8; ++j) ss += (float)b8[j] * (float)b8[j];
    for (int off = 1; off < lpu; off <<= 1) ss += __shfl_xor(ss, off, WAVE);
    inv = 1.0f / sqrtf(ss / (float)D + eps);
  }
  float ga[8], gb[8];
  if (w) {
    Gain8<W>::load(w + 8 * l, ga);
    Gain8<W>::load(w + half + 8 * l, gb);
  }
  // the angles of this lane's eight pairs: 64 contiguous bytes, four loads
  float4 turn[4];
  if (cs) {
    const float4* cs4 = reinterpret_cast<const float4*>(cs + t * half + 8 * l);
#pragma unroll
    for (int j = 0; j < 4; ++j) turn[j] = cs4[j];
  }
  bf16x8 oa, ob;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    float a = (float)a8[j] * inv, b = (float)b8[j] * inv;
    if (w) { a *= ga[j]; b *= gb[j]; }
    float c = 1.f, sn = 0.f;
    if (cs) { c = (j & 1) ? turn[j >> 1].z : turn[j >> 1].x; sn = (j & 1) ? turn[j >> 1].w : turn[j >> 1].y; }
    oa[j] = (bf16)(a * c - b * sn);
    ob[j] = (bf16)(b * c + a * sn);
    if (is_k) { oa[j] = finite_or_zero((bf16)oa[j]); ob[j] = finite_or_zero((bf16)ob[j]); }
  }
  *reinterpret_cast<bf16x8*>(dst + 8 * l) = oa;
  *reinterpret_cast<bf16x8*>(dst + half + 8 * l) = ob;
}

extern "C" int as_qk_norm_rope_store(const void* qkv, int dtype, const void* qw, const void* kw, int w_dtype,
                                     const float* cs, const int* slots, void* q_out, void* k_pages,
                                     void* v_pages, int num_tokens, int H, int KV, int D, int R, float eps,
                                     int block_size, int store_kv, hipStream_t stream) {
  if (num_tokens <= 0) return AS_OK;
  if (H <= 0 || KV <= 0 || D <= 0 || R < 0 || R > D || (R & 1) || block_size <= 0) return AS_BAD_SHAPE;
  if ((qw == nullptr) != (kw == nullptr)) return AS_BAD_SHAPE;
  const int lpu = D >> 4;
  if (dtype == DT_BF16 && R == D && (D & 15) == 0 && lpu <= WAVE && (lpu & (lpu - 1)) == 0) {
    const int heads = store_kv ? H + 2 * KV : H;
    const size_t units = (size_t)num_tokens * heads;
    const size_t blocks = (units * lpu + 255) / 256;
    if (blocks > 0x7fffffff) return AS_BAD_SHAPE;
#define LAUNCH8(W)                                                                                   \
  qk_norm_rope_store_bf16x8_kernel<W><<<(int)blocks, 256, 0, stream>>>(                              \
      (const bf16*)qkv, (const W*)qw, (const W*)kw, (const float2*)cs, slots, (bf16*)q_out,          \
      (bf16*)k_pages, (bf16*)v_pages, H, KV, D, eps, block_size, heads, units)
    if (w_dtype == DT_BF16) LAUNCH8(bf16);
    else if (w_dtype == DT_F32) LAUNCH8(float);
    else return AS_BAD_DTYPE;
#undef LAUNCH8
    return launch_status();
  }
  dim3 grid(num_tokens, store_kv ? H + 2 * KV : H);
#define LAUNCH(O, W)                                                                                   \
  qk_norm_rope_store_kernel<O, W><<<grid, WAVE, 0, stream>>>(                                          \
      (const O*)qkv, (const W*)qw, (const W*)kw, (const float2*)cs, slots, (O*)q_out, (O*)k_pages,    \
      (O*)v_pages, H, KV, D, R, eps, block_size)
  if (dtype == DT_F32 && w_dtype == DT_F32) LAUNCH(float, float);
  else if (dtype == DT_BF16 && w_dtype == DT_BF16) LAUNCH(bf16, bf16);
  else if (dtype == DT_BF16 && w_dtype == DT_F32) LAUNCH(bf16, float);
  else return AS_BAD_DTYPE;
#undef LAUNCH
  return launch_status();
}

// ---- gated activation -----------------------------------------------------------
// out[t, i] = silu(gu[t, i]) * gu[t, I + i], silu(g) = g / (1 + exp(-g)).
// Plain reference: reference atomserve/kernels.py:439-449, atomserve/model.py:358-359.
template <typename O>
__global__ void silu_mul_kernel(const O* __restrict__ gu, O* __restrict__ out, int inter, size_t total) {
  for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (size_t)gridDim.x * blockDim.x) {
    const size_t t = idx / inter;
    const int i = (int)(idx % inter);
    const float g = to_f32(gu[t * 2 * inter + i]);
    const float u = to_f32(gu[t * 2 * inter + inter + i]);
    out[idx] = from_f32<O>(g / (1.0f + expf(-g)) * u);
  }
}

// The same for bf16 rows whose width is a multiple of 8: 16-byte loads and stores, which is
// what a prompt's thousands of rows need to move at memory speed.
__global__ __launch_bounds__(256) void silu_mul_bf16x8_kernel(const bf16* __restrict__ gu, bf16* __restrict__ out,
                                                              int inter, size_t chunks) {
  typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
  const int per_row = inter >> 3;
  for (size_t c = (size_t)blockIdx.x * blockDim.x + threadIdx.x; c < chunks; c += (size_t)gridDim.x * blockDim.x) {
    const size_t t = c / per_row;
    const int i = (int)(c % per_row) * 8;
    const bf16x8 g8 = *reinterpret_cast<const bf16x8*>(gu + t * 2 * inter + i);
    const bf16x8 u8 = *reinterpret_cast<const bf16x8*>(gu + t * 2 * inter + inter + i);
    bf16x8 o8;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float g = (float)g8[j];
      o8[j] = (bf16)(g / (1.0f + expf(-g)) * (float)u8[j]);
    }
    *reinterpret_cast<bf16x8*>(out + t * inter + i) = o8;
  }
}

extern "C" int as_silu_mul(const void* gate_up, void* out, int dtype, int num_tokens, int inter,
                           hipStream_t stream) {
  if (num_tokens <= 0) return AS_OK;
  if (inter <= 0) return AS_BAD_SHAPE;
  const size_t total = (size_t)num_tokens * inter;
  const size_t want = (total + 255) / 256;
  const int blocks = (int)(want > 8192 ? 8192 : want);
  if (dtype == DT_BF16 && (inter & 7) == 0) {
    const size_t chunks = total >> 3, want8 = (chunks + 255) / 256;
    silu_mul_bf16x8_kernel<<<(int)(want8 > 16384 ? 16384 : want8), 256, 0, stream>>>((const bf16*)gate_up, (bf16*)out,
                                                                                    inter, chunks);
    return launch_status();
  }
  if (dtype == DT_F32) silu_mul_kernel<float><<<blocks, 256, 0, stream>>>((const float*)gate_up, (float*)out, inter, total);
  else if (dtype == DT_BF16) silu_mul_kernel<bf16><<<blocks, 256, 0, stream>>>((const bf16*)gate_up, (bf16*)out, inter, total);
  else return AS_BAD_DTYPE;
  return launch_status();
}
