// Matrix products out[M, N] = a[M, K] @ w[N, K]^T (weights keep the checkpoint's
// [out, in] layout).
//
// gemm_f32: genuine fp32 multiply-add on the vector ALU, no matrix-core mode of
// reduced precision.  Every output element is one fma chain over k = 0..K-1 in order,
// so a row's result does not depend on which other rows share the launch.
// Plain reference: reference atomserve/quant.py:89-91 (F.linear).
#include "common.h"

#define BM 64
#define BN 64
#define BK 16

__global__ __launch_bounds__(256) void gemm_f32_kernel(const float* __restrict__ a, const float* __restrict__ w,
                                                       float* __restrict__ out, int M, int N, int K) {
  __shared__ float as[BK][BM + 4];
  __shared__ float ws[BK][BN + 4];
  const int tid = threadIdx.x;
  const int tx = tid & 15, ty = tid >> 4;  // 16 x 16 threads, 4 x 4 outputs each
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  const int lr = tid >> 2, lk = (tid & 3) * 4;  // this thread loads 4 consecutive k of row lr
  float acc[4][4] = {};
  const bool vec = (K & 3) == 0;
  for (int kb = 0; kb < K; kb += BK) {
    float av[4] = {0.f, 0.f, 0.f, 0.f}, wv[4] = {0.f, 0.f, 0.f, 0.f};
    const int k = kb + lk;
    if (m0 + lr < M) {
      const float* p = a + (size_t)(m0 + lr) * K + k;
      if (vec && k + 3 < K) { const float4 r = *reinterpret_cast<const float4*>(p); av[0] = r.x; av[1] = r.y; av[2] = r.z; av[3] = r.w; }
      else { for (int i = 0; i < 4; ++i) if (k + i < K) av[i] = p[i]; }
    }
    if (n0 + lr < N) {
      const float* p = w + (size_t)(n0 + lr) * K + k;
      if (vec && k + 3 < K) { const float4 r = *reinterpret_cast<const float4*>(p); wv[0] = r.x; wv[1] = r.y; wv[2] = r.z; wv[3] = r.w; }
      else { for (int i = 0; i < 4; ++i) if (k + i < K) wv[i] = p[i]; }
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; ++i) { as[lk + i][lr] = av[i]; ws[lk + i][lr] = wv[i]; }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < BK; ++kk) {
      float ar[4], wr[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) { ar[i] = as[kk][ty * 4 + i]; wr[i] = ws[kk][tx * 4 + i]; }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int jn = 0; jn < 4; ++jn) acc[i][jn] = fmaf(ar[i], wr[jn], acc[i][jn]);
    }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int jn = 0; jn < 4; ++jn) {
      const int n = n0 + tx * 4 + jn;
      if (n < N) out[(size_t)m * N + n] = acc[i][jn];
    }
  }
}

extern "C" int as_gemm_f32(const float* a, const float* w, float* out, int M, int N, int K, hipStream_t stream) {
  if (M <= 0) return AS_OK;
  if (N <= 0 || K <= 0) return AS_BAD_SHAPE;
  dim3 grid((N + BN - 1) / BN, (M + BM - 1) / BM);
  if (grid.y > 65535) return AS_BAD_SHAPE;
  gemm_f32_kernel<<<grid, 256, 0, stream>>>(a, w, out, M, N, K);
  return launch_status();
}

// ---- bf16, few rows (decode): weights stream once from HBM through the matrix cores ----
//
// out[M, N] = a[M, K] @ w[N, K]^T for M <= 64, bf16 inputs, fp32 accumulation, bf16 or
// fp32 output.  The product is memory-bound on w, so the kernel is built around reading
// w exactly once with wide loads:
//   * a workgroup (8 waves) owns 16*S consecutive rows of w, i.e. one contiguous region;
//     its waves split K among themselves and their partial sums meet in LDS, added in a
//     fixed order;
//   * w is the A operand of v_mfma_f32_16x16x32_bf16 (rows of w = rows of the tile), the
//     activations are the B operand, so a lane's 4 results are 4 consecutive outputs of
//     one token;
//   * a lane loads 32 contiguous bytes of a row per 64-wide k step and feeds them to two
//     MFMAs; the k order inside a step is permuted the same way for both operands, which
//     leaves the dot product unchanged.
// Needs K % 8 == 0 (16-byte loads).
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

// ---- weights in the order in which a wave reads them ("wave order") ---------------------------
//
// A few-rows product walks w[R, K] in steps of 16 rows by 64 columns: lane (lr = lane % 16,
// lg = lane / 16) takes the 8 values at columns 64 step + 16 lg + 8 h of row 16 strip + lr, for
// h = 0 and 1.  From rows, one load instruction of a wave touches 64 bytes of each of 16 rows,
// and the two instructions of a step share every 128-byte line.  The copy in wave order holds the
// same values as the wave takes them: 16-byte piece ((strip * K / 64 + step) * 2 + h) * 64 + lane,
// so that an instruction reads 1 KB in one piece, every line once; the loads then carry the mark
// "will not be used again" (non-temporal), which lets memory stream them faster (from rows that
// mark makes the products slower: a line that is not kept is fetched twice).  Needs R % 16 == 0
// and K % 64 == 0.  Qwen3-8B sizes, 8 rows: the 144 products of a decode step 2.82 -> 2.6 ms.
#define WAVE_ORDER16(ptr) __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(ptr))

__global__ __launch_bounds__(256) void wave_order_kernel(const bf16* __restrict__ w, bf16* __restrict__ out,
                                                        int R, int K) {
  typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
  const size_t pieces = (size_t)R * K / 8;
  const int steps = K >> 6;
  for (size_t p = (size_t)blockIdx.x * 256 + threadIdx.x; p < pieces; p += (size_t)gridDim.x * 256) {
    const int lane = (int)(p & 63), h = (int)((p >> 6) & 1);
    const size_t tile = p >> 7;  // strip * steps + step
    const size_t strip = tile / steps;
    const int step = (int)(tile % steps);
    const size_t row = strip * 16 + (lane & 15);
    const int col = step * 64 + (lane >> 4) * 16 + h * 8;
    reinterpret_cast<u32x4_t*>(out)[p] = *reinterpret_cast<const u32x4_t*>(w + row * K + col);
  }
}

// out[R, K] = w[R, K] in wave order (bf16; R % 16 == 0, K % 64 == 0; out is not w).
extern "C" int as_wave_order(const void* w, void* out, int R, int K, hipStream_t stream) {
  if (R <= 0 || K <= 0 || (R & 15) || (K & 63) || !w || !out || w == out) return AS_BAD_SHAPE;
  const size_t pieces = (size_t)R * K / 8;
  const int blocks = (int)((pieces + 255) / 256 < 65536 ? (pieces + 255) / 256 : 65536);
  wave_order_kernel<<<blocks, 256, 0, stream>>>((const bf16*)w, (bf16*)out, R, K);
  return launch_status();
}
// s_waitcnt that only constrains the vector-memory counter (vmcnt: bits 3:0 and 15:14)
#define PF_WAIT_VM(N) __builtin_amdgcn_s_waitcnt(((N) & 15) | (((N) >> 4) << 14) | (7 << 4) | (15 << 8))


template <typename OutT> __device__ __forceinline__ void store4(OutT* p, floatx4 v, int valid);
template <> __device__ __forceinline__ void store4<float>(float* p, floatx4 v, int valid) {
  if (valid == 4 && (((uintptr_t)p) & 15) == 0) { *reinterpret_cast<floatx4*>(p) = v; return; }
  for (int i = 0; i < valid; ++i) p[i] = v[i];
}
template <> __device__ __forceinline__ void store4<bf16>(bf16* p, floatx4 v, int valid) {
  if (valid == 4 && (((uintptr_t)p) & 7) == 0) {
    typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
    bf16x4 o = {(bf16)v[0], (bf16)v[1], (bf16)v[2], (bf16)v[3]};
    *reinterpret_cast<bf16x4*>(p) = o;
    return;
  }
  for (int i = 0; i < valid; ++i) p[i] = (bf16)v[i];
}

// What a few-rows product carries along when the residual sum and the RMSNorm around it are
// folded into the products of a decode step (a pre-norm layer: x += part(norm(x))):
//
//   producer (LINK): out is the fp32 stream x[M, N] and receives the bf16-rounded product on
//     top; the same lanes then write scaled[m, n] = bf16(x * gain[n]), the input of the next
//     product without its 1/rms factor, and ssq[m, strip] = the sum of x^2 over the strip's 16
//     columns.  Every element belongs to one lane of one workgroup: no races, a fixed order.
//   consumer (SCALED): a is such a `scaled`; 1/rms of each row comes from the row's sums of
//     squares (added in a fixed order, in fp32) and multiplies the product's fp32 sums before
//     anything else happens to them.  x * gain / rms is rounded to bf16 once in the RMSNorm
//     kernel and x * gain once here: the same precision, not the same bits.
struct NormLink {
  const float* ssq_in;  // SCALED: [M, strips_in]
  int strips_in;
  float eps;
  const float* gain;    // LINK: [N], the gains of the norm that follows
  bf16* scaled;         // LINK: [M, N]
  float* ssq_out;       // LINK: [M, strips of this product]
};

// The LINK epilogue for the lane that holds columns n .. n+3 of row m (sum: the product's fp32
// sums).  All 64 lanes of the wave call it together.
__device__ __forceinline__ void link_epilogue(const NormLink& link, float* x, floatx4 sum, int m, int n, int M, int N,
                                              int strip, int nstrips) {
  float ss = 0.f;
  if (m < M && n < N) {
    const int valid = min(4, N - n);
    float* xp = x + (size_t)m * N + n;
    bf16* sp = link.scaled + (size_t)m * N + n;
    if (valid == 4) {  // N % 4 == 0 here or this is not the last group: 16-byte aligned
      floatx4 v = *reinterpret_cast<floatx4*>(xp);
      const floatx4 g = *reinterpret_cast<const floatx4*>(link.gain + n);
      typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
      bf16x4 sc;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        v[r] += (float)(bf16)sum[r];
        sc[r] = (bf16)(v[r] * g[r]);
        ss += v[r] * v[r];
      }
      *reinterpret_cast<floatx4*>(xp) = v;
      *reinterpret_cast<bf16x4*>(sp) = sc;
    } else {
      for (int r = 0; r < valid; ++r) {
        const float v = xp[r] + (float)(bf16)sum[r];
        xp[r] = v;
        sp[r] = (bf16)(v * link.gain[n + r]);
        ss += v * v;
      }
    }
  }
  ss += __shfl_xor(ss, 16, 64);  // the four lanes that hold the strip's 16 columns of row m
  ss += __shfl_xor(ss, 32, 64);
  if ((threadIdx.x & 63) < 16 && m < M) link.ssq_out[(size_t)m * nstrips + strip] = ss;
}

template <int S, int MT, int SK_WAVES, typename OutT, bool LINK = false, bool TILED = false>  // TILED: w in wave order
__global__ __launch_bounds__(SK_WAVES * 64) void gemm_bf16_skinny_kernel(const bf16* __restrict__ a,
                                                                        const bf16* __restrict__ w,
                                                                        OutT* __restrict__ out, int M, int N, int K,
                                                                        NormLink link = NormLink{}) {
  extern __shared__ floatx4 red[];  // [SK_WAVES][S * MT][64]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int lr = lane & 15, lg = lane >> 4;
  const int n0 = blockIdx.x * (16 * S);
  const int steps = (K + 63) >> 6;
  const int per = (steps + SK_WAVES - 1) / SK_WAVES;
  const int st0 = wave * per, st1 = min(steps, st0 + per);

  const bf16* wrow[S];
#pragma unroll
  for (int s = 0; s < S; ++s)
    wrow[s] = TILED ? w + (size_t)(blockIdx.x * S + s) * (K >> 6) * 1024 + lane * 8  // the strip's first step, this lane's piece
                    : w + (size_t)min(n0 + s * 16 + lr, N - 1) * K;
  const bf16* arow[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) arow[mt] = a + (size_t)min(mt * 16 + lr, M - 1) * K;
  floatx4 acc[S][MT];
#pragma unroll
  for (int s = 0; s < S; ++s)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[s][mt] = floatx4{0.f, 0.f, 0.f, 0.f};

  // Main loop: whole 64-wide steps, four at a time, every load unconditional (rows beyond M or
  // N were clamped to valid ones above; their results are never stored), so that sixteen or
  // more 16-byte loads per lane are in flight before the first MFMA waits for data.
  const int full_steps = K >> 6;
  const int st_full = min(st1, full_steps);
  int st = st0;
#define SK_LOAD(U, STEP)                                                                     \
  {                                                                                          \
    const int k = (STEP) * 64 + lg * 16;                                                     \
    _Pragma("unroll") for (int s = 0; s < S; ++s) {                                          \
      if constexpr (TILED) {                                                                 \
        wv[U][s][0] = WAVE_ORDER16(wrow[s] + (size_t)(STEP) * 1024);                         \
        wv[U][s][1] = WAVE_ORDER16(wrow[s] + (size_t)(STEP) * 1024 + 512);                   \
      } else {                                                                               \
        wv[U][s][0] = *reinterpret_cast<const bf16x8*>(wrow[s] + k);                         \
        wv[U][s][1] = *reinterpret_cast<const bf16x8*>(wrow[s] + k + 8);                     \
      }                                                                                      \
    }                                                                                        \
    _Pragma("unroll") for (int mt = 0; mt < MT; ++mt) {                                      \
      av[U][mt][0] = *reinterpret_cast<const bf16x8*>(arow[mt] + k);                         \
      av[U][mt][1] = *reinterpret_cast<const bf16x8*>(arow[mt] + k + 8);                     \
    }                                                                                        \
  }
#define SK_MATH(U)                                                                                        \
  _Pragma("unroll") for (int s = 0; s < S; ++s) _Pragma("unroll") for (int mt = 0; mt < MT; ++mt) {       \
    acc[s][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wv[U][s][0], av[U][mt][0], acc[s][mt], 0, 0, 0); \
    acc[s][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wv[U][s][1], av[U][mt][1], acc[s][mt], 0, 0, 0); \
  }
#ifdef SK_UN_OVERRIDE
  constexpr int UN = SK_UN_OVERRIDE;
#else
  constexpr int UN = (S * MT >= 4) ? 2 : 4;  // steps in flight; fewer when a step already holds many registers
#endif
  for (; st + UN <= st_full; st += UN) {
    bf16x8 wv[UN][S][2], av[UN][MT][2];
#pragma unroll
    for (int u = 0; u < UN; ++u) SK_LOAD(u, st + u)
#pragma unroll
    for (int u = 0; u < UN; ++u) SK_MATH(u)
  }
  for (; st < st_full; ++st) {
    bf16x8 wv[1][S][2], av[1][MT][2];
    SK_LOAD(0, st)
    SK_MATH(0)
  }
#undef SK_LOAD
  if (!TILED && st0 <= full_steps && st1 > full_steps && (K & 63)) {  // the wave owning the last, partial step: chunks of 8 beyond K count as zeros
    const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
    const int k = full_steps * 64 + lg * 16;
    const bool v0 = k + 8 <= K, v1 = k + 16 <= K;
    bf16x8 wv[1][S][2], av[1][MT][2];
#pragma unroll
    for (int s = 0; s < S; ++s) {
      wv[0][s][0] = v0 ? *reinterpret_cast<const bf16x8*>(wrow[s] + k) : zero;
      wv[0][s][1] = v1 ? *reinterpret_cast<const bf16x8*>(wrow[s] + k + 8) : zero;
    }
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      av[0][mt][0] = v0 ? *reinterpret_cast<const bf16x8*>(arow[mt] + k) : zero;
      av[0][mt][1] = v1 ? *reinterpret_cast<const bf16x8*>(arow[mt] + k + 8) : zero;
    }
    SK_MATH(0)
  }
#undef SK_MATH

#pragma unroll
  for (int s = 0; s < S; ++s)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) red[(wave * (S * MT) + s * MT + mt) * 64 + lane] = acc[s][mt];
  __syncthreads();
  for (int e = threadIdx.x; e < S * MT * 64; e += SK_WAVES * 64) {
    floatx4 sum = red[e];
#pragma unroll
    for (int wv_ = 1; wv_ < SK_WAVES; ++wv_) sum += red[wv_ * (S * MT * 64) + e];
    const int l = e & 63, tile = e >> 6, s = tile / MT, mt = tile % MT;
    const int m = mt * 16 + (l & 15), n = n0 + s * 16 + 4 * (l >> 4);
    if constexpr (LINK) {
      static_assert(!LINK || S == 1, "one strip a workgroup: its index names the sums of squares");
      link_epilogue(link, reinterpret_cast<float*>(out), sum, m, n, M, N, blockIdx.x, gridDim.x);
    } else {
      if (m < M && n < N) store4<OutT>(out + (size_t)m * N + n, sum, min(4, N - n));
    }
  }
}

// Whether a product of these sizes can read its weights in wave order (wt: that copy, or null).
static bool takes_wave_order(const void* wt, int N, int K) { return wt && !(N & 15) && !(K & 63); }

template <int S, int MT, int SK_WAVES>
static int launch_skinny(const void* a, const void* w, const void* wt, void* out, int out_dtype, int M, int N, int K,
                         hipStream_t stream) {
  const int blocks = (N + 16 * S - 1) / (16 * S);
  const size_t shmem = sizeof(floatx4) * SK_WAVES * S * MT * 64;
  if constexpr (S == 1) {
    if (takes_wave_order(wt, N, K) && (out_dtype == DT_BF16 || out_dtype == DT_F32)) {
      if (out_dtype == DT_BF16)
        gemm_bf16_skinny_kernel<1, MT, SK_WAVES, bf16, false, true><<<blocks, SK_WAVES * 64, shmem, stream>>>((const bf16*)a, (const bf16*)wt, (bf16*)out, M, N, K);
      else
        gemm_bf16_skinny_kernel<1, MT, SK_WAVES, float, false, true><<<blocks, SK_WAVES * 64, shmem, stream>>>((const bf16*)a, (const bf16*)wt, (float*)out, M, N, K);
      return launch_status();
    }
  }
  if (out_dtype == DT_BF16)
    gemm_bf16_skinny_kernel<S, MT, SK_WAVES, bf16><<<blocks, SK_WAVES * 64, shmem, stream>>>((const bf16*)a, (const bf16*)w, (bf16*)out, M, N, K);
  else if (out_dtype == DT_F32)
    gemm_bf16_skinny_kernel<S, MT, SK_WAVES, float><<<blocks, SK_WAVES * 64, shmem, stream>>>((const bf16*)a, (const bf16*)w, (float*)out, M, N, K);
  else
    return AS_BAD_DTYPE;
  return launch_status();
}

// The same product for up to 16 rows and K <= 64 * PIPE_WAVES * NST: persistent workgroups,
// one per compute unit.  Measured on the streaming kernel above: re-reading the activations
// for every strip costs as much as a fifth of the weights' own traffic.  Here each wave keeps
// its K-slice of the activations in registers for the whole kernel and walks over strips of
// 16 weight rows (strip = blockIdx.x, + gridDim.x, ...).  A strip's weights sit in two
// register buffers (first and second half of the wave's slice); as soon as a half has gone
// through the matrix cores, the same half of the NEXT strip is requested, so loads stay in
// flight while the partial sums of the waves meet in LDS.  The LDS buffer alternates between
// strips, which leaves one barrier per strip; the wave that adds and stores rotates.
// Chunks of 8 beyond K count as zeros (MASKED), so any K % 8 == 0 up to the limit is taken.
//
// GATED: w holds N gate rows followed by N up rows, and out[m, n] = silu(gate) * up with both
// sums rounded to OutT first, which is what the plain product followed by the activation
// kernel gives.  A workgroup then walks over pairs of strips (gate rows, then the up rows of
// the same outputs); the wave whose turn it is keeps the gate sums until the up sums arrive.
constexpr int PIPE_WAVES = 8;
constexpr int PIPE_MAX_NST = 12;
constexpr int PIPE_MAX_NST_TWO = 8;  // with two row tiles

template <typename OutT> __device__ __forceinline__ float rounded(float v);
template <> __device__ __forceinline__ float rounded<float>(float v) { return v; }
template <> __device__ __forceinline__ float rounded<bf16>(float v) { return (float)(bf16)v; }

template <int NST, bool MASKED, bool GATED, typename OutT, bool SCALED = false, bool LINK = false, int MT = 1,
          bool TILED = false>  // TILED: w in wave order (N % 16 == 0, not MASKED)
__global__ __launch_bounds__(PIPE_WAVES * 64) void gemm_bf16_skinny_pipe_kernel(const bf16* __restrict__ a,
                                                                               const bf16* __restrict__ w,
                                                                               OutT* __restrict__ out, int M, int N,
                                                                               int K, int nstrips,
                                                                               NormLink link = NormLink{}) {
  static_assert(NST >= 2, "a wave's slice is handled in two halves");
  static_assert(!TILED || !MASKED, "weights in wave order come in whole steps");
  static_assert(!LINK || (!GATED && !SCALED && sizeof(OutT) == 4), "the stream is fp32 and takes a plain product");
  constexpr int H = (NST + 1) / 2, H2 = NST - H;  // steps of the first and of the second half
  __shared__ floatx4 red[2][MT][PIPE_WAVES * 64];
  __shared__ float inv_rms[16 * MT];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int lr = lane & 15, lg = lane >> 4;
  const int kbase = wave * NST * 64 + lg * 16;  // this lane's first k; step u adds 64 u
  // A unit of work is 16 rows of w: `strip` counts strips of outputs, `up` says which half
  // of a gated w the rows come from.
  int strip = blockIdx.x;
  bool up = false;
  if (strip >= nstrips) return;
  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
#define PIPE_VALID(U, HALF) (!MASKED || kbase + (U) * 64 + (HALF) * 8 + 8 <= K)
#define PIPE_LOAD(BUF, ROW, OFF, CNT)                                                                         \
  _Pragma("unroll") for (int u = 0; u < CNT; ++u) {                                                           \
    if constexpr (TILED) {                                                                                    \
      BUF[u][0] = WAVE_ORDER16(ROW + ((OFF) + u) * 1024);                                                     \
      BUF[u][1] = WAVE_ORDER16(ROW + ((OFF) + u) * 1024 + 512);                                               \
    } else {                                                                                                  \
      BUF[u][0] = PIPE_VALID((OFF) + u, 0) ? *reinterpret_cast<const bf16x8*>(ROW + ((OFF) + u) * 64) : zero; \
      BUF[u][1] = PIPE_VALID((OFF) + u, 1) ? *reinterpret_cast<const bf16x8*>(ROW + ((OFF) + u) * 64 + 8) : zero; \
    }                                                                                                         \
  }
#define PIPE_MATH(BUF, OFF, CNT)                                                                              \
  _Pragma("unroll") for (int u = 0; u < CNT; ++u) _Pragma("unroll") for (int mt = 0; mt < MT; ++mt) {           \
    acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(BUF[u][0], av[mt][(OFF) + u][0], acc[mt], 0, 0, 0);       \
    acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(BUF[u][1], av[mt][(OFF) + u][1], acc[mt], 0, 0, 0);       \
  }
// where this lane's share of a strip begins: its row at its first k, or (wave order) its piece of the wave's first step
#define PIPE_ROWS(STRIP, UP)                                                                                          \
  (TILED ? w + (((size_t)(STRIP) + ((UP) ? (size_t)(N >> 4) : 0)) * (K >> 6) + wave * NST) * 1024 + lane * 8          \
         : w + ((size_t)min((STRIP) * 16 + lr, N - 1) + ((UP) ? (size_t)N : 0)) * K + kbase)
  bf16x8 w0[H][2], w1[H2][2];
  const bf16* wrow = PIPE_ROWS(strip, false);
  PIPE_LOAD(w0, wrow, 0, H)
  PIPE_LOAD(w1, wrow, H, H2)
  bf16x8 av[MT][NST][2];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const bf16* arow = a + (size_t)min(mt * 16 + lr, M - 1) * K + kbase;
#pragma unroll
    for (int u = 0; u < NST; ++u) {
      av[mt][u][0] = PIPE_VALID(u, 0) ? *reinterpret_cast<const bf16x8*>(arow + u * 64) : zero;
      av[mt][u][1] = PIPE_VALID(u, 1) ? *reinterpret_cast<const bf16x8*>(arow + u * 64 + 8) : zero;
    }
  }
  if constexpr (SCALED) {
    // 1 / rms of the rows, 32 threads a row and 16 rows at a time; published by the first strip's barrier
    const int j0 = threadIdx.x & 31;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const int row = mt * 16 + (threadIdx.x >> 5);
      float ss = 0.f;
      if (row < M)
        for (int j = j0; j < link.strips_in; j += 32) ss += link.ssq_in[(size_t)row * link.strips_in + j];
#pragma unroll
      for (int off = 1; off < 32; off <<= 1) ss += __shfl_xor(ss, off, 64);
      if (j0 == 0) inv_rms[row] = row < M ? 1.0f / sqrtf(ss / (float)K + link.eps) : 0.f;
    }
  }
  int buf = 0, turn = 0;
  floatx4 gate[MT];
  for (;;) {
    const bool next_up = GATED && !up;
    const int next = next_up ? strip : strip + gridDim.x;
    const bool more = next < nstrips;
    const bf16* nrow = PIPE_ROWS(next, next_up);
    floatx4 acc[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[mt] = floatx4{0.f, 0.f, 0.f, 0.f};
    PIPE_MATH(w0, 0, H)
    if (more) { PIPE_LOAD(w0, nrow, 0, H) }
    PIPE_MATH(w1, H, H2)
    if (more) { PIPE_LOAD(w1, nrow, H, H2) }
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) red[buf][mt][wave * 64 + lane] = acc[mt];
    __syncthreads();
    if (wave == turn) {  // sums in the order of the waves, whichever wave adds them
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        floatx4 sum = red[buf][mt][lane];
#pragma unroll
        for (int x = 1; x < PIPE_WAVES; ++x) sum += red[buf][mt][x * 64 + lane];
        const int m = mt * 16 + lr, n = strip * 16 + 4 * lg;
        if constexpr (SCALED) sum *= inv_rms[m];
        if constexpr (LINK) {
          link_epilogue(link, reinterpret_cast<float*>(out), sum, m, n, M, N, strip, nstrips);
        } else if (GATED && !up) {
          gate[mt] = sum;
        } else {
          if (GATED) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              const float g = rounded<OutT>(gate[mt][r]);
              sum[r] = g / (1.0f + expf(-g)) * rounded<OutT>(sum[r]);
            }
          }
          if (m < M && n < N) store4<OutT>(out + (size_t)m * N + n, sum, min(4, N - n));
        }
      }
    }
    if (!more) break;
    // The next strip writes the other LDS buffer, and its barrier comes before anyone writes
    // this one again; by then the adding wave has passed that barrier, so it has read this one.
    buf ^= 1;
    if (!next_up) turn = (turn + 1 == PIPE_WAVES) ? 0 : turn + 1;
    strip = next;
    up = next_up;
  }
#undef PIPE_ROWS
#undef PIPE_VALID
#undef PIPE_LOAD
#undef PIPE_MATH
}

template <int NST, bool GATED, typename OutT, bool SCALED, bool LINK, int MT>
static int launch_pipe(const void* a, const void* w, const void* wt, void* out, int M, int N, int K,
                       const NormLink& link, hipStream_t stream) {
  const int nstrips = (N + 15) / 16;
  const int blocks = min(nstrips, compute_units());
  if (K == 64 * PIPE_WAVES * NST && takes_wave_order(wt, N, K))
    gemm_bf16_skinny_pipe_kernel<NST, false, GATED, OutT, SCALED, LINK, MT, true><<<blocks, PIPE_WAVES * 64, 0, stream>>>(
        (const bf16*)a, (const bf16*)wt, (OutT*)out, M, N, K, nstrips, link);
  else if (K == 64 * PIPE_WAVES * NST)
    gemm_bf16_skinny_pipe_kernel<NST, false, GATED, OutT, SCALED, LINK, MT><<<blocks, PIPE_WAVES * 64, 0, stream>>>(
        (const bf16*)a, (const bf16*)w, (OutT*)out, M, N, K, nstrips, link);
  else
    gemm_bf16_skinny_pipe_kernel<NST, true, GATED, OutT, SCALED, LINK, MT><<<blocks, PIPE_WAVES * 64, 0, stream>>>(
        (const bf16*)a, (const bf16*)w, (OutT*)out, M, N, K, nstrips, link);
  return launch_status();
}

// Whether the persistent kernel takes a product of these sizes: the activations of a wave's
// K-slice stay in its registers, 8 per row tile and 64 columns, so 17 to 32 rows (two row tiles)
// leave room for K up to 64 * PIPE_WAVES * PIPE_MAX_NST_TWO only.  (Whether two row tiles pay is
// the caller's question: every workgroup reads all rows of the activations, which at 32 rows
// and K = 4096 is more than its share of the weights.)
static bool pipe_fits(int M, int K) {
  return (M <= 16 && K <= 64 * PIPE_WAVES * PIPE_MAX_NST) || (M <= 32 && K <= 64 * PIPE_WAVES * PIPE_MAX_NST_TWO);
}

template <bool GATED, typename OutT, bool SCALED = false, bool LINK = false>
static int dispatch_pipe(const void* a, const void* w, const void* wt, void* out, int M, int N, int K,
                         hipStream_t stream, const NormLink& link = NormLink{}) {
  if (!pipe_fits(M, K)) return AS_BAD_SHAPE;
  int nst = 2 * ((K + 128 * PIPE_WAVES - 1) / (128 * PIPE_WAVES));
  if (K > 64 * PIPE_WAVES * 4 && K <= 64 * PIPE_WAVES * 5) nst = 5;  // a width of 2,560 (Qwen3-4B) in five whole steps a wave, not six masked ones
  if (M > 16) {
    switch (nst) {
      case 2: return launch_pipe<2, GATED, OutT, SCALED, LINK, 2>(a, w, wt, out, M, N, K, link, stream);
      case 4: return launch_pipe<4, GATED, OutT, SCALED, LINK, 2>(a, w, wt, out, M, N, K, link, stream);
      case 5: return launch_pipe<5, GATED, OutT, SCALED, LINK, 2>(a, w, wt, out, M, N, K, link, stream);
      case 6: return launch_pipe<6, GATED, OutT, SCALED, LINK, 2>(a, w, wt, out, M, N, K, link, stream);
      case 8: return launch_pipe<8, GATED, OutT, SCALED, LINK, 2>(a, w, wt, out, M, N, K, link, stream);
    }
    return AS_BAD_SHAPE;
  }
  switch (nst) {
    case 2: return launch_pipe<2, GATED, OutT, SCALED, LINK, 1>(a, w, wt, out, M, N, K, link, stream);
    case 4: return launch_pipe<4, GATED, OutT, SCALED, LINK, 1>(a, w, wt, out, M, N, K, link, stream);
    case 5: return launch_pipe<5, GATED, OutT, SCALED, LINK, 1>(a, w, wt, out, M, N, K, link, stream);
    case 6: return launch_pipe<6, GATED, OutT, SCALED, LINK, 1>(a, w, wt, out, M, N, K, link, stream);
    case 8: return launch_pipe<8, GATED, OutT, SCALED, LINK, 1>(a, w, wt, out, M, N, K, link, stream);
    case 10: return launch_pipe<10, GATED, OutT, SCALED, LINK, 1>(a, w, wt, out, M, N, K, link, stream);
    case 12: return launch_pipe<12, GATED, OutT, SCALED, LINK, 1>(a, w, wt, out, M, N, K, link, stream);
  }
  return AS_BAD_SHAPE;
}

// out[M, N] = silu(a @ w[:N]^T) * (a @ w[N:]^T) for w[2N, K] in bf16, both products rounded
// to bf16 before the activation.  Only sizes of the persistent kernel; AS_BAD_SHAPE
// otherwise, and the caller runs the product and the activation kernel instead.
// wt (here and below): the same weights in wave order (as_wave_order), or null; taken where the sizes allow.
extern "C" int as_gemm_bf16_gated(const void* a, const void* w, const void* wt, void* out, int M, int N, int K,
                                  hipStream_t stream) {
  if (M <= 0) return AS_OK;
  if (N <= 0 || K <= 0 || (K & 7) || !pipe_fits(M, K)) return AS_BAD_SHAPE;
  return dispatch_pipe<true, bf16>(a, w, wt, out, M, N, K, stream);
}

// The producer of a NormLink: x[M, N] (fp32) += bf16(a @ w^T); scaled[M, N] = bf16(x * gain);
// ssq[M, ceil(N / 16)] = sums of x^2 per 16 columns.  M <= 32, K % 8 == 0, N % 4 == 0; a K beyond
// the persistent kernel goes through the streaming one.
extern "C" int as_gemm_bf16_link(const void* a, const void* w, const void* wt, float* x, const float* gain,
                                 void* scaled, float* ssq, int M, int N, int K, hipStream_t stream) {
  if (M <= 0) return AS_OK;
  if (M > 32 || N <= 0 || K <= 0 || (K & 7) || (N & 3) || !gain || !scaled || !ssq) return AS_BAD_SHAPE;
  const NormLink link{nullptr, 0, 0.f, gain, (bf16*)scaled, ssq};
  if (pipe_fits(M, K)) return dispatch_pipe<false, float, false, true>(a, w, wt, x, M, N, K, stream, link);
  const int blocks = (N + 15) / 16;
  const bool tiled = takes_wave_order(wt, N, K);
#define LINK_STREAM(MTV, WAVES)                                                                                 \
  if (tiled)                                                                                                    \
    gemm_bf16_skinny_kernel<1, MTV, WAVES, float, true, true><<<blocks, WAVES * 64, sizeof(floatx4) * WAVES * MTV * 64, stream>>>( \
        (const bf16*)a, (const bf16*)wt, x, M, N, K, link);                                                     \
  else                                                                                                          \
    gemm_bf16_skinny_kernel<1, MTV, WAVES, float, true><<<blocks, WAVES * 64, sizeof(floatx4) * WAVES * MTV * 64, stream>>>( \
        (const bf16*)a, (const bf16*)w, x, M, N, K, link)
  if (M <= 16) {
    if (blocks < 512) { LINK_STREAM(1, 16); } else { LINK_STREAM(1, 8); }
  } else {
    if (blocks < 512) { LINK_STREAM(2, 16); } else { LINK_STREAM(2, 8); }
  }
#undef LINK_STREAM
  return launch_status();
}

// The consumer of a NormLink: out[M, N] (bf16) = (scaled @ w^T) / rms(x) with rms from
// ssq[M, strips_in] (strips_in = ceil(K / 16)) and eps; gated != 0: the gated product of that.
// Only sizes of the persistent kernel.
extern "C" int as_gemm_bf16_scaled(const void* scaled, const float* ssq, int strips_in, float eps, const void* w,
                                   const void* wt, void* out, int M, int N, int K, int gated, hipStream_t stream) {
  if (M <= 0) return AS_OK;
  if (N <= 0 || K <= 0 || (K & 7) || !pipe_fits(M, K) || !ssq || strips_in != (K + 15) / 16) return AS_BAD_SHAPE;
  const NormLink link{ssq, strips_in, eps, nullptr, nullptr, nullptr};
  return gated ? dispatch_pipe<true, bf16, true, false>(scaled, w, wt, out, M, N, K, stream, link)
               : dispatch_pipe<false, bf16, true, false>(scaled, w, wt, out, M, N, K, stream, link);
}

// ---- bf16, 17 to 128 rows: tiles of weight rows with the activations staged in LDS ---------
//
// With more than 16 rows the activations no longer fit a wave's registers, and reading them from
// memory again for every strip of 16 weight rows costs as much as reading weights (a 16-byte load
// per lane costs the same whether it ends in L2 or in HBM).  Here a workgroup of 8 waves owns NS
// strips (NS = 8, 4 or 2; 8 / NS waves share a strip and split every chunk of K between them) and
// walks K in chunks of 256: the chunk's activations come into LDS once per workgroup by loads that
// pass through registers (requested one chunk ahead, in LDS for the chunk in use and the one
// before), every wave multiplies its strip's weights (straight from memory into registers, two
// chunks ahead) with them.  So a workgroup reads M rows of
// activations for 16 NS rows of weights; fewer strips make more workgroups where N is small.
//
//   GATED:   the first half of the strips are gate rows, the second half the up rows of the same
//            outputs; the up sums meet the gate sums in LDS and out = silu(gate) * up, both rounded
//            to OutT first.
//   PARTIAL: blockIdx.y names a range of K; the fp32 sums of that range go to
//            partial[split][m][n] for whoever adds the ranges up (the RMSNorm that follows does).
//
// LDS slot (16 bytes) of activation row r, k-block c (8 values) of a chunk: r * 32 + (c ^ (r & 15)):
// the 16 rows that the lanes of an MFMA operand read at one k-block lie in 16 different bank groups.
// Needs K % 256 == 0 (and ranges of K that are multiples of 256).
constexpr int TILE_KC = 256;
constexpr int tile_waves(int ns) { return ns == 6 ? 6 : 8; }
constexpr int TILE_RING = 2;

template <int MT, int NS, bool GATED, bool PARTIAL, typename OutT, bool TILED = false>  // TILED: w in wave order (N % 16 == 0)
__global__ __launch_bounds__(tile_waves(NS) * 64) void gemm_bf16_tile_kernel(const bf16* __restrict__ a,
                                                                        const bf16* __restrict__ w,
                                                                        OutT* __restrict__ out,
                                                                        float* __restrict__ partial, int M, int N,
                                                                        int K, int k_per_split) {
  typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
  typedef __attribute__((address_space(3))) void* lds_ptr_t;
  typedef const __attribute__((address_space(1))) void* global_ptr_t;
  constexpr int TILE_WAVES = tile_waves(NS), NT = TILE_WAVES * 64;
  constexpr int KW = TILE_WAVES / NS;  // waves that share a strip
  constexpr int STEPS = 4 / KW;        // 64-wide steps of a chunk that one wave multiplies
  constexpr int ROWS = MT * 16, SLOTS = ROWS * 32;  // 16-byte slots of one chunk
  constexpr int OUT_STRIPS = GATED ? NS / 2 : NS;   // strips of outputs per workgroup
  constexpr int COPIES = (SLOTS + NT - 1) / NT;  // 16-byte pieces of a chunk that one thread moves
  static_assert(NS == 8 || NS == 6 || NS == 4 || NS == 2, "8 waves divide into 8, 4 or 2 strips of 16 rows; 6 waves take 6");
  extern __shared__ __attribute__((aligned(16))) u32x4_t tile_lds[];  // [TILE_RING][SLOTS]
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lr = lane & 15, lg = lane >> 4;
  const int strip = wave % NS, kw = wave / NS;
  const int k0 = PARTIAL ? blockIdx.y * k_per_split : 0;
  const int k1 = PARTIAL ? min(K, k0 + k_per_split) : K;
  const int nchunks = (k1 - k0) / TILE_KC;
  // this wave's 16 weight rows (rows beyond N repeat the last one; their sums are not stored)
  const bool is_up = GATED && strip >= OUT_STRIPS;
  const int n0 = blockIdx.x * (16 * OUT_STRIPS) + (strip % OUT_STRIPS) * 16;  // first output column of the strip
  // Loads go through buffer descriptors: a load beyond the buffer's end returns zeros and moves no
  // data, so every chunk issues the same loads (those for chunks past the last are sent beyond the
  // end) and the count of loads in flight at any point of the loop is known exactly.
  const unsigned w_rows = (unsigned)(GATED ? 2 * N : N);
  const __amdgpu_buffer_rsrc_t w_buf = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<bf16*>(w), 0, (int)(w_rows * (unsigned)K * 2u), 0x00020000);
  const __amdgpu_buffer_rsrc_t a_buf = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<bf16*>(a), 0, (int)((unsigned)M * (unsigned)K * 2u), 0x00020000);
  constexpr unsigned BEYOND = 0xfffffff0u;
  // byte offset of this lane's first 16 bytes of the strip at k0: in its row, or (wave order) in the strip's run of
  // 2 KB steps; a step of 64 columns further lies 128 bytes further in a row and 2 KB further in wave order, the
  // second half of a lane's 32 bytes 16 bytes and 1 KB further
  constexpr unsigned W_STEP = TILED ? 2048u : 128u, W_HALF = TILED ? 1024u : 16u, W_AUX = TILED ? 2 : 0;  // 2: non-temporal
  const unsigned w_off =
      TILED ? (((unsigned)(n0 >> 4) + (is_up ? (unsigned)(N >> 4) : 0u)) * (unsigned)(K >> 6) + (unsigned)(k0 >> 6)) * 2048u + lane * 16u
            : (((unsigned)min(n0 + lr, N - 1) + (is_up ? (unsigned)N : 0u)) * (unsigned)K + k0 + lg * 16) * 2u;

  // ---- activations: chunk j travels through registers (requested one chunk ahead, 16-byte loads
  // spread over the threads) into LDS slot j % 2 just before it is used
  u32x4_t held[COPIES];
  unsigned a_off[COPIES];
#pragma unroll
  for (int i = 0; i < COPIES; ++i) {
    const int slot = i * NT + tid, r = slot >> 5, c = (slot & 31) ^ (r & 15);
    a_off[i] = slot < SLOTS ? ((unsigned)min(r, M - 1) * (unsigned)K + k0 + c * 8) * 2u : BEYOND;
  }
  // Workgroups start at different chunks of K and wrap round: side by side they would all ask for
  // the same 512 bytes of every weight row at the same time, which are the same few memory channels.
  const int turn = (int)((blockIdx.x * 5u + blockIdx.y * 3u) % (unsigned)max(nchunks, 1));
  auto where = [&](int j) { const int at = j + turn; return at >= nchunks ? at - nchunks : at; };
  auto request = [&](int j) {
    const int at = where(j);
#pragma unroll
    for (int i = 0; i < COPIES; ++i)
      held[i] = __builtin_amdgcn_raw_buffer_load_b128(
          a_buf, (j < nchunks && a_off[i] != BEYOND) ? a_off[i] + at * (TILE_KC * 2) : BEYOND, 0, 0);
  };
  auto deposit = [&](int j) {
    u32x4_t* dst = tile_lds + (j % TILE_RING) * SLOTS + tid;
#pragma unroll
    for (int i = 0; i < COPIES; ++i)
      if (SLOTS % NT == 0 || i * NT + tid < SLOTS) dst[i * NT] = held[i];
  };
  // Three sets of registers hold the weights of this chunk, the next and the one after; their
  // roles rotate with the chunks (copying one set into another would wait for the newest loads).
  u32x4_t wa[STEPS][2], wb[STEPS][2], wc[STEPS][2];
  auto fetch = [&](u32x4_t (&into)[STEPS][2], int j) {
    const unsigned base = j < nchunks ? w_off + where(j) * (4 * W_STEP) : BEYOND;  // a chunk is four steps
#pragma unroll
    for (int i = 0; i < STEPS; ++i) {
      const unsigned at = j < nchunks ? base + (kw + i * KW) * W_STEP : BEYOND;
      into[i][0] = __builtin_amdgcn_raw_buffer_load_b128(w_buf, at, 0, W_AUX);
      into[i][1] = __builtin_amdgcn_raw_buffer_load_b128(w_buf, j < nchunks ? at + W_HALF : BEYOND, 0, W_AUX);
    }
  };
  floatx4 acc[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) acc[mt] = floatx4{0.f, 0.f, 0.f, 0.f};
  // One chunk: its activations (in registers by now) go to LDS, whose slot everyone left before the
  // barrier of the chunk before; the next chunk's activations and the weights of the chunk after
  // next are requested; a bare barrier (a fence would wait for every load in flight); the products.
  auto chunk = [&](int j, u32x4_t (&now)[STEPS][2], u32x4_t (&later)[STEPS][2]) {
    deposit(j);
    request(j + 1);
    fetch(later, j + 2);
    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): this wave's LDS writes have landed
    __builtin_amdgcn_s_barrier();
    const u32x4_t* acts = tile_lds + (j % TILE_RING) * SLOTS;
#pragma unroll
    for (int i = 0; i < STEPS; ++i)
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int c = (kw + i * KW) * 8 + lg * 2 + h;
        const bf16x8 wv = __builtin_bit_cast(bf16x8, now[i][h]);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          const bf16x8 av = __builtin_bit_cast(bf16x8, acts[(mt * 16 + lr) * 32 + (c ^ lr)]);  // r & 15 == lr
          acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wv, av, acc[mt], 0, 0, 0);
        }
      }
  };

  request(0);
  fetch(wa, 0);
  fetch(wb, 1);
  const int rounds = nchunks / 3;
  for (int it = 0; it < rounds; ++it) {  // three chunks: the roles of the weight registers come round
    const int j = 3 * it;
    chunk(j, wa, wc);
    chunk(j + 1, wb, wa);
    chunk(j + 2, wc, wb);
  }
  if (nchunks - 3 * rounds >= 1) chunk(3 * rounds, wa, wc);
  if (nchunks - 3 * rounds == 2) chunk(3 * rounds + 1, wb, wa);

  // ---- results: lane (lr, lg) holds out[m = mt * 16 + lr][n0 + 4 lg .. + 3]
  floatx4* meet = reinterpret_cast<floatx4*>(tile_lds);  // [8 waves][MT][64], once the ring is done with
  if constexpr (KW > 1 || GATED) {
    __syncthreads();
    if (kw > 0 || is_up) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) meet[(wave * MT + mt) * 64 + lane] = acc[mt];
    }
    __syncthreads();
    if (kw > 0) return;
    if constexpr (KW > 1) {  // the sums of the waves that shared this strip, in their order
      if (!is_up) {
#pragma unroll
        for (int x = 1; x < KW; ++x)
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) acc[mt] += meet[((x * NS + strip) * MT + mt) * 64 + lane];
      }
    }
    if (is_up) return;
  }
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = mt * 16 + lr, n = n0 + 4 * lg;
    floatx4 res = acc[mt];
    if constexpr (GATED) {
      floatx4 u = meet[((strip + OUT_STRIPS) * MT + mt) * 64 + lane];
#pragma unroll
      for (int x = 1; x < KW; ++x) u += meet[((x * NS + strip + OUT_STRIPS) * MT + mt) * 64 + lane];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float g = rounded<OutT>(res[r]);
        res[r] = g / (1.0f + expf(-g)) * rounded<OutT>(u[r]);
      }
    }
    if (m >= M || n >= N) continue;
    if constexpr (PARTIAL) {
      store4<float>(partial + ((size_t)blockIdx.y * M + m) * N + n, res, min(4, N - n));
    } else {
      store4<OutT>(out + (size_t)m * N + n, res, min(4, N - n));
    }
  }
}

template <int MT, int NS>
static int launch_tile(const void* a, const void* w, const void* wt, void* out, float* partial, int out_dtype, int M,
                       int N, int K, int gated, int splits, hipStream_t stream) {
  constexpr int TILE_WAVES = tile_waves(NS);
  const size_t ring = (size_t)TILE_RING * MT * 16 * 32 * 16, meet = (size_t)TILE_WAVES * MT * 64 * 16;
  const size_t shmem = ring > meet ? ring : meet;
  // ranges of whole chunks, the last one possibly shorter
  const int k_per_split = splits > 0 ? (K / TILE_KC + splits - 1) / splits * TILE_KC : K;
  const int per_tile = 16 * (gated ? NS / 2 : NS);
  const dim3 grid((N + per_tile - 1) / per_tile, splits > 0 ? splits : 1);
#define TILE_GO(GATEDV, PARTIALV, T, TILEDV)                                                              \
  do {                                                                                                    \
    auto kernel = gemm_bf16_tile_kernel<MT, NS, GATEDV, PARTIALV, T, TILEDV>;                             \
    static bool raised = false;                                                                           \
    if (shmem > (48u << 10) && !raised) {                                                                 \
      if (hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize,            \
                              (int)shmem) != hipSuccess) return AS_LAUNCH_FAILED;                         \
      raised = true;                                                                                      \
    }                                                                                                     \
    kernel<<<grid, TILE_WAVES * 64, shmem, stream>>>((const bf16*)a, (const bf16*)(TILEDV ? wt : w), (T*)out, partial, \
                                                     M, N, K, k_per_split);                               \
  } while (0)
  // the two variants that decode steps run also read weights in wave order
  const bool tiled = takes_wave_order(wt, N, K);
  if (splits > 0 && tiled && NS == 4) {  // the split products of the engine have tiles of four strips
    if constexpr (NS == 4) TILE_GO(false, true, float, true);
  } else if (splits > 0) TILE_GO(false, true, float, false);
  else if (gated && out_dtype == DT_BF16 && tiled) TILE_GO(true, false, bf16, true);
  else if (gated && out_dtype == DT_BF16) TILE_GO(true, false, bf16, false);
  else if (!gated && out_dtype == DT_BF16 && tiled && NS <= 4) {  // narrow tiles: what a plain product of few columns takes
    if constexpr (NS <= 4) TILE_GO(false, false, bf16, true);
  } else if (!gated && out_dtype == DT_BF16) TILE_GO(false, false, bf16, false);
  else if (!gated && out_dtype == DT_F32) TILE_GO(false, false, float, false);
  else return AS_BAD_DTYPE;
#undef TILE_GO
  return launch_status();
}

// out[M, N] = a[M, K] @ w[N, K]^T for 1 <= M <= 128 and K % 256 == 0 through the tile kernel
// (row tiles of 16 up to 64 rows, 96 or 128 rows above; two chunks of 128 rows take 128 KB of LDS).
//   gated != 0:  w is [2 N, K] (gate rows, then up rows), out[M, N] = silu(gate) * up, bf16.
//   splits > 0:  K is cut into `splits` ranges of ceil(K / 256 / splits) chunks of 256 (the last range may be
//                shorter, none may be empty) and the fp32 sums of every range go to partial[splits, M, N];
//                `out` is not written.
//   strips:      weight rows per workgroup / 16: 8, 6, 4 or 2 (0: 8).
//   wt:          the weights in wave order or null; read where N % 16 == 0 by the gated variant, the split variant
//                (tiles of 4 strips) and the plain bf16 variant (tiles of 2 and 4 strips).
extern "C" int as_gemm_bf16_tile(const void* a, const void* w, const void* wt, void* out, float* partial,
                                 int out_dtype, int M, int N, int K, int gated, int splits, int strips,
                                 hipStream_t stream) {
  if (M <= 0) return AS_OK;
  if (M > 128 || N <= 0 || K <= 0 || (K % TILE_KC) || splits < 0) return AS_BAD_SHAPE;
  if (splits > 0) {  // every range gets at least one chunk
    const int chunks = K / TILE_KC, per = (chunks + splits - 1) / splits;
    if (gated || !partial || (long long)(splits - 1) * per >= chunks) return AS_BAD_SHAPE;
  }
  if (splits == 0 && !out) return AS_BAD_SHAPE;
  if (strips == 0) strips = 8;
  if (strips != 8 && strips != 6 && strips != 4 && strips != 2) return AS_BAD_SHAPE;
  if ((unsigned long long)(gated ? 2 : 1) * N * K * 2ull > 0xf0000000ull) return AS_BAD_SHAPE;  // 32-bit byte offsets
  int MT = (M + 15) / 16;
  if (MT > 4) MT = MT <= 6 ? 6 : 8;  // above 64 rows: tiles of 96 and 128 rows
#define TILE_CASE(MTV, NSV) \
  if (MT == MTV && strips == NSV) return launch_tile<MTV, NSV>(a, w, wt, out, partial, out_dtype, M, N, K, gated, splits, stream)
  TILE_CASE(1, 8); TILE_CASE(2, 8); TILE_CASE(3, 8); TILE_CASE(4, 8);
  TILE_CASE(1, 6); TILE_CASE(2, 6); TILE_CASE(3, 6); TILE_CASE(4, 6);
  TILE_CASE(1, 4); TILE_CASE(2, 4); TILE_CASE(3, 4); TILE_CASE(4, 4);
  TILE_CASE(1, 2); TILE_CASE(2, 2); TILE_CASE(3, 2); TILE_CASE(4, 2);
  TILE_CASE(6, 8); TILE_CASE(8, 8); TILE_CASE(6, 6); TILE_CASE(8, 6);
  TILE_CASE(6, 4); TILE_CASE(8, 4); TILE_CASE(6, 2); TILE_CASE(8, 2);
#undef TILE_CASE
  return AS_BAD_SHAPE;
}

// strips: rows of w per workgroup / 16 in the streaming kernel (1, 2 or 4); 0 lets this
// function choose, which for up to 16 rows and a K that fits is the persistent kernel (-1
// asks for that one and fails where it cannot run).  Few strips (a small N) get 16 waves
// per workgroup in the streaming kernel, so that K is split further and the GPU still has
// enough loads in flight.
extern "C" int as_gemm_bf16_skinny(const void* a, const void* w, const void* wt, void* out, int out_dtype, int M,
                                   int N, int K, int strips, hipStream_t stream) {
  if (M <= 0) return AS_OK;
  if (M > 64 || N <= 0 || K <= 0 || (K & 7)) return AS_BAD_SHAPE;
  const int MT = (M + 15) / 16;
  if (strips == 0 || strips == -1) {
    if (pipe_fits(M, K)) {
      if (out_dtype == DT_BF16) return dispatch_pipe<false, bf16>(a, w, wt, out, M, N, K, stream);
      if (out_dtype == DT_F32) return dispatch_pipe<false, float>(a, w, wt, out, M, N, K, stream);
      return AS_BAD_DTYPE;
    }
    if (strips == -1) return AS_BAD_SHAPE;
  }
  int S = strips;
  if (S == 0) S = 1;  // measured best at every size of interest; more strips only cost registers
  if (S * MT > 8) S = 8 / MT;  // the partial sums of 8 waves stay within 64 KB of LDS
  if (S == 3) S = 2;
  const bool wide = (N / (16 * S)) < 512 && MT <= 2 && S == 1;
#define CASE(SV, MTV)                                                                               \
  if (S == SV && MT == MTV)                                                                         \
    return wide ? launch_skinny<SV, MTV, 16>(a, w, wt, out, out_dtype, M, N, K, stream)             \
                : launch_skinny<SV, MTV, 8>(a, w, wt, out, out_dtype, M, N, K, stream)
  CASE(1, 1); CASE(2, 1); CASE(4, 1);
  CASE(1, 2); CASE(2, 2); CASE(4, 2);
  CASE(1, 3); CASE(1, 4); CASE(2, 3); CASE(2, 4);
#undef CASE
  return AS_BAD_SHAPE;
}
