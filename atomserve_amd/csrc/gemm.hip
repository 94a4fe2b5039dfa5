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

template <int S, int MT, int SK_WAVES, typename OutT>
__global__ __launch_bounds__(SK_WAVES * 64) void gemm_bf16_skinny_kernel(const bf16* __restrict__ a,
                                                                        const bf16* __restrict__ w,
                                                                        OutT* __restrict__ out, int M, int N, int K) {
  extern __shared__ floatx4 red[];  // [SK_WAVES][S * MT][64]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int lr = lane & 15, lg = lane >> 4;
  const int n0 = blockIdx.x * (16 * S);
  const int steps = (K + 63) >> 6;
  const int per = (steps + SK_WAVES - 1) / SK_WAVES;
  const int st0 = wave * per, st1 = min(steps, st0 + per);

  const bf16* wrow[S];
#pragma unroll
  for (int s = 0; s < S; ++s) wrow[s] = w + (size_t)min(n0 + s * 16 + lr, N - 1) * K;
  const bf16* arow[MT];
  bool aval[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = mt * 16 + lr;
    aval[mt] = m < M;
    arow[mt] = a + (size_t)min(m, M - 1) * K;
  }
  floatx4 acc[S][MT];
#pragma unroll
  for (int s = 0; s < S; ++s)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[s][mt] = floatx4{0.f, 0.f, 0.f, 0.f};

  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll 2
  for (int st = st0; st < st1; ++st) {
    const int k = st * 64 + lg * 16;
    const bool v0 = k + 8 <= K, v1 = k + 16 <= K;
    bf16x8 wv[S][2], av[MT][2];
#pragma unroll
    for (int s = 0; s < S; ++s) {
      wv[s][0] = v0 ? *reinterpret_cast<const bf16x8*>(wrow[s] + k) : zero;
      wv[s][1] = v1 ? *reinterpret_cast<const bf16x8*>(wrow[s] + k + 8) : zero;
    }
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      av[mt][0] = (v0 && aval[mt]) ? *reinterpret_cast<const bf16x8*>(arow[mt] + k) : zero;
      av[mt][1] = (v1 && aval[mt]) ? *reinterpret_cast<const bf16x8*>(arow[mt] + k + 8) : zero;
    }
#pragma unroll
    for (int s = 0; s < S; ++s)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        acc[s][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wv[s][0], av[mt][0], acc[s][mt], 0, 0, 0);
        acc[s][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wv[s][1], av[mt][1], acc[s][mt], 0, 0, 0);
      }
  }

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
    if (m < M && n < N) store4<OutT>(out + (size_t)m * N + n, sum, min(4, N - n));
  }
}

template <int S, int MT, int SK_WAVES>
static int launch_skinny(const void* a, const void* w, void* out, int out_dtype, int M, int N, int K,
                         hipStream_t stream) {
  const int blocks = (N + 16 * S - 1) / (16 * S);
  const size_t shmem = sizeof(floatx4) * SK_WAVES * S * MT * 64;
  if (out_dtype == DT_BF16)
    gemm_bf16_skinny_kernel<S, MT, SK_WAVES, bf16><<<blocks, SK_WAVES * 64, shmem, stream>>>((const bf16*)a, (const bf16*)w, (bf16*)out, M, N, K);
  else if (out_dtype == DT_F32)
    gemm_bf16_skinny_kernel<S, MT, SK_WAVES, float><<<blocks, SK_WAVES * 64, shmem, stream>>>((const bf16*)a, (const bf16*)w, (float*)out, M, N, K);
  else
    return AS_BAD_DTYPE;
  return launch_status();
}

// strips: rows of w per workgroup / 16 (1, 2 or 4); 0 lets the kernel choose.
// Few strips (a small N) get 16 waves per workgroup, so that K is split further and the
// GPU still has enough loads in flight.
extern "C" int as_gemm_bf16_skinny(const void* a, const void* w, void* out, int out_dtype, int M, int N, int K,
                                   int strips, hipStream_t stream) {
  if (M <= 0) return AS_OK;
  if (M > 64 || N <= 0 || K <= 0 || (K & 7)) return AS_BAD_SHAPE;
  const int MT = (M + 15) / 16;
  int S = strips;
  if (S == 0) S = (MT > 2) ? 1 : (N >= 65536 ? 4 : (N >= 6144 ? 2 : 1));
  if (MT > 2 && S > 1) S = 1;  // keeps the partial sums within LDS
  const bool wide = (N / (16 * S)) < 512 && MT <= 2 && S == 1;
#define CASE(SV, MTV)                                                                               \
  if (S == SV && MT == MTV)                                                                         \
    return wide ? launch_skinny<SV, MTV, 16>(a, w, out, out_dtype, M, N, K, stream)                 \
                : launch_skinny<SV, MTV, 8>(a, w, out, out_dtype, M, N, K, stream)
  CASE(1, 1); CASE(2, 1); CASE(4, 1);
  CASE(1, 2); CASE(2, 2); CASE(4, 2);
  CASE(1, 3); CASE(1, 4);
#undef CASE
  return AS_BAD_SHAPE;
}
