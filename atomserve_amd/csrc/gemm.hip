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
