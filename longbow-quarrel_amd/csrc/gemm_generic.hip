// y[M, N] = x[M, K] . W[N, K]^T  -- weights are [out, in], K contiguous in both
// (internal/device/kernels.metal:105-132: "y[b,row] = sum_k W[row,k] x[b,k]").
//
// This file holds the size-agnostic kernel: LDS-tiled, vector FMA, 32-bit
// accumulation, every output summed over k in ascending order (in slabs of 16, each summed by
// itself first), so a row's result does not depend on how many other rows the launch holds.  It is the whole of
// the float32 path (no matrix-core mode that would narrow the operands) and the
// fallback of the bfloat16 path for shapes the MFMA kernels refuse.
#include "common.h"

namespace {

constexpr int BM = 64, BN = 64, BK = 16;

template <typename T, typename TO>
__global__ __launch_bounds__(256) void gemm_tiled_kernel(const T* __restrict__ A, int lda,
                                                         const T* __restrict__ W, int ldw,
                                                         TO* __restrict__ C, int ldc, int M, int N,
                                                         int K) {
  // k-major tiles: a thread reads 4 consecutive m (or n) for one k
  __shared__ float As[BK][BM + 4];
  __shared__ float Ws[BK][BN + 4];
  const int tid = threadIdx.x;
  const int tx = tid & 15, ty = tid >> 4;  // 16 x 16 threads, 4 x 4 outputs each
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  // loader mapping: 64 rows x 16 k = 256 threads x 4 consecutive k
  const int lrow = tid >> 2, lk = (tid & 3) * 4;

  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

  for (int k0 = 0; k0 < K; k0 += BK) {
    {
      const int m = m0 + lrow;
      const T* src = A + (long long)m * lda + k0 + lk;
#pragma unroll
      for (int u = 0; u < 4; ++u)
        As[lk + u][lrow] = (m < M && k0 + lk + u < K) ? to_f32(src[u]) : 0.f;
      const int n = n0 + lrow;
      const T* wsrc = W + (long long)n * ldw + k0 + lk;
#pragma unroll
      for (int u = 0; u < 4; ++u)
        Ws[lk + u][lrow] = (n < N && k0 + lk + u < K) ? to_f32(wsrc[u]) : 0.f;
    }
    __syncthreads();
    // a slab's 16 products are summed by themselves and then added to the running sum: the rounding
    // error of a long row grows with K / 16 + 16 additions instead of K
    float part[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) part[i][j] = 0.f;
#pragma unroll
    for (int kk = 0; kk < BK; ++kk) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = Ws[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) part[i][j] = fmaf(a[i], b[j], part[i][j]);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[i][j] += part[i][j];
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n < N) C[(long long)m * ldc + n] = from_f32<TO>(acc[i][j]);
    }
  }
}

}  // namespace

int lq_gemm_generic(const void* x, const void* w, void* out, int in_dtype, int out_dtype, int M,
                    int N, int K, int lda, int ldw, int ldc, hipStream_t stream) {
  dim3 grid(lq_ceil_div(N, BN), lq_ceil_div(M, BM));
  LQ_REQUIRE(grid.y <= 65535, "linear: %d rows are too many for one launch", M);
#define LQ_GEMM_LAUNCH(T, TO)                                                                   \
  gemm_tiled_kernel<T, TO><<<grid, 256, 0, stream>>>((const T*)x, lda, (const T*)w, ldw, (TO*)out, \
                                                      ldc, M, N, K)
  if (in_dtype == LQ_F32 && out_dtype == LQ_F32)
    LQ_GEMM_LAUNCH(float, float);
  else if (in_dtype == LQ_BF16 && out_dtype == LQ_BF16)
    LQ_GEMM_LAUNCH(bf16_t, bf16_t);
  else if (in_dtype == LQ_BF16 && out_dtype == LQ_F32)
    LQ_GEMM_LAUNCH(bf16_t, float);
  else if (in_dtype == LQ_F32 && out_dtype == LQ_BF16)
    LQ_GEMM_LAUNCH(float, bf16_t);
  else
    LQ_REQUIRE(false, "linear: unsupported dtypes %d -> %d", in_dtype, out_dtype);
#undef LQ_GEMM_LAUNCH
  LQ_CHECK_LAUNCH("linear(generic)");
  return 0;
}
