// lq_linear: y[M, N] = x[M, K] . W[N, K]^T, dispatch over the kernels.
#include "common.h"

int lq_gemm_generic(const void* x, const void* w, void* out, int in_dtype, int out_dtype, int M,
                    int N, int K, int lda, int ldw, int ldc, hipStream_t stream);
bool lq_gemm_mfma_accepts(const void* x, const void* w, int in_dtype, int K, int lda, int ldw);
int lq_gemm_mfma(const void* x, const void* w, void* out, int out_dtype, int M, int N, int K, int lda,
                 int ldw, int ldc, hipStream_t stream);

extern "C" int lq_linear(const void* x, const void* w, void* out, int in_dtype, int out_dtype,
                         int M, int N, int K, int lda, int ldw, int ldc, int force_generic,
                         hipStream_t stream) {
  LQ_REQUIRE(M > 0 && N > 0 && K > 0, "linear: sizes M=%d N=%d K=%d must be positive", M, N, K);
  LQ_REQUIRE(lda >= K && ldw >= K && ldc >= N, "linear: a row stride is smaller than its row");
  LQ_REQUIRE(x && w && out, "linear: null pointer");
  if (!force_generic && lq_gemm_mfma_accepts(x, w, in_dtype, K, lda, ldw))
    return lq_gemm_mfma(x, w, out, out_dtype, M, N, K, lda, ldw, ldc, stream);
  return lq_gemm_generic(x, w, out, in_dtype, out_dtype, M, N, K, lda, ldw, ldc, stream);
}
