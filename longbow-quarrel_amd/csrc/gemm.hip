// lq_linear: y[M, N] = x[M, K] . W[N, K]^T, dispatch over the kernels.
#include "common.h"

int lq_gemm_generic(const void* x, const void* w, void* out, int in_dtype, int out_dtype, int M,
                    int N, int K, int lda, int ldw, int ldc, hipStream_t stream);
bool lq_gemm_mfma_accepts(const void* x, const void* w, int in_dtype, int K, int lda, int ldw);
int lq_gemm_mfma(const void* x, const void* w, void* out, int out_dtype, int M, int N, int K, int lda,
                 int ldw, int ldc, int epilogue, int splits, long long split_stride, int packed, hipStream_t stream);
bool lq_gemm_packable(int N, int K);
int lq_gemm_mfma_splits(int M, int N, int K);
int lq_gemm_fused_parts(int M, int N, int K);
int lq_gemm_residual(const void* act, const void* w, float* x, float* sq_out, const float* gain, void* scaled,
                     int ld_scaled, int M, int N, int K, int lda, int ldw, int ldx, int packed, hipStream_t stream);
int lq_gemm_scaled(const void* h, int ldh, const float* sq_parts, int n_parts, int width, float eps, const void* w,
                   void* out, int out_dtype, int M, int N, int K, int ldw, int ldc, int swiglu, int packed,
                   hipStream_t stream);

// In how many shares of K lq_linear wants to compute this product (1: whole).  With s > 1 shares the
// caller passes an output of s pieces, `split_stride` elements apart; their sum is the product, and
// whoever consumes it adds the pieces in ascending order.
extern "C" int lq_linear_splits(int in_dtype, int M, int N, int K, int force_generic) {
  if (force_generic || in_dtype != LQ_BF16 || K % 8 != 0) return 1;
  return lq_gemm_mfma_splits(M, N, K);
}

// Whether a bfloat16 weight [N, K] may be handed to the products packed (lq_pack_weight): only where every
// kernel that can meet it reads that layout.  `w_packed` below says that w is; its ldw is then K.
extern "C" int lq_weight_packable(int dtype, int N, int K) { return dtype == LQ_BF16 && lq_gemm_packable(N, K); }

extern "C" int lq_linear(const void* x, const void* w, void* out, int in_dtype, int out_dtype,
                         int M, int N, int K, int lda, int ldw, int ldc, int splits, long long split_stride,
                         int force_generic, int w_packed, hipStream_t stream) {
  LQ_REQUIRE(M > 0 && N > 0 && K > 0, "linear: sizes M=%d N=%d K=%d must be positive", M, N, K);
  LQ_REQUIRE(lda >= K && ldw >= K && ldc >= N, "linear: a row stride is smaller than its row");
  LQ_REQUIRE(x && w && out, "linear: null pointer");
  LQ_REQUIRE(splits >= 1 && (splits == 1 || split_stride >= (long long)M * ldc), "linear: bad split arguments");
  LQ_REQUIRE(!w_packed || (ldw == K && lq_weight_packable(in_dtype, N, K)), "linear: this weight cannot be packed");
  if (!force_generic && lq_gemm_mfma_accepts(x, w, in_dtype, K, lda, ldw))
    return lq_gemm_mfma(x, w, out, out_dtype, M, N, K, lda, ldw, ldc, 0, splits, split_stride, w_packed, stream);
  LQ_REQUIRE(splits == 1, "linear: only the matrix-core kernels split K");
  LQ_REQUIRE(!w_packed, "linear: only the matrix-core kernels read a packed weight (x must be 16-byte aligned rows)");
  return lq_gemm_generic(x, w, out, in_dtype, out_dtype, M, N, K, lda, ldw, ldc, stream);
}

// Whether lq_linear_swiglu takes this problem (else: lq_linear into [M, 2I] and lq_swiglu).
extern "C" int lq_linear_swiglu_supported(int in_dtype, int N, int K) {
  return in_dtype == LQ_BF16 && N % 16 == 0 && K % 8 == 0;
}

// out[M, N/2] = silu(gate) * up where [gate | up] = x . W^T and W's N rows hold gate and up rows
// interleaved in groups of 8 (rows 16j..16j+7 gate 8j..8j+7, rows 16j+8..16j+15 up 8j..8j+7).
extern "C" int lq_linear_swiglu(const void* x, const void* w, void* out, int in_dtype, int out_dtype, int M,
                                int N, int K, int lda, int ldw, int ldc, int w_packed, hipStream_t stream) {
  LQ_REQUIRE(M > 0 && N > 0 && K > 0, "linear+swiglu: sizes M=%d N=%d K=%d must be positive", M, N, K);
  LQ_REQUIRE(lda >= K && ldw >= K && ldc >= N / 2, "linear+swiglu: a row stride is smaller than its row");
  LQ_REQUIRE(x && w && out, "linear+swiglu: null pointer");
  LQ_REQUIRE(lq_linear_swiglu_supported(in_dtype, N, K) && lq_gemm_mfma_accepts(x, w, in_dtype, K, lda, ldw),
             "linear+swiglu: needs bfloat16, 16-byte aligned rows, K %% 8 == 0 and N %% 16 == 0");
  LQ_REQUIRE(!w_packed || (ldw == K && lq_weight_packable(in_dtype, N, K)), "linear+swiglu: this weight cannot be packed");
  return lq_gemm_mfma(x, w, out, out_dtype, M, N, K, lda, ldw, ldc, 1, 1, 0, w_packed, stream);
}

// ------------------------------------------------------------------ the products around a norm (decoding)
// A pre-norm block's x += act . w^T; out = rmsnorm(x) . w2^T in two kernels instead of three.  The first
// adds into the float32 stream, leaves per-row sums of squares, a part per block, and the rows times the
// norm's gain in bfloat16; the second multiplies those rows with w2 and scales each output row by
// 1 / sqrt(mean(x^2) + eps) from the parts.  (The rows are rounded to bfloat16 before the division by the
// root mean square, not after: the same relative rounding.)  lq_linear_fused_parts: the number of parts
// the first leaves for [M, K] x [N, K]^T, or 0 when these kernels do not take the size (then the caller
// uses the separate kernels).
extern "C" int lq_linear_fused_parts(int dtype, int M, int N, int K) {
  if (dtype != LQ_BF16) return 0;
  return lq_gemm_fused_parts(M, N, K);
}

extern "C" int lq_linear_residual(const void* act, const void* w, float* x, float* sq_out, const float* gain,
                                  void* scaled, int ld_scaled, int dtype, int M, int N, int K, int lda, int ldw,
                                  int ldx, int parts, int w_packed, hipStream_t stream) {
  LQ_REQUIRE(act && w && x && sq_out, "linear_residual: null pointer");
  LQ_REQUIRE((gain == nullptr) == (scaled == nullptr) && (scaled == nullptr || ld_scaled >= N),
             "linear_residual: a gain and a place for the scaled rows come together");
  LQ_REQUIRE(lda >= K && ldw >= K && ldx >= N, "linear_residual: a row stride is smaller than its row");
  LQ_REQUIRE(parts > 0 && parts == lq_linear_fused_parts(dtype, M, N, K),
             "linear_residual: M=%d N=%d K=%d leaves %d parts, not %d", M, N, K, lq_linear_fused_parts(dtype, M, N, K),
             parts);
  LQ_REQUIRE(lq_gemm_mfma_accepts(act, w, dtype, K, lda, ldw), "linear_residual: operands are not aligned");
  LQ_REQUIRE(!w_packed || (ldw == K && lq_weight_packable(dtype, N, K)), "linear_residual: this weight cannot be packed");
  return lq_gemm_residual(act, w, x, sq_out, gain, scaled, ld_scaled, M, N, K, lda, ldw, ldx, w_packed, stream);
}

extern "C" int lq_linear_scaled(const void* h, int ldh, const float* sq_parts, int parts, float eps, const void* w,
                                void* out, int dtype, int out_dtype, int M, int N, int K, int ldw, int ldc,
                                int swiglu, int w_packed, hipStream_t stream) {
  LQ_REQUIRE(h && sq_parts && w && out, "linear_scaled: null pointer");
  LQ_REQUIRE(parts > 0 && ldh >= K && ldw >= K && ldc >= (swiglu ? N / 2 : N), "linear_scaled: bad sizes");
  LQ_REQUIRE(lq_linear_fused_parts(dtype, M, N, K) > 0 && (!swiglu || N % 16 == 0),
             "linear_scaled: M=%d N=%d K=%d is not taken", M, N, K);
  LQ_REQUIRE(lq_gemm_mfma_accepts(h, w, dtype, K, ldh, ldw), "linear_scaled: operands are not aligned");
  LQ_REQUIRE(!w_packed || (ldw == K && lq_weight_packable(dtype, N, K)), "linear_scaled: this weight cannot be packed");
  return lq_gemm_scaled(h, ldh, sq_parts, parts, K, eps, w, out, out_dtype, M, N, K, ldw, ldc, swiglu, w_packed, stream);
}
