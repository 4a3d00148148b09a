// y[M, N] = x[M, K] . W[N, K]^T  -- weights are [out, in], K contiguous in both
// (internal/device/kernels.metal:105-132: "y[b,row] = sum_k W[row,k] x[b,k]").
//
// This file holds the size-agnostic product: the whole of the float32 path and the fallback of the
// bfloat16 path for shapes that the bfloat16 matrix-core kernels refuse.  Operands are widened to
// float32 (never narrowed) and multiplied on the matrix cores in their true 32-bit mode,
// v_mfma_f32_16x16x4_f32: float32 in, float32 accumulate, no reduced-precision step anywhere.
//
// One summation tree for every output, whatever kernel, tile or batch it is computed in, so that a
// row's result does not depend on how many other rows the launch holds (bit for bit):
//   * K is cut into chunks of CHUNK = 256 consecutive k, counted from k = 0;
//   * a chunk's sum starts from zero and runs through the chunk in slabs of 16 k, a slab being four
//     matrix instructions: instruction j of a slab multiplies k0 + 4 g + j for g = 0..3 (the four k that
//     one instruction takes are spread over the slab so that a lane can fetch its four k of a slab as
//     16 consecutive bytes);
//   * the chunks' sums are added one after the other in ascending order, in float32.
// k past K count as zeros, which change no sum.  The rounding error of a long row grows with
// K / 256 + 64 additions instead of K.
//
// Two kernels: an LDS-tiled one (block tiles of 64 x 64 or 128 x 128, any size and alignment), and one for
// up to 16 rows that streams the weights straight from memory, a block of waves a tile of 16 columns, its
// waves taking chunks in turn and adding their sums up in order through LDS.
#include "common.h"

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int CHUNK = 256, SLAB = 16;

// v_mfma_f32_16x16x4_f32: lane l gives A[row l % 16][k l / 16] and B[k l / 16][column l % 16] and holds
// D[4 (l / 16) + e][l % 16], e < 4.
__device__ inline f32x4 mfma4(float a, float b, f32x4 c) { return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0); }

// ---- tiled: 4 waves (2 x 2), a wave TM x TN tiles of 16 x 16 ---------------------------------------------
template <typename T, typename TO, int TM, int TN>
__global__ __launch_bounds__(256) void gemm_f32_tiled_kernel(const T* __restrict__ A, int lda, const T* __restrict__ W,
                                                             int ldw, TO* __restrict__ C, int ldc, int M, int N, int K) {
  constexpr int BM = 2 * TM * 16, BN = 2 * TN * 16;
  // k-major tiles; rows of BM + 4 floats put the four k that an instruction reads on different banks
  __shared__ float As[SLAB][BM + 4];
  __shared__ float Ws[SLAB][BN + 4];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r16 = lane & 15, g = lane >> 4;
  const int wm = wave >> 1, wn = wave & 1;
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  // loader: a thread takes 4 consecutive k of one row, 64 rows a pass
  const int lrow = tid >> 2, lk = (tid & 3) * 4;
  constexpr int PA = BM / 64, PW = BN / 64;

  f32x4 total[TM][TN], chunk[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      total[i][j] = (f32x4){0.f, 0.f, 0.f, 0.f};
      chunk[i][j] = (f32x4){0.f, 0.f, 0.f, 0.f};
    }

  float ra[PA][4], rw[PW][4];
  auto fetch = [&](int k0) {
#pragma unroll
    for (int p = 0; p < PA; ++p) {
      const int m = m0 + p * 64 + lrow;
      const T* src = A + (long long)min(m, M - 1) * lda + k0 + lk;
#pragma unroll
      for (int u = 0; u < 4; ++u) ra[p][u] = (m < M && k0 + lk + u < K) ? to_f32(src[u]) : 0.f;
    }
#pragma unroll
    for (int p = 0; p < PW; ++p) {
      const int n = n0 + p * 64 + lrow;
      const T* src = W + (long long)min(n, N - 1) * ldw + k0 + lk;
#pragma unroll
      for (int u = 0; u < 4; ++u) rw[p][u] = (n < N && k0 + lk + u < K) ? to_f32(src[u]) : 0.f;
    }
  };
  auto stage = [&]() {
#pragma unroll
    for (int p = 0; p < PA; ++p)
#pragma unroll
      for (int u = 0; u < 4; ++u) As[lk + u][p * 64 + lrow] = ra[p][u];
#pragma unroll
    for (int p = 0; p < PW; ++p)
#pragma unroll
      for (int u = 0; u < 4; ++u) Ws[lk + u][p * 64 + lrow] = rw[p][u];
  };

  fetch(0);
  for (int k0 = 0; k0 < K; k0 += SLAB) {
    stage();
    __syncthreads();
    if (k0 + SLAB < K) fetch(k0 + SLAB);  // the next slab is on its way while this one is multiplied
#pragma unroll
    for (int j4 = 0; j4 < 4; ++j4) {
      float a[TM], b[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i) a[i] = As[4 * g + j4][(wm * TM + i) * 16 + r16];
#pragma unroll
      for (int j = 0; j < TN; ++j) b[j] = Ws[4 * g + j4][(wn * TN + j) * 16 + r16];
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) chunk[i][j] = mfma4(a[i], b[j], chunk[i][j]);
    }
    if ((k0 + SLAB) % CHUNK == 0 || k0 + SLAB >= K) {
      // a chunk is complete: it joins the running sum, and the next starts from zero
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          total[i][j] += chunk[i][j];
          chunk[i][j] = (f32x4){0.f, 0.f, 0.f, 0.f};
        }
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int n = n0 + (wn * TN + j) * 16 + r16;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int m = m0 + (wm * TM + i) * 16 + 4 * g + e;
        if (m < M && n < N) C[(long long)m * ldc + n] = from_f32<TO>(total[i][j][e]);
      }
    }
}

// ---- at most 16 rows: the weights streamed from memory ---------------------------------------------------
// Four k of a row as float32: 16 bytes of float32 or 8 bytes of bfloat16.
__device__ inline f32x4 load4(const float* p) { return *(const f32x4*)p; }
__device__ inline f32x4 load4(const bf16_t* p) {
  const uint2 v = *(const uint2*)p;
  f32x4 r;
  r.x = __uint_as_float(v.x << 16);
  r.y = __uint_as_float(v.x & 0xffff0000u);
  r.z = __uint_as_float(v.y << 16);
  r.w = __uint_as_float(v.y & 0xffff0000u);
  return r;
}

constexpr int ROWS_WAVES = 8;  // waves a block; each takes every eighth chunk

template <typename T, typename TO>
__global__ __launch_bounds__(ROWS_WAVES * 64) void gemm_f32_rows_kernel(const T* __restrict__ X, int ldx,
                                                                        const T* __restrict__ W, int ldw,
                                                                        TO* __restrict__ C, int ldc, int M, int N, int K) {
  __shared__ float sums[2][ROWS_WAVES][256];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int c16 = lane & 15, g = lane >> 4;
  const int n0 = blockIdx.x * 16;
  const T* wp = W + (long long)min(n0 + c16, N - 1) * ldw + 4 * g;
  const T* xp = X + (long long)min(c16, M - 1) * ldx + 4 * g;
  const int chunks = (K + CHUNK - 1) / CHUNK;
  f32x4 total = {0.f, 0.f, 0.f, 0.f};
  const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
  for (int round = 0; round * ROWS_WAVES < chunks; ++round) {
    const int ch = round * ROWS_WAVES + wave;
    f32x4 sum = zero;
    if (ch < chunks) {
      const int k_begin = ch * CHUNK;
      // all of the chunk's weights are asked for together (16 loads of 1 KiB a wave), then its x
      f32x4 wv[CHUNK / SLAB], xv[CHUNK / SLAB];
#pragma unroll
      for (int s = 0; s < CHUNK / SLAB; ++s) {
        const int k = k_begin + s * SLAB;  // this lane's four k: k + 4 g .. k + 4 g + 3 (K is a multiple of 4)
        wv[s] = k + 4 * g < K ? load4(wp + k) : zero;
      }
#pragma unroll
      for (int s = 0; s < CHUNK / SLAB; ++s) {
        const int k = k_begin + s * SLAB;
        xv[s] = k + 4 * g < K ? load4(xp + k) : zero;
      }
#pragma unroll
      for (int s = 0; s < CHUNK / SLAB; ++s) {
#pragma unroll
        for (int j4 = 0; j4 < 4; ++j4) sum = mfma4(xv[s][j4], wv[s][j4], sum);
      }
    }
    // the round's chunks join the running sum in ascending order (every wave adds the same, wave 0 stores)
    float(*buf)[256] = sums[round & 1];
#pragma unroll
    for (int e = 0; e < 4; ++e) buf[wave][e * 64 + lane] = sum[e];
    __syncthreads();  // (two buffers: the one written two rounds ago has been read by then)
    const int n_round = min(ROWS_WAVES, chunks - round * ROWS_WAVES);
    for (int w = 0; w < n_round; ++w)
#pragma unroll
      for (int e = 0; e < 4; ++e) total[e] += buf[w][e * 64 + lane];
  }
  if (wave == 0) {
    const int n = n0 + c16;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int m = 4 * g + e;
      if (m < M && n < N) C[(long long)m * ldc + n] = from_f32<TO>(total[e]);
    }
  }
}

template <typename T, typename TO>
int launch(const void* x, const void* w, void* out, int M, int N, int K, int lda, int ldw, int ldc, hipStream_t stream) {
  const int el = (int)sizeof(T);
  // rows of four k each, fetched as one piece: K, the strides and the addresses must allow it
  const bool pieces = K % 4 == 0 && lda % 4 == 0 && ldw % 4 == 0 && ((uintptr_t)x % (4 * el)) == 0 &&
                      ((uintptr_t)w % (4 * el)) == 0;
  if (M <= 16 && pieces) {
    gemm_f32_rows_kernel<T, TO><<<lq_ceil_div(N, 16), ROWS_WAVES * 64, 0, stream>>>((const T*)x, lda, (const T*)w, ldw,
                                                                                   (TO*)out, ldc, M, N, K);
    LQ_CHECK_LAUNCH("linear(float32 rows)");
    return 0;
  }
  if (M > 64 && N > 64) {
    dim3 grid(lq_ceil_div(N, 128), lq_ceil_div(M, 128));
    LQ_REQUIRE(grid.y <= 65535, "linear: %d rows are too many for one launch", M);
    gemm_f32_tiled_kernel<T, TO, 4, 4><<<grid, 256, 0, stream>>>((const T*)x, lda, (const T*)w, ldw, (TO*)out, ldc, M, N, K);
  } else {
    dim3 grid(lq_ceil_div(N, 64), lq_ceil_div(M, 64));
    LQ_REQUIRE(grid.y <= 65535, "linear: %d rows are too many for one launch", M);
    gemm_f32_tiled_kernel<T, TO, 2, 2><<<grid, 256, 0, stream>>>((const T*)x, lda, (const T*)w, ldw, (TO*)out, ldc, M, N, K);
  }
  LQ_CHECK_LAUNCH("linear(float32 tiled)");
  return 0;
}

}  // namespace

int lq_gemm_generic(const void* x, const void* w, void* out, int in_dtype, int out_dtype, int M,
                    int N, int K, int lda, int ldw, int ldc, hipStream_t stream) {
  if (in_dtype == LQ_F32 && out_dtype == LQ_F32) return launch<float, float>(x, w, out, M, N, K, lda, ldw, ldc, stream);
  if (in_dtype == LQ_BF16 && out_dtype == LQ_BF16) return launch<bf16_t, bf16_t>(x, w, out, M, N, K, lda, ldw, ldc, stream);
  if (in_dtype == LQ_BF16 && out_dtype == LQ_F32) return launch<bf16_t, float>(x, w, out, M, N, K, lda, ldw, ldc, stream);
  if (in_dtype == LQ_F32 && out_dtype == LQ_BF16) return launch<float, bf16_t>(x, w, out, M, N, K, lda, ldw, ldc, stream);
  lq_set_error("linear: unsupported dtypes %d -> %d", in_dtype, out_dtype);
  return -1;
}
