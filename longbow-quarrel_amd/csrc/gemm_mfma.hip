// bfloat16 matrix products on the gfx950 matrix cores:  C[M, N] = A[M, K] . W[N, K]^T.
//
// Both operands have K contiguous, which is what the MFMA operand layout
// wants: a lane holds 8 consecutive k of one row (A) or one column (W row).
//
//   v_mfma_f32_32x32x16_bf16: lane l gives A[row l%32][k (l/32)*8 .. +8] and
//     B[col l%32][k (l/32)*8 .. +8]; it receives D[(e/4)*8 + (l/32)*4 + e%4][l%32], e < 16.
//   v_mfma_f32_16x16x32_bf16: lane l gives A[row l%16][k (l/16)*8 .. +8] and
//     B[col l%16][same k]; it receives D[(l/16)*4 + e][l%16], e < 4.
//
// Kernels:
//  * tiled, pipelined: 4 or 8 waves compute a 128 x 256 or 256 x 256 tile; operand slabs go from
//    memory straight into a ring of LDS stages (no registers in between).  For many rows (prefill)
//    and K a multiple of 32.  The same kernel with tiles of 64, 128 or 256 rows by 128, 64 or 32
//    columns and three or four stages takes 13 to 256 rows of a wide matrix (long decoding batches,
//    short prompts): the tile covers all rows, so every weight is read once, at streaming speed.
//  * tiled: a block of 4 waves (2 x 2) computes a (2*WM*32) x (2*WN*32) tile, operands staged
//    through padded LDS in steps of 64 k, next step prefetched into registers while the current one
//    is multiplied.  Takes any K that is a multiple of 8, and the small cases.
//  * skinny: at most 16 rows (decode).  A block owns 16 output columns; its KW waves split K,
//    stream their slice of the 16 weight rows straight from memory into MFMA operands (every
//    weight byte is read once, 16 bytes a lane), and add their partial tiles through LDS in
//    wave order, so the result does not depend on timing.
//
// Accumulation is 32-bit.  K must be a multiple of 8 and rows 16-byte aligned; the dispatcher
// sends everything else to the size-agnostic kernel.
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

namespace {

__device__ inline bf16x8 as_bf16x8(u32x4 v) {
  union {
    u32x4 u;
    bf16x8 b;
  } c;
  c.u = v;
  return c.b;
}

// A pointer that is the same in every lane, held in scalar registers.
__device__ inline const char* uniform_ptr(const char* p) {
  const unsigned long long v = (unsigned long long)p;
  const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)v), hi = __builtin_amdgcn_readfirstlane((unsigned)(v >> 32));
  return (const char*)(((unsigned long long)hi << 32) | lo);
}

template <typename TO>
__device__ inline void store_out(TO* p, float v);
template <>
__device__ inline void store_out<float>(float* p, float v) {
  *p = v;
}
template <>
__device__ inline void store_out<bf16_t>(bf16_t* p, float v) {
  *p = f32_to_bf16(v);
}

// Epilogues.  EPI_SWIGLU expects the weight rows interleaved in groups of 8: rows 16j..16j+7 are
// gate rows 8j..8j+7 and rows 16j+8..16j+15 the matching up rows, so that the lane holding gate
// column c (c % 16 < 8) finds its up value 8 lanes further; it writes silu(gate) * up to
// out[m][8j + c % 8], an [M, N / 2] matrix.
// EPI_RESIDUAL adds the product into C (the float32 residual stream, updated in place) and leaves, per
// row, the sum of squares of the block's updated columns in a table, for the norm that follows.
enum { EPI_NONE = 0, EPI_SWIGLU = 1, EPI_RESIDUAL = 2 };

// silu(g) u = g u / (1 + e^-g), for 16-bit outputs: the hardware's exponential and reciprocal (an ulp or so
// each, far below the rounding of the result) instead of a division and a library call per element
__device__ inline float silu_mul(float g, float u) { return g * __builtin_amdgcn_rcpf(1.0f + __expf(-g)) * u; }

// the value of the lane 8 places away within its row of 16 lanes (lane ^ 8), by a DPP rotation
__device__ inline float from_lane_xor8(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x128, 0xf, 0xf, true));
}

// A wave's WM x WN accumulators of 32 x 32 go to C (rows from row0, columns from col0).
template <int WM, int WN, int EPI, typename TO>
__device__ inline void tile_epilogue(f32x16 (&acc)[WM][WN], TO* __restrict__ C, int ldc, int M, int N, int row0,
                                     int col0, int lane) {
#pragma unroll
  for (int i = 0; i < WM; ++i)
#pragma unroll
    for (int j = 0; j < WN; ++j) {
      const int col = col0 + j * 32 + (lane & 31);
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int row = row0 + i * 32 + (e >> 2) * 8 + (lane >> 5) * 4 + (e & 3);
        if (EPI == EPI_SWIGLU) {
          // gate column c (c % 16 < 8) and its up column c + 8 sit 8 lanes apart
          const float up = __shfl(acc[i][j][e], lane + 8, 64);
          if ((col & 15) < 8 && row < M && col + 8 < N)
            store_out<TO>(C + (long long)row * ldc + ((col >> 4) << 3) + (col & 7), silu_mul(acc[i][j][e], up));
        } else {
          if (row < M && col < N) store_out<TO>(C + (long long)row * ldc + col, acc[i][j][e]);
        }
      }
    }
}

// The same for 16-bit outputs of a whole block, through LDS: the accumulator layout gives a lane one
// value of a row at a time (2-byte stores, 64 bytes a row), so the block first lays its output tile
// out in LDS, [BM][OUT_W] 16-bit, and then writes whole rows, 16 bytes a lane.  `tile` must hold
// BM * OUT_W * 2 bytes and be free (every wave past its last LDS read: the caller's barrier).
template <int WM, int WN, int BM, int BN, int EPI, int THREADS>
__device__ inline void block_epilogue_16(f32x16 (&acc)[WM][WN], bf16_t* __restrict__ C, int ldc, int M, int N, int m0,
                                         int n0, int wrow, int wcol, int lane, int tid, bf16_t* tile) {
  constexpr int OUT_W = EPI == EPI_SWIGLU ? BN / 2 : BN;
#pragma unroll
  for (int i = 0; i < WM; ++i)
#pragma unroll
    for (int j = 0; j < WN; ++j) {
      const int col = wcol + j * 32 + (lane & 31);  // within the block tile
      if constexpr (EPI == EPI_SWIGLU) {
        // Gate column c (c % 16 < 8) and its up column c + 8 sit 8 lanes apart.  Two rows at a time: the
        // gate lane takes the up value of the first row from its partner and gives it the gate value of the
        // second, so that every lane works out one product of the pair and no lane stands idle.
        const bool gate_lane = (lane & 8) == 0;
        const int out_col = ((col >> 4) << 3) + (col & 7);
#pragma unroll
        for (int e = 0; e < 16; e += 2) {
          const int row = wrow + i * 32 + (e >> 2) * 8 + (lane >> 5) * 4 + (e & 3) + (gate_lane ? 0 : 1);
          const float got = from_lane_xor8(gate_lane ? acc[i][j][e + 1] : acc[i][j][e]);
          const float v = gate_lane ? silu_mul(acc[i][j][e], got) : silu_mul(got, acc[i][j][e + 1]);
          tile[row * OUT_W + out_col] = f32_to_bf16(v);
        }
      } else {
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int row = wrow + i * 32 + (e >> 2) * 8 + (lane >> 5) * 4 + (e & 3);
          tile[row * OUT_W + col] = f32_to_bf16(acc[i][j][e]);
        }
      }
    }
  __syncthreads();
  const int n_out = EPI == EPI_SWIGLU ? N / 2 : N, c0 = EPI == EPI_SWIGLU ? n0 / 2 : n0;
  const bool vec = ldc % 8 == 0 && ((uintptr_t)C % 16) == 0;
  constexpr int CPR = OUT_W / 8;  // 16-byte chunks a row
  for (int c = tid; c < BM * CPR; c += THREADS) {
    const int row = c / CPR, cc = (c % CPR) * 8;
    const int grow = m0 + row, gcol = c0 + cc;
    if (grow >= M || gcol >= n_out) continue;
    bf16_t* dst = C + (long long)grow * ldc + gcol;
    const bf16_t* src = tile + row * OUT_W + cc;
    if (vec && gcol + 8 <= n_out) {
      *(u32x4*)dst = *(const u32x4*)src;
    } else {
      for (int q = 0; q < 8 && gcol + q < n_out; ++q) dst[q] = src[q];
    }
  }
}

// ------------------------------------------------------------------ tiled
constexpr int TBK = 64;           // k per stage
constexpr int TLD = TBK + 8;      // padded LDS row, in elements (144 bytes: conflict-free b128 reads)

template <int WM, int WN, int EPI, typename TO>
__global__ __launch_bounds__(256, (WM * WN <= 8 ? 2 : 1)) void gemm_bf16_tiled_kernel(const bf16_t* __restrict__ A, int lda,
                                                              const bf16_t* __restrict__ W, int ldw,
                                                              TO* __restrict__ C, int ldc, int M, int N,
                                                              int K, int tiles_m, int tiles_n) {
  constexpr int BM = 2 * WM * 32, BN = 2 * WN * 32;
  constexpr int A_CHUNKS = BM * (TBK / 8) / 256;  // 16-byte chunks a thread loads per stage
  constexpr int W_CHUNKS = BN * (TBK / 8) / 256;
  extern __shared__ __attribute__((aligned(16))) uint16_t lds[];
  uint16_t* As = lds;                 // [BM][TLD]
  uint16_t* Ws = lds + BM * TLD;      // [BN][TLD]

  // Consecutive blocks go to different XCDs (8 of them, each with its own L2).  Remap so that
  // one XCD gets a contiguous run of tiles, and let a run walk the m-tiles of one n-tile first:
  // its blocks then share the same weight tile in that XCD's L2.
  const int total = tiles_m * tiles_n;
  int pid = blockIdx.x;
  if (total % 8 == 0) pid = (pid % 8) * (total / 8) + pid / 8;  // ragged runs keep the plain order
  const int tm = pid % tiles_m, tn = pid / tiles_m;
  const int m0 = tm * BM, n0 = tn * BN;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;

  f32x16 acc[WM][WN];
#pragma unroll
  for (int i = 0; i < WM; ++i)
#pragma unroll
    for (int j = 0; j < WN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  u32x4 ra[A_CHUNKS], rw[W_CHUNKS];
  const u32x4 zero = {0u, 0u, 0u, 0u};

  auto load_stage = [&](int k0) {
#pragma unroll
    for (int i = 0; i < A_CHUNKS; ++i) {
      const int c = tid + i * 256;
      const int row = c >> 3, kc = (c & 7) * 8;
      const int m = min(m0 + row, M - 1);
      ra[i] = (k0 + kc < K) ? *(const u32x4*)(A + (long long)m * lda + k0 + kc) : zero;
    }
#pragma unroll
    for (int i = 0; i < W_CHUNKS; ++i) {
      const int c = tid + i * 256;
      const int row = c >> 3, kc = (c & 7) * 8;
      const int n = min(n0 + row, N - 1);
      rw[i] = (k0 + kc < K) ? *(const u32x4*)(W + (long long)n * ldw + k0 + kc) : zero;
    }
  };
  auto store_stage = [&]() {
#pragma unroll
    for (int i = 0; i < A_CHUNKS; ++i) {
      const int c = tid + i * 256;
      *(u32x4*)(As + (c >> 3) * TLD + (c & 7) * 8) = ra[i];
    }
#pragma unroll
    for (int i = 0; i < W_CHUNKS; ++i) {
      const int c = tid + i * 256;
      *(u32x4*)(Ws + (c >> 3) * TLD + (c & 7) * 8) = rw[i];
    }
  };

  load_stage(0);
  for (int k0 = 0; k0 < K; k0 += TBK) {
    __syncthreads();  // everyone is done reading the previous stage
    store_stage();
    __syncthreads();
    if (k0 + TBK < K) load_stage(k0 + TBK);  // in flight while this stage is multiplied
#pragma unroll
    for (int kk = 0; kk < TBK / 16; ++kk) {
      bf16x8 a[WM], b[WN];
      const int koff = kk * 16 + (lane >> 5) * 8;
#pragma unroll
      for (int i = 0; i < WM; ++i)
        a[i] = as_bf16x8(*(const u32x4*)(As + (wm * WM * 32 + i * 32 + (lane & 31)) * TLD + koff));
#pragma unroll
      for (int j = 0; j < WN; ++j)
        b[j] = as_bf16x8(*(const u32x4*)(Ws + (wn * WN * 32 + j * 32 + (lane & 31)) * TLD + koff));
#pragma unroll
      for (int i = 0; i < WM; ++i)
#pragma unroll
        for (int j = 0; j < WN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
    }
  }

  tile_epilogue<WM, WN, EPI, TO>(acc, C, ldc, M, N, m0 + wm * WM * 32, n0 + wn * WN * 32, lane);
}

template <int WM, int WN, int EPI, typename TO>
int launch_tiled(const void* A, const void* W, void* C, int M, int N, int K, int lda, int ldw, int ldc,
                 hipStream_t stream) {
  constexpr int BM = 2 * WM * 32, BN = 2 * WN * 32;
  const int tiles_m = lq_ceil_div(M, BM), tiles_n = lq_ceil_div(N, BN);
  const size_t smem = (size_t)(BM + BN) * TLD * sizeof(uint16_t);
  auto kernel = gemm_bf16_tiled_kernel<WM, WN, EPI, TO>;
  static bool configured = false;
  if (!configured && smem > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                       (int)smem);
    if (e != hipSuccess) {
      lq_set_error("linear: cannot reserve %zu bytes of LDS: %s", smem, hipGetErrorString(e));
      return -2;
    }
    configured = true;
  }
  const long long blocks = (long long)tiles_m * tiles_n;
  LQ_REQUIRE(blocks < (1ll << 31), "linear: too many tiles");
  kernel<<<(int)blocks, 256, smem, stream>>>((const bf16_t*)A, lda, (const bf16_t*)W, ldw, (TO*)C, ldc,
                                              M, N, K, tiles_m, tiles_n);
  LQ_CHECK_LAUNCH("linear(mfma tiled)");
  return 0;
}

// ------------------------------------------------------------------ tiled, pipelined
// What bounds a large product here is the traffic from L2 into the compute units, so this kernel
// makes the block tile large (GM x GN waves, each WM x WN accumulators of 32 x 32) and moves operand
// slabs of BK k from memory straight into LDS (global_load_lds_dwordx4: no registers, no LDS store
// instructions) into a ring of STAGES stages, STAGES - 1 slabs ahead of the one being multiplied, with
// one barrier a slab.  LDS rows are BK * 2 bytes, unpadded; the 16-byte chunk c of row r sits at chunk
// position c ^ swizzle(r), which keeps a fragment read (16 consecutive rows, one chunk) on 16
// different bank groups.  Fragment reads run two 16-k steps ahead of the products.
// blockIdx.y shares K: each share writes its partial product to C + y * split_stride.
// Needs K % (BK * shares) == 0.
#define LQ_GLOBAL_PTR(p) ((const __attribute__((address_space(1))) void*)(p))
#define LQ_LDS_PTR(p) ((__attribute__((address_space(3))) void*)(p))

// s_waitcnt vmcnt(n) alone (gfx9 encoding: vmcnt in bits 3:0 and 15:14, the other counters at their maxima)
#define LQ_WAIT_VMCNT(n) __builtin_amdgcn_s_waitcnt(0x0F70 | ((n) & 15) | (((n) >> 4) << 14))

template <int GM, int GN, int WM, int WN, int BK, int STAGES>
struct PipeShape {
  static constexpr int NW = GM * GN;                        // waves
  static constexpr int BM = GM * WM * 32, BN = GN * WN * 32;
  static constexpr int ROW_BYTES = BK * 2;
  static constexpr int CPR = BK / 8;                        // 16-byte chunks a row
  static constexpr int ROWS_PER_DMA = 1024 / ROW_BYTES;     // a wave's transfer is 64 lanes x 16 bytes
  // a stage is BM rows of A, then BN rows of W: TRANSFERS runs of 1 KiB, dealt out over the waves (DMA
  // each; where that does not come out even, the last run is fetched more than once)
  static constexpr int TRANSFERS = (BM + BN) / ROWS_PER_DMA, DMA = (TRANSFERS + NW - 1) / NW;
  static constexpr int A_BYTES = BM * ROW_BYTES, STAGE_BYTES = (BM + BN) * ROW_BYTES;
  static constexpr int LDS_BYTES = STAGES * STAGE_BYTES;
  static constexpr int KK = BK / 16;                        // 16-k steps a slab
  static_assert(BM % (ROWS_PER_DMA * NW) == 0 && BN % ROWS_PER_DMA == 0, "whole rounds of transfers for A, then W");
  static constexpr int A_ROUNDS = BM / (ROWS_PER_DMA * NW);  // transfers j < A_ROUNDS of every wave fetch A
  static_assert(DMA * (STAGES - 1) < 64, "vmcnt has 6 bits");
  // chunk position of chunk c in row r: rows that share a 256-byte bank row get different positions
  __device__ static int swizzle(int row) { return (row / (256 / ROW_BYTES)) & (CPR - 1); }
};

template <int GM, int GN, int WM, int WN, int BK, int STAGES, int EPI, typename TO, bool ALTERNATE = false>
__global__ __launch_bounds__(GM * GN * 64, 2) void gemm_bf16_pipelined_kernel(
    const bf16_t* __restrict__ A, int lda, const bf16_t* __restrict__ W, int ldw, TO* __restrict__ C, int ldc, int M,
    int N, int K, int tiles_m, int tiles_n, int k_share, long long split_stride, int packed) {
  using S = PipeShape<GM, GN, WM, WN, BK, STAGES>;
  extern __shared__ __attribute__((aligned(1024))) unsigned char plds[];

  const int total = tiles_m * tiles_n;
  int pid = blockIdx.x;
  if (total % 8 == 0) pid = (pid % 8) * (total / 8) + pid / 8;  // one XCD walks a contiguous run of tiles
  int tm = pid % tiles_m, tn = pid / tiles_m;
  if (total % 8 == 0 && tiles_m > 8 && (total / 8) % tiles_m == 0) {
    // The 32 tiles that an XCD works on together should share operands both ways: 8 row tiles by 4 column
    // tiles ask for 12 tiles' worth of operand rows, 32 row tiles of one column tile for 33.  The XCD's run
    // is whole columns of tiles: walk them four columns at a time, and each such band in windows of 8 row
    // tiles (the last window of a band has what is left).
    const int run = total / 8, cols = run / tiles_m, r = pid % run, first_col = (pid / run) * cols;
    const int band = r / (4 * tiles_m), in_band = r % (4 * tiles_m), width = min(4, cols - 4 * band);
    const int whole = tiles_m / 8, window = min(in_band / (8 * width), whole);
    const int in_window = in_band - window * 8 * width, height = window < whole ? 8 : tiles_m - 8 * whole;
    tm = window * 8 + in_window % height;
    tn = first_col + 4 * band + in_window / height;
  }
  const int m0 = tm * S::BM, n0 = tn * S::BN;
  const int k_begin = blockIdx.y * k_share;
  C += blockIdx.y * split_stride;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / GN, wn = wave % GN;

  // where this lane's 16 bytes of each transfer come from: transfer x = NW j + wave fills the stage's
  // chunks [64 x, 64 x + 64); chunk p is stage row p / CPR (A rows first), position p % CPR.  The address
  // is a wave-uniform origin (the operand's tile at this block's first k) plus a 32-bit lane offset.
  // (a packed W keeps 8 rows' 64-k slabs side by side: slab s of rows 8 i .. 8 i + 7 is the KiB at
  // element 8 i ldw + 512 s, a row's 64 k every 128 bytes in it; n0 and k_begin are multiples of 8 and 64)
  const int w_kmul = packed ? 16 : 2;  // bytes that one k moves a slab's address on
  const char* a_origin = (const char*)(A + (long long)m0 * lda + k_begin);
  const char* w_origin = (const char*)(W + (long long)n0 * ldw) + (long long)k_begin * w_kmul;
  unsigned off[S::DMA];
  int dst[S::DMA];
#pragma unroll
  for (int j = 0; j < S::DMA; ++j) {
    const int x = min(j * S::NW + wave, S::TRANSFERS - 1);
    const int p = x * 64 + lane, row = p / S::CPR, c = (p % S::CPR) ^ S::swizzle(row);
    const unsigned wr = (unsigned)(min(n0 + row - S::BM, N - 1) - n0);
    off[j] = row < S::BM ? (unsigned)(min(m0 + row, M - 1) - m0) * (unsigned)lda * 2u + c * 16
             : packed    ? (wr >> 3) * (unsigned)ldw * 16u + (wr & 7) * 128u + c * 16
                         : wr * (unsigned)ldw * 2u + c * 16;
    dst[j] = x * 1024;
  }
  auto dma = [&](int stage, int k0) {
    unsigned char* base = plds + stage * S::STAGE_BYTES;
#pragma unroll
    for (int j = 0; j < S::DMA; ++j) {
      // a scalar base and a 32-bit lane offset: one address register a transfer
      const char* origin = uniform_ptr(j < S::A_ROUNDS ? a_origin + (long long)k0 * 2 : w_origin + (long long)k0 * w_kmul);
      __builtin_amdgcn_global_load_lds(LQ_GLOBAL_PTR(origin + off[j]), LQ_LDS_PTR(base + dst[j]), 16, 0, 0);
    }
  };

  // fragment addresses within a 32-row group: row lane % 32, chunk 2 kk + lane / 32, swizzled
  int frag[S::KK];
#pragma unroll
  for (int kk = 0; kk < S::KK; ++kk)
    frag[kk] = (lane & 31) * S::ROW_BYTES + ((2 * kk + (lane >> 5)) ^ S::swizzle(lane & 31)) * 16;
  const unsigned char* a_base = plds + wm * WM * 32 * S::ROW_BYTES;
  const unsigned char* w_base = plds + S::A_BYTES + wn * WN * 32 * S::ROW_BYTES;

  f32x16 acc[WM][WN];
#pragma unroll
  for (int i = 0; i < WM; ++i)
#pragma unroll
    for (int j = 0; j < WN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  const int slabs = k_share / BK;

  auto step = [&](int stage, int t) {
    // this wave's transfers of slab t have landed (those of the slabs behind it may still fly) ...
    const int behind = min(STAGES - 2, slabs - 1 - t);
    if (STAGES >= 4 && behind == 2)
      LQ_WAIT_VMCNT(2 * S::DMA);
    else if (STAGES >= 3 && behind == 1)
      LQ_WAIT_VMCNT(S::DMA);
    else
      LQ_WAIT_VMCNT(0);
    // ... and so have everyone's; and everyone is done reading slab t - 1, whose stage is filled next
    asm volatile("s_barrier" ::: "memory");
    if (t + STAGES - 1 < slabs) dma((stage + STAGES - 1) % STAGES, (t + STAGES - 1) * BK);
    const unsigned char* as = a_base + stage * S::STAGE_BYTES;
    const unsigned char* ws = w_base + stage * S::STAGE_BYTES;
    bf16x8 a[2][WM], b[2][WN];
    auto read = [&](int kk) {
#pragma unroll
      for (int i = 0; i < WM; ++i)
        a[kk & 1][i] = as_bf16x8(*(const u32x4*)(as + i * 32 * S::ROW_BYTES + frag[kk]));
#pragma unroll
      for (int j = 0; j < WN; ++j)
        b[kk & 1][j] = as_bf16x8(*(const u32x4*)(ws + j * 32 * S::ROW_BYTES + frag[kk]));
    };
    read(0);
    read(1);
#pragma unroll
    for (int kk = 0; kk < S::KK; ++kk) {
      __builtin_amdgcn_sched_barrier(0);  // reads stay ahead of the products they do not feed
#pragma unroll
      for (int i = 0; i < WM; ++i)
#pragma unroll
        for (int j = 0; j < WN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[kk & 1][i], b[kk & 1][j], acc[i][j], 0, 0, 0);
      if (kk + 2 < S::KK) read(kk + 2);
    }
  };
  static_assert(STAGES >= 2 && STAGES <= 4, "the wait above knows 2 to 4 stages");
  if constexpr (!ALTERNATE) {
#pragma unroll
    for (int q = 0; q < STAGES - 1; ++q)
      if (q < slabs) dma(q, q * BK);
    for (int t = 0; t < slabs; t += STAGES) {
#pragma unroll
      for (int q = 0; q < STAGES; ++q)
        if (t + q < slabs) step(q, t + q);
    }
  } else {
    // Two groups of four waves (one wave of each on every SIMD) take turns: while one group multiplies
    // slab t, the other reads its fragments of slab t (or t + 1) from LDS, so the matrix pipe and the LDS
    // port of a SIMD work at the same time.  Every wave runs  fetch(t) | barrier | multiply(t) | barrier;
    // the second group has passed one barrier more before it starts, which puts it half a period behind.
    static_assert(!ALTERNATE || (STAGES == 2 && GM == 4 && GN == 2), "two stages, two groups of four waves");
    // Transfers are asked for in the fetch phases, after the wave's fragment reads are on their way: there
    // they cost nothing, while a wave that asks between its products (or before its reads) holds up the
    // matrix pipe (or the barrier) for as long as the address unit takes.  Group 0's waves fetch W, group 1's
    // fetch A, a wave every fourth transfer of its operand.  What may be overwritten when (stage s = t % 2
    // holds slab t; group 0 reads slab t + 1 while group 1 multiplies slab t; group 1 reads slab t + 1 while
    // group 0 multiplies it):
    //   W of slab t + 1, by group 0 after its reads of slab t: everyone has read W of slab t - 1 (group 1 last,
    //     before it multiplied slab t - 1, which it does now);
    //   group 1's own A rows of slab t + 1, by group 1 after its reads of slab t: it read those of slab t - 1 a
    //     period ago;
    //   group 0's A rows of slab t + 2, by group 1 at the same time, into the stage it is reading: group 0 has
    //     read its rows of slab t and multiplies them now.
    // Addresses: a buffer descriptor over the tile's valid rows (rows past the matrix read as zeros, no
    // clamping by hand), a lane offset (row within a transfer, swizzled chunk), the transfer's rows added to
    // it, and the slab's k as the scalar offset.
    const int group = wave >> 2, w4 = wave & 3;
    constexpr int NT = S::BM / S::ROWS_PER_DMA / 4;    // a wave's transfers of a slab of A (group 1)
    constexpr int NT_W = S::BN / S::ROWS_PER_DMA / 4;  // and of W (group 0)
    static_assert(S::BM % (S::ROWS_PER_DMA * 8) == 0 && S::BN % (S::ROWS_PER_DMA * 4) == 0,
                  "whole transfers for four waves, half of A group 0's rows");
    static_assert((4 * S::ROWS_PER_DMA) % ((256 / S::ROW_BYTES) * S::CPR) == 0, "a wave's transfers lie whole swizzle periods apart");
    const int lrow = lane / S::CPR;
    const int lchunk = ((lane % S::CPR) ^ S::swizzle(w4 * S::ROWS_PER_DMA + lrow)) * 16;
    const int ld = group == 0 ? ldw : lda;
    static_assert(!ALTERNATE || S::ROWS_PER_DMA == 8, "a transfer is the 8 rows that a packed W keeps together");
    const bool w_packed = group == 0 && packed;
    // this lane in the wave's transfer 0, and the way to the wave's next transfer
    const int t_voff = w_packed ? w4 * ld * 16 + lrow * 128 + lchunk : (w4 * S::ROWS_PER_DMA + lrow) * ld * 2 + lchunk;
    const int t_step = 4 * S::ROWS_PER_DMA * ld * 2;
    const int t_kmul = w_packed ? 16 : 2;
    const __amdgpu_buffer_rsrc_t t_rsrc =
        group == 0 ? __builtin_amdgcn_make_buffer_rsrc((void*)w_origin, 0, min(N - n0, S::BN) * ldw * 2, 0x00020000)
                   : __builtin_amdgcn_make_buffer_rsrc((void*)a_origin, 0, min(M - m0, S::BM) * lda * 2, 0x00020000);
    const int t_dst = (group == 0 ? S::A_BYTES : 0) + w4 * 1024;  // in a stage; 4 KiB on a transfer
    auto transfer = [&](int j, int stage, int k0) {
      int v = t_voff;
      asm volatile("" : "+v"(v));  // added up anew every time: kept across the loop it would cost a register a transfer
      __builtin_amdgcn_raw_ptr_buffer_load_lds(t_rsrc, LQ_LDS_PTR(plds + stage * S::STAGE_BYTES + t_dst + j * 4096), 16,
                                               v + j * t_step, k0 * t_kmul, 0, 0);
    };
    for (int q = 0; q < 2 && q < slabs; ++q)
#pragma unroll
      for (int j = 0; j < (NT > NT_W ? NT : NT_W); ++j)
        if (j < (group == 0 ? NT_W : NT)) transfer(j, q, q * BK);
    if (slabs == 1)
      LQ_WAIT_VMCNT(0);
    else if (group == 0)
      LQ_WAIT_VMCNT(NT_W);
    else
      LQ_WAIT_VMCNT(NT);
    asm volatile("s_barrier" ::: "memory");             // slab 0 is there
    if (group == 1) asm volatile("s_barrier" ::: "memory");  // half a period behind
    auto turn = [&](int stage, int t) {
      const unsigned char* as = a_base + stage * S::STAGE_BYTES;
      const unsigned char* ws = w_base + stage * S::STAGE_BYTES;
      bf16x8 a[S::KK][WM], b[S::KK][WN];
#pragma unroll
      for (int kk = 0; kk < S::KK; ++kk) {
#pragma unroll
        for (int i = 0; i < WM; ++i) a[kk][i] = as_bf16x8(*(const u32x4*)(as + i * 32 * S::ROW_BYTES + frag[kk]));
#pragma unroll
        for (int j = 0; j < WN; ++j) b[kk][j] = as_bf16x8(*(const u32x4*)(ws + j * 32 * S::ROW_BYTES + frag[kk]));
      }
      const bool next = t >= 1 && t + 1 < slabs, after_next = t + 2 < slabs;
      if (group == 0) {
        if (next) {
#pragma unroll
          for (int j = 0; j < NT_W; ++j) transfer(j, stage ^ 1, (t + 1) * BK);  // W of slab t + 1
        }
      } else {
        if (next) {
#pragma unroll
          for (int j = NT / 2; j < NT; ++j) transfer(j, stage ^ 1, (t + 1) * BK);  // own A rows of slab t + 1
        }
        if (after_next) {
#pragma unroll
          for (int j = 0; j < NT / 2; ++j) transfer(j, stage, (t + 2) * BK);  // group 0's A rows of slab t + 2
        }
        // group 0's A rows of slab t + 1, asked for a period ago, have landed: it reads them after the barrier
        if (next && after_next)
          LQ_WAIT_VMCNT(NT);
        else if (next || after_next)
          LQ_WAIT_VMCNT(NT / 2);
        else
          LQ_WAIT_VMCNT(0);
      }
      __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): the fragments are in registers
      __builtin_amdgcn_sched_barrier(0);
      asm volatile("s_barrier" ::: "memory");
      __builtin_amdgcn_sched_barrier(0);
      __builtin_amdgcn_s_setprio(1);
#pragma unroll
      for (int kk = 0; kk < S::KK; ++kk)
#pragma unroll
        for (int i = 0; i < WM; ++i)
#pragma unroll
          for (int j = 0; j < WN; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[kk][i], b[kk][j], acc[i][j], 0, 0, 0);
      __builtin_amdgcn_s_setprio(0);
      // what the next fetch phases read of slab t + 1 has landed: all of W (group 0's transfers), group 1's
      // own A rows (asked for before group 0's rows of slab t + 2, which may still fly)
      if (group == 0 || !after_next)
        LQ_WAIT_VMCNT(0);
      else
        LQ_WAIT_VMCNT(NT / 2);
      __builtin_amdgcn_sched_barrier(0);
      asm volatile("s_barrier" ::: "memory");
      __builtin_amdgcn_sched_barrier(0);
    };
    for (int t = 0; t < slabs; t += 2) {
      turn(0, t);
      if (t + 1 < slabs) turn(1, t + 1);
    }
    if (group == 0) asm volatile("s_barrier" ::: "memory");
  }
  if constexpr (sizeof(TO) == 2) {
    constexpr int OUT_BYTES = S::BM * (EPI == EPI_SWIGLU ? S::BN / 2 : S::BN) * 2;
    static_assert(OUT_BYTES <= S::LDS_BYTES, "the output tile must fit the stages");
    __syncthreads();  // every wave is past its last fragment read
    block_epilogue_16<WM, WN, S::BM, S::BN, EPI, S::NW * 64>(acc, C, ldc, M, N, m0, n0, wm * WM * 32, wn * WN * 32, lane,
                                                             tid, (bf16_t*)plds);
  } else {
    tile_epilogue<WM, WN, EPI, TO>(acc, C, ldc, M, N, m0 + wm * WM * 32, n0 + wn * WN * 32, lane);
  }
}

template <int GM, int GN, int WM, int WN, int BK, int STAGES, int EPI, typename TO, bool ALTERNATE = false>
int launch_pipelined(const void* A, const void* W, void* C, int M, int N, int K, int lda, int ldw, int ldc,
                     int splits, long long split_stride, hipStream_t stream, int packed = 0) {
  using S = PipeShape<GM, GN, WM, WN, BK, STAGES>;
  LQ_REQUIRE(!packed || (BK == 64 && N % 8 == 0), "linear: a packed weight needs slabs of 64 k and rows in eights");
  const int tiles_m = lq_ceil_div(M, S::BM), tiles_n = lq_ceil_div(N, S::BN);
  auto kernel = gemm_bf16_pipelined_kernel<GM, GN, WM, WN, BK, STAGES, EPI, TO, ALTERNATE>;
  static bool configured = false;
  if (!configured && S::LDS_BYTES > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                       S::LDS_BYTES);
    if (e != hipSuccess) {
      lq_set_error("linear: cannot reserve %d bytes of LDS: %s", S::LDS_BYTES, hipGetErrorString(e));
      return -2;
    }
    configured = true;
  }
  const long long blocks = (long long)tiles_m * tiles_n;
  LQ_REQUIRE(blocks < (1ll << 31), "linear: too many tiles");
  LQ_REQUIRE(splits >= 1 && K % (BK * splits) == 0, "linear: the pipelined kernel needs K to be a multiple of %d",
             BK * splits);
  LQ_REQUIRE(splits == 1 || EPI == EPI_NONE, "linear: no epilogue on partial products");
  LQ_REQUIRE((long long)lda * 2 * S::BM < (1ll << 31) && (long long)ldw * 2 * S::BN < (1ll << 31),
             "linear: rows too far apart for the tile's 32-bit offsets");
  kernel<<<dim3((int)blocks, splits), S::NW * 64, S::LDS_BYTES, stream>>>(
      (const bf16_t*)A, lda, (const bf16_t*)W, ldw, (TO*)C, ldc, M, N, K, tiles_m, tiles_n, K / splits, split_stride,
      packed);
  LQ_CHECK_LAUNCH("linear(mfma pipelined)");
  return 0;
}

// ------------------------------------------------------------------ skinny (M <= 64)
// 64-k chunks a wave keeps in flight (two weight loads of 1 KiB each): fewer when more row tiles
// need their own x operands in registers
constexpr int sk_unroll(int mt) { return mt == 1 ? 4 : 2; }

template <int KW, int MT, int EPI, typename TO>
__global__ __launch_bounds__(KW * 64) void gemm_bf16_skinny_kernel(const bf16_t* __restrict__ X, int ldx,
                                                                   const bf16_t* __restrict__ W, int ldw,
                                                                   TO* __restrict__ C, int ldc, int M,
                                                                   int N, int K) {
  constexpr int SK_UNROLL = sk_unroll(MT);
  __shared__ float red[KW][MT * 256];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n0 = blockIdx.x * 16;
  const int g = lane >> 4;
  const int nrow = min(n0 + (lane & 15), N - 1);
  const bf16_t* wp = W + (long long)nrow * ldw + g * 8;
  const bf16_t* xp[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) xp[t] = X + (long long)min(t * 16 + (lane & 15), M - 1) * ldx + g * 8;
  const u32x4 zero = {0u, 0u, 0u, 0u};

  f32x4 acc[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) acc[t] = (f32x4){0.f, 0.f, 0.f, 0.f};
  // wave w takes 64-k chunks w, w + KW, w + 2 KW, ... : the block reads KW * 128 bytes of every
  // weight row at a time
  for (int kc = wave * 64; kc < K; kc += KW * 64 * SK_UNROLL) {
    u32x4 wv[SK_UNROLL][2], xv[SK_UNROLL][MT][2];
#pragma unroll
    for (int u = 0; u < SK_UNROLL; ++u) {
      const int k = kc + u * KW * 64;
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const bool ok = k + h * 32 + g * 8 < K;
        wv[u][h] = ok ? *(const u32x4*)(wp + k + h * 32) : zero;
#pragma unroll
        for (int t = 0; t < MT; ++t) xv[u][t][h] = ok ? *(const u32x4*)(xp[t] + k + h * 32) : zero;
      }
    }
#pragma unroll
    for (int u = 0; u < SK_UNROLL; ++u)
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int t = 0; t < MT; ++t)
          acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(xv[u][t][h]), as_bf16x8(wv[u][h]), acc[t],
                                                           0, 0, 0);
  }
  // acc[t][e] = C[t * 16 + (lane / 16) * 4 + e][n0 + lane % 16], partial over this wave's k
#pragma unroll
  for (int t = 0; t < MT; ++t)
#pragma unroll
    for (int e = 0; e < 4; ++e) red[wave][t * 256 + e * 64 + lane] = acc[t][e];
  __syncthreads();
  if (wave == 0) {
    const int c16 = lane & 15;
    const int col = n0 + c16;
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float s = 0.f;
#pragma unroll
        for (int w = 0; w < KW; ++w) s += red[w][t * 256 + e * 64 + lane];
        const int row = t * 16 + g * 4 + e;
        if (EPI == EPI_SWIGLU) {
          const float up = __shfl(s, lane + 8, 64);
          if (c16 < 8 && row < M && col + 8 < N) store_out<TO>(C + (long long)row * ldc + (n0 >> 1) + c16, silu_mul(s, up));
        } else {
          if (row < M && col < N) store_out<TO>(C + (long long)row * ldc + col, s);
        }
      }
  }
}

template <int KW, int MT, int EPI, typename TO>
int launch_skinny(const void* X, const void* W, void* C, int M, int N, int K, int ldx, int ldw, int ldc,
                  hipStream_t stream) {
  gemm_bf16_skinny_kernel<KW, MT, EPI, TO><<<lq_ceil_div(N, 16), KW * 64, 0, stream>>>(
      (const bf16_t*)X, ldx, (const bf16_t*)W, ldw, (TO*)C, ldc, M, N, K);
  LQ_CHECK_LAUNCH("linear(mfma skinny)");
  return 0;
}

// ------------------------------------------------------------------ skinny, at most 16 rows
// One block per compute unit (or a small multiple): the N columns are dealt out in equal runs, so
// every compute unit streams the same number of weight bytes; a block walks its run in tiles of
// 16 columns.  The block's KW waves own contiguous K slices and keep their x fragments in
// registers across the tiles, so x is read once per block and each tile costs weight loads only
// (all of a tile's loads are in flight together).  Partial tiles meet in LDS, summed in wave order.
// Up to 64 rows: MT row tiles of 16 share every weight fragment.
constexpr int V3_MAXT = 8;  // tiles a block may own
// k-steps (of 32) whose x fragments a wave holds at a time, and waves per block: both shrink as the
// row tiles (each with x fragments and accumulators of its own) grow
constexpr int v3_kb(int mt) { return mt <= 2 ? 8 / mt : 2; }
constexpr int v3_kw(int mt) { return mt == 1 ? 16 : 8; }

// A product whose rows are scaled afterwards by the RMS statistic of the norm that its input stands for:
// the input holds x * gain (not yet divided by the root mean square), the rows' sums of squares come in
// parts (sq_parts[row][part], what the product before left), and out = rstd(row) * (input . w^T).
struct RowScale {
  const float* sq_parts;  // [M][n_parts]
  int n_parts;
  int width;              // of the normalised rows
  float eps;
};

// For EPI_RESIDUAL: where the sums of squares go, and optionally the next product's input.
struct ResidualOut {
  float* sq_out;          // [M][gridDim.x]
  const float* gain;      // [N] or null
  bf16_t* scaled;         // [M][ld_scaled]: bfloat16(x_new * gain), or null
  int ld_scaled;
};

template <int KW, int MT, int EPI, typename TO, bool SCALED, bool PACKED>
__global__ __launch_bounds__(KW * 64) void gemm_bf16_skinny_v3_kernel(const bf16_t* __restrict__ X, int ldx,
                                                                      const bf16_t* __restrict__ W, int ldw,
                                                                      TO* __restrict__ C, int ldc, int M, int N,
                                                                      int K, int cols_per_block, int ks_per_wave,
                                                                      long long split_stride, RowScale scale,
                                                                      ResidualOut res) {
  constexpr int KB = v3_kb(MT);
  constexpr int VALS = MT * 4;  // accumulator values a lane holds per tile
  // One row tile: the partial tiles of all the block's column tiles meet in LDS at once (dynamic, a KiB a tile
  // and wave), behind one barrier.  More row tiles: a tile at a time through a buffer of fixed size.
  constexpr bool BATCH = MT == 1;
  __shared__ float red_one[BATCH ? 1 : KW][BATCH ? 1 : VALS * 64];
  extern __shared__ __attribute__((aligned(16))) float red_all[];  // [tiles][KW][256] with BATCH
  __shared__ float fresh_sh[EPI == EPI_RESIDUAL ? 16 : 1][EPI == EPI_RESIDUAL ? V3_MAXT * 16 : 1];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int g = lane >> 4, c16 = lane & 15;
  const int col_begin = blockIdx.x * cols_per_block;
  const int col_end = min(N, col_begin + cols_per_block);
  if (col_begin >= N) return;
  const int ntiles = (col_end - col_begin + 15) / 16;
  // blockIdx.y: which share of K this block sums (its partial result goes to C + y * split_stride);
  // within the share, this wave's slice is [k_wave, k_stop)
  const int k_wave = (blockIdx.y * KW + wave) * ks_per_wave * 32;
  const int k_stop = min(K, k_wave + ks_per_wave * 32);
  C += blockIdx.y * split_stride;
  const bf16_t* xp[MT];  // k below already holds the lane's g * 8
#pragma unroll
  for (int m = 0; m < MT; ++m) xp[m] = X + (long long)min(m * 16 + c16, M - 1) * ldx;
  const u32x4 zero = {0u, 0u, 0u, 0u};

  // the parts of a row's sum of squares, asked for now and added up after the products
  __shared__ float rstd_sh[16];
  float sq_mine[4] = {0.f, 0.f, 0.f, 0.f};
  if (SCALED) {
    static_assert(!SCALED || MT == 1, "one row tile");
    if (wave < M) {  // 16 waves: wave w holds row w
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int b = lane + 64 * j;
        sq_mine[j] = b < scale.n_parts ? scale.sq_parts[(long long)wave * scale.n_parts + b] : 0.f;
      }
    }
  }

  f32x4 acc[V3_MAXT][MT];
#pragma unroll
  for (int t = 0; t < V3_MAXT; ++t)
#pragma unroll
    for (int m = 0; m < MT; ++m) acc[t][m] = (f32x4){0.f, 0.f, 0.f, 0.f};

  for (int kb = k_wave; kb < k_stop; kb += KB * 32) {
    u32x4 xv[KB][MT];
#pragma unroll
    for (int s = 0; s < KB; ++s) {
      const int k = kb + s * 32 + g * 8;
#pragma unroll
      for (int m = 0; m < MT; ++m) xv[s][m] = (k < k_stop) ? *(const u32x4*)(xp[m] + k) : zero;
    }
#pragma unroll
    for (int t = 0; t < V3_MAXT; ++t) {
      if (t < ntiles) {
        const int nrow = min(col_begin + t * 16 + c16, col_end - 1);
        // (packed: 8 rows' slabs of 64 k side by side; a wave's slice starts at a multiple of 64, so step s is
        // a constant number of bytes from the slice's first slab, as in a dense row)
        const bf16_t* wp = PACKED ? W + (long long)(nrow >> 3) * 8 * ldw + (nrow & 7) * 64 + ((kb >> 6) << 9) + g * 8
                                  : W + (long long)nrow * ldw + kb + g * 8;
        u32x4 wv[KB];
#pragma unroll
        for (int s = 0; s < KB; ++s) {
          const int k = kb + s * 32 + g * 8;
          wv[s] = (k < k_stop) ? *(const u32x4*)(wp + (PACKED ? (s >> 1) * 512 + (s & 1) * 32 : s * 32)) : zero;
        }
#pragma unroll
        for (int s = 0; s < KB; ++s)
#pragma unroll
          for (int m = 0; m < MT; ++m)
            acc[t][m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(xv[s][m]), as_bf16x8(wv[s]), acc[t][m],
                                                                0, 0, 0);
      }
    }
  }
  if (SCALED) {
    static_assert(!SCALED || KW == 16, "a wave a row");
    if (wave < M) {
      // more than 256 parts: the rest now
      float sum = (sq_mine[0] + sq_mine[1]) + (sq_mine[2] + sq_mine[3]);
      for (int b = lane + 256; b < scale.n_parts; b += 64) sum += scale.sq_parts[(long long)wave * scale.n_parts + b];
      for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off, 64);
      if (lane == 0) rstd_sh[wave] = 1.0f / sqrtf(sum / (float)scale.width + scale.eps);
    }
    // the barrier of the reduction below also publishes rstd_sh
  }
  // acc[t][m][e] = C[m * 16 + (lane / 16) * 4 + e][col_begin + 16 t + lane % 16], partial over this
  // wave's k.  The waves share out the (m, e) values of the tiles and each sums its share over all waves,
  // in wave order.
  auto finish = [&](int t, int v, float s, float x_old) {
    const int col = col_begin + t * 16 + c16;
    const int row = (v >> 2) * 16 + g * 4 + (v & 3);
    if (SCALED) s *= rstd_sh[min(row, M - 1)];
    if (EPI == EPI_SWIGLU) {
      const float up = __shfl(s, lane + 8, 64);
      if (c16 < 8 && row < M && col + 8 < col_end)
        store_out<TO>(C + (long long)row * ldc + ((col_begin + t * 16) >> 1) + c16, silu_mul(s, up));
    } else if constexpr (EPI == EPI_RESIDUAL) {
      static_assert(EPI != EPI_RESIDUAL || sizeof(TO) == 4, "the residual stream is float32");
      float fresh = 0.f;
      if (row < M && col < col_end) {
        fresh = x_old + s;
        *((float*)C + (long long)row * ldc + col) = fresh;
        if (res.scaled) res.scaled[(long long)row * res.ld_scaled + col] = f32_to_bf16(fresh * res.gain[col]);
      }
      if (row < 16) fresh_sh[row][t * 16 + c16] = fresh;  // zero beyond the matrix
    } else {
      if (row < M && col < col_end) store_out<TO>(C + (long long)row * ldc + col, s);
    }
  };
  auto stream_value = [&](int t, int v) -> float {  // the residual stream's old value at this lane's place
    if constexpr (EPI == EPI_RESIDUAL) {
      const int col = col_begin + t * 16 + c16, row = (v >> 2) * 16 + g * 4 + (v & 3);
      if (row < M && col < col_end) return *((const float*)C + (long long)row * ldc + col);
    }
    return 0.f;
  };
  if constexpr (BATCH) {
    // every tile's partial sums at once; the 4 value rows of each tile are dealt out over the waves (row
    // j = 4 t + v to wave j % KW), which ask for the stream's old values before they meet at the barrier
    static_assert(!BATCH || V3_MAXT * 4 <= 2 * KW, "at most two value rows a wave");
#pragma unroll
    for (int t = 0; t < V3_MAXT; ++t)
      if (t < ntiles) {
#pragma unroll
        for (int e = 0; e < 4; ++e) red_all[(t * KW + wave) * 256 + e * 64 + lane] = acc[t][0][e];
      }
    float x_old[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int j = wave + KW * i;
      x_old[i] = j < ntiles * 4 ? stream_value(j >> 2, j & 3) : 0.f;
    }
    __syncthreads();  // (also publishes rstd_sh)
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int j = wave + KW * i;
      if (j < ntiles * 4) {
        const int t = j >> 2, v = j & 3;
        float s = 0.f;
#pragma unroll
        for (int w = 0; w < KW; ++w) s += red_all[(t * KW + w) * 256 + v * 64 + lane];
        finish(t, v, s, x_old[i]);
      }
    }
  } else {
#pragma unroll
    for (int t = 0; t < V3_MAXT; ++t) {
      if (t < ntiles) {
        if (t > 0) __syncthreads();  // the tile before has been read
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
          for (int e = 0; e < 4; ++e) red_one[wave][(m * 4 + e) * 64 + lane] = acc[t][m][e];
        __syncthreads();
        for (int v = (wave + t) % KW; v < VALS; v += KW) {
          float s = 0.f;
#pragma unroll
          for (int w = 0; w < KW; ++w) s += red_one[w][v * 64 + lane];
          finish(t, v, s, stream_value(t, v));
        }
      }
    }
  }
  if (EPI == EPI_RESIDUAL) {
    // sum of squares of this block's columns of every row, in a fixed order: wave w takes row w
    __syncthreads();
    for (int r = wave; r < min(M, 16); r += KW) {
      float sum = 0.f;
      for (int c = lane; c < ntiles * 16; c += 64) sum += fresh_sh[r][c] * fresh_sh[r][c];
      for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off, 64);
      if (lane == 0) res.sq_out[(long long)r * gridDim.x + blockIdx.x] = sum;
    }
  }
}

// How many blocks should share K for an [M, K] x [N, K]^T product with the balanced kernel (1: no
// split).  With several row tiles a block wants several column tiles too, so that the x fragments it
// holds are used more than once; a matrix with few columns gets them by giving each block a wider run
// of columns and a share of K instead.
int v3_splits(int M, int N, int K) {
  if (M <= 16 || M > 64) return 1;
  if (!(N >= 8 * lq_compute_units() && K >= 512)) return 1;
  const int tiles_per_block = lq_ceil_div(lq_ceil_div(N, 16), lq_compute_units());
  int splits = 1;
  while (splits < 4 && tiles_per_block * splits < 4 && K / (splits * 2) >= 1024) splits *= 2;
  return splits;
}

// Runs of columns for the balanced kernel: equal, in units of 16 (8 without a paired epilogue), at most
// V3_MAXT tiles each; -> columns a block, blocks
inline void v3_runs(int N, int cus, int unit, int& cols, int& grid) {
  int blocks = cus;
  cols = lq_ceil_div(lq_ceil_div(N, blocks), unit) * unit;
  while (cols > V3_MAXT * 16) {
    blocks += cus;
    cols = lq_ceil_div(lq_ceil_div(N, blocks), unit) * unit;
  }
  grid = lq_ceil_div(N, cols);
}

template <int KW, int MT, int EPI, typename TO, bool SCALED, bool PACKED>
int launch_skinny_v3_as(const void* X, const void* W, void* C, int M, int N, int K, int ldx, int ldw, int ldc, int splits,
                        long long split_stride, hipStream_t stream, RowScale scale, ResidualOut res, int cols, int grid,
                        int ks_per_wave);

template <int MT, int EPI, typename TO, bool SCALED = false>
int launch_skinny_v3(const void* X, const void* W, void* C, int M, int N, int K, int ldx, int ldw, int ldc,
                     int splits, long long split_stride, hipStream_t stream, int packed = 0,
                     RowScale scale = RowScale(), ResidualOut res = ResidualOut()) {
  constexpr int KW = v3_kw(MT);
  LQ_REQUIRE(!packed || (K % 64 == 0 && N % 8 == 0), "linear: a packed weight has K in 64s and rows in eights");
  int cols, grid;
  v3_runs(N, lq_compute_units() / splits, EPI == EPI_SWIGLU ? 16 : 8, cols, grid);
  const int ksteps = lq_ceil_div(K, 32);
  // an even number of 32-k steps a wave: its slice starts at a multiple of 64, where a packed weight's slabs do
  const int ks_per_wave = (lq_ceil_div(ksteps, KW * splits) + 1) / 2 * 2;
  if (packed)
    return launch_skinny_v3_as<KW, MT, EPI, TO, SCALED, true>(X, W, C, M, N, K, ldx, ldw, ldc, splits, split_stride, stream,
                                                              scale, res, cols, grid, ks_per_wave);
  return launch_skinny_v3_as<KW, MT, EPI, TO, SCALED, false>(X, W, C, M, N, K, ldx, ldw, ldc, splits, split_stride, stream,
                                                             scale, res, cols, grid, ks_per_wave);
}

template <int KW, int MT, int EPI, typename TO, bool SCALED, bool PACKED>
int launch_skinny_v3_as(const void* X, const void* W, void* C, int M, int N, int K, int ldx, int ldw, int ldc, int splits,
                        long long split_stride, hipStream_t stream, RowScale scale, ResidualOut res, int cols, int grid,
                        int ks_per_wave) {
  auto kernel = gemm_bf16_skinny_v3_kernel<KW, MT, EPI, TO, SCALED, PACKED>;
  // one row tile: a KiB of LDS for every column tile and wave of a block
  const int lds = MT == 1 ? lq_ceil_div(cols, 16) * KW * 1024 : 0;
  static bool configured = false;
  if (!configured && MT == 1) {
    hipError_t e = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, V3_MAXT * KW * 1024);
    if (e != hipSuccess) {
      lq_set_error("linear: cannot reserve %d bytes of LDS: %s", V3_MAXT * KW * 1024, hipGetErrorString(e));
      return -2;
    }
    configured = true;
  }
  kernel<<<dim3(grid, splits), KW * 64, lds, stream>>>(
      (const bf16_t*)X, ldx, (const bf16_t*)W, ldw, (TO*)C, ldc, M, N, K, cols, ks_per_wave, split_stride, scale, res);
  LQ_CHECK_LAUNCH("linear(mfma skinny v3)");
  return 0;
}

template <int MT, int EPI, typename TO>
int pick_skinny(const void* x, const void* w, void* out, int M, int N, int K, int lda, int ldw, int ldc,
                hipStream_t stream) {
  // enough waves to keep the memory system busy: about 8 a CU
  const long long tiles = lq_ceil_div(N, 16);
  const int chunks = lq_ceil_div(K, 64);
  if (tiles * 4 >= 2048 || chunks < 8)
    return launch_skinny<4, MT, EPI, TO>(x, w, out, M, N, K, lda, ldw, ldc, stream);
  if (tiles * 8 >= 2048 || chunks < 16 || MT > 2)
    return launch_skinny<8, MT, EPI, TO>(x, w, out, M, N, K, lda, ldw, ldc, stream);
  return launch_skinny<16, MT, EPI, TO>(x, w, out, M, N, K, lda, ldw, ldc, stream);
}

// A weight may be kept packed (8 rows' slabs of 64 k side by side, see lq_pack_weight) if every product
// with it runs in the pipelined kernel with slabs of 64 k or in the balanced kernel: wide, K in 64s.
inline bool gemm_packable(int N, int K) {
  return N >= 8 * lq_compute_units() && N % 8 == 0 && K >= 512 && K % 64 == 0;
}

// The large pipelined tile pays once its tiles (times the shares of K) fill three quarters of the chip.
inline bool fills_chip(long long blocks) { return blocks * 4 >= 3ll * lq_compute_units(); }

// Shares of K for more than 64 rows: few tiles of 256 x 256 (a narrow weight matrix, a short prompt)
// leave compute units idle; sharing K out over blocks fills them.
int tiled_splits(int M, int N, int K) {
  if (K % 64 != 0) return 1;
  const long long t256 = (long long)lq_ceil_div(M, 256) * lq_ceil_div(N, 256);
  int splits = 1;
  while (splits < 8 && !fills_chip(t256 * splits) && K % (128 * splits) == 0 && K / (splits * 2) >= 1024) splits *= 2;
  return splits;
}

// ---- 13 to 256 rows of a wide matrix: the weights are what is read, once, at the speed of the memory.
// The pipelined kernel streams them best (transfers of three or four slabs in flight, no registers in
// between) when its tile covers all rows, so that a weight is read once, and is narrow enough, with K shared
// out over blocks, for about one block a compute unit: 64 x 128 (8 waves), 128 x 128 (8 waves) or 256 x 128
// tiles (8 waves) of 4, 4 and 3 stages.  A product that must come out whole (16-bit out: its consumer adds no
// pieces) and has few columns takes the 64- or 32-column sibling instead.
// (from 13 rows: with packed weights the tiles stream as fast as the matrix-vector kernels, whose time grows
// with every row beyond 8; 8B shape, a decoding step at batch 12 4.10 ms either way, at batch 16 4.30 -> 4.13, at
// batch 24 4.55 -> 4.10, at batch 32 4.74 -> 4.25)
#ifndef LQ_MID_ROWS_FROM
#define LQ_MID_ROWS_FROM 12
#endif
inline bool mid_rows(int M, int N, int K) {
  // (a head over a large vocabulary, a thousand tiles and more, stays with the matrix-vector kernel while one row
  // tile takes the rows: 1B shape at 16 rows 105 against 124 us)
  if (M <= 16 && N >= 128 * lq_compute_units()) return false;
  return M > LQ_MID_ROWS_FROM && M <= 256 && K % 64 == 0 && K >= 512 && N >= 8 * lq_compute_units();
}

inline int mid_splits_for(int tiles, int K) {
  const int want = 3 * lq_compute_units() / 4;
  int splits = 1;
  while (splits < 16 && tiles * splits < want && K % (128 * splits) == 0 && K / (2 * splits) >= 512) splits *= 2;
  return splits;
}

// Up to 64 rows, a product in pieces may take 64-column tiles (four waves) instead of 128-column ones (eight):
// as many blocks with half as many pieces for the consumer to add.  They are taken where they give more blocks,
// or as many when these fill every compute unit (then the chip's memory bounds the launch, and fewer pieces are
// what is left to gain: 8B shape at 64 rows, the norm after o and down 7.8 -> 6.9 us); where blocks are fewer
// than compute units a block's bytes in flight bound it, and the wide tile has twice as many (q, k and v at 64
// rows: 13.2 against 16.0 us).
inline bool mid_narrow(int M, int N, int K) {
  if (M > 64) return false;
  const int cus = lq_compute_units();
  const int wide = lq_ceil_div(N, 128) * mid_splits_for(lq_ceil_div(N, 128), K);
  const int narrow = lq_ceil_div(N, 64) * mid_splits_for(lq_ceil_div(N, 64), K);
  if (mid_splits_for(lq_ceil_div(N, 64), K) == 1) return false;  // whole: the 128-column tile or its siblings below
  return (narrow < cus ? narrow : cus) > (wide < cus ? wide : cus) || (narrow >= cus && wide >= cus);
}

int mid_splits(int M, int N, int K) {
  return mid_splits_for(lq_ceil_div(N, mid_narrow(M, N, K) ? 64 : 128), K);
}

template <int EPI, typename TO>
int launch_mid(const void* x, const void* w, void* out, int M, int N, int K, int lda, int ldw, int ldc, int splits,
               long long split_stride, hipStream_t stream, int packed) {
  // whole and with few columns: 64- or 32-column tiles (no epilogue pairs columns across them)
  if constexpr (EPI == EPI_NONE) {
    const int want = 3 * lq_compute_units() / 4;
    if (splits == 1 && lq_ceil_div(N, 64) < want) {
      if (M <= 64) return launch_pipelined<2, 1, 1, 1, 64, 4, EPI, TO>(x, w, out, M, N, K, lda, ldw, ldc, 1, 0, stream, packed);
      if (M <= 128) return launch_pipelined<4, 1, 1, 1, 64, 4, EPI, TO>(x, w, out, M, N, K, lda, ldw, ldc, 1, 0, stream, packed);
      return launch_pipelined<8, 1, 1, 1, 64, 3, EPI, TO>(x, w, out, M, N, K, lda, ldw, ldc, 1, 0, stream, packed);
    }
    if (splits == 1 && lq_ceil_div(N, 128) < want) {
      if (M <= 64) return launch_pipelined<2, 2, 1, 1, 64, 4, EPI, TO>(x, w, out, M, N, K, lda, ldw, ldc, 1, 0, stream, packed);
      if (M <= 128) return launch_pipelined<2, 2, 2, 1, 64, 4, EPI, TO>(x, w, out, M, N, K, lda, ldw, ldc, 1, 0, stream, packed);
      return launch_pipelined<4, 2, 2, 1, 64, 3, EPI, TO>(x, w, out, M, N, K, lda, ldw, ldc, 1, 0, stream, packed);
    }
  }
  if constexpr (EPI == EPI_NONE)
    if (splits > 1 && mid_narrow(M, N, K))
      return launch_pipelined<2, 2, 1, 1, 64, 4, EPI, TO>(x, w, out, M, N, K, lda, ldw, ldc, splits, split_stride, stream, packed);
  if (M <= 64)
    return launch_pipelined<2, 4, 1, 1, 64, 4, EPI, TO>(x, w, out, M, N, K, lda, ldw, ldc, splits, split_stride, stream, packed);
  if (M <= 128)
    return launch_pipelined<4, 2, 1, 2, 64, 4, EPI, TO>(x, w, out, M, N, K, lda, ldw, ldc, splits, split_stride, stream, packed);
  return launch_pipelined<4, 2, 2, 2, 64, 3, EPI, TO>(x, w, out, M, N, K, lda, ldw, ldc, splits, split_stride, stream, packed);
}

int mfma_splits(int M, int N, int K) {
  if (mid_rows(M, N, K)) return mid_splits(M, N, K);
  return M <= 64 ? v3_splits(M, N, K) : tiled_splits(M, N, K);
}

template <int EPI, typename TO>
int dispatch(const void* x, const void* w, void* out, int M, int N, int K, int lda, int ldw, int ldc,
             int splits, long long split_stride, hipStream_t stream, int packed) {
  // a packed weight is wide and has K in 64s (gemm_packable): every way below that it can take ends in the
  // pipelined kernel with slabs of 64 k or in the balanced one
  LQ_REQUIRE(!packed || gemm_packable(N, K), "linear: a %d x %d weight cannot be packed", N, K);
  if (splits > 1) {
    if (EPI != EPI_NONE || splits != mfma_splits(M, N, K)) {
      lq_set_error("linear: %d shares of K are not what this product takes (%d)", splits, mfma_splits(M, N, K));
      return -1;
    }
  }
  if (mid_rows(M, N, K)) return launch_mid<EPI, TO>(x, w, out, M, N, K, lda, ldw, ldc, splits, split_stride, stream, packed);
  if (splits > 1) {
    if (M <= 32) return launch_skinny_v3<2, EPI, TO>(x, w, out, M, N, K, lda, ldw, ldc, splits, split_stride, stream, packed);
    if (M <= 64) return launch_skinny_v3<4, EPI, TO>(x, w, out, M, N, K, lda, ldw, ldc, splits, split_stride, stream, packed);
    return launch_pipelined<4, 2, 2, 4, 64, 2, EPI, TO, true>(x, w, out, M, N, K, lda, ldw, ldc, splits, split_stride,
                                                              stream, packed);
  }
  // wide enough to give every compute unit a run of columns: the balanced kernel; else the simple one
  const bool wide = N >= 8 * lq_compute_units() && K >= 512;
  if (M <= 16) {
    if (wide) return launch_skinny_v3<1, EPI, TO>(x, w, out, M, N, K, lda, ldw, ldc, 1, 0, stream, packed);
    return pick_skinny<1, EPI, TO>(x, w, out, M, N, K, lda, ldw, ldc, stream);
  }
  if (M <= 32) {
    if (wide) return launch_skinny_v3<2, EPI, TO>(x, w, out, M, N, K, lda, ldw, ldc, 1, 0, stream, packed);
    return pick_skinny<2, EPI, TO>(x, w, out, M, N, K, lda, ldw, ldc, stream);
  }
  if (M <= 64) {
    if (wide) return launch_skinny_v3<4, EPI, TO>(x, w, out, M, N, K, lda, ldw, ldc, 1, 0, stream, packed);
    return pick_skinny<4, EPI, TO>(x, w, out, M, N, K, lda, ldw, ldc, stream);
  }
  // the largest tile that still fills the chip: 256 rows by 256, 224 or 192 columns (8 waves), 128 x 256
  // (4 waves, pipelined), then the register-staged kernels, which also take a K that is no multiple of 32
  const long long t256 = (long long)lq_ceil_div(M, 256) * lq_ceil_div(N, 256);
  const long long t128 = (long long)lq_ceil_div(M, 128) * lq_ceil_div(N, 256);
  if (K % 64 == 0 && fills_chip(t256)) {
    // Tiles run in rounds of one a compute unit; a narrower tile can save a round or fill a round that
    // a wider one leaves part empty.  Cost of a round relative to the 256-column tile, as measured.
    const int cus = lq_compute_units(), tm = lq_ceil_div(M, 256);
    // (A last round that is part empty costs less than a whole one, which the rounding up does not know: a
    // narrower tile has to win by a margin.)
    const double c256 = 0.95 * lq_ceil_div(tm * lq_ceil_div(N, 256), cus);
    const double c224 = 1.13 * lq_ceil_div(tm * lq_ceil_div(N, 224), cus);
    const double c192 = 0.78 * lq_ceil_div(tm * lq_ceil_div(N, 192), cus);
    if (c256 <= c224 && c256 <= c192) {
      // Whole rounds of 256-column tiles, and where what is left would fill half a round or less, that rest
      // as 128-column tiles in a launch of its own: a round of half-size tiles instead of a round of whole
      // tiles on half the chip (2 048 x 28 672: three rounds and 256 half tiles instead of 3.5 rounds).
      const int tn = lq_ceil_div(N, 256), rest = (tm * tn) % cus;
      if (N % 256 == 0 && tm * tn > cus && 4 * rest >= cus && rest % tm == 0 && 2 * rest <= cus + cus / 8) {
        const int n1 = (tn - rest / tm) * 256, n2 = N - n1;
        const int col2 = EPI == EPI_SWIGLU ? n1 / 2 : n1;  // where the second launch's columns start in out
        int rc = launch_pipelined<4, 2, 2, 4, 64, 2, EPI, TO, true>(x, w, out, M, n1, K, lda, ldw, ldc, 1, 0, stream, packed);
        if (rc != 0) return rc;
        return launch_pipelined<4, 2, 2, 2, 64, 2, EPI, TO, true>(x, (const bf16_t*)w + (long long)n1 * ldw,
                                                                  (TO*)out + col2, M, n2, K, lda, ldw, ldc, 1, 0, stream, packed);
      }
      return launch_pipelined<4, 2, 2, 4, 64, 2, EPI, TO, true>(x, w, out, M, N, K, lda, ldw, ldc, 1, 0, stream, packed);
    }
    if (c224 <= c192)
      return launch_pipelined<8, 1, 1, 7, 64, 2, EPI, TO>(x, w, out, M, N, K, lda, ldw, ldc, 1, 0, stream, packed);
    return launch_pipelined<4, 2, 2, 3, 64, 2, EPI, TO, true>(x, w, out, M, N, K, lda, ldw, ldc, 1, 0, stream, packed);
  }
  if (!packed && K % 32 == 0 && t128 >= lq_compute_units())
    return launch_pipelined<2, 2, 2, 4, 32, 3, EPI, TO>(x, w, out, M, N, K, lda, ldw, ldc, 1, 0, stream, packed);
  // few tiles even of 128 x 256 (some hundred rows of a narrow matrix): 128 x 128 tiles, four stages deep
  if (K % 64 == 0 && K >= 512)
    return launch_pipelined<4, 2, 1, 2, 64, 4, EPI, TO>(x, w, out, M, N, K, lda, ldw, ldc, 1, 0, stream, packed);
  if (t128 >= 2 * lq_compute_units()) return launch_tiled<2, 4, EPI, TO>(x, w, out, M, N, K, lda, ldw, ldc, stream);
  return launch_tiled<2, 2, EPI, TO>(x, w, out, M, N, K, lda, ldw, ldc, stream);
}

}  // namespace

int lq_gemm_mfma_splits(int M, int N, int K) { return mfma_splits(M, N, K); }

// The decode pair around a norm.  `residual`: x[M, N] (float32) += act[M, K] . w[N, K]^T; sq_out[M][parts]
// takes each row's sum of squares over a block's columns, and, with a gain, scaled[M, N] takes
// bfloat16(x * gain), the input of the product after the norm.  `scaled`: out = rstd(row) * (h . w^T) with
// rstd from those parts, optionally through the SwiGLU epilogue.  Both are the balanced kernel with one
// row tile; lq_gemm_fused_parts says how many parts it leaves (0: this size is not taken).
int lq_gemm_fused_parts(int M, int N, int K) {
  if (M < 1 || M > 16 || mid_rows(M, N, K) || !(N >= 8 * lq_compute_units() && K >= 512) || K % 8 != 0) return 0;
  int cols, grid;
  v3_runs(N, lq_compute_units(), 8, cols, grid);
  return grid;
}

int lq_gemm_residual(const void* act, const void* w, float* x, float* sq_out, const float* gain, void* scaled,
                     int ld_scaled, int M, int N, int K, int lda, int ldw, int ldx, int packed, hipStream_t stream) {
  ResidualOut res;
  res.sq_out = sq_out;
  res.gain = gain;
  res.scaled = (bf16_t*)scaled;
  res.ld_scaled = ld_scaled;
  return launch_skinny_v3<1, EPI_RESIDUAL, float>(act, w, x, M, N, K, lda, ldw, ldx, 1, 0, stream, packed, RowScale(), res);
}

int lq_gemm_scaled(const void* h, int ldh, const float* sq_parts, int n_parts, int width, float eps, const void* w,
                   void* out, int out_dtype, int M, int N, int K, int ldw, int ldc, int swiglu, int packed,
                   hipStream_t stream) {
  RowScale sc;
  sc.sq_parts = sq_parts;
  sc.n_parts = n_parts;
  sc.width = width;
  sc.eps = eps;
  if (swiglu) {
    if (out_dtype == LQ_BF16)
      return launch_skinny_v3<1, EPI_SWIGLU, bf16_t, true>(h, w, out, M, N, K, ldh, ldw, ldc, 1, 0, stream, packed, sc);
    if (out_dtype == LQ_F32)
      return launch_skinny_v3<1, EPI_SWIGLU, float, true>(h, w, out, M, N, K, ldh, ldw, ldc, 1, 0, stream, packed, sc);
  } else {
    if (out_dtype == LQ_BF16)
      return launch_skinny_v3<1, EPI_NONE, bf16_t, true>(h, w, out, M, N, K, ldh, ldw, ldc, 1, 0, stream, packed, sc);
    if (out_dtype == LQ_F32)
      return launch_skinny_v3<1, EPI_NONE, float, true>(h, w, out, M, N, K, ldh, ldw, ldc, 1, 0, stream, packed, sc);
  }
  lq_set_error("linear: unknown output dtype %d", out_dtype);
  return -1;
}

// Whether the MFMA kernels take this problem (the caller falls back to the generic kernel if not).
bool lq_gemm_mfma_accepts(const void* x, const void* w, int in_dtype, int K, int lda, int ldw) {
  return in_dtype == LQ_BF16 && K % 8 == 0 && lda % 8 == 0 && ldw % 8 == 0 &&
         ((uintptr_t)x % 16) == 0 && ((uintptr_t)w % 16) == 0;
}

bool lq_gemm_packable(int N, int K) { return gemm_packable(N, K); }

int lq_gemm_mfma(const void* x, const void* w, void* out, int out_dtype, int M, int N, int K, int lda,
                 int ldw, int ldc, int epilogue, int splits, long long split_stride, int packed, hipStream_t stream) {
  if (epilogue == EPI_NONE) {
    if (out_dtype == LQ_F32)
      return dispatch<EPI_NONE, float>(x, w, out, M, N, K, lda, ldw, ldc, splits, split_stride, stream, packed);
    if (out_dtype == LQ_BF16)
      return dispatch<EPI_NONE, bf16_t>(x, w, out, M, N, K, lda, ldw, ldc, splits, split_stride, stream, packed);
  } else if (epilogue == EPI_SWIGLU) {
    if (N % 16 != 0) {
      lq_set_error("linear+swiglu: %d interleaved rows are not a multiple of 16", N);
      return -1;
    }
    if (out_dtype == LQ_F32) return dispatch<EPI_SWIGLU, float>(x, w, out, M, N, K, lda, ldw, ldc, 1, 0, stream, packed);
    if (out_dtype == LQ_BF16) return dispatch<EPI_SWIGLU, bf16_t>(x, w, out, M, N, K, lda, ldw, ldc, 1, 0, stream, packed);
  }
  lq_set_error("linear: unknown out dtype %d or epilogue %d", out_dtype, epilogue);
  return -1;
}
