// Row-wise kernels of the decoder: embedding rows, RMSNorm (with the residual
// add folded in), rotation + cache write, SwiGLU, residual add, row gather, casts.
// Norm statistics, rotation angles and the residual sum are 32-bit (or wider).
#include "common.h"
#include <algorithm>

// ---------------------------------------------------------------- embedding
// out[r, :] = float(table[token[r], :])   (row copy, internal/device/kernels.metal:465-467)
// A token that is no row of the table (a replayed step can be handed the sampler's "no token" before the
// host has seen it) gives a row of zeros: nothing outside the table is read.
// A packed table (the layout of lq_pack_weight, for a table that is also the head's weight) keeps 8 rows'
// slabs of 64 elements side by side: element k of row n lies at (n / 8) 8 D + (k / 64) 512 + (n % 8) 64 + k % 64.
template <typename T>
__global__ void embed_kernel(const T* __restrict__ table, const int* __restrict__ tokens,
                             float* __restrict__ out, int D, int vocab, int packed) {
  const int r = blockIdx.x;
  const long long tok = tokens[r];
  const bool known = tok >= 0 && tok < vocab;
  const long long row = known ? tok : 0;
  const T* src = packed ? table + (row >> 3) * 8 * (long long)D + (row & 7) * 64 : table + row * (long long)D;
  float* dst = out + (long long)r * D;
  for (int j = threadIdx.x; j < D; j += blockDim.x)
    dst[j] = known ? to_f32(src[packed ? ((j >> 6) << 9) + (j & 63) : j]) : 0.0f;
}

// A bfloat16 row of a width that is a multiple of 8, 16 bytes a lane and load: all of a thread's loads are on
// their way before its first store (the loop above waits for every element in turn: 9.4 us for a step's eight
// rows of 4 096, this 4).
typedef unsigned embed_u32x4 __attribute__((ext_vector_type(4)));
typedef float embed_f32x4 __attribute__((ext_vector_type(4)));
template <int PER_THREAD>
__global__ __launch_bounds__(256) void embed_bf16_vec_kernel(const bf16_t* __restrict__ table,
                                                             const int* __restrict__ tokens, float* __restrict__ out,
                                                             int D, int vocab, int packed) {
  const int r = blockIdx.x;
  const long long tok = tokens[r];
  const bool known = tok >= 0 && tok < vocab;
  const long long row = known ? tok : 0;
  // (chunk c of 8 elements: packed, 8 chunks of a row every 64 chunks)
  const embed_u32x4* src = (const embed_u32x4*)(packed ? table + (row >> 3) * 8 * (long long)D + (row & 7) * 64
                                                       : table + row * (long long)D);
  embed_f32x4* dst = (embed_f32x4*)(out + (long long)r * D);
  const int chunks = D / 8;
  embed_u32x4 v[PER_THREAD];
#pragma unroll
  for (int i = 0; i < PER_THREAD; ++i) {
    const int c = threadIdx.x + i * 256;
    v[i] = (c < chunks && known) ? src[packed ? ((c >> 3) << 6) + (c & 7) : c] : (embed_u32x4){0u, 0u, 0u, 0u};
  }
#pragma unroll
  for (int i = 0; i < PER_THREAD; ++i) {
    const int c = threadIdx.x + i * 256;
    if (c < chunks) {
      dst[2 * c] = (embed_f32x4){__uint_as_float(v[i][0] << 16), __uint_as_float(v[i][0] & 0xffff0000u),
                                 __uint_as_float(v[i][1] << 16), __uint_as_float(v[i][1] & 0xffff0000u)};
      dst[2 * c + 1] = (embed_f32x4){__uint_as_float(v[i][2] << 16), __uint_as_float(v[i][2] & 0xffff0000u),
                                     __uint_as_float(v[i][3] << 16), __uint_as_float(v[i][3] & 0xffff0000u)};
    }
  }
}

extern "C" int lq_embed(const void* table, int table_dtype, const int* tokens, float* out, int rows,
                        int D, int vocab, int packed, hipStream_t stream) {
  LQ_REQUIRE(rows > 0 && D > 0 && vocab > 0, "embed: rows %d, width %d and table rows %d must be positive", rows, D, vocab);
  LQ_REQUIRE(!packed || (D % 64 == 0 && vocab % 8 == 0), "embed: a packed table has rows in eights and a width in 64s");
  const int threads = D >= 1024 ? 256 : 64;
  if (table_dtype == LQ_BF16 && D % 8 == 0 && D >= 2048 && D <= 8 * 256 * 8 && (uintptr_t)table % 16 == 0 &&
      (uintptr_t)out % 16 == 0) {
    if (D <= 8 * 256 * 2)
      embed_bf16_vec_kernel<2><<<rows, 256, 0, stream>>>((const bf16_t*)table, tokens, out, D, vocab, packed);
    else if (D <= 8 * 256 * 4)
      embed_bf16_vec_kernel<4><<<rows, 256, 0, stream>>>((const bf16_t*)table, tokens, out, D, vocab, packed);
    else
      embed_bf16_vec_kernel<8><<<rows, 256, 0, stream>>>((const bf16_t*)table, tokens, out, D, vocab, packed);
    LQ_CHECK_LAUNCH("embed");
    return 0;
  }
  if (table_dtype == LQ_F32)
    embed_kernel<float><<<rows, threads, 0, stream>>>((const float*)table, tokens, out, D, vocab, packed);
  else if (table_dtype == LQ_BF16)
    embed_kernel<bf16_t><<<rows, threads, 0, stream>>>((const bf16_t*)table, tokens, out, D, vocab, packed);
  else
    LQ_REQUIRE(false, "embed: unknown table dtype %d", table_dtype);
  LQ_CHECK_LAUNCH("embed");
  return 0;
}

// ---------------------------------------------------------------- packed weights
// dst = src [N, K] with 8 rows' slabs of 64 k side by side: element k of row n at
// (n / 8) 8 K + (k / 64) 512 + (n % 8) 64 + k % 64.  A kernel that fetches a slab of 64 k of 8 (or 128) rows
// then reads one run of 1 KiB (16 KiB) instead of 128 bytes from each of 8 (128) places a row apart, and the
// next slab is the next KiB: what the memory gives whole pages for.  N % 8 == 0, K % 64 == 0; 16 bytes a thread.
__global__ __launch_bounds__(256) void pack_weight_kernel(const embed_u32x4* __restrict__ src,
                                                          embed_u32x4* __restrict__ dst, long long chunks, int K) {
  const long long c = (long long)blockIdx.x * 256 + threadIdx.x;  // chunk of 8 elements, in the order of dst
  if (c >= chunks) return;
  const long long per8 = (long long)K;       // chunks in 8 rows: 8 K / 8
  const long long group = c / per8, in = c - group * per8;
  const int slab = (int)(in >> 6), row = (int)(in >> 3) & 7, part = (int)in & 7;
  dst[c] = src[((group * 8 + row) * (long long)K + slab * 64 + part * 8) >> 3];
}

extern "C" int lq_pack_weight(const void* src, void* dst, int N, int K, hipStream_t stream) {
  LQ_REQUIRE(src && dst && src != dst, "pack_weight: two different buffers");
  LQ_REQUIRE(N > 0 && K > 0 && N % 8 == 0 && K % 64 == 0, "pack_weight: %d rows in eights, %d columns in 64s", N, K);
  LQ_REQUIRE((uintptr_t)src % 16 == 0 && (uintptr_t)dst % 16 == 0, "pack_weight: 16-byte aligned buffers");
  const long long chunks = (long long)N * K / 8;
  LQ_REQUIRE((chunks + 255) / 256 < (1ll << 31), "pack_weight: too large");
  pack_weight_kernel<<<(unsigned)((chunks + 255) / 256), 256, 0, stream>>>((const embed_u32x4*)src, (embed_u32x4*)dst,
                                                                           chunks, K);
  LQ_CHECK_LAUNCH("pack_weight");
  return 0;
}

// ---------------------------------------------------------------- RMSNorm
// Per row: (x += delta, written back, if delta is given), s = sum x^2,
// r = 1 / sqrt(s / D + eps), out = x * r * w.  eps inside the root, weight
// after normalisation (internal/device/kernels.metal:905-942).
// delta may come in `parts` pieces (the partial sums of a product whose K was split over blocks),
// `part_stride` elements apart; they are added in ascending order.
template <typename TD, typename TO, bool HAS_DELTA>
__global__ void rmsnorm_kernel(float* __restrict__ x, const TD* __restrict__ delta, int parts,
                               long long part_stride, const float* __restrict__ w, TO* __restrict__ out, int D,
                               float eps) {
  __shared__ float red[16];
  const long long base = (long long)blockIdx.x * D;
  float ss = 0.f;
  for (int j = threadIdx.x; j < D; j += blockDim.x) {
    float v = x[base + j];
    if (HAS_DELTA) {
      for (int s = 0; s < parts; ++s) v += to_f32(delta[s * part_stride + base + j]);
      x[base + j] = v;
    }
    ss += v * v;
  }
  ss = block_sum(ss, red);
  const float r = 1.0f / sqrtf(ss / (float)D + eps);
  for (int j = threadIdx.x; j < D; j += blockDim.x) {
    // each thread re-reads what it wrote itself: no barrier needed
    out[base + j] = from_f32<TO>(x[base + j] * r * w[j]);
  }
}

// The same, for rows that fit the block's registers: width a multiple of 4 and at most
// 256 threads * NV * 4.  One read of x (and delta), one write of each output.
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2_t __attribute__((ext_vector_type(2)));

__device__ inline f32x4_t load4(const float* p) { return *(const f32x4_t*)p; }
__device__ inline f32x4_t load4(const bf16_t* p) {
  const u32x2_t r = *(const u32x2_t*)p;
  f32x4_t v;
  v[0] = __uint_as_float(r[0] << 16);
  v[1] = __uint_as_float(r[0] & 0xffff0000u);
  v[2] = __uint_as_float(r[1] << 16);
  v[3] = __uint_as_float(r[1] & 0xffff0000u);
  return v;
}
__device__ inline void store4(float* p, f32x4_t v) { *(f32x4_t*)p = v; }
__device__ inline void store4(bf16_t* p, f32x4_t v) {
  u32x2_t r;
  r[0] = (unsigned)f32_to_bf16(v[0]).bits | ((unsigned)f32_to_bf16(v[1]).bits << 16);
  r[1] = (unsigned)f32_to_bf16(v[2]).bits | ((unsigned)f32_to_bf16(v[3]).bits << 16);
  *(u32x2_t*)p = r;
}

// MANY: the delta comes in more than two pieces (few rows of a product whose K many blocks share): such a
// launch is bound by the latency of its loads, not by their number, and asks for four pieces of all of a
// thread's elements together.  Many rows with one or two pieces stream, and want few registers instead.
template <typename TD, typename TO, bool HAS_DELTA, int NV, bool MANY>
__global__ __launch_bounds__(256) void rmsnorm_regs_kernel(float* __restrict__ x, const TD* __restrict__ delta,
                                                           int parts, long long part_stride,
                                                           const float* __restrict__ w, TO* __restrict__ out,
                                                           int D, float eps) {
  __shared__ float red[16];
  const long long base = (long long)blockIdx.x * D;
  f32x4_t v[NV];
  float ss = 0.f;
  if constexpr (!MANY) {
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int j = (threadIdx.x + i * 256) * 4;
      if (j < D) {
        v[i] = load4(x + base + j);
        if (HAS_DELTA) {
          for (int s = 0; s < parts; ++s) v[i] += load4(delta + s * part_stride + base + j);
          store4(x + base + j, v[i]);
        }
        ss += v[i][0] * v[i][0] + v[i][1] * v[i][1] + v[i][2] * v[i][2] + v[i][3] * v[i][3];
      }
    }
  } else {
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int j = (threadIdx.x + i * 256) * 4;
      if (j < D) v[i] = load4(x + base + j);
    }
    // the pieces are added in ascending order, element by element, as above
    int s = 0;
    for (; s + 4 <= parts; s += 4) {
      f32x4_t d[4][NV];
#pragma unroll
      for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int i = 0; i < NV; ++i) {
          const int j = (threadIdx.x + i * 256) * 4;
          if (j < D) d[q][i] = load4(delta + (s + q) * part_stride + base + j);
        }
#pragma unroll
      for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int i = 0; i < NV; ++i) {
          const int j = (threadIdx.x + i * 256) * 4;
          if (j < D) v[i] += d[q][i];
        }
    }
    for (; s < parts; ++s) {
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        const int j = (threadIdx.x + i * 256) * 4;
        if (j < D) v[i] += load4(delta + s * part_stride + base + j);
      }
    }
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int j = (threadIdx.x + i * 256) * 4;
      if (j < D) {
        store4(x + base + j, v[i]);
        ss += v[i][0] * v[i][0] + v[i][1] * v[i][1] + v[i][2] * v[i][2] + v[i][3] * v[i][3];
      }
    }
  }
  ss = block_sum(ss, red);
  const float r = 1.0f / sqrtf(ss / (float)D + eps);
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int j = (threadIdx.x + i * 256) * 4;
    if (j < D) store4(out + base + j, v[i] * r * load4(w + j));
  }
}

template <typename TD, typename TO, bool HAS>
static void rmsnorm_launch(float* x, const void* delta, int parts, long long part_stride, const float* w, void* out,
                           int rows, int D, float eps, hipStream_t stream) {
  const bool aligned = D % 4 == 0 && ((uintptr_t)x % 16) == 0 && ((uintptr_t)out % 16) == 0 &&
                       ((uintptr_t)w % 16) == 0 && ((uintptr_t)delta % 16) == 0 && part_stride % 4 == 0;
  const int vecs = (D / 4 + 255) / 256;
  if (aligned && vecs <= 8) {
#define LQ_REGS(NV)                                                                                              \
  do {                                                                                                           \
    if (HAS && parts > 2)                                                                                        \
      rmsnorm_regs_kernel<TD, TO, HAS, NV, true><<<rows, 256, 0, stream>>>(x, (const TD*)delta, parts,           \
                                                                           part_stride, w, (TO*)out, D, eps);    \
    else                                                                                                         \
      rmsnorm_regs_kernel<TD, TO, HAS, NV, false><<<rows, 256, 0, stream>>>(x, (const TD*)delta, parts,          \
                                                                            part_stride, w, (TO*)out, D, eps);   \
  } while (0)
    if (vecs <= 1)
      LQ_REGS(1);
    else if (vecs <= 2)
      LQ_REGS(2);
    else if (vecs <= 4)
      LQ_REGS(4);
    else
      LQ_REGS(8);
#undef LQ_REGS
    return;
  }
  const int threads = D >= 2048 ? 512 : (D >= 512 ? 256 : 64);
  rmsnorm_kernel<TD, TO, HAS><<<rows, threads, 0, stream>>>(x, (const TD*)delta, parts, part_stride, w, (TO*)out, D,
                                                            eps);
}

extern "C" int lq_rmsnorm(float* x, const void* delta, int delta_dtype, int parts, long long part_stride,
                          const float* w, float eps, void* out, int out_dtype, int rows, int D,
                          hipStream_t stream) {
  LQ_REQUIRE(rows > 0 && D > 0, "rmsnorm: rows %d and width %d must be positive", rows, D);
  LQ_REQUIRE(delta == nullptr || (parts >= 1 && (parts == 1 || part_stride >= (long long)rows * D)),
             "rmsnorm: %d delta parts with stride %lld", parts, part_stride);
  LQ_REQUIRE(out_dtype == LQ_F32 || out_dtype == LQ_BF16, "rmsnorm: unknown out dtype %d", out_dtype);
#define LQ_NORM_LAUNCH(TD, TO, HAS) \
  rmsnorm_launch<TD, TO, HAS>(x, delta, parts, part_stride, w, out, rows, D, eps, stream)
  if (delta == nullptr) {
    if (out_dtype == LQ_F32)
      LQ_NORM_LAUNCH(float, float, false);
    else
      LQ_NORM_LAUNCH(float, bf16_t, false);
  } else if (delta_dtype == LQ_F32) {
    if (out_dtype == LQ_F32)
      LQ_NORM_LAUNCH(float, float, true);
    else
      LQ_NORM_LAUNCH(float, bf16_t, true);
  } else if (delta_dtype == LQ_BF16) {
    if (out_dtype == LQ_F32)
      LQ_NORM_LAUNCH(bf16_t, float, true);
    else
      LQ_NORM_LAUNCH(bf16_t, bf16_t, true);
  } else {
    LQ_REQUIRE(false, "rmsnorm: unknown delta dtype %d", delta_dtype);
  }
#undef LQ_NORM_LAUNCH
  LQ_CHECK_LAUNCH("rmsnorm");
  return 0;
}

// ---------------------------------------------------------------- residual add
template <typename TD>
__global__ void add_kernel(float* __restrict__ x, const TD* __restrict__ delta, long long n) {
  long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (; i < n; i += stride) x[i] += to_f32(delta[i]);
}

extern "C" int lq_add(float* x, const void* delta, int delta_dtype, long long n, hipStream_t stream) {
  LQ_REQUIRE(n > 0, "add: count %lld must be positive", n);
  const int threads = 256;
  const int blocks = (int)(lq_ceil_div64(n, threads) < 8192 ? lq_ceil_div64(n, threads) : 8192);
  if (delta_dtype == LQ_F32)
    add_kernel<float><<<blocks, threads, 0, stream>>>(x, (const float*)delta, n);
  else if (delta_dtype == LQ_BF16)
    add_kernel<bf16_t><<<blocks, threads, 0, stream>>>(x, (const bf16_t*)delta, n);
  else
    LQ_REQUIRE(false, "add: unknown delta dtype %d", delta_dtype);
  LQ_CHECK_LAUNCH("add");
  return 0;
}

// ---------------------------------------------------------------- casts
template <typename TI, typename TO>
__global__ void cast_kernel(const TI* __restrict__ in, TO* __restrict__ out, long long n) {
  long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (; i < n; i += stride) out[i] = from_f32<TO>(to_f32(in[i]));
}

extern "C" int lq_cast(const void* in, int in_dtype, void* out, int out_dtype, long long n,
                       hipStream_t stream) {
  LQ_REQUIRE(n > 0, "cast: count %lld must be positive", n);
  const int threads = 256;
  const int blocks = (int)(lq_ceil_div64(n, threads) < 8192 ? lq_ceil_div64(n, threads) : 8192);
  if (in_dtype == LQ_F32 && out_dtype == LQ_BF16)
    cast_kernel<float, bf16_t><<<blocks, threads, 0, stream>>>((const float*)in, (bf16_t*)out, n);
  else if (in_dtype == LQ_BF16 && out_dtype == LQ_F32)
    cast_kernel<bf16_t, float><<<blocks, threads, 0, stream>>>((const bf16_t*)in, (float*)out, n);
  else
    LQ_REQUIRE(false, "cast: unsupported pair %d -> %d", in_dtype, out_dtype);
  LQ_CHECK_LAUNCH("cast");
  return 0;
}

// ---------------------------------------------------------------- SwiGLU
// out[r, i] = silu(g) * u with g = gu[r, i], u = gu[r, I + i], silu(g) = g / (1 + e^-g).
// No clamps (internal/device/cpu_ref.go:132-149).
template <typename TI, typename TO>
__global__ void swiglu_kernel(const TI* __restrict__ gu, TO* __restrict__ out, int I, long long n) {
  long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (; i < n; i += stride) {
    const long long r = i / I;
    const int c = (int)(i - r * I);
    const float g = to_f32(gu[r * 2 * I + c]);
    const float u = to_f32(gu[r * 2 * I + I + c]);
    out[i] = from_f32<TO>(g / (1.0f + expf(-g)) * u);
  }
}

extern "C" int lq_swiglu(const void* gu, int in_dtype, void* out, int out_dtype, int rows, int I,
                         hipStream_t stream) {
  LQ_REQUIRE(rows > 0 && I > 0, "swiglu: rows %d and width %d must be positive", rows, I);
  const long long n = (long long)rows * I;
  const int threads = 256;
  const int blocks = (int)(lq_ceil_div64(n, threads) < 16384 ? lq_ceil_div64(n, threads) : 16384);
#define LQ_SWIGLU_LAUNCH(TI, TO) \
  swiglu_kernel<TI, TO><<<blocks, threads, 0, stream>>>((const TI*)gu, (TO*)out, I, n)
  if (in_dtype == LQ_F32 && out_dtype == LQ_F32)
    LQ_SWIGLU_LAUNCH(float, float);
  else if (in_dtype == LQ_F32 && out_dtype == LQ_BF16)
    LQ_SWIGLU_LAUNCH(float, bf16_t);
  else if (in_dtype == LQ_BF16 && out_dtype == LQ_BF16)
    LQ_SWIGLU_LAUNCH(bf16_t, bf16_t);
  else
    LQ_REQUIRE(false, "swiglu: unsupported dtypes %d -> %d", in_dtype, out_dtype);
#undef LQ_SWIGLU_LAUNCH
  LQ_CHECK_LAUNCH("swiglu");
  return 0;
}

// ---------------------------------------------------------------- row gather
// out[i, :] = x[rows[i], :] (+ delta[rows[i], :]); picks the rows whose logits
// are wanted before the final norm, carrying a not yet applied residual delta.
template <typename TD, bool HAS_DELTA>
__global__ void gather_rows_kernel(const float* __restrict__ x, const TD* __restrict__ delta, int parts,
                                   long long part_stride, const int* __restrict__ rows, float* __restrict__ out,
                                   int D) {
  const long long src = (long long)rows[blockIdx.x] * D;
  const long long dst = (long long)blockIdx.x * D;
  // (a launch of a few rows is bound by the latency of its loads: those of four turns are asked for together)
#pragma unroll 4
  for (int j = threadIdx.x; j < D; j += blockDim.x) {
    float v = x[src + j];
    if (HAS_DELTA) {
      // ascending order; four pieces are asked for together
      int s = 0;
      for (; s + 4 <= parts; s += 4) {
        const float d0 = to_f32(delta[s * part_stride + src + j]);
        const float d1 = to_f32(delta[(s + 1) * part_stride + src + j]);
        const float d2 = to_f32(delta[(s + 2) * part_stride + src + j]);
        const float d3 = to_f32(delta[(s + 3) * part_stride + src + j]);
        v += d0;
        v += d1;
        v += d2;
        v += d3;
      }
      for (; s < parts; ++s) v += to_f32(delta[s * part_stride + src + j]);
    }
    out[dst + j] = v;
  }
}

extern "C" int lq_gather_rows(const float* x, const void* delta, int delta_dtype, int parts, long long part_stride,
                              const int* rows, float* out, int n, int D, hipStream_t stream) {
  LQ_REQUIRE(n > 0 && D > 0, "gather_rows: count %d and width %d must be positive", n, D);
  const int threads = D >= 1024 ? 256 : 64;
  if (delta == nullptr)
    gather_rows_kernel<float, false><<<n, threads, 0, stream>>>(x, nullptr, 0, 0, rows, out, D);
  else if (delta_dtype == LQ_F32)
    gather_rows_kernel<float, true><<<n, threads, 0, stream>>>(x, (const float*)delta, parts, part_stride, rows, out, D);
  else if (delta_dtype == LQ_BF16)
    gather_rows_kernel<bf16_t, true><<<n, threads, 0, stream>>>(x, (const bf16_t*)delta, parts, part_stride, rows, out, D);
  else
    LQ_REQUIRE(false, "gather_rows: unknown delta dtype %d", delta_dtype);
  LQ_CHECK_LAUNCH("gather_rows");
  return 0;
}

// ---------------------------------------------------------------- rotation + cache write
// One block per row.  The row's position p comes from row_pos; its angles
// p * f_i are formed and reduced modulo 2 pi in double from the double table f
// (hd/2 entries), so the rotation is exact to 32-bit rounding at any position.  Pair (i, i + hd/2):
//   x_i' = x_i cos - x_{i+hd/2} sin ; x_{i+hd/2}' = x_i sin + x_{i+hd/2} cos
// (internal/device/kernels.metal:430-463).  q is rotated in place; rotated k
// and plain v go to the paged cache (internal/device/kernels.metal:1736-1749
// writes row p; here the row is found through the slot's block table):
//   K[block][kv head][offset][hd]      V[block][kv head][hd][offset]
// with block = table[slot][p / BS], offset = p % BS.
template <typename T>
__global__ void rope_store_kernel(T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v,
                                  int ldq, int ldk, int ldv, int nh, int nkv, int hd,
                                  const double* __restrict__ freqs, int has_rope,
                                  const int* __restrict__ row_pos, const int* __restrict__ row_seq,
                                  const int* __restrict__ seq_slot,
                                  const int* __restrict__ block_table, int bt_stride,
                                  T* __restrict__ kcache, T* __restrict__ vcache, int BS,
                                  int store) {
  extern __shared__ float cs[];  // cos[hd/2], sin[hd/2]
  const int r = blockIdx.x;
  const int half = hd / 2;
  const int p = row_pos[r];
  if (has_rope) {
    for (int i = threadIdx.x; i < half; i += blockDim.x) {
      // angle and its reduction to [-pi, pi] in double, sine and cosine of the remainder in 32-bit
      const double a = (double)p * freqs[i];
      const double n = rint(a * 0.15915494309189533577);
      double r = fma(-n, 6.283185307179586232, a);
      r = fma(-n, 2.4492935982947064e-16, r);
      float sn, c;
      sincosf((float)r, &sn, &c);
      cs[i] = c;
      cs[half + i] = sn;
    }
  } else {
    for (int i = threadIdx.x; i < half; i += blockDim.x) {
      cs[i] = 1.0f;
      cs[half + i] = 0.0f;
    }
  }
  __syncthreads();

  T* qr = q + (long long)r * ldq;
  for (int idx = threadIdx.x; idx < nh * half; idx += blockDim.x) {
    const int h = idx / half, i = idx - h * half;
    const float x0 = to_f32(qr[h * hd + i]);
    const float x1 = to_f32(qr[h * hd + i + half]);
    const float c = cs[i], s = cs[half + i];
    qr[h * hd + i] = from_f32<T>(x0 * c - x1 * s);
    qr[h * hd + i + half] = from_f32<T>(x0 * s + x1 * c);
  }
  if (!store) return;

  const int slot = seq_slot[row_seq[r]];
  const long long blk = block_table[(long long)slot * bt_stride + p / BS];
  const int off = p % BS;
  const T* kr = k + (long long)r * ldk;
  const T* vr = v + (long long)r * ldv;
  for (int idx = threadIdx.x; idx < nkv * half; idx += blockDim.x) {
    const int h = idx / half, i = idx - h * half;
    const float x0 = to_f32(kr[h * hd + i]);
    const float x1 = to_f32(kr[h * hd + i + half]);
    const float c = cs[i], s = cs[half + i];
    T* dst = kcache + ((blk * nkv + h) * BS + off) * (long long)hd;
    dst[i] = from_f32<T>(x0 * c - x1 * s);
    dst[i + half] = from_f32<T>(x0 * s + x1 * c);
  }
  for (int idx = threadIdx.x; idx < nkv * hd; idx += blockDim.x) {
    const int h = idx / hd, d = idx - h * hd;
    vcache[((blk * nkv + h) * hd + d) * (long long)BS + off] = vr[h * hd + d];
  }
}

// The same for bfloat16 rows that can be moved 16 bytes at a time (head size a multiple of 16, aligned
// rows): a thread takes 8 pairs, the pair (i, i + hd/2) from two loads, with the same 32-bit arithmetic.
typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));

__device__ inline void rotate8(u32x4_t& a, u32x4_t& b, const float* c, const float* s) {
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const float x0a = __uint_as_float(a[j] << 16), x0b = __uint_as_float(a[j] & 0xffff0000u);
    const float x1a = __uint_as_float(b[j] << 16), x1b = __uint_as_float(b[j] & 0xffff0000u);
    const float ca = c[2 * j], cb = c[2 * j + 1], sa = s[2 * j], sb = s[2 * j + 1];
    // one rounded product and one fused multiply-add, spelt out: left to the compiler, which of the two
    // products is fused differs from one caller to the next, and so does the last bit where they cancel
    const float ra = __fmaf_rn(x0a, ca, -__fmul_rn(x1a, sa)), rb = __fmaf_rn(x0b, cb, -__fmul_rn(x1b, sb));
    const float ia = __fmaf_rn(x0a, sa, __fmul_rn(x1a, ca)), ib = __fmaf_rn(x0b, sb, __fmul_rn(x1b, cb));
    a[j] = (unsigned)f32_to_bf16(ra).bits | ((unsigned)f32_to_bf16(rb).bits << 16);
    b[j] = (unsigned)f32_to_bf16(ia).bits | ((unsigned)f32_to_bf16(ib).bits << 16);
  }
}

__global__ __launch_bounds__(256) void rope_store_vec_kernel(
    bf16_t* __restrict__ q, const bf16_t* __restrict__ k, const bf16_t* __restrict__ v, int ldq, int ldk, int ldv,
    int nh, int nkv, int hd, const double* __restrict__ freqs, int has_rope, const int* __restrict__ row_pos,
    const int* __restrict__ row_seq, const int* __restrict__ seq_slot, const int* __restrict__ block_table,
    int bt_stride, bf16_t* __restrict__ kcache, bf16_t* __restrict__ vcache, int BS, int store) {
  extern __shared__ float cs[];  // cos[hd/2], sin[hd/2]
  const int r = blockIdx.x;
  const int half = hd / 2, hv = half / 8;
  const int p = row_pos[r];
  // what the cache write needs is asked for before the angles are worked out
  long long blk = 0;
  if (store) blk = block_table[(long long)seq_slot[row_seq[r]] * bt_stride + p / BS];
  for (int i = threadIdx.x; i < half; i += blockDim.x) {
    float c = 1.0f, sn = 0.0f;
    if (has_rope) {
      const double a = (double)p * freqs[i];
      const double n = rint(a * 0.15915494309189533577);
      double rem = fma(-n, 6.283185307179586232, a);
      rem = fma(-n, 2.4492935982947064e-16, rem);
      sincosf((float)rem, &sn, &c);
    }
    cs[i] = c;
    cs[half + i] = sn;
  }
  __syncthreads();
  bf16_t* qr = q + (long long)r * ldq;
  for (int idx = threadIdx.x; idx < nh * hv; idx += blockDim.x) {
    const int h = idx / hv, i = (idx - h * hv) * 8;
    u32x4_t a = *(const u32x4_t*)(qr + h * hd + i), b = *(const u32x4_t*)(qr + h * hd + half + i);
    rotate8(a, b, cs + i, cs + half + i);
    *(u32x4_t*)(qr + h * hd + i) = a;
    *(u32x4_t*)(qr + h * hd + half + i) = b;
  }
  if (!store) return;
  const int off = p % BS;
  const bf16_t* kr = k + (long long)r * ldk;
  const bf16_t* vr = v + (long long)r * ldv;
  for (int idx = threadIdx.x; idx < nkv * hv; idx += blockDim.x) {
    const int h = idx / hv, i = (idx - h * hv) * 8;
    u32x4_t a = *(const u32x4_t*)(kr + h * hd + i), b = *(const u32x4_t*)(kr + h * hd + half + i);
    rotate8(a, b, cs + i, cs + half + i);
    bf16_t* dst = kcache + ((blk * nkv + h) * BS + off) * (long long)hd;
    *(u32x4_t*)(dst + i) = a;
    *(u32x4_t*)(dst + half + i) = b;
  }
  for (int idx = threadIdx.x; idx < nkv * 2 * hv; idx += blockDim.x) {
    const int h = idx / (2 * hv), d = (idx - h * 2 * hv) * 8;
    const u32x4_t x = *(const u32x4_t*)(vr + h * hd + d);
    bf16_t* dst = vcache + ((blk * nkv + h) * hd + d) * (long long)BS + off;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      bf16_t lo, hi;
      lo.bits = (uint16_t)(x[j] & 0xffffu);
      hi.bits = (uint16_t)(x[j] >> 16);
      dst[(long long)(2 * j) * BS] = lo;
      dst[(long long)(2 * j + 1) * BS] = hi;
    }
  }
}

// The same from the float32 pieces that a product leaves where it shares K over blocks (`pieces` partial sums,
// `piece_stride` elements apart, each with q, k and v side by side in rows of ld elements): a thread adds the
// pieces of its 8 values up in ascending order, rounds the sums to bfloat16 as the whole product would have,
// and goes on as above; the rotated q goes to a buffer of its own.
__device__ inline u32x4_t sum_pieces8(const float* p, int pieces, long long piece_stride) {
  typedef float f32x4_t __attribute__((ext_vector_type(4)));
  f32x4_t lo = *(const f32x4_t*)p, hi = *(const f32x4_t*)(p + 4);
  // four pieces are asked for together (one round trip to memory, not four) and added in their order
  for (int s0 = 1; s0 < pieces; s0 += 4) {
    f32x4_t tl[4], th[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const long long at = (long long)min(s0 + j, pieces - 1) * piece_stride;
      tl[j] = *(const f32x4_t*)(p + at);
      th[j] = *(const f32x4_t*)(p + at + 4);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (s0 + j < pieces) {
        lo += tl[j];
        hi += th[j];
      }
    }
  }
  u32x4_t r;
  r[0] = (unsigned)f32_to_bf16(lo[0]).bits | ((unsigned)f32_to_bf16(lo[1]).bits << 16);
  r[1] = (unsigned)f32_to_bf16(lo[2]).bits | ((unsigned)f32_to_bf16(lo[3]).bits << 16);
  r[2] = (unsigned)f32_to_bf16(hi[0]).bits | ((unsigned)f32_to_bf16(hi[1]).bits << 16);
  r[3] = (unsigned)f32_to_bf16(hi[2]).bits | ((unsigned)f32_to_bf16(hi[3]).bits << 16);
  return r;
}

__global__ __launch_bounds__(256) void rope_store_pieces_kernel(
    const float* __restrict__ qkv, int ld, int pieces, long long piece_stride, bf16_t* __restrict__ q_out, int ldq,
    int nh, int nkv, int hd, const double* __restrict__ freqs, const int* __restrict__ row_pos,
    const int* __restrict__ row_seq, const int* __restrict__ seq_slot, const int* __restrict__ block_table,
    int bt_stride, bf16_t* __restrict__ kcache, bf16_t* __restrict__ vcache, int BS) {
  extern __shared__ float cs[];  // cos[hd/2], sin[hd/2]
  const int r = blockIdx.x;
  const int half = hd / 2, hv = half / 8;
  const int p = row_pos[r];
  const long long blk = block_table[(long long)seq_slot[row_seq[r]] * bt_stride + p / BS];
  for (int i = threadIdx.x; i < half; i += blockDim.x) {
    const double a = (double)p * freqs[i];
    const double n = rint(a * 0.15915494309189533577);
    double rem = fma(-n, 6.283185307179586232, a);
    rem = fma(-n, 2.4492935982947064e-16, rem);
    float sn, c;
    sincosf((float)rem, &sn, &c);
    cs[i] = c;
    cs[half + i] = sn;
  }
  __syncthreads();
  const float* qr = qkv + (long long)r * ld;
  const float* kr = qr + nh * hd;
  const float* vr = kr + nkv * hd;
  bf16_t* qo = q_out + (long long)r * ldq;
  for (int idx = threadIdx.x; idx < nh * hv; idx += blockDim.x) {
    const int h = idx / hv, i = (idx - h * hv) * 8;
    u32x4_t a = sum_pieces8(qr + h * hd + i, pieces, piece_stride);
    u32x4_t b = sum_pieces8(qr + h * hd + half + i, pieces, piece_stride);
    rotate8(a, b, cs + i, cs + half + i);
    *(u32x4_t*)(qo + h * hd + i) = a;
    *(u32x4_t*)(qo + h * hd + half + i) = b;
  }
  const int off = p % BS;
  for (int idx = threadIdx.x; idx < nkv * hv; idx += blockDim.x) {
    const int h = idx / hv, i = (idx - h * hv) * 8;
    u32x4_t a = sum_pieces8(kr + h * hd + i, pieces, piece_stride);
    u32x4_t b = sum_pieces8(kr + h * hd + half + i, pieces, piece_stride);
    rotate8(a, b, cs + i, cs + half + i);
    bf16_t* dst = kcache + ((blk * nkv + h) * BS + off) * (long long)hd;
    *(u32x4_t*)(dst + i) = a;
    *(u32x4_t*)(dst + half + i) = b;
  }
  for (int idx = threadIdx.x; idx < nkv * 2 * hv; idx += blockDim.x) {
    const int h = idx / (2 * hv), d = (idx - h * 2 * hv) * 8;
    const u32x4_t x = sum_pieces8(vr + h * hd + d, pieces, piece_stride);
    bf16_t* dst = vcache + ((blk * nkv + h) * hd + d) * (long long)BS + off;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      bf16_t lo, hi;
      lo.bits = (uint16_t)(x[j] & 0xffffu);
      hi.bits = (uint16_t)(x[j] >> 16);
      dst[(long long)(2 * j) * BS] = lo;
      dst[(long long)(2 * j + 1) * BS] = hi;
    }
  }
}

extern "C" int lq_rope_store_pieces(const float* qkv, int ld, int pieces, long long piece_stride, void* q_out, int ldq,
                                    int rows, int nh, int nkv, int hd, const double* freqs, const int* row_pos,
                                    const int* row_seq, const int* seq_slot, const int* block_table, int bt_stride,
                                    void* kcache, void* vcache, int block_size, hipStream_t stream) {
  LQ_REQUIRE(rows > 0 && pieces >= 1, "rope_store (pieces): rows %d, pieces %d", rows, pieces);
  LQ_REQUIRE(hd > 0 && hd % 16 == 0 && nh > 0 && nkv > 0, "rope_store (pieces): head size %d, heads %d / %d", hd, nh, nkv);
  LQ_REQUIRE(ld >= (nh + 2 * nkv) * hd && ldq >= nh * hd && ld % 4 == 0 && ldq % 8 == 0 && piece_stride % 4 == 0 &&
                 (pieces == 1 || piece_stride >= (long long)rows * ld),
             "rope_store (pieces): row strides %d / %d, piece stride %lld", ld, ldq, piece_stride);
  LQ_REQUIRE(((uintptr_t)qkv % 16) == 0 && ((uintptr_t)q_out % 16) == 0 && ((uintptr_t)kcache % 16) == 0,
             "rope_store (pieces): rows and caches must be 16-byte aligned");
  LQ_REQUIRE(block_size > 0 && bt_stride > 0, "rope_store: block size %d, table stride %d", block_size, bt_stride);
  LQ_REQUIRE(qkv && q_out && freqs && row_pos && row_seq && seq_slot && block_table && kcache && vcache,
             "rope_store (pieces): null argument");
  rope_store_pieces_kernel<<<rows, 256, (size_t)hd * sizeof(float), stream>>>(
      qkv, ld, pieces, piece_stride, (bf16_t*)q_out, ldq, nh, nkv, hd, freqs, row_pos, row_seq, seq_slot, block_table,
      bt_stride, (bf16_t*)kcache, (bf16_t*)vcache, block_size);
  LQ_CHECK_LAUNCH("rope_store (pieces)");
  return 0;
}

// The same for the rows of prompts, eight positions at a time: a block takes the rows of one sequence whose
// positions lie in one group [8 g, 8 g + 8), so that the values of a whole group go into the transposed V
// cache as runs of eight positions (16 bytes) instead of two bytes at a time, and takes cos and sin from
// the step's table (cs[row][pair][2], the same numbers that the kernels above work out for themselves).
// Blocks are counted sequence by sequence; a sequence's first and last group may be partial.
__global__ __launch_bounds__(256) void rope_store_groups_kernel(
    bf16_t* __restrict__ q, const bf16_t* __restrict__ k, const bf16_t* __restrict__ v, int ldq, int ldk, int ldv,
    int nh, int nkv, int hd, const float* __restrict__ cs, const int* __restrict__ row_pos,
    const int* __restrict__ cu_rows, int batch, const int* __restrict__ seq_slot,
    const int* __restrict__ block_table, int bt_stride, bf16_t* __restrict__ kcache, bf16_t* __restrict__ vcache,
    int BS) {
  int t = blockIdx.x, b = 0, r_begin = 0, n = 0, start = 0;
  for (; b < batch; ++b) {
    r_begin = cu_rows[b];
    n = cu_rows[b + 1] - r_begin;
    if (n <= 0) continue;
    start = row_pos[r_begin];
    const int groups = (start % 8 + n + 7) / 8;
    if (t < groups) break;
    t -= groups;
  }
  if (b >= batch) return;  // the whole block: the grid is an upper bound
  const int g8 = (start / 8 + t) * 8;
  const int p_lo = max(g8, start), p_hi = min(g8 + 8, start + n);
  const int r_lo = r_begin + (p_lo - start), cnt = p_hi - p_lo;  // rows r_lo .. r_lo + cnt - 1, positions p_lo ..
  const long long blk = block_table[(long long)seq_slot[b] * bt_stride + p_lo / BS];
  const int off0 = p_lo % BS;
  const int half = hd / 2, hv = half / 8;

  // A rotation item: 8 pairs (i .. i + 7, partners half further) of one head of one row.  Four items' loads
  // are asked for before the first is rotated: the items of a thread are independent, and their round trips
  // to memory would otherwise follow one another.
  struct Item {
    u32x4_t a, b;
    float4 t[4];
  };
  auto load_item = [&](const bf16_t* src, int row, int h, int i, Item& x) {
    x.a = *(const u32x4_t*)(src + h * hd + i);
    x.b = *(const u32x4_t*)(src + h * hd + half + i);
    const float4* t4 = (const float4*)(cs + ((long long)row * half + i) * 2);
#pragma unroll
    for (int j = 0; j < 4; ++j) x.t[j] = t4[j];
  };
  auto finish_item = [&](Item& x, bf16_t* dst, int i) {
    float c[8], sn[8];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      c[2 * j] = x.t[j].x;
      sn[2 * j] = x.t[j].y;
      c[2 * j + 1] = x.t[j].z;
      sn[2 * j + 1] = x.t[j].w;
    }
    rotate8(x.a, x.b, c, sn);
    *(u32x4_t*)(dst + i) = x.a;
    *(u32x4_t*)(dst + half + i) = x.b;
  };
  // the query heads are shared out over gridDim.y blocks; the last of them also takes the keys and the values
  const int parts = gridDim.y, part = blockIdx.y;
  const int h_lo = nh * part / parts, h_n = nh * (part + 1) / parts - h_lo;
  const int q_items = cnt * h_n * hv;
  for (int it0 = threadIdx.x; it0 < q_items; it0 += 4 * blockDim.x) {
    Item x[4];
    bf16_t* dst[4];
    int ii[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int it = min(it0 + u * (int)blockDim.x, q_items - 1);  // (a repeated last item is written twice alike)
      const int j = it / (h_n * hv), rem = it - j * (h_n * hv), h = h_lo + rem / hv;
      ii[u] = (rem % hv) * 8;
      bf16_t* qr = q + (long long)(r_lo + j) * ldq;
      dst[u] = qr + h * hd;
      load_item(qr, r_lo + j, h, ii[u], x[u]);
    }
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (it0 + u * (int)blockDim.x < q_items) finish_item(x[u], dst[u], ii[u]);
  }
  if (part != parts - 1) return;
  const int k_items = cnt * nkv * hv;
  for (int it0 = threadIdx.x; it0 < k_items; it0 += 2 * blockDim.x) {
    Item x[2];
    bf16_t* dst[2];
    int ii[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int it = min(it0 + u * (int)blockDim.x, k_items - 1);
      const int j = it / (nkv * hv), rem = it - j * (nkv * hv), h = rem / hv;
      ii[u] = (rem % hv) * 8;
      dst[u] = kcache + ((blk * nkv + h) * BS + off0 + j) * (long long)hd;
      load_item(k + (long long)(r_lo + j) * ldk, r_lo + j, h, ii[u], x[u]);
    }
#pragma unroll
    for (int u = 0; u < 2; ++u)
      if (it0 + u * (int)blockDim.x < k_items) finish_item(x[u], dst[u], ii[u]);
  }
  const bf16_t* vr = v + (long long)r_lo * ldv;
  if (cnt == 8) {  // a whole group: position off0 is a multiple of 8, the run is 16 bytes and aligned
    for (int c = threadIdx.x; c < nkv * hd; c += blockDim.x) {
      u32x4_t run;
#pragma unroll
      for (int j = 0; j < 4; ++j)
        run[j] = (unsigned)vr[(long long)(2 * j) * ldv + c].bits | ((unsigned)vr[(long long)(2 * j + 1) * ldv + c].bits << 16);
      *(u32x4_t*)(vcache + (blk * nkv * hd + c) * (long long)BS + off0) = run;
    }
  } else {
    for (int it = threadIdx.x; it < cnt * nkv * hd; it += blockDim.x) {
      const int j = it / (nkv * hd), c = it - j * (nkv * hd);
      vcache[(blk * nkv * hd + c) * (long long)BS + off0 + j] = vr[(long long)j * ldv + c];
    }
  }
}

// q rotated in place, rotated k and v into the cache, for the rows of a step that are laid out sequence by
// sequence (cu_rows) with consecutive positions: bfloat16, head sizes in steps of 16, aligned rows.
extern "C" int lq_rope_store_groups(void* q, const void* k, const void* v, int rows, int ldq, int ldk, int ldv,
                                    int nh, int nkv, int hd, const float* cos_sin, const int* row_pos,
                                    const int* cu_rows, int batch, const int* seq_slot, const int* block_table,
                                    int bt_stride, void* kcache, void* vcache, int block_size, hipStream_t stream) {
  LQ_REQUIRE(rows > 0 && batch > 0, "rope_store: rows %d and sequences %d must be positive", rows, batch);
  LQ_REQUIRE(hd > 0 && hd % 16 == 0 && nh > 0 && nkv > 0, "rope_store (groups): head size %d, heads %d / %d", hd, nh, nkv);
  LQ_REQUIRE(ldq >= nh * hd && ldk >= nkv * hd && ldv >= nkv * hd, "rope_store: a row stride is smaller than its row");
  LQ_REQUIRE(ldq % 8 == 0 && ldk % 8 == 0 && ((uintptr_t)q % 16) == 0 && ((uintptr_t)k % 16) == 0 &&
                 ((uintptr_t)kcache % 16) == 0 && ((uintptr_t)vcache % 16) == 0 && ((uintptr_t)cos_sin % 16) == 0,
             "rope_store (groups): rows and caches must be 16-byte aligned");
  LQ_REQUIRE(block_size > 0 && block_size % 8 == 0 && bt_stride > 0, "rope_store: block size %d, table stride %d",
             block_size, bt_stride);
  LQ_REQUIRE(q && k && v && cos_sin && row_pos && cu_rows && seq_slot && block_table && kcache && vcache,
             "rope_store (groups): null argument");
  const int blocks = rows / 8 + 2 * batch;  // every sequence has at most two partial groups
  // few groups (a short step): the query heads of a group are shared out over up to four blocks
  const int parts = std::max(1, std::min(std::min(4, nh), 2 * lq_compute_units() / blocks));
  rope_store_groups_kernel<<<dim3(blocks, parts), 256, 0, stream>>>(
      (bf16_t*)q, (const bf16_t*)k, (const bf16_t*)v, ldq, ldk, ldv, nh, nkv, hd, cos_sin, row_pos, cu_rows, batch,
      seq_slot, block_table, bt_stride, (bf16_t*)kcache, (bf16_t*)vcache, block_size);
  LQ_CHECK_LAUNCH("rope_store (groups)");
  return 0;
}

extern "C" int lq_rope_store(void* q, const void* k, const void* v, int dtype, int rows, int ldq,
                             int ldk, int ldv, int nh, int nkv, int hd, const double* freqs,
                             const int* row_pos, const int* row_seq, const int* seq_slot,
                             const int* block_table, int bt_stride, void* kcache, void* vcache,
                             int block_size, int store, hipStream_t stream) {
  LQ_REQUIRE(rows > 0, "rope_store: rows %d must be positive", rows);
  LQ_REQUIRE(hd > 0 && hd % 2 == 0, "rope_store: head size %d must be even", hd);
  LQ_REQUIRE(nh > 0 && nkv >= 0, "rope_store: head counts %d / %d", nh, nkv);
  LQ_REQUIRE(ldq >= nh * hd, "rope_store: q row stride %d is less than %d", ldq, nh * hd);
  if (store) {
    LQ_REQUIRE(ldk >= nkv * hd && ldv >= nkv * hd, "rope_store: k/v row stride too small");
    LQ_REQUIRE(block_size > 0 && bt_stride > 0, "rope_store: block size %d, table stride %d",
               block_size, bt_stride);
    LQ_REQUIRE(kcache && vcache && block_table && seq_slot && row_seq, "rope_store: null cache argument");
  }
  const int threads = 256;
  const size_t smem = (size_t)hd * sizeof(float);
  const int has_rope = freqs != nullptr;
  if (dtype == LQ_F32)
    rope_store_kernel<float><<<rows, threads, smem, stream>>>(
        (float*)q, (const float*)k, (const float*)v, ldq, ldk, ldv, nh, nkv, hd, freqs, has_rope,
        row_pos, row_seq, seq_slot, block_table, bt_stride, (float*)kcache, (float*)vcache,
        block_size, store);
  else if (dtype == LQ_BF16) {
    const bool vec = hd % 16 == 0 && ldq % 8 == 0 && ((uintptr_t)q % 16) == 0 &&
                     (!store || (ldk % 8 == 0 && ldv % 8 == 0 && ((uintptr_t)k % 16) == 0 && ((uintptr_t)v % 16) == 0 &&
                                 ((uintptr_t)kcache % 16) == 0));
    if (vec)
      rope_store_vec_kernel<<<rows, threads, smem, stream>>>(
          (bf16_t*)q, (const bf16_t*)k, (const bf16_t*)v, ldq, ldk, ldv, nh, nkv, hd, freqs, has_rope, row_pos,
          row_seq, seq_slot, block_table, bt_stride, (bf16_t*)kcache, (bf16_t*)vcache, block_size, store);
    else
      rope_store_kernel<bf16_t><<<rows, threads, smem, stream>>>(
          (bf16_t*)q, (const bf16_t*)k, (const bf16_t*)v, ldq, ldk, ldv, nh, nkv, hd, freqs, has_rope,
          row_pos, row_seq, seq_slot, block_table, bt_stride, (bf16_t*)kcache, (bf16_t*)vcache,
          block_size, store);
  }
  else
    LQ_REQUIRE(false, "rope_store: unknown dtype %d", dtype);
  LQ_CHECK_LAUNCH("rope_store");
  return 0;
}

// ---------------------------------------------------------------- cos/sin table of a step
// cs[r][i] = (cos, sin) of row_pos[r] * f_i, angles formed and reduced in double as in rope_store.
// Positions are the same for every layer of a step, so one launch serves them all.
__global__ void rope_table_kernel(const double* __restrict__ freqs, const int* __restrict__ row_pos,
                                  float* __restrict__ cs, int half) {
  const int r = blockIdx.x;
  const int p = row_pos[r];
  for (int i = threadIdx.x; i < half; i += blockDim.x) {
    const double a = (double)p * freqs[i];
    const double n = rint(a * 0.15915494309189533577);
    double rem = fma(-n, 6.283185307179586232, a);
    rem = fma(-n, 2.4492935982947064e-16, rem);
    float sn, c;
    sincosf((float)rem, &sn, &c);
    cs[((long long)r * half + i) * 2] = c;
    cs[((long long)r * half + i) * 2 + 1] = sn;
  }
}

extern "C" int lq_rope_table(const double* freqs, const int* row_pos, float* cs, int rows, int half,
                             hipStream_t stream) {
  LQ_REQUIRE(rows > 0 && half > 0, "rope_table: rows %d and pairs %d must be positive", rows, half);
  rope_table_kernel<<<rows, 64, 0, stream>>>(freqs, row_pos, cs, half);
  LQ_CHECK_LAUNCH("rope_table");
  return 0;
}
