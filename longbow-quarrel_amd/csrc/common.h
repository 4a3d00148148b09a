// Shared types and helpers of the gfx950 kernels.
//
// Every entry point is `extern "C"`, takes raw device pointers plus sizes and a
// hipStream_t, validates what its grid assumes, launches, and returns 0 or a
// negative code; lq_last_error() then holds the reason.  Nothing here
// allocates device memory: callers bring inputs, outputs and workspaces.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#define LQ_WAVE 64

// element types of activations / weights / cache as the Python side names them
enum LqDtype { LQ_F32 = 0, LQ_BF16 = 1 };

struct bf16_t {
  uint16_t bits;
};

__device__ __host__ inline float bf16_to_f32(bf16_t v) {
  union {
    uint32_t u;
    float f;
  } c;
  c.u = ((uint32_t)v.bits) << 16;
  return c.f;
}

// round to nearest even; NaN stays NaN
__device__ __host__ inline bf16_t f32_to_bf16(float f) {
  union {
    uint32_t u;
    float f;
  } c;
  c.f = f;
  bf16_t r;
  if ((c.u & 0x7fffffffu) > 0x7f800000u) {
    r.bits = (uint16_t)((c.u >> 16) | 0x0040u);
    return r;
  }
  uint32_t lsb = (c.u >> 16) & 1u;
  c.u += 0x7fffu + lsb;
  r.bits = (uint16_t)(c.u >> 16);
  return r;
}

__device__ inline float to_f32(float v) { return v; }
__device__ inline float to_f32(bf16_t v) { return bf16_to_f32(v); }

template <typename T>
__device__ inline T from_f32(float v);
template <>
__device__ inline float from_f32<float>(float v) {
  return v;
}
template <>
__device__ inline bf16_t from_f32<bf16_t>(float v) {
  return f32_to_bf16(v);
}

// ---- wave and block reductions (64-wide wavefronts) -------------------------

__device__ inline float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, LQ_WAVE);
  return v;
}

__device__ inline float wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, LQ_WAVE));
  return v;
}

// Sum over a block of up to 1024 threads; every thread gets the result.  The
// tree is fixed, so a row's sum does not depend on what else is in the launch.
__device__ inline float block_sum(float v, float* smem /* >= 16 floats */) {
  const int lane = threadIdx.x & (LQ_WAVE - 1);
  const int wave = threadIdx.x / LQ_WAVE;
  const int nwaves = (blockDim.x + LQ_WAVE - 1) / LQ_WAVE;
  v = wave_sum(v);
  __syncthreads();
  if (lane == 0) smem[wave] = v;
  __syncthreads();
  float total = 0.f;
  for (int w = 0; w < nwaves; ++w) total += smem[w];
  return total;
}

__device__ inline float block_max(float v, float* smem) {
  const int lane = threadIdx.x & (LQ_WAVE - 1);
  const int wave = threadIdx.x / LQ_WAVE;
  const int nwaves = (blockDim.x + LQ_WAVE - 1) / LQ_WAVE;
  v = wave_max(v);
  __syncthreads();
  if (lane == 0) smem[wave] = v;
  __syncthreads();
  float total = smem[0];
  for (int w = 1; w < nwaves; ++w) total = fmaxf(total, smem[w]);
  return total;
}

// ---- error reporting ---------------------------------------------------------

void lq_set_error(const char* fmt, ...);
int lq_compute_units();  // of the current device

#define LQ_REQUIRE(cond, ...)   \
  do {                          \
    if (!(cond)) {              \
      lq_set_error(__VA_ARGS__); \
      return -1;                \
    }                           \
  } while (0)

#define LQ_CHECK_LAUNCH(name)                                            \
  do {                                                                   \
    hipError_t e_ = hipGetLastError();                                   \
    if (e_ != hipSuccess) {                                              \
      lq_set_error("%s: launch failed: %s", name, hipGetErrorString(e_)); \
      return -2;                                                         \
    }                                                                    \
  } while (0)

// tokens by which a decoding attention launch rounds the bound of the lengths up before it shapes its grid
#define LQ_DECODE_LENGTH_BUCKET 1024

static inline int lq_ceil_div(int a, int b) { return (a + b - 1) / b; }
static inline long long lq_ceil_div64(long long a, long long b) { return (a + b - 1) / b; }
