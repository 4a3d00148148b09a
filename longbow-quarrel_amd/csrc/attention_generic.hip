// Causal grouped-query attention over the paged cache, size-agnostic version.
//
// One wavefront per (query row, query head).  Row r of the step has absolute
// position p = row_pos[r] and belongs to batch entry row_seq[r]; its keys are
// positions lo..p of that entry's slot, lo = 0 or p - window + 1 when a window
// is set (internal/device/kernels.metal:676).  Query head h reads kv head
// h / (nh / nkv) (:671).  score = q.k * scale, softmax with a running maximum
// that starts at -inf, out = sum softmax * v (:696-765), all in 32-bit.
//
// Keys are walked in chunks of 64 aligned to absolute positions, so the order
// of every sum depends on the row's position only: not on how the tokens were
// cut into steps nor on what else is in the batch.
//
// Cache layout: K[block][kv head][offset][hd], V[block][kv head][hd][offset],
// block = table[slot][t / BS], offset = t % BS.
#include "common.h"

namespace {

constexpr int MAX_HD = 512;  // 8 accumulators a lane

template <typename T>
__global__ __launch_bounds__(64) void attention_rows_kernel(
    const T* __restrict__ q, int ldq, T* __restrict__ out, int ldo, int nh, int nkv, int hd,
    const int* __restrict__ row_pos, const int* __restrict__ row_seq,
    const int* __restrict__ seq_slot, const int* __restrict__ block_table, int bt_stride,
    const T* __restrict__ kcache, const T* __restrict__ vcache, int BS, float scale, int window) {
  __shared__ float qs[MAX_HD];
  __shared__ float ps[64];
  __shared__ long long kbase[64];
  __shared__ long long vbase[64];

  const int r = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int g = h / (nh / nkv);
  const int p = row_pos[r];
  const int slot = seq_slot[row_seq[r]];
  const int lo = (window > 0 && p >= window) ? p - window + 1 : 0;
  const int* table = block_table + (long long)slot * bt_stride;

  for (int d = lane; d < hd; d += 64) qs[d] = to_f32(q[(long long)r * ldq + h * hd + d]);

  float m = -INFINITY, l = 0.f;
  float acc[MAX_HD / 64];
#pragma unroll
  for (int j = 0; j < MAX_HD / 64; ++j) acc[j] = 0.f;

  for (int t0 = (lo / 64) * 64; t0 <= p; t0 += 64) {
    const int t = t0 + lane;
    const bool valid = t >= lo && t <= p;
    __syncthreads();  // the previous chunk's readers of ps / kbase / vbase are done (and qs is written)
    float s = -INFINITY;
    if (valid) {
      const long long blk = table[t / BS];
      const int off = t % BS;
      const long long kb = ((blk * nkv + g) * BS + off) * (long long)hd;
      kbase[lane] = kb;
      vbase[lane] = (blk * nkv + g) * (long long)hd * BS + off;
      float dot = 0.f;
      const T* kr = kcache + kb;
      for (int d = 0; d < hd; ++d) dot = fmaf(qs[d], to_f32(kr[d]), dot);
      s = dot * scale;
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float alpha = expf(m - m_new);  // m = -inf on the first chunk gives 0
    const float pj = valid ? expf(s - m_new) : 0.f;
    ps[lane] = pj;
    // fixed-order sum of the chunk's weights: lane 0..63 ascending through LDS
    __syncthreads();
    const int nvalid = min(64, p - t0 + 1);
    float psum = 0.f;
    for (int i = 0; i < nvalid; ++i) psum += ps[i];
    l = l * alpha + psum;
#pragma unroll
    for (int j = 0; j < MAX_HD / 64; ++j) {
      const int d = lane + 64 * j;
      if (d < hd) {
        float a = acc[j] * alpha;
        for (int i = 0; i < nvalid; ++i) {
          const float w = ps[i];
          if (w != 0.f) a = fmaf(w, to_f32(vcache[vbase[i] + (long long)d * BS]), a);
        }
        acc[j] = a;
      }
    }
    m = m_new;
  }
  const float inv = 1.0f / l;
#pragma unroll
  for (int j = 0; j < MAX_HD / 64; ++j) {
    const int d = lane + 64 * j;
    if (d < hd) out[(long long)r * ldo + h * hd + d] = from_f32<T>(acc[j] * inv);
  }
}

}  // namespace

int lq_attention_generic(const void* q, int ldq, void* out, int ldo, int dtype, int rows, int nh,
                         int nkv, int hd, const int* row_pos, const int* row_seq,
                         const int* seq_slot, const int* block_table, int bt_stride,
                         const void* kcache, const void* vcache, int block_size, float scale,
                         int window, hipStream_t stream) {
  LQ_REQUIRE(hd <= MAX_HD, "attention: head size %d exceeds %d", hd, MAX_HD);
  LQ_REQUIRE(nh <= 65535, "attention: %d heads are too many for one launch", nh);
  dim3 grid(rows, nh);
  if (dtype == LQ_F32)
    attention_rows_kernel<float><<<grid, 64, 0, stream>>>(
        (const float*)q, ldq, (float*)out, ldo, nh, nkv, hd, row_pos, row_seq, seq_slot,
        block_table, bt_stride, (const float*)kcache, (const float*)vcache, block_size, scale,
        window);
  else if (dtype == LQ_BF16)
    attention_rows_kernel<bf16_t><<<grid, 64, 0, stream>>>(
        (const bf16_t*)q, ldq, (bf16_t*)out, ldo, nh, nkv, hd, row_pos, row_seq, seq_slot,
        block_table, bt_stride, (const bf16_t*)kcache, (const bf16_t*)vcache, block_size, scale,
        window);
  else
    LQ_REQUIRE(false, "attention: unknown dtype %d", dtype);
  LQ_CHECK_LAUNCH("attention(generic)");
  return 0;
}
