// Causal grouped-query attention over the paged cache, size-agnostic version.
//
// Two kernels.  Head sizes that are multiples of 16 (up to 256) with blocks of a multiple of 16 positions
// run on the matrix cores in their true 32-bit mode (attention_tiles_kernel, below the first); everything
// else takes the first kernel: one wavefront per (query row, query head).  Row r of the step has absolute
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

// ---- on the matrix cores, float32 in and float32 accumulate (v_mfma_f32_16x16x4_f32) -------------------------
// A wavefront takes a tile of up to 16 consecutive rows of the step and one query head.  For every sequence
// that has rows in the tile it walks that sequence's keys in chunks of 64 aligned to absolute positions, from
// the first chunk that any of these rows sees to the last; rows of other sequences, and keys that a row does
// not see, take part with weight zero, which changes nothing.  Per chunk: S^T = K . Q^T (16 keys by 16 rows a
// product, summed over the head's dimensions in slabs of 16, a slab four instructions: instruction j takes
// dimensions d0 + 4 g + j, g = 0..3), then the online softmax of every row over its own 64 scores, then
// O += P . V with the probabilities straight from the registers that the scores came in (a lane holds keys
// 4 g .. 4 g + 3 of its row, which is what the second product wants of it).  Every sum of a row is made of
// its own numbers in an order that depends on its position only: the same bits whatever else is in the tile,
// the step or the batch (`rows_per_tile` 1, for steps of single tokens, gives every row a tile of its own).
typedef float f32x4 __attribute__((ext_vector_type(4)));

__device__ inline f32x4 load4f(const float* p) { return *(const f32x4*)p; }
__device__ inline f32x4 load4f(const bf16_t* p) {
  const uint2 v = *(const uint2*)p;
  f32x4 r;
  r.x = __uint_as_float(v.x << 16);
  r.y = __uint_as_float(v.x & 0xffff0000u);
  r.z = __uint_as_float(v.y << 16);
  r.w = __uint_as_float(v.y & 0xffff0000u);
  return r;
}

template <typename T, int HS>  // HS: head size / 16
__global__ __launch_bounds__(64) void attention_tiles_kernel(
    const T* __restrict__ q, int ldq, T* __restrict__ out, int ldo, int rows, int rows_per_tile, int nh, int nkv,
    const int* __restrict__ row_pos, const int* __restrict__ row_seq, const int* __restrict__ seq_slot,
    const int* __restrict__ block_table, int bt_stride, const T* __restrict__ kcache, const T* __restrict__ vcache,
    int BS, float scale, int window) {
  constexpr int HD = HS * 16;
  const int lane = threadIdx.x, c = lane & 15, g = lane >> 4;
  const int h = blockIdx.y, kvh = h / (nh / nkv);
  const int r0 = blockIdx.x * rows_per_tile;
  const int n_rows = min(rows_per_tile, rows - r0);
  // lane (c, g) looks after row r0 + c (every g alike); rows past the tile repeat its last row and are not stored
  const int my_row = r0 + min(c, n_rows - 1);
  const int my_pos = row_pos[my_row], my_seq = row_seq[my_row];
  const int my_lo = (window > 0 && my_pos >= window) ? my_pos - window + 1 : 0;
  f32x4 qv[HS];
#pragma unroll
  for (int sl = 0; sl < HS; ++sl) qv[sl] = load4f(q + (long long)my_row * ldq + h * HD + sl * 16 + 4 * g);

  float m = -INFINITY, l = 0.f;
  f32x4 o[HS];  // o[dt][e]: row 4 g + e of the tile, dimension 16 dt + c
#pragma unroll
  for (int dt = 0; dt < HS; ++dt) o[dt] = (f32x4){0.f, 0.f, 0.f, 0.f};

  // one pass for every sequence with rows in the tile (a step's rows lie sequence by sequence, so these are
  // the sequences of its first to its last row)
  const int seq_first = __builtin_amdgcn_readfirstlane(row_seq[r0]);
  const int seq_last = __builtin_amdgcn_readfirstlane(row_seq[r0 + n_rows - 1]);
  for (int seq = seq_first; seq <= seq_last; ++seq) {
    const bool mine = my_seq == seq && c < n_rows;
    // the chunks that any row of this pass sees
    int lo_min = mine ? my_lo : 0x7fffffff, pos_max = mine ? my_pos : -1;
#pragma unroll
    for (int off = 1; off < 16; off <<= 1) {
      lo_min = min(lo_min, __shfl_xor(lo_min, off, 64));
      pos_max = max(pos_max, __shfl_xor(pos_max, off, 64));
    }
    lo_min = __builtin_amdgcn_readfirstlane(lo_min);
    pos_max = __builtin_amdgcn_readfirstlane(pos_max);
    if (pos_max < 0) continue;  // (a sequence number without rows here)
    const int* table = block_table + (long long)seq_slot[seq] * bt_stride;
    for (int t0 = (lo_min / 64) * 64; t0 <= pos_max; t0 += 64) {
      // S^T: st[kt][e] = score of key t0 + 16 kt + 4 g + e for row c
      f32x4 st[4];
#pragma unroll
      for (int kt = 0; kt < 4; ++kt) {
        st[kt] = (f32x4){0.f, 0.f, 0.f, 0.f};
        const int t = min(t0 + 16 * kt + c, pos_max);  // this lane's key as an operand row (clamped: finite, masked below)
        const long long blk = table[t / BS];
        const T* kr = kcache + ((blk * nkv + kvh) * BS + t % BS) * (long long)HD + 4 * g;
        f32x4 kv[HS];
#pragma unroll
        for (int sl = 0; sl < HS; ++sl) kv[sl] = load4f(kr + sl * 16);
#pragma unroll
        for (int sl = 0; sl < HS; ++sl)
#pragma unroll
          for (int j = 0; j < 4; ++j)
            st[kt] = __builtin_amdgcn_mfma_f32_16x16x4f32(kv[sl][j], qv[sl][j], st[kt], 0, 0, 0);
      }
      // the row's own 64 scores: 16 in this lane, the rest in the lanes 16, 32 and 48 further
      float cmax = -INFINITY;
#pragma unroll
      for (int kt = 0; kt < 4; ++kt)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int t = t0 + 16 * kt + 4 * g + e;
          const bool valid = mine && t >= my_lo && t <= my_pos;
          st[kt][e] = valid ? st[kt][e] * scale : -INFINITY;
          cmax = fmaxf(cmax, st[kt][e]);
        }
      cmax = fmaxf(cmax, __shfl_xor(cmax, 16, 64));
      cmax = fmaxf(cmax, __shfl_xor(cmax, 32, 64));
      const float m_new = fmaxf(m, cmax);
      const bool none = m_new == -INFINITY;  // no key of this row so far: nothing changes
      const float alpha = none ? 1.f : expf(m - m_new);
      float psum = 0.f;
#pragma unroll
      for (int kt = 0; kt < 4; ++kt)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          st[kt][e] = none ? 0.f : expf(st[kt][e] - m_new);
          psum += st[kt][e];
        }
      psum += __shfl_xor(psum, 16, 64);
      psum += __shfl_xor(psum, 32, 64);
      l = l * alpha + psum;
      m = m_new;
      // O = O * alpha + P . V: the accumulators hold rows 4 g + e, whose alpha lanes 4 g + e know
      float a4[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) a4[e] = __shfl(alpha, 4 * g + e, 64);
#pragma unroll
      for (int dt = 0; dt < HS; ++dt)
#pragma unroll
        for (int e = 0; e < 4; ++e) o[dt][e] *= a4[e];
#pragma unroll
      for (int kt = 0; kt < 4; ++kt) {
        // V^T of this lane's dimension 16 dt + c at keys t0 + 16 kt + 4 g .. + 3 (within one block)
        const int t = min(t0 + 16 * kt + 4 * g, pos_max) & ~3;
        const long long blk = table[t / BS];
        const T* vr = vcache + ((blk * nkv + kvh) * (long long)HD + c) * BS + t % BS;
        f32x4 vv[HS];
#pragma unroll
        for (int dt = 0; dt < HS; ++dt) vv[dt] = load4f(vr + (long long)dt * 16 * BS);
#pragma unroll
        for (int dt = 0; dt < HS; ++dt)
#pragma unroll
          for (int j = 0; j < 4; ++j)
            o[dt] = __builtin_amdgcn_mfma_f32_16x16x4f32(st[kt][j], vv[dt][j], o[dt], 0, 0, 0);
      }
    }
  }
  float inv4[4];
  const float inv = 1.0f / l;
#pragma unroll
  for (int e = 0; e < 4; ++e) inv4[e] = __shfl(inv, 4 * g + e, 64);
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const int row = 4 * g + e;
    if (row < n_rows) {
      T* orow = out + (long long)(r0 + row) * ldo + h * HD + c;
#pragma unroll
      for (int dt = 0; dt < HS; ++dt) orow[dt * 16] = from_f32<T>(o[dt][e] * inv4[e]);
    }
  }
}

template <typename T, int HS>
void launch_tiles(const void* q, int ldq, void* out, int ldo, int rows, int rows_per_tile, int nh, int nkv,
                  const int* row_pos, const int* row_seq, const int* seq_slot, const int* block_table, int bt_stride,
                  const void* kcache, const void* vcache, int BS, float scale, int window, hipStream_t stream) {
  dim3 grid(lq_ceil_div(rows, rows_per_tile), nh);
  attention_tiles_kernel<T, HS><<<grid, 64, 0, stream>>>((const T*)q, ldq, (T*)out, ldo, rows, rows_per_tile, nh, nkv,
                                                         row_pos, row_seq, seq_slot, block_table, bt_stride,
                                                         (const T*)kcache, (const T*)vcache, BS, scale, window);
}

template <typename T>
bool try_tiles(const void* q, int ldq, void* out, int ldo, int rows, int batch, int nh, int nkv, int hd,
               const int* row_pos, const int* row_seq, const int* seq_slot, const int* block_table, int bt_stride,
               const void* kcache, const void* vcache, int BS, float scale, int window, hipStream_t stream) {
  const int el = (int)sizeof(T);
  if (hd % 16 != 0 || hd > 256 || BS % 16 != 0 || ldq % 4 != 0 || ((uintptr_t)q % (4 * el)) != 0 ||
      ((uintptr_t)kcache % (4 * el)) != 0 || ((uintptr_t)vcache % (4 * el)) != 0)
    return false;
  // a step of single tokens (as many sequences as rows): a tile a row; else 16 rows a tile
  const int rpt = rows == batch ? 1 : 16;
#define LQ_TILES(HS)                                                                                                  \
  case HS:                                                                                                            \
    launch_tiles<T, HS>(q, ldq, out, ldo, rows, rpt, nh, nkv, row_pos, row_seq, seq_slot, block_table, bt_stride,     \
                        kcache, vcache, BS, scale, window, stream);                                                   \
    return true;
  switch (hd / 16) {
    LQ_TILES(1) LQ_TILES(2) LQ_TILES(3) LQ_TILES(4) LQ_TILES(5) LQ_TILES(6) LQ_TILES(7) LQ_TILES(8) LQ_TILES(9)
    LQ_TILES(10) LQ_TILES(12) LQ_TILES(16)
  }
#undef LQ_TILES
  return false;
}

}  // namespace

int lq_attention_generic(const void* q, int ldq, void* out, int ldo, int dtype, int rows, int batch, int nh,
                         int nkv, int hd, const int* row_pos, const int* row_seq,
                         const int* seq_slot, const int* block_table, int bt_stride,
                         const void* kcache, const void* vcache, int block_size, float scale,
                         int window, hipStream_t stream) {
  LQ_REQUIRE(hd <= MAX_HD, "attention: head size %d exceeds %d", hd, MAX_HD);
  LQ_REQUIRE(nh <= 65535, "attention: %d heads are too many for one launch", nh);
  LQ_REQUIRE(dtype == LQ_F32 || dtype == LQ_BF16, "attention: unknown dtype %d", dtype);
  const bool on_tiles =
      dtype == LQ_F32 ? try_tiles<float>(q, ldq, out, ldo, rows, batch, nh, nkv, hd, row_pos, row_seq, seq_slot, block_table,
                                         bt_stride, kcache, vcache, block_size, scale, window, stream)
                      : try_tiles<bf16_t>(q, ldq, out, ldo, rows, batch, nh, nkv, hd, row_pos, row_seq, seq_slot,
                                          block_table, bt_stride, kcache, vcache, block_size, scale, window, stream);
  if (on_tiles) {
    LQ_CHECK_LAUNCH("attention(generic, tiles)");
    return 0;
  }
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
