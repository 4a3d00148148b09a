// Causal grouped-query attention over the paged bfloat16 cache on the matrix cores.
//
// One wavefront owns 16 query columns and walks its keys in chunks of 32.  The score tile is
// computed transposed, S^T[key][q] = K . Q^T, so that after the softmax each lane already holds
// the probabilities of one query column in the layout the second product wants as its B operand
// (O^T[d][q] += V^T[d][key] . P^T[key][q]); nothing goes through LDS.  The cache stores V
// transposed per block for exactly this read: V[block][kv head][d][offset].
//
//   v_mfma_f32_16x16x32_bf16: lane l gives A[row l%16][k (l/16)*8 .. +8], B[col l%16][same k],
//   receives D[(l/16)*4 + e][l%16].
//   First product: A = 16 keys x 32 of head_dim, B = 16 queries x the same 32.
//   Second product: its 32 k are keys; MFMA k index (l/16)*8 + j stands for key
//   (l/16)*4 + j of the chunk's first 16 keys when j < 4, else 16 + (l/16)*4 + (j - 4):
//   the keys whose scores lane l already holds.
//
// Softmax statistics, scores and the output accumulator are 32-bit; probabilities are rounded to
// bfloat16 only as MFMA operands (their sum is taken before rounding).
//
// Two launch shapes share the inner loop:
//  * rows:  16 consecutive rows of one sequence for one query head (prompts).
//  * heads: one row of one sequence for the query heads of one kv head (decoding); keys are
//    cut into splits of SPLIT positions, aligned to absolute positions, each split a block of its
//    own, partial results merged by a second kernel in ascending split order.
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

namespace {

constexpr int BS = 64;      // positions per cache block (the only block size this file takes)
constexpr int SPLIT = 128;  // keys per split when decoding

__device__ inline bf16x8 as_bf16x8(u32x4 v) {
  union {
    u32x4 u;
    bf16x8 b;
  } c;
  c.u = v;
  return c.b;
}

__device__ inline unsigned pack_bf16(float lo, float hi) {
  return (unsigned)f32_to_bf16(lo).bits | ((unsigned)f32_to_bf16(hi).bits << 16);
}

struct AttnArgs {
  const bf16_t* q;
  int ldq;
  bf16_t* out;
  int ldo;
  int nh, nkv;
  const int* row_pos;
  const int* seq_slot;
  const int* cu_rows;
  const int* block_table;
  int bt_stride;
  const bf16_t* kcache;
  const bf16_t* vcache;
  float scale_log2;  // scale * log2(e)
  int window;
  int batch;
  // decode only
  float* part_o;   // [rows][nh][nsplit][HD]
  float* part_ml;  // [rows][nh][nsplit][2]
  int nsplit;
};

// The shared inner loop.  Query column c = lane % 16 is valid if c < ncols; its position is
// p_c, its first key lo_c.  Keys t_begin..t_end (inclusive) are walked; t_begin is a multiple of 32.
// On return o[dt][e] holds the unnormalised O^T[dt*16 + (lane/16)*4 + e][c], m the running maximum
// (in the log2 domain) and l this lane's share of the normaliser (to be summed over lane/16).
// One chunk's operands as they come from memory: 16 bytes a lane for each K fragment, two 8-byte
// pieces a lane for each V^T fragment.
template <int HD>
struct ChunkRegs {
  u32x4 k[2][HD / 32];
  u32x2 v[HD / 16][2];
};

template <int HD>
__device__ inline void load_chunk(const AttnArgs& a, int kvh, long long blk, int koff, ChunkRegs<HD>& r) {
  const int lane = threadIdx.x & 63, c16 = lane & 15, g = lane >> 4;
  const bf16_t* kb = a.kcache + ((blk * a.nkv + kvh) * BS + koff) * (long long)HD;
#pragma unroll
  for (int j = 0; j < 2; ++j)
#pragma unroll
    for (int kk = 0; kk < HD / 32; ++kk)
      r.k[j][kk] = *(const u32x4*)(kb + (16 * j + c16) * HD + kk * 32 + g * 8);
  const bf16_t* vb = a.vcache + ((blk * a.nkv + kvh) * (long long)HD) * BS + koff;
#pragma unroll
  for (int dt = 0; dt < HD / 16; ++dt) {
    const bf16_t* vr = vb + (long long)(dt * 16 + c16) * BS;
    r.v[dt][0] = *(const u32x2*)(vr + g * 4);
    r.v[dt][1] = *(const u32x2*)(vr + 16 + g * 4);
  }
}

template <int HD>
__device__ inline void attend(const AttnArgs& a, const bf16x8 (&qf)[HD / 32], int kvh, const int* table,
                              int t_begin, int t_end, bool col_valid, int p_c, int lo_c,
                              f32x4 (&o)[HD / 16], float& m, float& l) {
  const int lane = threadIdx.x & 63, g = lane >> 4;
  // the next chunk's keys and values are already on their way while this chunk is computed, and
  // the block number of the chunk after that while those are loaded
  ChunkRegs<HD> cur, nxt;
  long long blk_next = table[t_begin / BS];
  load_chunk<HD>(a, kvh, blk_next, t_begin % BS, nxt);
  blk_next = (t_begin + 32 <= t_end) ? table[(t_begin + 32) / BS] : 0;
  for (int t0 = t_begin; t0 <= t_end; t0 += 32) {
    cur = nxt;
    if (t0 + 32 <= t_end) {
      load_chunk<HD>(a, kvh, blk_next, (t0 + 32) % BS, nxt);
      blk_next = (t0 + 64 <= t_end) ? table[(t0 + 64) / BS] : 0;
    }
    f32x4 s[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      s[j] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kk = 0; kk < HD / 32; ++kk)
        s[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(cur.k[j][kk]), qf[kk], s[j], 0, 0, 0);
    }
    float sv[8];
    float cmax = -INFINITY;
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int t = t0 + 16 * j + g * 4 + e;
        const bool ok = col_valid && t >= lo_c && t <= p_c;
        const float v = ok ? s[j][e] * a.scale_log2 : -INFINITY;
        sv[j * 4 + e] = v;
        cmax = fmaxf(cmax, v);
      }
    cmax = fmaxf(cmax, __shfl_xor(cmax, 16, 64));
    cmax = fmaxf(cmax, __shfl_xor(cmax, 32, 64));
    const float m_new = fmaxf(m, cmax);
    const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;  // a column with no key yet
    const float alpha = exp2f(m - m_safe);
    float psum = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      sv[i] = exp2f(sv[i] - m_safe);
      psum += sv[i];
    }
    l = l * alpha + psum;
    m = m_new;
    u32x4 pw;
    pw[0] = pack_bf16(sv[0], sv[1]);
    pw[1] = pack_bf16(sv[2], sv[3]);
    pw[2] = pack_bf16(sv[4], sv[5]);
    pw[3] = pack_bf16(sv[6], sv[7]);
    const bf16x8 pb = as_bf16x8(pw);

    // keys past t_end lie in the block but were never written: their values must not reach the
    // product (0 * garbage may be NaN), so they are zeroed
    const bool tail = t0 + 31 > t_end;
#pragma unroll
    for (int dt = 0; dt < HD / 16; ++dt) {
      u32x2 v0 = cur.v[dt][0];
      u32x2 v1 = cur.v[dt][1];
      if (tail) {
        const int ta = t0 + g * 4, tb = t0 + 16 + g * 4;
        if (ta + 0 > t_end) v0[0] &= 0xffff0000u;
        if (ta + 1 > t_end) v0[0] &= 0x0000ffffu;
        if (ta + 2 > t_end) v0[1] &= 0xffff0000u;
        if (ta + 3 > t_end) v0[1] &= 0x0000ffffu;
        if (tb + 0 > t_end) v1[0] &= 0xffff0000u;
        if (tb + 1 > t_end) v1[0] &= 0x0000ffffu;
        if (tb + 2 > t_end) v1[1] &= 0xffff0000u;
        if (tb + 3 > t_end) v1[1] &= 0x0000ffffu;
      }
      u32x4 vv;
      vv[0] = v0[0];
      vv[1] = v0[1];
      vv[2] = v1[0];
      vv[3] = v1[1];
#pragma unroll
      for (int e = 0; e < 4; ++e) o[dt][e] *= alpha;
      o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(vv), pb, o[dt], 0, 0, 0);
    }
  }
}

// ------------------------------------------------------------------ rows (prompts)
template <int HD>
__global__ __launch_bounds__(64) void attn_rows_kernel(AttnArgs a) {
  // find this block's tile: tiles of 16 rows, counted sequence by sequence
  int t = blockIdx.x, b = 0, r0 = -1, nrows = 0;
  for (; b < a.batch; ++b) {
    const int begin = a.cu_rows[b], n = a.cu_rows[b + 1] - begin;
    const int tiles = (n + 15) / 16;
    if (t < tiles) {
      r0 = begin + t * 16;
      nrows = min(16, n - t * 16);
      break;
    }
    t -= tiles;
  }
  if (r0 < 0) return;
  const int lane = threadIdx.x & 63, c16 = lane & 15, g = lane >> 4;
  const int h = blockIdx.y, kvh = h / (a.nh / a.nkv);
  const int* table = a.block_table + (long long)a.seq_slot[b] * a.bt_stride;
  const int p0 = a.row_pos[r0];
  const bool col_valid = c16 < nrows;
  const int p_c = p0 + min(c16, nrows - 1);
  const int lo_c = (a.window > 0 && p_c >= a.window) ? p_c - a.window + 1 : 0;
  const int lo_tile = (a.window > 0 && p0 >= a.window) ? p0 - a.window + 1 : 0;

  bf16x8 qf[HD / 32];
  {
    const bf16_t* qr = a.q + (long long)(r0 + min(c16, nrows - 1)) * a.ldq + h * HD + g * 8;
#pragma unroll
    for (int kk = 0; kk < HD / 32; ++kk) qf[kk] = as_bf16x8(*(const u32x4*)(qr + kk * 32));
  }
  f32x4 o[HD / 16];
#pragma unroll
  for (int dt = 0; dt < HD / 16; ++dt) o[dt] = (f32x4){0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;
  attend<HD>(a, qf, kvh, table, (lo_tile / 32) * 32, p0 + nrows - 1, col_valid, p_c, lo_c, o, m, l);
  l += __shfl_xor(l, 16, 64);
  l += __shfl_xor(l, 32, 64);
  if (!col_valid) return;
  const float inv = 1.0f / l;
  bf16_t* orow = a.out + (long long)(r0 + c16) * a.ldo + h * HD + g * 4;
#pragma unroll
  for (int dt = 0; dt < HD / 16; ++dt) {
    u32x2 w;
    w[0] = pack_bf16(o[dt][0] * inv, o[dt][1] * inv);
    w[1] = pack_bf16(o[dt][2] * inv, o[dt][3] * inv);
    *(u32x2*)(orow + dt * 16) = w;
  }
}

// ------------------------------------------------------------------ heads (decoding)
template <int HD>
__global__ __launch_bounds__(64) void attn_heads_kernel(AttnArgs a) {
  const int b = blockIdx.x, kvh = blockIdx.y, split = blockIdx.z;
  const int lane = threadIdx.x & 63, c16 = lane & 15, g = lane >> 4;
  const int G = a.nh / a.nkv;
  const int r = a.cu_rows[b];
  const int p = a.row_pos[r];
  const int lo = (a.window > 0 && p >= a.window) ? p - a.window + 1 : 0;
  const int t_begin = max(split * SPLIT, (lo / 32) * 32);
  const int t_end = min(split * SPLIT + SPLIT - 1, p);
  if (t_begin > t_end || split * SPLIT + SPLIT - 1 < lo) return;
  const int* table = a.block_table + (long long)a.seq_slot[b] * a.bt_stride;
  const bool col_valid = c16 < G;
  const int h = kvh * G + min(c16, G - 1);

  bf16x8 qf[HD / 32];
  {
    const bf16_t* qr = a.q + (long long)r * a.ldq + h * HD + g * 8;
#pragma unroll
    for (int kk = 0; kk < HD / 32; ++kk) qf[kk] = as_bf16x8(*(const u32x4*)(qr + kk * 32));
  }
  f32x4 o[HD / 16];
#pragma unroll
  for (int dt = 0; dt < HD / 16; ++dt) o[dt] = (f32x4){0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;
  attend<HD>(a, qf, kvh, table, t_begin, t_end, col_valid, p, lo, o, m, l);
  l += __shfl_xor(l, 16, 64);
  l += __shfl_xor(l, 32, 64);
  if (!col_valid) return;
  if (a.nsplit == 1) {
    const float inv = 1.0f / l;
    bf16_t* orow = a.out + (long long)r * a.ldo + h * HD + g * 4;
#pragma unroll
    for (int dt = 0; dt < HD / 16; ++dt) {
      u32x2 w;
      w[0] = pack_bf16(o[dt][0] * inv, o[dt][1] * inv);
      w[1] = pack_bf16(o[dt][2] * inv, o[dt][3] * inv);
      *(u32x2*)(orow + dt * 16) = w;
    }
    return;
  }
  const long long slot = ((long long)r * a.nh + h) * a.nsplit + split;
  float* po = a.part_o + slot * HD + g * 4;
#pragma unroll
  for (int dt = 0; dt < HD / 16; ++dt) *(f32x4*)(po + dt * 16) = o[dt];
  if (g == 0) {
    a.part_ml[slot * 2] = m;
    a.part_ml[slot * 2 + 1] = l;
  }
}

// Merges the splits of one (row, head): out = sum_s 2^(m_s - M) o_s / sum_s 2^(m_s - M) l_s,
// splits in ascending order.
template <int HD>
__global__ __launch_bounds__(64) void attn_merge_kernel(AttnArgs a) {
  const int b = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int r = a.cu_rows[b];
  const int p = a.row_pos[r];
  const int lo = (a.window > 0 && p >= a.window) ? p - a.window + 1 : 0;
  const int s_first = lo / SPLIT, s_last = p / SPLIT;
  const long long base = ((long long)r * a.nh + h) * a.nsplit;
  float M = -INFINITY;
  for (int s = s_first; s <= s_last; ++s) M = fmaxf(M, a.part_ml[(base + s) * 2]);
  float L = 0.f;
  float acc[HD / 64 + 1];
#pragma unroll
  for (int j = 0; j < HD / 64 + 1; ++j) acc[j] = 0.f;
  for (int s = s_first; s <= s_last; ++s) {
    const float w = exp2f(a.part_ml[(base + s) * 2] - M);
    L += w * a.part_ml[(base + s) * 2 + 1];
#pragma unroll
    for (int j = 0; j < HD / 64 + 1; ++j) {
      const int d = lane + 64 * j;
      if (d < HD) acc[j] += w * a.part_o[(base + s) * HD + d];
    }
  }
  const float inv = 1.0f / L;
#pragma unroll
  for (int j = 0; j < HD / 64 + 1; ++j) {
    const int d = lane + 64 * j;
    if (d < HD) a.out[(long long)r * a.ldo + h * HD + d] = f32_to_bf16(acc[j] * inv);
  }
}

template <int HD>
int launch(const AttnArgs& a, int rows, int decode, hipStream_t stream) {
  if (!decode) {
    dim3 grid(lq_ceil_div(rows, 16) + a.batch, a.nh);
    attn_rows_kernel<HD><<<grid, 64, 0, stream>>>(a);
    LQ_CHECK_LAUNCH("attention(mfma rows)");
    return 0;
  }
  dim3 grid(a.batch, a.nkv, a.nsplit);
  attn_heads_kernel<HD><<<grid, 64, 0, stream>>>(a);
  LQ_CHECK_LAUNCH("attention(mfma heads)");
  if (a.nsplit > 1) {
    dim3 mgrid(a.batch, a.nh);
    attn_merge_kernel<HD><<<mgrid, 64, 0, stream>>>(a);
    LQ_CHECK_LAUNCH("attention(mfma merge)");
  }
  return 0;
}

}  // namespace

bool lq_attention_mfma_accepts(int dtype, int nh, int nkv, int hd, int block_size, int ldq, int ldo,
                               const void* q, const void* out, int decode) {
  if (dtype != LQ_BF16 || block_size != BS) return false;
  if (!(hd == 32 || hd == 64 || hd == 96 || hd == 128 || hd == 192 || hd == 256)) return false;
  if (ldq % 8 != 0 || ldo % 4 != 0 || ((uintptr_t)q % 16) != 0 || ((uintptr_t)out % 8) != 0) return false;
  if (decode && nh / nkv > 16) return false;
  if (nh > 65535 || nkv > 65535) return false;
  return true;
}

// Floats of workspace a decode launch needs (0 when one split is enough).
long long lq_attention_mfma_workspace(int rows, int nh, int hd, int max_len) {
  const int nsplit = lq_ceil_div(max_len, SPLIT);
  if (nsplit <= 1) return 0;
  return (long long)rows * nh * nsplit * (hd + 2);
}

int lq_attention_mfma(const void* q, int ldq, void* out, int ldo, int rows, int batch, int nh, int nkv,
                      int hd, const int* row_pos, const int* seq_slot, const int* cu_rows,
                      const int* block_table, int bt_stride, const void* kcache, const void* vcache,
                      float scale, int window, int decode, int max_len, float* workspace,
                      long long workspace_floats, hipStream_t stream) {
  AttnArgs a;
  a.q = (const bf16_t*)q;
  a.ldq = ldq;
  a.out = (bf16_t*)out;
  a.ldo = ldo;
  a.nh = nh;
  a.nkv = nkv;
  a.row_pos = row_pos;
  a.seq_slot = seq_slot;
  a.cu_rows = cu_rows;
  a.block_table = block_table;
  a.bt_stride = bt_stride;
  a.kcache = (const bf16_t*)kcache;
  a.vcache = (const bf16_t*)vcache;
  a.scale_log2 = scale * 1.44269504088896340736f;
  a.window = window;
  a.batch = batch;
  a.part_o = nullptr;
  a.part_ml = nullptr;
  a.nsplit = 1;
  if (decode) {
    LQ_REQUIRE(rows == batch, "attention: decoding needs one row a sequence (%d rows, %d sequences)", rows, batch);
    LQ_REQUIRE(max_len > 0, "attention: decoding needs the longest sequence length");
    a.nsplit = lq_ceil_div(max_len, SPLIT);
    LQ_REQUIRE(a.nsplit <= 65535, "attention: %d tokens are too many splits", max_len);
    if (a.nsplit > 1) {
      const long long need = lq_attention_mfma_workspace(rows, nh, hd, max_len);
      LQ_REQUIRE(workspace != nullptr && workspace_floats >= need,
                 "attention: workspace of %lld floats needed, %lld given", need, workspace_floats);
      a.part_o = workspace;
      a.part_ml = workspace + (long long)rows * nh * a.nsplit * hd;
    }
  }
  switch (hd) {
    case 32: return launch<32>(a, rows, decode, stream);
    case 64: return launch<64>(a, rows, decode, stream);
    case 96: return launch<96>(a, rows, decode, stream);
    case 128: return launch<128>(a, rows, decode, stream);
    case 192: return launch<192>(a, rows, decode, stream);
    case 256: return launch<256>(a, rows, decode, stream);
  }
  lq_set_error("attention: head size %d has no matrix-core kernel", hd);
  return -1;
}
