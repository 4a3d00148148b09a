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
//  * rows (prompts): a wave owns QT tiles of 16 consecutive rows of one sequence for one query head
//    and reuses every key/value fragment it loads for all of them; the waves of a block are the
//    query heads of one kv head over the same rows, so that they read the same keys at the same time.
//  * heads (decoding): one row of one sequence, the query heads of one kv head as the 16 columns.
//    The waves of a block take the cache blocks (64 positions: two chunks) of a split of
//    `split_len` positions in turn (wave w: blocks w, w + NW, ...) and combine their partial results
//    through LDS in wave order.  A compute unit keeps about a hundred memory requests in flight,
//    whatever their size, so a sequence's keys are spread over many workgroups: a split is 256
//    positions or, where that would make more than MAX_DECODE_BLOCKS workgroups, the multiple of 64
//    that leaves the fullest compute unit the fewest keys (decode_split_len).  A row with several
//    splits is finished by whichever of its blocks comes last (a ticket counter per row and kv
//    head), which adds the partial results up in ascending split order: no second kernel, and the
//    result does not depend on which block that was.  Splits and chunks are aligned to absolute
//    positions.
#include <map>
#include <mutex>
#include <tuple>

#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

namespace {

constexpr int BS = 64;      // positions per cache block (the only block size this file takes)
constexpr int MAX_DECODE_BLOCKS = 512;  // beyond this, decoding splits grow instead of multiplying

__device__ inline bf16x8 as_bf16x8(u32x4 v) {
  union {
    u32x4 u;
    bf16x8 b;
  } c;
  c.u = v;
  return c.b;
}

typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

// two floats to packed bfloat16, round to nearest even (v_cvt_pk_bf16_f32)
__device__ inline unsigned pack_bf16(float lo, float hi) {
  union {
    bf16x2 b;
    unsigned u;
  } c;
  c.b = __builtin_convertvector((f32x2){lo, hi}, bf16x2);
  return c.u;
}

// Reductions over the four 16-lane rows of a wave (the lanes that share lane % 16) with the row-swap
// instructions of gfx950, which stay in the vector unit (a shuffle goes through LDS and back).
// v_permlane16_swap exchanges the odd rows of its first operand with the even rows of its second;
// with the same value in both, every lane then holds its own and its xor-16 partner's value, the
// lower row's first.  v_permlane32_swap does the same with the wave's halves.
__device__ inline float rows_max(float x) {
  auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  x = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
  auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
__device__ inline float rows_sum(float x) {
  auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  x = __uint_as_float(a[0]) + __uint_as_float(a[1]);
  auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

// 2^x for x <= 0 (v_exp_f32; results below the normal range flush to zero, which is what a
// probability that small is worth)
__device__ inline float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// The running maximum that the probabilities are taken against follows the scores' maximum lazily: it moves
// (and what has been summed is rescaled) only when some row of the wave meets a score more than this far
// above it, in the log2 domain.  Probabilities then reach 2^8 at most, which float32 sums and bfloat16
// operands (eight bits of exponent) hold as well as values below 1; the quotient at the end is the same.
// After a row's first keys the branch is taken rarely; with a slack of zero it ran whenever any row's maximum
// moved at all, and its multiplications of every accumulator cost 5 to 8 % of a long prompt's time.
constexpr float RESCALE_SLACK = 8.0f;

// Which key of a 32-key chunk row r of score tile j stands for: the rows are dealt out so that the
// eight probabilities a lane ends up with (rows (lane/16)*4 + e of both tiles) belong to eight
// consecutive keys, (lane/16)*8 .. +7: the second product then takes its V^T operand as one
// 16-byte run of keys.
__device__ inline int chunk_key(int j, int r) { return (r >> 2) * 8 + j * 4 + (r & 3); }

// One chunk of 32 keys for one query tile: from the raw score tiles s[2] (S^T, lane holds rows
// (lane/16)*4 + e of each 16-row tile, i.e. keys (lane/16)*8 + 4 j + e, for column lane%16) to the packed probabilities, updating the
// running maximum m (log2 domain, scores scaled by c = scale * log2 e) and normaliser share l.
// Returns the factor the output accumulator has to be multiplied with (1 if the maximum stayed).
// `masked` is wave-uniform: false when every key of the chunk is visible to every column.
__device__ inline float softmax_chunk(const f32x4 (&s)[2], float c, bool masked, bool col_valid, int t0, int lo,
                                      int pos, float& m, float& l, u32x4& pw) {
  const int g = (threadIdx.x & 63) >> 4;
  float sv[8];
#pragma unroll
  for (int j = 0; j < 2; ++j)
#pragma unroll
    for (int e = 0; e < 4; ++e) sv[j * 4 + e] = s[j][e];
  if (masked) {
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int t = t0 + g * 8 + j * 4 + e;
        if (!(col_valid && t >= lo && t <= pos)) sv[j * 4 + e] = -INFINITY;
      }
  }
  float cmax = fmaxf(fmaxf(fmaxf(sv[0], sv[1]), fmaxf(sv[2], sv[3])), fmaxf(fmaxf(sv[4], sv[5]), fmaxf(sv[6], sv[7])));
  cmax = rows_max(cmax) * c;  // c > 0: scaling commutes with the maximum
  float alpha = 1.0f;
  if (__any(cmax > m + RESCALE_SLACK)) {  // (false for -inf against -inf, true for anything against -inf)
    const float m_new = fmaxf(m, cmax);
    alpha = fast_exp2(m - ((m_new == -INFINITY) ? 0.f : m_new));
    l *= alpha;
    m = m_new;
  }
  const float m_safe = (m == -INFINITY) ? 0.f : m;  // a column with no key yet
  float psum = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    sv[i] = fast_exp2(fmaf(sv[i], c, -m_safe));  // -inf stays -inf, 2^-inf = 0
    psum += sv[i];
  }
  l += psum;
  pw[0] = pack_bf16(sv[0], sv[1]);
  pw[1] = pack_bf16(sv[2], sv[3]);
  pw[2] = pack_bf16(sv[4], sv[5]);
  pw[3] = pack_bf16(sv[6], sv[7]);
  return alpha;
}

// Partial results that cross from one block of a launch to another.  The L2 caches of the chip's
// dies are not coherent with each other for ordinary accesses, and the fences that make them so
// write back and invalidate a whole L2 for everybody.  Device-scope atomic stores and loads go
// past those caches instead: the writer waits until its stores have completed before it takes its
// ticket, the reader reads after it has seen the last ticket.
__device__ inline void publish_result(float* p, float v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ inline float other_blocks_result(const float* p) {
  return __hip_atomic_load(const_cast<float*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
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
  int split_len;   // positions per split, a multiple of 64
  int units;       // > 0: workgroups a kv head, which share the sequences' splits out among themselves
  int* tickets;    // [rows][nkv], zero between launches: how many splits of the row have finished
  // decode with the rotation and the cache write folded in (all null otherwise): the step's
  // unrotated keys and values, and cos/sin of every row's angles [rows][HD/2][2]
  const bf16_t* k_new;
  const bf16_t* v_new;
  int ldk, ldv;
  const float* cs;
  // > 1 (folded launches only): q, k_new and v_new are float32, the partial sums that a product whose K was
  // shared over blocks left, `pieces` of them `piece_stride` floats apart; ldq, ldk and ldv count floats.
  // The kernel adds them up in order and rounds the sums as the whole product would have.
  int pieces;
  long long piece_stride;
};

// One chunk's operands as they come from memory: 16 bytes a lane for each K fragment and for each
// V^T fragment.
template <int HD>
struct ChunkRegs {
  u32x4 k[2][HD / 32];
  u32x4 v[HD / 16];
};

// A whole cache block: both chunks of 32 keys.  Every line of the cache is asked for by two
// instructions next to each other (a key row's k-steps, a value row's two halves), which the L1
// turns into one request of 128 bytes; halves asked for by different waves go out as two of 64,
// and it is the number of requests in flight that a compute unit is short of.
// (Head sizes above 128 have no registers for a whole block: they load chunk by chunk, FIRST to
// FIRST + N - 1, into r[0 .. N-1].)
template <int HD, int FIRST, int N>
__device__ inline void load_block(const AttnArgs& a, int kvh, long long blk, ChunkRegs<HD> (&r)[N]) {
  const int lane = threadIdx.x & 63, c16 = lane & 15, g = lane >> 4;
  const bf16_t* kb = a.kcache + ((blk * a.nkv + kvh) * BS) * (long long)HD;
#pragma unroll
  for (int hf = 0; hf < N; ++hf)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int kk = 0; kk < HD / 32; ++kk)
        r[hf].k[j][kk] = *(const u32x4*)(kb + ((FIRST + hf) * 32 + chunk_key(j, c16)) * HD + kk * 32 + g * 8);
  const bf16_t* vb = a.vcache + ((blk * a.nkv + kvh) * (long long)HD) * BS;
#pragma unroll
  for (int dt = 0; dt < HD / 16; ++dt) {
    const bf16_t* vr = vb + (long long)(dt * 16 + c16) * BS;
#pragma unroll
    for (int hf = 0; hf < N; ++hf) r[hf].v[dt] = *(const u32x4*)(vr + (FIRST + hf) * 32 + g * 8);
  }
}

// What a wave carries for each of its QT query tiles.  Column c = lane % 16 of tile qt is valid if
// valid[qt]; its position is pos[qt], its first key lo[qt].  o[qt][dt][e] is the unnormalised
// O^T[dt*16 + (lane/16)*4 + e][c], m the running maximum (log2 domain), l this lane's share of
// the normaliser (to be summed over lane/16).
template <int HD, int QT>
struct QTiles {
  bf16x8 q[QT][HD / 32];
  f32x4 o[QT][HD / 16];
  float m[QT], l[QT];
  bool valid[QT];
  int pos[QT], lo[QT];
  int last_key[QT];   // largest position any column of the tile may see (wave-uniform)
  int first_key[QT];  // smallest (wave-uniform)
  int free_to[QT];    // chunks that end at or before this key and start at or after free_from are
  int free_from[QT];  //   visible to every column: no masking needed (wave-uniform; free_to = -1: never)
};

// Walks the cache blocks that start at t_first, t_first + t_step, ... while <= t_end (all multiples
// of 64).  Keys beyond t_written were never written and are kept out of the second product.
template <int HD, int QT>
__device__ inline void attend(const AttnArgs& a, QTiles<HD, QT>& w, int kvh, const int* table, int t_first,
                              int t_step, int t_end, int t_written) {
  const int lane = threadIdx.x & 63, g = lane >> 4;
  if (t_first > t_end) return;
  // One block a wave is in flight (it fills the compute unit's queue of requests by itself); only
  // the block number is fetched one round ahead.
  constexpr int AT_ONCE = HD <= 128 ? 2 : 1;
  ChunkRegs<HD> blk[AT_ONCE];
  long long blk_next = table[t_first / BS];
  for (int tb = t_first; tb <= t_end; tb += t_step) {
    const long long blk_now = blk_next;
    load_block<HD, 0, AT_ONCE>(a, kvh, blk_now, blk);
    blk_next = (tb + t_step <= t_end) ? table[(tb + t_step) / BS] : 0;
#pragma unroll
    for (int hf = 0; hf < 2; ++hf) {
      const int t0 = tb + hf * 32;
      if (t0 > t_end) break;
      if (AT_ONCE == 1 && hf == 1) load_block<HD, 1, AT_ONCE>(a, kvh, blk_now, blk);
      ChunkRegs<HD>& cur = blk[AT_ONCE == 2 ? hf : 0];
      // values of keys that were never written must not reach the product (0 * garbage may be NaN)
      if (t0 + 31 > t_written) {
        const int ta = t0 + g * 8;  // this lane's eight keys
#pragma unroll
        for (int dt = 0; dt < HD / 16; ++dt)
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            if (ta + 2 * e > t_written) cur.v[dt][e] &= 0xffff0000u;
            if (ta + 2 * e + 1 > t_written) cur.v[dt][e] &= 0x0000ffffu;
          }
      }
#pragma unroll
      for (int qt = 0; qt < QT; ++qt) {
        if (t0 > w.last_key[qt] || t0 + 31 < w.first_key[qt]) continue;  // nothing of this chunk is visible
        f32x4 s[2];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          s[j] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int kk = 0; kk < HD / 32; ++kk)
            s[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(cur.k[j][kk]), w.q[qt][kk], s[j], 0, 0, 0);
        }
        const bool masked = !(t0 + 31 <= w.free_to[qt] && t0 >= w.free_from[qt]);
        u32x4 pw;
        const float alpha = softmax_chunk(s, a.scale_log2, masked, w.valid[qt], t0, w.lo[qt], w.pos[qt], w.m[qt],
                                          w.l[qt], pw);
        const bf16x8 pb = as_bf16x8(pw);
        if (!__all(alpha == 1.0f)) {  // the maximum moved for some column: rescale what has been summed
#pragma unroll
          for (int dt = 0; dt < HD / 16; ++dt)
#pragma unroll
            for (int e = 0; e < 4; ++e) w.o[qt][dt][e] *= alpha;
        }
#pragma unroll
        for (int dt = 0; dt < HD / 16; ++dt)
          w.o[qt][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(cur.v[dt]), pb, w.o[qt][dt], 0, 0, 0);
      }
    }
  }
}

template <int HD, int QT>
__device__ inline void init_tiles(QTiles<HD, QT>& w) {
#pragma unroll
  for (int qt = 0; qt < QT; ++qt) {
#pragma unroll
    for (int dt = 0; dt < HD / 16; ++dt) w.o[qt][dt] = (f32x4){0.f, 0.f, 0.f, 0.f};
    w.m[qt] = -INFINITY;
    w.l[qt] = 0.f;
  }
}

// ------------------------------------------------------------------ rows (prompts)
// Block = NW waves = NW query heads of one kv head over the same QT * 16 rows.  The block walks
// the keys one cache block (64 positions) at a time: all threads copy the block's K [64][HD] and
// V^T [HD][64] from memory into padded LDS (next block's copy in registers while the current one is
// multiplied), and every wave reads its MFMA operands from there, so a key is fetched once for
// all the heads that share it.  LDS rows are padded (K: +16 bytes, V^T: +16 bytes) so that the
// operand reads of a quarter wave fall into distinct banks.  Keys lie in LDS in the order the score
// tiles read them (chunk_key).
template <int HD>
struct RowsLds {
  static constexpr int K_STRIDE = HD * 2 + 16;   // bytes per key row
  static constexpr int V_STRIDE = BS * 2 + 16;   // bytes per d row
  static constexpr int K_BYTES = BS * K_STRIDE;
  static constexpr int V_BYTES = HD * V_STRIDE;
  static constexpr int STAGE = K_BYTES + V_BYTES;
  static constexpr int PIECES = HD * 8;          // 16-byte pieces of K (and of V^T) in one cache block
};

template <int HD, int QT, int HW, int RT>
__global__ __launch_bounds__(HW * RT * 64, (HD <= 128 && HW * RT > 1 ? 2 : 1)) void attn_rows_kernel(AttnArgs a, int heads_per_block_group, int tiles, int units) {
  using L = RowsLds<HD>;
  constexpr int NW = HW * RT;  // wave = row group * HW + head: HW query heads of one kv head, RT groups of QT row tiles
  constexpr int ROWS = QT * 16 * RT;
  constexpr int THREADS = NW * 64;
  constexpr int PER_THREAD = (L::PIECES + THREADS - 1) / THREADS;  // pieces of K, and of V, per thread
  constexpr bool EARLY = PER_THREAD <= 8;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

  // Tasks (a tile of ROWS rows, counted sequence by sequence, for one group of heads) in descending
  // order of their keys: late tiles first.  Workgroups i, i + units, i + 2 units, ... land on the
  // same compute unit, so the tasks are dealt out in a snake (0 .. units-1, then back): a unit's
  // heavy task gets a light partner and the units finish together.
  const int per_tile = gridDim.x / tiles;  // groups of heads
  const int round = blockIdx.x / units, place = blockIdx.x % units;
  int task = round * units + ((round & 1) ? units - 1 - place : place);
  if ((round + 1) * units > (int)gridDim.x) task = blockIdx.x;  // the last, partial round stays in order
  const int head_group = task % per_tile;
  int t = tiles - 1 - task / per_tile, b = 0, r0 = -1, nrows = 0;
  for (; b < a.batch; ++b) {
    const int begin = a.cu_rows[b], n = a.cu_rows[b + 1] - begin;
    const int tiles = (n + ROWS - 1) / ROWS;
    if (t < tiles) {
      r0 = begin + t * ROWS;
      nrows = min(ROWS, n - t * ROWS);
      break;
    }
    t -= tiles;
  }
  if (r0 < 0) return;  // the whole block
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, c16 = lane & 15, g = lane >> 4;
  const int G = a.nh / a.nkv;
  // blockIdx.y = kv head * groups + group, a group being HW consecutive query heads of the kv head
  const int kvh = head_group / heads_per_block_group;
  const int hq = (head_group % heads_per_block_group) * HW + wave % HW;
  const int tile0 = (wave / HW) * QT;  // this wave's first row tile within the block
  const bool wave_active = hq < G;  // an idle wave still copies and meets the barriers
  const int h = kvh * G + min(hq, G - 1);
  const int* table = a.block_table + (long long)a.seq_slot[b] * a.bt_stride;
  const int p0 = a.row_pos[r0];

  QTiles<HD, QT> w;
  init_tiles<HD, QT>(w);
#pragma unroll
  for (int qt = 0; qt < QT; ++qt) {
    const int rows_here = min(16, nrows - (tile0 + qt) * 16);  // may be <= 0: the tile is empty
    const int rc = (tile0 + qt) * 16 + min(c16, max(rows_here, 1) - 1);
    const int row = r0 + min(rc, nrows - 1);
    w.valid[qt] = wave_active && c16 < rows_here;
    w.pos[qt] = p0 + min(rc, nrows - 1);
    w.lo[qt] = (a.window > 0 && w.pos[qt] >= a.window) ? w.pos[qt] - a.window + 1 : 0;
    const int first_pos = p0 + min((tile0 + qt) * 16, nrows - 1);
    w.last_key[qt] = (wave_active && rows_here > 0) ? p0 + (tile0 + qt) * 16 + rows_here - 1 : -1;
    w.first_key[qt] = (a.window > 0 && first_pos >= a.window) ? first_pos - a.window + 1 : 0;
    // keys up to the tile's first row's position and from its last row's window start on are visible to
    // all of its columns (those past a partial tile's rows run as copies of its last row, never stored)
    const int last_pos = p0 + (tile0 + qt) * 16 + rows_here - 1;
    w.free_to[qt] = (wave_active && rows_here > 0) ? first_pos : -1;
    w.free_from[qt] = (a.window > 0 && last_pos >= a.window) ? last_pos - a.window + 1 : 0;
    const bf16_t* qr = a.q + (long long)row * a.ldq + h * HD + g * 8;
#pragma unroll
    for (int kk = 0; kk < HD / 32; ++kk) w.q[qt][kk] = as_bf16x8(*(const u32x4*)(qr + kk * 32));
  }
  const int t_end = p0 + nrows - 1;  // the last key anyone here sees, and the last one written
  const int lo_tile = (a.window > 0 && p0 >= a.window) ? p0 - a.window + 1 : 0;
  const int blk_first = lo_tile / BS, blk_last = t_end / BS;

  u32x4 rk[PER_THREAD], rv[PER_THREAD];
  auto fetch = [&](int lb) {
    const long long blk = table[lb];
    const bf16_t* kb = a.kcache + (blk * a.nkv + kvh) * (long long)(BS * HD);
    const bf16_t* vb = a.vcache + (blk * a.nkv + kvh) * (long long)(HD * BS);
#pragma unroll
    for (int i = 0; i < PER_THREAD; ++i) {
      const int pc = tid + i * THREADS;
      if (pc < L::PIECES) {
        rk[i] = *(const u32x4*)(kb + pc * 8);
        rv[i] = *(const u32x4*)(vb + pc * 8);
      }
    }
  };
  auto stash = [&](int lb, unsigned char* stage) {
    // values of keys that were never written must not reach the product (0 * garbage may be NaN)
    const int base_key = lb * BS;
    const bool tail = base_key + BS - 1 > t_end;
#pragma unroll
    for (int i = 0; i < PER_THREAD; ++i) {
      const int pc = tid + i * THREADS;
      if (pc < L::PIECES) {
        // keys go to the row their score tile reads them from: row 16 j + r holds key chunk_key(j, r)
        const int key = pc / (HD / 8), part = pc % (HD / 8);
        const int k32 = key & 31;
        const int krow = (key & 32) + ((k32 >> 2) & 1) * 16 + (k32 >> 3) * 4 + (k32 & 3);
        *(u32x4*)(stage + krow * L::K_STRIDE + part * 16) = rk[i];
        const int d = pc >> 3, vpart = pc & 7;
        u32x4 v = rv[i];
        if (tail) {
          const int k0 = base_key + vpart * 8;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            if (k0 + 2 * e > t_end) v[e] &= 0xffff0000u;
            if (k0 + 2 * e + 1 > t_end) v[e] &= 0x0000ffffu;
          }
        }
        *(u32x4*)(stage + L::K_BYTES + d * L::V_STRIDE + vpart * 16) = v;
      }
    }
  };

  fetch(blk_first);
  stash(blk_first, smem);
  __syncthreads();
  for (int lb = blk_first; lb <= blk_last; ++lb) {
    unsigned char* cur = smem + ((lb - blk_first) & 1) * L::STAGE;
    unsigned char* nxt = smem + ((lb - blk_first + 1) & 1) * L::STAGE;
    const bool more = lb < blk_last;
    // The next block's loads are on their way during this block's products where a thread's share
    // of them is small enough to stay in registers meanwhile; else they follow the products.
    if (EARLY && more) fetch(lb + 1);
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      const int t0 = lb * BS + half * 32;
      if (t0 > t_end) break;
#pragma unroll
      for (int qt = 0; qt < QT; ++qt) {
        if (t0 > w.last_key[qt] || t0 + 31 < w.first_key[qt]) continue;  // nothing of this chunk is visible
        f32x4 sc[2];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          sc[j] = (f32x4){0.f, 0.f, 0.f, 0.f};
          const unsigned char* kr = cur + (half * 32 + 16 * j + c16) * L::K_STRIDE + g * 16;
#pragma unroll
          for (int kk = 0; kk < HD / 32; ++kk)
            sc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(*(const u32x4*)(kr + kk * 64)), w.q[qt][kk],
                                                            sc[j], 0, 0, 0);
        }
        const bool masked = !(t0 + 31 <= w.free_to[qt] && t0 >= w.free_from[qt]);
        u32x4 pw;
        const float alpha = softmax_chunk(sc, a.scale_log2, masked, w.valid[qt], t0, w.lo[qt], w.pos[qt], w.m[qt],
                                          w.l[qt], pw);
        const bf16x8 pb = as_bf16x8(pw);
        if (!__all(alpha == 1.0f)) {  // the maximum moved for some column: rescale what has been summed
#pragma unroll
          for (int dt = 0; dt < HD / 16; ++dt)
#pragma unroll
            for (int e = 0; e < 4; ++e) w.o[qt][dt][e] *= alpha;
        }
#pragma unroll
        for (int dt = 0; dt < HD / 16; ++dt) {
          const u32x4 vv = *(const u32x4*)(cur + L::K_BYTES + (dt * 16 + c16) * L::V_STRIDE + half * 64 + g * 16);
          w.o[qt][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(vv), pb, w.o[qt][dt], 0, 0, 0);
        }
      }
    }
    // Nobody reads nxt: its last readers passed the barrier below one round ago.
    if (more) {
      if (!EARLY) fetch(lb + 1);
      stash(lb + 1, nxt);
    }
    __syncthreads();
  }
#pragma unroll
  for (int qt = 0; qt < QT; ++qt) {
    float l = w.l[qt];
    l = rows_sum(l);
    if (!w.valid[qt]) continue;
    const float inv = 1.0f / l;
    bf16_t* orow = a.out + (long long)(r0 + (tile0 + qt) * 16 + c16) * a.ldo + h * HD + g * 4;
#pragma unroll
    for (int dt = 0; dt < HD / 16; ++dt) {
      u32x2 ww;
      ww[0] = pack_bf16(w.o[qt][dt][0] * inv, w.o[qt][dt][1] * inv);
      ww[1] = pack_bf16(w.o[qt][dt][2] * inv, w.o[qt][dt][3] * inv);
      *(u32x2*)(orow + dt * 16) = ww;
    }
  }
}

template <int HD, int QT, int HW, int RT>
int launch_rows(const AttnArgs& a, int rows, int groups, hipStream_t stream) {
  using L = RowsLds<HD>;
  constexpr int ROWS = QT * 16 * RT, NW = HW * RT;
  const size_t smem = 2 * (size_t)L::STAGE;
  auto kernel = attn_rows_kernel<HD, QT, HW, RT>;
  static bool configured = false;
  if (!configured && smem > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) {
      lq_set_error("attention: cannot reserve %zu bytes of LDS: %s", smem, hipGetErrorString(e));
      return -2;
    }
    configured = true;
  }
  const int tiles = lq_ceil_div(rows, ROWS) + a.batch;  // an upper bound: a sequence's last tile may be partial
  kernel<<<dim3(tiles * a.nkv * groups), NW * 64, smem, stream>>>(a, groups, tiles, lq_compute_units());
  LQ_CHECK_LAUNCH("attention(mfma rows)");
  return 0;
}

// ------------------------------------------------------------------ rows, 32 x 32 score tiles
// The same launch shape with the wider product, v_mfma_f32_32x32x16_bf16: a wave owns 32 consecutive
// rows of one query head, a block is the HW query heads of one kv head over the same 32 rows.  A K or
// V^T fragment read from LDS (1 KB) now feeds a product of 32 x 32 x 16 instead of 16 x 16 x 32: half
// the LDS traffic a flop, which is what bounded the narrower tile.
//   lane l gives A[row l%32][k (l/32)*8 .. +8] and B[col l%32][the same k]; it receives
//   D[(e/4)*8 + (l/32)*4 + e%4][l%32], e < 16.
//   First product: A = 32 keys x 16 of head_dim (LDS), B = 32 rows x the same 16 (registers):
//   S^T[key][row]; lane (row r, half h) holds keys (e/4)*8 + 4 h + e%4 of the chunk.
//   Second product, two steps of 16 keys: step s takes the lane's probabilities e = 8 s .. 8 s + 7 as
//   they are, so its k index 8 h + j stands for key 16 s + (j/4)*8 + 4 h + j%4; V^T lies in LDS with
//   the keys of every 16 in the order [0-3][8-11][4-7][12-15], which makes those eight one 16-byte run.
typedef float f32x16 __attribute__((ext_vector_type(16)));

// With KS = 2 a head's 32 rows are shared by two waves that take the first and the second 32 keys of every
// cache block and add their results up through LDS at the end: a tile's time is set by its last row tile's
// walk through all the keys before it, and on a short prompt, where the chip holds every tile at once, that
// walk is the launch's time.
template <int HD, int HW, int KS>
__global__ __launch_bounds__(HW * KS * 64, KS == 2 ? 1 : 2) void attn_rows32_kernel(AttnArgs a, int heads_per_block_group,
                                                                                   int tiles, int units) {
  using L = RowsLds<HD>;
  constexpr int ROWS = 32, THREADS = HW * KS * 64;
  constexpr int MERGE_FLOATS = HD / 32 * 16 * 64 + 2 * 64;  // a wave's accumulators, maxima and normaliser shares
  static_assert(KS == 1 || (KS == 2 && HW * MERGE_FLOATS * 4 <= 2 * L::STAGE), "the second waves' results fit the stages");
  constexpr int PER_THREAD = (L::PIECES + THREADS - 1) / THREADS;  // pieces of K, and of V, per thread
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

  // tasks as in attn_rows_kernel: late (heavy) tiles first, dealt out over the compute units in a snake
  const int per_tile = gridDim.x / tiles;
  const int round = blockIdx.x / units, place = blockIdx.x % units;
  int task = round * units + ((round & 1) ? units - 1 - place : place);
  if ((round + 1) * units > (int)gridDim.x) task = blockIdx.x;
  const int head_group = task % per_tile;
  int t = tiles - 1 - task / per_tile, b = 0, r0 = -1, nrows = 0;
  for (; b < a.batch; ++b) {
    const int begin = a.cu_rows[b], n = a.cu_rows[b + 1] - begin;
    const int tiles_b = (n + ROWS - 1) / ROWS;
    if (t < tiles_b) {
      r0 = begin + t * ROWS;
      nrows = min(ROWS, n - t * ROWS);
      break;
    }
    t -= tiles_b;
  }
  if (r0 < 0) return;  // the whole block
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, c32 = lane & 31, hf = lane >> 5;
  const int head_slot = wave % HW, ks = wave / HW;  // (ks: which 32 keys of a cache block, with KS = 2)
  const int G = a.nh / a.nkv;
  const int kvh = head_group / heads_per_block_group;
  const int hq = (head_group % heads_per_block_group) * HW + head_slot;
  const bool wave_active = hq < G;  // an idle wave still copies and meets the barriers
  const int h = kvh * G + min(hq, G - 1);
  const int* table = a.block_table + (long long)a.seq_slot[b] * a.bt_stride;
  const int p0 = a.row_pos[r0];

  // this lane's row (column of the score tile)
  const int rc = min(c32, nrows - 1);
  const bool valid = wave_active && c32 < nrows;
  const int pos = p0 + rc;
  const int lo = (a.window > 0 && pos >= a.window) ? pos - a.window + 1 : 0;
  const int last_key = wave_active ? p0 + nrows - 1 : -1;                       // wave-uniform
  const int first_key = (a.window > 0 && p0 >= a.window) ? p0 - a.window + 1 : 0;
  // keys up to the first row's position and from the last row's window start on are visible to all 32 rows
  // (the columns past a partial tile run as copies of its last row and are never stored: they see these keys too)
  const int free_to = wave_active ? p0 : -1;
  const int free_from = (a.window > 0 && p0 + nrows - 1 >= a.window) ? p0 + nrows - 1 - a.window + 1 : 0;
  bf16x8 q[HD / 16];
  {
    const bf16_t* qr = a.q + (long long)(r0 + rc) * a.ldq + h * HD + hf * 8;
#pragma unroll
    for (int kk = 0; kk < HD / 16; ++kk) q[kk] = as_bf16x8(*(const u32x4*)(qr + kk * 16));
  }
  f32x16 o[HD / 32];
#pragma unroll
  for (int dt = 0; dt < HD / 32; ++dt)
#pragma unroll
    for (int e = 0; e < 16; ++e) o[dt][e] = 0.f;
  float m = -INFINITY, l = 0.f;  // running maximum of the row (log2 domain); this lane's share of the normaliser

  const int t_end = p0 + nrows - 1;  // the last key anyone here sees, and the last one written
  const int blk_first = first_key / BS, blk_last = t_end / BS;

  u32x4 rk[PER_THREAD], rv[PER_THREAD];
  auto fetch = [&](int lb) {
    const long long blk = table[lb];
    const bf16_t* kb = a.kcache + (blk * a.nkv + kvh) * (long long)(BS * HD);
    const bf16_t* vb = a.vcache + (blk * a.nkv + kvh) * (long long)(HD * BS);
#pragma unroll
    for (int i = 0; i < PER_THREAD; ++i) {
      const int pc = tid + i * THREADS;
      if (pc < L::PIECES) {
        rk[i] = *(const u32x4*)(kb + pc * 8);
        rv[i] = *(const u32x4*)(vb + pc * 8);
      }
    }
  };
  auto stash = [&](int lb, unsigned char* stage) {
    // values of keys that were never written must not reach the product (0 * garbage may be NaN)
    const int base_key = lb * BS;
    const bool tail = base_key + BS - 1 > t_end;
#pragma unroll
    for (int i = 0; i < PER_THREAD; ++i) {
      const int pc = tid + i * THREADS;
      if (pc < L::PIECES) {
        const int key = pc / (HD / 8), part = pc % (HD / 8);  // keys in their own order: row = key
        *(u32x4*)(stage + key * L::K_STRIDE + part * 16) = rk[i];
        const int d = pc >> 3, vpart = pc & 7;  // eight keys of one d: 8 vpart .. + 7
        u32x4 v = rv[i];
        if (tail) {
          const int k0 = base_key + vpart * 8;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            if (k0 + 2 * e > t_end) v[e] &= 0xffff0000u;
            if (k0 + 2 * e + 1 > t_end) v[e] &= 0x0000ffffu;
          }
        }
        // within every 16 keys the order in LDS is [0-3][8-11][4-7][12-15]
        unsigned char* vrow = stage + L::K_BYTES + d * L::V_STRIDE + (vpart >> 1) * 32;
        const int odd = vpart & 1;
        *(u32x2*)(vrow + (odd ? 8 : 0)) = (u32x2){v[0], v[1]};
        *(u32x2*)(vrow + (odd ? 24 : 16)) = (u32x2){v[2], v[3]};
      }
    }
  };

  fetch(blk_first);
  stash(blk_first, smem);
  __syncthreads();
  for (int lb = blk_first; lb <= blk_last; ++lb) {
    unsigned char* cur = smem + ((lb - blk_first) & 1) * L::STAGE;
    unsigned char* nxt = smem + ((lb - blk_first + 1) & 1) * L::STAGE;
    const bool more = lb < blk_last;
    if (more) fetch(lb + 1);  // on their way during this block's products
#pragma unroll
    for (int hh = 0; hh < 2 / KS; ++hh) {
      const int half = KS == 2 ? ks : hh;
      const int t0 = lb * BS + half * 32;
      if (t0 > t_end) break;
      if (t0 > last_key || t0 + 31 < first_key) continue;  // nothing of this chunk is visible to this wave
      f32x16 sc;
#pragma unroll
      for (int e = 0; e < 16; ++e) sc[e] = 0.f;
      const unsigned char* kr = cur + (half * 32 + c32) * L::K_STRIDE + hf * 16;
      const unsigned char* vr = cur + L::K_BYTES + c32 * L::V_STRIDE + half * 64 + hf * 16;
      // All of the half's K fragments are asked for before the first product, and its V^T fragments as soon
      // as the products have been issued, so that they arrive during the products and the softmax: a wave
      // that asks for each fragment just before its product waits out the LDS latency sixteen times a half.
      u32x4 kf[HD / 16], vf[2][HD / 32];
#pragma unroll
      for (int kk = 0; kk < HD / 16; ++kk) kf[kk] = *(const u32x4*)(kr + kk * 32);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int kk = 0; kk < HD / 16; ++kk)
        sc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(kf[kk]), q[kk], sc, 0, 0, 0);
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2)
#pragma unroll
        for (int dt = 0; dt < HD / 32; ++dt) vf[s2][dt] = *(const u32x4*)(vr + dt * 32 * L::V_STRIDE + s2 * 32);
      __builtin_amdgcn_sched_barrier(0);
      const bool masked = !(t0 + 31 <= free_to && t0 >= free_from);
      if (masked) {
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int tk = t0 + (e >> 2) * 8 + hf * 4 + (e & 3);
          if (!(valid && tk >= lo && tk <= pos)) sc[e] = -INFINITY;
        }
      }
      float cmax = sc[0];
#pragma unroll
      for (int e = 1; e < 16; ++e) cmax = fmaxf(cmax, sc[e]);
      {  // the row's other sixteen keys are in the lane 32 places away
        auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(cmax), __float_as_uint(cmax), false, false);
        cmax = fmaxf(__uint_as_float(sw[0]), __uint_as_float(sw[1]));
      }
      cmax *= a.scale_log2;  // the scale is positive: it commutes with the maximum
      if (__any(cmax > m + RESCALE_SLACK)) {  // some row's maximum moved far: rescale what has been summed
        const float m_new = fmaxf(m, cmax);
        const float alpha = fast_exp2(m - ((m_new == -INFINITY) ? 0.f : m_new));
        l *= alpha;
        m = m_new;
#pragma unroll
        for (int dt = 0; dt < HD / 32; ++dt)
#pragma unroll
          for (int e = 0; e < 16; ++e) o[dt][e] *= alpha;
      }
      const float m_safe = (m == -INFINITY) ? 0.f : m;  // a row with no key yet
      float psum = 0.f;
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        sc[e] = fast_exp2(fmaf(sc[e], a.scale_log2, -m_safe));  // -inf stays -inf, 2^-inf = 0
        psum += sc[e];
      }
      l += psum;
      u32x4 pw[2];
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2)
#pragma unroll
        for (int j = 0; j < 4; ++j) pw[s2][j] = pack_bf16(sc[8 * s2 + 2 * j], sc[8 * s2 + 2 * j + 1]);
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2)
#pragma unroll
        for (int dt = 0; dt < HD / 32; ++dt)
          o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(vf[s2][dt]), as_bf16x8(pw[s2]), o[dt], 0, 0, 0);
    }
    // Nobody reads nxt: its last readers passed the barrier below one round ago.
    if (more) stash(lb + 1, nxt);
    __syncthreads();
  }
  if constexpr (KS == 2) {
    // the second waves' sums go to the first through LDS (everyone is past the last stage's reads)
    float* mine = (float*)smem + head_slot * MERGE_FLOATS;
    if (ks == 1) {
#pragma unroll
      for (int dt = 0; dt < HD / 32; ++dt)
#pragma unroll
        for (int e = 0; e < 16; ++e) mine[(dt * 16 + e) * 64 + lane] = o[dt][e];
      mine[HD / 32 * 16 * 64 + lane] = m;
      mine[HD / 32 * 16 * 64 + 64 + lane] = l;
    }
    __syncthreads();
    if (ks == 1) return;
    const float m1 = mine[HD / 32 * 16 * 64 + lane], l1 = mine[HD / 32 * 16 * 64 + 64 + lane];
    const float m_all = fmaxf(m, m1);
    const float m_safe = (m_all == -INFINITY) ? 0.f : m_all;
    const float f0 = fast_exp2(m - m_safe), f1 = fast_exp2(m1 - m_safe);  // 2^-inf = 0: a wave that saw no key
    l = l * f0 + l1 * f1;
#pragma unroll
    for (int dt = 0; dt < HD / 32; ++dt)
#pragma unroll
      for (int e = 0; e < 16; ++e) o[dt][e] = o[dt][e] * f0 + mine[(dt * 16 + e) * 64 + lane] * f1;
  }
  {
    auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(l), __float_as_uint(l), false, false);
    l = __uint_as_float(sw[0]) + __uint_as_float(sw[1]);
  }
  if (!valid) return;
  const float inv = 1.0f / l;
  bf16_t* orow = a.out + (long long)(r0 + c32) * a.ldo + h * HD + hf * 4;
#pragma unroll
  for (int dt = 0; dt < HD / 32; ++dt)
#pragma unroll
    for (int g4 = 0; g4 < 4; ++g4) {  // d = dt*32 + g4*8 + hf*4 + (0..3)
      u32x2 ww;
      ww[0] = pack_bf16(o[dt][g4 * 4 + 0] * inv, o[dt][g4 * 4 + 1] * inv);
      ww[1] = pack_bf16(o[dt][g4 * 4 + 2] * inv, o[dt][g4 * 4 + 3] * inv);
      *(u32x2*)(orow + dt * 32 + g4 * 8) = ww;
    }
}

template <int HD, int HW, int KS>
int launch_rows32(const AttnArgs& a, int rows, int groups, hipStream_t stream) {
  using L = RowsLds<HD>;
  const size_t smem = 2 * (size_t)L::STAGE;
  auto kernel = attn_rows32_kernel<HD, HW, KS>;
  static bool configured = false;
  if (!configured && smem > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) {
      lq_set_error("attention: cannot reserve %zu bytes of LDS: %s", smem, hipGetErrorString(e));
      return -2;
    }
    configured = true;
  }
  const int tiles = lq_ceil_div(rows, 32) + a.batch;  // an upper bound: a sequence's last tile may be partial
  kernel<<<dim3(tiles * a.nkv * groups), HW * KS * 64, smem, stream>>>(a, groups, tiles, lq_compute_units());
  LQ_CHECK_LAUNCH("attention(mfma rows, 32 x 32)");
  return 0;
}

// ------------------------------------------------------------------ heads (decoding)
// Block = NW waves over one split of one (sequence, kv head).  LDS: per wave HD x G floats of
// partial output (the valid columns only), G maxima, G normalisers.
// Which split of which sequence unit u of a kv head takes, when the units share the work out themselves
// (a few sequences, no window).  Every sequence's keys are cut into splits of one length: the smallest
// multiple of 256 with which the splits that hold keys number no more than the launch has units for a kv
// head.  Those splits are numbered through (the whole ones first, sequence after sequence, then every
// sequence's last, part-filled one), and unit u takes number u.  With sequences of unequal lengths a launch
// whose grid is (sequence, split) leaves the splits of the short ones empty and makes the long ones' as large
// as if all were long; here a unit has work or ends at once, and the units with work follow one another, so
// that the compute units (which take workgroups in turn) get equal numbers of them.  Lane l holds sequence l;
// every wave of the workgroup works out the same answer.
struct DecodeItem {
  int row, pos, slot, split_len, split;
  int first_unit, n_full, last_unit;  // the row's whole splits sit in units first_unit .., its last, part-filled one in last_unit
};

// Inclusive prefix sums over the wave's 64 lanes with data-parallel-primitive moves (no trip through LDS):
// within rows of 16 lanes by shifts of 1, 2, 4 and 8 (lanes shifted in from outside a row read zero), then
// lane 15 of a row into the odd rows and lane 31 into the upper half.
__device__ inline int wave_prefix_sums(int v) {
  v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xf, 0xf, true);   // row_shr:1
  v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xf, 0xf, true);   // row_shr:2
  v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xf, 0xf, true);   // row_shr:4
  v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xf, 0xf, true);   // row_shr:8
  v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xa, 0xf, false);  // row_bcast:15 into rows 1 and 3
  v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xc, 0xf, false);  // row_bcast:31 into rows 2 and 3
  return v;
}

// Splits of length 256 k that hold keys of a sequence whose newest position is `pos` (position p lies in block
// p / 256; blocks of 256 positions and their quotients are small integers, which a float division gives exactly).
// One function for the kernel's search and for the host's check of it.
__host__ __device__ inline int splits_with_keys(int pos, int k) {
  return (int)(((float)(pos >> 8) + 0.5f) / (float)k) + 1;
}
constexpr int UNIT_SEARCH_TRIES = 1024;

// -> 1: unit u has work (in `it`); 0: it has none; -1: no split length was found within the tries, which the
// host's choice of the units rules out (decode_units) as long as the lengths lie within the launch's bound.
__device__ inline int balanced_item(const AttnArgs& a, int u, DecodeItem& it) {
  const int lane = threadIdx.x & 63;
  const bool mine = lane < a.batch;
  const int pl = mine ? a.row_pos[lane] : -1;  // lane l looks after sequence l (at most 64 of them)
  const int sl = mine ? a.seq_slot[lane] : 0;
  const int total = __builtin_amdgcn_readlane(wave_prefix_sums(pl + 1), 63);
  // the smallest multiple of 256 with which the splits that hold keys are no more than the units; blocks of
  // 256 positions and their quotients are small integers, which a float division gives exactly
  int k = max(1, (total + 256 * a.units - 1) / (256 * a.units)), cnt = 0;
  for (int tries = 0; tries < UNIT_SEARCH_TRIES; ++tries, ++k) {
    cnt = mine ? splits_with_keys(pl, k) : 0;  // splits of this lane's sequence that hold keys
    if (__builtin_amdgcn_readlane(wave_prefix_sums(cnt), 63) <= a.units) break;
  }
  const int SL = 256 * k;
  // whole splits first, sequence after sequence, then the last splits (the part-filled ones): the two
  // workgroups that share a compute unit, c and c + 32 of a die's run, then differ as little as may be
  const int part = mine && (pl + 1) % SL != 0 ? 1 : 0, full = cnt - part;
  const int full_incl = wave_prefix_sums(full), part_incl = wave_prefix_sums(part);
  const int n_full = __builtin_amdgcn_readlane(full_incl, 63), n_part = __builtin_amdgcn_readlane(part_incl, 63);
  if (n_full + n_part > a.units) return -1;
  if (u >= n_full + n_part) return 0;
  const bool whole = u < n_full;
  const int row = whole ? __popcll(__ballot(mine && full_incl <= u))
                        : __popcll(__ballot(mine && part_incl <= u - n_full));
  it.row = row;
  it.pos = __builtin_amdgcn_readlane(pl, row);
  it.slot = __builtin_amdgcn_readlane(sl, row);
  it.split_len = SL;
  it.n_full = __builtin_amdgcn_readlane(full, row);
  it.first_unit = __builtin_amdgcn_readlane(full_incl - full, row);
  it.last_unit = n_full + __builtin_amdgcn_readlane(part_incl - part, row);
  it.split = whole ? u - it.first_unit : it.n_full;
  return 1;
}

template <int HD, int NW, bool PIECES = false>
__global__ __launch_bounds__(NW * 64, (HD <= 128 ? 2 : 1)) void attn_heads_kernel(AttnArgs a) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  const int G = a.nh / a.nkv;
  float* lds_o = lds;                    // [NW][HD][G]
  float* lds_m = lds + NW * HD * G;      // [NW][G]
  float* lds_l = lds_m + NW * G;         // [NW][G]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, c16 = lane & 15, g = lane >> 4;
  // grid (sequence, kv head, split), or (kv head, unit) when the units share the splits out themselves
  int b = blockIdx.x, kvh = blockIdx.y, split = blockIdx.z, SL = a.split_len, p, slot;
  int first_unit = 0, n_full = 0, last_unit = 0;
  if (a.units > 0) {
    DecodeItem it;
    kvh = blockIdx.x;
    const int found = balanced_item(a, blockIdx.y, it);
    if (found < 0) {
      // Nobody would write the output: make that loud instead of leaving what the buffer held.  Units 0 ..
      // batch - 1 (there are at least two a sequence) fill their row's heads of this kv head with NaN.
      if ((int)blockIdx.y < a.batch) {
        bf16_t nan;
        nan.bits = 0x7FC0;
        bf16_t* o = a.out + (long long)blockIdx.y * a.ldo + (long long)kvh * G * HD;
        for (int i = threadIdx.x; i < G * HD; i += NW * 64) o[i] = nan;
      }
      return;
    }
    if (found == 0) return;  // the whole block: more units than splits with keys
    b = it.row;
    p = it.pos;
    slot = it.slot;
    SL = it.split_len;
    split = it.split;
    first_unit = it.first_unit;
    n_full = it.n_full;
    last_unit = it.last_unit;
  } else {
    p = a.row_pos[b];
    slot = a.seq_slot[b];
  }
  const int r = b;  // a decoding step has one row a sequence, in the order of the sequences
  // Everything that depends on the row alone is asked for at once, before the position is known
  // (or, with units, together with the block table): a block's time is a chain of memory round trips
  // (position, block table, keys), and these join the first of them.
  const int h = kvh * G + min(c16, G - 1);
  const bool folded = HD % 64 == 0 && a.cs != nullptr;
  u32x4 qraw[HD / 32];
  constexpr int KP = (HD / 2 + 63) / 64, VP = (HD + 63) / 64;
  // (with pieces: the sums of this row's key pairs and value elements, lane i pair i and element i)
  float pk0[KP], pk1[KP], pv[VP];
  if constexpr (PIECES) {
    // A few pieces are asked for together, everything a lane needs of them at once, and added in ascending
    // order: one round trip for up to PC pieces.
    constexpr int PC = HD <= 128 ? 4 : 2;
    const float* qr = (const float*)a.q + (long long)r * a.ldq + h * HD + g * 8;
    const float* kf = (const float*)a.k_new + (long long)r * a.ldk + kvh * HD;
    const float* vf = (const float*)a.v_new + (long long)r * a.ldv + kvh * HD;
    f32x4 sq[HD / 32][2];
    for (int pc = 0; pc < a.pieces; pc += PC) {
      f32x4 tq[PC][HD / 32][2];
      float tk0[PC][KP], tk1[PC][KP], tv[PC][VP];
#pragma unroll
      for (int j = 0; j < PC; ++j) {
        const long long at = (long long)min(pc + j, a.pieces - 1) * a.piece_stride;
#pragma unroll
        for (int kk = 0; kk < HD / 32; ++kk) {
          tq[j][kk][0] = *(const f32x4*)(qr + at + kk * 32);
          tq[j][kk][1] = *(const f32x4*)(qr + at + kk * 32 + 4);
        }
#pragma unroll
        for (int e = 0; e < KP; ++e) {
          const int i = min(lane + 64 * e, HD / 2 - 1);
          tk0[j][e] = kf[at + i];
          tk1[j][e] = kf[at + i + HD / 2];
        }
#pragma unroll
        for (int e = 0; e < VP; ++e) tv[j][e] = vf[at + min(lane + 64 * e, HD - 1)];
      }
#pragma unroll
      for (int j = 0; j < PC; ++j) {
        if (pc + j >= a.pieces) continue;
        const bool first = pc + j == 0;
#pragma unroll
        for (int kk = 0; kk < HD / 32; ++kk) {
          sq[kk][0] = first ? tq[j][kk][0] : sq[kk][0] + tq[j][kk][0];
          sq[kk][1] = first ? tq[j][kk][1] : sq[kk][1] + tq[j][kk][1];
        }
#pragma unroll
        for (int e = 0; e < KP; ++e) {
          pk0[e] = first ? tk0[j][e] : pk0[e] + tk0[j][e];
          pk1[e] = first ? tk1[j][e] : pk1[e] + tk1[j][e];
        }
#pragma unroll
        for (int e = 0; e < VP; ++e) pv[e] = first ? tv[j][e] : pv[e] + tv[j][e];
      }
    }
#pragma unroll
    for (int kk = 0; kk < HD / 32; ++kk) {
      qraw[kk][0] = pack_bf16(sq[kk][0][0], sq[kk][0][1]);
      qraw[kk][1] = pack_bf16(sq[kk][0][2], sq[kk][0][3]);
      qraw[kk][2] = pack_bf16(sq[kk][1][0], sq[kk][1][1]);
      qraw[kk][3] = pack_bf16(sq[kk][1][2], sq[kk][1][3]);
    }
  } else {
    const bf16_t* qr = a.q + (long long)r * a.ldq + h * HD + g * 8;
#pragma unroll
    for (int kk = 0; kk < HD / 32; ++kk) qraw[kk] = *(const u32x4*)(qr + kk * 32);
  }
  // the row's own key and value (lane i: pair i of the key, elements d of the value), for the wave
  // that will turn out to write them
  float kx0[KP], kx1[KP], kc[KP], ks[KP];
  bf16_t vx[VP];
  if (folded) {
    const float* cs = a.cs + (long long)r * HD;  // [HD/2][2]
    const bf16_t* kr = a.k_new + (long long)r * a.ldk + kvh * HD;
    const bf16_t* vr = a.v_new + (long long)r * a.ldv + kvh * HD;
#pragma unroll
    for (int j = 0; j < KP; ++j) {
      const int i = min(lane + 64 * j, HD / 2 - 1);
      if constexpr (PIECES) {
        kx0[j] = bf16_to_f32(f32_to_bf16(pk0[j]));
        kx1[j] = bf16_to_f32(f32_to_bf16(pk1[j]));
      } else {
        kx0[j] = bf16_to_f32(kr[i]);
        kx1[j] = bf16_to_f32(kr[i + HD / 2]);
      }
      kc[j] = cs[2 * i];
      ks[j] = cs[2 * i + 1];
    }
#pragma unroll
    for (int j = 0; j < VP; ++j) {
      if constexpr (PIECES) vx[j] = f32_to_bf16(pv[j]);
      else vx[j] = vr[min(lane + 64 * j, HD - 1)];
    }
    // The rotation of this step's query, folded in.  Pair (i, i + HD/2): a lane's
    // fragment kk holds i = kk*32 + (lane/16)*8 + j and its fragment kk + HD/64 the partners.
#pragma unroll
    for (int kk = 0; kk < HD / 64; ++kk) {
      const int i0 = kk * 32 + g * 8;
      u32x4 lo4 = qraw[kk], hi4 = qraw[kk + HD / 64];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const f32x4 c2 = *(const f32x4*)(cs + (i0 + 2 * j) * 2);  // cos, sin of i0+2j and of i0+2j+1
        const float x0a = __uint_as_float(lo4[j] << 16), x0b = __uint_as_float(lo4[j] & 0xffff0000u);
        const float x1a = __uint_as_float(hi4[j] << 16), x1b = __uint_as_float(hi4[j] & 0xffff0000u);
        lo4[j] = pack_bf16(x0a * c2[0] - x1a * c2[1], x0b * c2[2] - x1b * c2[3]);
        hi4[j] = pack_bf16(x0a * c2[1] + x1a * c2[0], x0b * c2[3] + x1b * c2[2]);
      }
      qraw[kk] = lo4;
      qraw[kk + HD / 64] = hi4;
    }
#pragma unroll
    for (int j = 0; j < KP; ++j) {  // the key's rotation, by every wave: whoever writes it has it ready
      const float x0 = kx0[j], x1 = kx1[j];
      kx0[j] = x0 * kc[j] - x1 * ks[j];
      kx1[j] = x0 * ks[j] + x1 * kc[j];
    }
  }
  const int lo = (a.window > 0 && p >= a.window) ? p - a.window + 1 : 0;
  const int lo64 = (lo / BS) * BS;
  const int s_begin = max(split * SL, lo64);
  const int s_end = min(split * SL + SL - 1, p);
  if (s_begin > s_end) return;  // the whole block: this split holds no key of the row
  const int s_first = lo64 / SL, s_last = p / SL;  // the row's splits that hold keys
  const int* table = a.block_table + (long long)slot * a.bt_stride;

  QTiles<HD, 1> w;
  init_tiles<HD, 1>(w);
  w.valid[0] = c16 < G;
  w.pos[0] = p;
  w.lo[0] = lo;
  w.last_key[0] = p;
  w.first_key[0] = lo;
  w.free_to[0] = -1;  // columns beyond the group's heads are never valid: always the masked path
  w.free_from[0] = 0;
  // The wave that will read the block holding position p writes the row's rotated key and its
  // value there first; a workgroup-scope fence orders its lanes' stores before its lanes' loads.
  // No other wave (and no other workgroup) reads that block.
  if (folded && split == s_last && wave == ((p - split * SL) / BS) % NW) {
    const long long blk = table[p / BS];
    const int off = p % BS;
    bf16_t* kdst = const_cast<bf16_t*>(a.kcache) + ((blk * a.nkv + kvh) * BS + off) * (long long)HD;
    bf16_t* vdst = const_cast<bf16_t*>(a.vcache) + ((blk * a.nkv + kvh) * (long long)HD) * BS + off;
#pragma unroll
    for (int j = 0; j < KP; ++j) {
      const int i = lane + 64 * j;
      if (i < HD / 2) {
        bf16_t r0, r1;
        r0.bits = (uint16_t)(pack_bf16(kx0[j], 0.f) & 0xffffu);
        r1.bits = (uint16_t)(pack_bf16(kx1[j], 0.f) & 0xffffu);
        kdst[i] = r0;
        kdst[i + HD / 2] = r1;
      }
    }
#pragma unroll
    for (int j = 0; j < VP; ++j) {
      const int d = lane + 64 * j;
      if (d < HD) vdst[(long long)d * BS] = vx[j];
    }
    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "workgroup");
  }
#pragma unroll
  for (int kk = 0; kk < HD / 32; ++kk) w.q[0][kk] = as_bf16x8(qraw[kk]);
  // block numbering is absolute within the split, so that a wave's blocks depend on positions only
  int t_first = split * SL + wave * BS;
  while (t_first < s_begin) t_first += NW * BS;
  attend<HD, 1>(a, w, kvh, table, t_first, NW * BS, s_end, p);
  float l = w.l[0];
  l = rows_sum(l);

  // combine the waves' partial results in wave order
  if (c16 < G) {
    float* my_o = lds_o + (long long)wave * HD * G;
#pragma unroll
    for (int dt = 0; dt < HD / 16; ++dt)
#pragma unroll
      for (int e = 0; e < 4; ++e) my_o[(dt * 16 + g * 4 + e) * G + c16] = w.o[0][dt][e];
    if (g == 0) {
      lds_m[wave * G + c16] = w.m[0];
      lds_l[wave * G + c16] = l;
    }
  }
  __syncthreads();
  // every thread finishes some (d, column) pairs: HD * G of them over NW * 64 threads
  for (int idx = threadIdx.x; idx < HD * G; idx += NW * 64) {
    const int d = idx / G, c = idx - d * G;
    float M = -INFINITY;
#pragma unroll
    for (int j = 0; j < NW; ++j) M = fmaxf(M, lds_m[j * G + c]);
    float acc = 0.f, L = 0.f;
#pragma unroll
    for (int j = 0; j < NW; ++j) {
      const float mj = lds_m[j * G + c];
      const float wgt = (mj == -INFINITY) ? 0.f : exp2f(mj - M);
      acc += wgt * lds_o[((long long)j * HD + d) * G + c];
      L += wgt * lds_l[j * G + c];
    }
    const int hh = kvh * G + c;
    if (s_first == s_last) {
      a.out[(long long)r * a.ldo + hh * HD + d] = f32_to_bf16(acc / L);
    } else {
      // a split's partial results lie by (row, head, split), or by (kv head, unit, head of the group)
      const long long at = a.units > 0 ? ((long long)kvh * a.units + (split < n_full ? first_unit + split : last_unit)) * G + c
                                       : ((long long)r * a.nh + hh) * a.nsplit + split;
      publish_result(a.part_o + at * HD + d, acc);
      if (d == 0) {
        publish_result(a.part_ml + at * 2, M);
        publish_result(a.part_ml + at * 2 + 1, L);
      }
    }
  }
  if (s_first == s_last) return;

  // The row has other splits.  Once every thread's stores have completed the block takes a ticket;
  // the block that takes the last one adds the splits up.
  __shared__ int last_block;
  __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this thread's stores have been acknowledged
  __syncthreads();
  if (threadIdx.x == 0) {
    const int done = __hip_atomic_fetch_add(&a.tickets[(long long)r * a.nkv + kvh], 1, __ATOMIC_RELAXED,
                                            __HIP_MEMORY_SCOPE_AGENT);
    last_block = done == s_last - s_first;
  }
  __syncthreads();
  if (!last_block) return;
  for (int idx = threadIdx.x; idx < HD * G; idx += NW * 64) {
    const int d = idx / G, c = idx - d * G;
    const int hh = kvh * G + c;
    // split s of the row lies at place(s): by (row, head, split), or by (kv head, unit, head of the group)
    auto place = [&](int sidx) -> long long {
      if (a.units > 0) return ((long long)kvh * a.units + (sidx < n_full ? first_unit + sidx : last_unit)) * G + c;
      return ((long long)r * a.nh + hh) * a.nsplit + sidx;
    };
    // four splits' values are asked for together; the sum runs in ascending split order under a
    // running maximum
    float M = -INFINITY, acc = 0.f, L = 0.f;
    for (int s0 = s_first; s0 <= s_last; s0 += 4) {
      float pm[4], pl[4], po[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const long long sp = place(min(s0 + j, s_last));
        pm[j] = other_blocks_result(a.part_ml + sp * 2);
        pl[j] = other_blocks_result(a.part_ml + sp * 2 + 1);
        po[j] = other_blocks_result(a.part_o + sp * HD + d);
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (s0 + j > s_last || pm[j] == -INFINITY) continue;  // (a split whose keys the window hides)
        const float m_new = fmaxf(M, pm[j]);
        const float keep = exp2f(M - m_new), wgt = exp2f(pm[j] - m_new);
        acc = acc * keep + wgt * po[j];
        L = L * keep + wgt * pl[j];
        M = m_new;
      }
    }
    a.out[(long long)r * a.ldo + hh * HD + d] = f32_to_bf16(acc / L);
  }
  if (threadIdx.x == 0)  // for the next launch
    __hip_atomic_store(&a.tickets[(long long)r * a.nkv + kvh], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <int HD>
int launch(const AttnArgs& a, int rows, int decode, hipStream_t stream) {
  const int G = a.nh / a.nkv;
  if (!decode) {
    constexpr int QT = HD <= 64 ? 4 : (HD <= 128 ? 2 : 1);
    constexpr int QT2 = QT > 1 ? QT / 2 : 1;  // with two row groups of waves: the same rows a block, half a wave
    if constexpr (HD % 32 == 0 && HD <= 128) {
      // The 32 x 32 score tile (its accumulators fit up to this head size) reads half as much from LDS for a
      // product, with half as many waves on a compute unit to hide one wave's softmax behind another's
      // products.  As measured (32 heads over 8): at head size 64 it wins at every length (46 against 68 us at
      // 2 048 tokens, 353 against 429 at 8 192); at head size 128 it wins or ties at every length too (one
      // sequence of 256 tokens 16.7 against 16.6 us, of 1 000 tokens 33.8 against 34.2, of 2 048 tokens 65.9
      // against 67.7, of 8 192 tokens 612 against 682; sixteen sequences of 512 tokens 79 against 84, eight of 300
      // tokens 29.0 against 28.5) since its fragments are asked for early and partial tiles take the unmasked
      // path below the diagonal.  With one head a kv head a workgroup would be one wave that stages a whole
      // cache block through its own registers: then the narrow tiles stay for head sizes above 64.
      // Two waves a head (each half of every cache block's keys) where the workgroups would not even be one a
      // compute unit: the chip then holds twice the waves and a tile's walk through its keys takes half as
      // long (one sequence of 1 000 tokens 32.6 -> 28.5 us, of 700 tokens 24.8 -> 22.2).  With more workgroups
      // than that they would run one after the other, eight waves each, where two of four waves run side by
      // side (2 048 tokens 64.8 -> 72.8 us, 8 192 tokens 597 -> 648).
      const int hw = G >= 4 ? 4 : (G >= 2 ? 2 : 1);
      const bool two = (long long)lq_ceil_div(rows, 32) * a.nkv * lq_ceil_div(G, hw) <= lq_compute_units();
      if (G >= 4)
        return two ? launch_rows32<HD, 4, 2>(a, rows, lq_ceil_div(G, 4), stream)
                   : launch_rows32<HD, 4, 1>(a, rows, lq_ceil_div(G, 4), stream);
      if (G >= 2)
        return two ? launch_rows32<HD, 2, 2>(a, rows, lq_ceil_div(G, 2), stream)
                   : launch_rows32<HD, 2, 1>(a, rows, lq_ceil_div(G, 2), stream);
      if constexpr (HD <= 64)
        return two ? launch_rows32<HD, 1, 2>(a, rows, 1, stream) : launch_rows32<HD, 1, 1>(a, rows, 1, stream);
      else
        return launch_rows<HD, QT, 1, 1>(a, rows, 1, stream);
    } else {
      if (G >= 4) return launch_rows<HD, QT2, 4, 2>(a, rows, lq_ceil_div(G, 4), stream);
      if (G >= 2) return launch_rows<HD, QT, 2, 1>(a, rows, lq_ceil_div(G, 2), stream);
      return launch_rows<HD, QT, 1, 1>(a, rows, 1, stream);
    }
  }
  // Four waves a block (two where their partial outputs would not fit 48 KiB of LDS): small blocks
  // of which a compute unit holds several, each wave with one chunk in flight.
  const int per_wave = (HD * G + 2 * G) * (int)sizeof(float);
  dim3 grid(a.batch, a.nkv, a.nsplit);
  if (a.units > 0) grid = dim3(a.nkv, a.units, 1);
  if (a.pieces > 1) {
    if (4 * per_wave <= 48 * 1024)
      attn_heads_kernel<HD, 4, true><<<grid, 4 * 64, (size_t)4 * per_wave, stream>>>(a);
    else
      attn_heads_kernel<HD, 2, true><<<grid, 2 * 64, (size_t)2 * per_wave, stream>>>(a);
  } else if (4 * per_wave <= 48 * 1024)
    attn_heads_kernel<HD, 4><<<grid, 4 * 64, (size_t)4 * per_wave, stream>>>(a);
  else
    attn_heads_kernel<HD, 2><<<grid, 2 * 64, (size_t)2 * per_wave, stream>>>(a);
  LQ_CHECK_LAUNCH("attention(mfma heads)");
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

// Positions per block of a decoding launch: a multiple of 64 from 256 up, chosen so that the compute unit
// with the most keys has as few as may be.  Workgroups go to the chip's dies in turn and within a die to its
// compute units in turn, so with n workgroups the fullest unit has ceil(ceil(n / 8) / (units a die)) of them,
// each with a split's keys; more than MAX_DECODE_BLOCKS workgroups (two resident a unit) only where that pays
// for the waiting (33 to 63 long sequences, which one workgroup each would put two on some units and one on
// others), and of two lengths that come to the same the shorter (more waves to hide each other's round
// trips).  It depends on the
// bound rounded up to LQ_DECODE_LENGTH_BUCKET, so that launches whose bounds differ less than that add up their sums in the same
// order.
static int decode_split_len(int rows, int nkv, int max_len) {
  const long long bound = (long long)lq_ceil_div(max_len, LQ_DECODE_LENGTH_BUCKET) * LQ_DECODE_LENGTH_BUCKET;
  // (asked for at every launch: the answers are kept)
  static std::mutex guard;
  static std::map<std::tuple<int, int, long long>, int> known;
  const auto key = std::make_tuple(rows, nkv, bound);
  {
    std::lock_guard<std::mutex> lock(guard);
    const auto it = known.find(key);
    if (it != known.end()) return it->second;
  }
  const int per_die = lq_compute_units() / 8 > 0 ? lq_compute_units() / 8 : 1;
  long long best = 0, best_cost = 0, best_on = 0;
  for (long long sl = 256; sl <= bound; sl += 64) {
    const long long nsplit = (bound + sl - 1) / sl, blocks = (long long)rows * nkv * nsplit;
    if (blocks > 4 * MAX_DECODE_BLOCKS && nsplit > 1) continue;
    // (beyond the two workgroups that a compute unit holds at a time, each costs about 512 keys' worth of
    // waiting for its turn and of round trips that nothing hides; where two lengths come to the same, the one
    // with fewer workgroups a unit, and then the shorter)
    const long long on_fullest = ((blocks + 7) / 8 + per_die - 1) / per_die;
    const long long cost = on_fullest * sl + (on_fullest > 2 ? (on_fullest - 2) * 512 : 0);
    if (best == 0 || cost < best_cost || (cost == best_cost && on_fullest < best_on)) {
      best = sl;
      best_cost = cost;
      best_on = on_fullest;
    }
  }
  const int answer = (int)(best > 0 ? best : bound);
  std::lock_guard<std::mutex> lock(guard);
  known[key] = answer;
  return answer;
}

// Units a kv head for a decoding launch whose workgroups share the splits out themselves (0: the grid is
// (sequence, kv head, split)): as many as keep the launch within MAX_DECODE_BLOCKS workgroups, or, where that
// is less than two a sequence, LQ_UNITS_A_SEQUENCE a sequence (the workgroups beyond what a compute unit holds
// wait their turn); no more than the sequences have splits of 256 within their bound, and at least two a
// sequence, with which a split length that fits is sure to exist.  Taken for 2 to 64 sequences (a wave's
// lanes) without a window.
#ifndef LQ_UNITS_A_SEQUENCE
#define LQ_UNITS_A_SEQUENCE 4
#endif
static int decode_units(int rows, int nkv, int max_len, int window) {
  if (window > 0 || rows < 2 || rows > 64) return 0;
  const long long bound = (long long)lq_ceil_div(max_len, LQ_DECODE_LENGTH_BUCKET) * LQ_DECODE_LENGTH_BUCKET;
  long long by_cap = MAX_DECODE_BLOCKS / nkv;
  if (by_cap < 2 * rows) by_cap = (long long)LQ_UNITS_A_SEQUENCE * rows;
  const long long by_bound = (long long)rows * (bound / 256);
  const long long units = by_cap < by_bound ? by_cap : by_bound;
  if (units < 2 * rows || units > 65535) return 0;
  // The kernel looks for the split length upwards from (all keys) / (256 units) and finds it before twice
  // that; it gives the search 1 024 steps.
  if (rows * bound / (256 * units) > 512) return 0;
  return (int)units;
}

// The host's check of the search that the kernel's units make for their split length (balanced_item): the tries
// it takes for sequences whose newest positions are `pos[0..rows)`, or -1 if it does not end within
// UNIT_SEARCH_TRIES (which the choice of the units is meant to rule out), or 0 where the launch would not take
// the units' way at all.  The same arithmetic, one sequence after another instead of a lane each.
int lq_attention_mfma_unit_search(const int* pos, int rows, int nkv, int max_len) {
  const int units = decode_units(rows, nkv, max_len, 0);
  if (units <= 0) return 0;
  long long total = 0;
  for (int i = 0; i < rows; ++i) total += pos[i] + 1;
  int k = (int)((total + 256LL * units - 1) / (256LL * units));
  if (k < 1) k = 1;
  for (int tries = 0; tries < UNIT_SEARCH_TRIES; ++tries, ++k) {
    long long cnt = 0;
    for (int i = 0; i < rows; ++i) cnt += splits_with_keys(pos[i], k);
    if (cnt <= units) return tries + 1;
  }
  return -1;
}

// Floats of workspace a decode launch needs (0 when one split is enough): enough for either grid, the
// window being unknown here.
long long lq_attention_mfma_workspace(int rows, int nh, int nkv, int hd, int max_len) {
  const int nsplit = lq_ceil_div(max_len, decode_split_len(rows, nkv, max_len));
  const long long classic = nsplit <= 1 ? 0 : (long long)rows * nh * nsplit * (hd + 2);
  const long long shared = (long long)decode_units(rows, nkv, max_len, 0) * nh * (hd + 2);
  return classic > shared ? classic : shared;
}

int lq_attention_mfma(const void* q, int ldq, void* out, int ldo, int rows, int batch, int nh, int nkv,
                      int hd, const int* row_pos, const int* seq_slot, const int* cu_rows,
                      const int* block_table, int bt_stride, const void* kcache, const void* vcache,
                      float scale, int window, int decode, int max_len, float* workspace,
                      long long workspace_floats, int* tickets, long long tickets_n, const void* k_new,
                      const void* v_new, int ldk, int ldv, const float* cs, int uneven, int pieces,
                      long long piece_stride, hipStream_t stream) {
  AttnArgs a;
  a.pieces = pieces;
  a.piece_stride = piece_stride;
  if (pieces > 1) {
    LQ_REQUIRE(cs != nullptr, "attention: pieces of q, k and v are taken by the launch that rotates them only");
    LQ_REQUIRE(pieces <= 64 && piece_stride > 0 && piece_stride % 4 == 0 && ldq % 4 == 0,
               "attention: %d pieces %lld floats apart with rows of %d floats are not taken", pieces, piece_stride, ldq);
  }
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
  a.split_len = 256;
  a.units = 0;
  a.tickets = tickets;
  a.k_new = (const bf16_t*)k_new;
  a.v_new = (const bf16_t*)v_new;
  a.ldk = ldk;
  a.ldv = ldv;
  a.cs = cs;
  if (cs != nullptr) {
    LQ_REQUIRE(decode && hd % 64 == 0 && k_new && v_new && ldk >= nkv * hd && ldv >= nkv * hd,
               "attention: the folded rotation needs a decoding step, a head size that is a multiple of 64 and the step's keys and values");
    LQ_REQUIRE(((uintptr_t)cs % 16) == 0, "attention: the cos/sin table must be 16-byte aligned");
  }
  if (decode) {
    LQ_REQUIRE(rows == batch, "attention: decoding needs one row a sequence (%d rows, %d sequences)", rows, batch);
    LQ_REQUIRE(max_len > 0, "attention: decoding needs the longest sequence length");
    a.split_len = decode_split_len(rows, nkv, max_len);
    a.nsplit = lq_ceil_div(max_len, a.split_len);
    LQ_REQUIRE(a.nsplit <= 65535, "attention: %d tokens are too many splits", max_len);
    a.units = uneven ? decode_units(rows, nkv, max_len, window) : 0;  // (by the bound in 1 024s, as everything here)
    if (a.units > 0) {
      const long long need = (long long)a.units * nh * (hd + 2);
      LQ_REQUIRE(workspace != nullptr && workspace_floats >= need,
                 "attention: workspace of %lld floats needed, %lld given", need, workspace_floats);
      LQ_REQUIRE(tickets != nullptr && tickets_n >= (long long)rows * nkv,
                 "attention: %lld ticket counters needed for %d rows and %d kv heads, %lld given",
                 (long long)rows * nkv, rows, nkv, tickets_n);
      a.part_o = workspace;
      a.part_ml = workspace + (long long)a.units * nh * hd;
    } else if (a.nsplit > 1) {
      const long long need = lq_attention_mfma_workspace(rows, nh, nkv, hd, max_len);
      LQ_REQUIRE(workspace != nullptr && workspace_floats >= need,
                 "attention: workspace of %lld floats needed, %lld given", need, workspace_floats);
      LQ_REQUIRE(tickets != nullptr && tickets_n >= (long long)rows * nkv,
                 "attention: %lld ticket counters needed for %d rows and %d kv heads, %lld given",
                 (long long)rows * nkv, rows, nkv, tickets_n);
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
