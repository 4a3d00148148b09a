// Sampling on the device: repetition penalty, greedy arg-max, and temperature sampling with
// top-k and top-p, one block per sequence.
//
// The law follows the reference's sampler (internal/engine/sampler.go:72-105):
//   penalty on the distinct ids among the last 64 of the history (:249-275): logit /= pen if
//   positive, else *= pen; temperature 0 picks the first maximal index (:282-307); else
//   p = softmax(logits / T) (:125-156), candidates with p <= 1e-10 dropped (:158-166), order
//   by descending probability, keep the first k (:309-314), then the shortest prefix whose mass
//   reaches top_p (:316-339), draw r = U[0,1) * mass and take the candidate where the running
//   sum passes r (:168-184).
// Two things differ on purpose.  No sort: the kept set is a prefix of the descending order, so
// it is found as a threshold on the 64-bit key (logit bits, then lower index first) by bisection
// over counts and masses.  A histogram of the row first cuts off a short list of the largest keys
// that surely holds the kept set (more than top_k keys, or mass past top_p); the bisection and the
// draw then run on that list in LDS, and on the whole row only when no such list fits.  And the running sum of the draw walks the kept candidates
// in index order, not in order of probability: the law of the drawn token is the same, which
// token a given random number picks is not.
// Sums are double with a fixed tree, so a sequence's draw does not depend on the batch.
//
// Per-sequence sampler state lives in device arrays indexed by slot: a 64-bit key and counter for
// the random numbers (counter-based: draw n of a sequence depends on key and n only) and a ring
// of the last 64 token ids.
#include "common.h"
#include "lq_no_alloc.h"

#include <mutex>

typedef float f32x4 __attribute__((ext_vector_type(4)));

namespace {

constexpr int THREADS = 1024;
constexpr int RECENT = 64;

__device__ inline unsigned ordered_bits(float f) {
  // monotone map float -> unsigned (larger float, larger key); NaN sorts below everything
  if (f != f) return 0u;
  unsigned u = __float_as_uint(f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

__device__ inline float from_ordered_bits(unsigned k) {
  unsigned u = (k & 0x80000000u) ? (k & 0x7fffffffu) : ~k;
  return __uint_as_float(u);
}

__device__ inline unsigned long long shfl_xor_u64(unsigned long long v, int off) {
  unsigned lo = (unsigned)v, hi = (unsigned)(v >> 32);
  lo = __shfl_xor(lo, off, 64);
  hi = __shfl_xor(hi, off, 64);
  return ((unsigned long long)hi << 32) | lo;
}

__device__ inline unsigned long long shfl_up_u64(unsigned long long v, int off) {
  unsigned lo = (unsigned)v, hi = (unsigned)(v >> 32);
  lo = __shfl_up(lo, off, 64);
  hi = __shfl_up(hi, off, 64);
  return ((unsigned long long)hi << 32) | lo;
}

__device__ inline double shfl_f64(double v, int src) {
  const unsigned long long bits = (unsigned long long)__double_as_longlong(v);
  const unsigned hi = __shfl((unsigned)(bits >> 32), src, 64), lo = __shfl((unsigned)bits, src, 64);
  return __longlong_as_double((long long)(((unsigned long long)hi << 32) | lo));
}

__device__ inline double shfl_xor_f64(double v, int off) {
  return __longlong_as_double((long long)shfl_xor_u64((unsigned long long)__double_as_longlong(v), off));
}

// Block-wide reductions over THREADS threads with a fixed tree; every thread gets the result.
__device__ inline double block_sum_f64(double v, double* sm) {
  for (int off = 32; off > 0; off >>= 1) v += shfl_xor_f64(v, off);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) sm[threadIdx.x >> 6] = v;
  __syncthreads();
  double t = 0.0;
  for (int w = 0; w < THREADS / 64; ++w) t += sm[w];
  return t;
}

__device__ inline unsigned long long block_min_u64(unsigned long long v, unsigned long long* sm) {
  for (int off = 32; off > 0; off >>= 1) {
    const unsigned long long o = shfl_xor_u64(v, off);
    v = o < v ? o : v;
  }
  __syncthreads();
  if ((threadIdx.x & 63) == 0) sm[threadIdx.x >> 6] = v;
  __syncthreads();
  unsigned long long t = sm[0];
  for (int w = 1; w < THREADS / 64; ++w) t = sm[w] < t ? sm[w] : t;
  return t;
}

__device__ inline unsigned long long block_max_u64(unsigned long long v, unsigned long long* sm) {
  return ~block_min_u64(~v, sm);
}

__device__ inline long long block_sum_i64(long long v, unsigned long long* sm) {
  for (int off = 32; off > 0; off >>= 1) v += (long long)shfl_xor_u64((unsigned long long)v, off);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) sm[threadIdx.x >> 6] = (unsigned long long)v;
  __syncthreads();
  long long t = 0;
  for (int w = 0; w < THREADS / 64; ++w) t += (long long)sm[w];
  return t;
}

__device__ inline unsigned long long key_of(float logit, int index) {
  return ((unsigned long long)ordered_bits(logit) << 32) | (unsigned long long)(0xffffffffu - (unsigned)index);
}

// A row that holds a NaN or an infinity is not sampled from: its token comes out as NO_TOKEN, its
// generator and ring stay as they are, and the host reports it (the reference scans the row the same
// way and then takes the first finite index instead: internal/engine/sampler.go:72-75, 107-123).
// BAD_ROW is larger than any key (the largest, of +inf at index 0, has 0xff800000 as its upper half).
constexpr unsigned long long BAD_ROW = ~0ull;
constexpr int NO_TOKEN = -1;

__device__ inline bool non_finite(float f) { return (__float_as_uint(f) & 0x7f800000u) == 0x7f800000u; }

// the key, or BAD_ROW for a NaN or an infinity
__device__ inline unsigned long long checked_key_of(float logit, int index) {
  return non_finite(logit) ? BAD_ROW : key_of(logit, index);
}

// splitmix64 of (key, counter): the n-th uniform of a sequence, 53 bits in [0, 1)
__device__ inline double uniform_of(unsigned long long key, unsigned long long counter) {
  unsigned long long z = key + 0x9e3779b97f4a7c15ull * (counter + 1ull);
  z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
  z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
  z = z ^ (z >> 31);
  return (double)(z >> 11) * (1.0 / 9007199254740992.0);
}

__device__ inline void push_recent(int* recent, int* recent_n, int slot, int tok) {
  const int n = recent_n[slot];
  recent[(long long)slot * RECENT + (n % RECENT)] = tok;
  recent_n[slot] = n + 1;
}

// ------------------------------------------------------------------ penalty
__global__ __launch_bounds__(RECENT) void penalty_kernel(float* __restrict__ logits, int ld, int V,
                                                         const int* __restrict__ seq_slot,
                                                         const int* __restrict__ recent,
                                                         const int* __restrict__ recent_n, float penalty) {
  const int row = blockIdx.x, i = threadIdx.x;
  const int slot = seq_slot[row];
  const int n = min(recent_n[slot], RECENT);
  if (i >= n) return;
  const int* ring = recent + (long long)slot * RECENT;
  const int tok = ring[i];
  if (tok < 0 || tok >= V) return;
  for (int j = 0; j < i; ++j)
    if (ring[j] == tok) return;  // each distinct id once
  float* p = logits + (long long)row * ld + tok;
  const float v = *p;
  *p = v > 0.f ? v / penalty : v * penalty;
}

// ------------------------------------------------------------------ greedy
// Two stages so that a few rows still use many compute units: ARGMAX_PARTS blocks a row reduce a
// slice of the vocabulary each to its best key, one block a row reduces those.  Keys order by logit,
// then by lower index, so the result is the first maximal index whatever the slicing.
constexpr int ARGMAX_PARTS = 32;

__global__ __launch_bounds__(256) void argmax_part_kernel(const float* __restrict__ logits, int ld, int V,
                                                          unsigned long long* __restrict__ part) {
  __shared__ unsigned long long sm[4];
  const int row = blockIdx.y, slice = blockIdx.x;
  const float* lr = logits + (long long)row * ld;
  const int per = (V + ARGMAX_PARTS - 1) / ARGMAX_PARTS;
  const int i1 = min(V, (slice + 1) * per);
  unsigned long long best = 0ull;
  // eight loads a thread on their way at once: a slice of 4 000 logits is two round trips to memory, not sixteen
  for (int base = slice * per + threadIdx.x; base < i1; base += 8 * 256) {
    float v[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = base + j * 256 < i1 ? lr[base + j * 256] : 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      if (base + j * 256 < i1) {
        const unsigned long long k = checked_key_of(v[j], base + j * 256);
        best = k > best ? k : best;
      }
    }
  }
  for (int off = 32; off > 0; off >>= 1) {
    const unsigned long long o = shfl_xor_u64(best, off);
    best = o > best ? o : best;
  }
  if ((threadIdx.x & 63) == 0) sm[threadIdx.x >> 6] = best;
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < 4; ++w) best = sm[w] > best ? sm[w] : best;
    part[(long long)row * ARGMAX_PARTS + slice] = best;
  }
}

__global__ __launch_bounds__(64) void argmax_final_kernel(const unsigned long long* __restrict__ part,
                                                          const int* __restrict__ seq_slot, int* __restrict__ out,
                                                          int* __restrict__ recent, int* __restrict__ recent_n) {
  const int row = blockIdx.x;
  unsigned long long best = threadIdx.x < ARGMAX_PARTS ? part[(long long)row * ARGMAX_PARTS + threadIdx.x] : 0ull;
  for (int off = 32; off > 0; off >>= 1) {
    const unsigned long long o = shfl_xor_u64(best, off);
    best = o > best ? o : best;
  }
  if (threadIdx.x == 0) {
    if (best == BAD_ROW) {
      out[row] = NO_TOKEN;
      return;
    }
    const int tok = (int)(0xffffffffu - (unsigned)(best & 0xffffffffull));
    out[row] = tok;
    if (recent) push_recent(recent, recent_n, seq_slot[row], tok);
  }
}

// ------------------------------------------------------------------ temperature, top-k, top-p
struct SampleArgs {
  const float* logits;
  int ld, V;
  const int* seq_slot;
  float inv_temperature;
  int top_k;
  float top_p;
  long long* rng_key;
  long long* rng_ctr;
  int* recent;
  int* recent_n;
  int* out;
  int* kept_count;    // optional, per row
  double* kept_mass;  // optional, per row: mass of the kept set / total mass
};

// One pass over a set of logits: how many keys are >= theta, their mass (if wanted) and the smallest of them.
struct PassResult {
  long long count;
  double mass;
  unsigned long long kmin;
};

// f(logit, index) for every logit of the row, 16 bytes a lane where the row's alignment allows; the
// order in which a thread meets its elements depends on V and the row's address only.
template <typename F>
__device__ inline void for_each_logit(const float* lr, int V, F f) {
  const int tid = threadIdx.x;
  const int head = min(V, (int)(((16u - (unsigned)((uintptr_t)lr & 15u)) & 15u) / 4u));
  if (tid < head) f(lr[tid], tid);
  const int n4 = (V - head) / 4;
  const f32x4* p4 = (const f32x4*)(lr + head);
#pragma unroll 4
  for (int j = tid; j < n4; j += THREADS) {
    const f32x4 x = p4[j];
    const int i = head + 4 * j;
    f(x[0], i);
    f(x[1], i + 1);
    f(x[2], i + 2);
    f(x[3], i + 3);
  }
  const int tail = head + 4 * n4 + tid;
  if (tail < V) f(lr[tail], tail);
}

// The whole row in memory, all threads of the block.
struct RowPass {
  const float* lr;
  int V;
  float mx, invT;
  unsigned long long* smu;
  double* smd;
  __device__ PassResult over(unsigned long long theta, bool want_mass) const {
    long long cnt = 0;
    double mass = 0.0;
    unsigned long long kmin = ~0ull;
    for_each_logit(lr, V, [&](float v, int i) {
      const unsigned long long k = key_of(v, i);
      if (k >= theta) {
        ++cnt;
        if (want_mass) mass += (double)expf((v - mx) * invT);
        kmin = k < kmin ? k : kmin;
      }
    });
    PassResult r;
    r.count = block_sum_i64(cnt, smu);
    r.mass = want_mass ? block_sum_f64(mass, smd) : 0.0;
    r.kmin = block_min_u64(kmin, smu);
    return r;
  }
  // largest logit bits below lo, if any
  __device__ bool max_below(unsigned long long lo, unsigned long long& below) const {
    unsigned long long loc = 0ull;  // bits + 1, so that 0 means none
    for_each_logit(lr, V, [&](float v, int) {
      const unsigned long long hk = (unsigned long long)ordered_bits(v);
      if (hk < lo && hk + 1ull > loc) loc = hk + 1ull;
    });
    loc = block_max_u64(loc, smu);
    below = loc - 1ull;
    return loc > 0ull;
  }
};

// A short list of (logit, index) in LDS, ascending by index, worked on by one wave: no barriers.
struct ListPass {
  const float* val;
  const int* idx;
  int n;
  float mx, invT;
  __device__ PassResult over(unsigned long long theta, bool want_mass) const {
    const int lane = threadIdx.x & 63;
    long long cnt = 0;
    double mass = 0.0;
    unsigned long long kmin = ~0ull;
    for (int j = lane; j < n; j += 64) {
      const float v = val[j];
      const unsigned long long k = key_of(v, idx[j]);
      if (k >= theta) {
        ++cnt;
        if (want_mass) mass += (double)expf((v - mx) * invT);
        kmin = k < kmin ? k : kmin;
      }
    }
    for (int off = 32; off > 0; off >>= 1) {
      cnt += (long long)shfl_xor_u64((unsigned long long)cnt, off);
      mass += shfl_xor_f64(mass, off);
      const unsigned long long o = shfl_xor_u64(kmin, off);
      kmin = o < kmin ? o : kmin;
    }
    PassResult r;
    r.count = cnt;
    r.mass = mass;
    r.kmin = kmin;
    return r;
  }
  __device__ bool max_below(unsigned long long lo, unsigned long long& below) const {
    const int lane = threadIdx.x & 63;
    unsigned long long loc = 0ull;
    for (int j = lane; j < n; j += 64) {
      const unsigned long long hk = (unsigned long long)ordered_bits(val[j]);
      if (hk < lo && hk + 1ull > loc) loc = hk + 1ull;
    }
    for (int off = 32; off > 0; off >>= 1) {
      const unsigned long long o = shfl_xor_u64(loc, off);
      loc = o > loc ? o : loc;
    }
    below = loc - 1ull;
    return loc > 0ull;
  }
};

// The kept set is the longest allowed prefix of the descending order: at most k_limit members, all
// above the floor, and without its last member not yet at the top_p mass.  As a set it is
// {key >= theta}; allowed() is monotone in theta, so theta is found by bisection: first on the logit
// bits (whole groups of equal logits) from lo_bits up, then, only if the group below the boundary has
// several members, on the index bits inside that group.  `pass` must see every key >= lo_bits << 32,
// and the set of all of them must not be allowed unless lo_bits is 0.
template <typename P>
__device__ inline unsigned long long find_theta(const P& pass, unsigned long long best, unsigned long long lo_bits,
                                                long long k_limit, double e_floor, bool use_p, double p_mass) {
  auto allowed = [&](unsigned long long theta) -> bool {
    const PassResult r = pass.over(theta, use_p);
    if (r.count == 0) return true;
    const double e_min = (double)expf((from_ordered_bits((unsigned)(r.kmin >> 32)) - pass.mx) * pass.invT);
    return r.count <= k_limit && e_min > e_floor && (!use_p || r.mass - e_min < p_mass);
  };
  unsigned long long lo = lo_bits, hi = best >> 32;
  // the group of the maximum may itself be too large for k; then the index bisection below handles it
  if (!allowed(hi << 32)) {
    lo = hi = (best >> 32) + 1ull;  // nothing of the top group fits as a whole
  } else {
    while (lo < hi) {
      const unsigned long long mid = lo + (hi - lo) / 2ull;
      if (allowed(mid << 32))
        hi = mid;
      else
        lo = mid + 1ull;
    }
  }
  unsigned long long theta = lo << 32;  // 2^32 << 32 would need best >> 32 == 0xffffffff, a NaN: excluded
  if (lo > lo_bits) {
    unsigned long long below = 0ull;
    if (pass.max_below(lo, below) && below >= lo_bits) {
      const PassResult grp = pass.over(below << 32, false);
      const PassResult above = pass.over(lo << 32, false);
      if (grp.count - above.count > 1) {
        // several equal logits: admit them one by one in index order while allowed;
        // allowed(lo << 32) holds, allowed(below << 32) does not
        unsigned long long a2 = (below << 32) + 1ull, b2 = lo << 32;
        while (a2 < b2) {
          const unsigned long long mid = a2 + (b2 - a2) / 2ull;
          if (allowed(mid))
            b2 = mid;
          else
            a2 = mid + 1ull;
        }
        theta = a2;
      }
    }
  }
  return theta;
}

// The threshold and the draw on a short list of (logit, index), ascending by index, by one wave.  The
// list must hold the kept set, and whatever it holds besides must rank below it (then the longest allowed
// prefix of the list's descending order is that of the row's).
struct ListResult {
  int tok, kept;
  double mass;
};

__device__ inline ListResult list_draw(const float* list_val, const int* list_idx, int n_list, unsigned long long theta,
                                       float mx, float invT, double u);

__device__ inline ListResult list_threshold_and_draw(const float* list_val, const int* list_idx, int n_list,
                                                     unsigned long long best, float mx, float invT, long long k_limit,
                                                     double e_floor, bool use_p, double p_mass, double u) {
  const int lane = threadIdx.x & 63;
  ListPass pass{list_val, list_idx, n_list, mx, invT};
  unsigned long long lo_key = ~0ull;
  for (int j = lane; j < n_list; j += 64) {
    const unsigned long long k = key_of(list_val[j], list_idx[j]);
    lo_key = k < lo_key ? k : lo_key;
  }
  for (int off = 32; off > 0; off >>= 1) {
    const unsigned long long o = shfl_xor_u64(lo_key, off);
    lo_key = o < lo_key ? o : lo_key;
  }
  const unsigned long long theta = find_theta(pass, best, lo_key >> 32, k_limit, e_floor, use_p, p_mass);
  return list_draw(list_val, list_idx, n_list, theta, mx, invT, u);
}

// The same threshold for a list of a few dozen entries, without a search: every entry's rank and the mass
// of the entries before it in the descending order, by comparing it with all others (reads of one LDS
// word by all lanes at a time).  An entry is kept if fewer than k_limit rank before it, it is above the
// floor, and the mass before it is below the top_p mass: the longest allowed prefix, entry by entry.
__device__ inline unsigned long long list_threshold_by_ranks(const float* list_val, const int* list_idx, int n_list,
                                                             float mx, float invT, long long k_limit, double e_floor,
                                                             bool use_p, double p_mass, unsigned long long* key_sh,
                                                             float* e_sh) {
  const int lane = threadIdx.x & 63;
  // every entry's key and weight once (key_sh, e_sh: n_list entries of LDS that this wave owns)
  for (int j = lane; j < n_list; j += 64) {
    key_sh[j] = key_of(list_val[j], list_idx[j]);
    e_sh[j] = expf((list_val[j] - mx) * invT);
  }
  unsigned long long theta = ~0ull;  // the smallest kept key
  for (int i0 = 0; i0 < n_list; i0 += 64) {
    const int i = i0 + lane;
    const bool has = i < n_list;
    const unsigned long long ki = has ? key_sh[i] : ~0ull;
    int rank = 0;
    double before = 0.0;
    for (int j = 0; j < n_list; ++j) {
      const bool ahead = key_sh[j] > ki;
      rank += ahead ? 1 : 0;
      before += ahead ? (double)e_sh[j] : 0.0;  // in index order
    }
    const bool kept = has && rank < k_limit && (double)e_sh[min(i, n_list - 1)] > e_floor && (!use_p || before < p_mass);
    if (kept && ki < theta) theta = ki;
  }
  for (int off = 32; off > 0; off >>= 1) {
    const unsigned long long o = shfl_xor_u64(theta, off);
    theta = o < theta ? o : theta;
  }
  return theta;  // ~0: nothing is kept (then the draw falls back to the maximum)
}

__device__ inline ListResult list_draw(const float* list_val, const int* list_idx, int n_list, unsigned long long theta,
                                       float mx, float invT, double u) {
  const int lane = threadIdx.x & 63;
  // the draw: running sum over the kept entries in index order, a contiguous run of the list a lane
  const int chunk = (n_list + 63) / 64;
  const int j0 = min(n_list, lane * chunk), j1 = min(n_list, j0 + chunk);
  double mine = 0.0;
  int cnt = 0;
  for (int j = j0; j < j1; ++j)
    if (key_of(list_val[j], list_idx[j]) >= theta) {
      mine += (double)expf((list_val[j] - mx) * invT);
      ++cnt;
    }
  double incl = mine;
  for (int off = 1; off < 64; off <<= 1) {
    const unsigned long long bits = (unsigned long long)__double_as_longlong(incl);
    const unsigned hi32 = __shfl_up((unsigned)(bits >> 32), off, 64);
    const unsigned lo32 = __shfl_up((unsigned)bits, off, 64);
    const double o = __longlong_as_double((long long)(((unsigned long long)hi32 << 32) | lo32));
    if (lane >= off) incl += o;
  }
  const double all = shfl_f64(incl, 63);  // the mass of the kept set
  int kept = cnt;
  for (int off = 32; off > 0; off >>= 1) kept += __shfl_xor(kept, off, 64);
  const double r = u * all;
  const double lo_excl = incl - mine;
  int tok = -1;
  if (cnt > 0 && r >= lo_excl && r < incl) {
    double acc = lo_excl;
    for (int j = j0; j < j1; ++j)
      if (key_of(list_val[j], list_idx[j]) >= theta) {
        acc += (double)expf((list_val[j] - mx) * invT);
        tok = list_idx[j];
        if (r < acc) break;
      }
  }
  // at most one lane's range holds r
  for (int off = 32; off > 0; off >>= 1) tok = max(tok, __shfl_xor(tok, off, 64));
  ListResult res;
  res.tok = tok;
  res.kept = kept;
  res.mass = all;
  return res;
}

// Histogram of the row over (max - logit): bin width chosen so that every candidate (p > 1e-10) falls
// into the bins before the last.  Counts and masses are integers (mass in units of 2^-40), so that the
// order of the atomic additions does not matter.
constexpr int HIST_BINS = 1024;
constexpr int LIST_CAP = 6144;   // entries of the short list in LDS
constexpr double MASS_UNIT = 1099511627776.0;  // 2^40

__global__ __launch_bounds__(THREADS) void sample_kernel(SampleArgs a, const int* only) {
  __shared__ unsigned long long smu[THREADS / 64];
  __shared__ double smd[THREADS / 64];
  __shared__ double scan[THREADS];
  __shared__ int winner;
  __shared__ unsigned hist_count[HIST_BINS];
  __shared__ unsigned long long hist_mass[HIST_BINS];
  __shared__ float list_val[LIST_CAP];
  __shared__ int list_idx[LIST_CAP];
  __shared__ int wave_count[THREADS / 64 + 1];
  __shared__ int cut_bin;
  __shared__ unsigned long long theta_sh;
  __shared__ int tok_sh, kept_sh;
  __shared__ double total_sh;
  const int row = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  if (only != nullptr && only[row] == 0) return;  // the parts have dealt with this row
  const float* lr = a.logits + (long long)row * a.ld;
  const int V = a.V;
  const float invT = a.inv_temperature;

  // maximum logit (as a key: also gives the arg-max)
  unsigned long long best = 0ull;
  for_each_logit(lr, V, [&](float v, int i) {
    const unsigned long long k = checked_key_of(v, i);
    best = k > best ? k : best;
  });
  best = block_max_u64(best, smu);
  if (best == BAD_ROW) {  // the same for every thread of the block
    if (tid == 0) {
      a.out[row] = NO_TOKEN;
      if (a.kept_count) a.kept_count[row] = 0;
      if (a.kept_mass) a.kept_mass[row] = 0.0;
    }
    return;
  }
  const float mx = from_ordered_bits((unsigned)(best >> 32));

  // e_i = exp((l_i - max) / T) in 32-bit, sums in double; Z = sum e_i; candidates need p > 1e-10
  double zloc = 0.0;
  for_each_logit(lr, V, [&](float v, int) { zloc += (double)expf((v - mx) * invT); });
  const double Z = block_sum_f64(zloc, smd);
  const double e_floor = 1e-10 * Z;
  const bool use_p = a.top_p > 0.f && a.top_p < 1.f;
  const double p_mass = (double)a.top_p * Z;

  // candidates: their number, the smallest of them; and the histogram
  for (int bin = tid; bin < HIST_BINS; bin += THREADS) {
    hist_count[bin] = 0u;
    hist_mass[bin] = 0ull;
  }
  __syncthreads();
  // a candidate has (max - l) / T < ln(1e10) + ln(Z) <= 23.03 + ln(V): all of them lie in bins < HIST_BINS - 1
  const float span = (23.1f + logf((float)V)) / invT;
  const float inv_width = (float)(HIST_BINS - 1) / span;
  const bool select = a.top_k > 0 || use_p;
  long long ncand_loc = 0;
  unsigned long long cand_min = ~0ull;
  for_each_logit(lr, V, [&](float v, int i) {
    const float e = expf((v - mx) * invT);
    if ((double)e > e_floor) {
      ++ncand_loc;
      const unsigned long long k = key_of(v, i);
      cand_min = k < cand_min ? k : cand_min;
    }
    if (select) {
      const float d = (mx - v) * inv_width;
      if (d >= 0.f && d < (float)(HIST_BINS - 1)) {  // beyond: no candidate (and NaN); the cut never looks there
        const int bin = (int)d;
        atomicAdd(&hist_count[bin], 1u);
        atomicAdd(&hist_mass[bin], (unsigned long long)((double)e * MASS_UNIT));
      }
    }
  });
  const long long ncand = block_sum_i64(ncand_loc, smu);
  cand_min = block_min_u64(cand_min, smu);
  const long long k_limit = (a.top_k > 0 && a.top_k < ncand) ? a.top_k : ncand;
  __syncthreads();

  // A cut in the histogram: the first bins that surely hold more than the kept set (more than top_k
  // keys, or a mass past top_p by a margin and then one more non-empty bin).  The keys of these bins
  // become a short list in LDS, on which the threshold is then found exactly.
  if (wave == 0) {
    int cut = -1;
    if (select) {
      // lane l owns bins [16 l, 16 l + 16); running totals up to its first bin by a wave scan
      constexpr int PER = HIST_BINS / 64;
      const unsigned long long m_need = (unsigned long long)(p_mass * (1.0 + 1e-9) * MASS_UNIT) + (unsigned long long)V + 1ull;
      unsigned long long n_mine = 0ull, m_mine = 0ull;
      for (int j = 0; j < PER; ++j) {
        n_mine += hist_count[lane * PER + j];
        m_mine += hist_mass[lane * PER + j];
      }
      unsigned long long n_incl = n_mine, m_incl = m_mine;
      for (int off = 1; off < 64; off <<= 1) {
        const unsigned long long on = shfl_up_u64(n_incl, off), om = shfl_up_u64(m_incl, off);
        if (lane >= off) {
          n_incl += on;
          m_incl += om;
        }
      }
      unsigned long long cum_n = n_incl - n_mine, cum_m = m_incl - m_mine;
      int bin_k = HIST_BINS, bin_m = HIST_BINS;  // the first bin after which more than top_k keys / the mass are in
      for (int j = 0; j < PER; ++j) {
        const int bin = lane * PER + j;
        cum_n += hist_count[bin];
        cum_m += hist_mass[bin];
        if (a.top_k > 0 && cum_n > (unsigned long long)a.top_k && bin_k == HIST_BINS) bin_k = bin;
        if (use_p && cum_m >= m_need && bin_m == HIST_BINS) bin_m = bin;
      }
      for (int off = 32; off > 0; off >>= 1) {
        bin_k = min(bin_k, __shfl_xor(bin_k, off, 64));
        bin_m = min(bin_m, __shfl_xor(bin_m, off, 64));
      }
      // past the mass: one more non-empty bin
      int after = HIST_BINS;
      for (int j = PER - 1; j >= 0; --j) {
        const int bin = lane * PER + j;
        if (bin > bin_m && hist_count[bin] > 0u) after = bin;
      }
      for (int off = 32; off > 0; off >>= 1) after = min(after, __shfl_xor(after, off, 64));
      const int first = min(bin_k, after);
      if (first < HIST_BINS - 1) cut = first;
    }
    if (lane == 0) cut_bin = cut;
  }
  __syncthreads();
  const int cut = cut_bin;
  int n_list = 0;
  if (cut >= 0) {
    for (int bin = tid; bin <= cut; bin += THREADS) n_list += (int)hist_count[bin];
    n_list = (int)block_sum_i64(n_list, smu);
  }
  const bool short_list = cut >= 0 && n_list <= LIST_CAP;

  const int slot = a.seq_slot[row];
  const unsigned long long ctr = (unsigned long long)a.rng_ctr[slot];
  const double u = uniform_of((unsigned long long)a.rng_key[slot], ctr);

  if (short_list) {
    // the list, ascending by index: every wave owns a contiguous run of the row
    const int head = min(V, (int)(((16u - (unsigned)((uintptr_t)lr & 15u)) & 15u) / 4u));
    const int n4 = (V - head) / 4;
    const int per_wave = (n4 + THREADS / 64 - 1) / (THREADS / 64);
    const int j_begin = min(n4, wave * per_wave), j_end = min(n4, j_begin + per_wave);
    const f32x4* p4 = (const f32x4*)(lr + head);
    auto in_cut = [&](float v) -> bool {
      const float d = (mx - v) * inv_width;
      return d >= 0.f && d < (float)(HIST_BINS - 1) && (int)d <= cut;
    };
    for (int phase = 0; phase < 2; ++phase) {
      int at = phase == 0 ? 0 : wave_count[wave];  // where this wave's next entry goes
      auto put = [&](bool take, float v, int i, unsigned long long before_mask) {
        const unsigned long long m = __ballot(take);
        if (phase == 1 && take) {
          const int pos = at + __popcll(m & before_mask);
          list_val[pos] = v;
          list_idx[pos] = i;
        }
        at += __popcll(m);
      };
      const unsigned long long lt = (1ull << lane) - 1ull;
      if (wave == 0) {  // the unaligned head of the row
        const bool has = lane < head;
        const float v = has ? lr[lane] : 0.f;
        put(has && in_cut(v), v, lane, lt);
      }
      for (int j0 = j_begin; j0 < j_end; j0 += 64) {
        const int j = j0 + lane;
        const bool has = j < j_end;
        const f32x4 x = has ? p4[j] : (f32x4){0.f, 0.f, 0.f, 0.f};
        const int i = head + 4 * j;
        // index order: lane by lane, and a lane's four in turn
        const bool t0 = has && in_cut(x[0]), t1 = has && in_cut(x[1]), t2 = has && in_cut(x[2]), t3 = has && in_cut(x[3]);
        const int mine = (int)t0 + (int)t1 + (int)t2 + (int)t3;
        int incl = mine;
        for (int off = 1; off < 64; off <<= 1) {
          const int o = __shfl_up(incl, off, 64);
          if (lane >= off) incl += o;
        }
        if (phase == 1) {
          int pos = at + incl - mine;
          if (t0) { list_val[pos] = x[0]; list_idx[pos] = i; ++pos; }
          if (t1) { list_val[pos] = x[1]; list_idx[pos] = i + 1; ++pos; }
          if (t2) { list_val[pos] = x[2]; list_idx[pos] = i + 2; ++pos; }
          if (t3) { list_val[pos] = x[3]; list_idx[pos] = i + 3; ++pos; }
        }
        at += __shfl(incl, 63, 64);
      }
      if (wave == THREADS / 64 - 1) {  // the row's last few
        const int i = head + 4 * n4 + lane;
        const bool has = i < V;
        const float v = has ? lr[i] : 0.f;
        put(has && in_cut(v), v, i, lt);
      }
      if (phase == 0) {
        __syncthreads();
        if (lane == 0) wave_count[wave + 1] = at;  // counts first, shifted by one
        __syncthreads();
        if (tid == 0) {
          wave_count[0] = 0;
          for (int w = 1; w <= THREADS / 64; ++w) wave_count[w] += wave_count[w - 1];
        }
        __syncthreads();
      }
    }
    __syncthreads();
    // one wave finds the threshold and draws; the list holds every key >= its smallest one
    if (wave == 0) {
      const ListResult res = list_threshold_and_draw(list_val, list_idx, n_list, best, mx, invT, k_limit, e_floor, use_p,
                                                     p_mass, u);
      if (lane == 0) {
        tok_sh = res.tok;
        kept_sh = res.kept;
        total_sh = res.mass;
      }
    }
    __syncthreads();
  } else {
    // the row itself: when nothing is cut (all candidates are kept) or the list would not fit
    unsigned long long theta;
    if (!select) {
      theta = ncand > 0 ? cand_min : 0ull;  // every candidate: the floor is the only rule
    } else {
      RowPass pass{lr, V, mx, invT, smu, smd};
      theta = find_theta(pass, best, 0ull, k_limit, e_floor, use_p, p_mass);
    }
    // the draw: running sum over the kept candidates in index order
    const int chunk = (V + THREADS - 1) / THREADS;
    const int i0 = min(V, tid * chunk), i1 = min(V, i0 + chunk);
    double mine = 0.0;
    long long cnt_loc = 0;
    for (int i = i0; i < i1; ++i)
      if (key_of(lr[i], i) >= theta) {
        mine += (double)expf((lr[i] - mx) * invT);
        ++cnt_loc;
      }
    scan[tid] = mine;
    __syncthreads();
    // inclusive prefix sums of scan[]: lane j of wave 0 sums its 16 entries serially, a wave scan
    // gives each lane what lies before it
    if (tid < 64) {
      double run = 0.0;
      for (int j = 0; j < THREADS / 64; ++j) {
        run += scan[tid * (THREADS / 64) + j];
        scan[tid * (THREADS / 64) + j] = run;
      }
      double incl = run;
      for (int off = 1; off < 64; off <<= 1) {
        const unsigned long long bits = (unsigned long long)__double_as_longlong(incl);
        const unsigned hi32 = __shfl_up((unsigned)(bits >> 32), off, 64);
        const unsigned lo32 = __shfl_up((unsigned)bits, off, 64);
        const double o = __longlong_as_double((long long)(((unsigned long long)hi32 << 32) | lo32));
        if (tid >= off) incl += o;
      }
      const double before = incl - run;
      for (int j = 0; j < THREADS / 64; ++j) scan[tid * (THREADS / 64) + j] += before;
    }
    if (tid == 0) winner = -1;
    __syncthreads();
    const double total = scan[THREADS - 1];
    const long long kept = block_sum_i64(cnt_loc, smu);
    const double r = u * total;
    const double hi_incl = scan[tid];
    const double lo_excl = hi_incl - mine;
    if (cnt_loc > 0 && r >= lo_excl && r < hi_incl) {
      double acc = lo_excl;
      int tok = -1;
      for (int i = i0; i < i1; ++i)
        if (key_of(lr[i], i) >= theta) {
          acc += (double)expf((lr[i] - mx) * invT);
          tok = i;
          if (r < acc) break;
        }
      winner = tok;  // the ranges are disjoint: at most one thread's range holds r
    }
    __syncthreads();
    if (tid == 0) {
      tok_sh = winner;
      kept_sh = (int)kept;
      total_sh = total;
    }
    __syncthreads();
  }
  if (tid == 0) {
    int tok = tok_sh;
    if (tok < 0) tok = (int)(0xffffffffu - (unsigned)(best & 0xffffffffull));  // r fell on a rounding seam
    a.out[row] = tok;
    a.rng_ctr[slot] = (long long)(ctr + 1ull);
    if (a.recent) push_recent(a.recent, a.recent_n, slot, tok);
    if (a.kept_count) a.kept_count[row] = kept_sh;
    if (a.kept_mass) a.kept_mass[row] = total_sh / Z;
  }
}

// ------------------------------------------------------------------ top-k in parts
// With a small top_k the kept set lies among the k largest of the row, and those lie among the k largest
// of every slice of the row.  So the row is first cut into SAMPLE_PARTS slices, a block each: it leaves
// its slice's largest key, the slice's sum of exp((l - slice max) / T), and the entries that rank among
// the slice's k largest values (all that tie with the k-th: at most PART_CAP, else the row is flagged
// and goes the long way), in index order.  One block a row then puts the parts together: the row's
// maximum, Z = sum over the slices of their sums scaled to it, the list, and on it the same threshold
// search and draw as above.  Five passes of one compute unit over the row become one pass of 32.
constexpr int SAMPLE_PARTS = 32;
constexpr int PART_THREADS = 256;
constexpr int PART_PER_LANE = 16;                                     // a block takes up to 4096 entries
constexpr int PART_MAX_SLICE = PART_THREADS * PART_PER_LANE;
constexpr int PART_CAP = 96;                                          // entries a part may leave
constexpr int PART_MAX_K = 64;
constexpr int WAVE_CAP = 128;                                         // entries a wave may hand to its block

struct PartOut {          // what a part leaves, rows x SAMPLE_PARTS of each
  unsigned long long* best;  // largest key of the slice (BAD_ROW: a NaN or an infinity)
  double* z;                 // sum of exp((l - slice max) / T)
  int* count;                // entries left, or -1: more than PART_CAP rank with the k largest
  float* val;                // [PART_CAP]
  int* idx;                  // [PART_CAP]
};

__device__ inline PartOut part_out(unsigned char* scratch, int rows) {
  const long long n = (long long)rows * SAMPLE_PARTS;
  PartOut o;
  o.best = (unsigned long long*)scratch;
  o.z = (double*)(o.best + n);
  o.val = (float*)(o.z + n);
  o.idx = (int*)(o.val + n * PART_CAP);
  o.count = o.idx + n * PART_CAP;
  return o;
}
static long long part_scratch_bytes(int rows) {
  return (long long)rows * SAMPLE_PARTS * (8 + 8 + 4 + PART_CAP * 8);
}

// A value v with at least k and at most `cap` of a wave's ordered-bit values >= v (a lane's PER of them
// in registers); if no value cuts that finely (ties), the largest v with at least k values >= v, whatever
// their number; with fewer than k values: 0.  The k largest are among the values >= v either way.
template <int PER>
__device__ inline unsigned cut_for_k_largest(const unsigned (&bits)[PER], int k, int cap) {
  unsigned lo = 0u, hi = 0xffffffffu;  // count(>= lo) >= k holds for lo = 0 (if there are k at all)
  while (lo < hi) {
    const unsigned mid = lo + (hi - lo) / 2u + 1u;  // upper middle: lo < mid <= hi
    int c = 0;  // counted with ballots: no lane waits for another
#pragma unroll
    for (int j = 0; j < PER; ++j) c += __popcll(__ballot(bits[j] >= mid));
    if (c >= k) {
      lo = mid;
      if (c <= cap) break;
    } else {
      hi = mid - 1u;
    }
  }
  return lo;
}

__global__ __launch_bounds__(PART_THREADS) void sample_parts_kernel(const float* __restrict__ logits, int ld, int V,
                                                                    float invT, int top_k, unsigned char* scratch) {
  __shared__ float wv[PART_THREADS / 64][WAVE_CAP];
  __shared__ int wi[PART_THREADS / 64][WAVE_CAP];
  __shared__ int wn[PART_THREADS / 64];
  __shared__ unsigned long long wbest[PART_THREADS / 64];
  __shared__ double wz[PART_THREADS / 64];
  const int part = blockIdx.x, row = blockIdx.y, rows = gridDim.y;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const PartOut o = part_out(scratch, rows);
  const long long at = (long long)row * SAMPLE_PARTS + part;
  const int per = (V + SAMPLE_PARTS - 1) / SAMPLE_PARTS;
  const int i0 = part * per, i1 = min(V, i0 + per);
  const float* lr = logits + (long long)row * ld;
  // a wave takes 1024 consecutive entries, 64 at a time (entry j of lane l: 64 j + l), so that loads are
  // whole lines and (j, lane) order is index order
  float v[PART_PER_LANE];
  unsigned bits[PART_PER_LANE];
  unsigned long long best = 0ull;
  const int mine0 = i0 + wave * (64 * PART_PER_LANE) + lane;
#pragma unroll
  for (int j = 0; j < PART_PER_LANE; ++j) {
    const int i = mine0 + 64 * j;
    const bool has = i < i1;
    v[j] = has ? lr[i] : 0.f;
    bits[j] = has ? ordered_bits(v[j]) : 0u;  // (0 ranks below every number)
    if (has) {
      const unsigned long long k = checked_key_of(v[j], i);
      best = k > best ? k : best;
    }
  }
  for (int off = 32; off > 0; off >>= 1) {
    const unsigned long long ob = shfl_xor_u64(best, off);
    best = ob > best ? ob : best;
  }
  if (lane == 0) wbest[wave] = best;
  __syncthreads();
  best = wbest[0];
  for (int w = 1; w < PART_THREADS / 64; ++w) best = wbest[w] > best ? wbest[w] : best;
  if (best == BAD_ROW || i0 >= i1) {  // the same for every thread of the block
    if (tid == 0) {
      o.best[at] = i0 >= i1 ? 0ull : BAD_ROW;
      o.z[at] = 0.0;
      o.count[at] = 0;
    }
    return;
  }
  const float mx = from_ordered_bits((unsigned)(best >> 32));
  double z = 0.0;
#pragma unroll
  for (int j = 0; j < PART_PER_LANE; ++j)
    if (mine0 + 64 * j < i1) z += (double)expf((v[j] - mx) * invT);
  for (int off = 32; off > 0; off >>= 1) z += shfl_xor_f64(z, off);
  if (lane == 0) wz[wave] = z;
  // every wave: the entries that rank with its k largest values, to LDS in index order
  const unsigned cut = cut_for_k_largest<PART_PER_LANE>(bits, top_k, WAVE_CAP);
  const unsigned long long before = (1ull << lane) - 1ull;
  int total = 0;
  bool fits = true;
#pragma unroll
  for (int j = 0; j < PART_PER_LANE; ++j) {
    const bool take = mine0 + 64 * j < i1 && bits[j] >= cut;
    const unsigned long long m = __ballot(take);
    const int pos = total + __popcll(m & before);
    total += __popcll(m);
    fits = fits && total <= WAVE_CAP;
    if (take && fits) {
      wv[wave][pos] = v[j];
      wi[wave][pos] = mine0 + 64 * j;
    }
  }
  if (lane == 0) wn[wave] = fits ? total : -1;
  __syncthreads();
  // wave 0: the k largest values among what the four waves left, again with their ties
  if (wave != 0) return;
  double zsum = 0.0;
  bool over = false;
  int n_all = 0;
  for (int w = 0; w < PART_THREADS / 64; ++w) {
    zsum += wz[w];
    over = over || wn[w] < 0;
    n_all += max(wn[w], 0);
  }
  if (lane == 0) {
    o.best[at] = best;
    o.z[at] = zsum;
  }
  if (over) {
    if (lane == 0) o.count[at] = -1;
    return;
  }
  // the waves' lists one after the other are in index order; a lane takes a run of 8 of them
  constexpr int RUN = PART_THREADS / 64 * WAVE_CAP / 64;  // 8
  float cv[RUN];
  int ci[RUN];
  unsigned cb[RUN];
#pragma unroll
  for (int j = 0; j < RUN; ++j) {
    int q = lane * RUN + j;  // place in the concatenation
    int w = 0;
    while (w < PART_THREADS / 64 - 1 && q >= wn[w]) {
      q -= wn[w];
      ++w;
    }
    const bool has = lane * RUN + j < n_all;
    cv[j] = has ? wv[w][q] : 0.f;
    ci[j] = has ? wi[w][q] : -1;
    cb[j] = has ? ordered_bits(cv[j]) : 0u;
  }
  const unsigned cut2 = cut_for_k_largest<RUN>(cb, top_k, PART_CAP);
  int take2 = 0;
#pragma unroll
  for (int j = 0; j < RUN; ++j) take2 += (ci[j] >= 0 && cb[j] >= cut2) ? 1 : 0;
  int incl2 = take2;
  for (int off = 1; off < 64; off <<= 1) {
    const int up = __shfl_up(incl2, off, 64);
    if (lane >= off) incl2 += up;
  }
  const int total2 = __shfl(incl2, 63, 64);
  if (total2 <= PART_CAP) {
    int pos = incl2 - take2;
#pragma unroll
    for (int j = 0; j < RUN; ++j)
      if (ci[j] >= 0 && cb[j] >= cut2) {
        o.val[at * PART_CAP + pos] = cv[j];
        o.idx[at * PART_CAP + pos] = ci[j];
        ++pos;
      }
  }
  if (lane == 0) o.count[at] = total2 <= PART_CAP ? total2 : -1;
}

// One block a row: puts the parts together and draws.  Rows whose parts were flagged are left for the
// long way (redo[row] = 1), which the host launches over all rows right after: it skips the others.
__global__ __launch_bounds__(256) void sample_merge_kernel(SampleArgs a, const unsigned char* scratch, int* redo) {
  __shared__ float list_val[SAMPLE_PARTS * PART_CAP];
  __shared__ int list_idx[SAMPLE_PARTS * PART_CAP];
  __shared__ int offset[SAMPLE_PARTS + 1];
  __shared__ unsigned long long key_sh[4 * PART_MAX_K];
  __shared__ float e_sh[4 * PART_MAX_K];
  __shared__ unsigned long long best_sh;
  __shared__ double z_sh;
  __shared__ int floor_count;
  const int row = blockIdx.x, rows = gridDim.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const PartOut o = part_out(const_cast<unsigned char*>(scratch), rows);
  const long long at0 = (long long)row * SAMPLE_PARTS;
  const float invT = a.inv_temperature;
  if (wave == 0) {
    // the row's maximum, the flags, the places of the parts' lists
    unsigned long long best = lane < SAMPLE_PARTS ? o.best[at0 + lane] : 0ull;
    int cnt = lane < SAMPLE_PARTS ? o.count[at0 + lane] : 0;
    int flagged = cnt < 0 ? 1 : 0;
    for (int off = 32; off > 0; off >>= 1) {
      const unsigned long long ob = shfl_xor_u64(best, off);
      best = ob > best ? ob : best;
      flagged |= __shfl_xor(flagged, off, 64);
    }
    int incl = max(cnt, 0);
    for (int off = 1; off < 64; off <<= 1) {
      const int up = __shfl_up(incl, off, 64);
      if (lane >= off) incl += up;
    }
    if (lane < SAMPLE_PARTS) offset[lane + 1] = incl;
    if (lane == 0) offset[0] = 0;
    // Z = sum over the parts of z_p * exp((m_p - m) / T), in part order
    const float mx = from_ordered_bits((unsigned)(best >> 32));
    double term = 0.0;
    if (lane < SAMPLE_PARTS && best != BAD_ROW && o.best[at0 + lane] != 0ull) {
      const float mp = from_ordered_bits((unsigned)(o.best[at0 + lane] >> 32));
      term = o.z[at0 + lane] * exp(((double)mp - (double)mx) * (double)invT);
    }
    double zsum = 0.0;
    for (int p = 0; p < SAMPLE_PARTS; ++p) zsum += shfl_f64(term, p);
    if (lane == 0) {
      best_sh = flagged && best != BAD_ROW ? 1ull : best;  // 1: the long way
      z_sh = zsum;
      floor_count = 0;
    }
  }
  __syncthreads();
  const unsigned long long best = best_sh;
  if (best == BAD_ROW || best == 1ull) {
    if (tid == 0) {
      if (best == BAD_ROW) {
        a.out[row] = NO_TOKEN;
        if (a.kept_count) a.kept_count[row] = 0;
        if (a.kept_mass) a.kept_mass[row] = 0.0;
        redo[row] = 0;
      } else {
        redo[row] = 1;
      }
    }
    return;
  }
  const float mx = from_ordered_bits((unsigned)(best >> 32));
  const double Z = z_sh;
  const double e_floor = 1e-10 * Z;
  const bool use_p = a.top_p > 0.f && a.top_p < 1.f;
  const double p_mass = (double)a.top_p * Z;
  const int n_list = offset[SAMPLE_PARTS];
  int above = 0;
  // every thread asks for its entries of the list at once: which part an entry belongs to is looked up
  // in the parts' offsets (the loads of all parts are then in flight together)
  for (int j = tid; j < n_list; j += 256) {
    int p = 0;
#pragma unroll
    for (int step = SAMPLE_PARTS / 2; step > 0; step >>= 1)
      if (offset[p + step] <= j) p += step;
    const long long src = (at0 + p) * PART_CAP + (j - offset[p]);
    const float v = o.val[src];
    list_val[j] = v;
    list_idx[j] = o.idx[src];
    above += (double)expf((v - mx) * invT) > e_floor ? 1 : 0;
  }
  for (int off = 32; off > 0; off >>= 1) above += __shfl_xor(above, off, 64);
  if (lane == 0) atomicAdd(&floor_count, above);
  __syncthreads();
  if (wave != 0) return;
  // every candidate of the row (p > 1e-10) that ranks among the k largest is in the list; if the row has
  // fewer than k candidates, all of them are
  const long long k_limit = min((long long)a.top_k, (long long)floor_count);
  // the list is 32 times what is needed: keep what ranks with its k largest values (a coarse cut by
  // counting alone), in place and in order, and search that
  int n_short = n_list;
  {
    constexpr int PER = SAMPLE_PARTS * PART_CAP / 64;  // 48
    // entry j of lane l is 64 j + l: neighbouring lanes read neighbouring words, and (j, lane) order is
    // index order.  Everything is read before anything is written, and an entry moves to its own place or
    // one before it.
    float mv[PER];
    int mi[PER];
    unsigned lb[PER];
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const bool has = 64 * j + lane < n_list;
      mv[j] = has ? list_val[64 * j + lane] : 0.f;
      mi[j] = has ? list_idx[64 * j + lane] : -1;
      lb[j] = has ? ordered_bits(mv[j]) : 0u;
    }
    const unsigned cut = cut_for_k_largest<PER>(lb, a.top_k, 4 * PART_MAX_K);
    const unsigned long long before = (1ull << lane) - 1ull;
    int total = 0;
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const bool take = mi[j] >= 0 && lb[j] >= cut;
      const unsigned long long m = __ballot(take);
      if (take) {
        const int pos = total + __popcll(m & before);
        list_val[pos] = mv[j];
        list_idx[pos] = mi[j];
      }
      total += __popcll(m);
    }
    n_short = total;
  }
  const int slot = a.seq_slot[row];
  const unsigned long long ctr = (unsigned long long)a.rng_ctr[slot];
  const double u = uniform_of((unsigned long long)a.rng_key[slot], ctr);
  ListResult res;
  if (n_short <= 4 * PART_MAX_K)
    res = list_draw(list_val, list_idx, n_short,
                    list_threshold_by_ranks(list_val, list_idx, n_short, mx, invT, k_limit, e_floor, use_p, p_mass, key_sh, e_sh), mx,
                    invT, u);
  else  // (ties beyond what the coarse cut could separate)
    res = list_threshold_and_draw(list_val, list_idx, n_short, best, mx, invT, k_limit, e_floor, use_p, p_mass, u);
  if (lane == 0) {
    int tok = res.tok;
    if (tok < 0) tok = (int)(0xffffffffu - (unsigned)(best & 0xffffffffull));  // r fell on a rounding seam
    a.out[row] = tok;
    a.rng_ctr[slot] = (long long)(ctr + 1ull);
    if (a.recent) push_recent(a.recent, a.recent_n, slot, tok);
    if (a.kept_count) a.kept_count[row] = res.kept;
    if (a.kept_mass) a.kept_mass[row] = res.mass / Z;
    redo[row] = 0;
  }
}

// ------------------------------------------------------------------ state upkeep
__global__ void advance_kernel(int* row_pos, int* seq_start, int* seq_len, int batch) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < batch) {
    row_pos[i] += 1;
    seq_start[i] += 1;
    seq_len[i] += 1;
  }
}

}  // namespace

// Ids of a sequence's history that the repetition penalty looks at: the width of the ring that lq_apply_penalty,
// lq_argmax and lq_sample take (whoever allocates the ring asks here).
extern "C" int lq_penalty_window() { return RECENT; }

extern "C" int lq_apply_penalty(float* logits, int ld, int rows, int V, const int* seq_slot, const int* recent,
                                const int* recent_n, float penalty, hipStream_t stream) {
  LQ_REQUIRE(rows > 0 && V > 0 && ld >= V, "penalty: bad sizes");
  LQ_REQUIRE(penalty > 0.f, "penalty: factor %f must be positive", penalty);
  penalty_kernel<<<rows, RECENT, 0, stream>>>(logits, ld, V, seq_slot, recent, recent_n, penalty);
  LQ_CHECK_LAUNCH("penalty");
  return 0;
}

// `scratch`: rows * 32 64-bit words the two stages pass their partial results through
extern "C" int lq_argmax(const float* logits, int ld, int rows, int V, const int* seq_slot, int* out, int* recent,
                         int* recent_n, unsigned long long* scratch, hipStream_t stream) {
  LQ_REQUIRE(rows > 0 && V > 0 && ld >= V, "argmax: bad sizes");
  LQ_REQUIRE(rows <= 65535, "argmax: %d rows are too many for one launch", rows);
  LQ_REQUIRE(scratch != nullptr, "argmax: scratch of rows * %d 64-bit words is needed", ARGMAX_PARTS);
  LQ_REQUIRE(recent == nullptr || (recent_n != nullptr && seq_slot != nullptr), "argmax: ring without its counters");
  argmax_part_kernel<<<dim3(ARGMAX_PARTS, rows), 256, 0, stream>>>(logits, ld, V, scratch);
  argmax_final_kernel<<<rows, 64, 0, stream>>>(scratch, seq_slot, out, recent, recent_n);
  LQ_CHECK_LAUNCH("argmax");
  return 0;
}

// ---- arg-max for callers that cannot allocate (lq_no_alloc.h) ----
// The stages' scratch: a fixed array in device memory, a copy on every GPU, each at its own address.
// `scratch` itself is a host-side stand-in and no device address: the pointer that kernels and other
// HIP calls take comes from hipGetSymbolAddress, asked once per device and kept.
static __device__ __align__(256) unsigned long long scratch[LQ_ARGMAX_NO_ALLOC_MAX_ROWS * ARGMAX_PARTS];

constexpr int MAX_DEVICES = 64;
static unsigned long long* scratch_on_device[MAX_DEVICES];  // null until the first call on that device
static std::mutex scratch_lock;

// the current device's copy of `scratch`
static int scratch_pointer(unsigned long long** ptr) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  LQ_REQUIRE(e == hipSuccess, "argmax_no_alloc: no current device: %s", hipGetErrorString(e));
  LQ_REQUIRE(dev >= 0 && dev < MAX_DEVICES, "argmax_no_alloc: device %d is beyond the %d this library keeps scratch for",
             dev, MAX_DEVICES);
  std::lock_guard<std::mutex> hold(scratch_lock);
  if (scratch_on_device[dev] == nullptr) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    LQ_REQUIRE(e == hipSuccess && p != nullptr, "argmax_no_alloc: the scratch array has no address on device %d: %s", dev,
               hipGetErrorString(e));
    scratch_on_device[dev] = (unsigned long long*)p;
  }
  *ptr = scratch_on_device[dev];
  return 0;
}

extern "C" int lq_argmax_no_alloc(const float* logits, int ld, int rows, int V, int* out, hipStream_t stream) {
  LQ_REQUIRE(rows > 0 && V > 0 && ld >= V, "argmax_no_alloc: bad sizes");
  LQ_REQUIRE(rows <= LQ_ARGMAX_NO_ALLOC_MAX_ROWS,
             "argmax_no_alloc: %d rows are more than the %d that the fixed scratch array holds (use lq_argmax with a "
             "scratch buffer of your own)", rows, LQ_ARGMAX_NO_ALLOC_MAX_ROWS);
  LQ_REQUIRE(logits != nullptr && out != nullptr, "argmax_no_alloc: null pointer");
  unsigned long long* part = nullptr;
  if (scratch_pointer(&part) != 0) return -1;
  argmax_part_kernel<<<dim3(ARGMAX_PARTS, rows), 256, 0, stream>>>(logits, ld, V, part);
  argmax_final_kernel<<<rows, 64, 0, stream>>>(part, nullptr, out, nullptr, nullptr);
  LQ_CHECK_LAUNCH("argmax_no_alloc");
  return 0;
}

// Bytes of scratch with which lq_sample takes the short way for `rows` rows (top_k in 1..64 and a
// vocabulary of 8 192 to 131 072 entries); without it, or outside these sizes, it goes the long way.
extern "C" long long lq_sample_scratch_bytes(int rows) { return part_scratch_bytes(rows) + (long long)rows * 4; }

extern "C" int lq_sample(const float* logits, int ld, int rows, int V, const int* seq_slot, float temperature,
                         int top_k, float top_p, long long* rng_key, long long* rng_ctr, int* recent,
                         int* recent_n, int* out, int* kept_count, double* kept_mass, void* scratch,
                         long long scratch_bytes, hipStream_t stream) {
  LQ_REQUIRE(rows > 0 && V > 0 && ld >= V, "sample: bad sizes");
  LQ_REQUIRE(temperature > 0.f, "sample: temperature %f must be positive (0 is the greedy kernel)", temperature);
  LQ_REQUIRE(seq_slot && rng_key && rng_ctr && out, "sample: null pointer");
  LQ_REQUIRE(rows <= 65535, "sample: %d rows are too many for one launch", rows);
  SampleArgs a;
  a.logits = logits;
  a.ld = ld;
  a.V = V;
  a.seq_slot = seq_slot;
  a.inv_temperature = 1.0f / temperature;
  a.top_k = top_k;
  a.top_p = top_p;
  a.rng_key = rng_key;
  a.rng_ctr = rng_ctr;
  a.recent = recent;
  a.recent_n = recent_n;
  a.out = out;
  a.kept_count = kept_count;
  a.kept_mass = kept_mass;
  const bool parts = scratch != nullptr && scratch_bytes >= lq_sample_scratch_bytes(rows) && top_k >= 1 &&
                     top_k <= PART_MAX_K && V >= 8192 && V <= SAMPLE_PARTS * PART_MAX_SLICE &&
                     ((uintptr_t)scratch % 8) == 0;
  if (!parts) {
    sample_kernel<<<rows, THREADS, 0, stream>>>(a, nullptr);
    LQ_CHECK_LAUNCH("sample");
    return 0;
  }
  int* redo = (int*)((unsigned char*)scratch + part_scratch_bytes(rows));
  sample_parts_kernel<<<dim3(SAMPLE_PARTS, rows), PART_THREADS, 0, stream>>>(logits, ld, V, a.inv_temperature, top_k,
                                                                            (unsigned char*)scratch);
  sample_merge_kernel<<<rows, 256, 0, stream>>>(a, (const unsigned char*)scratch, redo);
  // rows with more ties at a slice's k-th value than a part can hold (redo = 1): the long way, the others
  // leave at once
  sample_kernel<<<rows, THREADS, 0, stream>>>(a, redo);
  LQ_CHECK_LAUNCH("sample");
  return 0;
}

// row_pos, seq_start and seq_len of a decoding batch move on by one (keeps a captured step replayable)
extern "C" int lq_advance(int* row_pos, int* seq_start, int* seq_len, int batch, hipStream_t stream) {
  LQ_REQUIRE(batch > 0, "advance: batch %d must be positive", batch);
  advance_kernel<<<lq_ceil_div(batch, 256), 256, 0, stream>>>(row_pos, seq_start, seq_len, batch);
  LQ_CHECK_LAUNCH("advance");
  return 0;
}
