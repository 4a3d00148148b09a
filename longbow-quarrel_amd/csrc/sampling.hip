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
// with block-wide counts and masses.  And the running sum of the draw walks the kept candidates
// in index order, not in order of probability: the law of the drawn token is the same, which
// token a given random number picks is not.
// Sums are double with a fixed tree, so a sequence's draw does not depend on the batch.
//
// Per-sequence sampler state lives in device arrays indexed by slot: a 64-bit key and counter for
// the random numbers (counter-based: draw n of a sequence depends on key and n only) and a ring
// of the last 64 token ids.
#include "common.h"

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
  for (int i = slice * per + threadIdx.x; i < i1; i += 256) {
    const unsigned long long k = key_of(lr[i], i);
    best = k > best ? k : best;
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

// One pass over the row: how many keys are >= theta, their mass (if wanted) and the smallest of them.
struct PassResult {
  long long count;
  double mass;
  unsigned long long kmin;
};

__device__ inline PassResult pass_over(const float* lr, int V, unsigned long long theta, float mx, float invT,
                                       bool want_mass, unsigned long long* smu, double* smd) {
  long long cnt = 0;
  double mass = 0.0;
  unsigned long long kmin = ~0ull;
  for (int i = threadIdx.x; i < V; i += THREADS) {
    const float v = lr[i];
    const unsigned long long k = key_of(v, i);
    if (k >= theta) {
      ++cnt;
      if (want_mass) mass += (double)expf((v - mx) * invT);
      kmin = k < kmin ? k : kmin;
    }
  }
  PassResult r;
  r.count = block_sum_i64(cnt, smu);
  r.mass = want_mass ? block_sum_f64(mass, smd) : 0.0;
  r.kmin = block_min_u64(kmin, smu);
  return r;
}

__global__ __launch_bounds__(THREADS) void sample_kernel(SampleArgs a) {
  __shared__ unsigned long long smu[THREADS / 64];
  __shared__ double smd[THREADS / 64];
  __shared__ double scan[THREADS];
  __shared__ int winner;
  const int row = blockIdx.x, tid = threadIdx.x;
  const float* lr = a.logits + (long long)row * a.ld;
  const int V = a.V;
  const float invT = a.inv_temperature;

  // maximum logit (as a key: also gives the arg-max)
  unsigned long long best = 0ull;
  for (int i = tid; i < V; i += THREADS) {
    const unsigned long long k = key_of(lr[i], i);
    best = k > best ? k : best;
  }
  best = block_max_u64(best, smu);
  const float mx = from_ordered_bits((unsigned)(best >> 32));

  // e_i = exp((l_i - max) / T) in 32-bit, sums in double; Z = sum e_i; candidates need p > 1e-10
  double zloc = 0.0;
  for (int i = tid; i < V; i += THREADS) zloc += (double)expf((lr[i] - mx) * invT);
  const double Z = block_sum_f64(zloc, smd);
  const double e_floor = 1e-10 * Z;
  long long ncand_loc = 0;
  for (int i = tid; i < V; i += THREADS)
    if ((double)expf((lr[i] - mx) * invT) > e_floor) ++ncand_loc;
  const long long ncand = block_sum_i64(ncand_loc, smu);
  const long long k_limit = (a.top_k > 0 && a.top_k < ncand) ? a.top_k : ncand;
  const bool use_p = a.top_p > 0.f && a.top_p < 1.f;
  const double p_mass = (double)a.top_p * Z;

  // The kept set is the longest allowed prefix of the descending order: at most k_limit members,
  // all above the floor, and without its last member not yet at the top_p mass.  As a set it is
  // {key >= theta}; allowed() is monotone in theta, so theta is found by bisection: first on the
  // logit bits (whole groups of equal logits), then, only if the group below the boundary has
  // several members, on the index bits inside that group.
  auto allowed = [&](unsigned long long theta) -> bool {
    const PassResult r = pass_over(lr, V, theta, mx, invT, use_p, smu, smd);
    if (r.count == 0) return true;
    const double e_min = (double)expf((from_ordered_bits((unsigned)(r.kmin >> 32)) - mx) * invT);
    return r.count <= k_limit && e_min > e_floor && (!use_p || r.mass - e_min < p_mass);
  };
  unsigned long long theta;
  if (!use_p && k_limit == (long long)V) {
    theta = 0ull;  // everything is kept
  } else {
    unsigned long long lo = 0ull, hi = best >> 32;  // allowed(hi << 32): the arg-max's group... checked below
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
    theta = lo << 32;  // may be 2^32 << 32 = overflow only if best>>32 == 0xffffffff, i.e. +NaN: excluded
    if (lo > 0ull) {
      // the next group below the boundary: largest logit bits < lo
      unsigned long long below = 0ull;
      bool any = false;
      {
        unsigned long long loc = 0ull;
        for (int i = tid; i < V; i += THREADS) {
          const unsigned long long hk = (unsigned long long)ordered_bits(lr[i]);
          if (hk < lo && hk + 1ull > loc) loc = hk + 1ull;  // store hk + 1 so that 0 means none
        }
        loc = block_max_u64(loc, smu);
        any = loc > 0ull;
        below = loc - 1ull;
      }
      if (any) {
        const PassResult grp = pass_over(lr, V, below << 32, mx, invT, false, smu, smd);
        const PassResult above = pass_over(lr, V, lo << 32, mx, invT, false, smu, smd);
        if (grp.count - above.count > 1) {
          // several equal logits: admit them one by one in index order while allowed
          unsigned long long l2 = below << 32, h2 = lo << 32;  // allowed(h2) holds, allowed(l2) does not
          // find the smallest allowed theta in (l2, h2]
          unsigned long long a2 = l2 + 1ull, b2 = h2;
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
  }

  // the draw: running sum over the kept candidates in index order
  const int chunk = (V + THREADS - 1) / THREADS;
  const int i0 = tid * chunk, i1 = min(V, i0 + chunk);
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

  const int slot = a.seq_slot[row];
  const unsigned long long ctr = (unsigned long long)a.rng_ctr[slot];
  const double u = uniform_of((unsigned long long)a.rng_key[slot], ctr);
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
    int tok = winner;
    if (tok < 0) tok = (int)(0xffffffffu - (unsigned)(best & 0xffffffffull));  // r fell on a rounding seam
    a.out[row] = tok;
    a.rng_ctr[slot] = (long long)(ctr + 1ull);
    if (a.recent) push_recent(a.recent, a.recent_n, slot, tok);
    if (a.kept_count) a.kept_count[row] = (int)kept;
    if (a.kept_mass) a.kept_mass[row] = total / Z;
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

extern "C" int lq_sample(const float* logits, int ld, int rows, int V, const int* seq_slot, float temperature,
                         int top_k, float top_p, long long* rng_key, long long* rng_ctr, int* recent,
                         int* recent_n, int* out, int* kept_count, double* kept_mass, hipStream_t stream) {
  LQ_REQUIRE(rows > 0 && V > 0 && ld >= V, "sample: bad sizes");
  LQ_REQUIRE(temperature > 0.f, "sample: temperature %f must be positive (0 is the greedy kernel)", temperature);
  LQ_REQUIRE(seq_slot && rng_key && rng_ctr && out, "sample: null pointer");
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
  sample_kernel<<<rows, THREADS, 0, stream>>>(a);
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
