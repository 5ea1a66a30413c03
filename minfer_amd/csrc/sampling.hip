// Sampling on the device, one block per row of float32 logits [rows][ld], vocab <= ld.
// Semantics follow src/sampler.rs of yusiwen/minfer:
//   greedy: first maximum under strict '>' (:16-26)
//   penalties over the recent-token window (:44-76)
//   top-k: entries below the k-th largest value -> -inf, ties at the threshold stay (:125-137)
//   top-p: softmax over finite entries, descending stable order, shortest prefix whose
//          cumulative probability exceeds p is kept (:149-196)
//   temperature: l/temp, exp(l - max), sum, walk indices upward until the running sum
//          reaches the uniform draw r in [0,1) (:224-267)
// The uniform comes from a counter-based generator keyed (seed, sequence key, step), so a
// sequence's draws do not depend on what else is in the batch.  Sums run in double in a
// fixed order (top-p's per-bin masses excepted, which only matter within rounding of p).
#include "common.h"

// No fused multiply-add in this file: a probability is exp(l * (1/temp) - max) * (1/sum) with one
// rounding per operation wherever it is formed, so that the whole-row kernels, the fused ones and
// a plain host implementation arrive at the same numbers (left to itself the compiler fuses the
// multiply into the subtraction in some places and not in others).
#pragma clang fp contract(off)

namespace {

constexpr int NT = 1024;

__device__ __forceinline__ uint64_t mix64(uint64_t z) {
  z += 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

// uniform in [0,1) with 24 bits; mirrored by minfer_amd.sampling.rng.uniform.  `stream` is the
// host's mix64(seed ^ mix64(key)) of a sequence (minfer_amd.sampling.rng.stream): the seed reaches
// the kernels as data, so a captured step serves every seed.
__device__ __forceinline__ float uniform01(uint64_t stream, uint64_t step) {
  const uint64_t h = mix64(stream ^ step);
  return (float)(uint32_t)(h >> 40) * (1.0f / 16777216.0f);
}

// the one way a probability is formed
__device__ __forceinline__ float scaled(float x, float s) { return x * s; }
__device__ __forceinline__ float exp_rel(float l, float mx) { return expf(l - mx); }
__device__ __forceinline__ float prob_of(float l, float mx, float inv) { return exp_rel(l, mx) * inv; }
__device__ __forceinline__ float share_of(float l, float mx, float tot) { return exp_rel(l, mx) / tot; }

// f(i, row[i]) for i in [lo, hi) in index order, until f returns false.  A thread's run of
// consecutive entries is read 16 bytes at a time where the row allows: the lanes of such a load
// sit in 64 different cache lines, each a look-up of its own in the CU's cache, so four entries a
// look-up instead of one.
template <typename F>
__device__ __forceinline__ void for_run(const float* __restrict__ row, int lo, int hi, F f) {
  int i = lo;
  if ((reinterpret_cast<uintptr_t>(row + lo) & 15) == 0) {
    for (; i + 3 < hi; i += 4) {
      const float4 v = *reinterpret_cast<const float4*>(row + i);
      if (!f(i, v.x) || !f(i + 1, v.y) || !f(i + 2, v.z) || !f(i + 3, v.w)) return;
    }
  }
  for (; i < hi; ++i)
    if (!f(i, row[i])) return;
}

// entries per thread when a row is cut into runs: a multiple of 4, for the 16-byte reads
__device__ __forceinline__ int run_length(int vocab) { return (((vocab + NT - 1) / NT) + 3) & ~3; }

__device__ __forceinline__ double wave_sum_d(double v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, MF_WAVE);
  return v;
}

__device__ __forceinline__ double block_sum_d(double v, double* scratch) {
  v = wave_sum_d(v);
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  __syncthreads();
  if (lane == 0) scratch[w] = v;
  __syncthreads();
  double t = 0.0;
  for (int i = 0; i < NT / 64; ++i) t += scratch[i];
  return t;
}

// (value, index) of the first maximum of a row; every thread gets it.
__device__ __forceinline__ void block_argmax(const float* __restrict__ row, int vocab, float scale,
                                             float* s_val, int* s_idx, float& best_v, int& best_i) {
  float bv = -INFINITY;
  int bi = 0x7fffffff;
  for (int i = threadIdx.x; i < vocab; i += NT) {
    const float v = scaled(row[i], scale);
    if (v > bv || (v == bv && i < bi)) { bv = v; bi = i; }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_xor(bv, o, MF_WAVE);
    const int oi = __shfl_xor(bi, o, MF_WAVE);
    if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
  }
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  __syncthreads();
  if (lane == 0) { s_val[w] = bv; s_idx[w] = bi; }
  __syncthreads();
  bv = s_val[0];
  bi = s_idx[0];
  for (int i = 1; i < NT / 64; ++i)
    if (s_val[i] > bv || (s_val[i] == bv && s_idx[i] < bi)) { bv = s_val[i]; bi = s_idx[i]; }
  best_v = bv;
  best_i = (bi == 0x7fffffff) ? 0 : bi;   // a row of NaN or -inf: index 0, as the reference
}

__global__ __launch_bounds__(NT) void argmax_kernel(const float* __restrict__ logits, int ld, int vocab,
                                                    int* __restrict__ out, float* __restrict__ out_val) {
  __shared__ float s_val[NT / 64];
  __shared__ int s_idx[NT / 64];
  float bv;
  int bi;
  block_argmax(logits + (size_t)blockIdx.x * ld, vocab, 1.0f, s_val, s_idx, bv, bi);
  if (threadIdx.x == 0) {
    out[blockIdx.x] = bi;
    if (out_val) out_val[blockIdx.x] = bv;
  }
}

// Greedy over a large vocabulary with few rows: a row is cut into `chunks` pieces, one block
// each, and a second pass picks among the pieces (still the first maximum).
__global__ __launch_bounds__(NT) void argmax_part_kernel(const float* __restrict__ logits, int ld, int vocab,
                                                         int chunks, float* __restrict__ pval,
                                                         int* __restrict__ pidx) {
  __shared__ float s_val[NT / 64];
  __shared__ int s_idx[NT / 64];
  const int per = (vocab + chunks - 1) / chunks;
  const int lo = blockIdx.y * per, n = min(per, vocab - lo);
  float bv = -INFINITY;
  int bi = 0;
  if (n > 0) {
    block_argmax(logits + (size_t)blockIdx.x * ld + lo, n, 1.0f, s_val, s_idx, bv, bi);
    bi += lo;
  }
  if (threadIdx.x == 0) {
    pval[blockIdx.x * chunks + blockIdx.y] = n > 0 ? bv : -INFINITY;
    pidx[blockIdx.x * chunks + blockIdx.y] = bi;
  }
}

__global__ __launch_bounds__(64) void argmax_final_kernel(const float* __restrict__ pval,
                                                          const int* __restrict__ pidx, int chunks,
                                                          int* __restrict__ out) {
  float bv = -INFINITY;
  int bi = 0x7fffffff;
  for (int c = threadIdx.x; c < chunks; c += 64) {
    const float v = pval[blockIdx.x * chunks + c];
    const int i = pidx[blockIdx.x * chunks + c];
    if (v > bv || (v == bv && i < bi)) { bv = v; bi = i; }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_xor(bv, o, MF_WAVE);
    const int oi = __shfl_xor(bi, o, MF_WAVE);
    if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
  }
  if (threadIdx.x == 0) out[blockIdx.x] = (bi == 0x7fffffff) ? 0 : bi;
}

// temperature draw; temp < 1e-6 falls back to greedy (src/sampler.rs:225-227)
__device__ __forceinline__ void sample_row(const float* __restrict__ row, int rowi, int vocab, float temp,
                                           const long long* __restrict__ streams,
                                           const int* __restrict__ steps, const float* __restrict__ forced_r,
                                           int* __restrict__ out) {
  __shared__ float s_val[NT / 64];
  __shared__ int s_idx[NT / 64];
  __shared__ double s_d[NT / 64];
  __shared__ double s_wave_tot[NT / 64];
  __shared__ int s_found;
  float mx;
  int amax;
  const bool greedy = temp < 1e-6f;
  const float inv_t = greedy ? 1.0f : 1.0f / temp;
  block_argmax(row, vocab, inv_t, s_val, s_idx, mx, amax);
  if (greedy) {
    if (threadIdx.x == 0) out[rowi] = amax;
    return;
  }
  // contiguous chunk per thread so that the walk is in index order
  const int chunk = run_length(vocab);
  const int lo = min(vocab, (int)threadIdx.x * chunk), hi = min(vocab, lo + chunk);
  double mine = 0.0;
  for_run(row, lo, hi, [&](int, float x) {
    const float l = scaled(x, inv_t);
    if (l > -INFINITY) mine += (double)exp_rel(l, mx);
    return true;
  });
  const double total = block_sum_d(mine, s_d);
  const float inv = (float)(1.0 / total);
  // probabilities as the reference forms them: e * (1/sum as f32)
  double pm = 0.0;
  for_run(row, lo, hi, [&](int, float x) {
    const float l = scaled(x, inv_t);
    if (l > -INFINITY) pm += (double)prob_of(l, mx, inv);
    return true;
  });
  // exclusive scan of pm over threads: within the wave, then over wave totals
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  double incl = pm;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const double up = __shfl_up(incl, o, MF_WAVE);
    if (lane >= o) incl += up;
  }
  if (threadIdx.x == 0) s_found = vocab - 1;    // fallback: the last index (src/sampler.rs:266)
  __syncthreads();
  if (lane == 63) s_wave_tot[w] = incl;
  __syncthreads();
  double before = 0.0;
  for (int i = 0; i < w; ++i) before += s_wave_tot[i];
  const double prefix = before + incl - pm;
  float r = forced_r ? forced_r[rowi]
                     : uniform01((uint64_t)streams[rowi], (uint64_t)(uint32_t)steps[rowi]);
  const double rr = fmax((double)r, 1e-30);
  if (pm > 0.0 && prefix < rr && rr <= prefix + pm) {
    double cum = prefix;
    int pick = -1;
    for_run(row, lo, hi, [&](int i, float x) {
      const float l = scaled(x, inv_t);
      if (!(l > -INFINITY)) return true;
      const float p = prob_of(l, mx, inv);
      if (p <= 0.f) return true;
      cum += (double)p;
      pick = i;
      return !(rr <= cum);
    });
    if (pick >= 0) s_found = pick;
  }
  __syncthreads();
  if (threadIdx.x == 0) out[rowi] = s_found;
}

__global__ __launch_bounds__(NT) void sample_kernel(const float* __restrict__ logits, int ld, int vocab,
                                                    float temp,
                                                    const long long* __restrict__ streams,
                                                    const int* __restrict__ steps,
                                                    const float* __restrict__ forced_r,
                                                    int* __restrict__ out) {
  sample_row(logits + (size_t)blockIdx.x * ld, blockIdx.x, vocab, temp, streams, steps, forced_r, out);
}

// penalties in place; prev is [rows][max_prev], n_prev[row] entries are used
__global__ __launch_bounds__(64) void penalties_kernel(float* __restrict__ logits, int ld, int vocab,
                                                       const int* __restrict__ prev, int max_prev,
                                                       const int* __restrict__ n_prev, float repeat,
                                                       float frequency, float presence) {
  const int rowi = blockIdx.x;
  float* row = logits + (size_t)rowi * ld;
  const int* pv = prev + (size_t)rowi * max_prev;
  const int n = min(n_prev[rowi], max_prev);
  for (int i = threadIdx.x; i < n; i += 64) {
    const int tok = pv[i];
    if (tok < 0 || tok >= vocab) continue;
    int count = 0;
    bool first = true;
    for (int j = 0; j < n; ++j) {
      if (pv[j] == tok) {
        ++count;
        if (j < i) first = false;
      }
    }
    if (!first) continue;
    float v = row[tok];
    if (fabsf(frequency) >= 1e-6f || fabsf(presence) >= 1e-6f) {
      v -= (float)count * frequency;
      v -= presence;
    }
    if (fabsf(repeat - 1.0f) >= 1e-6f && repeat >= 1.0f) v = (v <= 0.f) ? v * repeat : v / repeat;
    row[tok] = v;
  }
}

// monotone map float -> uint32 (larger float, larger key); NaN sorts above +inf
__device__ __forceinline__ uint32_t order_key(float f) {
  const uint32_t u = __float_as_uint(f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

__device__ __forceinline__ float key_value(uint32_t key) {      // the float that order_key maps to `key`
  return __uint_as_float((key & 0x80000000u) ? (key ^ 0x80000000u) : ~key);
}

// top-k by radix select of the k-th largest key, 8 bits a pass
__device__ __forceinline__ void top_k_row(float* __restrict__ row, int vocab, int k) {
  __shared__ unsigned int hist[256];
  __shared__ uint32_t s_prefix;
  __shared__ int s_remaining;
  if (k <= 0 || k >= vocab) return;
  if (threadIdx.x == 0) { s_prefix = 0; s_remaining = k; }
  for (int pass = 0; pass < 4; ++pass) {
    const int shift = 24 - 8 * pass;
    for (int i = threadIdx.x; i < 256; i += NT) hist[i] = 0;
    __syncthreads();
    const uint32_t prefix = s_prefix;
    const uint32_t mask = pass == 0 ? 0u : (0xFFFFFFFFu << (shift + 8));
    for (int i = threadIdx.x; i < vocab; i += NT) {
      const uint32_t key = order_key(row[i]);
      if ((key & mask) == prefix) atomicAdd(&hist[(key >> shift) & 255u], 1u);
    }
    __syncthreads();
    if (threadIdx.x == 0) {
      int remaining = s_remaining;
      int b = 255;
      for (; b > 0; --b) {
        if ((int)hist[b] >= remaining) break;
        remaining -= (int)hist[b];
      }
      s_prefix = prefix | ((uint32_t)b << shift);
      s_remaining = remaining;
    }
    __syncthreads();
  }
  const uint32_t thr = s_prefix;    // key of the k-th largest value
  for (int i = threadIdx.x; i < vocab; i += NT)
    if (order_key(row[i]) < thr) row[i] = -INFINITY;
  __syncthreads();      // what follows in the same block reads the row
}

__global__ __launch_bounds__(NT) void top_k_kernel(float* __restrict__ logits, int ld, int vocab, int k) {
  top_k_row(logits + (size_t)blockIdx.x * ld, vocab, k);
}

// top-p.  Probabilities p_i = exp(l_i - max) / sum over finite entries.  The kept set is
// {p_i > tau} plus the first c entries (in index order) with p_i == tau, where tau is the
// probability at which the descending cumulative mass first exceeds p.  tau is found by
// radix select over the probabilities' bit patterns, accumulating mass per bin in double.
__device__ __forceinline__ void top_p_row(float* __restrict__ row, int vocab, float p) {
  __shared__ float s_val[NT / 64];
  __shared__ int s_idx[NT / 64];
  __shared__ double s_d[NT / 64];
  __shared__ double bin_mass[256];
  __shared__ unsigned int bin_count[256];
  __shared__ uint32_t s_prefix;
  __shared__ double s_above;
  __shared__ unsigned int s_ties;
  __shared__ unsigned int s_wave_cnt[NT / 64];
  if (!(p > 0.f && p < 1.f)) return;
  float mx;
  int amax;
  block_argmax(row, vocab, 1.0f, s_val, s_idx, mx, amax);
  if (!(mx > -INFINITY)) return;
  const int chunk = run_length(vocab);
  const int lo = min(vocab, (int)threadIdx.x * chunk), hi = min(vocab, lo + chunk);
  double mine = 0.0;
  for_run(row, lo, hi, [&](int, float x) {
    if (x > -INFINITY) mine += exp((double)(x - mx));
    return true;
  });
  const double total = block_sum_d(mine, s_d);
  const float tot_f = (float)total;
  if (threadIdx.x == 0) { s_prefix = 0; s_above = 0.0; }
  for (int pass = 0; pass < 4; ++pass) {
    const int shift = 24 - 8 * pass;
    for (int i = threadIdx.x; i < 256; i += NT) { bin_mass[i] = 0.0; bin_count[i] = 0; }
    __syncthreads();
    const uint32_t prefix = s_prefix;
    const uint32_t mask = pass == 0 ? 0u : (0xFFFFFFFFu << (shift + 8));
    for_run(row, lo, hi, [&](int, float x) {
      if (!(x > -INFINITY)) return true;
      const float pr = share_of(x, mx, tot_f);
      const uint32_t key = __float_as_uint(pr);        // pr >= 0: bit order is value order
      if ((key & mask) == prefix) {
        atomicAdd(&bin_mass[(key >> shift) & 255u], (double)pr);
        atomicAdd(&bin_count[(key >> shift) & 255u], 1u);
      }
      return true;
    });
    __syncthreads();
    if (threadIdx.x == 0) {
      double above = s_above;
      int b = 255;
      for (; b > 0; --b) {
        if (bin_count[b] && above + bin_mass[b] > (double)p) break;
        above += bin_mass[b];
      }
      s_prefix = prefix | ((uint32_t)b << shift);
      s_above = above;
      s_ties = bin_count[b];
    }
    __syncthreads();
  }
  const uint32_t tau_key = s_prefix;
  const double tau = (double)__uint_as_float(tau_key);
  const unsigned int n_ties = s_ties;
  unsigned int keep_ties = n_ties;
  if (tau > 0.0) {
    const double need = ((double)p - s_above) / tau;     // ties needed so that mass exceeds p
    const double c = floor(need) + 1.0;
    keep_ties = c < 1.0 ? 1u : (c > (double)n_ties ? n_ties : (unsigned int)c);
  }
  // rank of each tie in index order: count per thread chunk, exclusive scan
  unsigned int my_ties = 0;
  for_run(row, lo, hi, [&](int, float x) {
    if (x > -INFINITY && __float_as_uint(share_of(x, mx, tot_f)) == tau_key) ++my_ties;
    return true;
  });
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  unsigned int incl = my_ties;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const unsigned int up = __shfl_up(incl, o, MF_WAVE);
    if (lane >= o) incl += up;
  }
  __syncthreads();
  if (lane == 63) s_wave_cnt[w] = incl;
  __syncthreads();
  unsigned int rank = incl - my_ties;
  for (int i = 0; i < w; ++i) rank += s_wave_cnt[i];
  for_run(row, lo, hi, [&](int i, float x) {
    if (!(x > -INFINITY)) return true;
    const uint32_t key = __float_as_uint(share_of(x, mx, tot_f));
    if (key > tau_key) return true;
    if (key == tau_key && rank++ < keep_ties) return true;
    row[i] = -INFINITY;
    return true;
  });
  __syncthreads();      // what follows in the same block reads the row
}

__global__ __launch_bounds__(NT) void top_p_kernel(float* __restrict__ logits, int ld, int vocab,
                                                   float p) {
  top_p_row(logits + (size_t)blockIdx.x * ld, vocab, p);
}

// ---------------------------------------------------------------- top-k, top-p and the draw in one
// With a small k the three steps above need the row only once.  A first kernel cuts the row
// into CAND_CHUNKS pieces, one block each, and lists each piece's k largest entries and every
// further entry equal to the k-th (largest first, equal values in index order): the row's k
// largest and their ties are among them.  A second kernel, one block per row, merges the lists
// into the row's survivors (the k largest and the ties of the k-th), and then does on these few
// what top_p_row and sample_row do on the whole row, with the same arithmetic in the same order
// (probabilities as float, sums in double in index order).  The logits are not changed.  A piece
// or a row with more ties than a list holds (a constant row, say) takes the kernels above
// instead, inside the second kernel, which then does change the row.
constexpr int CAND_CHUNKS = 32;      // pieces of a row
constexpr int CAND_CAP = 64;         // entries of a piece's list
constexpr int CAND_EPT = 32;         // entries per thread of a piece: vocab <= 32 * 256 * 32
constexpr int FAST_K_MAX = 48;       // the largest k that takes this path
constexpr int SURV_CAP = 128;        // survivors of a row

__global__ __launch_bounds__(256) void topk_candidates_kernel(const float* __restrict__ logits, int ld,
                                                              int vocab, int k, float* __restrict__ cand_val,
                                                              int* __restrict__ cand_idx,
                                                              int* __restrict__ cand_n) {
  __shared__ uint32_t s_key[2][4];
  __shared__ int s_idx[2][4];
  __shared__ float l_val[CAND_CAP];
  __shared__ int l_idx[CAND_CAP];
  const int rowi = blockIdx.y, chunk = blockIdx.x;
  const float* row = logits + (size_t)rowi * ld;
  const int per = (vocab + CAND_CHUNKS - 1) / CAND_CHUNKS;
  const int lo = chunk * per, n = max(0, min(per, vocab - lo));
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  // this thread's entries: lo + j * 256 + tid, as keys; 0 marks one that is out of play (no entry
  // above -inf has a key that small, and those at or below -inf are never listed)
  uint32_t key[CAND_EPT];
#pragma unroll
  for (int j = 0; j < CAND_EPT; ++j) {
    const int i = j * 256 + (int)threadIdx.x;
    key[j] = i < n ? order_key(row[lo + i]) : 0u;
  }
  int count = 0, over = 0;
  uint32_t kth = 0;
  for (int it = 0;; ++it) {
    // the largest entry of the block that is still in play, the lowest index among equals
    uint32_t bk = 0;
    int bj = 0;
#pragma unroll
    for (int j = 0; j < CAND_EPT; ++j)
      if (key[j] > bk) { bk = key[j]; bj = j; }
    const int bi = bj * 256 + (int)threadIdx.x;
    uint32_t rk = bk;
    int ri = bi;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const uint32_t ok = __shfl_xor(rk, o, MF_WAVE);
      const int oi = __shfl_xor(ri, o, MF_WAVE);
      if (ok > rk || (ok == rk && oi < ri)) { rk = ok; ri = oi; }
    }
    const int b = it & 1;
    if (lane == 0) { s_key[b][w] = rk; s_idx[b][w] = ri; }
    __syncthreads();
    uint32_t gk = s_key[b][0];
    int gi = s_idx[b][0];
#pragma unroll
    for (int ww = 1; ww < 4; ++ww) {
      const uint32_t ok = s_key[b][ww];
      const int oi = s_idx[b][ww];
      if (ok > gk || (ok == gk && oi < gi)) { gk = ok; gi = oi; }
    }
    if (gk <= 0x007FFFFFu) break;                      // nothing left above -inf (which no step keeps alive)
    if (count >= k && gk != kth) break;                // past the k-th and its ties
    if (count == CAND_CAP) { over = 1; break; }        // more ties than the list holds
    if (count == k - 1) kth = gk;
    if (threadIdx.x == 0) {
      l_val[count] = key_value(gk);
      l_idx[count] = lo + gi;
    }
    if (bk == gk && bi == gi) {
#pragma unroll
      for (int j = 0; j < CAND_EPT; ++j)
        if (j == bj) key[j] = 0u;
    }
    ++count;
  }
  __syncthreads();
  const size_t base = ((size_t)rowi * CAND_CHUNKS + chunk) * CAND_CAP;
  for (int i = threadIdx.x; i < count; i += 256) {
    cand_val[base + i] = l_val[i];
    cand_idx[base + i] = l_idx[i];
  }
  if (threadIdx.x == 0) cand_n[rowi * CAND_CHUNKS + chunk] = over ? -1 : count;
}

__global__ __launch_bounds__(NT) void sample_filtered_kernel(float* __restrict__ logits, int ld, int vocab, int k,
                                                             float top_p, float temp,
                                                             const long long* __restrict__ streams,
                                                             const int* __restrict__ steps,
                                                             const float* __restrict__ forced_r,
                                                             const float* __restrict__ cand_val,
                                                             const int* __restrict__ cand_idx,
                                                             const int* __restrict__ cand_n,
                                                             int* __restrict__ out) {
  __shared__ float v[SURV_CAP];        // survivors: value, index, probability, rank, alive
  __shared__ int ix[SURV_CAP];
  __shared__ float pr[SURV_CAP];
  __shared__ int rank_p[SURV_CAP];     // place in (probability descending, index ascending)
  __shared__ int rank_i[SURV_CAP];     // place in index order
  __shared__ int alive[SURV_CAP];
  __shared__ int order[SURV_CAP];      // survivor at a place
  __shared__ int s_n, s_over;
  __shared__ float c_val[CAND_CHUNKS * CAND_CAP];      // the pieces' lists
  __shared__ int c_idx[CAND_CHUNKS * CAND_CAP];
  __shared__ int c_n[CAND_CHUNKS];
  const int rowi = blockIdx.x;
  float* row = logits + (size_t)rowi * ld;
  const int tid = threadIdx.x, lane = tid & 63;
  if (tid == 0) { s_n = 0; s_over = 0; }
  if (tid < CAND_CHUNKS) c_n[tid] = cand_n[rowi * CAND_CHUNKS + tid];
  __syncthreads();
  for (int i = tid; i < CAND_CHUNKS * CAND_CAP; i += NT) {
    if ((i % CAND_CAP) < c_n[i / CAND_CAP]) {
      c_val[i] = cand_val[(size_t)rowi * CAND_CHUNKS * CAND_CAP + i];
      c_idx[i] = cand_idx[(size_t)rowi * CAND_CHUNKS * CAND_CAP + i];
    }
  }
  __syncthreads();
  if (tid < 64) {
    // the pieces' lists are sorted: lane c holds the head of piece c's, the wave takes the best
    // head (the lower piece among equals, which is the lower index) until the k-th and its ties are out
    const int c = lane;
    int cn = c < CAND_CHUNKS ? c_n[c] : 0;
    const bool piece_over = __builtin_amdgcn_ballot_w64(cn < 0) != 0;
    const int base = c * CAND_CAP;
    int head = 0, count = 0, over = piece_over ? 1 : 0;
    uint32_t kth = 0;
    while (!over) {
      const bool has = head < cn;
      uint32_t hk = has ? order_key(c_val[base + head]) : 0;
      uint32_t rk = hk;
      int rc = has ? c : 0x7fffffff;
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) {
        const uint32_t ok = __shfl_xor(rk, o, MF_WAVE);
        const int oc = __shfl_xor(rc, o, MF_WAVE);
        if (oc != 0x7fffffff && (rc == 0x7fffffff || ok > rk || (ok == rk && oc < rc))) { rk = ok; rc = oc; }
      }
      if (rc == 0x7fffffff) break;
      if (count >= k && rk != kth) break;
      if (count == SURV_CAP) { over = 1; break; }
      if (count == k - 1) kth = rk;
      if (c == rc) {
        v[count] = c_val[base + head];
        ix[count] = c_idx[base + head];
        ++head;
      }
      ++count;
    }
    if (lane == 0) { s_n = count; s_over = over; }
  }
  __syncthreads();
  if (s_over) {            // too many equal values for the lists: the whole-row kernels, in place
    top_k_row(row, vocab, k);
    top_p_row(row, vocab, top_p);
    sample_row(row, rowi, vocab, temp, streams, steps, forced_r, out);
    return;
  }
  const int n = s_n;       // survivors, largest first, equal values in index order
  if (tid < n) alive[tid] = 1;
  __syncthreads();
  const float mx = n > 0 ? v[0] : -INFINITY;
  if (top_p > 0.f && top_p < 1.f && mx > -INFINITY) {
    // as top_p_row: p_i = exp(l_i - max) / sum over finite entries, the sum in double
    __shared__ double s_tot;
    __shared__ double ed[SURV_CAP];
    if (tid < n) ed[tid] = v[tid] > -INFINITY ? exp((double)(v[tid] - mx)) : 0.0;
    __syncthreads();
    if (tid == 0) {
      double t = 0.0;
      for (int i = 0; i < n; ++i) t += ed[i];
      s_tot = t;
    }
    __syncthreads();
    const float tot_f = (float)s_tot;
    if (tid < n) pr[tid] = v[tid] > -INFINITY ? share_of(v[tid], mx, tot_f) : -1.f;    // -1: not finite, last
    __syncthreads();
    if (tid < n) {
      int r = 0;
      for (int j = 0; j < n; ++j)
        if (pr[j] > pr[tid] || (pr[j] == pr[tid] && ix[j] < ix[tid])) ++r;
      rank_p[tid] = r;
      order[r] = tid;
    }
    __syncthreads();
    if (tid == 0) {
      // descending, stable: the shortest prefix whose mass exceeds p stays
      double cum = 0.0;
      int keep = n;
      for (int r = 0; r < n; ++r) {
        const int i = order[r];
        if (pr[i] < 0.f) { keep = min(keep, r); break; }       // entries that are not finite stay as they are
        cum += (double)pr[i];
        if (cum > (double)top_p) { keep = r + 1; break; }
      }
      for (int r = keep; r < n; ++r)
        if (pr[order[r]] >= 0.f) alive[order[r]] = 0;
    }
    __syncthreads();
  }
  // as sample_row on what is left, in index order
  if (tid < n) {
    int r = 0;
    for (int j = 0; j < n; ++j)
      if (ix[j] < ix[tid]) ++r;
    rank_i[tid] = r;
  }
  __syncthreads();
  if (tid < n) order[rank_i[tid]] = tid;
  __shared__ float s_mxt, s_inv;
  __shared__ float ev[SURV_CAP];       // exp(l - max) of a survivor, 0 for one that is out
  const float inv_t = 1.0f / temp;
  __syncthreads();
  if (tid == 0) {
    float mxt = -INFINITY;
    for (int i = 0; i < n; ++i)
      if (alive[i]) mxt = fmaxf(mxt, scaled(v[i], inv_t));
    s_mxt = mxt;
  }
  __syncthreads();
  if (tid < n) {
    const float l = scaled(v[tid], inv_t);
    ev[tid] = (alive[tid] && l > -INFINITY) ? exp_rel(l, s_mxt) : 0.f;
  }
  __syncthreads();
  if (tid == 0) {
    double total = 0.0;
    for (int r = 0; r < n; ++r) total += (double)ev[order[r]];
    s_inv = (float)(1.0 / total);
  }
  __syncthreads();
  if (tid < n) ev[tid] = ev[tid] * s_inv;              // the probability, as prob_of forms it
  __syncthreads();
  if (tid == 0) {
    const float rnd = forced_r ? forced_r[rowi]
                               : uniform01((uint64_t)streams[rowi], (uint64_t)(uint32_t)steps[rowi]);
    const double rr = fmax((double)rnd, 1e-30);
    double cum = 0.0;
    int pick = vocab - 1;                // fallback: the last index (src/sampler.rs:266)
    for (int r = 0; r < n; ++r) {
      const int i = order[r];
      const float p = ev[i];
      if (p <= 0.f) continue;
      cum += (double)p;
      if (rr <= cum) { pick = ix[i]; break; }
    }
    out[rowi] = pick;
  }
}

// after a decode step: feed the sampled token back, move every sequence on by one, and (when
// prev is given) put the token into the sequence's window of recent tokens: prev[i] holds the
// last n_prev[i] <= max_prev tokens in no particular order (the penalties count, they do not
// look at the order), cursor[i] is where the next one goes, the oldest once the window is full.
__global__ void advance_kernel(int* __restrict__ next_ids, const int* __restrict__ sampled,
                               int* __restrict__ positions, int* __restrict__ steps, int n,
                               int* __restrict__ prev, int max_prev, int* __restrict__ n_prev,
                               int* __restrict__ cursor) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int tok = sampled[i];
  next_ids[i] = tok;
  positions[i] += 1;
  steps[i] += 1;
  if (prev) {
    const int c = cursor[i];
    prev[(size_t)i * max_prev + c] = tok;
    cursor[i] = c + 1 == max_prev ? 0 : c + 1;
    if (n_prev[i] < max_prev) n_prev[i] += 1;
  }
}

}  // namespace

// `work` (chunks * rows floats and as many ints, chunks <= 64) lets few rows of a large
// vocabulary spread over the chip; without it a row is one block.
MF_API int mf_argmax(const float* logits, int ld, int rows, int vocab, int* out, float* work, int chunks,
                     hipStream_t stream) {
  if (rows <= 0) return 0;
  if (vocab <= 0 || ld < vocab || chunks > 64) return (int)hipErrorInvalidValue;
  if (work && chunks > 1) {
    int* pidx = reinterpret_cast<int*>(work + (size_t)rows * chunks);
    argmax_part_kernel<<<dim3(rows, chunks), NT, 0, stream>>>(logits, ld, vocab, chunks, work, pidx);
    int rc = mf_launch_status();
    if (rc) return rc;
    argmax_final_kernel<<<rows, 64, 0, stream>>>(work, pidx, chunks, out);
    return mf_launch_status();
  }
  argmax_kernel<<<rows, NT, 0, stream>>>(logits, ld, vocab, out, nullptr);
  return mf_launch_status();
}

MF_API int mf_sample(const float* logits, int ld, int rows, int vocab, float temp,
                     const long long* streams, const int* steps, const float* forced_r, int* out,
                     hipStream_t stream) {
  if (rows <= 0) return 0;
  if (vocab <= 0 || ld < vocab) return (int)hipErrorInvalidValue;
  sample_kernel<<<rows, NT, 0, stream>>>(logits, ld, vocab, temp, streams, steps, forced_r, out);
  return mf_launch_status();
}

// top-k (1 <= k <= 48), top-p (outside (0,1): off) and the temperature draw (temp >= 1e-6) in two
// kernels that read the row once; `work` holds rows * 32 * 64 floats, as many ints, and rows * 32
// ints.  The logits stay as they are unless a row has more equal values than the lists hold.
MF_API int mf_sample_filtered(float* logits, int ld, int rows, int vocab, int k, float top_p, float temp,
                              const long long* streams, const int* steps, const float* forced_r,
                              void* work, int* out, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (vocab <= 0 || ld < vocab || k < 1 || k > FAST_K_MAX || !(temp >= 1e-6f) || !work ||
      vocab > CAND_CHUNKS * 256 * CAND_EPT)
    return (int)hipErrorInvalidValue;
  float* cand_val = (float*)work;
  int* cand_idx = (int*)(cand_val + (size_t)rows * CAND_CHUNKS * CAND_CAP);
  int* cand_n = cand_idx + (size_t)rows * CAND_CHUNKS * CAND_CAP;
  topk_candidates_kernel<<<dim3(CAND_CHUNKS, rows), 256, 0, stream>>>(logits, ld, vocab, k, cand_val, cand_idx,
                                                                      cand_n);
  int rc = mf_launch_status();
  if (rc) return rc;
  sample_filtered_kernel<<<rows, NT, 0, stream>>>(logits, ld, vocab, k, top_p, temp, streams, steps, forced_r,
                                                  cand_val, cand_idx, cand_n, out);
  return mf_launch_status();
}

MF_API int mf_penalties(float* logits, int ld, int rows, int vocab, const int* prev, int max_prev,
                        const int* n_prev, float repeat, float frequency, float presence,
                        hipStream_t stream) {
  if (rows <= 0 || max_prev <= 0) return 0;
  if (vocab <= 0 || ld < vocab) return (int)hipErrorInvalidValue;
  penalties_kernel<<<rows, 64, 0, stream>>>(logits, ld, vocab, prev, max_prev, n_prev, repeat, frequency,
                                            presence);
  return mf_launch_status();
}

MF_API int mf_top_k(float* logits, int ld, int rows, int vocab, int k, hipStream_t stream) {
  if (rows <= 0 || k <= 0 || k >= vocab) return 0;
  if (ld < vocab) return (int)hipErrorInvalidValue;
  top_k_kernel<<<rows, NT, 0, stream>>>(logits, ld, vocab, k);
  return mf_launch_status();
}

MF_API int mf_top_p(float* logits, int ld, int rows, int vocab, float p, hipStream_t stream) {
  if (rows <= 0 || !(p > 0.f && p < 1.f)) return 0;
  if (vocab <= 0 || ld < vocab) return (int)hipErrorInvalidValue;
  top_p_kernel<<<rows, NT, 0, stream>>>(logits, ld, vocab, p);
  return mf_launch_status();
}

MF_API int mf_advance(int* next_ids, const int* sampled, int* positions, int* steps, int n, int* prev,
                      int max_prev, int* n_prev, int* cursor, hipStream_t stream) {
  if (n <= 0) return 0;
  if (prev && (max_prev <= 0 || !n_prev || !cursor)) return (int)hipErrorInvalidValue;
  advance_kernel<<<(n + 255) / 256, 256, 0, stream>>>(next_ids, sampled, positions, steps, n, prev, max_prev,
                                                      n_prev, cursor);
  return mf_launch_status();
}
