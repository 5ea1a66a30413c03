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
// into CAND_CHUNKS pieces, one wave each, and lists each piece's k largest entries and every
// further entry equal to the k-th (largest first, equal values in index order): the row's k
// largest and their ties are among them.  A second kernel, one block per row, merges the lists
// into the row's survivors (the k largest and the ties of the k-th), and then does on these few
// what top_p_row and sample_row do on the whole row, with the same arithmetic in the same order
// (probabilities as float, sums in double in index order).  The logits are not changed.  A piece
// or a row with more ties than a list holds (a constant row, say) takes the kernels above
// instead, inside the second kernel, which then does change the row.
constexpr int CAND_CHUNKS = 64;      // pieces of a row (the merge gives a lane to each)
constexpr int CAND_CAP = 64;         // entries of a piece's list
constexpr int CAND_EPT = 64;         // most entries per lane of a piece: vocab <= 64 * 64 * 64
constexpr int FAST_K_MAX = 48;       // the largest k that takes this path
constexpr int SURV_CAP = 128;        // survivors of a row

// The largest entry of every piece, as a key (0: the piece has none above -inf).  The k-th largest
// of a row's piece maxima is a bound from below on the row's k-th largest entry (they are k entries
// of the row themselves), so the lists need nothing smaller: most pieces then list nothing or one.
__global__ __launch_bounds__(256) void piece_max_kernel(const float* __restrict__ logits, int ld, int vocab,
                                                        uint32_t* __restrict__ piece_max) {
  const int lane = threadIdx.x & 63;
  const int rowi = blockIdx.y, chunk = blockIdx.x * 4 + (threadIdx.x >> 6);
  const float* row = logits + (size_t)rowi * ld;
  const int per = (vocab + CAND_CHUNKS - 1) / CAND_CHUNKS;
  const int lo = chunk * per, n = max(0, min(per, vocab - lo));
  uint32_t best = 0;
  for (int i0 = 0; i0 < n; i0 += 8 * 64) {            // eight loads on their way at a time
    float x[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) x[u] = row[lo + min(i0 + u * 64 + lane, n - 1)];     // (the last one again: a maximum does not mind)
#pragma unroll
    for (int u = 0; u < 8; ++u) best = max(best, order_key(x[u]));
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) best = max(best, (uint32_t)__shfl_xor((int)best, o, MF_WAVE));
  if (lane == 0) piece_max[rowi * CAND_CHUNKS + chunk] = best <= 0x007FFFFFu ? 0u : best;
}

// One wave lists one piece (no barrier anywhere: a block is four pieces that know nothing of each
// other): each lane holds its entries of the piece as keys, the wave takes the largest that is
// still in play until the k-th and its ties are out or the next one is below the row's bound,
// lane 0 writes it out.
template <int EPT>      // entries per lane: a piece has at most 64 EPT
__global__ __launch_bounds__(256) void topk_candidates_kernel(const float* __restrict__ logits, int ld,
                                                              int vocab, int k,
                                                              const uint32_t* __restrict__ piece_max,
                                                              float* __restrict__ cand_val,
                                                              int* __restrict__ cand_idx,
                                                              int* __restrict__ cand_n) {
  const int lane = threadIdx.x & 63;
  const int rowi = blockIdx.y, chunk = blockIdx.x * 4 + (threadIdx.x >> 6);
  const float* row = logits + (size_t)rowi * ld;
  const int per = (vocab + CAND_CHUNKS - 1) / CAND_CHUNKS;
  const int lo = chunk * per, n = max(0, min(per, vocab - lo));
  // the bound: lane c holds piece c's maximum; its place among the 64 (larger first, the lower piece
  // among equals) is the number of lanes that come before it; the one at place k - 1 is the bound
  static_assert(CAND_CHUNKS == 64 && FAST_K_MAX <= CAND_CHUNKS, "a lane for every piece, k pieces at least");
  const uint32_t mine = piece_max[rowi * CAND_CHUNKS + lane];
  int place = 0;
  for (int c = 0; c < 64; ++c) {
    const uint32_t other = (uint32_t)__shfl((int)mine, c, MF_WAVE);
    place += (other > mine || (other == mine && c < lane)) ? 1 : 0;
  }
  const unsigned long long at = __builtin_amdgcn_ballot_w64(place == k - 1);
  const uint32_t bound = (uint32_t)__shfl((int)mine, (int)__builtin_ctzll(at), MF_WAVE);    // 0: no bound
  // this lane's entries: lo + j * 64 + lane, as keys; 0 marks one that is out of play (no entry
  // above -inf has a key that small, and those at or below -inf are never listed)
  uint32_t key[EPT];
#pragma unroll
  for (int j = 0; j < EPT; ++j) {
    const int i = j * 64 + lane;
    key[j] = i < n ? order_key(row[lo + i]) : 0u;
  }
  const size_t base = ((size_t)rowi * CAND_CHUNKS + chunk) * CAND_CAP;
  int count = 0, over = 0;
  uint32_t kth = 0;
  for (;;) {
    // the largest entry of the piece that is still in play, the lowest index among equals
    uint32_t bk = 0;
    int bj = 0;
#pragma unroll
    for (int j = 0; j < EPT; ++j)
      if (key[j] > bk) { bk = key[j]; bj = j; }
    const int bi = bj * 64 + lane;
    uint32_t gk = bk;
    int gi = bi;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const uint32_t ok = __shfl_xor(gk, o, MF_WAVE);
      const int oi = __shfl_xor(gi, o, MF_WAVE);
      if (ok > gk || (ok == gk && oi < gi)) { gk = ok; gi = oi; }
    }
    if (gk <= 0x007FFFFFu) break;                      // nothing left above -inf (which no step keeps alive)
    if (gk < bound) break;                             // below the row's k-th largest for certain
    if (count >= k && gk != kth) break;                // past the k-th and its ties
    if (count == CAND_CAP) { over = 1; break; }        // more ties than the list holds
    if (count == k - 1) kth = gk;
    if (lane == 0) {
      cand_val[base + count] = key_value(gk);
      cand_idx[base + count] = lo + gi;
    }
    if (bk == gk && bi == gi) {
#pragma unroll
      for (int j = 0; j < EPT; ++j)
        if (j == bj) key[j] = 0u;
    }
    ++count;
  }
  if (lane == 0) cand_n[rowi * CAND_CHUNKS + chunk] = over ? -1 : count;
}

// Sums that have to run one after the other (doubles, in a fixed order) run in wave 0 with the
// terms in registers, place r in lane r % 64 (register r / 64), read out by lane number: a
// thread that walks an LDS array instead waits for every element in turn.
__device__ __forceinline__ float at_place(float lo, float hi, int r) {       // r the same in every lane
  const int l = __builtin_amdgcn_readfirstlane(r & 63);
  return __int_as_float(r < 64 ? __builtin_amdgcn_readlane(__float_as_int(lo), l)
                               : __builtin_amdgcn_readlane(__float_as_int(hi), l));
}
__device__ __forceinline__ int at_place(int lo, int hi, int r) {
  const int l = __builtin_amdgcn_readfirstlane(r & 63);
  return r < 64 ? __builtin_amdgcn_readlane(lo, l) : __builtin_amdgcn_readlane(hi, l);
}
__device__ __forceinline__ double at_place(double lo, double hi, int r) {
  const int l = __builtin_amdgcn_readfirstlane(r & 63);
  const double x = r < 64 ? lo : hi;
  const int a = __builtin_amdgcn_readlane(__double2loint(x), l), b = __builtin_amdgcn_readlane(__double2hiint(x), l);
  return __hiloint2double(b, a);
}

constexpr int RANK_MAX = 512;        // candidates up to which each finds its place by counting the ones before it

__global__ __launch_bounds__(NT) void sample_filtered_kernel(float* __restrict__ logits, int ld, int vocab, int k,
                                                             float top_p, float temp,
                                                             const long long* __restrict__ streams,
                                                             const int* __restrict__ steps,
                                                             const float* __restrict__ forced_r,
                                                             const float* __restrict__ cand_val,
                                                             const int* __restrict__ cand_idx,
                                                             const int* __restrict__ cand_n,
                                                             int* __restrict__ out) {
  __shared__ float v[SURV_CAP];        // survivors: value, index, probability, alive
  __shared__ int ix[SURV_CAP];
  __shared__ float pr[SURV_CAP];
  __shared__ int alive[SURV_CAP];
  __shared__ int order[SURV_CAP];      // survivor at a place
  __shared__ int s_n, s_over, s_total, s_keep;
  __shared__ uint32_t s_kth;
  __shared__ uint32_t d_key[CAND_CHUNKS * CAND_CAP];   // the pieces' lists one after the other, as keys
  __shared__ int d_idx[CAND_CHUNKS * CAND_CAP];
  __shared__ int c_n[CAND_CHUNKS], c_off[CAND_CHUNKS];
  const int rowi = blockIdx.x;
  float* row = logits + (size_t)rowi * ld;
  const int tid = threadIdx.x, lane = tid & 63;
  if (tid == 0) { s_n = 0; s_over = 0; s_kth = 0; }
  __syncthreads();
  if (tid < 64) {
    // where each piece's list begins in the row's list
    static_assert(CAND_CHUNKS == 64, "a lane for every piece");
    const int cn = cand_n[rowi * CAND_CHUNKS + lane];
    const bool piece_over = __builtin_amdgcn_ballot_w64(cn < 0) != 0;
    const int cnt = max(cn, 0);
    int incl = cnt;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const int up = __shfl_up(incl, o, MF_WAVE);
      if (lane >= o) incl += up;
    }
    c_n[lane] = cnt;
    c_off[lane] = incl - cnt;
    if (lane == 63) s_total = incl;
    if (lane == 0 && piece_over) s_over = 1;
  }
  __syncthreads();
  const int C = s_total;
  if (!s_over) {
    // every piece's first entries in the first round (the lists are short as a rule: one wait for
    // memory, not one per piece)
    for (int s0 = 0; s0 < CAND_CAP; s0 += NT / CAND_CHUNKS) {
      const int piece = tid % CAND_CHUNKS, slot = s0 + tid / CAND_CHUNKS;
      if (slot < c_n[piece]) {
        const size_t src = (size_t)rowi * CAND_CHUNKS * CAND_CAP + piece * CAND_CAP + slot;
        d_key[c_off[piece] + slot] = order_key(cand_val[src]);
        d_idx[c_off[piece] + slot] = cand_idx[src];
      }
    }
  }
  __syncthreads();
  if (!s_over && C <= RANK_MAX) {
    // Few candidates (the rule): each counts the ones that come before it (larger first, the lower
    // index among equals), which is its place; the one at place k - 1 names the k-th value, and
    // what is at least that survives, at its place.
    static_assert(RANK_MAX <= NT, "a thread for every candidate");
    uint32_t mk = 0;
    int mi = 0, place = 0;
    if (tid < C) {
      mk = d_key[tid];
      mi = d_idx[tid];
      for (int j = 0; j < C; ++j) {
        const uint32_t ok = d_key[j];
        const int oi = d_idx[j];
        place += (ok > mk || (ok == mk && oi < mi)) ? 1 : 0;
      }
      if (place == k - 1) s_kth = mk;
    }
    __syncthreads();
    if (tid < C && mk >= s_kth) {
      if (place < SURV_CAP) {
        v[place] = key_value(mk);
        ix[place] = mi;
      } else {
        s_over = 1;
      }
      atomicAdd(&s_n, 1);
    }
  } else if (!s_over && tid < 64) {
    // many candidates: the pieces' lists are sorted, lane c holds the head of piece c's, the wave
    // takes the best head (the lower piece among equals, which is the lower index) until the k-th
    // and its ties are out
    const int c = lane;
    const int cn = c_n[c], base = c_off[c];
    int head = 0, count = 0, over = 0;
    uint32_t kth = 0;
    for (;;) {
      const bool has = head < cn;
      const uint32_t hk = has ? d_key[base + head] : 0;
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
        v[count] = key_value(d_key[base + head]);
        ix[count] = d_idx[base + head];
        ++head;
      }
      ++count;
    }
    if (lane == 0) { s_n = count; if (over) s_over = 1; }
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
  const int r0 = lane, r1 = lane + 64;                 // wave 0: the two places of a lane
  if (top_p > 0.f && top_p < 1.f && mx > -INFINITY) {
    // as top_p_row: p_i = exp(l_i - max) / sum over finite entries, the sum in double
    __shared__ double s_tot;
    if (tid < 64) {
      const double e0 = r0 < n && v[r0] > -INFINITY ? exp((double)(v[r0] - mx)) : 0.0;
      const double e1 = r1 < n && v[r1] > -INFINITY ? exp((double)(v[r1] - mx)) : 0.0;
      double t = 0.0;
      for (int i = 0; i < n; ++i) t += at_place(e0, e1, i);
      if (lane == 0) s_tot = t;
    }
    __syncthreads();
    const float tot_f = (float)s_tot;
    if (tid < n) pr[tid] = v[tid] > -INFINITY ? share_of(v[tid], mx, tot_f) : -1.f;    // -1: not finite, last
    __syncthreads();
    if (tid < n) {
      int r = 0;
      for (int j = 0; j < n; ++j)
        if (pr[j] > pr[tid] || (pr[j] == pr[tid] && ix[j] < ix[tid])) ++r;
      order[r] = tid;
    }
    __syncthreads();
    if (tid < 64) {
      // descending, stable: the shortest prefix whose mass exceeds p stays
      const float p0 = r0 < n ? pr[order[r0]] : -1.f, p1 = r1 < n ? pr[order[r1]] : -1.f;
      double cum = 0.0;
      int keep = n;
      for (int r = 0; r < n; ++r) {
        const float p = at_place(p0, p1, r);
        if (p < 0.f) { keep = min(keep, r); break; }           // entries that are not finite stay as they are
        cum += (double)p;
        if (cum > (double)top_p) { keep = r + 1; break; }
      }
      if (r0 < n && r0 >= keep && p0 >= 0.f) alive[order[r0]] = 0;
      if (r1 < n && r1 >= keep && p1 >= 0.f) alive[order[r1]] = 0;
    }
    __syncthreads();
  }
  // as sample_row on what is left, in index order
  if (tid < n) {
    int r = 0;
    for (int j = 0; j < n; ++j)
      if (ix[j] < ix[tid]) ++r;
    order[r] = tid;
  }
  __syncthreads();
  if (tid >= 64) return;
  // wave 0 alone from here on: lane holds the survivors at places r0 and r1 of the index order
  const float inv_t = 1.0f / temp;
  const int i0 = r0 < n ? order[r0] : 0, i1 = r1 < n ? order[r1] : 0;
  const bool on0 = r0 < n && alive[i0], on1 = r1 < n && alive[i1];
  const float l0 = on0 ? scaled(v[i0], inv_t) : -INFINITY, l1 = on1 ? scaled(v[i1], inv_t) : -INFINITY;
  float mxt = fmaxf(l0, l1);
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) mxt = fmaxf(mxt, __shfl_xor(mxt, o, MF_WAVE));
  const float e0 = l0 > -INFINITY ? exp_rel(l0, mxt) : 0.f, e1 = l1 > -INFINITY ? exp_rel(l1, mxt) : 0.f;
  double total = 0.0;
  for (int r = 0; r < n; ++r) total += (double)at_place(e0, e1, r);
  const float inv = (float)(1.0 / total);
  const float q0 = e0 * inv, q1 = e1 * inv;            // the probability, as prob_of forms it
  const int x0 = r0 < n ? ix[i0] : 0, x1 = r1 < n ? ix[i1] : 0;
  const float rnd = forced_r ? forced_r[rowi]
                             : uniform01((uint64_t)streams[rowi], (uint64_t)(uint32_t)steps[rowi]);
  const double rr = fmax((double)rnd, 1e-30);
  double cum = 0.0;
  int pick = vocab - 1;                // fallback: the last index (src/sampler.rs:266)
  for (int r = 0; r < n; ++r) {
    const float p = at_place(q0, q1, r);
    if (p <= 0.f) continue;
    cum += (double)p;
    if (rr <= cum) { pick = at_place(x0, x1, r); break; }
  }
  if (lane == 0) out[rowi] = pick;
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
// kernels that read the row once (and a small one before them that reads it for the pieces'
// maxima); `work` holds rows * 64 * 64 floats, as many ints, and twice rows * 64 ints.  The logits stay as they are unless a row has more equal values than the lists hold.
MF_API int mf_sample_filtered(float* logits, int ld, int rows, int vocab, int k, float top_p, float temp,
                              const long long* streams, const int* steps, const float* forced_r,
                              void* work, int* out, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (vocab <= 0 || ld < vocab || k < 1 || k > FAST_K_MAX || !(temp >= 1e-6f) || !work ||
      vocab > CAND_CHUNKS * 64 * CAND_EPT)
    return (int)hipErrorInvalidValue;
  float* cand_val = (float*)work;
  int* cand_idx = (int*)(cand_val + (size_t)rows * CAND_CHUNKS * CAND_CAP);
  int* cand_n = cand_idx + (size_t)rows * CAND_CHUNKS * CAND_CAP;
  uint32_t* piece_max = (uint32_t*)(cand_n + (size_t)rows * CAND_CHUNKS);
  const dim3 grid(CAND_CHUNKS / 4, rows);
  piece_max_kernel<<<grid, 256, 0, stream>>>(logits, ld, vocab, piece_max);
  if (int rc0 = mf_launch_status()) return rc0;
  const int ept = ((vocab + CAND_CHUNKS - 1) / CAND_CHUNKS + 63) / 64;     // entries per lane of a piece
  if (ept <= 16) topk_candidates_kernel<16><<<grid, 256, 0, stream>>>(logits, ld, vocab, k, piece_max, cand_val, cand_idx, cand_n);
  else if (ept <= 32) topk_candidates_kernel<32><<<grid, 256, 0, stream>>>(logits, ld, vocab, k, piece_max, cand_val, cand_idx, cand_n);
  else if (ept <= 48) topk_candidates_kernel<48><<<grid, 256, 0, stream>>>(logits, ld, vocab, k, piece_max, cand_val, cand_idx, cand_n);
  else topk_candidates_kernel<CAND_EPT><<<grid, 256, 0, stream>>>(logits, ld, vocab, k, piece_max, cand_val, cand_idx, cand_n);
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
