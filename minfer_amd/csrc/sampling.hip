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

namespace {

constexpr int NT = 1024;

__device__ __forceinline__ uint64_t mix64(uint64_t z) {
  z += 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

// uniform in [0,1) with 24 bits; mirrored by minfer_amd.sampling.rng.uniform
__device__ __forceinline__ float uniform01(uint64_t seed, uint64_t key, uint64_t step) {
  const uint64_t h = mix64(mix64(seed ^ mix64(key)) ^ step);
  return (float)(uint32_t)(h >> 40) * (1.0f / 16777216.0f);
}

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
    const float v = row[i] * scale;
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
__global__ __launch_bounds__(NT) void sample_kernel(const float* __restrict__ logits, int ld, int vocab,
                                                    float temp, uint64_t seed,
                                                    const long long* __restrict__ keys,
                                                    const int* __restrict__ steps,
                                                    const float* __restrict__ forced_r,
                                                    int* __restrict__ out) {
  __shared__ float s_val[NT / 64];
  __shared__ int s_idx[NT / 64];
  __shared__ double s_d[NT / 64];
  __shared__ double s_wave_tot[NT / 64];
  __shared__ int s_found;
  const int rowi = blockIdx.x;
  const float* row = logits + (size_t)rowi * ld;
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
  const int chunk = (vocab + NT - 1) / NT;
  const int lo = min(vocab, (int)threadIdx.x * chunk), hi = min(vocab, lo + chunk);
  double mine = 0.0;
  for (int i = lo; i < hi; ++i) {
    const float l = row[i] * inv_t;
    if (l > -INFINITY) mine += (double)expf(l - mx);
  }
  const double total = block_sum_d(mine, s_d);
  const float inv = (float)(1.0 / total);
  // probabilities as the reference forms them: e * (1/sum as f32)
  double pm = 0.0;
  for (int i = lo; i < hi; ++i) {
    const float l = row[i] * inv_t;
    if (l > -INFINITY) pm += (double)(expf(l - mx) * inv);
  }
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
                     : uniform01(seed, (uint64_t)keys[rowi], (uint64_t)(uint32_t)steps[rowi]);
  const double rr = fmax((double)r, 1e-30);
  if (pm > 0.0 && prefix < rr && rr <= prefix + pm) {
    double cum = prefix;
    int pick = -1;
    for (int i = lo; i < hi; ++i) {
      const float l = row[i] * inv_t;
      if (!(l > -INFINITY)) continue;
      const float p = expf(l - mx) * inv;
      if (p <= 0.f) continue;
      cum += (double)p;
      pick = i;
      if (rr <= cum) break;
    }
    if (pick >= 0) s_found = pick;
  }
  __syncthreads();
  if (threadIdx.x == 0) out[rowi] = s_found;
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

// top-k by radix select of the k-th largest key, 8 bits a pass
__global__ __launch_bounds__(NT) void top_k_kernel(float* __restrict__ logits, int ld, int vocab, int k) {
  __shared__ unsigned int hist[256];
  __shared__ uint32_t s_prefix;
  __shared__ int s_remaining;
  float* row = logits + (size_t)blockIdx.x * ld;
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
}

// top-p.  Probabilities p_i = exp(l_i - max) / sum over finite entries.  The kept set is
// {p_i > tau} plus the first c entries (in index order) with p_i == tau, where tau is the
// probability at which the descending cumulative mass first exceeds p.  tau is found by
// radix select over the probabilities' bit patterns, accumulating mass per bin in double.
__global__ __launch_bounds__(NT) void top_p_kernel(float* __restrict__ logits, int ld, int vocab,
                                                   float p) {
  __shared__ float s_val[NT / 64];
  __shared__ int s_idx[NT / 64];
  __shared__ double s_d[NT / 64];
  __shared__ double bin_mass[256];
  __shared__ unsigned int bin_count[256];
  __shared__ uint32_t s_prefix;
  __shared__ double s_above;
  __shared__ unsigned int s_ties;
  __shared__ unsigned int s_wave_cnt[NT / 64];
  float* row = logits + (size_t)blockIdx.x * ld;
  if (!(p > 0.f && p < 1.f)) return;
  float mx;
  int amax;
  block_argmax(row, vocab, 1.0f, s_val, s_idx, mx, amax);
  if (!(mx > -INFINITY)) return;
  const int chunk = (vocab + NT - 1) / NT;
  const int lo = min(vocab, (int)threadIdx.x * chunk), hi = min(vocab, lo + chunk);
  double mine = 0.0;
  for (int i = lo; i < hi; ++i)
    if (row[i] > -INFINITY) mine += exp((double)(row[i] - mx));
  const double total = block_sum_d(mine, s_d);
  const float tot_f = (float)total;
  if (threadIdx.x == 0) { s_prefix = 0; s_above = 0.0; }
  for (int pass = 0; pass < 4; ++pass) {
    const int shift = 24 - 8 * pass;
    for (int i = threadIdx.x; i < 256; i += NT) { bin_mass[i] = 0.0; bin_count[i] = 0; }
    __syncthreads();
    const uint32_t prefix = s_prefix;
    const uint32_t mask = pass == 0 ? 0u : (0xFFFFFFFFu << (shift + 8));
    for (int i = lo; i < hi; ++i) {
      if (!(row[i] > -INFINITY)) continue;
      const float pr = expf(row[i] - mx) / tot_f;
      const uint32_t key = __float_as_uint(pr);        // pr >= 0: bit order is value order
      if ((key & mask) == prefix) {
        atomicAdd(&bin_mass[(key >> shift) & 255u], (double)pr);
        atomicAdd(&bin_count[(key >> shift) & 255u], 1u);
      }
    }
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
  for (int i = lo; i < hi; ++i)
    if (row[i] > -INFINITY && __float_as_uint(expf(row[i] - mx) / tot_f) == tau_key) ++my_ties;
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
  for (int i = lo; i < hi; ++i) {
    if (!(row[i] > -INFINITY)) continue;
    const uint32_t key = __float_as_uint(expf(row[i] - mx) / tot_f);
    if (key > tau_key) continue;
    if (key == tau_key && rank++ < keep_ties) continue;
    row[i] = -INFINITY;
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

MF_API int mf_sample(const float* logits, int ld, int rows, int vocab, float temp, uint64_t seed,
                     const long long* keys, const int* steps, const float* forced_r, int* out,
                     hipStream_t stream) {
  if (rows <= 0) return 0;
  if (vocab <= 0 || ld < vocab) return (int)hipErrorInvalidValue;
  sample_kernel<<<rows, NT, 0, stream>>>(logits, ld, vocab, temp, seed, keys, steps, forced_r, out);
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
