// Attention of single query tokens over the paged cache, split along the keys.
//
// For a query token t of sequence b at position p and kv head hk, the G = nh/nk query
// heads of the group read the same keys: cache rows j with lo <= j <= p, lo = 0 or
// p - window + 1.  s_j = dot(q, K_j) * scale; softmax over j; o = sum_j p_j V_j
// (src/graph/cpu_backend.rs:437-494 of yusiwen/minfer; the causal rule "rows 0..=pos" is
// its `vl = pos + 1`, :462).  The softmax is the online form of the reference's CUDA
// kernel (running max, running sum, rescaled accumulator, src/cuda_kernels.cu:673-790),
// all in 32-bit.
//
// Work split: a block owns (token, kv head, chunk of up to GC query heads, key split).
// 16 lanes share one key row, each holding EPL = head_dim/16 consecutive elements; each
// group of 16 lanes takes R rows per step so that 2R independent loads are in flight and
// the running maximum is updated once per R rows.  A block of 4 waves (16 groups) walks
// 16 R rows per step, a divisor of the page size, so a step stays inside one page.  With
// several key splits each block writes an unnormalised partial (acc, max, sum) and
// `attn_combine_kernel` merges them; the merge order is fixed, so results are the same
// bits run to run.
//
// Used for decode in both precisions and for whole prompts in the 32-bit path.
#pragma once
#include <type_traits>
#include "common.h"

namespace attn_tokens {

template <int EPL> struct Chunk { static constexpr int GC = (EPL <= 8) ? 8 : 4; };
// rows per 16-lane group per step: 16 bytes of a row per lane -> 4 rows, more -> fewer
template <typename T, int EPL> struct Rows {
  static constexpr int BYTES = EPL * (int)sizeof(T);
  static constexpr int R = BYTES <= 16 ? 4 : (BYTES <= 32 ? 2 : 1);
};

template <typename T> __device__ __forceinline__ float exp_for(float x);
template <> __device__ __forceinline__ float exp_for<float>(float x) { return expf(x); }
template <> __device__ __forceinline__ float exp_for<bf16>(float x) { return __expf(x); }

template <typename T, int EPL>
__device__ __forceinline__ void load_elems(const T* __restrict__ p, float (&dst)[EPL]) {
  constexpr int BYTES = EPL * (int)sizeof(T);
  constexpr int ALIGN = (BYTES % 16 == 0) ? 16 : (BYTES % 8 == 0) ? 8 : (BYTES % 4 == 0) ? 4 : 2;
  const T* a = (const T*)__builtin_assume_aligned(p, ALIGN);
#pragma unroll
  for (int e = 0; e < EPL; ++e) dst[e] = to_f32(a[e]);
}

// the same elements kept in their storage type (for loads issued a step ahead)
template <typename T, int EPL>
__device__ __forceinline__ void load_raw(const T* __restrict__ p, T (&dst)[EPL]) {
  constexpr int BYTES = EPL * (int)sizeof(T);
  constexpr int ALIGN = (BYTES % 16 == 0) ? 16 : (BYTES % 8 == 0) ? 8 : (BYTES % 4 == 0) ? 4 : 2;
  const T* a = (const T*)__builtin_assume_aligned(p, ALIGN);
#pragma unroll
  for (int e = 0; e < EPL; ++e) dst[e] = a[e];
}

// sum over the 16 lanes of a row group, result in every lane (DPP, no LDS traffic)
__device__ __forceinline__ float group16_sum(float v) {
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));   // lane ^ 1
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));   // lane ^ 2
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xF, 0xF, true));  // mirror in 8
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xF, 0xF, true));  // mirror in 16
  return v;
}

template <typename T, int EPL>
__global__ __launch_bounds__(256) void attn_tokens_kernel(
    const T* __restrict__ q, const T* __restrict__ kc, const T* __restrict__ vc,
    const int* __restrict__ page_table, int pt_stride, const int* __restrict__ positions,
    const int* __restrict__ seq_of_tok, T* __restrict__ out, float* __restrict__ part, int nh, int nk,
    float scale, int window, int n_splits, int split_len) {
  constexpr int GC = Chunk<EPL>::GC;
  constexpr int R = Rows<T, EPL>::R;
  constexpr int TILE = 16 * R;
  constexpr int HD = 16 * EPL;
  __shared__ float sm_acc[4][GC][HD];
  __shared__ float sm_ml[4][GC][2];

  const int t = blockIdx.x;
  const int G = nh / nk;
  const int n_gc = (G + GC - 1) / GC;
  const int hk = blockIdx.y / n_gc;
  const int g0 = (blockIdx.y % n_gc) * GC;
  const int gcount = min(GC, G - g0);
  const int h0 = hk * G + g0;
  const int split = blockIdx.z;
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int sub = lane & 15, rg = lane >> 4;
  const int gi = w * 4 + rg;

  const int p = positions[t];
  const int* pt = page_table + (size_t)seq_of_tok[t] * pt_stride;
  const int lo = window > 0 ? max(0, p - window + 1) : 0;
  const int j_begin = max(lo, split * split_len);
  const int j_end = min(p + 1, (split + 1) * split_len);

  float qr[GC][EPL], acc[GC][EPL], m[GC], l[GC];
#pragma unroll
  for (int g = 0; g < GC; ++g) {
    m[g] = -INFINITY;
    l[g] = 0.f;
#pragma unroll
    for (int e = 0; e < EPL; ++e) { acc[g][e] = 0.f; qr[g][e] = 0.f; }
    if (g < gcount) load_elems<T, EPL>(q + ((size_t)t * nh + h0 + g) * HD + sub * EPL, qr[g]);
  }

  // K and V of a step are loaded one step ahead, in their storage type
  T kn[R][EPL], vn[R][EPL];
  auto issue = [&](int tile) {
    const int page = pt[tile / MF_PAGE];
    const size_t base = (((size_t)page * nk + hk) * MF_PAGE + (tile % MF_PAGE)) * HD + sub * EPL;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int row = gi * R + r;                    // row inside the tile
      const int j = tile + row;
      const bool ok = j >= j_begin && j < j_end;
      const int rr = ok ? row : (j_begin > tile ? j_begin - tile : 0);   // a row that exists
      load_raw<T, EPL>(kc + base + (size_t)rr * HD, kn[r]);
      load_raw<T, EPL>(vc + base + (size_t)rr * HD, vn[r]);
    }
  };
  const int tile0 = j_begin & ~(TILE - 1);
  if (tile0 < j_end) issue(tile0);
  for (int tile = tile0; tile < j_end; tile += TILE) {
    float kr[R][EPL], vr[R][EPL];
    bool valid[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int j = tile + gi * R + r;
      valid[r] = j >= j_begin && j < j_end;
#pragma unroll
      for (int e = 0; e < EPL; ++e) { kr[r][e] = to_f32(kn[r][e]); vr[r][e] = to_f32(vn[r][e]); }
    }
    if (tile + TILE < j_end) issue(tile + TILE);
#pragma unroll
    for (int g = 0; g < GC; ++g) {
      if (g < gcount) {
        float s[R];
        float m_new = m[g];
#pragma unroll
        for (int r = 0; r < R; ++r) {
          float d = 0.f;
#pragma unroll
          for (int e = 0; e < EPL; ++e) d = fmaf(qr[g][e], kr[r][e], d);
          d = group16_sum(d);
          s[r] = valid[r] ? d * scale : -INFINITY;
          m_new = fmaxf(m_new, s[r]);
        }
        const float corr = (m_new == -INFINITY) ? 1.f : exp_for<T>(m[g] - m_new);
        float lsum = l[g] * corr;
#pragma unroll
        for (int e = 0; e < EPL; ++e) acc[g][e] *= corr;
#pragma unroll
        for (int r = 0; r < R; ++r) {
          const float pe = valid[r] ? exp_for<T>(s[r] - m_new) : 0.f;
          lsum += pe;
#pragma unroll
          for (int e = 0; e < EPL; ++e) acc[g][e] = fmaf(pe, vr[r][e], acc[g][e]);
        }
        l[g] = lsum;
        m[g] = m_new;
      }
    }
  }

  // merge the 4 row groups of the wave
#pragma unroll
  for (int off = 16; off <= 32; off <<= 1) {
#pragma unroll
    for (int g = 0; g < GC; ++g) {
      const float m_o = __shfl_xor(m[g], off, MF_WAVE);
      const float l_o = __shfl_xor(l[g], off, MF_WAVE);
      const float m_new = fmaxf(m[g], m_o);
      const float c1 = (m_new == -INFINITY) ? 0.f : exp_for<T>(m[g] - m_new);
      const float c2 = (m_new == -INFINITY) ? 0.f : exp_for<T>(m_o - m_new);
      l[g] = l[g] * c1 + l_o * c2;
#pragma unroll
      for (int e = 0; e < EPL; ++e) {
        const float a_o = __shfl_xor(acc[g][e], off, MF_WAVE);
        acc[g][e] = acc[g][e] * c1 + a_o * c2;
      }
      m[g] = m_new;
    }
  }
  if (rg == 0) {
#pragma unroll
    for (int g = 0; g < GC; ++g) {
#pragma unroll
      for (int e = 0; e < EPL; ++e) sm_acc[w][g][sub * EPL + e] = acc[g][e];
      if (sub == 0) { sm_ml[w][g][0] = m[g]; sm_ml[w][g][1] = l[g]; }
    }
  }
  __syncthreads();

  // merge the 4 waves: thread (g, sub) for the first GC*16 threads
  const int g = threadIdx.x >> 4;
  if (g >= gcount) return;
  const int fsub = threadIdx.x & 15;
  float mm = -INFINITY;
#pragma unroll
  for (int ww = 0; ww < 4; ++ww) mm = fmaxf(mm, sm_ml[ww][g][0]);
  float c[4], L = 0.f;
#pragma unroll
  for (int ww = 0; ww < 4; ++ww) {
    c[ww] = (mm == -INFINITY) ? 0.f : exp_for<T>(sm_ml[ww][g][0] - mm);
    L += sm_ml[ww][g][1] * c[ww];
  }
  const int h = h0 + g;
  if (n_splits == 1) {
    T* o = out + ((size_t)t * nh + h) * HD + fsub * EPL;
    const float inv = L > 0.f ? 1.0f / L : 0.f;
#pragma unroll
    for (int e = 0; e < EPL; ++e) {
      float a = 0.f;
#pragma unroll
      for (int ww = 0; ww < 4; ++ww) a += sm_acc[ww][g][fsub * EPL + e] * c[ww];
      o[e] = from_f32<T>(a * inv);
    }
  } else {
    float* o = part + (((size_t)t * nh + h) * n_splits + split) * (HD + 2);
#pragma unroll
    for (int e = 0; e < EPL; ++e) {
      float a = 0.f;
#pragma unroll
      for (int ww = 0; ww < 4; ++ww) a += sm_acc[ww][g][fsub * EPL + e] * c[ww];
      o[fsub * EPL + e] = a;
    }
    if (fsub == 0) { o[HD] = mm; o[HD + 1] = L; }
  }
}

// out[t][h][:] = sum_s acc_s exp(m_s - M) / sum_s l_s exp(m_s - M); at most 64 splits.
// One block per (token, head), a thread per element of the head (64 ceil(hd / 64) threads): in
// every wave lane s weighs split s, for itself, so the waves need nothing from each other; then a
// thread adds its element's weighted sums one after another, in the order of the splits.
template <typename T>
__global__ __launch_bounds__(256) void attn_combine_kernel(const float* __restrict__ part,
                                                           T* __restrict__ out, int hd, int n_splits) {
  const size_t th = blockIdx.x;   // t * nh + h
  const float* base = part + th * n_splits * (hd + 2);
  const int lane = threadIdx.x & 63, d = threadIdx.x;
  const float ms = lane < n_splits ? base[(size_t)lane * (hd + 2) + hd] : -INFINITY;
  const float ls = lane < n_splits ? base[(size_t)lane * (hd + 2) + hd + 1] : 0.f;
  const float mm = wave_max(ms);
  const float wv = (ms == -INFINITY) ? 0.f : exp_for<T>(ms - mm);
  // the splits behind the last one with keys (places a token does not use) are not read at all
  const unsigned long long with_keys = __ballot(ms != -INFINITY);
  const int n_used = with_keys ? 64 - __clzll((long long)with_keys) : 0;
  auto of_split = [](float x, int s) { return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(x), s)); };
  float L = 0.f;
  for (int s = 0; s < n_used; ++s) L += of_split(ls, s) * of_split(wv, s);
  const float inv = L > 0.f ? 1.0f / L : 0.f;
  if (d >= hd) return;
  // Eight splits a round (sixteen where there are more than eight), their loads in flight together:
  // a round that is not full, left to a plain loop, would run split by split, a trip to memory
  // each.  Weight 0: a split without keys, whose sums nobody wrote, or one behind the last; its
  // load goes to the first split's line instead and counts as 0.
  auto rounds = [&](auto WIDTH) {
    constexpr int W = decltype(WIDTH)::value;
    float a = 0.f;
    for (int s0 = 0; s0 < n_used; s0 += W) {
      float w[W], v[W];
#pragma unroll
      for (int j = 0; j < W; ++j) {
        w[j] = s0 + j < 64 ? of_split(wv, s0 + j) : 0.f;
        v[j] = base[(w[j] != 0.f ? (size_t)(s0 + j) * (hd + 2) : 0) + d];
      }
#pragma unroll
      for (int j = 0; j < W; ++j) a += (w[j] != 0.f ? v[j] : 0.f) * w[j];
    }
    return a;
  };
  const float a = n_used <= 8 ? rounds(std::integral_constant<int, 8>{}) : rounds(std::integral_constant<int, 16>{});
  out[th * hd + d] = from_f32<T>(a * inv);
}

template <typename T, int EPL>
int launch_one(const T* q, const T* kc, const T* vc, const int* page_table, int pt_stride,
               const int* positions, const int* seq_of_tok, T* out, float* part, int n_tok, int nh,
               int nk, float scale, int window, int n_splits, int split_len, hipStream_t stream) {
  constexpr int GC = Chunk<EPL>::GC;
  const int G = nh / nk;
  dim3 grid(n_tok, nk * ((G + GC - 1) / GC), n_splits);
  attn_tokens_kernel<T, EPL><<<grid, 256, 0, stream>>>(q, kc, vc, page_table, pt_stride, positions,
                                                       seq_of_tok, out, part, nh, nk, scale, window,
                                                       n_splits, split_len);
  int rc = mf_launch_status();
  if (rc == 0 && n_splits > 1) {
    attn_combine_kernel<T><<<n_tok * nh, 64 * ((16 * EPL + 63) / 64), 0, stream>>>(part, out, 16 * EPL, n_splits);
    rc = mf_launch_status();
  }
  return rc;
}

template <typename T>
int launch(const void* q, const void* kc, const void* vc, const int* page_table, int pt_stride,
           const int* positions, const int* seq_of_tok, void* out, float* part, int n_tok, int nh,
           int nk, int hd, float scale, int window, int n_splits, int split_len, hipStream_t stream) {
  if (n_tok <= 0) return 0;
  if (hd % 16 != 0 || hd < 16 || hd > 256 || nk <= 0 || nh % nk != 0 || n_splits < 1 || n_splits > 64 ||
      split_len < MF_PAGE || split_len % MF_PAGE != 0 || (n_splits > 1 && part == nullptr))
    return (int)hipErrorInvalidValue;
#define MF_CASE(E)                                                                                  \
  case E:                                                                                           \
    return launch_one<T, E>((const T*)q, (const T*)kc, (const T*)vc, page_table, pt_stride,         \
                            positions, seq_of_tok, (T*)out, part, n_tok, nh, nk, scale, window,     \
                            n_splits, split_len, stream);
  switch (hd / 16) {
    MF_CASE(1) MF_CASE(2) MF_CASE(3) MF_CASE(4) MF_CASE(5) MF_CASE(6) MF_CASE(7) MF_CASE(8)
    MF_CASE(9) MF_CASE(10) MF_CASE(11) MF_CASE(12) MF_CASE(13) MF_CASE(14) MF_CASE(15) MF_CASE(16)
  }
#undef MF_CASE
  return (int)hipErrorInvalidValue;
}

}  // namespace attn_tokens
