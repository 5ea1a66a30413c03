// Attention of single query tokens over the paged cache in bfloat16 on the gfx950 matrix
// cores (decode), split along the keys.
//
// For a query token t of sequence b at position p and kv head hk, the G = nh/nk query heads
// of the group read the same keys: cache rows j with lo <= j <= p, lo = 0 or p - window + 1.
// s_j = dot(q, K_j) * scale; softmax over j; o = sum_j p_j V_j (src/graph/cpu_backend.rs:
// 437-494 of yusiwen/minfer; the causal rule "rows 0..=pos" is its `vl = pos + 1`, :462).
// The softmax is the online form of the reference's CUDA kernel (running max, running sum,
// rescaled accumulator, src/cuda_kernels.cu:673-790), in 32-bit; probabilities are rounded to
// bfloat16 for the second product, as in the prompt kernel.
//
// The heads of a group share every key, so up to 16 of them are the second matrix of one
// product: a wave takes 32 keys at a time and computes, with 16x16x32 MFMAs,
//   S^T[key][head] = K Q^T      A = K rows straight from the cache, B = Q held in registers
//   O^T[col][head] += V^T P^T   A = V^T rows straight from the cache, B = P^T
// The cache keeps V transposed inside a page in bfloat16, in two halves of 32 keys
// ([2][head_dim][32 keys]), so V^T rows are contiguous over the keys of a step like K rows are
// over head_dim, the 16 rows a load takes are one contiguous kilobyte (whole 128-byte lines: what
// a CU can have in flight is counted in lines, and rows of 64 keys would ask for half of each),
// and neither operand passes through LDS.  In both results a lane owns one head (lane % 16): the softmax statistics are
// per-lane scalars, and the scores a lane holds (8 consecutive keys, by the choice of which
// key each K row of a tile is) are exactly the 8 k-slots of its B operand in the second
// product, so P never leaves its registers.
//
// A block is (token, kv head, chunk of 16 heads, key split); its 4 waves take the 32-key steps
// of the split in turn and merge through LDS.  The split length follows the token's own
// length, so every split has work.  With several splits each block writes an unnormalised
// partial (acc, max, sum) and attn_combine_kernel merges them in a fixed order.
#include "attn_tokens_impl.h"
#include "noalloc.h"

namespace {

constexpr int STEP = 32;       // keys per wave step
static_assert(STEP * 2 == MF_PAGE, "a step is one half of a page of V");

// ROPE: the step's q|k|v come as the 32-bit output of their product, [(nh + 2 nk) hd] per token,
// not yet rotated and not yet in the cache.  The kernel rotates q on the way into its operand
// (half-split pairs i, i + hd/2; x0' = x0 c - x1 s, x1' = x0 s + x1 c; src/graph/
// cpu_backend.rs:421-431), and the blocks of the last split, which holds the token's own
// position, rotate k, take v, put both into their operands in place of what the cache row
// holds, and (one block per kv head, when write_kv) store them into the cache for later
// steps: no rotation kernel and no q buffer between the product and the attention.
struct RopeArgs {
  const float* qkv;      // [n_tok][(nh + 2 nk) hd]
  const float* cs;       // [positions][hd / 2]
  const float* sn;
  int write_kv;
};

// 8 rotated elements d .. d + 7 of one head (src, hd floats) at position pos
template <int HD>
__device__ __forceinline__ bf16x8 rotated8(const float* __restrict__ src, const float* __restrict__ cs,
                                           const float* __restrict__ sn, int pos, int d) {
  constexpr int HALF = HD / 2;
  const bool upper = d >= HALF;
  const int i = upper ? d - HALF : d;               // index into the table and of the lower partner
  const float4 a0 = *reinterpret_cast<const float4*>(src + i), a1 = *reinterpret_cast<const float4*>(src + i + 4);
  const float4 b0 = *reinterpret_cast<const float4*>(src + i + HALF);
  const float4 b1 = *reinterpret_cast<const float4*>(src + i + HALF + 4);
  const float4 c0 = *reinterpret_cast<const float4*>(cs + (size_t)pos * HALF + i);
  const float4 c1 = *reinterpret_cast<const float4*>(cs + (size_t)pos * HALF + i + 4);
  const float4 s0 = *reinterpret_cast<const float4*>(sn + (size_t)pos * HALF + i);
  const float4 s1 = *reinterpret_cast<const float4*>(sn + (size_t)pos * HALF + i + 4);
  const float x0[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
  const float x1[8] = {b0.x, b0.y, b0.z, b0.w, b1.x, b1.y, b1.z, b1.w};
  const float c[8] = {c0.x, c0.y, c0.z, c0.w, c1.x, c1.y, c1.z, c1.w};
  const float sv[8] = {s0.x, s0.y, s0.z, s0.w, s1.x, s1.y, s1.z, s1.w};
  bf16x8 r;
#pragma unroll
  for (int e = 0; e < 8; ++e) r[e] = (bf16)(upper ? x0[e] * sv[e] + x1[e] * c[e] : x0[e] * c[e] - x1[e] * sv[e]);
  return r;
}

template <int HD, bool ROPE>
__global__ __launch_bounds__(256) void attn_decode_kernel(
    const bf16* __restrict__ q, bf16* kc, bf16* vt,
    const int* __restrict__ page_table, int pt_stride, const int* __restrict__ positions,
    const int* __restrict__ seq_of_tok, bf16* __restrict__ out, float* __restrict__ part, int n_tok, int nh, int nk,
    float scale, int window, int n_splits, int base_splits, RopeArgs rope) {
  constexpr int KS = (HD + 31) / 32;      // 32-wide steps over head_dim in the first product
  constexpr int CT = HD / 16;             // 16-wide column tiles of the output
  constexpr int O_LD = HD + 4;
  __shared__ float sm_o[4][16][O_LD];
  __shared__ float sm_ml[4][16][2];

  const int lane = threadIdx.x & 63;
  const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r16 = lane & 15, q4 = lane >> 4;
  const int G = nh / nk;
  const int n_gc = (G + 15) / 16;
  // Which token, group of heads and split this block has, and how many splits the token's keys go
  // over (`active`, at most its n_splits places in `part`).
  int t, hg, split, active, p;
  if (base_splits == 0) {
    // Every token has n_splits splits.  Blocks are numbered with the split running fastest, then
    // the group of heads, then the token: consecutive blocks go to consecutive dies, so a
    // sequence's splits are dealt over all of them (with the token running fastest and 8 sequences
    // on 8 dies every die had one sequence to itself).
    split = blockIdx.x % n_splits;
    hg = (blockIdx.x / n_splits) % (nk * n_gc);
    t = blockIdx.x / (n_splits * nk * n_gc);
    active = n_splits;
    p = positions[t];
  } else {
    // The step's tokens (at most 64) share n_tok * base_splits splits, as many blocks per group of
    // heads as without sharing (one per CU is what the plan aims at; a block more on some CUs
    // would double their time): one split each, and the rest in proportion to their keys (token
    // i's part ends where the keys up to and with its own end on that scale, rounded down), so
    // that blocks have about equal work whatever the lengths: a step is as long as its longest
    // block.  Blocks are numbered through the tokens' splits one after the other; every wave works
    // the shares out for itself, lane i for token i, in integers, so all blocks of a launch agree.
    const int nb = n_tok * base_splits;
    const int b = blockIdx.x % nb;
    hg = blockIdx.x / nb;
    const int p_i = lane < n_tok ? positions[lane] : 0;
    const int len_i = lane < n_tok ? (window > 0 ? min(p_i + 1, window) : p_i + 1) : 0;
    long long keys = len_i;                // of the tokens up to and with lane's
    for (int o = 1; o < n_tok; o <<= 1) {
      const long long v = __shfl_up(keys, o, MF_WAVE);
      if (lane >= o) keys += v;
    }
    const long long total = __shfl(keys, n_tok - 1, MF_WAVE);
    const int end_i = (int)(keys * (nb - n_tok) / total);
    const int begin_i = __shfl_up(end_i, 1, MF_WAVE);
    const int s_i = lane < n_tok ? min(n_splits, 1 + end_i - (lane ? begin_i : 0)) : 0;
    int behind = s_i;                      // splits of the tokens up to and with lane's
    for (int o = 1; o < n_tok; o <<= 1) {
      const int v = __shfl_up(behind, o, MF_WAVE);
      if (lane >= o) behind += v;
    }
    const unsigned long long mine = __ballot(b >= behind - s_i && b < behind);
    if (mine == 0) return;                 // a block beyond the shares (a token whose share its places cut)
    t = __ffsll((long long)mine) - 1;
    split = __builtin_amdgcn_readfirstlane(b - (__shfl(behind, t, MF_WAVE) - __shfl(s_i, t, MF_WAVE)));
    active = __builtin_amdgcn_readfirstlane(__shfl(s_i, t, MF_WAVE));
    p = __builtin_amdgcn_readfirstlane(__shfl(p_i, t, MF_WAVE));
  }
  const int hk = hg / n_gc;
  const int g0 = (hg % n_gc) * 16;
  const int gcount = min(16, G - g0);
  const int h0 = hk * G + g0;

  const int* pt = page_table + (size_t)seq_of_tok[t] * pt_stride;
  const int lo = window > 0 ? max(0, p - window + 1) : 0;
  if (split == 0 && active < n_splits) {
    // the places this token leaves unused say "nothing here" (maximum -inf, sum 0; the merge reads
    // no further)
    for (int i = threadIdx.x; i < (n_splits - active) * gcount; i += 256) {
      float* o = part + (((size_t)t * nh + h0 + i % gcount) * n_splits + active + i / gcount) * (HD + 2);
      o[HD] = -INFINITY;
      o[HD + 1] = 0.f;
    }
  }
  // split length: this token's keys over its splits, in whole block rounds of 4 steps
  const int per = (p + 1 - lo + active - 1) / active;
  const int split_len = (per + 4 * STEP - 1) / (4 * STEP) * (4 * STEP);
  const int j_begin = lo + split * split_len;
  const int j_end = min(p + 1, j_begin + split_len);
  if (j_begin >= j_end) {
    // A split past the token's keys (a short sequence under a split count made for long ones):
    // the same mark, and the block is done.
    for (int g = threadIdx.x; g < gcount; g += 256) {
      float* o = part + (((size_t)t * nh + h0 + g) * n_splits + split) * (HD + 2);
      o[HD] = -INFINITY;
      o[HD + 1] = 0.f;
    }
    return;
  }

  // B operand of the first product: row = head r16, 8 elements of head_dim at 32 ks + 8 q4.
  // ROPE: the block rotates its 16 heads once, one 8-element chunk per thread, into LDS.
  __shared__ __attribute__((aligned(16))) bf16 sm_q[ROPE ? 16 * KS * 32 : 8];
  if constexpr (ROPE) {
    for (int c = threadIdx.x; c < 16 * KS * 4; c += 256) {
      const int head = c / (KS * 4), d = (c % (KS * 4)) * 8;
      bf16x8 q8 = bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
      if (head < gcount && d < HD)
        q8 = rotated8<HD>(rope.qkv + ((size_t)t * (nh + 2 * nk) + h0 + head) * HD, rope.cs, rope.sn, p, d);
      *reinterpret_cast<bf16x8*>(&sm_q[head * KS * 32 + d]) = q8;
    }
  }
  // ROPE: the token's own key and value, for the blocks whose split ends at its position:
  // rotated (k) and rounded once here, kept in LDS until the step that holds position p.
  // Key p is row `krow + 4 a` of tile a in its step for exactly one a, in the four lanes of one
  // r16; value p is element p % 8 of the lanes with q4 = (p % 32) / 8.
  const int krow = 8 * (r16 >> 2) + (r16 & 3);
  const bool own_split = ROPE && rope.write_kv && j_end == p + 1 && j_begin <= p;
  const int po = p % STEP;
  const int own_a = (po - krow) >> 2;                      // 0 or 1 where this lane holds key p
  const bool own_k = own_split && (po - krow == 0 || po - krow == 4);
  const bool own_v = own_split && q4 == (po >> 3);
  __shared__ __attribute__((aligned(16))) bf16 sm_k[ROPE ? KS * 32 : 8];
  __shared__ bf16 sm_v[ROPE ? HD : 8];
  if constexpr (ROPE) {
    if (own_split) {
      const int tid = threadIdx.x;
      const float* row = rope.qkv + (size_t)t * (nh + 2 * nk) * HD;
      const bool store = g0 == 0;                          // one block per kv head fills the cache
      const int page = pt[p / MF_PAGE];
      if (tid < KS * 4) {
        bf16x8 k8 = bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
        if (tid * 8 < HD) {
          k8 = rotated8<HD>(row + (size_t)(nh + hk) * HD, rope.cs, rope.sn, p, tid * 8);
          if (store)
            *reinterpret_cast<bf16x8*>(kc + (((size_t)page * nk + hk) * MF_PAGE + p % MF_PAGE) * HD + tid * 8) = k8;
        }
        *reinterpret_cast<bf16x8*>(&sm_k[tid * 8]) = k8;
      }
      for (int d = tid; d < HD; d += 256) {
        const bf16 v = (bf16)row[(size_t)(nh + nk + hk) * HD + d];
        sm_v[d] = v;
        if (store)
          vt[((((size_t)page * nk + hk) * 2 + (p % MF_PAGE) / STEP) * HD + d) * STEP + p % STEP] = v;
      }
    }
    __syncthreads();
  }
  bf16x8 qf[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    const int d = ks * 32 + q4 * 8;
    if constexpr (ROPE) {
      qf[ks] = *reinterpret_cast<const bf16x8*>(&sm_q[r16 * KS * 32 + d]);
    } else {
      qf[ks] = bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
      if (r16 < gcount && d < HD) qf[ks] = *reinterpret_cast<const bf16x8*>(q + ((size_t)t * nh + h0 + r16) * HD + d);
    }
  }

  floatx4 oacc[CT];                       // O^T: head r16, columns 16 c + 4 q4 + r
#pragma unroll
  for (int c = 0; c < CT; ++c) oacc[c] = floatx4{0.f, 0.f, 0.f, 0.f};
  float m_run = -INFINITY, l_run = 0.f;   // of head r16 (the same in the four lanes that share it)

  // Steps are 32-key blocks of the cache, so a step lies in one page.  Row r16 of K tile a is
  // key 8 (r16 / 4) + 4 a + r16 % 4 of the step: the scores of lane (r16, q4) then belong to
  // keys 8 q4 + 4 a + r, r = 0..3, eight consecutive keys over the two tiles.
  const int step0 = j_begin / STEP;
  const int n_steps = j_begin < j_end ? (j_end - 1) / STEP - step0 + 1 : 0;
  bf16x8 kn[2][KS], vn[CT];
  // The page of a step is looked up a whole step before its keys are asked for, so that the
  // look-up's latency does not stand in front of every step's loads.  One step in flight per wave
  // is enough: with two, at twice the registers, nothing was faster.
  auto page_of = [&](int i) { return pt[(step0 + i) * STEP / MF_PAGE]; };
  auto issue = [&](int i, int page) {
    const int jb = (step0 + i) * STEP;
    const int off = jb % MF_PAGE;
    const bf16* kp = kc + (((size_t)page * nk + hk) * MF_PAGE + off + krow) * HD + q4 * 8;
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        kn[a][ks] = bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
        if (ks * 32 + q4 * 8 < HD) kn[a][ks] = *reinterpret_cast<const bf16x8*>(kp + (size_t)(4 * a) * HD + ks * 32);
      }
    const bf16* vp = vt + ((((size_t)page * nk + hk) * 2 + off / STEP) * HD + r16) * STEP + q4 * 8;
#pragma unroll
    for (int c = 0; c < CT; ++c) vn[c] = *reinterpret_cast<const bf16x8*>(vp + (size_t)(16 * c) * STEP);
  };
  int page_ahead = 0;                    // of the step after the one in flight
  if (w < n_steps) {
    const int page_first = page_of(w);
    if (w + 4 < n_steps) page_ahead = page_of(w + 4);
    issue(w, page_first);
  }
  for (int i = w; i < n_steps; i += 4) {
    bf16x8 kf[2][KS], vf[CT];
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) kf[a][ks] = kn[a][ks];
#pragma unroll
    for (int c = 0; c < CT; ++c) vf[c] = vn[c];
    if (i + 4 < n_steps) issue(i + 4, page_ahead);
    if (i + 8 < n_steps) page_ahead = page_of(i + 8);

    const int jb = (step0 + i) * STEP;
    const int key0 = jb + 8 * q4;                  // this lane's eight keys: key0 .. key0 + 7
    const bool edge = jb < j_begin || jb + STEP > j_end;
    if constexpr (ROPE) {
      if (own_split && jb + po == p) {             // the step of the token's own position
        if (own_k) {
#pragma unroll
          for (int ks = 0; ks < KS; ++ks) {
            const bf16x8 k8 = *reinterpret_cast<const bf16x8*>(&sm_k[ks * 32 + q4 * 8]);
            if (own_a == 0) kf[0][ks] = k8;
            else kf[1][ks] = k8;
          }
        }
        if (own_v) {
#pragma unroll
          for (int c = 0; c < CT; ++c) {
            const bf16 v = sm_v[16 * c + r16];
#pragma unroll
            for (int e = 0; e < 8; ++e)
              if (e == (po & 7)) vf[c][e] = v;
          }
        }
      }
    }
    if (edge) {
      // Keys outside the split are masked out of P below, but their V may never have been
      // written (a page is not cleared when it is taken) and 0 * garbage could be NaN:
      // they enter as zeros.
#pragma unroll
      for (int c = 0; c < CT; ++c)
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (key0 + e < j_begin || key0 + e >= j_end) vf[c][e] = (bf16)0.f;
    }
    floatx4 s[2];
#pragma unroll
    for (int a = 0; a < 2; ++a) {
      s[a] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
        s[a] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[a][ks], qf[ks], s[a], 0, 0, 0);
    }
    float sc[8];
    float mx = -INFINITY;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int j = key0 + e;
      const float v = s[e >> 2][e & 3] * scale;
      sc[e] = (!edge || (j >= j_begin && j < j_end)) ? v : -INFINITY;
      mx = fmaxf(mx, sc[e]);
    }
    mx = fmaxf(mx, __shfl_xor(mx, 16, MF_WAVE));
    mx = fmaxf(mx, __shfl_xor(mx, 32, MF_WAVE));
    const float m_new = fmaxf(m_run, mx);
    const float corr = (m_new == -INFINITY) ? 1.f : __expf(m_run - m_new);
    float lsum = 0.f;
    bf16x8 pf;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float pe = (sc[e] == -INFINITY) ? 0.f : __expf(sc[e] - m_new);
      lsum += pe;
      pf[e] = (bf16)pe;
    }
    lsum += __shfl_xor(lsum, 16, MF_WAVE);
    lsum += __shfl_xor(lsum, 32, MF_WAVE);
    l_run = l_run * corr + lsum;
    m_run = m_new;
#pragma unroll
    for (int c = 0; c < CT; ++c) {
#pragma unroll
      for (int r = 0; r < 4; ++r) oacc[c][r] *= corr;
      oacc[c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[c], pf, oacc[c], 0, 0, 0);
    }
  }

  // merge the 4 waves
#pragma unroll
  for (int c = 0; c < CT; ++c)
    *reinterpret_cast<floatx4*>(&sm_o[w][r16][16 * c + 4 * q4]) = oacc[c];
  if (q4 == 0) { sm_ml[w][r16][0] = m_run; sm_ml[w][r16][1] = l_run; }
  __syncthreads();
  // thread -> (head g, 16 threads over the columns)
  const int g = threadIdx.x >> 4;
  if (g >= gcount) return;
  const int sub = threadIdx.x & 15;
  float mm = -INFINITY;
#pragma unroll
  for (int ww = 0; ww < 4; ++ww) mm = fmaxf(mm, sm_ml[ww][g][0]);
  float cw[4], L = 0.f;
#pragma unroll
  for (int ww = 0; ww < 4; ++ww) {
    cw[ww] = (mm == -INFINITY) ? 0.f : __expf(sm_ml[ww][g][0] - mm);
    L += sm_ml[ww][g][1] * cw[ww];
  }
  const int h = h0 + g;
  if (n_splits == 1) {
    bf16* o = out + ((size_t)t * nh + h) * HD;
    const float inv = L > 0.f ? 1.0f / L : 0.f;
    for (int d = sub; d < HD; d += 16) {
      float a = 0.f;
#pragma unroll
      for (int ww = 0; ww < 4; ++ww) a += sm_o[ww][g][d] * cw[ww];
      o[d] = (bf16)(a * inv);
    }
  } else {
    float* o = part + (((size_t)t * nh + h) * n_splits + split) * (HD + 2);
    for (int d = sub; d < HD; d += 16) {
      float a = 0.f;
#pragma unroll
      for (int ww = 0; ww < 4; ++ww) a += sm_o[ww][g][d] * cw[ww];
      o[d] = a;
    }
    if (sub == 0) { o[HD] = mm; o[HD + 1] = L; }
  }
}

template <int HD>
int launch(const bf16* q, bf16* kc, bf16* vt, const int* page_table, int pt_stride, const int* positions,
           const int* seq_of_tok, bf16* out, float* part, int n_tok, int nh, int nk, float scale, int window,
           int n_splits, int base_splits, const RopeArgs* rope, hipStream_t stream) {
  const int G = nh / nk;
  const long blocks = (long)n_tok * nk * ((G + 15) / 16) * (base_splits ? base_splits : n_splits);
  if (blocks > 0x7fffffffL) return (int)hipErrorInvalidValue;
  dim3 grid((unsigned)blocks);
  if (rope)
    attn_decode_kernel<HD, true><<<grid, 256, 0, stream>>>(q, kc, vt, page_table, pt_stride, positions, seq_of_tok,
                                                           out, part, n_tok, nh, nk, scale, window, n_splits,
                                                           base_splits, *rope);
  else
    attn_decode_kernel<HD, false><<<grid, 256, 0, stream>>>(q, kc, vt, page_table, pt_stride, positions,
                                                            seq_of_tok, out, part, n_tok, nh, nk, scale, window,
                                                            n_splits, base_splits,
                                                            RopeArgs{nullptr, nullptr, nullptr, 0});
  int rc = mf_launch_status();
  if (rc == 0 && n_splits > 1) {
    attn_tokens::attn_combine_kernel<bf16><<<n_tok * nh, 64 * ((HD + 63) / 64), 0, stream>>>(part, out, HD, n_splits);
    rc = mf_launch_status();
  }
  return rc;
}

int dispatch(const void* q, void* kc, void* vt, const int* page_table, int pt_stride, const int* positions,
             const int* seq_of_tok, void* out, float* part, int n_tok, int nh, int nk, int hd, float scale,
             int window, int n_splits, int base_splits, const RopeArgs* rope, hipStream_t stream) {
  if (n_tok <= 0) return 0;
  if (base_splits == n_splits) base_splits = 0;       // nothing to share out
  if (hd % 16 != 0 || hd < 16 || hd > 256 || nk <= 0 || nh % nk != 0 || n_splits < 1 || n_splits > 64 ||
      (n_splits > 1 && part == nullptr) || base_splits < 0 || base_splits > n_splits || (base_splits && n_tok > 64))
    return (int)hipErrorInvalidValue;
#define MF_CASE(E)                                                                                          \
  case E:                                                                                                   \
    return launch<16 * E>((const bf16*)q, (bf16*)kc, (bf16*)vt, page_table, pt_stride, positions,           \
                          seq_of_tok, (bf16*)out, part, n_tok, nh, nk, scale, window, n_splits,    \
                          base_splits, rope, stream);
  switch (hd / 16) {
    MF_CASE(1) MF_CASE(2) MF_CASE(3) MF_CASE(4) MF_CASE(5) MF_CASE(6) MF_CASE(7) MF_CASE(8)
    MF_CASE(9) MF_CASE(10) MF_CASE(11) MF_CASE(12) MF_CASE(13) MF_CASE(14) MF_CASE(15) MF_CASE(16)
  }
#undef MF_CASE
  return (int)hipErrorInvalidValue;
}

}  // namespace

// q, out: [n_tok][nh][hd]; kc: [pages][nk][64][hd]; vt: [pages][nk][2][hd][32] (V transposed inside
// a page, in two halves of 32 keys); part: n_tok * nh * n_splits * (hd + 2) floats when n_splits > 1 (at most 64 splits).
// base_splits: 0 or n_splits: every token's keys go over n_splits splits; a number below n_splits
// (and at most 64 tokens): the step's tokens share n_tok * base_splits splits, one each and the
// rest in proportion to their keys, none taking more than n_splits (the places it leaves unused
// are marked empty), so that a long sequence among short ones does not make the step as long as
// its own n_splits-th.
MF_API int mf_attn_decode_bf16(const void* q, const void* kc, const void* vt, const int* page_table,
                               int pt_stride, const int* positions, const int* seq_of_tok, void* out,
                               float* part, int n_tok, int nh, int nk, int hd, float scale, int window,
                               int n_splits, int base_splits, hipStream_t stream) {
  return dispatch(q, const_cast<void*>(kc), const_cast<void*>(vt), page_table, pt_stride, positions, seq_of_tok,
                  out, part, n_tok, nh, nk, hd, scale, window, n_splits, base_splits, nullptr, stream);
}

// The same with the rotation and the cache write of the step's own q|k|v folded in: qkv is the
// 32-bit [n_tok][(nh + 2 nk) hd] output of their product, cs/sn the [positions][hd / 2] tables.
// Each token must be the last position of its sequence (a decode step); hd must be a multiple
// of 16 so that 8-element chunks do not straddle the half.  With write_kv = 0 nothing is
// stored and k, v come from the cache (a layer that reads another layer's cache).
MF_API int mf_attn_decode_rope_bf16(const float* qkv, const float* cs, const float* sn, void* kc, void* vt,
                                    const int* page_table, int pt_stride, const int* positions,
                                    const int* seq_of_tok, void* out, float* part, int n_tok, int nh, int nk,
                                    int hd, float scale, int window, int n_splits, int base_splits, int write_kv,
                                    hipStream_t stream) {
  const RopeArgs rope{qkv, cs, sn, write_kv};
  return dispatch(nullptr, kc, vt, page_table, pt_stride, positions, seq_of_tok, out, part, n_tok, nh, nk, hd,
                  scale, window, n_splits, base_splits, &rope, stream);
}

// ------------------------------------------------------------------ the entry point that allocates nothing
// (see noalloc.h)
namespace {

// The partials of the key splits.  In host code this name is only a handle for the runtime: the
// memory's address on a device comes from hipGetSymbolAddress, once per device, below.
static __device__ __align__(256) float scratch[MF_NOALLOC_SCRATCH_FLOATS];

constexpr int MAX_DEVICES = 64;
float* scratch_on_device[MAX_DEVICES] = {};      // each GPU holds its own copy of the array, at its own address

// the array's address on the current device; nullptr and `rc` set on failure
float* scratch_address(int* rc) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) { *rc = (int)e; return nullptr; }
  if (dev < 0 || dev >= MAX_DEVICES) { *rc = (int)hipErrorInvalidDevice; return nullptr; }
  float* p = __atomic_load_n(&scratch_on_device[dev], __ATOMIC_ACQUIRE);
  if (p) return p;
  void* addr = nullptr;
  e = hipGetSymbolAddress(&addr, HIP_SYMBOL(scratch));
  if (e != hipSuccess || !addr) { *rc = e != hipSuccess ? (int)e : (int)hipErrorUnknown; return nullptr; }
  p = (float*)addr;
  __atomic_store_n(&scratch_on_device[dev], p, __ATOMIC_RELEASE);    // two first calls at once store the same address
  return p;
}

}  // namespace

MF_API size_t mf_attn_decode_bf16_noalloc_capacity(void) { return MF_NOALLOC_SCRATCH_FLOATS; }

MF_API int mf_attn_decode_bf16_noalloc(const void* q, const void* kc, const void* vt, const int* page_table,
                                       int pt_stride, const int* positions, const int* seq_of_tok, void* out,
                                       int n_tok, int nh, int nk, int hd, float scale, int window, int n_splits,
                                       hipStream_t stream) {
  if (n_tok <= 0) return 0;
  if (n_splits < 1 || n_splits > 64 || nh <= 0 || hd <= 0) return (int)hipErrorInvalidValue;
  float* part = nullptr;
  if (n_splits > 1) {
    const size_t need = (size_t)n_tok * (size_t)nh * (size_t)n_splits * (size_t)(hd + 2);
    if (need > MF_NOALLOC_SCRATCH_FLOATS) return MF_NOALLOC_TOO_LARGE;
    int rc = 0;
    part = scratch_address(&rc);
    if (!part) return rc;
  }
  return dispatch(q, const_cast<void*>(kc), const_cast<void*>(vt), page_table, pt_stride, positions, seq_of_tok,
                  out, part, n_tok, nh, nk, hd, scale, window, n_splits, 0, nullptr, stream);
}
