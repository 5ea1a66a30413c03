// Causal grouped-query attention for many query tokens per sequence (prompts), bfloat16,
// on the gfx950 matrix cores, reading keys and values from the paged cache.
//
// Semantics as the reference's attention (src/graph/cpu_backend.rs:437-494 of
// yusiwen/minfer): a query at position p sees cache rows lo..p of its own sequence
// (lo = 0, or p - window + 1), scores q.k * scale, softmax, weighted sum of v; query head h
// reads kv head h / (nh / nk).  The softmax is the online form of the reference's CUDA
// kernel (src/cuda_kernels.cu:673-790); scores, maxima, sums and the output accumulate in
// 32-bit, probabilities are rounded to bfloat16 for the second product.
//
// The query heads of a group read the same keys and values, so the rows of the problem are
// (token, head of the group) pairs: a block owns `tq` consecutive new tokens of one sequence
// times `gh` heads of one kv head (gh * tq rows, at most 32 a wave), and every page of K and V
// it brings into LDS serves all of them.  (One head a block, as a first form of this kernel had
// it, pulls every page once per head through each CU, and a CU draws only so much: at 7 heads a
// group the pages' way into the CU, not the matrix cores, set the time.)
// The time of a prompt's attention is that of its last tile, whose block walks every page of the
// sequence one after the other, so the host may give a tile to several blocks, which take its
// pages in turn (block s of n the pages first + s, first + s + n, ...): each leaves its maxima,
// sums and output in `parts`, counts itself in, and the one that comes last adds all of them up,
// in the order of s, and writes the result.
// A page (64 keys) of K and of V travels from the cache straight into LDS (global_load_lds, no
// registers in between), one or two pages ahead of the one being multiplied, one barrier a
// page.  LDS holds K as stored, [64 keys][head_dim], and V as stored, transposed in two halves
// [2][head_dim][32 keys]; the 16-byte chunks of a row sit at swizzled places so that the lanes
// of a fragment read fall on different banks (the copy's lanes pick their source chunk to suit).
//   S^T[key][row] = K Q^T    32x32x16 MFMA, A = K rows from LDS, B = Q held in registers
//   lane <-> row, so the row statistics of the softmax are per-lane scalars
//   O^T[d][row]  += V^T P^T  A = V^T from LDS, B = P^T, which is S^T's own register layout
// The k index of the second product is permuted the same way on both operands (the sum
// does not care), which is what lets P stay in registers.
#include "common.h"

namespace {

constexpr int KT = MF_PAGE;         // keys per step: one page
constexpr int LDS_MAX = 160 * 1024;

// 16 bytes per lane from base + off (a wave-uniform base and a 32-bit byte offset per lane) to
// LDS at lds_byte + 16 * lane
__device__ __forceinline__ void dma16(const bf16* base, unsigned off, unsigned lds_byte) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(off), "s"(base), "s"(lds_byte)
               : "memory", "m0");
}

// Sizes of the kernel for head_dim = 16 NKS.  Four waves, 32 rows each.  Up to a head size of 128 a
// wave keeps within 256 registers and a block within 64 KB of LDS (two pages in flight), so two
// blocks share a CU, one wave of each on every SIMD: they drift apart, and one multiplies while the
// other is at its softmax.  (Eight waves of one block, in step at the block's barrier, wait for the
// same unit at the same time; giving the two waves of a SIMD the step's halves in opposite order,
// the second product a step late, measured the same to 3 % at twice the code.)
template <int NKS>
struct Shape {
  static constexpr int HD = NKS * 16;
  static constexpr int NW = 4;
  static constexpr int ROWS = NW * 32;
  static constexpr int NDT = (NKS + 1) / 2;          // 32-wide output tiles over head_dim
  static constexpr int HDP = NDT * 32;
  static constexpr int CPR = 2 * NKS;                // 16-byte chunks of a row of K
  static constexpr bool POW2 = (CPR & (CPR - 1)) == 0;
  static constexpr int KDIV = 16 / CPR > 1 ? 16 / CPR : 1;   // rows that share a swizzle (power-of-two CPR)
  static constexpr int KBYTES = KT * HD * 2;
  // V in LDS: [2][HDP][32 keys] in groups of 16 rows (a kilobyte, one copy instruction), every other
  // group 8 bytes further on: the lanes of a fragment read take 8 bytes at the same place of rows d and
  // d + 16, which would meet in one bank.  Rows from HD on are never written nor used.
  static constexpr int VGROUP = 1024 + 16;
  static constexpr int VBYTES = 2 * (HDP / 16) * VGROUP + 16;
  static constexpr int STAGE = KBYTES + VBYTES;
  static constexpr int NI = (CPR + NW - 1) / NW;     // copies per wave and page, of K and of V each
  static constexpr bool SURPLUS = CPR % NW != 0;     // some waves' last copy has no chunk: it goes to a dump
  static constexpr int DUMP = SURPLUS ? NW * 1024 : 0;
  static constexpr int K_LD = HD + 8;                // row stride of the output staging
  static constexpr int OBYTES = NW * 32 * K_LD * 2;
  static constexpr int PER_CU = NKS <= 8 ? 2 : 1;    // blocks that share a CU
  static constexpr int NST = PER_CU == 2 ? 2 : 3 * STAGE + DUMP <= LDS_MAX ? 3 : 2;   // pages of a block in LDS
  static constexpr int SMEM = NST * STAGE + DUMP > OBYTES ? NST * STAGE + DUMP : OBYTES;
  static constexpr int XW = NDT * 16 + 2;            // values a thread leaves in `parts`
};

// chunk c of K row `row` sits at chunk c ^ kswz(row) of the row in LDS
template <int NKS>
__device__ __forceinline__ int kswz(int row) {
  using S = Shape<NKS>;
  return S::POW2 ? (row / S::KDIV) & (S::CPR - 1) : 0;
}

template <int NKS>
__global__ __launch_bounds__(Shape<NKS>::NW * 64, Shape<NKS>::PER_CU) void attn_prefill_kernel(
    const bf16* __restrict__ q, const bf16* __restrict__ kc, const bf16* __restrict__ vc,
    const int* __restrict__ page_table, int pt_stride, const int* __restrict__ cu_seqlens,
    const int* __restrict__ start_pos, const int* __restrict__ tile_seq,
    const int* __restrict__ tile_q0, const int* __restrict__ tile_share, float* __restrict__ parts,
    int* __restrict__ arrived, int max_shares, bf16* __restrict__ out, int nh, int nk, int gh, int tq,
    float scale, int window, int pair_slots) {
  using S = Shape<NKS>;
  constexpr int HD = S::HD, NW = S::NW, NT = NW * 64, NDT = S::NDT, HDP = S::HDP, CPR = S::CPR;
  constexpr int STAGE = S::STAGE, KBYTES = S::KBYTES, NI = S::NI, NST = S::NST, K_LD = S::K_LD, XW = S::XW;
  constexpr int PER = 2 * NI;                        // copies a wave has in flight per page
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const unsigned lds0 = (unsigned)(uintptr_t)smem;

  // Work items are (tile, kv head, chunk of the group's heads) with the tiles longest first (the
  // host sorts them), one block each, in this order: the longest start first and the short ones
  // fill in behind them.
  const int G = nh / nk, n_chunks = (G + gh - 1) / gh, ipt = nk * n_chunks;
  // Where all items are on the chip at once, two to a CU, nothing fills in, and what counts is
  // which two share a CU: blocks i and i + CUs do, so the second lot runs shortest first and every
  // CU gets about the same number of pages (the longest and the shortest tile together).
  int item = blockIdx.x;
  if (pair_slots > 0 && (int)gridDim.x <= 2 * pair_slots && item >= pair_slots) item = (int)gridDim.x - 1 - (item - pair_slots);
  const int tile = item / ipt, it = item % ipt;
  const int hk = it / n_chunks, chunk = it % n_chunks;
  const int h0 = hk * G + chunk * gh, ghc = min(gh, G - chunk * gh);      // this block's heads: h0 .. h0 + ghc - 1
  const int b = tile_seq[tile], q0 = tile_q0[tile];
  // tile_share[tile]: which of how many blocks of these queries this one is, and the number of the
  // queries' slot in `parts` and `arrived`: share + 256 * shares + 65536 * slot (0 shares: alone)
  const int share_word = tile_share ? tile_share[tile] : 0;
  const int share = share_word & 255, n_shares = max(1, (share_word >> 8) & 255), share_slot = share_word >> 16;
  const int tok0 = cu_seqlens[b], n_new = cu_seqlens[b + 1] - tok0, start = start_pos[b];
  const int* pt = page_table + (size_t)b * pt_stride;
  const int tid = threadIdx.x, lane = tid & 63, wid = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int ql = lane & 31, hf = lane >> 5;

  // this lane's row: token q0 + tl of the sequence's new ones, head h0 + g
  const int n_tok = min(tq, n_new - q0);                 // tokens of this tile
  const int r = wid * 32 + ql;
  const int tl = r / ghc, g = r - tl * ghc;
  const bool q_ok = tl < n_tok;
  const int pq = start + q0 + tl;                        // its position
  bf16x8 qf[NKS];
#pragma unroll
  for (int ks = 0; ks < NKS; ++ks) {
    qf[ks] = bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
    if (q_ok)
      qf[ks] = *reinterpret_cast<const bf16x8*>(q + ((size_t)(tok0 + q0 + tl) * nh + h0 + g) * HD + ks * 16 + hf * 8);
  }
  // positions this wave and this block need
  const float sl2 = scale * 1.44269504088896340736f;    // scores -> exponents of 2
  const int wave_tl_lo = (wid * 32) / ghc, wave_tl_hi = (wid * 32 + 31) / ghc;
  const bool wave_any = wave_tl_lo < n_tok;              // the wave has a row at all
  const int wave_p_lo = start + q0 + wave_tl_lo;
  const int wave_p_hi = wave_any ? start + q0 + min(wave_tl_hi, n_tok - 1) : -1;
  const int blk_p_lo = start + q0;
  const int blk_p_hi = start + q0 + n_tok - 1;
  const int key_lo = window > 0 ? max(0, blk_p_lo - window + 1) : 0;

  floatx16 oacc[NDT];
#pragma unroll
  for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
    for (int e = 0; e < 16; ++e) oacc[dt][e] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;

  // ---- the copies: copy n of this wave is instruction i = wid + NW n of the page's CPR, 64 chunks each
  unsigned koff[NI], voff[NI], kdst[NI], vdst[NI];
  bool real[NI];
#pragma unroll
  for (int n = 0; n < NI; ++n) {
    const int i = wid + NW * n;
    real[n] = !S::SURPLUS || i < CPR;
    const int ii = real[n] ? i : i % CPR;
    // K: place p = 64 ii + lane of the stage is row p / CPR, chunk position p % CPR
    const int p = 64 * ii + lane, row = p / CPR, c = (p % CPR) ^ kswz<NKS>(row);
    koff[n] = (unsigned)(row * HD + c * 8) * 2u;
    kdst[n] = real[n] ? ii * 1024 : NST * STAGE + wid * 1024;
    // V: rows (half, d) of 64 bytes, 16 an instruction; chunk position lane % 4 holds chunk (lane % 4) ^ ((d >> 2) & 3)
    const int R = 16 * ii + (lane >> 2), half = R / HD, d = R - half * HD;
    voff[n] = (unsigned)((half * HD + d) * 4 + ((lane & 3) ^ ((d >> 2) & 3))) * 16u;
    const int group = half * (HDP / 16) + (16 * ii - half * HD) / 16;
    vdst[n] = real[n] ? KBYTES + group * S::VGROUP + (group & 1) * 8 : NST * STAGE + wid * 1024;
  }
  auto issue = [&](int page, int stage) {
    const bf16* kp = kc + ((size_t)page * nk + hk) * KT * HD;
    const bf16* vp = vc + ((size_t)page * nk + hk) * HD * KT;     // a page of V is [2][HD][KT / 2]
    const unsigned base = lds0 + (unsigned)stage * STAGE;
#pragma unroll
    for (int n = 0; n < NI; ++n)
      dma16(kp, koff[n], __builtin_amdgcn_readfirstlane(real[n] ? base + kdst[n] : lds0 + kdst[n]));
#pragma unroll
    for (int n = 0; n < NI; ++n)
      dma16(vp, voff[n], __builtin_amdgcn_readfirstlane(real[n] ? base + vdst[n] : lds0 + vdst[n]));
  };
  // ---- the fragment reads
  // K: row 32 kt + ql, chunk 2 ks + hf at position (2 ks + hf) ^ kswz(row); the swizzle of row + 32 is that of row
  unsigned kaddr[NKS];
#pragma unroll
  for (int ks = 0; ks < NKS; ++ks) kaddr[ks] = (unsigned)(ql * HD * 2 + (((2 * ks + hf) ^ kswz<NKS>(ql)) * 16));
  // V^T: row d = 32 dt + ql of a half, the four keys 4 hf .. of chunk cl at position cl ^ ((ql >> 2) & 3)
  unsigned vaddr[4];
#pragma unroll
  for (int cl = 0; cl < 4; ++cl)
    vaddr[cl] = (unsigned)(KBYTES + (ql >> 4) * (S::VGROUP + 8) + ((ql & 15) * 4 + (cl ^ ((ql >> 2) & 3))) * 16 + hf * 8);

  // this block's pages: first + share, first + share + n_shares, ...
  const int page_first = key_lo / KT + share, page_last = blk_p_hi / KT;
  const int n_steps = page_first <= page_last ? (page_last - page_first) / n_shares + 1 : 0;
  for (int j = 0; j < NST - 1 && j < n_steps; ++j) issue(pt[page_first + j * n_shares], j);
  // The queries are in their registers before the loop: left to itself the compiler waits for them
  // at their first use inside it, with a count of zero on every trip (it cannot know on the way
  // back that they have long arrived), and that wait would take in the copies just set out.
#pragma unroll
  for (int ks = 0; ks < NKS; ++ks) asm volatile("" ::"v"(qf[ks]));
  int pid_next = n_steps > NST - 1 ? pt[page_first + (NST - 1) * n_shares] : 0;     // asked for a step ahead of its use

  // ---- the three parts of a step
  // The step's turn: page j has landed and is readable by all, the stage of the page that nobody
  // reads any more takes the copies of a page further on, and the last page's unwritten keys are
  // taken out of V.  Stage of page j: j % NST.
  auto turn = [&](int j) {
    // page j has landed (for this wave) when only the copies of the pages behind it are in flight
    const int behind = min(n_steps - 1 - j, NST - 2);
    if (behind <= 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(%0)" ::"n"(PER) : "memory");
    __syncthreads();          // ... for every wave; and every wave is done with the step before
    const int ahead = j + NST - 1;
    if (ahead < n_steps) {
      issue(pid_next, ahead % NST);
      if (ahead + 1 < n_steps) pid_next = pt[page_first + (ahead + 1) * n_shares];
    }
    // Keys after the block's last position were never written (a page is not cleared when it is
    // taken): they are masked out of P, but 0 * garbage could still be NaN, so their V becomes zero.
    const int n_written = blk_p_hi - (page_first + j * n_shares) * KT + 1;
    if (n_written < KT) {
      unsigned char* st = smem + (j % NST) * STAGE;
      for (int x = tid; x < 2 * HD * 4; x += NT) {
        const int cs = x & 3, R = x >> 2, half = R / HD, d = R - half * HD;
        const int k0 = half * 32 + (cs ^ ((d >> 2) & 3)) * 8;
        if (k0 + 8 > n_written) {
          const int group = half * (HDP / 16) + d / 16;
          bf16x4* at = reinterpret_cast<bf16x4*>(st + KBYTES + group * S::VGROUP + (group & 1) * 8 + ((d & 15) * 4 + cs) * 16);
          bf16x4 v0 = at[0], v1 = at[1];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            if (k0 + e >= n_written) v0[e] = (bf16)0.f;
            if (k0 + 4 + e >= n_written) v1[e] = (bf16)0.f;
          }
          at[0] = v0;
          at[1] = v1;
        }
      }
      __syncthreads();
    }
  };
  // S^T = K Q^T of page j, two tiles of 32 keys, their sums in turn; the fragments are asked for two steps ahead
  floatx16 s[2];
  auto scores = [&](int j) {
    const unsigned char* st = smem + (j % NST) * STAGE;
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int e = 0; e < 16; ++e) s[kt][e] = 0.f;
    constexpr int AHEAD = NKS < 2 ? NKS : 2;
    bf16x8 a[AHEAD + 1][2];
    auto read_k = [&](int ks, int slot) {
#pragma unroll
      for (int kt = 0; kt < 2; ++kt) a[slot][kt] = *reinterpret_cast<const bf16x8*>(st + kaddr[ks] + kt * 32 * HD * 2);
    };
#pragma unroll
    for (int ks = 0; ks < AHEAD; ++ks) read_k(ks, ks);
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) {
      if (ks + AHEAD < NKS) read_k(ks + AHEAD, (ks + AHEAD) % (AHEAD + 1));
      __builtin_amdgcn_sched_barrier(0);       // (the compiler would move every read down to its use)
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
        s[kt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[ks % (AHEAD + 1)][kt], qf[ks], s[kt], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  // Mask, running maximum, probabilities of page j from its scores: reg e of tile kt is key
  // key0 + 32 kt + 8 (e / 4) + 4 hf + e % 4.  Scores stay unscaled; the maximum is kept in units of
  // scale * log2(e), so that exp((s - m) scale) is one fused multiply-add and one 2^x per score.  A
  // page that every row of the wave sees whole needs no mask (the lanes past the block's last row
  // have zeros for a query and nobody reads their result); one that no row sees is masked whole
  // (every probability 0).
  bf16x8 pb[4];
  auto softmax = [&](int j) {
    const int key0 = (page_first + j * n_shares) * KT;
    const bool whole = key0 + KT - 1 <= wave_p_lo && (window <= 0 || key0 > wave_p_hi - window);
    if (!whole) {
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int key = key0 + kt * 32 + (e >> 2) * 8 + hf * 4 + (e & 3);
          const bool vis = q_ok && key <= pq && (window <= 0 || key > pq - window);
          s[kt][e] = vis ? s[kt][e] : -INFINITY;
        }
    }
    float s_max = -INFINITY;
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int e = 0; e < 16; ++e) s_max = fmaxf(s_max, s[kt][e]);
    float m_new = fmaxf(m_run, s_max * sl2);             // (scale > 0: the maximum of the products is the product of the maximum)
    m_new = fmaxf(m_new, __shfl_xor(m_new, 32, MF_WAVE));
    const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
    float psum = 0.f;
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const float pe = __builtin_amdgcn_exp2f(fmaf(s[kt][e], sl2, -m_use));    // 2^(-inf) = 0 for masked keys
        psum += pe;
        pb[kt * 2 + (e >> 3)][e & 7] = (bf16)pe;
      }
    // the accumulators are rescaled only when some row's maximum moved
    if (__builtin_amdgcn_ballot_w64(m_new != m_run) != 0) {
      const float corr = (m_new == -INFINITY) ? 1.f : __builtin_amdgcn_exp2f(m_run - m_new);
      l_run *= corr;
#pragma unroll
      for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
        for (int e = 0; e < 16; ++e) oacc[dt][e] *= corr;
      m_run = m_new;
    }
    l_run += psum;
  };
  // O^T += V^T P^T of page j; operand element e of group kg is key 16 kg + 8 (e / 4) + 4 hf + e % 4: two
  // runs of four keys, in chunks 2 (kg % 2) and 2 (kg % 2) + 1 of half kg / 2.  Groups of keys
  // outermost: the NDT products of a group are independent of each other.
  auto weighted = [&](int j) {
    const unsigned char* st = smem + (j % NST) * STAGE;
    constexpr int NV = 4 * NDT, VAHEAD = 2;
    bf16x4 v[VAHEAD + 1][2];
    auto read_v = [&](int i, int slot) {
      const int kg = i / NDT, dt = i % NDT;
      const unsigned char* vrow = st + ((kg >> 1) * (HDP / 16) + dt * 2) * S::VGROUP;
      v[slot][0] = *reinterpret_cast<const bf16x4*>(vrow + vaddr[2 * (kg & 1)]);
      v[slot][1] = *reinterpret_cast<const bf16x4*>(vrow + vaddr[2 * (kg & 1) + 1]);
    };
#pragma unroll
    for (int i = 0; i < VAHEAD; ++i) read_v(i, i);
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      if (i + VAHEAD < NV) read_v(i + VAHEAD, (i + VAHEAD) % (VAHEAD + 1));
      __builtin_amdgcn_sched_barrier(0);
      const bf16x4 lo4 = v[i % (VAHEAD + 1)][0], hi4 = v[i % (VAHEAD + 1)][1];
      const bf16x8 a = {lo4[0], lo4[1], lo4[2], lo4[3], hi4[0], hi4[1], hi4[2], hi4[3]};
      oacc[i % NDT] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, pb[i / NDT], oacc[i % NDT], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  for (int j = 0; j < n_steps; ++j) {
    turn(j);
    // nothing to do for this wave where every key is later than every query here, or left of every window
    const int key0 = (page_first + j * n_shares) * KT;
    if (key0 > wave_p_hi || (window > 0 && key0 + KT - 1 <= wave_p_lo - window)) continue;
    scores(j);
    softmax(j);
    weighted(j);
  }
  __syncthreads();            // every wave is past its last read of the pages: LDS is free

  if (n_shares > 1) {
    // This block's part goes to memory (lane-major: value v of thread t at v * NT + t), written
    // through and read past the caches, since the blocks of a tile may sit behind different L2s.
    float* slot0 = parts + ((size_t)share_slot * ipt + it) * max_shares * XW * NT + tid;
    float* mine = slot0 + (size_t)share * XW * NT;
    __hip_atomic_store(mine, m_run, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    __hip_atomic_store(mine + NT, l_run, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
      for (int e = 0; e < 16; ++e)
        __hip_atomic_store(mine + (2 + dt * 16 + e) * NT, oacc[dt][e], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    __builtin_amdgcn_s_waitcnt(0);                       // this wave's stores have reached memory
    __syncthreads();
    int* last = reinterpret_cast<int*>(smem);
    if (tid == 0) {
      // Counting in releases this block's part and, for the block that arrives last, acquires the
      // others': the block's stores are ordered before the increment by the barrier above (and are
      // atomic stores themselves), the increments on one counter form a release sequence, and the
      // last arriver's loads below are ordered behind its increment by the barrier that follows.
      int* count = arrived + share_slot * ipt + it;
      const int before = __hip_atomic_fetch_add(count, 1, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
      if (before == n_shares - 1) __hip_atomic_store(count, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // as it was found
      *last = before == n_shares - 1;
    }
    __syncthreads();
    const bool is_last = *last != 0;
    __syncthreads();                                     // the word is in the output staging's place
    if (!is_last) return;
    m_run = -INFINITY;
    l_run = 0.f;
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
      for (int e = 0; e < 16; ++e) oacc[dt][e] = 0.f;
    for (int s = 0; s < n_shares; ++s) {                 // every part, this block's own too, in the order of s
      const float* theirs = slot0 + (size_t)s * XW * NT;
      const float m_o = __hip_atomic_load(theirs, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
      const float l_o = __hip_atomic_load(theirs + NT, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
      const float m_new = fmaxf(m_run, m_o);
      const float c_mine = (m_run == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(m_run - m_new);
      const float c_theirs = (m_o == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(m_o - m_new);
      l_run = l_run * c_mine + l_o * c_theirs;
#pragma unroll
      for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
        for (int e = 0; e < 16; ++e)
          oacc[dt][e] = oacc[dt][e] * c_mine +
                        __hip_atomic_load(theirs + (2 + dt * 16 + e) * NT, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM) * c_theirs;
      m_run = m_new;
    }
  }
  // normalise; O^T regs: d = 32 dt + 8 (e / 4) + 4 hf + e % 4 for this lane's row
  const float l_tot = l_run + __shfl_xor(l_run, 32, MF_WAVE);
  const float inv = l_tot > 0.f ? 1.0f / l_tot : 0.f;
  bf16* ow = reinterpret_cast<bf16*>(smem) + (size_t)wid * 32 * K_LD;
#pragma unroll
  for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
    for (int rb = 0; rb < 4; ++rb) {
      const int d = dt * 32 + rb * 8 + hf * 4;
      if (d < HD) {
        const bf16x4 v = {(bf16)(oacc[dt][rb * 4 + 0] * inv), (bf16)(oacc[dt][rb * 4 + 1] * inv),
                          (bf16)(oacc[dt][rb * 4 + 2] * inv), (bf16)(oacc[dt][rb * 4 + 3] * inv)};
        *reinterpret_cast<bf16x4*>(&ow[ql * K_LD + d]) = v;
      }
    }
  __syncthreads();
  // the rows of this wave, 16 bytes per lane
  for (int c = lane; c < 32 * (HD / 8); c += 64) {
    const int row = c / (HD / 8), ch = c % (HD / 8);
    const int rr = wid * 32 + row, t = rr / ghc, gg = rr - t * ghc;
    if (t < n_tok)
      *reinterpret_cast<bf16x8*>(out + ((size_t)(tok0 + q0 + t) * nh + h0 + gg) * HD + ch * 8) =
          *reinterpret_cast<const bf16x8*>(&ow[row * K_LD + ch * 8]);
  }
}

template <int NKS>
int launch(const bf16* q, const bf16* kc, const bf16* vc, const int* page_table, int pt_stride,
           const int* cu_seqlens, const int* start_pos, const int* tile_seq, const int* tile_q0,
           const int* tile_share, float* parts, int* arrived, int max_shares, bf16* out, int n_tiles, int nh, int nk,
           int gh, int tq, float scale, int window, hipStream_t stream) {
  using S = Shape<NKS>;
  if (gh * tq > S::ROWS) return (int)hipErrorInvalidValue;
  static bool configured = false;
  auto kern = attn_prefill_kernel<NKS>;
  if (!configured) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, S::SMEM);
    if (e != hipSuccess) return (int)e;
    configured = true;
  }
  static int n_cu = 0;                 // compute units of the device (asked once)
  if (n_cu == 0) {
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) return (int)hipErrorUnknown;
    n_cu = prop.multiProcessorCount;
  }
  const int G = nh / nk, ipt = nk * ((G + gh - 1) / gh);
  kern<<<n_tiles * ipt, S::NW * 64, S::SMEM, stream>>>(q, kc, vc, page_table, pt_stride, cu_seqlens, start_pos, tile_seq,
                                                       tile_q0, tile_share, parts, arrived, max_shares, out, nh, nk, gh,
                                                       tq, scale, window, S::PER_CU == 2 && !tile_share ? n_cu : 0);
  return mf_launch_status();
}

}  // namespace

// (token, head) pairs a workgroup takes at this head size: the host gives it `gh` heads of a kv
// head's group (all of them, unless the group has more heads than that) times tq = rows / gh
// consecutive new tokens.
MF_API int mf_attn_prefill_rows(int hd) { return 128; }
// workgroups of this kernel that run on a CU at once
MF_API int mf_attn_prefill_per_cu(int hd) { return hd <= 128 ? 2 : 1; }

// tile_seq[i], tile_q0[i]: sequence (index in the step's batch) and first new token of the
// i-th block of tq query tokens; the host lists them, longest first.  Every block of tokens is
// worked by nk * ceil((nh / nk) / gh) workgroups, one for each kv head and each chunk of gh heads of
// its group.  tile_share (or null: every workgroup has its rows to itself): entry i is share + 256 *
// shares + 65536 * slot, workgroup `share` of `shares` (at most max_shares, which is at most 255)
// that take the pages of these queries in turn; their parts meet in
// parts[slot][workgroup of the block][max_shares][mf_attn_prefill_part_floats(hd)] and
// arrived[slot][workgroup of the block], which is zero before the call and after it.  Calls that use
// the same parts and arrived run on one stream.
MF_API int mf_attn_prefill_part_floats(int hd) {
  return (((hd / 16 + 1) / 2) * 16 + 2) * 256;
}

MF_API int mf_attn_prefill_bf16(const void* q, const void* kc, const void* vc, const int* page_table,
                                int pt_stride, const int* cu_seqlens, const int* start_pos,
                                const int* tile_seq, const int* tile_q0, const int* tile_share, float* parts,
                                int* arrived, int max_shares, void* out, int n_tiles, int nh, int nk, int hd,
                                int gh, int tq, float scale, int window, hipStream_t stream) {
  if (n_tiles <= 0) return 0;
  if (hd % 16 != 0 || hd < 16 || hd > 256 || nk <= 0 || nh % nk != 0) return (int)hipErrorInvalidValue;
  if (gh < 1 || tq < 1 || gh > nh / nk) return (int)hipErrorInvalidValue;
  if (tile_share && (!parts || !arrived || max_shares < 1 || max_shares > 255)) return (int)hipErrorInvalidValue;
#define MF_CASE(E)                                                                                        \
  case E:                                                                                                 \
    return launch<E>((const bf16*)q, (const bf16*)kc, (const bf16*)vc, page_table, pt_stride, cu_seqlens, \
                     start_pos, tile_seq, tile_q0, tile_share, parts, arrived, max_shares, (bf16*)out, n_tiles, nh, \
                     nk, gh, tq, scale, window, stream);
  switch (hd / 16) {
    MF_CASE(1) MF_CASE(2) MF_CASE(3) MF_CASE(4) MF_CASE(5) MF_CASE(6) MF_CASE(7) MF_CASE(8)
    MF_CASE(9) MF_CASE(10) MF_CASE(11) MF_CASE(12) MF_CASE(13) MF_CASE(14) MF_CASE(15) MF_CASE(16)
  }
#undef MF_CASE
  return (int)hipErrorInvalidValue;
}
