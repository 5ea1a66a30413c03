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
// A block (4 waves) owns 128 consecutive query tokens of one sequence and one query head;
// each wave 32 of them.  The time of a prompt's attention is that of its last tile, whose block
// walks every page of the sequence one after the other, so the host may give a tile to several
// blocks, which take its pages in turn (block s of n the pages first + s, first + s + n, ...):
// each leaves its maxima, sums and output in `parts`, counts itself in, and the one that comes
// last adds all of them up, in the order of s, and writes the result.
// Per cache page (64 keys): K goes to LDS as stored and V^T as rows of 64
// keys (the cache keeps a page of V transposed in two halves, [2][head_dim][32 keys], which the
// copy puts side by side), into one of two buffers.
//   S^T[key][q] = K Q^T      32x32x16 MFMA, A = K rows from LDS, B = Q held in registers
//   lane <-> query column, so the row statistics of the softmax are per-lane scalars
//   O^T[d][q]  += V^T P^T    A = V^T from LDS, B = P^T, which is S^T's own register layout
// The k index of the second product is permuted the same way on both operands (the sum
// does not care), which is what lets P stay in registers.
#include "common.h"

namespace {

constexpr int BQ = 128;             // query tokens per block
constexpr int KT = MF_PAGE;         // keys per step: one page
constexpr int VT_LD = KT + 4;       // LDS row stride of V^T in elements: 34 words, conflict-free 8-byte reads

// Two blocks per CU up to head size 128: left to itself the compiler takes more than 256 registers
// there (one wave per SIMD) and shuffles the accumulators between the two register files; held to
// 256 it needs no scratch and runs nearly twice as fast.
template <int NKS>                  // head_dim / 16
__global__ __launch_bounds__(256, NKS <= 8 ? 2 : 1) void attn_prefill_kernel(
    const bf16* __restrict__ q, const bf16* __restrict__ kc, const bf16* __restrict__ vc,
    const int* __restrict__ page_table, int pt_stride, const int* __restrict__ cu_seqlens,
    const int* __restrict__ start_pos, const int* __restrict__ tile_seq,
    const int* __restrict__ tile_q0, const int* __restrict__ tile_share, float* __restrict__ parts,
    int* __restrict__ arrived, int max_shares, bf16* __restrict__ out, int n_tiles, int nh, int nk, float scale,
    int window, int pair_slots) {
  constexpr int HD = NKS * 16;
  constexpr int NDT = (NKS + 1) / 2;          // 32-wide output tiles over head_dim
  constexpr int HDP = NDT * 32;
  constexpr int K_LD = HD + 8;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  constexpr int BUF = KT * K_LD + HDP * VT_LD;           // elements of one buffer: K [KT][K_LD], V^T [HDP][VT_LD]
  bf16* const kv = reinterpret_cast<bf16*>(smem);        // two such buffers
  bf16* Os = reinterpret_cast<bf16*>(smem);              // [4][32][K_LD], after the last step

  // Work items are (tile, head) with the tiles longest first (the host sorts them), one block
  // each, in this order: the longest start first and the short ones fill in behind them.  Where
  // all items are on the chip at once, two to a CU (a prompt of 2,048 tokens and 28 heads: 448),
  // nothing fills in, and what counts is which two share a CU: blocks i and i + CUs do, so the
  // second lot runs shortest first and every CU gets about the same number of pages (the
  // longest and the shortest tile together: 34 pages where two of the longest were 64).
  const int n_items = n_tiles * nh;
  int item = blockIdx.x;
  if (pair_slots > 0 && n_items <= 2 * pair_slots && item >= pair_slots) item = n_items - 1 - (item - pair_slots);
  const int tile = item / nh;
  const int b = tile_seq[tile], q0 = tile_q0[tile];
  const int h = item % nh, hk = h / (nh / nk);
  // tile_share[tile]: which of how many blocks of these queries this one is, and the number of the
  // queries' slot in `parts` and `arrived`: share + 256 * shares + 65536 * slot (0 shares: alone)
  const int share_word = tile_share ? tile_share[tile] : 0;
  const int share = share_word & 255, n_shares = max(1, (share_word >> 8) & 255), share_slot = share_word >> 16;
  const int tok0 = cu_seqlens[b], n_new = cu_seqlens[b + 1] - tok0, start = start_pos[b];
  const int* pt = page_table + (size_t)b * pt_stride;
  const int tid = threadIdx.x, lane = tid & 63, wid = tid >> 6;
  const int ql = lane & 31, hf = lane >> 5;

  // this lane's query
  const int qi = q0 + wid * 32 + ql;                     // index among the sequence's new tokens
  const bool q_ok = qi < n_new;
  const int pq = start + qi;                             // its position
  bf16x8 qf[NKS];
#pragma unroll
  for (int ks = 0; ks < NKS; ++ks) {
    qf[ks] = bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
    if (q_ok)
      qf[ks] = *reinterpret_cast<const bf16x8*>(q + ((size_t)(tok0 + qi) * nh + h) * HD + ks * 16 + hf * 8);
  }
  // positions this wave and this block need
  const float sl2 = scale * 1.44269504088896340736f;    // scores -> exponents of 2
  const bool wave_q_last_ok = q0 + wid * 32 + 31 < n_new;   // all 32 queries of the wave exist
  const int wave_q_last = min(q0 + wid * 32 + 31, n_new - 1);
  const int wave_p_hi = start + wave_q_last;
  const int wave_p_lo = start + q0 + wid * 32;
  const int blk_p_hi = start + min(q0 + BQ - 1, n_new - 1);
  const int blk_p_lo = start + q0;
  const int key_lo = window > 0 ? max(0, blk_p_lo - window + 1) : 0;

  floatx16 oacc[NDT];
#pragma unroll
  for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
    for (int r = 0; r < 16; ++r) oacc[dt][r] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;

  if (HDP > HD) {   // rows of V^T beyond head_dim stay zero
    for (int i = tid; i < (HDP - HD) * VT_LD; i += 256) {
      kv[KT * K_LD + HD * VT_LD + i] = (bf16)0.f;
      kv[BUF + KT * K_LD + HD * VT_LD + i] = (bf16)0.f;
    }
  }

  // K and V of a page travel global -> registers while the page before is multiplied
  constexpr int KCH = (KT * (HD / 8) + 255) / 256;       // K chunks of 8 elements per thread
  constexpr int VCH = (HD * (KT / 8) + 255) / 256;       // V^T chunks of 8 keys per thread
  bf16x8 kreg[KCH], vreg[VCH];
  auto fetch = [&](int page_i) {
    const int page = pt[page_i];
    const bf16* kp = kc + ((size_t)page * nk + hk) * KT * HD;
    const bf16* vp = vc + ((size_t)page * nk + hk) * HD * KT;     // a page of V is [2][HD][KT / 2]
#pragma unroll
    for (int i = 0; i < KCH; ++i) {
      const int c = i * 256 + tid;
      if (c < KT * (HD / 8)) kreg[i] = *reinterpret_cast<const bf16x8*>(kp + (size_t)(c / (HD / 8)) * HD + (c % (HD / 8)) * 8);
    }
    // Keys after the block's last position were never written (a page is not cleared when
    // it is taken): they are masked out of P, but 0 * garbage could still be NaN, so they
    // enter as zeros.
    const int n_written = blk_p_hi - page_i * KT + 1;    // keys of this page that exist
#pragma unroll
    for (int i = 0; i < VCH; ++i) {
      const int c = i * 256 + tid;         // chunk: half c / (4 HD), column (c / 4) % HD, 8 keys from 8 (c % 4)
      if (c < HD * (KT / 8)) {
        vreg[i] = *reinterpret_cast<const bf16x8*>(vp + (size_t)c * 8);
        if (n_written < KT) {
          const int k0 = (c / (HD * 4)) * (KT / 2) + (c % 4) * 8;
#pragma unroll
          for (int e = 0; e < 8; ++e)
            if (k0 + e >= n_written) vreg[i][e] = (bf16)0.f;
        }
      }
    }
  };
  // registers -> LDS, as stored: K thread -> (row, 8-element chunk); V^T thread -> (column,
  // 8-key chunk), whose row stride keeps 8-byte alignment only
  auto stage = [&](int buf) {
    bf16* Ks = kv + buf * BUF;
    bf16* Vt = Ks + KT * K_LD;
#pragma unroll
    for (int i = 0; i < KCH; ++i) {
      const int c = i * 256 + tid;
      if (c < KT * (HD / 8)) *reinterpret_cast<bf16x8*>(&Ks[(c / (HD / 8)) * K_LD + (c % (HD / 8)) * 8]) = kreg[i];
    }
#pragma unroll
    for (int i = 0; i < VCH; ++i) {
      const int c = i * 256 + tid;
      if (c < HD * (KT / 8)) {
        bf16* dst = &Vt[((c / 4) % HD) * VT_LD + (c / (HD * 4)) * (KT / 2) + (c % 4) * 8];
        *reinterpret_cast<bf16x4*>(dst) = bf16x4{vreg[i][0], vreg[i][1], vreg[i][2], vreg[i][3]};
        *reinterpret_cast<bf16x4*>(dst + 4) = bf16x4{vreg[i][4], vreg[i][5], vreg[i][6], vreg[i][7]};
      }
    }
  };
  // Two buffers, one barrier a page: while page i is multiplied from one buffer, page i + 1
  // (fetched a step ago) goes from registers into the other and page i + 2 sets out from memory.
  const int page_first = key_lo / KT + share, page_last = blk_p_hi / KT;
  if (page_first <= page_last) {
    fetch(page_first);
    stage(0);
    if (page_first + n_shares <= page_last) fetch(page_first + n_shares);
  }
  __syncthreads();
  int buf = 0;
  for (int page_i = page_first; page_i <= page_last; page_i += n_shares, buf ^= 1) {
    if (page_i + n_shares <= page_last) {
      stage(buf ^ 1);             // every wave is past the barrier behind its last read of that buffer
      if (page_i + 2 * n_shares <= page_last) fetch(page_i + 2 * n_shares);
    }
    const bf16* Ks = kv + buf * BUF;
    const bf16* Vt = Ks + KT * K_LD;
    const int key0 = page_i * KT;
    // nothing to do for this wave where every key is later than every query here, or left of every window
    const bool skip = key0 > wave_p_hi || (window > 0 && key0 + KT - 1 <= wave_p_lo - window);
    if (skip) {
      __syncthreads();
      continue;
    }

    // S^T = K Q^T, two tiles of 32 keys
    floatx16 s[2];
#pragma unroll
    for (int kt = 0; kt < 2; ++kt) {
#pragma unroll
      for (int r = 0; r < 16; ++r) s[kt][r] = 0.f;
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks) {
        const bf16x8 a = *reinterpret_cast<const bf16x8*>(&Ks[(kt * 32 + ql) * K_LD + ks * 16 + hf * 8]);
        s[kt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, qf[ks], s[kt], 0, 0, 0);
      }
    }
    // Mask, running maximum: reg r of tile kt is key key0 + 32 kt + 8 (r / 4) + 4 hf + r % 4.
    // Scores stay unscaled; the maximum is kept in units of scale * log2(e), so that
    // exp((s - m) scale) is one fused multiply-add and one 2^x per score.  A page that every
    // query of the wave sees whole needs no mask.
    float m_new = m_run;
    const bool whole = key0 + KT - 1 <= wave_p_lo && wave_q_last_ok && (window <= 0 || key0 > wave_p_hi - window);
    if (whole) {
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int r = 0; r < 16; ++r) m_new = fmaxf(m_new, s[kt][r] * sl2);
    } else {
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int key = key0 + kt * 32 + (r >> 2) * 8 + hf * 4 + (r & 3);
          const bool vis = q_ok && key <= pq && (window <= 0 || key > pq - window);
          s[kt][r] = vis ? s[kt][r] : -INFINITY;
          m_new = fmaxf(m_new, s[kt][r] * sl2);
        }
    }
    m_new = fmaxf(m_new, __shfl_xor(m_new, 32, MF_WAVE));
    const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
    float psum = 0.f;
    bf16x8 pb[4];
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float pe = __builtin_amdgcn_exp2f(fmaf(s[kt][r], sl2, -m_use));    // 2^(-inf) = 0 for masked keys
        psum += pe;
        pb[kt * 2 + (r >> 3)][r & 7] = (bf16)pe;
      }
    // the accumulators are rescaled only when some query's maximum moved
    if (__builtin_amdgcn_ballot_w64(m_new != m_run) != 0) {
      const float corr = (m_new == -INFINITY) ? 1.f : __builtin_amdgcn_exp2f(m_run - m_new);
      l_run *= corr;
#pragma unroll
      for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[dt][r] *= corr;
      m_run = m_new;
    }
    l_run += psum;
    // O^T += V^T P^T; operand element e of group kg is key 16 kg + 8 (e / 4) + 4 hf + e % 4
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
      for (int kg = 0; kg < 4; ++kg) {
        const bf16* vrow = &Vt[(dt * 32 + ql) * VT_LD + kg * 16 + hf * 4];
        const bf16x4 lo4 = *reinterpret_cast<const bf16x4*>(vrow);
        const bf16x4 hi4 = *reinterpret_cast<const bf16x4*>(vrow + 8);
        const bf16x8 a = {lo4[0], lo4[1], lo4[2], lo4[3], hi4[0], hi4[1], hi4[2], hi4[3]};
        oacc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, pb[kg], oacc[dt], 0, 0, 0);
      }
    __syncthreads();
  }

  if (n_shares > 1) {
    // This block's part goes to memory (lane-major: value v of thread t at v * 256 + t), written
    // through and read past the caches, since the blocks of a tile may sit behind different L2s.
    constexpr int XW = NDT * 16 + 2;
    float* slot0 = parts + ((size_t)share_slot * nh + h) * max_shares * XW * 256 + tid;
    float* mine = slot0 + (size_t)share * XW * 256;
    __hip_atomic_store(mine, m_run, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    __hip_atomic_store(mine + 256, l_run, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        __hip_atomic_store(mine + (2 + dt * 16 + r) * 256, oacc[dt][r], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    __builtin_amdgcn_s_waitcnt(0);                       // this wave's stores have reached memory
    __syncthreads();
    int* last = reinterpret_cast<int*>(smem);            // (the page buffers are free behind the loop's last barrier)
    if (tid == 0) {
      // Counting in releases this block's part and, for the block that arrives last, acquires the
      // others': the block's stores are ordered before the increment by the barrier above (and are
      // atomic stores themselves), the increments on one counter form a release sequence, and the
      // last arriver's loads below are ordered behind its increment by the barrier that follows.
      int* count = arrived + share_slot * nh + h;
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
      for (int r = 0; r < 16; ++r) oacc[dt][r] = 0.f;
    for (int s = 0; s < n_shares; ++s) {                 // every part, this block's own too, in the order of s
      const float* theirs = slot0 + (size_t)s * XW * 256;
      const float m_o = __hip_atomic_load(theirs, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
      const float l_o = __hip_atomic_load(theirs + 256, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
      const float m_new = fmaxf(m_run, m_o);
      const float c_mine = (m_run == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(m_run - m_new);
      const float c_theirs = (m_o == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(m_o - m_new);
      l_run = l_run * c_mine + l_o * c_theirs;
#pragma unroll
      for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r)
          oacc[dt][r] = oacc[dt][r] * c_mine +
                        __hip_atomic_load(theirs + (2 + dt * 16 + r) * 256, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM) * c_theirs;
      m_run = m_new;
    }
  }
  // normalise; O^T regs: d = 32 dt + 8 (r / 4) + 4 hf + r % 4 for this lane's query
  const float l_tot = l_run + __shfl_xor(l_run, 32, MF_WAVE);
  const float inv = l_tot > 0.f ? 1.0f / l_tot : 0.f;
  // (all waves are past the last page's barrier: the buffers are free)
  bf16* ow = Os + (size_t)wid * 32 * K_LD;
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
  // rows of this wave's 32 queries, 16 bytes per lane
  for (int c = lane; c < 32 * (HD / 8); c += 64) {
    const int row = c / (HD / 8), ch = c % (HD / 8);
    const int qrow = q0 + wid * 32 + row;
    if (qrow < n_new)
      *reinterpret_cast<bf16x8*>(out + ((size_t)(tok0 + qrow) * nh + h) * HD + ch * 8) =
          *reinterpret_cast<const bf16x8*>(&ow[row * K_LD + ch * 8]);
  }
}

template <int NKS>
int launch(const bf16* q, const bf16* kc, const bf16* vc, const int* page_table, int pt_stride,
           const int* cu_seqlens, const int* start_pos, const int* tile_seq, const int* tile_q0,
           const int* tile_share, float* parts, int* arrived, int max_shares, bf16* out, int n_tiles, int nh, int nk,
           float scale, int window, hipStream_t stream) {
  constexpr int HD = NKS * 16, HDP = ((NKS + 1) / 2) * 32, K_LD = HD + 8;
  static int n_cu = 0;                 // compute units of the device (asked once)
  if (n_cu == 0) {
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) return (int)hipErrorUnknown;
    n_cu = prop.multiProcessorCount;
  }
  const int pair_slots = NKS <= 8 ? n_cu : 0;      // where two blocks share a CU (head sizes up to 128)
  constexpr int kv_bytes = 2 * (KT * K_LD + HDP * VT_LD) * 2;      // two buffers
  constexpr int o_bytes = 4 * 32 * K_LD * 2;
  constexpr int smem = kv_bytes > o_bytes ? kv_bytes : o_bytes;
  static bool configured = false;
  auto kern = attn_prefill_kernel<NKS>;
  if (!configured) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e != hipSuccess) return (int)e;
    configured = true;
  }
  kern<<<n_tiles * nh, 256, smem, stream>>>(q, kc, vc, page_table, pt_stride, cu_seqlens, start_pos, tile_seq,
                                            tile_q0, tile_share, parts, arrived, max_shares, out, n_tiles, nh, nk, scale,
                                            window, tile_share ? 0 : pair_slots);
  return mf_launch_status();
}

}  // namespace

// tile_seq[i], tile_q0[i]: sequence (index in the step's batch) and first new token of the
// i-th block of 128 query tokens; the host lists them, longest first.  tile_share (or null: every
// block has its queries to itself): entry i is share + 256 * shares + 65536 * slot, block `share`
// of `shares` (at most max_shares, which is at most 255) that take the pages of these queries in
// turn; their parts meet in parts[slot][head][max_shares][mf_attn_prefill_part_floats(hd)] and
// arrived[slot][head], which is zero before the call and after it.  Calls that use the same parts and arrived run on one stream.
MF_API int mf_attn_prefill_part_floats(int hd) { return (((hd / 16 + 1) / 2) * 16 + 2) * 256; }

MF_API int mf_attn_prefill_bf16(const void* q, const void* kc, const void* vc, const int* page_table,
                                int pt_stride, const int* cu_seqlens, const int* start_pos,
                                const int* tile_seq, const int* tile_q0, const int* tile_share, float* parts,
                                int* arrived, int max_shares, void* out, int n_tiles, int nh, int nk, int hd,
                                float scale, int window, hipStream_t stream) {
  if (n_tiles <= 0) return 0;
  if (hd % 16 != 0 || hd < 16 || hd > 256 || nk <= 0 || nh % nk != 0) return (int)hipErrorInvalidValue;
  if (tile_share && (!parts || !arrived || max_shares < 1 || max_shares > 255)) return (int)hipErrorInvalidValue;
#define MF_CASE(E)                                                                                        \
  case E:                                                                                                 \
    return launch<E>((const bf16*)q, (const bf16*)kc, (const bf16*)vc, page_table, pt_stride, cu_seqlens, \
                     start_pos, tile_seq, tile_q0, tile_share, parts, arrived, max_shares, (bf16*)out, n_tiles, nh, \
                     nk, scale, window, stream);
  switch (hd / 16) {
    MF_CASE(1) MF_CASE(2) MF_CASE(3) MF_CASE(4) MF_CASE(5) MF_CASE(6) MF_CASE(7) MF_CASE(8)
    MF_CASE(9) MF_CASE(10) MF_CASE(11) MF_CASE(12) MF_CASE(13) MF_CASE(14) MF_CASE(15) MF_CASE(16)
  }
#undef MF_CASE
  return (int)hipErrorInvalidValue;
}
