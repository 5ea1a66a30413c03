// bfloat16 matrix products on the gfx950 matrix cores, 32-bit accumulation:
//   C[M][N] (+)= A[M][K] * W[N][K]^T (+ bias[N])
// (out[t][o] = dot(W[o][:], x[t][:]) + b[o], src/graph/cpu_backend.rs:214-248 of
// yusiwen/minfer; the reference's own matrix kernels are quantised and are not followed.)
//
// The kernels:
//  * `tile_kernel`: many rows (prompts).  A BM x BN block tile per 4 or 8 waves, K walked in
//    steps of BK through double-buffered LDS, 32x32x16 MFMA, each wave a WM x WN tile.
//  * `tile_dma_kernel`: tiles of 256 x 256, 256 x 192 or 256 x 128 with their k tiles copied
//    straight into LDS; the choice for large aligned products (the width by how the tiles fill
//    the chip's rounds).
//  * `stationary16_kernel`: at most 16 rows and K of 896, 1536, 2048, 3584, 4096, 5120 or 8192 (decode):
//    one block per CU keeps the activations in registers and walks over weight tiles.
//  * `rolling16_kernel`, `skinny16_kernel`: at most 16 rows, any K (decode).  The time is the
//    weight stream: the waves of a block split K, each reads weights and activations straight
//    into MFMA operands (16x16x32) and the partial sums meet in LDS.
//  * `panel_kernel`: 17 to 64 rows against a wide matrix: one block per CU over the whole of K.
//  * `skinny_ring_kernel`, `skinny_kernel` (any alignment): 17 to 64 rows.  Each wave owns 16
//    weight rows and reads them from HBM straight into MFMA operands, the activation rows are
//    staged in LDS and shared by the block, K may be split over blocks with a fixed-order
//    reduction afterwards.
// Both operands have K contiguous, which is exactly the MFMA operand layout (8 consecutive
// k per lane), so nothing is transposed.  The kernels for at most 64 rows (all but the guarded
// skinny16_kernel) can read the weights from a tiled copy instead (`w_operand`), where the
// caller has one.
//
// Epilogues: 0 store fp32, 1 add into fp32 (residual stream), 2 store bf16, 3 SwiGLU.
// SwiGLU (y = silu(g) * u, silu(z) = z / (1 + exp(-z)), src/graph/cpu_backend.rs:323-329):
// the weight rows come interleaved in groups of 64, 32 gate rows then the 32 up rows of the
// same outputs (the last group padded with zero rows), so a gate column and its up column
// are 32 apart inside one wave's tile; the epilogue writes bfloat16 y[M][ldc], ldc = number
// of outputs, straight from the 32-bit accumulators and the [M][2 nf] intermediate is never
// stored.
#include <stdio.h>
#include <stdlib.h>

#include "common.h"

namespace {

enum { EPI_F32 = 0, EPI_ACC_F32 = 1, EPI_BF16 = 2, EPI_SWIGLU = 3 };

__device__ __forceinline__ void store_out(void* C, int ldc, int m, int n, float v, int epi) {
  if (epi == EPI_BF16) {
    ((bf16*)C)[(size_t)m * ldc + n] = (bf16)v;
  } else {
    float* c = (float*)C + (size_t)m * ldc + n;
    *c = (epi == EPI_ACC_F32) ? *c + v : v;
  }
}

__device__ __forceinline__ float swiglu_f(float g, float u) { return g / (1.0f + expf(-g)) * u; }

// 8 consecutive k of one row, zero at and beyond k_end.  Rows are clamped by the caller to a
// row that exists (results of such rows are never stored), so the fast form has no branch:
// VEC needs 16-byte aligned rows and K a multiple of 8, so a chunk is inside or outside whole.
template <bool VEC>
__device__ __forceinline__ bf16x8 load8(const bf16* __restrict__ base, int ld, int row, int k, int k_end) {
  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
  if (VEC) {
    const int kk = min(k, k_end - 8);
    const bf16x8 v = *reinterpret_cast<const bf16x8*>(base + (size_t)row * ld + kk);
    return k + 8 <= k_end ? v : zero;
  } else {
    bf16x8 v = zero;
    const bf16* p = base + (size_t)row * ld + k;
#pragma unroll
    for (int e = 0; e < 8; ++e)
      if (k + e < k_end) v[e] = p[e];
    return v;
  }
}

// 8 consecutive k with no guard at all: the caller knows the chunk lies inside the row.
__device__ __forceinline__ bf16x8 load8_inside(const bf16* __restrict__ base, int ld, int row, int k) {
  return *reinterpret_cast<const bf16x8*>(base + (size_t)row * ld + k);
}

// The epilogue of a wave's TM x TN tiles of 32 x 32 (D[m][n]: lane holds n = lane % 32,
// m = 8 (r / 4) + 4 (lane / 32) + r % 4): bias, then store / accumulate / round / SwiGLU.
template <int TM, int TN>
__device__ __forceinline__ void tile_epilogue(floatx16 (&acc)[TM][TN], const float* __restrict__ bias,
                                              void* __restrict__ C, int ldc, int M, int N, int epi, int m0,
                                              int wm, int n0, int wn, int lane) {
  const int fr = lane & 31;
  // D[m][n]: lane holds n = lane % 32, m = 8 (r / 4) + 4 (lane / 32) + r % 4
  if (epi == EPI_SWIGLU) {
    if constexpr (TN % 2 == 0) {
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; j += 2) {
          const int ng = n0 + wn + j * 32 + fr;            // gate column; its up column is ng + 32
          const int col = (ng >> 6) * 32 + (ng & 63);
          if (col >= ldc) continue;
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int m = m0 + wm + i * 32 + (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
            if (m < M) ((bf16*)C)[(size_t)m * ldc + col] = (bf16)swiglu_f(acc[i][j][r], acc[i][j + 1][r]);
          }
        }
    }
    return;
  }
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int n = n0 + wn + j * 32 + fr;
      if (n >= N) continue;
      const float b = bias ? bias[n] : 0.f;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = m0 + wm + i * 32 + (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
        if (m < M) store_out(C, ldc, m, n, acc[i][j][r] + b, epi);
      }
    }
}

// Tile number -> (row of tiles, column of tiles).  The tiles are numbered in bands of 8 rows of
// tiles, down a band's rows first: 32 neighbouring numbers (what an XCD has in flight, see the
// kernels) are then 8 x 4 tiles, which share 12 operand panels between them (a whole column of
// 32 tile rows would share 33).
__device__ __forceinline__ void tile_position(int tile, int tiles_m, int tiles_n, int& bm, int& bn) {
  constexpr int BAND = 8;
  const int band = tile / (BAND * tiles_n), first = band * BAND;
  const int rows = min(tiles_m - first, BAND);
  const int in_band = tile - band * BAND * tiles_n;
  bm = first + in_band % rows;
  bn = in_band / rows;
}

// ------------------------------------------------------------------ tiled kernel
// LDS row stride is BK + 8 elements (144 bytes for BK 64, 80 for BK 32): conflict-free b128 reads
template <int BM, int BN, int WM, int WN, int BK, bool VEC>
__global__ __launch_bounds__(64 * (BM / WM) * (BN / WN)) void tile_kernel(const bf16* __restrict__ A, int lda,
                                                   const bf16* __restrict__ W, int ldw,
                                                   const float* __restrict__ bias, void* __restrict__ C,
                                                   int ldc, int M, int N, int K, int epi, int tiles_m,
                                                   int xcd_remap, int k_per_split) {
  constexpr int NTHR = 64 * (BM / WM) * (BN / WN);
  constexpr int LDS_LD = BK + 8;
  if (k_per_split > 0) {
    // K split over blockIdx.y: this block multiplies k_per_split of K and stores its sums, 32-bit
    // and without bias, into its own [M][N] slab of C; another kernel adds the slabs
    const int kb = blockIdx.y * k_per_split;
    A += kb;
    W += kb;
    K = min(k_per_split, K - kb);
    C = (float*)C + (size_t)blockIdx.y * M * N;
  }
  constexpr int TM = WM / 32, TN = WN / 32;
  constexpr int RP = NTHR / (BK / 8);         // rows per load pass
  constexpr int PA = BM / RP, PW = BN / RP;
  static_assert(BM % RP == 0 && BN % RP == 0, "load passes cover the tile");
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  bf16* As = reinterpret_cast<bf16*>(smem);               // [2][BM][LDS_LD]
  bf16* Ws = As + 2 * BM * LDS_LD;                        // [2][BN][LDS_LD]

  // Workgroups go to the 8 XCDs in turn, each with an L2 of its own: give every XCD one
  // contiguous eighth of the tile numbers, so that the tiles an XCD has in flight are neighbours
  // and share their operands' rows in its L2.
  int tile = blockIdx.x;
  if (xcd_remap) {
    const int n_tiles = gridDim.x, per = n_tiles / 8, rem = n_tiles % 8;
    const int x = blockIdx.x % 8, qq = blockIdx.x / 8;
    tile = x * per + min(x, rem) + qq;
  }
  int bm, bn;
  tile_position(tile, tiles_m, gridDim.x / tiles_m, bm, bn);
  const int m0 = bm * BM, n0 = bn * BN;
  const int tid = threadIdx.x, lane = tid & 63, wid = tid >> 6;
  const int wm = (wid % (BM / WM)) * WM, wn = (wid / (BM / WM)) * WN;
  const int lrow = tid / (BK / 8), lk = (tid % (BK / 8)) * 8;
  const int fr = lane & 31, fk = (lane >> 5) * 8;

  floatx16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  bf16x8 ra[PA], rw[PW];
  int arow[PA], wrow[PW];                       // rows past the matrix read its last row
#pragma unroll
  for (int p = 0; p < PA; ++p) arow[p] = min(m0 + p * RP + lrow, M - 1);
#pragma unroll
  for (int p = 0; p < PW; ++p) wrow[p] = min(n0 + p * RP + lrow, N - 1);
  const int nkt = (K + BK - 1) / BK;
  const int nkt_inside = VEC ? K / BK : 0;      // k tiles that need no guard (the loop's fast form:
                                                // a guard's select would wait for the load at once)
  auto load_tile = [&](int kt) {
    const int k = kt * BK + lk;
    if (kt < nkt_inside) {
#pragma unroll
      for (int p = 0; p < PA; ++p) ra[p] = load8_inside(A, lda, arow[p], k);
#pragma unroll
      for (int p = 0; p < PW; ++p) rw[p] = load8_inside(W, ldw, wrow[p], k);
    } else {
#pragma unroll
      for (int p = 0; p < PA; ++p) ra[p] = load8<VEC>(A, lda, arow[p], k, K);
#pragma unroll
      for (int p = 0; p < PW; ++p) rw[p] = load8<VEC>(W, ldw, wrow[p], k, K);
    }
  };
  load_tile(0);
#pragma unroll
  for (int p = 0; p < PA; ++p)
    *reinterpret_cast<bf16x8*>(&As[(p * RP + lrow) * LDS_LD + lk]) = ra[p];
#pragma unroll
  for (int p = 0; p < PW; ++p)
    *reinterpret_cast<bf16x8*>(&Ws[(p * RP + lrow) * LDS_LD + lk]) = rw[p];
  __syncthreads();

  for (int kt = 0; kt < nkt; ++kt) {
    const int cur = kt & 1;
    const bool more = kt + 1 < nkt;
    if (more) load_tile(kt + 1);
    const bf16* as = As + cur * BM * LDS_LD;
    const bf16* ws = Ws + cur * BN * LDS_LD;
    // The fragments of k-step ks + 1 are asked for before the products of k-step ks are issued,
    // into the other half of fa / fw, so the matrix cores do not wait for LDS inside a tile.
    bf16x8 fa[2][TM], fw[2][TN];
    auto read_frags = [&](int ks, int h) {
#pragma unroll
      for (int i = 0; i < TM; ++i)
        fa[h][i] = *reinterpret_cast<const bf16x8*>(&as[(wm + i * 32 + fr) * LDS_LD + ks * 16 + fk]);
#pragma unroll
      for (int j = 0; j < TN; ++j)
        fw[h][j] = *reinterpret_cast<const bf16x8*>(&ws[(wn + j * 32 + fr) * LDS_LD + ks * 16 + fk]);
    };
    read_frags(0, 0);
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) {
      if (ks + 1 < BK / 16) read_frags(ks + 1, (ks + 1) & 1);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[ks & 1][i], fw[ks & 1][j], acc[i][j], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
    if (more) {
      bf16* an = As + (cur ^ 1) * BM * LDS_LD;
      bf16* wn_ = Ws + (cur ^ 1) * BN * LDS_LD;
#pragma unroll
      for (int p = 0; p < PA; ++p)
        *reinterpret_cast<bf16x8*>(&an[(p * RP + lrow) * LDS_LD + lk]) = ra[p];
#pragma unroll
      for (int p = 0; p < PW; ++p)
        *reinterpret_cast<bf16x8*>(&wn_[(p * RP + lrow) * LDS_LD + lk]) = rw[p];
    }
    __syncthreads();
  }

  tile_epilogue<TM, TN>(acc, bias, C, ldc, M, N, epi, m0, wm, n0, wn, lane);
}

// ------------------------------------------------------------------ tiled kernel, loads straight into LDS
// A tile of 256 rows by BN weight rows on 8 waves, but k tiles of 64 travel global -> LDS
// without passing registers (global_load_lds_dwordx4: lane i's 16 bytes land at the wave's LDS
// base + 16 i), in two or three stages of (256 + BN) * 128 bytes, and the staging registers are
// gone.  The widths: 256 (waves of 128 x 64, two stages of 64 KB) has the most products per
// byte copied and is the fastest where its tiles fill the chip's rounds; 192 (waves of 64 x 96)
// and 128 (waves of 64 x 64, three stages) make more, smaller tiles for products whose 256-wide
// tiles would leave a round half empty (q|k|v and o of a prompt of 2,048 tokens: 144 and 112
// such tiles for 256 CUs).
//
// A row of a k tile is one 128-byte line, fetched by 8 adjacent lanes: what a CU can have in
// flight towards L2 is counted in requests, so every request should be a whole line (k tiles of
// 32, half lines, drew markedly less).
//
// There is no room for padding in such a copy, so a row's eight 16-byte chunks are stored
// permuted: chunk c of row r sits at position c ^ ((r >> 1) & 7), which spreads the 16 rows
// that one pass of a 16-byte fragment read covers over all 64 banks.  Which chunk a lane fetches
// is free (its global address), so the permutation costs nothing on the way in.
//
// The compiler does not know that these loads write LDS and so does not wait for them; the
// kernel does, with vmcnt counts it keeps itself (4 + BN / 64 loads per wave and tile, in order)
// and one barrier per tile: behind it, tile kt + 1 has landed for every wave, and the stage of
// tile kt, which every wave holds in registers by then, is free to take tile kt + STAGES.
// Needs 16-byte aligned rows and K a multiple of 64.  What keeps this kernel from the matrix
// cores' own rate is where the copies' lines come from (HBM and other dies' share of the data),
// not how the copies are issued: blocks that run side by side on an XCD must walk K in step, so
// that a line one of them fetches is in that XCD's L2 for the others.
constexpr int DMA_BM = 256, DMA_BK = 64;

// 16 bytes per lane from base + off (a wave-uniform base and a 32-bit byte offset per lane: one
// register where a 64-bit address takes two, and no address arithmetic per copy)
__device__ __forceinline__ void dma16(const bf16* base, unsigned off, unsigned lds_byte) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(off), "s"(base), "s"(lds_byte)
               : "memory", "m0");
}

// waits until at most `tiles` of the youngest k tiles' copies (LOADS a wave and tile) are in flight
template <int LOADS>
__device__ __forceinline__ void dma_wait(int tiles) {
  if (tiles <= 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  else if (tiles == 1) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(LOADS) : "memory");
  else asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * LOADS) : "memory");
}

// BN: the tile's width (256 or 128); WAVES_M x (8 / WAVES_M): the grid of the 8 waves over the
// tile; STAGES: k tiles of a tile in LDS (2 or 3), (256 + BN) * 128 bytes each.
template <int BN, int WAVES_M, int STAGES>
__global__ __launch_bounds__(512) void tile_dma_kernel(const bf16* __restrict__ A, int lda,
                                                       const bf16* __restrict__ W, int ldw,
                                                       const float* __restrict__ bias, void* __restrict__ C,
                                                       int ldc, int M, int N, int K, int epi, int tiles_m,
                                                       int xcd_remap, int k_per_split) {
  constexpr int WAVES_N = 8 / WAVES_M;
  constexpr int WM = DMA_BM / WAVES_M, WN = BN / WAVES_N;
  constexpr int TM = WM / 32, TN = WN / 32;
  constexpr int ROW = DMA_BK * 2;              // bytes of a row in LDS
  constexpr int STAGE_BYTES = (DMA_BM + BN) * ROW;
  constexpr int WB = BN / 64;                  // 1 KB blocks of the W tile that a wave copies
  constexpr int LOADS = 4 + WB;                // copies per wave and k tile
  static_assert(STAGES == 2 || STAGES == 3, "the waits count one or two tiles in flight");
  if (k_per_split > 0) {
    // K split over blockIdx.y (k_per_split a multiple of 64): this block multiplies its part of K
    // and stores 32-bit sums into its own [M][N] slab of C; another kernel adds the slabs
    const int kb = blockIdx.y * k_per_split;
    A += kb;
    W += kb;
    K = min(k_per_split, K - kb);
    C = (float*)C + (size_t)blockIdx.y * M * N;
  }
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  int tile = blockIdx.x;
  if (xcd_remap) {
    const int n_tiles = gridDim.x, per = n_tiles / 8, rem = n_tiles % 8;
    const int x = blockIdx.x % 8, qq = blockIdx.x / 8;
    tile = x * per + min(x, rem) + qq;
  }
  int bm, bn;
  tile_position(tile, tiles_m, gridDim.x / tiles_m, bm, bn);
  const int m0 = bm * DMA_BM, n0 = bn * BN;
  const int lane = threadIdx.x & 63;
  const int wid = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wm = (wid % WAVES_M) * WM, wn = (wid / WAVES_M) * WN;
  const int fr = lane & 31, fk = lane >> 5;

  floatx16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // this lane's share of a tile's copy: wave `wid` moves the 1 KB blocks wid, 8 + wid, ... (8 rows
  // each) of the A tile and of the W tile; the lane fetches row 8 b + lane / 8, the chunk that
  // belongs at position lane % 8
  const unsigned lds0 = (unsigned)(uintptr_t)smem;
  unsigned ga[4], gw[WB];                      // byte offsets from A and W (the host checks that they fit)
#pragma unroll
  for (int jj = 0; jj < 4; ++jj) {
    const int r = 8 * (jj * 8 + wid) + (lane >> 3);
    const int chunk = (lane & 7) ^ ((r >> 1) & 7);
    ga[jj] = ((unsigned)min(m0 + r, M - 1) * (unsigned)lda + chunk * 8) * 2u;
    if (jj < WB) gw[jj] = ((unsigned)min(n0 + r, N - 1) * (unsigned)ldw + chunk * 8) * 2u;
  }
  // the copies of a wave for tile kt into stage st: four blocks of the A tile, then WB of the W tile
  auto issue = [&](int kt, int st) {
    const unsigned base = lds0 + (unsigned)st * STAGE_BYTES + wid * 1024;
    const int k = kt * DMA_BK;
#pragma unroll
    for (int q = 0; q < 4; ++q) dma16(A + k, ga[q], __builtin_amdgcn_readfirstlane(base + q * 8192));
#pragma unroll
    for (int q = 0; q < WB; ++q)
      dma16(W + k, gw[q], __builtin_amdgcn_readfirstlane(base + DMA_BM * ROW + q * 8192));
  };
  // fragment reads: row R of a tile, chunk 4 half + 2 ks + fk of its 8, at position chunk ^ ((R >> 1) & 7)
  const int sw = (fr >> 1) & 7;
  int offa[TM], offw[TN];
#pragma unroll
  for (int i = 0; i < TM; ++i) offa[i] = (wm + i * 32 + fr) * ROW;
#pragma unroll
  for (int j = 0; j < TN; ++j) offw[j] = DMA_BM * ROW + (wn + j * 32 + fr) * ROW;

  const int nkt = K / DMA_BK;
  // A tile is multiplied in two halves of two k-steps, from two register sets: the fragments of
  // the next half are read from LDS while the second k-step of this one runs, so that behind the
  // barrier there is always work for the matrix cores.
  bf16x8 fa[2][2][TM], fw[2][2][TN];          // [set][k-step][tile]
  auto read_frags = [&](int stage, auto HALF) {
    constexpr int half = decltype(HALF)::value;          // which is also the register set
    const unsigned char* st = smem + stage * STAGE_BYTES;
    const int pos0 = ((half * 4 + fk) ^ sw) * 16, pos1 = ((half * 4 + 2 + fk) ^ sw) * 16;
#pragma unroll
    for (int i = 0; i < TM; ++i) fa[half][0][i] = *reinterpret_cast<const bf16x8*>(st + offa[i] + pos0);
#pragma unroll
    for (int j = 0; j < TN; ++j) fw[half][0][j] = *reinterpret_cast<const bf16x8*>(st + offw[j] + pos0);
#pragma unroll
    for (int i = 0; i < TM; ++i) fa[half][1][i] = *reinterpret_cast<const bf16x8*>(st + offa[i] + pos1);
#pragma unroll
    for (int j = 0; j < TN; ++j) fw[half][1][j] = *reinterpret_cast<const bf16x8*>(st + offw[j] + pos1);
  };
  auto multiply = [&](int ks, auto SET) {
    constexpr int set = decltype(SET)::value;
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[set][ks][i], fw[set][ks][j], acc[i][j], 0, 0, 0);
  };
  using S0 = std::integral_constant<int, 0>;
  using S1 = std::integral_constant<int, 1>;
  // tiles 0 .. STAGES - 1 set out at once; tile 0 has landed (for this wave) when only the ones
  // after it are in flight
  int issued = 0;                              // tiles set out so far
  for (; issued < STAGES && issued < nkt; ++issued) issue(issued, issued);
  dma_wait<LOADS>(issued - 1);
  __syncthreads();
  read_frags(0, S0{});
  int stage = 0;                               // of tile kt
  // All tiles but the last run the same straight line of code, the last one a copy without the
  // barrier section.  (With that section under an `if` inside one loop, the compiler joins the
  // two paths in front of the last eight products and waits there for every LDS read in flight,
  // the next tile's fragments included, which those products do not use.)
  for (int kt = 0; kt + 1 < nkt; ++kt) {
    // first half, from set 0; the second half of the same stage goes into set 1
    multiply(0, S0{});
    __builtin_amdgcn_sched_barrier(0);
    read_frags(stage, S1{});
    __builtin_amdgcn_sched_barrier(0);
    multiply(1, S0{});
    __builtin_amdgcn_sched_barrier(0);
    // second half, from set 1; in its middle the barrier that makes tile kt + 1 readable and
    // this tile's stage free
    multiply(0, S1{});
    __builtin_amdgcn_sched_barrier(0);
    dma_wait<LOADS>(issued - kt - 2);          // tile kt + 1 has landed when only the later ones are in flight
    __syncthreads();
    // Tile kt + STAGES goes into the stage of tile kt: waves 0..3 set their copies out here, waves
    // 4..7 (the other wave of each SIMD) behind the tile's last products, a quarter of a k tile
    // later.  All eight at once measured 2 to 11 % slower (the down product of a prompt most):
    // the copies' requests reach the L2 in one burst from every CU of the XCD, which walk K in
    // step, and meet the fragment reads of the new tile in LDS.  (Four groups a quarter apart,
    // or every wave's copies in two halves, measured worse than two groups: the last ones land late.)
    const int freed = stage;
    if (wid < 4 && issued < nkt) { issue(issued, freed); ++issued; }
    stage = stage + 1 == STAGES ? 0 : stage + 1;
    read_frags(stage, S0{});
    __builtin_amdgcn_sched_barrier(0);
    multiply(1, S1{});
    __builtin_amdgcn_sched_barrier(0);
    if (wid >= 4 && issued < nkt) { issue(issued, freed); ++issued; }
    __builtin_amdgcn_sched_barrier(0);
  }
  multiply(0, S0{});
  __builtin_amdgcn_sched_barrier(0);
  read_frags(stage, S1{});
  __builtin_amdgcn_sched_barrier(0);
  multiply(1, S0{});
  multiply(0, S1{});
  multiply(1, S1{});
  tile_epilogue<TM, TN>(acc, bias, C, ldc, M, N, epi, m0, wm, n0, wn, lane);
}

template <int BN, int WAVES_M, int STAGES>
int launch_tile_dma(const bf16* A, int lda, const bf16* W, int ldw, const float* bias, void* C, int ldc, int M,
                    int N, int K, int epi, hipStream_t stream, int splits = 1, int k_per_split = 0) {
  constexpr int smem = STAGES * (DMA_BM + BN) * DMA_BK * 2;
  static bool configured = false;
  auto kern = tile_dma_kernel<BN, WAVES_M, STAGES>;
  if (!configured) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e != hipSuccess) return (int)e;
    configured = true;
  }
  const int tiles_m = (M + DMA_BM - 1) / DMA_BM, tiles_n = (N + BN - 1) / BN;
  kern<<<dim3(tiles_m * tiles_n, splits), 512, smem, stream>>>(A, lda, W, ldw, bias, C, ldc, M, N, K, epi, tiles_m,
                                                               tiles_m * tiles_n >= 16, k_per_split);
  return mf_launch_status();
}

template <int BM, int BN, int WM, int WN, int BK, bool VEC>
int launch_tile_v(const bf16* A, int lda, const bf16* W, int ldw, const float* bias, void* C, int ldc,
                  int M, int N, int K, int epi, hipStream_t stream, int splits = 1, int k_per_split = 0) {
  constexpr int smem = 2 * (BM + BN) * (BK + 8) * (int)sizeof(bf16);
  constexpr int NTHR = 64 * (BM / WM) * (BN / WN);
  static bool configured = false;
  auto kern = tile_kernel<BM, BN, WM, WN, BK, VEC>;
  if (!configured) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e != hipSuccess) return (int)e;
    configured = true;
  }
  const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
  kern<<<dim3(tiles_m * tiles_n, splits), NTHR, smem, stream>>>(A, lda, W, ldw, bias, C, ldc, M, N, K, epi,
                                                                tiles_m, tiles_m * tiles_n >= 16, k_per_split);
  return mf_launch_status();
}

template <int BM, int BN, int WM, int WN, int BK = 64>
int launch_tile(const bf16* A, int lda, const bf16* W, int ldw, const float* bias, void* C, int ldc,
                int M, int N, int K, int epi, int vec_ok, hipStream_t stream, int splits = 1,
                int k_per_split = 0) {
  return vec_ok ? launch_tile_v<BM, BN, WM, WN, BK, true>(A, lda, W, ldw, bias, C, ldc, M, N, K, epi, stream,
                                                          splits, k_per_split)
                : launch_tile_v<BM, BN, WM, WN, BK, false>(A, lda, W, ldw, bias, C, ldc, M, N, K, epi, stream,
                                                           splits, k_per_split);
}

// ------------------------------------------------------------------ skinny kernel
constexpr int KC = 256;          // k per staging step
constexpr int SK_LD = KC + 8;    // LDS row stride in elements

// The tiled copy of a weight matrix (K a multiple of 32, rows padded to a multiple of 16):
// [rows / 16][K / 32][16 rows][32 k], 1 KB a tile.  A wave's load of an MFMA operand (lane ->
// row lane % 16, eight k at 8 (lane / 16)) is one tile: a contiguous kilobyte of whole 128-byte
// lines, where the row-major matrix gives it sixteen halves of lines K elements apart, and a
// wave that walks along K reads tile after tile.  The kernels for at most 64 rows, which take their
// weights straight from memory into MFMA operands, read this copy where the caller has one (the
// down product at 8 rows: 26.7 us from 34.1).  WSTEP: elements from one step of 32 k to the next.
template <bool TILED>
__device__ __forceinline__ const bf16* w_operand(const bf16* W, int ldw, int K, int row, int k) {
  if constexpr (TILED) return W + ((size_t)(row >> 4) * (K >> 5) + (k >> 5)) * 512 + (row & 15) * 32 + (k & 31);
  else return W + (size_t)row * ldw + k;
}

// 17 to 64 rows.  A block of 8 waves owns 128 weight rows; each wave streams its 16 rows from
// HBM straight into MFMA operands, a chunk (256 k) ahead; the activation rows of a chunk are
// staged in LDS once per block (double-buffered: the next chunk travels global -> registers
// while this one is multiplied, and is written to the other buffer afterwards, so there is
// one barrier per chunk).  Partial sums go to part[split][M][N]; with one split the epilogue
// runs in place.
template <int MT, bool VEC, bool TILED>
__global__ __launch_bounds__(512) void skinny_kernel(const bf16* __restrict__ A, int lda,
                                                     const bf16* __restrict__ W, int ldw,
                                                     const float* __restrict__ bias, void* __restrict__ C,
                                                     int ldc, float* __restrict__ part, int M, int N,
                                                     int K, int k_per_split, int epi) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  bf16* As = reinterpret_cast<bf16*>(smem);                     // [2][MT * 16][SK_LD]
  constexpr int ROWS = MT * 16;
  const int tid = threadIdx.x, lane = tid & 63, wid = tid >> 6;
  const int n_row = blockIdx.x * 128 + wid * 16 + (lane & 15);  // weight row of this lane
  const int n_ld = min(n_row, N - 1);                           // the row it reads
  const int kq = (lane >> 4) * 8;                               // k offset inside a 32-step
  const int k_begin = blockIdx.y * k_per_split;
  const int k_end = min(K, k_begin + k_per_split);

  floatx4 acc[MT];
#pragma unroll
  for (int i = 0; i < MT; ++i) acc[i] = floatx4{0.f, 0.f, 0.f, 0.f};

  // staging slots of this thread: MT chunks of 8 k; chunk c -> row c / 32, k (c % 32) * 8
  int srow[MT], sk[MT];
#pragma unroll
  for (int i = 0; i < MT; ++i) {
    const int c = i * 512 + tid;
    srow[i] = c / (KC / 8);
    sk[i] = (c % (KC / 8)) * 8;
  }
  bf16x8 wcur[KC / 32], wnext[KC / 32], stage[MT];
  auto load_chunk = [&](int k0, bf16x8 (&wd)[KC / 32]) {
    if (VEC && k0 + KC <= k_end) {                     // inside: no guards, nothing waits
#pragma unroll
      for (int s = 0; s < KC / 32; ++s)
        wd[s] = *reinterpret_cast<const bf16x8*>(w_operand<TILED>(W, ldw, K, n_ld, k0 + s * 32 + kq));
#pragma unroll
      for (int i = 0; i < MT; ++i) stage[i] = load8_inside(A, lda, min(srow[i], M - 1), k0 + sk[i]);
    } else {
#pragma unroll
      for (int s = 0; s < KC / 32; ++s) {
        const int k = k0 + s * 32 + kq;
        if constexpr (TILED) {          // K in whole steps of 32: eight elements are all inside or all outside
          const bf16x8 v = *reinterpret_cast<const bf16x8*>(w_operand<true>(W, ldw, K, n_ld, min(k, K - 8)));
          wd[s] = k + 8 <= k_end ? v : bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
        } else {
          wd[s] = load8<VEC>(W, ldw, n_ld, k, k_end);
        }
      }
#pragma unroll
      for (int i = 0; i < MT; ++i) stage[i] = load8<VEC>(A, lda, min(srow[i], M - 1), k0 + sk[i], k_end);
    }
  };
  auto store_stage = [&](int buf) {
#pragma unroll
    for (int i = 0; i < MT; ++i)
      *reinterpret_cast<bf16x8*>(&As[(buf * ROWS + srow[i]) * SK_LD + sk[i]]) = stage[i];
  };
  load_chunk(k_begin, wcur);
  store_stage(0);
  __syncthreads();
  int buf = 0;
  for (int k0 = k_begin; k0 < k_end; k0 += KC) {
    const bool more = k0 + KC < k_end;
    if (more) load_chunk(k0 + KC, wnext);
    const bf16* as = As + buf * ROWS * SK_LD;
#pragma unroll
    for (int s = 0; s < KC / 32; ++s) {
#pragma unroll
      for (int i = 0; i < MT; ++i) {
        const bf16x8 a = *reinterpret_cast<const bf16x8*>(&as[(i * 16 + (lane & 15)) * SK_LD + s * 32 + kq]);
        acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, wcur[s], acc[i], 0, 0, 0);
      }
    }
    if (more) {
      store_stage(buf ^ 1);
#pragma unroll
      for (int s = 0; s < KC / 32; ++s) wcur[s] = wnext[s];
    }
    __syncthreads();
    buf ^= 1;
  }

  // D[m][n]: lane holds n = lane % 16, m = 4 (lane / 16) + r
  if (n_row >= N) return;
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int m = i * 16 + (lane >> 4) * 4 + r;
      if (m >= M) continue;
      if (part) {
        part[((size_t)blockIdx.y * M + m) * N + n_row] = acc[i][r];
      } else {
        store_out(C, ldc, m, n_row, acc[i][r] + (bias ? bias[n_row] : 0.f), epi);
      }
    }
}

// The same product where every chunk is whole (K and the splits in multiples of 256, aligned rows),
// as a ring: each wave keeps its 8 weight fragments of a chunk in registers and refills one right
// behind the MFMA that used it, with the next chunk's, so the loads in flight never run dry at a
// chunk's end as they do above; the sums leave through an LDS tile, in rows of 512 bytes.
constexpr int SR_LD = 128 + 4;      // row stride of that tile (floats)

template <int MT, bool TILED>
__global__ __launch_bounds__(512) void skinny_ring_kernel(const bf16* __restrict__ A, int lda,
                                                          const bf16* __restrict__ W, int ldw,
                                                          const float* __restrict__ bias,
                                                          void* __restrict__ C, int ldc,
                                                          float* __restrict__ part, int M, int N, int K,
                                                          int k_per_split, int epi) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  constexpr int ROWS = MT * 16;
  bf16* As = reinterpret_cast<bf16*>(smem);                                            // [2][ROWS][SK_LD]
  float* ot = reinterpret_cast<float*>(smem + 2 * ROWS * SK_LD * sizeof(bf16));        // [ROWS][SR_LD]
  const int tid = threadIdx.x, lane = tid & 63, wid = tid >> 6;
  const int r16 = lane & 15, kq = (lane >> 4) * 8;
  const int n0 = blockIdx.x * 128;
  constexpr int WSTEP = TILED ? 512 : 32;
  const bf16* wrow = w_operand<TILED>(W, ldw, K, min(n0 + wid * 16 + r16, N - 1), kq);
  const int k_begin = blockIdx.y * k_per_split;
  const int k_end = min(K, k_begin + k_per_split);
  const int sk = (tid & 31) * 8;
  const bf16* src[MT];
#pragma unroll
  for (int i = 0; i < MT; ++i) src[i] = A + (size_t)min(i * 16 + (tid >> 5), M - 1) * lda + sk;
  bf16x8 stage[MT], wr[KC / 32];
#pragma unroll
  for (int i = 0; i < MT; ++i) stage[i] = *reinterpret_cast<const bf16x8*>(src[i] + k_begin);
#pragma unroll
  for (int s = 0; s < KC / 32; ++s) wr[s] = *reinterpret_cast<const bf16x8*>(wrow + ((k_begin >> 5) + s) * WSTEP);
#pragma unroll
  for (int i = 0; i < MT; ++i)
    *reinterpret_cast<bf16x8*>(&As[(i * 16 + (tid >> 5)) * SK_LD + sk]) = stage[i];
  __syncthreads();
  floatx4 acc[MT];
#pragma unroll
  for (int i = 0; i < MT; ++i) acc[i] = floatx4{0.f, 0.f, 0.f, 0.f};
  int buf = 0;
  for (int k0 = k_begin; k0 < k_end; k0 += KC) {
    const int kn = k0 + KC < k_end ? k0 + KC : k_begin;     // behind the last chunk: the first again, dropped
#pragma unroll
    for (int i = 0; i < MT; ++i) stage[i] = *reinterpret_cast<const bf16x8*>(src[i] + kn);
    __builtin_amdgcn_sched_barrier(0);
    const bf16* as = As + buf * ROWS * SK_LD;
#pragma unroll
    for (int s = 0; s < KC / 32; ++s) {
#pragma unroll
      for (int i = 0; i < MT; ++i) {
        const bf16x8 a = *reinterpret_cast<const bf16x8*>(&as[(i * 16 + r16) * SK_LD + s * 32 + kq]);
        acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, wr[s], acc[i], 0, 0, 0);
      }
      wr[s] = *reinterpret_cast<const bf16x8*>(wrow + ((kn >> 5) + s) * WSTEP);
      __builtin_amdgcn_sched_barrier(0);      // use a register, then refill it, in this order
    }
    buf ^= 1;
#pragma unroll
    for (int i = 0; i < MT; ++i)
      *reinterpret_cast<bf16x8*>(&As[(buf * ROWS + i * 16 + (tid >> 5)) * SK_LD + sk]) = stage[i];
    __syncthreads();
  }
  // D[m][n]: n = lane % 16, m = 4 (lane / 16) + r
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int r = 0; r < 4; ++r) ot[(i * 16 + (lane >> 4) * 4 + r) * SR_LD + wid * 16 + r16] = acc[i][r];
  __syncthreads();
  const int c = tid & 127, n = n0 + c;
  if (n >= N) return;
  if (part) {
    for (int m = tid >> 7; m < M; m += 4) part[((size_t)blockIdx.y * M + m) * N + n] = ot[m * SR_LD + c];
  } else {
    const float b = bias ? bias[n] : 0.f;
    for (int m = tid >> 7; m < M; m += 4) store_out(C, ldc, m, n, ot[m * SR_LD + c] + b, epi);
  }
}

// At most 16 rows: no LDS staging at all.  A block owns 16 NT weight rows; its NW waves split
// K between them, each streaming its slice of the weights from HBM and the matching slice of
// the few activation rows from L2 straight into MFMA operands, S steps (32 S k) of loads in
// flight ahead of the matrix cores.  The waves' sums meet in LDS and wave 0 adds them in a
// fixed order and runs the epilogue, so there is no second kernel and no atomics.
template <int NW, int NT, int S, bool VEC, bool PAIR = false>
__global__ __launch_bounds__(NW * 64) void skinny16_kernel(const bf16* __restrict__ A, int lda,
                                                           const bf16* __restrict__ W, int ldw,
                                                           const float* __restrict__ bias,
                                                           void* __restrict__ C, int ldc, int M, int N,
                                                           int K, int k_per_wave, int epi) {
  __shared__ float red[NW][NT][64][4];
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
  // PAIR (SwiGLU, NT = 2): block b owns 16 gate rows of group b / 2 and the 16 up rows of
  // the same outputs, 32 rows further on
  constexpr int TSTRIDE = PAIR ? 32 : 16;
  const int n_base = (PAIR ? (blockIdx.x >> 1) * 64 + (blockIdx.x & 1) * 16 : blockIdx.x * 16 * NT) + (lane & 15);
  const int m_row = min(lane & 15, M - 1);               // rows past M read row M - 1; never stored
  int n_ld[NT];
#pragma unroll
  for (int j = 0; j < NT; ++j) n_ld[j] = min(n_base + TSTRIDE * j, N - 1);
  const int kq = (lane >> 4) * 8;
  const int k_begin = wid * k_per_wave;
  const int k_end = min(K, k_begin + k_per_wave);
  floatx4 acc[NT];
#pragma unroll
  for (int j = 0; j < NT; ++j) acc[j] = floatx4{0.f, 0.f, 0.f, 0.f};
  bf16x8 wc[NT][S], ac[S], wn[NT][S], an[S];
  // a batch that lies inside [k_begin, k_end) is loaded without guards (a guard's select
  // would make the wave wait for the load right away, and nothing would be in flight)
  auto load_batch = [&](int k0, bf16x8 (&wd)[NT][S], bf16x8 (&ad)[S]) {
    if (VEC && k0 + S * 32 <= k_end) {
#pragma unroll
      for (int s = 0; s < S; ++s) {
#pragma unroll
        for (int j = 0; j < NT; ++j) wd[j][s] = load8_inside(W, ldw, n_ld[j], k0 + s * 32 + kq);
        ad[s] = load8_inside(A, lda, m_row, k0 + s * 32 + kq);
      }
    } else {
      // the slice's last batch: whole steps still go unguarded, the rest is guarded or zero
#pragma unroll
      for (int s = 0; s < S; ++s) {
        const int k = k0 + s * 32;
        if (VEC && k + 32 <= k_end) {
#pragma unroll
          for (int j = 0; j < NT; ++j) wd[j][s] = load8_inside(W, ldw, n_ld[j], k + kq);
          ad[s] = load8_inside(A, lda, m_row, k + kq);
        } else {
#pragma unroll
          for (int j = 0; j < NT; ++j) wd[j][s] = load8<VEC>(W, ldw, n_ld[j], k + kq, k_end);
          ad[s] = load8<VEC>(A, lda, m_row, k + kq, k_end);
        }
      }
    }
  };
  if (k_begin < k_end) load_batch(k_begin, wc, ac);
  for (int k0 = k_begin; k0 < k_end; k0 += S * 32) {
    const bool more = k0 + S * 32 < k_end;
    if (more) load_batch(k0 + S * 32, wn, an);
#pragma unroll
    for (int s = 0; s < S; ++s)
#pragma unroll
      for (int j = 0; j < NT; ++j)
        acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ac[s], wc[j][s], acc[j], 0, 0, 0);
    if (more) {
#pragma unroll
      for (int s = 0; s < S; ++s) {
#pragma unroll
        for (int j = 0; j < NT; ++j) wc[j][s] = wn[j][s];
        ac[s] = an[s];
      }
    }
  }
#pragma unroll
  for (int j = 0; j < NT; ++j)
#pragma unroll
    for (int r = 0; r < 4; ++r) red[wid][j][lane][r] = acc[j][r];
  __syncthreads();
  if (wid != 0) return;
  if (epi == EPI_SWIGLU) {       // tile 0 gate, tile 1 up
    if constexpr (PAIR && NT == 2) {
      const int col = blockIdx.x * 16 + (lane & 15);
      if (col < ldc) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int m = (lane >> 4) * 4 + r;
          if (m >= M) continue;
          float g = 0.f, u = 0.f;
#pragma unroll
          for (int w = 0; w < NW; ++w) { g += red[w][0][lane][r]; u += red[w][1][lane][r]; }
          ((bf16*)C)[(size_t)m * ldc + col] = (bf16)swiglu_f(g, u);
        }
      }
    }
    return;
  }
#pragma unroll
  for (int j = 0; j < NT; ++j) {
    const int n = n_base + 16 * j;
    if (n >= N) continue;
    const float b = bias ? bias[n] : 0.f;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int m = (lane >> 4) * 4 + r;      // D[m][n]: n = lane % 16, m = 4 (lane / 16) + r
      if (m >= M) continue;
      float v = 0.f;
#pragma unroll
      for (int w = 0; w < NW; ++w) v += red[w][j][lane][r];
      store_out(C, ldc, m, n, v + b, epi);
    }
  }
}

// compute units of the current device (0 on error)
static int cu_count() {
  static int n_cu = 0;
  if (n_cu == 0) {
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) return 0;
    n_cu = prop.multiProcessorCount;
  }
  return n_cu;
}

// ---- which shapes each decode kernel takes (the launchers and `mf_gemm_bf16_plan` both ask here)

// K = 256 NS for which the register-resident kernel is instantiated
#define MF_STATIONARY_NS(X) X(4) X(6) X(8) X(10) X(12) X(14) X(16) X(20) X(24) X(28) X(32)

// weights in flight per wave of the register-resident kernel: a whole slice up to NS 16, else the
// largest divisor of NS that leaves the activations (4 NS registers) and the ring within budget
constexpr int stationary_ring(int NS, int NT) {
  if (NS <= 16) return NS;
  for (int r = 10; r > 1; --r)
    if (NS % r == 0 && 4 * NS + 4 * NT * r <= 176) return r;
  return 1;
}

constexpr int STATIONARY_K7 = 896;       // the one K that runs as 7 waves of 4 steps

bool stationary_takes(int M, int N, int K, int epi, bool normed) {
  if (epi == EPI_SWIGLU && N % 64 != 0) return false;
  // (a model that narrow has few weight rows as well, and its steps are their kernels' starts, not
  // the stream: there the fold of the norm is what this kernel is taken for, from 64 tiles on)
  if (K == STATIONARY_K7) return M <= 16 && (N + 15) / 16 >= 64;
  if (M > 16 || (N + 15) / 16 < 128) return false;
  if (K % 256 != 0) return false;
  // a K above 5120 without a norm or SwiGLU to fold in (the o product of the widest models): the
  // rolling kernel is the faster one there
  if (K > 5120 && !normed && epi != EPI_SWIGLU) return false;
  switch (K / 256) {
#define MF_X(NS_) case NS_:
    MF_STATIONARY_NS(MF_X)
#undef MF_X
    return true;
  }
  return false;
}

// one block per CU over the whole of K, for 17 to 64 rows against a matrix that gives every CU at
// least 8 tiles of 16 weight rows
bool panel_takes(int M, int N, int K, bool aligned, int epi, int n_cu) {
  if (M <= 16 || M > 64 || K % 256 != 0 || !aligned) return false;
  if (epi == EPI_SWIGLU && N % 64 != 0) return false;
  return (N + 31) / 32 >= 4 * n_cu;
}

// the ring form of the K-split kernel needs whole chunks of 256 in every split
bool ring_takes(bool aligned, int K, int splits, int k_per_split) {
  return aligned && K % 256 == 0 && (long)(splits - 1) * k_per_split < K;
}

// The RMS norm folded around the products of at most 64 rows, across two kernels (y = x /
// sqrt(mean(x^2) + eps) * g, src/vec_ops.rs:500-522):
//  * a product that adds into the residual stream x and knows the weight g of the norm that reads
//    the stream next leaves, beside the stream's new rows, xg = bf16(x g) and for every row the
//    sums of x^2 in parts (`out_*`): over runs of 256 columns where the kernel that adds the parts
//    of a K split does it (17 to 64 rows: it has every new value of x in its hands), one part per
//    block where a one-kernel product of at most 16 rows does it in its epilogue (every block
//    owns some columns; `out_parts` places a row, the ones past the grid set to zero);
//  * the product that follows takes xg as its activations and multiplies its own sums by the
//    row's 1 / sqrt(sum / K + eps) in its epilogue (`in_*`), the partial sums of squares added up
//    in their order.
// No norm kernel, no pass over the stream between the two products.  The same arithmetic as the
// fold of the register-resident kernel above (bf16(x g) to the matrix cores, the row's factor in
// the epilogue).
constexpr int MF_NOT_BUILT = -2;     // an entry point's answer for a shape it has no kernel for; nothing was launched

struct FusedNorm {
  const float* in_ssq;     // [M][in_parts] partial sums of squares of the rows this product reads (null: none)
  int in_parts;
  float in_eps;
  const float* out_g;      // [N] weight of the norm that reads the output next (null: none)
  bf16* out_xg;            // [M][N]
  float* out_ssq;          // [M][ceil(N / 256)], or [M][out_parts] from a one-kernel product of at most 16 rows
  int out_parts;
};

// 1 / sqrt(mean(x^2) + eps) of NR rows from their partial sums, K the rows' length, in two steps
// so that a kernel can ask for the sums early and use them late; all lanes of a wave call both with
// the same rows (a row outside [0, M) gives 1).  The lanes take the partial sums between them, all
// rows' loads in flight together, and add up in a fixed tree.
template <int NR>
__device__ __forceinline__ void row_sums_ask(const FusedNorm& f, const int (&rows)[NR], int M, int lane, float (&t)[NR]) {
#pragma unroll
  for (int i = 0; i < NR; ++i) {
    t[i] = 0.f;
    if (rows[i] >= 0 && rows[i] < M)
      for (int p = lane; p < f.in_parts; p += 64) t[i] += f.in_ssq[(size_t)rows[i] * f.in_parts + p];
  }
}

template <int NR>
__device__ __forceinline__ void row_factors_of(const FusedNorm& f, const int (&rows)[NR], int M, int K, float (&t)[NR]) {
#pragma unroll
  for (int i = 0; i < NR; ++i) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) t[i] += __shfl_xor(t[i], o, MF_WAVE);
    t[i] = (rows[i] >= 0 && rows[i] < M) ? 1.0f / sqrtf(t[i] / (float)K + f.in_eps) : 1.f;
  }
}


// End of a one-kernel product of at most 16 rows that prepares the next norm (FusedNorm::out_*):
// every lane has the squares of its own outputs of row e_m in `sq` (0 where it has none), the
// COLS lanes of a row sit side by side; their sum is this block's part of the row.  Block 0 also
// sets the places past the grid to zero.
template <int COLS>
__device__ __forceinline__ void norm_part_out(const FusedNorm& f, float sq, int e_m, int e_c, int M) {
#pragma unroll
  for (int o = COLS / 2; o > 0; o >>= 1) sq += __shfl_xor(sq, o, MF_WAVE);
  if (e_c == 0 && e_m < M) f.out_ssq[(size_t)e_m * f.out_parts + blockIdx.x] = sq;
  if (blockIdx.x == 0) {
    const int spare = f.out_parts - (int)gridDim.x;
    for (int i = threadIdx.x; i < M * spare; i += blockDim.x)
      f.out_ssq[(size_t)(i / spare) * f.out_parts + gridDim.x + i % spare] = 0.f;
  }
}

// The same split of the work as skinny16_kernel (a block owns 16 NT weight rows, its waves split
// K), for aligned operands and K a multiple of 32, with the loads rolling: a wave holds S steps
// of weights and activations in registers, and the refill of a register is issued right behind
// the MFMA that read it, so S steps of loads stay in flight the whole time in half the
// registers of the two-buffer scheme above.  With K of many thousands and few weight rows
// (the down projection) the chip is filled by loads in flight, not by blocks, and this is
// what the time depends on.
template <int NW, int NT, int S, bool PAIR, bool TILED>
__global__ __launch_bounds__(NW * 64) void rolling16_kernel(const bf16* __restrict__ A, int lda,
                                                            const bf16* __restrict__ W, int ldw,
                                                            const float* __restrict__ bias,
                                                            void* __restrict__ C, int ldc, int M, int N,
                                                            int K, int steps_per_wave, int epi, int rpb,
                                                            FusedNorm fused) {
  constexpr int COLS = 16 * NT;
  constexpr int RS = COLS + 4;
  constexpr int WSTEP = TILED ? 512 : 32;
  __shared__ float red[NW][16][RS];
  const int lane = threadIdx.x & 63;
  const int wid = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);     // the same in the whole wave
  const int r16 = lane & 15;
  // rpb: weight rows per block (at most 16 NT; fewer when that spreads the rows over every CU:
  // a CU draws only so much from memory, so an idle CU is bandwidth lost).  Lanes past the
  // block's rows read its last row again, from the CU's own cache.
  auto tile_row = [&](int j) {
    return PAIR ? (blockIdx.x >> 1) * 64 + (blockIdx.x & 1) * 16 + j * 32 : blockIdx.x * rpb + j * 16;
  };
  auto lane_row = [&](int j) {           // the weight row this lane reads in tile j
    return PAIR ? tile_row(j) + r16 : blockIdx.x * rpb + min(j * 16 + r16, rpb - 1);
  };
  const int total = K / 32;
  const int first = min(wid * steps_per_wave, total);
  const int T = min(steps_per_wave, total - first);       // steps of this wave
  const int kq = first * 32 + (lane >> 4) * 8;
  const bf16* arow = A + (size_t)min(r16, M - 1) * lda + kq;
  const bf16* wrow[NT];
#pragma unroll
  for (int j = 0; j < NT; ++j) wrow[j] = w_operand<TILED>(W, ldw, K, min(lane_row(j), N - 1), kq);
  floatx4 acc[NT];
#pragma unroll
  for (int j = 0; j < NT; ++j) acc[j] = floatx4{0.f, 0.f, 0.f, 0.f};
  // The epilogue's place of this lane: wave w adds up the sums of activation rows
  // [w 64 / COLS, (w + 1) 64 / COLS), every wave one pass at the same time.  Where the product is
  // added to what the output holds, the old value is asked for here, in front of the whole stream:
  // behind it, its way from memory would be the kernel's tail, once per pass.
  constexpr int ROWS_PER_PASS = 64 / COLS;
  static_assert(NW * ROWS_PER_PASS >= 16, "a pass for every activation row");
  const int e_c = lane % COLS;
  const int e_n = tile_row(e_c >> 4) + (e_c & 15);
  const int e_m = wid * ROWS_PER_PASS + lane / COLS;
  const bool e_mine = e_m < M && e_n < N && (PAIR || e_c < rpb);
  float c_old = 0.f, e_g = 0.f;
  if (epi == EPI_ACC_F32 && e_mine) c_old = ((const float*)C)[(size_t)e_m * ldc + e_n];
  if (fused.out_g && e_mine) e_g = fused.out_g[e_n];       // the next norm's weight, where this product prepares it
  const int R = T / S, rem = T % S;
  if (R == 0) {       // a slice shorter than the registers hold: step by step
    for (int s = 0; s < T; ++s) {
      const bf16x8 a1 = *reinterpret_cast<const bf16x8*>(arow + s * 32);
#pragma unroll
      for (int j = 0; j < NT; ++j)
        acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
            a1, *reinterpret_cast<const bf16x8*>(wrow[j] + s * WSTEP), acc[j], 0, 0, 0);
    }
  } else {
    bf16x8 a[S], w[NT][S];
#pragma unroll
    for (int s = 0; s < S; ++s) {
      a[s] = *reinterpret_cast<const bf16x8*>(arow + s * 32);
#pragma unroll
      for (int j = 0; j < NT; ++j) w[j][s] = *reinterpret_cast<const bf16x8*>(wrow[j] + s * WSTEP);
    }
    // rounds whose refills all exist: no branch in the body
    int base = 0;
    for (int i = 0; i + 1 < R; ++i, base += S) {
#pragma unroll
      for (int s = 0; s < S; ++s) {
#pragma unroll
        for (int j = 0; j < NT; ++j) {
          acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[s], w[j][s], acc[j], 0, 0, 0);
          w[j][s] = *reinterpret_cast<const bf16x8*>(wrow[j] + (base + S + s) * WSTEP);
        }
        a[s] = *reinterpret_cast<const bf16x8*>(arow + (base + S + s) * 32);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    // the last whole round refills only what the remainder needs
#pragma unroll
    for (int s = 0; s < S; ++s) {
#pragma unroll
      for (int j = 0; j < NT; ++j) acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[s], w[j][s], acc[j], 0, 0, 0);
      if (s < rem) {
        a[s] = *reinterpret_cast<const bf16x8*>(arow + (base + S + s) * 32);
#pragma unroll
        for (int j = 0; j < NT; ++j) w[j][s] = *reinterpret_cast<const bf16x8*>(wrow[j] + (base + S + s) * WSTEP);
      }
    }
#pragma unroll
    for (int s = 0; s < S; ++s) {
      if (s < rem) {
#pragma unroll
        for (int j = 0; j < NT; ++j) acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[s], w[j][s], acc[j], 0, 0, 0);
      }
    }
  }
  // D[m][n]: n = lane % 16, m = 4 (lane / 16) + r
#pragma unroll
  for (int j = 0; j < NT; ++j)
#pragma unroll
    for (int r = 0; r < 4; ++r) red[wid][(lane >> 4) * 4 + r][j * 16 + r16] = acc[j][r];
  __syncthreads();
  if (epi == EPI_SWIGLU) {
    if constexpr (PAIR && NT == 2) {
      const int col = blockIdx.x * 16 + r16;
      const int m = wid * 4 + (lane >> 4);
      if (col < ldc && m < M) {
        float g = 0.f, u = 0.f;
#pragma unroll
        for (int ww = 0; ww < NW; ++ww) { g += red[ww][m][r16]; u += red[ww][m][16 + r16]; }
        ((bf16*)C)[(size_t)m * ldc + col] = (bf16)swiglu_f(g, u);
      }
    }
    return;
  }
  float sq = 0.f;
  if (e_mine) {
    float v = bias ? bias[e_n] : 0.f;
#pragma unroll
    for (int ww = 0; ww < NW; ++ww) v += red[ww][e_m][e_c];
    if (epi == EPI_ACC_F32) v += c_old;
    if (epi == EPI_ACC_F32) ((float*)C)[(size_t)e_m * ldc + e_n] = v;
    else store_out(C, ldc, e_m, e_n, v, epi);
    if (fused.out_g) {
      fused.out_xg[(size_t)e_m * ldc + e_n] = (bf16)(v * e_g);
      sq = v * v;
    }
  }
  if (fused.out_g) norm_part_out<COLS>(fused, sq, e_m, e_c, M);
}

template <int NW, int NT, int S, bool PAIR = false, bool TILED = false>
int launch_rolling16(const bf16* A, int lda, const bf16* W, int ldw, const float* bias, void* C, int ldc,
                     int M, int N, int K, int epi, hipStream_t stream, const FusedNorm& fused = FusedNorm{}) {
  const int steps_per_wave = (K / 32 + NW - 1) / NW;
  int rpb = 16 * NT, blocks = N / 32;
  if (!PAIR) {
    const int n_cu = cu_count();
    if (n_cu <= 0) return (int)hipErrorUnknown;
    rpb = (N + n_cu - 1) / n_cu;                 // one block per CU when the rows are few
    rpb = rpb < 1 ? 1 : (rpb > 16 * NT ? 16 * NT : rpb);
    blocks = (N + rpb - 1) / rpb;
  }
  if (fused.out_g && (PAIR || blocks > fused.out_parts)) return MF_NOT_BUILT;
  rolling16_kernel<NW, NT, S, PAIR, TILED><<<blocks, NW * 64, 0, stream>>>(A, lda, W, ldw, bias, C, ldc, M, N, K,
                                                                           steps_per_wave, epi, rpb, fused);
  return mf_launch_status();
}

template <int NW, int NT, int S, bool PAIR = false>
int launch_skinny16(const bf16* A, int lda, const bf16* W, int ldw, const float* bias, void* C, int ldc,
                    int M, int N, int K, int epi, int vec_ok, hipStream_t stream) {
  const int k_per_wave = ((K + NW - 1) / NW + 31) / 32 * 32;      // even shares; a slice's last batch may be short
  const int blocks = (N + 16 * NT - 1) / (16 * NT);
  if (vec_ok)
    skinny16_kernel<NW, NT, S, true, PAIR><<<blocks, NW * 64, 0, stream>>>(A, lda, W, ldw, bias, C, ldc, M, N,
                                                                           K, k_per_wave, epi);
  else
    skinny16_kernel<NW, NT, S, false, PAIR><<<blocks, NW * 64, 0, stream>>>(A, lda, W, ldw, bias, C, ldc, M,
                                                                            N, K, k_per_wave, epi);
  return mf_launch_status();
}

// At most 16 rows and K = 256 NS (NS steps of 32 k for each of 8 waves): the activations are
// read once per block and stay in registers.  The grid is one block per CU; a block walks
// over its share of the 16-row weight tiles (items), and the load of the next item's
// weights is issued right behind the MFMA that frees the register, so the weight stream
// never pauses between items.  After an item the waves' sums meet in LDS (two buffers, one
// barrier per item) and the waves take turns at adding them and running the epilogue.
// Against the kernel above this removes the per-tile re-read of the activations (which
// cost a quarter of the time at 8 rows) and the start-up of a block per tile.
//
// NORM: the activations are rows of the 32-bit residual stream, to be RMS-normalised on the way
// in (y = x / sqrt(mean(x^2) + eps) * g, src/vec_ops.rs:500-522).  The 1 / sqrt(..) is one
// number per row, so it can wait for the epilogue: the matrix cores get bf16(x * g), every
// wave sums x^2 over its own slice of K while it converts, and the epilogue multiplies the
// row's sums by 1 / sqrt(total / K + eps).  No pass over the row beforehand, no kernel and no
// activation buffer between the norm and the product.
struct NormArgs {
  const float* g;          // [K] norm weight
  const int* row_idx;      // activation row m is residual row row_idx[m] (null: m)
  float eps;
};

//
// RING: how many of a slice's NS steps of weights a wave keeps in flight (a divisor of NS).  With
// RING = NS the registers hold a whole item; for a long K (5120, 8192) the activations alone take
// up to half the registers, so the weights go through a shorter ring, and a register is refilled
// with the step RING further on, of this item or of the next one.
// NW: waves of a block, each with a slice of NS steps of K: 8, K = 256 NS; or 7 with NS = 4 for a K
// of 896 (14 heads of 64, the narrowest model of the family), which is no multiple of 256.
template <int NS, int RING, int NT, bool PAIR, bool NORM, bool TILED, int NW = 8>
__global__ __launch_bounds__(NW * 64) void stationary16_kernel(const void* __restrict__ Av, int lda,
                                                               const bf16* __restrict__ W, int ldw,
                                                               const float* __restrict__ bias,
                                                               void* __restrict__ C, int ldc, int M, int N,
                                                               int cols_total, int unit, int share, int extra, int epi,
                                                               NormArgs norm, FusedNorm fused) {
  constexpr int KK = NW * NS * 32;         // K
  constexpr int WSTEP = TILED ? 512 : 32;  // elements from one step's weights to the next's
  constexpr int COLS = 16 * NT;            // weight rows (output columns) of an item
  constexpr int RS = COLS + 4;             // row stride of the sums in LDS: conflict-free writes
  __shared__ float red[2][NW][16][RS];     // [buffer][wave][activation row][weight row of the item]
  __shared__ float ssq[NW][16];            // NORM: sum of x^2 over a wave's slice, per activation row
  __shared__ float rfac[16];               // not NORM: the rows' factors of a norm prepared by the product before (1 where none)
  extern __shared__ __attribute__((aligned(16))) float gs[];   // NORM: the norm's weight, K floats
  static_assert(NS % RING == 0, "the ring divides a slice");
  static_assert(PAIR ? NW * 4 >= 16 : NW * (64 / COLS) >= 16, "an epilogue pass for every activation row");
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
  const int r16 = lane & 15;
  const int k0 = wid * NS * 32 + (lane >> 4) * 8;         // this lane's k in step 0 of its slice
  // The block's share: output columns [c_begin, c_end), the same number for every block up to
  // one `unit`, so that every CU streams the same bytes (a CU draws only so much from memory;
  // whole items per block would leave some with a fifth more than others).  PAIR: a column is
  // a gate row and the up row 32 further on, in groups of 64 weight rows.  An item is CH
  // columns; lanes past c_end read the share's last row again, from the CU's own cache.
  // (`share` units a block and one more for the first `extra` blocks: the host has divided, so
  // that a block's first loads do not wait behind a division in software)
  constexpr int CH = PAIR ? 16 : COLS;
  const int b = blockIdx.x;
  const int c_begin = (b * share + min(b, extra)) * unit;
  const int c_end = min(((b + 1) * share + min(b + 1, extra)) * unit, cols_total);
  const int n_items = (c_end - c_begin + CH - 1) / CH;
  auto lane_wrow = [&](int c0, int j) {      // weight row of this lane in tile j of the item at c0
    if (PAIR) {
      const int col = min(c0 + r16, c_end - 1);
      return (col >> 5) * 64 + (col & 31) + 32 * j;
    }
    return min(c0 + 16 * j + r16, c_end - 1);
  };
  const bf16* Wp = W;            // the weights, through a name whose use can be held back
  bf16x8 w[NT][RING];
  const bf16* wrow[NT];          // this lane's rows in the next item
  const bf16* wcur[NT];          // and in the current one (used when RING < NS)
  // The first item's loads are asked for without a condition (every block has an item: the grid is
  // no larger than the units to share): a load behind a branch makes the compiler count, for every
  // wait after it, with the path that has fewer loads in flight, and the prologue would wait for
  // the activations until most of the first weights have arrived as well.
  auto first_loads = [&](int j) {
    wcur[j] = w_operand<TILED>(Wp, ldw, KK, lane_wrow(c_begin, j), k0);
#pragma unroll
    for (int s = 0; s < RING; ++s) w[j][s] = *reinterpret_cast<const bf16x8*>(wcur[j] + s * WSTEP);
  };
  bf16x8 afr[NS];
  float ss = 0.f;
  if constexpr (NORM) {
    const int m_src = min(r16, M - 1);
    const float* xrow = (const float*)Av + (size_t)(norm.row_idx ? norm.row_idx[m_src] : m_src) * lda + k0;
    // step s of the slice: sum of squares, and bf16(x * g) into the operand registers
    auto convert_step = [&](int s, const float4 x0, const float4 x1) {
      const float4 g0 = *reinterpret_cast<const float4*>(&gs[k0 + s * 32]);
      const float4 g1 = *reinterpret_cast<const float4*>(&gs[k0 + s * 32 + 4]);
      ss = fmaf(x0.x, x0.x, ss); ss = fmaf(x0.y, x0.y, ss); ss = fmaf(x0.z, x0.z, ss); ss = fmaf(x0.w, x0.w, ss);
      ss = fmaf(x1.x, x1.x, ss); ss = fmaf(x1.y, x1.y, ss); ss = fmaf(x1.z, x1.z, ss); ss = fmaf(x1.w, x1.w, ss);
      afr[s][0] = (bf16)(x0.x * g0.x); afr[s][1] = (bf16)(x0.y * g0.y);
      afr[s][2] = (bf16)(x0.z * g0.z); afr[s][3] = (bf16)(x0.w * g0.w);
      afr[s][4] = (bf16)(x1.x * g1.x); afr[s][5] = (bf16)(x1.y * g1.y);
      afr[s][6] = (bf16)(x1.z * g1.z); afr[s][7] = (bf16)(x1.w * g1.w);
      // the packed value is wanted here and now (left alone, the compiler keeps x and g
      // alive and converts in front of the first MFMA, at twice the registers)
      // (and for a long row the sum as well: put off, it keeps x alive in 32 bits)
      if constexpr (NS <= 16) asm volatile("" : "+v"(afr[s]));
      else asm volatile("" : "+v"(afr[s]), "+v"(ss));
    };
    if constexpr (NS <= 16) {
      // Everything the prologue needs is asked for at once, oldest first in the order it is
      // used: the norm's weight (staged in LDS for all waves), this lane's x, and the first
      // item's tile 0, which keeps HBM at work while the activations are converted.  The order is
      // pinned: left alone, the compiler asks for the weights first and then waits for them
      // before it stages g.
      static_assert(NS > 16 || NW * NS * 32 <= 2 * NW * 64 * 4, "two float4 of g per thread cover K");
      const int ge0 = min((int)threadIdx.x * 4, NW * NS * 32 - 4);                 // the last ones twice
      const int ge1 = min((NW * 64 + (int)threadIdx.x) * 4, NW * NS * 32 - 4);
      const float4 gt0 = *reinterpret_cast<const float4*>(norm.g + ge0);
      const float4 gt1 = *reinterpret_cast<const float4*>(norm.g + ge1);
      float4 x[NS][2];
#pragma unroll
      for (int s = 0; s < NS; ++s) {
        x[s][0] = *reinterpret_cast<const float4*>(xrow + s * 32);
        x[s][1] = *reinterpret_cast<const float4*>(xrow + s * 32 + 4);
      }
      __builtin_amdgcn_sched_barrier(0);
      first_loads(0);
      __builtin_amdgcn_sched_barrier(0);
      *reinterpret_cast<float4*>(&gs[ge0]) = gt0;
      *reinterpret_cast<float4*>(&gs[ge1]) = gt1;
      __syncthreads();
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int s = 0; s < NS; ++s) convert_step(s, x[s][0], x[s][1]);
    } else {
      // A long row does not fit the registers in 32 bits beside its own bf16 copy: x comes in
      // sets of XC steps, the next set asked for before this one is converted, and the first
      // weights wait until the activations are in place.
      constexpr int XC = 4, SETS = NS / XC;
      static_assert(NS % XC == 0, "whole sets");
      float4 x[2][XC][2];
      const float* xp = xrow;
      auto load_set = [&](int c, int b) {
#pragma unroll
        for (int i = 0; i < XC; ++i) {
          x[b][i][0] = *reinterpret_cast<const float4*>(xp + (c * XC + i) * 32);
          x[b][i][1] = *reinterpret_cast<const float4*>(xp + (c * XC + i) * 32 + 4);
        }
      };
      load_set(0, 0);
      for (int e = (int)threadIdx.x * 4; e < NW * NS * 32; e += NW * 64 * 4)
        *reinterpret_cast<float4*>(&gs[e]) = *reinterpret_cast<const float4*>(norm.g + e);
      __syncthreads();
#pragma unroll
      for (int c = 0; c < SETS; ++c) {
        if (c + 1 < SETS) load_set(c + 1, (c + 1) & 1);
#pragma unroll
        for (int i = 0; i < XC; ++i) convert_step(c * XC + i, x[c & 1][i][0], x[c & 1][i][1]);
        // the address of the sets further on hangs on this set's last operand: asked for all at
        // once (which is what the compiler does with loads off one pointer) the row in 32 bits
        // would not fit the registers
        asm volatile("" : "+v"(xp), "+v"(afr[c * XC + XC - 1]));
        __builtin_amdgcn_sched_barrier(0);
      }
      asm volatile("" : "+s"(Wp), "+v"(afr[NS - 1]));     // no weights before the activations are in place
      first_loads(0);
    }
    ss += __shfl_xor(ss, 16);
    ss += __shfl_xor(ss, 32);
    if (lane < 16) ssq[wid][lane] = ss;    // read behind the first item's barrier
    __builtin_amdgcn_sched_barrier(0);
  } else {
    const bf16* arow = (const bf16*)Av + (size_t)min(r16, M - 1) * lda + k0;
#pragma unroll
    for (int s = 0; s < NS; ++s) afr[s] = *reinterpret_cast<const bf16x8*>(arow + s * 32);
  }
  // Not NORM: the activations may be bf16(x g) of rows whose sums of squares the product before has
  // left in parts (FusedNorm::in_*): wave w adds up rows w, w + NW, ..., asked for here, between the
  // activations and the first weights, and used behind them; the epilogue multiplies by the factors.
  constexpr int FR = (16 + NW - 1) / NW;
  int frow[FR];
  float ffac[FR];
#pragma unroll
  for (int i = 0; i < FR; ++i) frow[i] = (!NORM && fused.in_ssq && wid + NW * i < 16) ? wid + NW * i : -1;
  if constexpr (!NORM) {
    row_sums_ask<FR>(fused, frow, M, lane, ffac);
    __builtin_amdgcn_sched_barrier(0);
    first_loads(0);
  }
#pragma unroll
  for (int j = 1; j < NT; ++j) first_loads(j);
  if constexpr (!NORM) {
    row_factors_of<FR>(fused, frow, M, KK, ffac);
    if (lane == 0)
#pragma unroll
      for (int i = 0; i < FR; ++i)
        if (wid + NW * i < 16) rfac[wid + NW * i] = ffac[i];       // read behind the first item's barrier
  }
  float sq = 0.f;                      // a product that prepares the next norm: squares of this lane's outputs
  for (int it = 0; it < n_items; ++it) {
    // The loop body has no branch, so that the compiler can count the loads in flight and wait
    // for the oldest one only: behind the last item the loads go to the head of the matrix,
    // the same few lines for every lane, and their values are dropped.
    const int c0 = c_begin + it * CH;
    const bool has_next = it + 1 < n_items;
#pragma unroll
    for (int j = 0; j < NT; ++j)
      wrow[j] = w_operand<TILED>(Wp, ldw, KK, has_next ? lane_wrow(c0 + CH, j) : 0, k0);
    floatx4 acc[NT];
#pragma unroll
    for (int j = 0; j < NT; ++j) acc[j] = floatx4{0.f, 0.f, 0.f, 0.f};
    // The epilogue's place of this lane in this item: wave w adds up the sums of activation rows
    // [w 64 / COLS, (w + 1) 64 / COLS), all waves at once.  What the epilogue needs from memory (the
    // bias, and the output's old value where the product is added to it) is asked for here, in
    // front of the item's refills and without a condition (a lane with no place, or no such
    // operand, reads the head of the weights and drops it): behind the barrier it would make
    // the wave wait for every load it has in flight, and the kernel's last item for memory.
    const int e_c = lane % COLS;
    const int e_n = c0 + e_c;
    const int e_m = wid * (64 / COLS) + lane / COLS;
    const bool e_mine = !PAIR && e_n < c_end && e_m < M;
    float c_old = 0.f, e_bias = 0.f, e_g = 0.f;
    if constexpr (!PAIR) {
      const float* dummy = reinterpret_cast<const float*>(W);
      c_old = *((e_mine && epi == EPI_ACC_F32) ? (const float*)C + (size_t)e_m * ldc + e_n : dummy);
      e_bias = *((e_mine && bias) ? bias + e_n : dummy);
      e_g = *((e_mine && fused.out_g) ? fused.out_g + e_n : dummy);
    }
#pragma unroll
    for (int s = 0; s < NS; ++s) {
#pragma unroll
      for (int j = 0; j < NT; ++j) {
        acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(afr[s], w[j][s % RING], acc[j], 0, 0, 0);
        // the step RING further on: of this item, or of the next one.  (The load stays behind
        // the MFMA: moved in front of it, it needs a register of its own.)
        if constexpr (RING < NS) {
          asm volatile("" : "+v"(acc[j]) : : "memory");
          __builtin_amdgcn_sched_barrier(0);
        }
        w[j][s % RING] = s + RING < NS ? *reinterpret_cast<const bf16x8*>(wcur[j] + (s + RING) * WSTEP)
                                       : *reinterpret_cast<const bf16x8*>(wrow[j] + (s + RING - NS) * WSTEP);
        __builtin_amdgcn_sched_barrier(0);      // keep "use a register, then refill it" in this order
      }
      // (held here, or the compiler moves the two loads to where they are used)
      if (s == 0) asm volatile("" : "+v"(c_old), "+v"(e_bias), "+v"(e_g));
    }
#pragma unroll
    for (int j = 0; j < NT; ++j) wcur[j] = wrow[j];
    // D[m][n]: n = lane % 16, m = 4 (lane / 16) + r
    const int buf = it & 1;
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int r = 0; r < 4; ++r) red[buf][wid][(lane >> 4) * 4 + r][j * 16 + r16] = acc[j][r];
    __syncthreads();
    // The buffer is written again two items on, behind the next barrier, which this wave
    // reaches only after it has read its sums here.
    auto row_scale = [&](int m) {          // NORM: 1 / sqrt(mean(x^2) + eps) of activation row m
      float t = 0.f;
#pragma unroll
      for (int ww = 0; ww < NW; ++ww) t += ssq[ww][m];
      return 1.0f / sqrtf(t / (float)(NW * NS * 32) + norm.eps);
    };
    if constexpr (PAIR) {
      static_assert(NT == 2, "a gate tile and an up tile");
      const int col = c0 + r16;
      const int m = wid * 4 + (lane >> 4);
      if (epi == EPI_SWIGLU && col < c_end && col < ldc && m < M) {
        float g = 0.f, u = 0.f;
#pragma unroll
        for (int ww = 0; ww < NW; ++ww) { g += red[buf][ww][m][r16]; u += red[buf][ww][m][16 + r16]; }
        const float sc = NORM ? row_scale(m) : rfac[m];
        g *= sc;
        u *= sc;
        ((bf16*)C)[(size_t)m * ldc + col] = (bf16)swiglu_f(g, u);
      }
    } else {
      if (e_mine) {
        float v = 0.f;
#pragma unroll
        for (int ww = 0; ww < NW; ++ww) v += red[buf][ww][e_m][e_c];
        v *= NORM ? row_scale(e_m) : rfac[e_m];
        v += (bias ? e_bias : 0.f);
        if (epi == EPI_ACC_F32) v += c_old;
        if (epi == EPI_ACC_F32) ((float*)C)[(size_t)e_m * ldc + e_n] = v;
        else store_out(C, ldc, e_m, e_n, v, epi);
        if (fused.out_g) {
          fused.out_xg[(size_t)e_m * ldc + e_n] = (bf16)(v * e_g);
          sq = fmaf(v, v, sq);
        }
      }
    }
  }
  if constexpr (!PAIR)
    if (fused.out_g) norm_part_out<COLS>(fused, sq, wid * (64 / COLS) + lane / COLS, lane % COLS, M);
}

// true when the shape is one the register-resident kernel is built for
template <int NS, int NT, bool PAIR, bool TILED, int NW = 8>
int launch_stationary16(const void* A, int lda, const bf16* W, int ldw, const float* bias, void* C, int ldc,
                        int M, int N, int epi, const NormArgs* norm, const FusedNorm& fused, hipStream_t stream) {
  const int n_cu = cu_count();
  if (n_cu <= 0) return (int)hipErrorUnknown;
  const int cols_total = PAIR ? N / 2 : N;
  // shares in whole 128-byte lines of 32-bit output where the output is large enough for the
  // cost of partial lines to show; else in pairs of columns
  const int unit = (!PAIR && cols_total / 32 >= 8 * n_cu) ? 32 : 2;
  const int units = (cols_total + unit - 1) / unit;
  const int grid = units < n_cu ? units : n_cu;
  // registers: 4 NS for the activations and 4 NT RING for the weights in flight, of 256.  A long
  // K keeps 8 to 10 loads of 1 KB in flight per wave, far more than a CU has outstanding anyway.
  constexpr int RING = stationary_ring(NS, NT);
  static_assert(NS % RING == 0 && 4 * NS + 4 * NT * RING <= 200, "activations and weight ring fit the registers");
  if (norm) {
    constexpr int smem = NW * NS * 32 * (int)sizeof(float);      // the norm's weight
    auto kern = stationary16_kernel<NS, RING, NT, PAIR, true, TILED, NW>;
    static bool configured = false;
    if (!configured) {
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, smem);
      if (e != hipSuccess) return (int)e;
      configured = true;
    }
    if (fused.in_ssq || fused.out_g) return MF_NOT_BUILT;
    kern<<<grid, NW * 64, smem, stream>>>(A, lda, W, ldw, bias, C, ldc, M, N, cols_total, unit, units / grid, units % grid,
                                      epi, *norm, FusedNorm{});
  } else {
    if (fused.out_g && (PAIR || grid > fused.out_parts)) return MF_NOT_BUILT;
    stationary16_kernel<NS, RING, NT, PAIR, false, TILED, NW><<<grid, NW * 64, 0, stream>>>(A, lda, W, ldw, bias, C, ldc, M, N,
                                                                             cols_total, unit, units / grid,
                                                                             units % grid, epi,
                                                                             NormArgs{nullptr, nullptr, 0.f}, fused);
  }
  return mf_launch_status();
}

// 17 to 64 rows against a wide matrix (at least 8 tiles of 16 weight rows for every CU): one block
// per CU with an equal share of the matrix, the whole of K, no partial sums between blocks and no
// second kernel.  The share is cut into passes of at most 16 tiles; wave w multiplies tiles w and
// w + 8 of the pass.  A slot with no tile multiplies the matrix's first bytes, read by all lanes
// alike, and its sums are dropped: every wave runs the same instructions, so the loads in flight
// can be counted, and such a load is one look-up in the CU's cache where a tile's (64 lanes in
// 16 rows) is 64 -- repeating a real tile there made the cache's tag rate the limit.  Weights go
// from HBM straight into MFMA operands through a ring of 16 fragments a wave: the load of the
// next chunk's fragment is issued right behind the MFMA that frees the register, and runs on
// into the next pass (a ring of two chunks measured the same).  The activations of a chunk
// (256 k) are staged in LDS once per block, double-buffered, as in skinny_kernel; a pass re-reads
// them from L2.  At the end of a pass the sums go through an LDS tile so that rows are stored in
// whole lines, and SwiGLU pairs a gate tile with its up tile there.  (Folding the RMS norm into
// the staging, as the 16-row kernel does, measured slower here: every block would re-read the
// activations in 32 bits.)
constexpr int PANEL_TILES = 16;                 // tiles of a pass
constexpr int OT_LD = PANEL_TILES * 16 + 4;     // row stride of the output tile in LDS (floats)

template <int MT, bool TILED>
__global__ __launch_bounds__(512) void panel_kernel(const bf16* __restrict__ A, int lda,
                                                    const bf16* __restrict__ W, int ldw,
                                                    const float* __restrict__ bias, void* __restrict__ C,
                                                    int ldc, int M, int N, int K, int units_total, int epi,
                                                    FusedNorm fused) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  constexpr int ROWS = MT * 16;
  bf16* As = reinterpret_cast<bf16*>(smem);                                            // [2][ROWS][SK_LD]
  float* ot = reinterpret_cast<float*>(smem + 2 * ROWS * SK_LD * sizeof(bf16));        // [ROWS][OT_LD]
  __shared__ float rfac[ROWS];                 // the rows' norm factors (1 where no norm is folded in)
  const int tid = threadIdx.x, lane = tid & 63, wid = tid >> 6;

  const int r16 = lane & 15, kq = (lane >> 4) * 8;
  constexpr int WSTEP = TILED ? 512 : 32;
  const bool pair = epi == EPI_SWIGLU;
  // a unit is 32 weight rows: 32 outputs, or (pair) 16 gate rows and the 16 up rows of the same outputs
  const int u_begin = (int)((long)blockIdx.x * units_total / gridDim.x);
  const int u_end = (int)((long)(blockIdx.x + 1) * units_total / gridDim.x);
  const int n_u = u_end - u_begin;
  if (n_u <= 0) return;
  const int n_pass = (2 * n_u + PANEL_TILES - 1) / PANEL_TILES;
  const int per_u = (n_u + n_pass - 1) / n_pass;          // units of a pass (the last may have fewer)
  const int nch = K / KC;
  // what this lane reads for slot j of pass p, as a pointer at chunk 0
  auto slot_ptr = [&](int p, int j) -> const bf16* {
    if (p >= n_pass) return W;                             // behind the last pass: dropped
    const int cnt = 2 * min(per_u, n_u - p * per_u);       // tiles of the pass
    const int t = wid + 8 * j;
    if (t >= cnt) return W;                                // no tile
    const int u = u_begin + p * per_u + (t >> 1), which = t & 1;
    const int row0 = pair ? (u >> 1) * 64 + (u & 1) * 16 + 32 * which : u * 32 + 16 * which;
    return w_operand<TILED>(W, ldw, K, min(row0 + r16, N - 1), kq);
  };
  // staging: this thread handles rows i * 16 + tid / 32, k (tid % 32) * 8 of a chunk
  const int sk = (tid & 31) * 8;
  const bf16* src[MT];
#pragma unroll
  for (int i = 0; i < MT; ++i) src[i] = A + (size_t)min(i * 16 + (tid >> 5), M - 1) * lda + sk;
  bf16x8 stage[MT];
  auto load_stage = [&](int k0) {
#pragma unroll
    for (int i = 0; i < MT; ++i) stage[i] = *reinterpret_cast<const bf16x8*>(src[i] + k0);
  };
  auto store_stage = [&](int buf) {
#pragma unroll
    for (int i = 0; i < MT; ++i)
      *reinterpret_cast<bf16x8*>(&As[(buf * ROWS + i * 16 + (tid >> 5)) * SK_LD + sk]) = stage[i];
  };

  const bf16* wp[2] = {slot_ptr(0, 0), slot_ptr(0, 1)};
  bf16x8 wr[2][KC / 32];
  load_stage(0);
  // the rows' norm factors: wave w has rows w, w + 8, ...  Their partial sums are asked for between
  // the first activations and the first weights and used behind the activations' staging, so that
  // nothing the weight stream needs waits for them.
  int frow[2 * MT];
  float ffac[2 * MT];
#pragma unroll
  for (int i = 0; i < 2 * MT; ++i) frow[i] = fused.in_ssq ? wid + 8 * i : -1;
  row_sums_ask<2 * MT>(fused, frow, M, lane, ffac);
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int s = 0; s < KC / 32; ++s) {
    wr[0][s] = *reinterpret_cast<const bf16x8*>(wp[0] + s * WSTEP);
    wr[1][s] = *reinterpret_cast<const bf16x8*>(wp[1] + s * WSTEP);
  }
  __builtin_amdgcn_sched_barrier(0);
  store_stage(0);
  row_factors_of<2 * MT>(fused, frow, M, K, ffac);
  if (lane == 0)
#pragma unroll
    for (int i = 0; i < 2 * MT; ++i) rfac[wid + 8 * i] = ffac[i];
  __syncthreads();
  floatx4 acc[2][MT];
#pragma unroll
  for (int j = 0; j < 2; ++j)
#pragma unroll
    for (int i = 0; i < MT; ++i) acc[j][i] = floatx4{0.f, 0.f, 0.f, 0.f};
  int buf = 0, pass = 0, kc = 0;
  const int total = n_pass * nch;
  for (int t = 0; t < total; ++t) {
    // the next step: the pass's next chunk, or chunk 0 of the next pass
    const bool last_chunk = kc + 1 == nch;
    const int kn = last_chunk ? 0 : (kc + 1) * KC;
    const bf16* wnext[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) wnext[j] = last_chunk ? slot_ptr(pass + 1, j) : wp[j];
    load_stage(kn);
    __builtin_amdgcn_sched_barrier(0);
    const bf16* as = As + buf * ROWS * SK_LD;
#pragma unroll
    for (int s = 0; s < KC / 32; ++s) {
      bf16x8 a[MT];
#pragma unroll
      for (int i = 0; i < MT; ++i)
        a[i] = *reinterpret_cast<const bf16x8*>(&as[(i * 16 + r16) * SK_LD + s * 32 + kq]);
#pragma unroll
      for (int j = 0; j < 2; ++j) {
#pragma unroll
        for (int i = 0; i < MT; ++i)
          acc[j][i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i], wr[j][s], acc[j][i], 0, 0, 0);
        wr[j][s] = *reinterpret_cast<const bf16x8*>(wnext[j] + ((kn >> 5) + s) * WSTEP);
        __builtin_amdgcn_sched_barrier(0);      // use a register, then refill it, in this order
      }
    }
    store_stage(buf ^ 1);
    buf ^= 1;
    __syncthreads();        // the next chunk is staged
    if (!last_chunk) {
      ++kc;
      continue;
    }
    // ---- end of a pass
    const int cnt = 2 * min(per_u, n_u - pass * per_u);
    // D[m][n]: n = lane % 16, m = 4 (lane / 16) + r
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int tl = wid + 8 * j;
      if (tl < cnt) {
#pragma unroll
        for (int i = 0; i < MT; ++i)
#pragma unroll
          for (int r = 0; r < 4; ++r)
            ot[(i * 16 + (lane >> 4) * 4 + r) * OT_LD + tl * 16 + r16] = acc[j][i][r];
      }
#pragma unroll
      for (int i = 0; i < MT; ++i) acc[j][i] = floatx4{0.f, 0.f, 0.f, 0.f};
    }
    __syncthreads();        // the tile is whole; the next pass writes it behind its own barriers
    {
      const int c = tid & 255;
      const int u0 = u_begin + pass * per_u;
      if (pair) {
        const int col = u0 * 16 + c;                       // unit c / 16 holds gate at 32 (c / 16), up 16 further
        if (c < cnt * 8 && col < ldc) {
          const int o = (c >> 4) * 32 + (c & 15);
          for (int m = tid >> 8; m < M; m += 2)
            ((bf16*)C)[(size_t)m * ldc + col] = (bf16)swiglu_f(ot[m * OT_LD + o] * rfac[m], ot[m * OT_LD + o + 16] * rfac[m]);
        }
      } else {
        const int col = u0 * 32 + c;
        if (c < cnt * 16 && col < N) {
          const float b = bias ? bias[col] : 0.f;
          for (int m = tid >> 8; m < M; m += 2) store_out(C, ldc, m, col, ot[m * OT_LD + c] * rfac[m] + b, epi);
        }
      }
    }
    wp[0] = wnext[0];
    wp[1] = wnext[1];
    ++pass;
    kc = 0;
  }
}

// The parts of a split are added in rounds of up to eight, a round's loads in flight together, in
// the order of the splits (a plain loop over a count that is not known here is left to run split
// by split, a trip to memory each).
template <int CNT>
__device__ __forceinline__ float add_parts(float v, const float* __restrict__ p, size_t stride) {
  float x[CNT];
#pragma unroll
  for (int j = 0; j < CNT; ++j) x[j] = p[(size_t)j * stride];
#pragma unroll
  for (int j = 0; j < CNT; ++j) v += x[j];
  return v;
}

__device__ __forceinline__ float sum_of_parts(const float* __restrict__ part, size_t stride, size_t at, int splits) {
  float v = 0.f;
  for (int s0 = 0; s0 < splits; s0 += 8) {
    const float* p = part + (size_t)s0 * stride + at;
    switch (min(8, splits - s0)) {
      case 8: v = add_parts<8>(v, p, stride); break;
      case 7: v = add_parts<7>(v, p, stride); break;
      case 6: v = add_parts<6>(v, p, stride); break;
      case 5: v = add_parts<5>(v, p, stride); break;
      case 4: v = add_parts<4>(v, p, stride); break;
      case 3: v = add_parts<3>(v, p, stride); break;
      case 2: v = add_parts<2>(v, p, stride); break;
      default: v = add_parts<1>(v, p, stride); break;
    }
  }
  return v;
}

__global__ __launch_bounds__(256) void skinny_reduce_kernel(const float* __restrict__ part,
                                                            const float* __restrict__ bias,
                                                            void* __restrict__ C, int ldc, int M, int N, int K,
                                                            int splits, int epi, FusedNorm fused) {
  const int n = blockIdx.x * 256 + threadIdx.x, m = blockIdx.y;
  const size_t stride = (size_t)M * N;
  const int frow[1] = {fused.in_ssq ? m : -1};
  float ffac[1];
  row_sums_ask<1>(fused, frow, M, threadIdx.x & 63, ffac);
  row_factors_of<1>(fused, frow, M, K, ffac);
  const float rf = ffac[0];
  if (epi == EPI_SWIGLU) {       // n runs over the ldc outputs
    if (n >= ldc) return;
    const int ng = (n >> 5) * 64 + (n & 31);
    const float g = sum_of_parts(part, stride, (size_t)m * N + ng, splits);
    const float u = sum_of_parts(part, stride, (size_t)m * N + ng + 32, splits);
    ((bf16*)C)[(size_t)m * ldc + n] = (bf16)swiglu_f(g * rf, u * rf);
    return;
  }
  float v = 0.f;                 // the output's new value (0 beyond the row's end)
  if (n < N) {
    v = sum_of_parts(part, stride, (size_t)m * N + n, splits) * rf + (bias ? bias[n] : 0.f);
    if (epi == EPI_BF16) {
      ((bf16*)C)[(size_t)m * ldc + n] = (bf16)v;
    } else {
      float* c = (float*)C + (size_t)m * ldc + n;
      if (epi == EPI_ACC_F32) v += *c;
      *c = v;
    }
  }
  if (fused.out_g) {
    // for the norm that reads these rows next: bf16(x g), and this block's sum of x^2, the waves'
    // sums added in their order
    if (n < N) fused.out_xg[(size_t)m * N + n] = (bf16)(v * fused.out_g[n]);
    __shared__ float wsum[4];
    float sq = v * v;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) sq += __shfl_xor(sq, o, MF_WAVE);
    if ((threadIdx.x & 63) == 0) wsum[threadIdx.x >> 6] = sq;
    __syncthreads();
    if (threadIdx.x == 0) fused.out_ssq[(size_t)m * fused.out_parts + blockIdx.x] = ((wsum[0] + wsum[1]) + wsum[2]) + wsum[3];
    // (a row's places past the runs, where it has more of them: zero)
    if (blockIdx.x == 0)
      for (int p = gridDim.x + threadIdx.x; p < fused.out_parts; p += blockDim.x) fused.out_ssq[(size_t)m * fused.out_parts + p] = 0.f;
  }
}

// The same for rows whose length is a multiple of 4 (16-byte aligned parts, bias and output): a
// thread adds up four neighbouring outputs, a wave a run of 256 columns (so that a run's sum of
// squares is one wave's and needs no barrier), a block four runs.  A quarter of the blocks and of
// the loads of the kernel above, which is what its time is made of.
__global__ __launch_bounds__(256) void skinny_reduce4_kernel(const float* __restrict__ part,
                                                             const float* __restrict__ bias,
                                                             void* __restrict__ C, int ldc, int M, int N, int K,
                                                             int splits, int epi, FusedNorm fused) {
  const int run = blockIdx.x * 4 + (threadIdx.x >> 6);       // of 256 columns
  const int n = run * 256 + (threadIdx.x & 63) * 4, m = blockIdx.y;
  if (run * 256 >= N) return;                                // (whole waves leave: the shuffles below stay among those that stay)
  const size_t stride = (size_t)M * N;
  const int frow[1] = {fused.in_ssq ? m : -1};
  float ffac[1];
  row_sums_ask<1>(fused, frow, M, threadIdx.x & 63, ffac);
  float4 v = float4{0.f, 0.f, 0.f, 0.f};
  const bool in = n < N;                                     // N in fours: all four inside, or none
  if (in) {
    const float* p = part + (size_t)m * N + n;
    for (int s0 = 0; s0 < splits; s0 += 8) {                 // eight parts' loads in flight together, added in their order
      float4 x[8];
#pragma unroll
      for (int j = 0; j < 8; ++j)
        x[j] = s0 + j < splits ? *reinterpret_cast<const float4*>(p + (size_t)(s0 + j) * stride) : float4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int j = 0; j < 8; ++j) { v.x += x[j].x; v.y += x[j].y; v.z += x[j].z; v.w += x[j].w; }
    }
  }
  row_factors_of<1>(fused, frow, M, K, ffac);
  if (in) {
    const float rf = ffac[0];
    const float4 b = bias ? *reinterpret_cast<const float4*>(bias + n) : float4{0.f, 0.f, 0.f, 0.f};
    v = float4{v.x * rf + b.x, v.y * rf + b.y, v.z * rf + b.z, v.w * rf + b.w};
    if (epi == EPI_BF16) {
      bf16* c = (bf16*)C + (size_t)m * ldc + n;
      c[0] = (bf16)v.x; c[1] = (bf16)v.y; c[2] = (bf16)v.z; c[3] = (bf16)v.w;
    } else {
      float4* c = reinterpret_cast<float4*>((float*)C + (size_t)m * ldc + n);
      if (epi == EPI_ACC_F32) { const float4 o = *c; v = float4{v.x + o.x, v.y + o.y, v.z + o.z, v.w + o.w}; }
      *c = v;
    }
  }
  if (fused.out_g) {
    if (in) {
      const float4 g = *reinterpret_cast<const float4*>(fused.out_g + n);
      bf16* xg = fused.out_xg + (size_t)m * N + n;
      xg[0] = (bf16)(v.x * g.x); xg[1] = (bf16)(v.y * g.y); xg[2] = (bf16)(v.z * g.z); xg[3] = (bf16)(v.w * g.w);
    }
    float sq = ((v.x * v.x + v.y * v.y) + v.z * v.z) + v.w * v.w;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) sq += __shfl_xor(sq, o, MF_WAVE);
    if ((threadIdx.x & 63) == 0 && run < (N + 255) / 256) fused.out_ssq[(size_t)m * fused.out_parts + run] = sq;
    if (blockIdx.x == 0 && threadIdx.x < 64)                 // (a row's places past its runs, where it has more of them: zero)
      for (int p = (N + 255) / 256 + threadIdx.x; p < fused.out_parts; p += 64) fused.out_ssq[(size_t)m * fused.out_parts + p] = 0.f;
  }
}

// adds the parts of a K split and runs the epilogue: the kernel in fours where the operands allow it
int launch_reduce(const float* part, const float* bias, void* C, int ldc, int M, int N, int K, int splits, int epi,
                  const FusedNorm& fused, hipStream_t stream) {
  const bool fours = epi != EPI_SWIGLU && N % 4 == 0 && ldc % 4 == 0 && (uintptr_t)part % 16 == 0 &&
                     (uintptr_t)bias % 16 == 0 && (uintptr_t)C % 16 == 0 && (uintptr_t)fused.out_g % 16 == 0 &&
                     (uintptr_t)fused.out_xg % 8 == 0;
  if (fours) {
    dim3 g4((N + 1023) / 1024, M);
    skinny_reduce4_kernel<<<g4, 256, 0, stream>>>(part, bias, C, ldc, M, N, K, splits, epi, fused);
  } else {
    dim3 g2(((epi == EPI_SWIGLU ? ldc : N) + 255) / 256, M);
    skinny_reduce_kernel<<<g2, 256, 0, stream>>>(part, bias, C, ldc, M, N, K, splits, epi, fused);
  }
  return mf_launch_status();
}

template <int MT, bool VEC>
int launch_skinny_v(const bf16* A, int lda, const bf16* W, const bf16* Wt, int ldw, const float* bias, void* C,
                    int ldc, float* part, int M, int N, int K, int splits, int k_per_split, int epi,
                    const FusedNorm& fused, hipStream_t stream) {
  constexpr int smem = 2 * MT * 16 * SK_LD * (int)sizeof(bf16);
  static bool configured = false;
  const bool tiled = VEC && Wt != nullptr;
  auto kern = tiled ? skinny_kernel<MT, VEC, VEC> : skinny_kernel<MT, VEC, false>;
  if (!configured) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(skinny_kernel<MT, VEC, false>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e == hipSuccess)
      e = hipFuncSetAttribute(reinterpret_cast<const void*>(skinny_kernel<MT, VEC, VEC>),
                              hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e != hipSuccess) return (int)e;
    configured = true;
  }
  dim3 grid((N + 127) / 128, splits);
  const bool two_pass = splits > 1 || epi == EPI_SWIGLU;   // gate and up columns sit in different waves
  if (!two_pass && (fused.in_ssq || fused.out_g)) return MF_NOT_BUILT;     // the second kernel is what folds the norm in
  if (ring_takes(VEC, K, splits, k_per_split)) {
    constexpr int smem_ring = smem + MT * 16 * SR_LD * (int)sizeof(float);
    static bool ring_configured = false;
    if (!ring_configured) {
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(skinny_ring_kernel<MT, false>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, smem_ring);
      if (e == hipSuccess)
        e = hipFuncSetAttribute(reinterpret_cast<const void*>(skinny_ring_kernel<MT, true>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, smem_ring);
      if (e != hipSuccess) return (int)e;
      ring_configured = true;
    }
    if (Wt)
      skinny_ring_kernel<MT, true><<<grid, 512, smem_ring, stream>>>(A, lda, Wt, ldw, bias, C, ldc, two_pass ? part : nullptr,
                                                                     M, N, K, k_per_split, epi);
    else
      skinny_ring_kernel<MT, false><<<grid, 512, smem_ring, stream>>>(A, lda, W, ldw, bias, C, ldc, two_pass ? part : nullptr,
                                                                      M, N, K, k_per_split, epi);
  } else {
    kern<<<grid, 512, smem, stream>>>(A, lda, tiled ? Wt : W, ldw, bias, C, ldc, two_pass ? part : nullptr, M, N, K,
                                      k_per_split, epi);
  }
  int rc = mf_launch_status();
  if (rc == 0 && two_pass) rc = launch_reduce(part, bias, C, ldc, M, N, K, splits, epi, fused, stream);
  return rc;
}

template <int MT>
int launch_skinny(const bf16* A, int lda, const bf16* W, const bf16* Wt, int ldw, const float* bias, void* C,
                  int ldc, float* part, int M, int N, int K, int splits, int k_per_split, int epi, int vec_ok,
                  const FusedNorm& fused, hipStream_t stream) {
  return vec_ok ? launch_skinny_v<MT, true>(A, lda, W, Wt, ldw, bias, C, ldc, part, M, N, K, splits, k_per_split,
                                            epi, fused, stream)
                : launch_skinny_v<MT, false>(A, lda, W, nullptr, ldw, bias, C, ldc, part, M, N, K, splits,
                                             k_per_split, epi, fused, stream);
}

// The whole-K kernel for 17 to 64 rows, where the matrix is wide enough to give every CU at least
// 8 tiles; MF_NOT_BUILT (nothing launched) for any other shape.
template <int MT, bool TILED>
int launch_panel_mt(const bf16* A, int lda, const bf16* W, int ldw, const float* bias, void* C, int ldc, int M,
                    int N, int K, int epi, int grid, int units, const FusedNorm& fused, hipStream_t stream) {
  constexpr int smem = 2 * MT * 16 * SK_LD * (int)sizeof(bf16) + MT * 16 * OT_LD * (int)sizeof(float);
  static bool configured = false;
  if (!configured) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(panel_kernel<MT, TILED>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e != hipSuccess) return (int)e;
    configured = true;
  }
  panel_kernel<MT, TILED><<<grid, 512, smem, stream>>>(A, lda, W, ldw, bias, C, ldc, M, N, K, units, epi, fused);
  return mf_launch_status();
}

int launch_panel(const bf16* A, int lda, const bf16* W, const bf16* Wt, int ldw, const float* bias, void* C, int ldc,
                 int M, int N, int K, int epi, const FusedNorm& fused, hipStream_t stream) {
  const int n_cu = cu_count();
  if (n_cu <= 0) return (int)hipErrorUnknown;
  const bool aligned = ldw % 8 == 0 && (uintptr_t)W % 16 == 0 && lda % 8 == 0 && (uintptr_t)A % 16 == 0;
  if (!panel_takes(M, N, K, aligned, epi, n_cu) || fused.out_g) return MF_NOT_BUILT;
  const int units = (N + 31) / 32;
  switch ((M + 15) / 16) {
    case 2:
      return Wt ? launch_panel_mt<2, true>(A, lda, Wt, ldw, bias, C, ldc, M, N, K, epi, n_cu, units, fused, stream)
                : launch_panel_mt<2, false>(A, lda, W, ldw, bias, C, ldc, M, N, K, epi, n_cu, units, fused, stream);
    case 3:
      return Wt ? launch_panel_mt<3, true>(A, lda, Wt, ldw, bias, C, ldc, M, N, K, epi, n_cu, units, fused, stream)
                : launch_panel_mt<3, false>(A, lda, W, ldw, bias, C, ldc, M, N, K, epi, n_cu, units, fused, stream);
    case 4:
      return Wt ? launch_panel_mt<4, true>(A, lda, Wt, ldw, bias, C, ldc, M, N, K, epi, n_cu, units, fused, stream)
                : launch_panel_mt<4, false>(A, lda, W, ldw, bias, C, ldc, M, N, K, epi, n_cu, units, fused, stream);
  }
  return MF_NOT_BUILT;
}

// ---- which tile kernel a product of many rows takes
// Variants: 2: 128 x 128 tiles through registers (two blocks a CU), 3: 64 x 64, 9: 256 x 256 through
// registers, and the direct-to-LDS kernel (aligned operands, K in 64s) with tiles of 256 x 256
// (12), 256 x 192 (15, no SwiGLU) and 256 x 128 in three stages (13).  With `splits` > 1 the K
// dimension is cut over blocks (variants 12 and 2) and skinny_reduce_kernel adds the parts.
struct TilePlan { int variant, splits, k_per_split; double us; };

// The estimate behind the choice: a kernel's tiles go over its slots (blocks that fit the chip at
// once) in rounds; a round takes the product's k tiles of 64 times the variant's time per k tile
// (measured at the 7B widths with every CU busy), a last round that is not full somewhat less
// (fewer blocks pull on the fabric); a start, the epilogue's traffic, and for a K split the
// parts' way to memory and back come on top.
double rounds_us(long blocks, long slots, double step_us, long nkt) {
  const long full = blocks / slots;
  const double fill = (double)(blocks % slots) / (double)slots;
  return (double)nkt * step_us * ((double)full + (fill > 0. ? 0.7 + 0.3 * fill : 0.));
}

TilePlan plan_tiles(int M, int N, int K, bool dma_ok, int epi, int n_cu) {
  const long cu = n_cu > 0 ? n_cu : 1;
  const long nkt = (K + 63) / 64, chunks = (K + 255) / 256;
  const double mn = (double)M * (double)N;
  const double epi_us = (epi == EPI_ACC_F32 ? 8. : epi == EPI_F32 ? 4. : epi == EPI_BF16 ? 2. : 1.) * mn / 4e6;
  const double start_us = 12.;
  auto tiles = [&](int bm, int bn) { return (long)((M + bm - 1) / bm) * ((N + bn - 1) / bn); };
  auto cut = [&](long parts, int& splits, int& per) {          // K in `parts` runs of whole chunks of 256
    const long c = (chunks + parts - 1) / parts;
    splits = (int)((chunks + c - 1) / c);
    per = (int)(c * 256);
  };
  auto parts_us = [&](int splits) { return (double)(splits + 2) * mn * 4. / 3.5e6 + 5.; };
  TilePlan best{0, 1, K, 1e30};
  auto offer = [&](int variant, int splits, int per, double us) {
    if (us < best.us) best = TilePlan{variant, splits, per, us};
  };
  if (dma_ok) {
    offer(12, 1, K, rounds_us(tiles(256, 256), cu, 1.75, nkt) + start_us + epi_us);
    // (the narrower tiles must promise 4 % to be taken: where the estimates are that close, the
    // 256-wide tile has measured the faster)
    offer(13, 1, K, 1.04 * (rounds_us(tiles(256, 128), cu, 1.00, nkt) + start_us + epi_us));
    if (epi != EPI_SWIGLU) offer(15, 1, K, 1.04 * (rounds_us(tiles(256, 192), cu, 1.35, nkt) + start_us + epi_us));
    // many rows against few weight rows and a long K (the down product of a prompt): K cut over
    // the big tiles, each part at least 2,048 of K
    if (epi != EPI_SWIGLU && M >= 768)
      for (long parts = 2; parts <= std::min<long>(8, K / 2048); ++parts) {
        int splits, per;
        cut(parts, splits, per);
        if (splits < 2) continue;
        offer(12, splits, per, rounds_us(tiles(256, 256) * splits, cu, 1.75, per / 64) + start_us + parts_us(splits));
      }
  } else {
    offer(9, 1, K, rounds_us(tiles(256, 256), cu, 2.1, nkt) + start_us + epi_us);
  }
  const long t128 = tiles(128, 128);
  offer(M <= 64 && t128 < 64 && epi != EPI_SWIGLU ? 3 : 2, 1, K,
        rounds_us(t128, 2 * cu, 1.45, nkt) + start_us + epi_us);
  // a few hundred rows against a few thousand weight rows (some 50 tiles of 128 x 128, bound by
  // the weight stream): K over about two blocks per CU, each with at least 512 of K
  const long parts = std::min(chunks / 2, (2 * cu) / std::max(1L, t128));
  if (t128 < cu && parts >= 2) {
    int splits, per;
    cut(parts, splits, per);
    if (splits >= 2) offer(2, splits, per, rounds_us(t128 * splits, 2 * cu, 1.45, per / 64) + start_us + parts_us(splits));
  }
  return best;
}

// Which kernel a product of at most 64 rows takes.
enum SkinnyChoice {
  SK_STATIONARY, SK_ROLLING, SK_GUARDED_PAIR, SK_GUARDED_4X2, SK_GUARDED_8X2, SK_GUARDED_8X1, SK_PANEL, SK_RING,
  SK_STAGED
};

SkinnyChoice skinny_choice(int M, int N, int K, bool aligned, int epi, int splits, int k_per_split, int n_cu) {
  if (M <= 16 && splits == 1) {
    // the register-resident kernel where it is built; other aligned shapes the rolling K-split
    // kernel; the rest (and SwiGLU outside the first) the guarded kernel
    if (aligned && stationary_takes(M, N, K, epi, false)) return SK_STATIONARY;
    if (aligned && K % 32 == 0 && epi != EPI_SWIGLU) return SK_ROLLING;
    if (epi == EPI_SWIGLU) return SK_GUARDED_PAIR;
    // many weight rows: 4 waves with two 16-row tiles each (less activation traffic per weight
    // byte); a row count that would leave a short second round of 16-row blocks: 8 waves with
    // two tiles; otherwise 8 waves, one tile
    const int blocks16 = (N + 15) / 16;
    if (blocks16 >= 1024) return SK_GUARDED_4X2;
    if (blocks16 > 256 && blocks16 <= 512) return SK_GUARDED_8X2;
    return SK_GUARDED_8X1;
  }
  if (M > 16 && panel_takes(M, N, K, aligned, epi, n_cu)) return SK_PANEL;
  return ring_takes(aligned, K, splits, k_per_split) ? SK_RING : SK_STAGED;
}

}  // namespace

// `variant`: 0 picks by shape among the whole-K kernels; 1: 256x256 tile with 4 waves, 2: 128x128,
// 3: 64x64, 6: 256x128 with 8 waves, 9: 256x256 with 8 waves; through the direct-to-LDS pipeline, K in
// 64s: 12: 256x256, 13: 256x128 in three stages, 15: 256x192 (tests name them).
MF_API int mf_gemm_bf16(const void* A, int lda, const void* W, int ldw, const float* bias, void* C,
                        int ldc, int M, int N, int K, int epi, int variant, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || lda < K || ldw < K || epi < 0 || epi > 3) return (int)hipErrorInvalidValue;
  if (epi == EPI_SWIGLU ? (N % 64 != 0 || ldc > N / 2 || ldc <= N / 2 - 32 || bias) : ldc < N)
    return (int)hipErrorInvalidValue;
  const int vec_ok = (lda % 8 == 0) && (ldw % 8 == 0) && ((uintptr_t)A % 16 == 0) &&
                     ((uintptr_t)W % 16 == 0) && (K % 8 == 0);
  const bf16* a = (const bf16*)A;
  const bf16* w = (const bf16*)W;
  // the direct-to-LDS kernel addresses its operands with 32-bit byte offsets
  const bool dma_ok = vec_ok && K % DMA_BK == 0 && (size_t)M * lda * 2 < (1ull << 32) && (size_t)N * ldw * 2 < (1ull << 32);
  if (variant == 0) {
    const TilePlan plan = plan_tiles(M, N, K, dma_ok, epi, cu_count());
    if (plan.splits > 1) return (int)hipErrorInvalidValue;       // a K split needs the caller's workspace
    variant = plan.variant;
  }
  if (epi == EPI_SWIGLU && variant == 3) variant = 2;      // needs two 32-column tiles per wave
  switch (variant) {
    case 1: return launch_tile<256, 256, 128, 128>(a, lda, w, ldw, bias, C, ldc, M, N, K, epi, vec_ok, stream);
    case 2: return launch_tile<128, 128, 64, 64>(a, lda, w, ldw, bias, C, ldc, M, N, K, epi, vec_ok, stream);
    case 3: return launch_tile<64, 64, 32, 32>(a, lda, w, ldw, bias, C, ldc, M, N, K, epi, vec_ok, stream);
    case 6: return launch_tile<256, 128, 64, 64, 32>(a, lda, w, ldw, bias, C, ldc, M, N, K, epi, vec_ok, stream);
    case 9: return launch_tile<256, 256, 128, 64, 64>(a, lda, w, ldw, bias, C, ldc, M, N, K, epi, vec_ok, stream);
    case 12:
      if (!dma_ok) return (int)hipErrorInvalidValue;
      return launch_tile_dma<256, 2, 2>(a, lda, w, ldw, bias, C, ldc, M, N, K, epi, stream);
    case 13:
      if (!dma_ok) return (int)hipErrorInvalidValue;
      return launch_tile_dma<128, 4, 3>(a, lda, w, ldw, bias, C, ldc, M, N, K, epi, stream);
    case 15:
      if (!dma_ok || epi == EPI_SWIGLU) return (int)hipErrorInvalidValue;
      return launch_tile_dma<192, 4, 2>(a, lda, w, ldw, bias, C, ldc, M, N, K, epi, stream);
  }
  return (int)hipErrorInvalidValue;
}

// Few rows for the tile kernel (a prompt of a few hundred tokens against 3584 weight rows makes
// some 50 tiles for 256 CUs): K is split over `splits` blocks per tile, which store 32-bit sums
// into part[splits][M][N], and skinny_reduce_kernel adds them and runs the epilogue.
// k_per_split is a multiple of 64.
MF_API int mf_gemm_bf16_splitk(const void* A, int lda, const void* W, int ldw, const float* bias, void* C,
                               int ldc, float* part, int M, int N, int K, int splits, int k_per_split,
                               int epi, int variant, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || lda < K || ldw < K || epi < 0 || epi > 3 || splits < 2 || !part || k_per_split % 64 != 0 ||
      (long)splits * k_per_split < K || (long)(splits - 1) * k_per_split >= K)
    return (int)hipErrorInvalidValue;
  if (epi == EPI_SWIGLU ? (N % 64 != 0 || ldc > N / 2 || ldc <= N / 2 - 32 || bias) : ldc < N)
    return (int)hipErrorInvalidValue;
  const int vec_ok = (lda % 8 == 0) && (ldw % 8 == 0) && ((uintptr_t)A % 16 == 0) &&
                     ((uintptr_t)W % 16 == 0) && (K % 8 == 0);
  // variant 12: 256 x 256 tiles through the direct-to-LDS pipeline (many rows against few weight
  // rows and a long K: the down product of a prompt); 2: 128 x 128 (few rows)
  if (variant != 12 && variant != 2) return (int)hipErrorInvalidValue;
  const bool big_tiles = variant == 12;
  if (big_tiles && (!vec_ok || K % DMA_BK != 0 || (size_t)M * lda * 2 >= (1ull << 32) ||
                    (size_t)N * ldw * 2 >= (1ull << 32)))
    return (int)hipErrorInvalidValue;
  int rc = big_tiles ? launch_tile_dma<256, 2, 2>((const bf16*)A, lda, (const bf16*)W, ldw, nullptr, part, N, M, N, K,
                                       EPI_F32, stream, splits, k_per_split)
                     : launch_tile<128, 128, 64, 64>((const bf16*)A, lda, (const bf16*)W, ldw, nullptr, part, N, M,
                                                     N, K, EPI_F32, vec_ok, stream, splits, k_per_split);
  if (rc) return rc;
  return launch_reduce(part, bias, C, ldc, M, N, K, splits, epi, FusedNorm{}, stream);
}

// The register-resident kernel for the shapes it is built for (K = 256 NS with enough tiles to
// go round); MF_NOT_BUILT for any other, and nothing is launched.
static int stationary16(const void* a, int lda, const bf16* w, const bf16* wt, int ldw, const float* bias, void* C,
                        int ldc, int M, int N, int K, int epi, const NormArgs* norm, hipStream_t stream,
                        const FusedNorm& fused = FusedNorm{}) {
  if (!stationary_takes(M, N, K, epi, norm != nullptr)) return MF_NOT_BUILT;
  // two tiles an item where a block's share is more than one: 128-byte rows of 32-bit output
  const int n_cu = cu_count();
  if (n_cu <= 0) return (int)hipErrorUnknown;
  const bool two = (N + n_cu - 1) / n_cu > 16;
#define MF_STATIONARY_T(NS_, T_, W_)                                                                          \
  (epi == EPI_SWIGLU ? launch_stationary16<NS_, 2, true, T_>(a, lda, W_, ldw, bias, C, ldc, M, N, epi, norm, fused, stream) \
   : two             ? launch_stationary16<NS_, 2, false, T_>(a, lda, W_, ldw, bias, C, ldc, M, N, epi, norm, fused, stream) \
                     : launch_stationary16<NS_, 1, false, T_>(a, lda, W_, ldw, bias, C, ldc, M, N, epi, norm, fused, stream))
#define MF_STATIONARY(NS_) \
  case NS_: return wt ? MF_STATIONARY_T(NS_, true, wt) : MF_STATIONARY_T(NS_, false, w);
  if (K == STATIONARY_K7) {
    // seven waves: one tile an item outside SwiGLU (the epilogue gives every wave 64 / (16 NT) rows)
#define MF_STATIONARY_7(T_, W_)                                                                                  \
  (epi == EPI_SWIGLU ? launch_stationary16<4, 2, true, T_, 7>(a, lda, W_, ldw, bias, C, ldc, M, N, epi, norm, fused, stream) \
                     : launch_stationary16<4, 1, false, T_, 7>(a, lda, W_, ldw, bias, C, ldc, M, N, epi, norm, fused, stream))
    return wt ? MF_STATIONARY_7(true, wt) : MF_STATIONARY_7(false, w);
#undef MF_STATIONARY_7
  }
  switch (K / 256) { MF_STATIONARY_NS(MF_STATIONARY) }
#undef MF_STATIONARY
#undef MF_STATIONARY_T
  return MF_NOT_BUILT;
}

static int skinny_product(const void* A, int lda, const void* W, const void* Wt, int ldw, const float* bias,
                          void* C, int ldc, float* part, int M, int N, int K, int splits, int k_per_split, int epi,
                          const FusedNorm& fused, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (M > 64 || K <= 0 || lda < K || ldw < K || epi < 0 || epi > 3 || splits < 1 ||
      k_per_split % KC != 0 || (long)splits * k_per_split < K || (splits > 1 && !part))
    return (int)hipErrorInvalidValue;
  if (epi == EPI_SWIGLU ? (N % 64 != 0 || ldc > N / 2 || ldc <= N / 2 - 32 || bias || (M > 16 && !part))
                        : ldc < N)
    return (int)hipErrorInvalidValue;
  const int vec_ok = (lda % 8 == 0) && (ldw % 8 == 0) && ((uintptr_t)A % 16 == 0) &&
                     ((uintptr_t)W % 16 == 0) && (K % 8 == 0);
  const bf16* a = (const bf16*)A;
  const bf16* w = (const bf16*)W;
  const bf16* wt = (K % 32 == 0 && (uintptr_t)Wt % 16 == 0) ? (const bf16*)Wt : nullptr;
  const bool folds = fused.in_ssq || fused.out_g;
  const SkinnyChoice choice = skinny_choice(M, N, K, vec_ok, epi, splits, k_per_split, cu_count());
  // at most 16 rows: the register-resident kernel takes a prepared norm and prepares the next one, the
  // rolling kernel prepares the next one; the K-split kernels' second kernel counts its parts otherwise
  if (folds && M <= 16 && choice != SK_STATIONARY && choice != SK_RING && choice != SK_STAGED &&
      !(choice == SK_ROLLING && !fused.in_ssq))
    return MF_NOT_BUILT;
  switch (choice) {
    case SK_STATIONARY: return stationary16(a, lda, w, wt, ldw, bias, C, ldc, M, N, K, epi, nullptr, stream, fused);
    case SK_ROLLING:
      return wt ? launch_rolling16<8, 1, 16, false, true>(a, lda, wt, ldw, bias, C, ldc, M, N, K, epi, stream, fused)
                : launch_rolling16<8, 1, 16>(a, lda, w, ldw, bias, C, ldc, M, N, K, epi, stream, fused);
    case SK_GUARDED_PAIR: return launch_skinny16<4, 2, 4, true>(a, lda, w, ldw, bias, C, ldc, M, N, K, epi, vec_ok, stream);
    case SK_GUARDED_4X2: return launch_skinny16<4, 2, 4>(a, lda, w, ldw, bias, C, ldc, M, N, K, epi, vec_ok, stream);
    case SK_GUARDED_8X2: return launch_skinny16<8, 2, 4>(a, lda, w, ldw, bias, C, ldc, M, N, K, epi, vec_ok, stream);
    case SK_GUARDED_8X1: return launch_skinny16<8, 1, 8>(a, lda, w, ldw, bias, C, ldc, M, N, K, epi, vec_ok, stream);
    case SK_PANEL: return launch_panel(a, lda, w, wt, ldw, bias, C, ldc, M, N, K, epi, fused, stream);
    default: break;
  }
  switch ((M + 15) / 16) {
    case 1: return launch_skinny<1>(a, lda, w, wt, ldw, bias, C, ldc, part, M, N, K, splits, k_per_split, epi, vec_ok, fused, stream);
    case 2: return launch_skinny<2>(a, lda, w, wt, ldw, bias, C, ldc, part, M, N, K, splits, k_per_split, epi, vec_ok, fused, stream);
    case 3: return launch_skinny<3>(a, lda, w, wt, ldw, bias, C, ldc, part, M, N, K, splits, k_per_split, epi, vec_ok, fused, stream);
    case 4: return launch_skinny<4>(a, lda, w, wt, ldw, bias, C, ldc, part, M, N, K, splits, k_per_split, epi, vec_ok, fused, stream);
  }
  return (int)hipErrorInvalidValue;
}

// M <= 64.  `part` holds splits*M*N floats when splits > 1; k_per_split is a multiple of 256.
// `Wt`: the tiled copy of W (see w_operand), or null; the kernels that have a form for it read it
// instead of W.
MF_API int mf_gemm_bf16_skinny(const void* A, int lda, const void* W, const void* Wt, int ldw, const float* bias,
                               void* C, int ldc, float* part, int M, int N, int K, int splits,
                               int k_per_split, int epi, hipStream_t stream) {
  return skinny_product(A, lda, W, Wt, ldw, bias, C, ldc, part, M, N, K, splits, k_per_split, epi, FusedNorm{}, stream);
}

// The same with an RMS norm folded in on either side (see FusedNorm), for the shapes whose kernels
// have a place for it (17 to 64 rows: the whole-K kernel on the reading side, the K-split kernels
// with more than one split on both; at most 16 rows: the register-resident kernel on both sides,
// the rolling kernel on the writing side); MF_NOT_BUILT (-2), having launched nothing, for any other.
//  * in_ssq [M][in_parts], in_eps: A holds bf16(x g) of rows x whose sums of squares these are; the
//    product's sums are multiplied by the row's 1 / sqrt(sum / K + eps) before bias and epilogue.
//  * out_g [N], out_xg [M][N] bf16, out_ssq [M][out_parts]: beside C (32-bit, stored or added
//    to), bf16(C g) and the sums of C^2 in parts are written: over runs of 256 columns (out_parts =
//    ceil(N / 256)) for 17 to 64 rows; for at most 16 rows one part per block of the product's one
//    kernel, out_parts at least the number of CUs (the places past the grid are set to zero).
MF_API int mf_gemm_bf16_skinny_fused(const void* A, int lda, const void* W, const void* Wt, int ldw,
                                     const float* bias, void* C, int ldc, float* part, int M, int N, int K,
                                     int splits, int k_per_split, int epi, const float* in_ssq, int in_parts,
                                     float in_eps, const float* out_g, void* out_xg, float* out_ssq,
                                     int out_parts, hipStream_t stream) {
  if (in_ssq && in_parts < 1) return (int)hipErrorInvalidValue;
  if (out_g && (!out_xg || !out_ssq || out_parts < 1 || ldc != N || (epi != EPI_F32 && epi != EPI_ACC_F32)))
    return (int)hipErrorInvalidValue;
  if (out_g && out_parts < (N + 255) / 256) return (int)hipErrorInvalidValue;
  const FusedNorm fused{in_ssq, in_parts, in_eps, out_g, (bf16*)out_xg, out_ssq, out_parts};
  return skinny_product(A, lda, W, Wt, ldw, bias, C, ldc, part, M, N, K, splits, k_per_split, epi, fused, stream);
}

// RMS norm of rows of the 32-bit residual stream x (row m of the product is x[row_idx[m]]), then
// the product with W, in one kernel.  Returns MF_NOT_BUILT (-2), having launched nothing, for
// shapes the register-resident kernel does not cover: the caller then runs the norm and the
// product one after the other.
MF_API int mf_gemm_bf16_normed(const float* x, int ldx, const int* row_idx, const float* g, float eps,
                               const void* W, const void* Wt, int ldw, const float* bias, void* C, int ldc, int M,
                               int N, int K, int epi, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || epi < 0 || epi > EPI_SWIGLU) return (int)hipErrorInvalidValue;
  if (ldx % 4 != 0 || ldw % 8 != 0 || (uintptr_t)x % 16 != 0 || (uintptr_t)g % 16 != 0 || (uintptr_t)W % 16 != 0)
    return MF_NOT_BUILT;
  const NormArgs norm{g, row_idx, eps};
  const bf16* wt = (uintptr_t)Wt % 16 == 0 ? (const bf16*)Wt : nullptr;
  return stationary16(x, ldx, (const bf16*)W, wt, ldw, bias, C, ldc, M, N, K, epi, &norm, stream);
}

// How a product of more than 64 rows is run: out[0] the variant for mf_gemm_bf16, or with out[1] > 1
// for mf_gemm_bf16_splitk with out[1] splits of out[2] of K each.  `aligned`: 16-byte aligned
// operands with row strides and K in multiples of 8.
MF_API int mf_gemm_bf16_tile_plan(int M, int N, int K, int aligned, int epi, int n_cu, int* out) {
  if (!out || M <= 0 || N <= 0 || K <= 0 || epi < 0 || epi > 3 || n_cu <= 0) return (int)hipErrorInvalidValue;
  const bool dma_ok = aligned && K % DMA_BK == 0 && (size_t)M * K * 2 < (1ull << 32) && (size_t)N * K * 2 < (1ull << 32);
  const TilePlan plan = plan_tiles(M, N, K, dma_ok, epi, n_cu);
  out[0] = plan.variant;
  out[1] = plan.splits;
  out[2] = plan.k_per_split;
  return 0;
}

// The name of the kernel that a product of this shape takes, without launching anything: `rows`
// activation rows against `N` weight rows of length `K`; `aligned`: 16-byte aligned operands with
// row strides and K in multiples of 8; for at most 64 rows `splits`, `k_per_split`: the caller's K
// split (1, K for none); `normed`: the RMS norm is to be folded in (an empty name then means "no
// such kernel": norm and product run one after the other); `n_cu`: compute units of the device.
MF_API int mf_gemm_bf16_plan(int M, int N, int K, int aligned, int epi, int splits, int k_per_split,
                             int normed, int n_cu, char* name, int cap) {
  if (!name || cap < 48 || M <= 0 || N <= 0 || K <= 0 || epi < 0 || epi > 3 || n_cu <= 0) return (int)hipErrorInvalidValue;
  const char* what = "";
  if (normed) {
    what = (aligned && stationary_takes(M, N, K, epi, true)) ? "stationary16_kernel(norm)" : "";
  } else if (M <= 64) {
    switch (skinny_choice(M, N, K, aligned != 0, epi, splits, k_per_split, n_cu)) {
      case SK_STATIONARY: what = "stationary16_kernel"; break;
      case SK_ROLLING: what = "rolling16_kernel"; break;
      case SK_GUARDED_PAIR: case SK_GUARDED_4X2: case SK_GUARDED_8X2: case SK_GUARDED_8X1: what = "skinny16_kernel"; break;
      case SK_PANEL: what = "panel_kernel"; break;
      case SK_RING: what = "skinny_ring_kernel"; break;
      case SK_STAGED: what = "skinny_kernel"; break;
    }
  } else {
    const bool dma_ok = aligned && K % DMA_BK == 0 && (size_t)M * K * 2 < (1ull << 32) && (size_t)N * K * 2 < (1ull << 32);
    const TilePlan plan = plan_tiles(M, N, K, dma_ok, epi, n_cu);
    switch (plan.variant) {
      case 12: what = plan.splits > 1 ? "tile_dma_kernel<256>(split K)" : "tile_dma_kernel<256>"; break;
      case 13: what = "tile_dma_kernel<128>"; break;
      case 15: what = "tile_dma_kernel<192>"; break;
      case 9: what = "tile_kernel<256,256>"; break;
      case 2: what = plan.splits > 1 ? "tile_kernel<128,128>(split K)" : "tile_kernel<128,128>"; break;
      default: what = "tile_kernel<64,64>"; break;
    }
  }
  snprintf(name, (size_t)cap, "%s", what);
  return 0;
}
