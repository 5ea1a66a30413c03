// True 32-bit matrix product: C[M][N] (+)= A[M][K] * W[N][K]^T (+ bias[N]).
// out[t][o] = dot(W[o][:], x[t][:]) + b[o], as src/graph/cpu_backend.rs:214-248 of
// yusiwen/minfer.  Plain fp32 FMA, no reduced-precision matrix mode: this is the path
// that shows faults bfloat16 hides.  Any M, N, K; vector loads only where they are aligned.
// A dot product is summed in blocks of 128 terms whose sums are then added up: the rounding
// error of one long chain grows with the root of its length (18944 terms in the down product;
// the reference's scalar path sums in 64 bits, src/vec_ops.rs:31-35), that of blocks with the
// roots of the block's and of the number of blocks.
#include "common.h"

namespace {

constexpr int BM = 64, BN = 64, BK = 16, PAD = 4;

// Loads 4 consecutive k of one row into a float4, zero beyond the row count or K.
__device__ __forceinline__ float4 load4(const float* __restrict__ base, int ld, int row, int rows,
                                        int k, int K, bool vec_ok) {
  float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
  if (row < rows) {
    const float* p = base + (size_t)row * ld + k;
    if (vec_ok && k + 4 <= K) {
      v = *reinterpret_cast<const float4*>(p);
    } else {
      if (k + 0 < K) v.x = p[0];
      if (k + 1 < K) v.y = p[1];
      if (k + 2 < K) v.z = p[2];
      if (k + 3 < K) v.w = p[3];
    }
  }
  return v;
}

template <bool ACCUMULATE>
__global__ __launch_bounds__(256) void gemm_f32_kernel(const float* __restrict__ A, int lda,
                                                       const float* __restrict__ W, int ldw,
                                                       const float* __restrict__ bias,
                                                       float* __restrict__ C, int ldc, int M, int N,
                                                       int K, int vec_ok) {
  __shared__ float As[BK][BM + PAD];
  __shared__ float Ws[BK][BN + PAD];
  const int tid = threadIdx.x;
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  const int lrow = tid >> 2, lk = (tid & 3) * 4;   // 64 rows x 4 chunks of 4 k
  const int ty = tid >> 4, tx = tid & 15;
  constexpr int FLUSH = 128 / BK;                   // chunks per block of the sum
  float acc[4][4] = {}, tot[4][4] = {};
  int chunk = 0;
  for (int k0 = 0; k0 < K; k0 += BK) {
    const float4 a = load4(A, lda, m0 + lrow, M, k0 + lk, K, vec_ok);
    const float4 w = load4(W, ldw, n0 + lrow, N, k0 + lk, K, vec_ok);
    __syncthreads();
    As[lk + 0][lrow] = a.x; As[lk + 1][lrow] = a.y; As[lk + 2][lrow] = a.z; As[lk + 3][lrow] = a.w;
    Ws[lk + 0][lrow] = w.x; Ws[lk + 1][lrow] = w.y; Ws[lk + 2][lrow] = w.z; Ws[lk + 3][lrow] = w.w;
    __syncthreads();
#pragma unroll
    for (int k = 0; k < BK; ++k) {
      const float4 av = *reinterpret_cast<const float4*>(&As[k][ty * 4]);
      const float4 wv = *reinterpret_cast<const float4*>(&Ws[k][tx * 4]);
      const float ar[4] = {av.x, av.y, av.z, av.w};
      const float wr[4] = {wv.x, wv.y, wv.z, wv.w};
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(ar[i], wr[j], acc[i][j]);
    }
    if (++chunk == FLUSH) {
      chunk = 0;
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          tot[i][j] += acc[i][j];
          acc[i][j] = 0.f;
        }
    }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] += tot[i][j];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n >= N) continue;
      float v = acc[i][j];
      if (bias) v += bias[n];
      float* c = C + (size_t)m * ldc + n;
      *c = ACCUMULATE ? *c + v : v;
    }
  }
}

}  // namespace

MF_API int mf_gemm_f32(const float* A, int lda, const float* W, int ldw, const float* bias, float* C,
                       int ldc, int M, int N, int K, int accumulate, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || lda < K || ldw < K || ldc < N) return (int)hipErrorInvalidValue;
  const int vec_ok = (lda % 4 == 0) && (ldw % 4 == 0) && ((uintptr_t)A % 16 == 0) &&
                     ((uintptr_t)W % 16 == 0);
  dim3 grid((N + BN - 1) / BN, (M + BM - 1) / BM);
  if (accumulate)
    gemm_f32_kernel<true><<<grid, 256, 0, stream>>>(A, lda, W, ldw, bias, C, ldc, M, N, K, vec_ok);
  else
    gemm_f32_kernel<false><<<grid, 256, 0, stream>>>(A, lda, W, ldw, bias, C, ldc, M, N, K, vec_ok);
  return mf_launch_status();
}
