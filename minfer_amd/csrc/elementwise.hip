// Row-wise and element-wise kernels: embedding gather, RMSNorm (with optional row
// gather), SwiGLU, rotation table, rotation fused with the cache write, type conversion,
// seeded normal fill.  Formulas follow yusiwen/minfer's CPU path; each kernel names its
// source.  Statistics, angles and the residual stream are 32-bit.
#include "common.h"
#include "random_normal.h"

// ---------------------------------------------------------------- embedding
// h[t][:] = table[ids[t]][:], no scaling (src/graph/cpu_backend.rs:269-285).  The host
// checks ids before upload; an id outside the table gives a row of NaN so that it shows.
template <typename TT>
__global__ __launch_bounds__(256) void embed_kernel(const TT* __restrict__ table,
                                                    const int* __restrict__ ids,
                                                    float* __restrict__ out, int d, int vocab) {
  const int row = blockIdx.x;
  const int id = ids[row];
  float* o = out + (size_t)row * d;
  if (id < 0 || id >= vocab) {
    for (int i = threadIdx.x; i < d; i += 256) o[i] = __builtin_nanf("");
    return;
  }
  const TT* src = table + (size_t)id * d;
  for (int i = threadIdx.x; i < d; i += 256) o[i] = to_f32(src[i]);
}

MF_API int mf_embed(const void* table, int table_is_bf16, const int* ids, float* out, int rows,
                    int d, int vocab, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (table_is_bf16)
    embed_kernel<bf16><<<rows, 256, 0, stream>>>((const bf16*)table, ids, out, d, vocab);
  else
    embed_kernel<float><<<rows, 256, 0, stream>>>((const float*)table, ids, out, d, vocab);
  return mf_launch_status();
}

// ---------------------------------------------------------------- RMSNorm
// y = x * (1/sqrt(mean(x^2) + eps)) * w  (src/vec_ops.rs:500-522; eps inside the root).
// Row r of the output reads row row_idx[r] of x when row_idx is given.
// A row of at most 256 * 4 * KEEP elements stays in registers between the sum and the scaling.
template <typename OT, int KEEP>
__device__ __forceinline__ void rmsnorm_row_kept(const float* __restrict__ xr, const float* __restrict__ w,
                                                 OT* __restrict__ o, int d, float eps, float* scratch) {
  float4 v[KEEP];
  float ss = 0.f;
#pragma unroll
  for (int c = 0; c < KEEP; ++c) {
    const int i = (c * 256 + threadIdx.x) * 4;
    v[c] = i < d ? *reinterpret_cast<const float4*>(xr + i) : make_float4(0.f, 0.f, 0.f, 0.f);
    ss = fmaf(v[c].x, v[c].x, ss);
    ss = fmaf(v[c].y, v[c].y, ss);
    ss = fmaf(v[c].z, v[c].z, ss);
    ss = fmaf(v[c].w, v[c].w, ss);
  }
  ss = block_sum<256>(ss, scratch);
  const float scale = 1.0f / sqrtf(ss / (float)d + eps);
#pragma unroll
  for (int c = 0; c < KEEP; ++c) {
    const int i = (c * 256 + threadIdx.x) * 4;
    if (i < d) {
      const float4 g = w ? *reinterpret_cast<const float4*>(w + i) : make_float4(1.f, 1.f, 1.f, 1.f);
      o[i + 0] = from_f32<OT>(v[c].x * scale * g.x);
      o[i + 1] = from_f32<OT>(v[c].y * scale * g.y);
      o[i + 2] = from_f32<OT>(v[c].z * scale * g.z);
      o[i + 3] = from_f32<OT>(v[c].w * scale * g.w);
    }
  }
}

template <typename OT>
__global__ __launch_bounds__(256) void rmsnorm_kernel(const float* __restrict__ x,
                                                      const int* __restrict__ row_idx,
                                                      const float* __restrict__ w,
                                                      OT* __restrict__ out, int d, float eps) {
  __shared__ float scratch[4];
  const int row = blockIdx.x;
  const float* xr = x + (size_t)(row_idx ? row_idx[row] : row) * d;
  OT* o = out + (size_t)row * d;
  if (d % 4 == 0 && d <= 256 * 4 * 16) {
    if (d <= 256 * 4 * 4) rmsnorm_row_kept<OT, 4>(xr, w, o, d, eps, scratch);
    else if (d <= 256 * 4 * 8) rmsnorm_row_kept<OT, 8>(xr, w, o, d, eps, scratch);
    else rmsnorm_row_kept<OT, 16>(xr, w, o, d, eps, scratch);
    return;
  }
  float ss = 0.f;
  for (int i = threadIdx.x; i < d; i += 256) {
    const float v = xr[i];
    ss = fmaf(v, v, ss);
  }
  ss = block_sum<256>(ss, scratch);
  const float scale = 1.0f / sqrtf(ss / (float)d + eps);
  for (int i = threadIdx.x; i < d; i += 256) {
    const float g = w ? w[i] : 1.0f;
    o[i] = from_f32<OT>(xr[i] * scale * g);
  }
}

MF_API int mf_rmsnorm(const float* x, const int* row_idx, const float* w, void* out,
                      int out_is_bf16, int rows, int d, float eps, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (out_is_bf16)
    rmsnorm_kernel<bf16><<<rows, 256, 0, stream>>>(x, row_idx, w, (bf16*)out, d, eps);
  else
    rmsnorm_kernel<float><<<rows, 256, 0, stream>>>(x, row_idx, w, (float*)out, d, eps);
  return mf_launch_status();
}

// out[r][:] = x[idx[r]][:]  (generic row selection, src/graph/cpu_backend.rs:255-268)
__global__ __launch_bounds__(256) void gather_rows_kernel(const float* __restrict__ x,
                                                          const int* __restrict__ idx,
                                                          float* __restrict__ out, int d) {
  const float* src = x + (size_t)idx[blockIdx.x] * d;
  float* o = out + (size_t)blockIdx.x * d;
  for (int i = threadIdx.x; i < d; i += 256) o[i] = src[i];
}

MF_API int mf_gather_rows(const float* x, const int* idx, float* out, int rows, int d,
                          hipStream_t stream) {
  if (rows <= 0) return 0;
  gather_rows_kernel<<<rows, 256, 0, stream>>>(x, idx, out, d);
  return mf_launch_status();
}

// ---------------------------------------------------------------- SwiGLU
// y[r][i] = silu(g[r][i]) * u[r][i], silu(z) = z / (1 + exp(-z))
// (src/vec_ops.rs:131-146, src/graph/cpu_backend.rs:323-329).  g and u are the two halves
// of one [rows][2*nf] buffer.
template <typename IT, typename OT>
__global__ __launch_bounds__(256) void swiglu_kernel(const IT* __restrict__ gu, OT* __restrict__ out,
                                                     int nf) {
  const IT* g = gu + (size_t)blockIdx.y * 2 * nf;
  const IT* u = g + nf;
  OT* o = out + (size_t)blockIdx.y * nf;
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i < nf) {
    const float z = to_f32(g[i]);
    o[i] = from_f32<OT>(z / (1.0f + expf(-z)) * to_f32(u[i]));
  }
}

MF_API int mf_swiglu(const void* gu, int in_is_bf16, void* out, int out_is_bf16, int rows, int nf,
                     hipStream_t stream) {
  if (rows <= 0) return 0;
  dim3 grid((nf + 255) / 256, rows);
  if (in_is_bf16 && out_is_bf16)
    swiglu_kernel<bf16, bf16><<<grid, 256, 0, stream>>>((const bf16*)gu, (bf16*)out, nf);
  else if (!in_is_bf16 && out_is_bf16)
    swiglu_kernel<float, bf16><<<grid, 256, 0, stream>>>((const float*)gu, (bf16*)out, nf);
  else if (!in_is_bf16 && !out_is_bf16)
    swiglu_kernel<float, float><<<grid, 256, 0, stream>>>((const float*)gu, (float*)out, nf);
  else
    return (int)hipErrorInvalidValue;
  return mf_launch_status();
}

// ---------------------------------------------------------------- type conversion
template <typename IT, typename OT>
__global__ __launch_bounds__(256) void convert_kernel(const IT* __restrict__ in, OT* __restrict__ out,
                                                      size_t n) {
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256)
    out[i] = from_f32<OT>(to_f32(in[i]));
}

MF_API int mf_convert(const void* in, int in_is_bf16, void* out, int out_is_bf16, size_t n,
                      hipStream_t stream) {
  if (n == 0) return 0;
  const int blocks = (int)((n + 255) / 256 < 65535 ? (n + 255) / 256 : 65535);
  if (in_is_bf16 && !out_is_bf16)
    convert_kernel<bf16, float><<<blocks, 256, 0, stream>>>((const bf16*)in, (float*)out, n);
  else if (!in_is_bf16 && out_is_bf16)
    convert_kernel<float, bf16><<<blocks, 256, 0, stream>>>((const float*)in, (bf16*)out, n);
  else
    return (int)hipErrorInvalidValue;
  return mf_launch_status();
}

// ---------------------------------------------------------------- rotation
// cos/sin[pos][i] of angle = pos * scale / theta^(2i/hd), computed in double and rounded
// once (the reference forms the same angle in f32 per element and call,
// src/graph/cpu_backend.rs:403-420).
__global__ __launch_bounds__(256) void rope_table_kernel(float* __restrict__ cs, float* __restrict__ sn,
                                                         int n_pos, int half, double theta,
                                                         double freq_scale) {
  const int idx = blockIdx.x * 256 + threadIdx.x;
  if (idx >= n_pos * half) return;
  const int pos = idx / half, i = idx % half;
  const double freq = freq_scale / pow(theta, (2.0 * i) / (2.0 * half));
  const double ang = (double)pos * freq;
  cs[idx] = (float)cos(ang);
  sn[idx] = (float)sin(ang);
}

MF_API int mf_rope_table(float* cs, float* sn, int n_pos, int half, double theta,
                         double freq_scale, hipStream_t stream) {
  const int n = n_pos * half;
  if (n <= 0) return 0;
  rope_table_kernel<<<(n + 255) / 256, 256, 0, stream>>>(cs, sn, n_pos, half, theta, freq_scale);
  return mf_launch_status();
}

// Half-split rotation of q and k (pair i with i + hd/2; x0' = x0 c - x1 s, x1' = x0 s + x1 c;
// src/graph/cpu_backend.rs:421-431), v copied, k and v stored into the paged cache at the
// token's position before attention reads it (src/graph/cpu_backend.rs:118-149).  Without
// tables (cs null) nothing is rotated: the kernel then only rounds q and stores k and v that
// some other position encoding has already treated.
// qkv is [T][(nh + 2 nk) hd] in 32-bit with biases already added.  One block per
// (token, head of q|k|v).
// In bfloat16 a page of V is stored transposed in two halves, [2][hd][32 keys], the layout the
// attention kernels read as a matrix-core operand; in 32-bit it lies like K, [64 keys][hd].
template <typename OT, bool V_TRANSPOSED>
__global__ __launch_bounds__(64) void rope_kvwrite_kernel(
    const float* __restrict__ qkv, const float* __restrict__ cs, const float* __restrict__ sn,
    const int* __restrict__ positions, const int* __restrict__ seq_of_tok,
    const int* __restrict__ page_table, int pt_stride, OT* __restrict__ q_out,
    OT* __restrict__ kcache, OT* __restrict__ vcache, int nh, int nk, int hd, int write_kv) {
  const int t = blockIdx.x, head = blockIdx.y;
  const int half = hd >> 1;
  const int pos = positions[t];
  const float* src = qkv + ((size_t)t * (nh + 2 * nk) + head) * hd;
  if (head < nh) {
    OT* dst = q_out + ((size_t)t * nh + head) * hd;
    for (int i = threadIdx.x; i < half; i += 64) {
      const float c = cs ? cs[(size_t)pos * half + i] : 1.f, s = cs ? sn[(size_t)pos * half + i] : 0.f;
      const float x0 = src[i], x1 = src[i + half];
      dst[i] = from_f32<OT>(x0 * c - x1 * s);
      dst[i + half] = from_f32<OT>(x0 * s + x1 * c);
    }
    return;
  }
  if (!write_kv) return;
  const int page = page_table[(size_t)seq_of_tok[t] * pt_stride + pos / MF_PAGE];
  if (page < 0) return;
  const bool is_k = head < nh + nk;
  const int hk = is_k ? head - nh : head - nh - nk;
  if (is_k) {
    OT* dst = kcache + (((size_t)page * nk + hk) * MF_PAGE + pos % MF_PAGE) * hd;
    for (int i = threadIdx.x; i < half; i += 64) {
      const float c = cs ? cs[(size_t)pos * half + i] : 1.f, s = cs ? sn[(size_t)pos * half + i] : 0.f;
      const float x0 = src[i], x1 = src[i + half];
      dst[i] = from_f32<OT>(x0 * c - x1 * s);
      dst[i + half] = from_f32<OT>(x0 * s + x1 * c);
    }
  } else if (V_TRANSPOSED) {      // a page of V is [2][hd][32 keys]
    constexpr int VH = MF_PAGE / 2;
    const int off = pos % MF_PAGE;
    OT* dst = vcache + (((size_t)page * nk + hk) * 2 + off / VH) * hd * VH + off % VH;
    for (int i = threadIdx.x; i < hd; i += 64) dst[(size_t)i * VH] = from_f32<OT>(src[i]);
  } else {
    OT* dst = vcache + (((size_t)page * nk + hk) * MF_PAGE + pos % MF_PAGE) * hd;
    for (int i = threadIdx.x; i < hd; i += 64) dst[i] = from_f32<OT>(src[i]);
  }
}

// The same for head sizes that are multiples of 8 and 16-byte aligned rows: one block per token,
// a thread takes four neighbouring pairs at a time (float4 loads of x, cos and sin, one 8- or
// 16-byte store per half), q and k heads first, then v: the same bytes as one wave per token and
// head with 4-byte accesses moves, in wide accesses.
template <typename OT>
__device__ __forceinline__ void store4(OT* dst, float a, float b, float c, float d);
template <>
__device__ __forceinline__ void store4<float>(float* dst, float a, float b, float c, float d) {
  *reinterpret_cast<float4*>(dst) = make_float4(a, b, c, d);
}
template <>
__device__ __forceinline__ void store4<bf16>(bf16* dst, float a, float b, float c, float d) {
  *reinterpret_cast<bf16x4*>(dst) = bf16x4{(bf16)a, (bf16)b, (bf16)c, (bf16)d};
}

template <typename OT, bool V_TRANSPOSED>
__global__ __launch_bounds__(256) void rope_kvwrite_vec_kernel(
    const float* __restrict__ qkv, const float* __restrict__ cs, const float* __restrict__ sn,
    const int* __restrict__ positions, const int* __restrict__ seq_of_tok,
    const int* __restrict__ page_table, int pt_stride, OT* __restrict__ q_out,
    OT* __restrict__ kcache, OT* __restrict__ vcache, int nh, int nk, int hd, int write_kv) {
  const int t = blockIdx.x;
  const int half = hd >> 1, groups = half >> 2;           // groups of four pairs per head
  const int pos = positions[t];
  const float* row = qkv + (size_t)t * (nh + 2 * nk) * hd;
  const int page = write_kv ? page_table[(size_t)seq_of_tok[t] * pt_stride + pos / MF_PAGE] : -1;
  const int off = pos % MF_PAGE;
  const int n_rot = (nh + (write_kv && page >= 0 ? nk : 0)) * groups;
  for (int it = threadIdx.x; it < n_rot; it += 256) {
    const int head = it / groups, i = (it % groups) * 4;
    const float* src = row + (size_t)head * hd;
    const float4 x0 = *reinterpret_cast<const float4*>(src + i);
    const float4 x1 = *reinterpret_cast<const float4*>(src + i + half);
    const float4 c = cs ? *reinterpret_cast<const float4*>(cs + (size_t)pos * half + i) : make_float4(1.f, 1.f, 1.f, 1.f);
    const float4 s = cs ? *reinterpret_cast<const float4*>(sn + (size_t)pos * half + i) : make_float4(0.f, 0.f, 0.f, 0.f);
    OT* dst = head < nh ? q_out + ((size_t)t * nh + head) * hd
                        : kcache + (((size_t)page * nk + (head - nh)) * MF_PAGE + off) * hd;
    store4<OT>(dst + i, x0.x * c.x - x1.x * s.x, x0.y * c.y - x1.y * s.y, x0.z * c.z - x1.z * s.z,
               x0.w * c.w - x1.w * s.w);
    store4<OT>(dst + i + half, x0.x * s.x + x1.x * c.x, x0.y * s.y + x1.y * c.y, x0.z * s.z + x1.z * c.z,
               x0.w * s.w + x1.w * c.w);
  }
  if (!write_kv || page < 0) return;
  const float* vsrc = row + (size_t)(nh + nk) * hd;
  for (int it = threadIdx.x; it < nk * (hd >> 2); it += 256) {
    const int hk = it / (hd >> 2), i = (it % (hd >> 2)) * 4;
    const float4 v = *reinterpret_cast<const float4*>(vsrc + (size_t)hk * hd + i);
    if (V_TRANSPOSED) {                   // a page of V is [2][hd][32 keys]
      constexpr int VH = MF_PAGE / 2;
      OT* dst = vcache + ((((size_t)page * nk + hk) * 2 + off / VH) * hd + i) * VH + off % VH;
      dst[0] = from_f32<OT>(v.x);
      dst[VH] = from_f32<OT>(v.y);
      dst[2 * VH] = from_f32<OT>(v.z);
      dst[3 * VH] = from_f32<OT>(v.w);
    } else {
      store4<OT>(vcache + (((size_t)page * nk + hk) * MF_PAGE + off) * hd + i, v.x, v.y, v.z, v.w);
    }
  }
}

// The rotation alone, in place, on the first n_rot heads of every token's [n_heads_total][hd] row
// of 32-bit values (q and k of a q|k|v row; v is left as it is).
__global__ __launch_bounds__(256) void rope_inplace_kernel(float* __restrict__ x, const float* __restrict__ cs,
                                                           const float* __restrict__ sn,
                                                           const int* __restrict__ positions, int n_rot,
                                                           int n_heads_total, int hd) {
  const int t = blockIdx.x, half = hd >> 1;
  const int pos = positions[t];
  float* row = x + (size_t)t * n_heads_total * hd;
  for (int it = threadIdx.x; it < n_rot * half; it += 256) {
    const int head = it / half, i = it % half;
    const float c = cs[(size_t)pos * half + i], s = sn[(size_t)pos * half + i];
    float* p = row + (size_t)head * hd;
    const float x0 = p[i], x1 = p[i + half];
    p[i] = x0 * c - x1 * s;
    p[i + half] = x0 * s + x1 * c;
  }
}

MF_API int mf_rope_inplace(float* x, const float* cs, const float* sn, const int* positions, int n_tok, int n_rot,
                           int n_heads_total, int hd, hipStream_t stream) {
  if (n_tok <= 0 || n_rot <= 0) return 0;
  if (hd % 2 != 0 || n_rot > n_heads_total || !cs || !sn) return (int)hipErrorInvalidValue;
  rope_inplace_kernel<<<n_tok, 256, 0, stream>>>(x, cs, sn, positions, n_rot, n_heads_total, hd);
  return mf_launch_status();
}

MF_API int mf_rope_kvwrite(const float* qkv, const float* cs, const float* sn, const int* positions,
                           const int* seq_of_tok, const int* page_table, int pt_stride, void* q_out,
                           void* kcache, void* vcache, int is_bf16, int n_tok, int nh, int nk, int hd,
                           int write_kv, hipStream_t stream) {
  if (n_tok <= 0) return 0;
  if ((cs == nullptr) != (sn == nullptr)) return (int)hipErrorInvalidValue;
  const bool vec = hd % 8 == 0 && (uintptr_t)qkv % 16 == 0 && (uintptr_t)cs % 16 == 0 && (uintptr_t)sn % 16 == 0 &&
                   (uintptr_t)q_out % 16 == 0 && (uintptr_t)kcache % 16 == 0 && (uintptr_t)vcache % 16 == 0;
  if (vec) {
    if (is_bf16)
      rope_kvwrite_vec_kernel<bf16, true><<<n_tok, 256, 0, stream>>>(qkv, cs, sn, positions, seq_of_tok, page_table,
                                                                     pt_stride, (bf16*)q_out, (bf16*)kcache,
                                                                     (bf16*)vcache, nh, nk, hd, write_kv);
    else
      rope_kvwrite_vec_kernel<float, false><<<n_tok, 256, 0, stream>>>(qkv, cs, sn, positions, seq_of_tok,
                                                                       page_table, pt_stride, (float*)q_out,
                                                                       (float*)kcache, (float*)vcache, nh, nk, hd,
                                                                       write_kv);
    return mf_launch_status();
  }
  dim3 grid(n_tok, write_kv ? nh + 2 * nk : nh);
  if (is_bf16)
    rope_kvwrite_kernel<bf16, true><<<grid, 64, 0, stream>>>(qkv, cs, sn, positions, seq_of_tok, page_table,
                                                       pt_stride, (bf16*)q_out, (bf16*)kcache,
                                                       (bf16*)vcache, nh, nk, hd, write_kv);
  else
    rope_kvwrite_kernel<float, false><<<grid, 64, 0, stream>>>(qkv, cs, sn, positions, seq_of_tok, page_table,
                                                        pt_stride, (float*)q_out, (float*)kcache,
                                                        (float*)vcache, nh, nk, hd, write_kv);
  return mf_launch_status();
}

// ---------------------------------------------------------------- seeded normal fill
// value(i) depends only on (seed, i) and is the same bits as the host's fill of the same
// (seed, i) (random_normal.h, host_random.cpp).  A thread makes both members of a pair.
template <typename OT>
__global__ __launch_bounds__(256) void fill_normal_kernel(OT* __restrict__ out, size_t n, uint64_t seed,
                                                          float std, int round_bf16) {
  const size_t pairs = (n + 1) / 2;
  for (size_t j = (size_t)blockIdx.x * 256 + threadIdx.x; j < pairs; j += (size_t)gridDim.x * 256) {
    double z0, z1;
    mf_normal_pair(seed, j, &z0, &z1);
    float v0, v1;
    {
#pragma clang fp contract(off)
      v0 = (float)z0 * std;
      v1 = (float)z1 * std;
    }
    if (round_bf16) {
      v0 = mf_bf16_value(mf_bf16_bits(v0));
      v1 = mf_bf16_value(mf_bf16_bits(v1));
    }
    out[2 * j] = from_f32<OT>(v0);
    if (2 * j + 1 < n) out[2 * j + 1] = from_f32<OT>(v1);
  }
}

// `round_bf16`: a float32 output holds values that bfloat16 represents (what a tensor written in
// bfloat16 and widened gives); a bfloat16 output is rounded in any case.
MF_API int mf_fill_normal(void* out, int is_bf16, size_t n, uint64_t seed, float std, int round_bf16,
                          hipStream_t stream) {
  if (n == 0) return 0;
  const size_t pairs = (n + 1) / 2;
  const int blocks = (int)((pairs + 255) / 256 < 16384 ? (pairs + 255) / 256 : 16384);
  if (is_bf16)
    fill_normal_kernel<bf16><<<blocks, 256, 0, stream>>>((bf16*)out, n, seed, std, 1);
  else
    fill_normal_kernel<float><<<blocks, 256, 0, stream>>>((float*)out, n, seed, std, round_bf16);
  return mf_launch_status();
}
