// Memory-bound kernels of the Muon / NorMuon / Dion2 step for gfx950: everything around the
// Newton-Schulz GEMMs.  All of them are single-pass over their big operands, use 16-byte
// per-lane accesses where alignment allows, and reduce in a fixed order (no float atomics) so a
// step is bit-reproducible run to run.
#include "elementwise.h"

namespace dion {

static __device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

// Block-wide sum in a fixed order; result valid in every thread.  red: >= 16 floats of LDS.
static __device__ __forceinline__ float block_sum(float v, float* red) {
  v = wave_sum(v);
  const int w = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[w] = v;
  __syncthreads();
  float s = 0.f;
  for (int i = 0; i < nw; ++i) s += red[i];
  return s;
}

template <typename T>
static __device__ __forceinline__ float load_as_bf16_f32(const T* p, int64_t i);
template <>
__device__ __forceinline__ float load_as_bf16_f32<bf16_t>(const bf16_t* p, int64_t i) {
  return bf16_to_f32(p[i]);
}
template <>
__device__ __forceinline__ float load_as_bf16_f32<float>(const float* p, int64_t i) {
  return bf16_to_f32(f32_to_bf16(p[i]));
}

// ------------------------------------------------------------------------------------------
// Frobenius pre-normalisation:  partial sums of squares of bf16(in), then 1/(||.||*s + eps).
// ------------------------------------------------------------------------------------------
// 8 consecutive elements of `p` (16-byte aligned chunk index i) as bf16-rounded floats.
template <typename T>
static __device__ __forceinline__ void load8_as_bf16(const T* p, int64_t i, float v[8]) {
  if (sizeof(T) == 2) {
    const uint4 raw = ((const uint4*)p)[i];
    const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      v[2 * e] = __uint_as_float(w[e] << 16);
      v[2 * e + 1] = __uint_as_float(w[e] & 0xffff0000u);
    }
  } else {
    const float4 a = ((const float4*)p)[2 * i], c = ((const float4*)p)[2 * i + 1];
    const float f[8] = {a.x, a.y, a.z, a.w, c.x, c.y, c.z, c.w};
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = bf16_to_f32(f32_to_bf16(f[e]));
  }
}

template <typename T, bool VEC>
__global__ __launch_bounds__(256) void sumsq_partial_kernel(const T* __restrict__ in, int64_t numel,
                                                            int nblk, float* __restrict__ partial) {
  __shared__ float red[16];
  const int b = blockIdx.y;
  const T* src = in + (int64_t)b * numel;
  float s = 0.f;
  if (VEC) {
    const int64_t nv = numel >> 3;
    const int64_t per = (nv + nblk - 1) / nblk;
    const int64_t lo = (int64_t)blockIdx.x * per;
    int64_t hi = lo + per;
    if (hi > nv) hi = nv;
    for (int64_t i = lo + threadIdx.x; i < hi; i += 256) {
      float v[8];
      load8_as_bf16<T>(src, i, v);
#pragma unroll
      for (int e = 0; e < 8; ++e) s += v[e] * v[e];
    }
  } else {
    const int64_t per = (numel + nblk - 1) / nblk;
    const int64_t lo = (int64_t)blockIdx.x * per;
    int64_t hi = lo + per;
    if (hi > numel) hi = numel;
    for (int64_t i = lo + threadIdx.x; i < hi; i += 256) {
      const float v = load_as_bf16_f32<T>(src, i);
      s += v * v;
    }
  }
  s = block_sum(s, red);
  if (threadIdx.x == 0) partial[(int64_t)b * nblk + blockIdx.x] = s;
}

__global__ __launch_bounds__(256) void norm_finalize_kernel(const float* __restrict__ partial, int nblk,
                                                            float norm_scale, float eps,
                                                            float* __restrict__ inv_norm) {
  // Fixed summation order: thread t adds partials t, t + 256, ... (four independent running sums,
  // so four loads are in flight), then the block sum.
  __shared__ float red[16];
  const int b = blockIdx.x;
  const float* src = partial + (int64_t)b * nblk;
  float s4[4] = {0.f, 0.f, 0.f, 0.f};
  int i = threadIdx.x;
  for (; i + 3 * 256 < nblk; i += 4 * 256) {
#pragma unroll
    for (int j = 0; j < 4; ++j) s4[j] += src[i + j * 256];
  }
  for (int j = 0; i < nblk; i += 256, ++j) s4[j] += src[i];
  const float s = block_sum((s4[0] + s4[1]) + (s4[2] + s4[3]), red);
  if (threadIdx.x == 0) inv_norm[b] = 1.0f / (sqrtf(s) * norm_scale + eps);
}

// in [B,R,C] -> same [B,Rp,Cp] (scaled, zero padded) and trans [B,Cp,Rp] = same^T, both bf16.
// 64x64 tiles through LDS so both stores are row-contiguous.
template <typename T>
__global__ __launch_bounds__(256) void ns_prepare_kernel(const T* __restrict__ in, int R, int C,
                                                         const float* __restrict__ inv_norm,
                                                         bf16_t* __restrict__ same, int Rp, int Cp,
                                                         int ld_same, int64_t stride_same,
                                                         bf16_t* __restrict__ trans, int ld_trans,
                                                         int64_t stride_trans) {
  __shared__ bf16_t tile[64][66];
  const int b = blockIdx.z;
  const int r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
  const float sc = inv_norm ? inv_norm[b] : 1.0f;  // (no factor: the values are copied as they are)
  const T* src = in + (int64_t)b * R * C;
  bf16_t* ds = same + (int64_t)b * stride_same;
  bf16_t* dt = trans + (int64_t)b * stride_trans;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
#pragma unroll 4
  for (int i = ty; i < 64; i += 4) {
    const int r = r0 + i, c = c0 + tx;
    bf16_t v = 0;
    if (r < R && c < C) v = f32_to_bf16(load_as_bf16_f32<T>(src, (int64_t)r * C + c) * sc);
    tile[i][tx] = v;
    if (same) ds[(int64_t)r * ld_same + c] = v;
  }
  __syncthreads();
  if (!trans) return;
#pragma unroll 4
  for (int i = ty; i < 64; i += 4) {
    // trans row (c0 + i), column (r0 + tx)
    dt[(int64_t)(c0 + i) * ld_trans + r0 + tx] = tile[tx][i];
  }
}

// Same operation (either output may be null), 16-byte accesses: needs C % 8 == 0, 16-byte aligned input and row pitches.
template <typename T>
__global__ __launch_bounds__(256) void ns_prepare_vec_kernel(const T* __restrict__ in, int R, int C,
                                                             const float* __restrict__ inv_norm,
                                                             bf16_t* __restrict__ same, int ld_same,
                                                             int64_t stride_same,
                                                             bf16_t* __restrict__ trans, int ld_trans,
                                                             int64_t stride_trans) {
  __shared__ __attribute__((aligned(16))) bf16_t tile[64][72];
  const int b = blockIdx.z;
  const int r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
  const float sc = inv_norm ? inv_norm[b] : 1.0f;  // (no factor: the values are copied as they are)
  const T* src = in + (int64_t)b * R * C;
  bf16_t* ds = same + (int64_t)b * stride_same;
  bf16_t* dt = trans + (int64_t)b * stride_trans;
  const int chunk = threadIdx.x & 7, rr = threadIdx.x >> 3;  // 8 chunks x 32 rows per pass
#pragma unroll
  for (int pass = 0; pass < 2; ++pass) {
    const int i = rr + pass * 32;
    const int r = r0 + i, c = c0 + chunk * 8;
    uint4 o = make_uint4(0, 0, 0, 0);
    if (r < R && c < C) {
      float v[8];
      load8_as_bf16<T>(src, ((int64_t)r * C + c) >> 3, v);
      o.x = pack_bf16x2(v[0] * sc, v[1] * sc);
      o.y = pack_bf16x2(v[2] * sc, v[3] * sc);
      o.z = pack_bf16x2(v[4] * sc, v[5] * sc);
      o.w = pack_bf16x2(v[6] * sc, v[7] * sc);
    }
    *(uint4*)&tile[i][chunk * 8] = o;
    if (same) *(uint4*)(ds + (int64_t)r * ld_same + c) = o;
  }
  __syncthreads();
  if (!trans) return;
  // transposed: thread -> (trans row = column rr + 32*pass of the tile, 8 consecutive source rows)
#pragma unroll
  for (int pass = 0; pass < 2; ++pass) {
    const int col = rr + pass * 32;
    uint32_t w[4];
#pragma unroll
    for (int e = 0; e < 4; ++e)
      w[e] = (uint32_t)tile[chunk * 8 + 2 * e][col] | ((uint32_t)tile[chunk * 8 + 2 * e + 1][col] << 16);
    *(uint4*)(dt + (int64_t)(c0 + col) * ld_trans + r0 + chunk * 8) = make_uint4(w[0], w[1], w[2], w[3]);
  }
}

// Dense [B,R,C] <- padded [B,*,ld] (drops padding).
__global__ __launch_bounds__(256) void unpad_kernel(const bf16_t* __restrict__ src, int64_t src_stride,
                                                    int ld, bf16_t* __restrict__ dst, int R, int C) {
  const int b = blockIdx.z;
  for (int r = blockIdx.y; r < R; r += gridDim.y) {
    const bf16_t* s = src + (int64_t)b * src_stride + (int64_t)r * ld;
    bf16_t* d = dst + ((int64_t)b * R + r) * C;
    for (int c = blockIdx.x * 256 + threadIdx.x; c < C; c += gridDim.x * 256) d[c] = s[c];
  }
}

hipError_t launch_frobenius_inv(const void* in, int in_dtype, int batch, int64_t numel,
                                float norm_scale, float eps, float* partial, int nblk,
                                float* inv_norm, hipStream_t st) {
  const bool vec = (numel % 8 == 0) && (((uintptr_t)in) & 15) == 0;
#define SUMSQ_LAUNCH(T, V)                                                                      \
  hipLaunchKernelGGL((sumsq_partial_kernel<T, V>), dim3(nblk, batch), dim3(256), 0, st, (const T*)in, \
                     numel, nblk, partial)
  if (in_dtype == 0) {
    if (vec) SUMSQ_LAUNCH(bf16_t, true); else SUMSQ_LAUNCH(bf16_t, false);
  } else {
    if (vec) SUMSQ_LAUNCH(float, true); else SUMSQ_LAUNCH(float, false);
  }
#undef SUMSQ_LAUNCH
  return launch_norm_finalize(partial, nblk, batch, norm_scale, eps, inv_norm, st);
}

hipError_t launch_norm_finalize(const float* partial, int nblk, int batch, float norm_scale, float eps,
                                float* inv_norm, hipStream_t st) {
  hipLaunchKernelGGL(norm_finalize_kernel, dim3(batch), dim3(256), 0, st, partial, nblk, norm_scale, eps,
                     inv_norm);
  return hipGetLastError();
}

hipError_t launch_ns_prepare(const void* in, int in_dtype, int batch, int R, int C,
                             const float* inv_norm, bf16_t* same, int Rp, int Cp, int ld_same,
                             int64_t stride_same, bf16_t* trans, int ld_trans, int64_t stride_trans,
                             hipStream_t st) {
  dim3 grid(Cp / 64, Rp / 64, batch);
  const bool vec = (C % 8 == 0) && (((uintptr_t)in) & 15) == 0 && (ld_same % 8 == 0) &&
                   (ld_trans % 8 == 0) && (stride_same % 8 == 0) && (stride_trans % 8 == 0) &&
                   (((uintptr_t)same) & 15) == 0 && (((uintptr_t)trans) & 15) == 0;
  if (vec) {
    if (in_dtype == 0)
      hipLaunchKernelGGL(ns_prepare_vec_kernel<bf16_t>, grid, dim3(256), 0, st, (const bf16_t*)in, R, C,
                         inv_norm, same, ld_same, stride_same, trans, ld_trans, stride_trans);
    else
      hipLaunchKernelGGL(ns_prepare_vec_kernel<float>, grid, dim3(256), 0, st, (const float*)in, R, C,
                         inv_norm, same, ld_same, stride_same, trans, ld_trans, stride_trans);
    return hipGetLastError();
  }
  if (in_dtype == 0)
    hipLaunchKernelGGL(ns_prepare_kernel<bf16_t>, grid, dim3(256), 0, st, (const bf16_t*)in, R, C,
                       inv_norm, same, Rp, Cp, ld_same, stride_same, trans, ld_trans, stride_trans);
  else
    hipLaunchKernelGGL(ns_prepare_kernel<float>, grid, dim3(256), 0, st, (const float*)in, R, C,
                       inv_norm, same, Rp, Cp, ld_same, stride_same, trans, ld_trans, stride_trans);
  return hipGetLastError();
}

hipError_t launch_unpad(const bf16_t* src, int64_t src_stride, int ld, bf16_t* dst, int batch, int R,
                        int C, hipStream_t st) {
  int gx = (C + 255) / 256;
  if (gx > 64) gx = 64;
  hipLaunchKernelGGL(unpad_kernel, dim3(gx, R < 65535 ? R : 65535, batch), dim3(256), 0, st, src,
                     src_stride, ld, dst, R, C);
  return hipGetLastError();
}

// ------------------------------------------------------------------------------------------
// Muon pre: momentum + Nesterov + bf16 cast, list-of-parameters in, one arena out.
// ------------------------------------------------------------------------------------------
// SUMSQ (VEC only, one tile per workgroup): the workgroup also writes the sum of squares of the 4096
// bf16 values it stored, sumsq[p * gridDim.x + blockIdx.x] -- partial sums of ||U||_F^2 per matrix when
// a matrix is a whole number of tiles.
template <typename GT, typename MT, bool VEC, bool SUMSQ = false>
__global__ __launch_bounds__(256) void muon_pre_kernel(PtrTab G, PtrTab M, bf16_t* __restrict__ U,
                                                       int64_t numel, float mu, int nesterov,
                                                       float* __restrict__ sumsq = nullptr) {
  __shared__ float red[16];
  float ss = 0.f;
  const int p = blockIdx.y;
  const GT* __restrict__ g = (const GT*)G.p[p];
  MT* __restrict__ m = (MT*)M.p[p];
  bf16_t* __restrict__ u = U + (int64_t)p * numel;
  const int64_t stride = (int64_t)gridDim.x * 256;
  if (VEC) {
    // Two 8-element chunks per thread per trip, all loads issued before the arithmetic: up to 96
    // bytes of reads in flight per lane.
    // A workgroup owns contiguous tiles of 512 chunks (4096 elements), one tile per trip and normally
    // one trip: the workgroups in flight sweep one window of memory front to back.
    const int64_t nv = numel >> 3;
    for (int64_t i0 = (int64_t)blockIdx.x * 512 + threadIdx.x; i0 < nv; i0 += 2 * stride) {
      const int64_t i1 = i0 + 256;
      const bool has1 = i1 < nv;
      float gv[2][8], mv[2][8];
      st_load8<GT>(g, i0, gv[0]);
      if (has1) st_load8<GT>(g, i1, gv[1]);
      st_load8<MT>(m, i0, mv[0]);
      if (has1) st_load8<MT>(m, i1, mv[1]);
#pragma unroll
      for (int c = 0; c < 2; ++c) {
        if (c == 1 && !has1) break;
        const int64_t i = c == 0 ? i0 : i1;
        float uv[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          mv[c][e] = __fadd_rn(__fmul_rn(mv[c][e], mu), gv[c][e]);
          uv[e] = nesterov ? __fadd_rn(__fmul_rn(mv[c][e], mu), gv[c][e]) : mv[c][e];
        }
        st_store8<MT>(m, i, mv[c]);
        st_store8<bf16_t>(u, i, uv);
        if (SUMSQ) {
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const float r = st_round<bf16_t>(uv[e]);
            ss += r * r;
          }
        }
      }
    }
    if (SUMSQ) {
      ss = block_sum(ss, red);
      if (threadIdx.x == 0) sumsq[(int64_t)p * gridDim.x + blockIdx.x] = ss;
    }
  } else {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < numel; i += stride) {
      const float gv = st_load<GT>(g, i);
      const float mv = __fadd_rn(__fmul_rn(st_load<MT>(m, i), mu), gv);
      st_store<MT>(m, i, mv);
      u[i] = f32_to_bf16(nesterov ? __fadd_rn(__fmul_rn(mv, mu), gv) : mv);
    }
  }
}

// The same update for tall matrices (rows > cols) whose orthogonalization input is wanted with the short
// side along rows: U[p][mat] is written transposed, [cols][rows].  One 64 x 64 tile per workgroup, staged
// through LDS so that G / M rows are read and U^T rows written as whole 128-byte (bf16) runs; every thread
// handles two 8-element chunks, like the flat kernel.  sumsq[(p * mats + mat) * tiles + tile]: sum of
// squares of the tile's bf16 values, tile = (row tile) * (cols / 64) + column tile.
// Needs rows % 64 == 0, cols % 64 == 0, 16-byte aligned pointers.
template <typename GT, typename MT>
__global__ __launch_bounds__(256) void muon_pre_transposed_kernel(PtrTab G, PtrTab M, bf16_t* __restrict__ U,
                                                                  int mats, int rows, int cols, float mu,
                                                                  int nesterov, float* __restrict__ sumsq) {
  __shared__ __attribute__((aligned(16))) bf16_t tile[64][72];
  __shared__ float red[16];
  const int p = blockIdx.z / mats, mat = blockIdx.z - p * mats;
  const int r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
  const int64_t mat_off = (int64_t)mat * rows * cols;
  const GT* __restrict__ g = (const GT*)G.p[p] + mat_off;
  MT* __restrict__ m = (MT*)M.p[p] + mat_off;
  bf16_t* __restrict__ ut = U + ((int64_t)p * mats + mat) * rows * cols;
  const int chunk = threadIdx.x & 7, rr = threadIdx.x >> 3;  // 8 chunks x 32 rows per pass
  float gv[2][8], mv[2][8];
#pragma unroll
  for (int pass = 0; pass < 2; ++pass) {
    const int64_t i8 = ((int64_t)(r0 + rr + pass * 32) * cols + c0 + chunk * 8) >> 3;
    st_load8<GT>(g, i8, gv[pass]);
    st_load8<MT>(m, i8, mv[pass]);
  }
  float ss = 0.f;
#pragma unroll
  for (int pass = 0; pass < 2; ++pass) {
    const int64_t i8 = ((int64_t)(r0 + rr + pass * 32) * cols + c0 + chunk * 8) >> 3;
    float uv[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      mv[pass][e] = __fadd_rn(__fmul_rn(mv[pass][e], mu), gv[pass][e]);
      uv[e] = nesterov ? __fadd_rn(__fmul_rn(mv[pass][e], mu), gv[pass][e]) : mv[pass][e];
    }
    st_store8<MT>(m, i8, mv[pass]);
    uint4 o;
    o.x = pack_bf16x2(uv[0], uv[1]);
    o.y = pack_bf16x2(uv[2], uv[3]);
    o.z = pack_bf16x2(uv[4], uv[5]);
    o.w = pack_bf16x2(uv[6], uv[7]);
    *(uint4*)&tile[rr + pass * 32][chunk * 8] = o;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float r = st_round<bf16_t>(uv[e]);
      ss += r * r;
    }
  }
  ss = block_sum(ss, red);  // (its barriers also order the tile writes before the reads below)
  if (threadIdx.x == 0)
    sumsq[((int64_t)blockIdx.z * gridDim.y + blockIdx.y) * gridDim.x + blockIdx.x] = ss;
  // transposed: thread -> (U^T row = column rr + 32 * pass of the tile, 8 consecutive source rows)
#pragma unroll
  for (int pass = 0; pass < 2; ++pass) {
    const int col = rr + pass * 32;
    uint32_t w[4];
#pragma unroll
    for (int e = 0; e < 4; ++e)
      w[e] = (uint32_t)tile[chunk * 8 + 2 * e][col] | ((uint32_t)tile[chunk * 8 + 2 * e + 1][col] << 16);
    *(uint4*)(ut + (int64_t)(c0 + col) * rows + r0 + chunk * 8) = make_uint4(w[0], w[1], w[2], w[3]);
  }
}

// Workgroups for the tile-per-workgroup kernels: one per 512 chunks, at most 2^20.
static int ew_tiles(int64_t chunks) {
  int64_t b = (chunks + 511) / 512;
  if (b > (1 << 20)) b = 1 << 20;
  if (b < 1) b = 1;
  return (int)b;
}

static int ew_blocks(int64_t work_items) {
  int64_t b = (work_items + 255) / 256;
  if (b > 2048) b = 2048;
  if (b < 1) b = 1;
  return (int)b;
}

hipError_t launch_muon_pre(const PtrTab& G, int g_dtype, const PtrTab& M, int m_dtype, bf16_t* U, int n,
                           int64_t numel, float mu, int nesterov, bool vec, hipStream_t st) {
  dim3 grid(vec ? ew_tiles(numel >> 3) : ew_blocks(numel), n);
#define PRE_LAUNCH(GT, MT, V) \
  hipLaunchKernelGGL((muon_pre_kernel<GT, MT, V>), grid, dim3(256), 0, st, G, M, U, numel, mu, nesterov)
#define PRE_LAUNCH_M(GT, V) \
  do { if (m_dtype == 0) PRE_LAUNCH(GT, bf16_t, V); else PRE_LAUNCH(GT, float, V); } while (0)
  if (g_dtype == 0) {
    if (vec) PRE_LAUNCH_M(bf16_t, true); else PRE_LAUNCH_M(bf16_t, false);
  } else {
    if (vec) PRE_LAUNCH_M(float, true); else PRE_LAUNCH_M(float, false);
  }
#undef PRE_LAUNCH_M
#undef PRE_LAUNCH
  return hipGetLastError();
}

hipError_t launch_muon_pre_prepared(const PtrTab& G, int g_dtype, const PtrTab& M, int m_dtype, bf16_t* U,
                                    float* sumsq, int n, int mats, int rows, int cols, float mu,
                                    int nesterov, hipStream_t st) {
  if (rows > cols) {
    dim3 grid(cols / 64, rows / 64, n * mats);
#define PRET_LAUNCH(GT, MT)                                                                            \
  hipLaunchKernelGGL((muon_pre_transposed_kernel<GT, MT>), grid, dim3(256), 0, st, G, M, U, mats, rows, cols, \
                     mu, nesterov, sumsq)
    if (g_dtype == 0) {
      if (m_dtype == 0) PRET_LAUNCH(bf16_t, bf16_t); else PRET_LAUNCH(bf16_t, float);
    } else {
      if (m_dtype == 0) PRET_LAUNCH(float, bf16_t); else PRET_LAUNCH(float, float);
    }
#undef PRET_LAUNCH
    return hipGetLastError();
  }
  // one 4096-element tile per workgroup, so that blockIdx.x is the tile number within the parameter
  const int64_t numel = (int64_t)mats * rows * cols;
  dim3 grid((unsigned)(numel / 4096), n);
#define PRES_LAUNCH(GT, MT)                                                                             \
  hipLaunchKernelGGL((muon_pre_kernel<GT, MT, true, true>), grid, dim3(256), 0, st, G, M, U, numel, mu, \
                     nesterov, sumsq)
  if (g_dtype == 0) {
    if (m_dtype == 0) PRES_LAUNCH(bf16_t, bf16_t); else PRES_LAUNCH(bf16_t, float);
  } else {
    if (m_dtype == 0) PRES_LAUNCH(float, bf16_t); else PRES_LAUNCH(float, float);
  }
#undef PRES_LAUNCH
  return hipGetLastError();
}

// ------------------------------------------------------------------------------------------
// Muon / NorMuon post: decoupled weight decay (plain or cautious) + scaled update.
// ------------------------------------------------------------------------------------------
template <typename UT, typename XT, bool VEC>
__global__ __launch_bounds__(256) void muon_post_kernel(PtrTab X, const UT* __restrict__ U,
                                                        int64_t numel, int cols,
                                                        const float* __restrict__ row_scale,
                                                        const float* __restrict__ lr_dev,
                                                        const float* __restrict__ adj_lr_dev,
                                                        float adj_ratio,
                                                        const float* __restrict__ wd_dev,
                                                        float wd_host, int cautious) {
  const int p = blockIdx.y;
  XT* __restrict__ x = (XT*)X.p[p];
  const UT* __restrict__ u = U + (int64_t)p * numel;
  const float lr = *lr_dev;
  const float wd = wd_dev ? *wd_dev : wd_host;
  const float coeff = __fmul_rn(lr, wd);
  const float a = __fsub_rn(1.0f, coeff);
  const float b = adj_lr_dev ? *adj_lr_dev : __fmul_rn(lr, adj_ratio);
  const int64_t rows = numel / cols;
  const float* rs = row_scale ? row_scale + (int64_t)p * rows : nullptr;
  const int64_t stride = (int64_t)gridDim.x * 256;
  if (VEC) {
    // contiguous tiles of 512 chunks (4096 elements) per workgroup, two chunks per lane, all loads first
    const int64_t nv = numel >> 3;
    for (int64_t i0 = (int64_t)blockIdx.x * 512 + threadIdx.x; i0 < nv; i0 += 2 * stride) {
      const int64_t i1 = i0 + 256;
      const bool has1 = i1 < nv;
      float uv[2][8], xv[2][8];
      st_load8<UT>(u, i0, uv[0]);
      if (has1) st_load8<UT>(u, i1, uv[1]);
      st_load8<XT>(x, i0, xv[0]);
      if (has1) st_load8<XT>(x, i1, xv[1]);
#pragma unroll
      for (int c = 0; c < 2; ++c) {
        if (c == 1 && !has1) break;
        const int64_t i = c == 0 ? i0 : i1;
        if (rs) {  // cols % 8 == 0 on this path, so the 8 elements share a row
          const float s = rs[(i << 3) / cols];
#pragma unroll
          for (int e = 0; e < 8; ++e) uv[c][e] = __fmul_rn(uv[c][e], s);
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) xv[c][e] = muon_post_one(xv[c][e], uv[c][e], a, coeff, b, cautious);
        st_store8<XT>(x, i, xv[c]);
      }
    }
  } else {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < numel; i += stride) {
      float uv = st_load<UT>(u, i);
      if (rs) uv = __fmul_rn(uv, rs[i / cols]);
      st_store<XT>(x, i, muon_post_one(st_load<XT>(x, i), uv, a, coeff, b, cautious));
    }
  }
}

hipError_t launch_muon_post(const PtrTab& X, int x_dtype, const void* U, int u_dtype, int n, int64_t numel,
                            int cols, const float* row_scale, const float* lr_dev, const float* adj_lr_dev,
                            float adj_ratio, const float* wd_dev, float wd_host, int cautious, bool vec,
                            hipStream_t st) {
  dim3 grid(vec ? ew_tiles(numel >> 3) : ew_blocks(numel), n);
#define POST_LAUNCH(UT, XT, V)                                                                      \
  hipLaunchKernelGGL((muon_post_kernel<UT, XT, V>), grid, dim3(256), 0, st, X, (const UT*)U, numel, \
                     cols, row_scale, lr_dev, adj_lr_dev, adj_ratio, wd_dev, wd_host, cautious)
#define POST_LAUNCH_X(UT, V) \
  do { if (x_dtype == 0) POST_LAUNCH(UT, bf16_t, V); else POST_LAUNCH(UT, float, V); } while (0)
  if (u_dtype == 0) {
    if (vec) POST_LAUNCH_X(bf16_t, true); else POST_LAUNCH_X(bf16_t, false);
  } else {
    if (vec) POST_LAUNCH_X(float, true); else POST_LAUNCH_X(float, false);
  }
#undef POST_LAUNCH_X
#undef POST_LAUNCH
  return hipGetLastError();
}

// ------------------------------------------------------------------------------------------
// out[row][:] = U[row][:] * scale[row]: the normalised update itself, for callers that want it as a
// tensor (the optimizers fold the scale into the update kernels instead).
// ------------------------------------------------------------------------------------------
template <typename OT>
__global__ __launch_bounds__(256) void scale_rows_kernel(const bf16_t* __restrict__ U,
                                                         const float* __restrict__ scale,
                                                         OT* __restrict__ out, int cols) {
  const int64_t row = blockIdx.x;
  const float s = scale[row];
  const bf16_t* u = U + row * cols;
  OT* o = out + row * cols;
  for (int c = threadIdx.x; c < cols; c += 256) st_store<OT>(o, c, __fmul_rn(bf16_to_f32(u[c]), s));
}

hipError_t launch_scale_rows(const bf16_t* U, const float* scale, void* out, int out_dtype, int64_t n_rows,
                             int cols, hipStream_t st) {
  if (n_rows <= 0 || cols <= 0) return hipSuccess;
  if (n_rows > 0x7fffffff) return hipErrorInvalidValue;
  if (out_dtype == 0)
    hipLaunchKernelGGL((scale_rows_kernel<bf16_t>), dim3((unsigned)n_rows), dim3(256), 0, st, U, scale,
                       (bf16_t*)out, cols);
  else
    hipLaunchKernelGGL((scale_rows_kernel<float>), dim3((unsigned)n_rows), dim3(256), 0, st, U, scale,
                       (float*)out, cols);
  return hipGetLastError();
}

// ------------------------------------------------------------------------------------------
// NorMuon: per-row second moment EMA and the Frobenius-preserving row scales.
// ------------------------------------------------------------------------------------------
// Row r of matrix mat keeps its second moment at V[mat][row_idx ? row_idx[mat][r] : r]; V holds
// v_rows entries per matrix (v_rows == rows without row_idx).  The indirection serves updates made
// of selected rows only (NorDion2, dion/nordion2.py:430-447).  A negative row_idx entry marks a row
// that is not part of the update (an all-zero row of a masked full-size tensor,
// dion/nordion2.py:485-497): its second moment is left alone and its scale is 0.
// Pass 1: one wavefront per row.  V <- lerp(V, mean(u^2), w);  tmp[row] = sum(u^2).
template <typename VT>
__global__ __launch_bounds__(256) void normuon_rows_kernel(const bf16_t* __restrict__ U, PtrTab V,
                                                           int mats_per_ptr, int rows, int cols,
                                                           const int32_t* __restrict__ row_idx,
                                                           int v_rows, float w,
                                                           float* __restrict__ rowsq) {
  const int mat = blockIdx.y;
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const int lane = threadIdx.x & 63;
  const bf16_t* u = U + ((int64_t)mat * rows + row) * cols;
  float s = 0.f;
  if ((cols & 7) == 0 && (((uintptr_t)u) & 15) == 0) {
    for (int c = lane * 8; c < cols; c += 512) {
      const uint4 raw = *(const uint4*)(u + c);
      const uint32_t wv[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float lo = __uint_as_float(wv[e] << 16), hi = __uint_as_float(wv[e] & 0xffff0000u);
        s += lo * lo;
        s += hi * hi;
      }
    }
  } else {
    for (int c = lane; c < cols; c += 64) {
      const float v = bf16_to_f32(u[c]);
      s += v * v;
    }
  }
  s = wave_sum(s);
  if (lane == 0) {
    const int vr = row_idx ? row_idx[(int64_t)mat * rows + row] : row;
    if (vr >= 0) {
      VT* v = (VT*)V.p[mat / mats_per_ptr] + (int64_t)(mat % mats_per_ptr) * v_rows + vr;
      const float mean = s / (float)cols;
      const float vo = st_load<VT>(v, 0);
      st_store<VT>(v, 0, vo + w * (mean - vo));  // torch.lerp for weight < 0.5
    }
    rowsq[(int64_t)mat * rows + row] = vr >= 0 ? s : 0.f;
  }
}

// Pass 2: one block per matrix.  scale[row] = (1/d) * sqrt(S1) / max(sqrt(S2), 1e-8) with
// d = sqrt(V)+1e-8, S1 = sum rowsq, S2 = sum rowsq/d^2.  In place over rowsq.
template <typename VT>
__global__ __launch_bounds__(1024) void normuon_scale_kernel(PtrTab V, int mats_per_ptr, int rows,
                                                             const int32_t* __restrict__ row_idx,
                                                             int v_rows, float* __restrict__ scale) {
  __shared__ float red[16];
  const int mat = blockIdx.x;
  const VT* v = (const VT*)V.p[mat / mats_per_ptr] + (int64_t)(mat % mats_per_ptr) * v_rows;
  const int32_t* ri = row_idx ? row_idx + (int64_t)mat * rows : nullptr;
  float* sc = scale + (int64_t)mat * rows;
  float s1 = 0.f, s2 = 0.f;
  for (int r = threadIdx.x; r < rows; r += 1024) {
    const float q = sc[r];
    const int vr = ri ? ri[r] : r;
    const float inv = vr >= 0 ? 1.0f / (sqrtf(st_load<VT>(v, vr)) + 1e-8f) : 0.f;
    s1 += q;
    s2 += q * inv * inv;
  }
  s1 = block_sum(s1, red);
  s2 = block_sum(s2, red);
  const float ratio = sqrtf(s1) / fmaxf(sqrtf(s2), 1e-8f);
  __syncthreads();
  for (int r = threadIdx.x; r < rows; r += 1024) {
    const int vr = ri ? ri[r] : r;
    sc[r] = vr >= 0 ? (1.0f / (sqrtf(st_load<VT>(v, vr)) + 1e-8f)) * ratio : 0.f;
  }
}

hipError_t launch_normuon_stats(const bf16_t* U, const PtrTab& V, int v_dtype, int n_mat, int mats_per_ptr,
                                int rows, int cols, const int32_t* row_idx, int v_rows, float w,
                                float* row_scale, hipStream_t st) {
  // U / row_scale / row_idx are offset to the first matrix by the caller; V is the table chunk
  // covering them.
  if (v_dtype == 0) {
    hipLaunchKernelGGL(normuon_rows_kernel<bf16_t>, dim3((rows + 3) / 4, n_mat), dim3(256), 0, st, U, V,
                       mats_per_ptr, rows, cols, row_idx, v_rows, w, row_scale);
    hipLaunchKernelGGL(normuon_scale_kernel<bf16_t>, dim3(n_mat), dim3(1024), 0, st, V, mats_per_ptr, rows,
                       row_idx, v_rows, row_scale);
  } else {
    hipLaunchKernelGGL(normuon_rows_kernel<float>, dim3((rows + 3) / 4, n_mat), dim3(256), 0, st, U, V,
                       mats_per_ptr, rows, cols, row_idx, v_rows, w, row_scale);
    hipLaunchKernelGGL(normuon_scale_kernel<float>, dim3(n_mat), dim3(1024), 0, st, V, mats_per_ptr, rows,
                       row_idx, v_rows, row_scale);
  }
  return hipGetLastError();
}

// ------------------------------------------------------------------------------------------
// Dion2: accumulate + slice L1 norms, top-k, gather with error-feedback decay, fused post.
// ------------------------------------------------------------------------------------------
template <typename GT>
static __device__ __forceinline__ float g_load(const GT* g, int64_t i) {
  return sizeof(GT) == 2 ? bf16_to_f32(((const bf16_t*)g)[i]) : ((const float*)g)[i];
}

// select rows: one wavefront per row, norms[mat][row] = sum_j |M+G| (of the values as stored).
template <typename GT, typename MT>
__global__ __launch_bounds__(256) void dion2_acc_rows_kernel(PtrTab G, PtrTab M, int mats_per_ptr,
                                                             int rows, int cols,
                                                             float* __restrict__ norms) {
  const int mat = blockIdx.y;
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const int lane = threadIdx.x & 63;
  const int64_t base = ((int64_t)(mat % mats_per_ptr) * rows + row) * cols;
  const GT* g = (const GT*)G.p[mat / mats_per_ptr] + base;
  MT* m = (MT*)M.p[mat / mats_per_ptr] + base;
  float s = 0.f;
  for (int c = lane; c < cols; c += 64) {
    const float v = st_round<MT>(__fadd_rn(st_load<MT>(m, c), g_load<GT>(g, c)));
    st_store<MT>(m, c, v);
    s += fabsf(v);
  }
  s = wave_sum(s);
  if (lane == 0) norms[(int64_t)mat * rows + row] = s;
}

// select columns: each block owns 64 columns of one matrix and walks all rows (4 rows at a time).
template <typename GT, typename MT>
__global__ __launch_bounds__(256) void dion2_acc_cols_kernel(PtrTab G, PtrTab M, int mats_per_ptr,
                                                             int rows, int cols,
                                                             float* __restrict__ norms) {
  __shared__ float red[4][64];
  const int mat = blockIdx.y;
  const int c = blockIdx.x * 64 + (threadIdx.x & 63);
  const int ry = threadIdx.x >> 6;
  const int64_t base = (int64_t)(mat % mats_per_ptr) * rows * cols;
  const GT* g = (const GT*)G.p[mat / mats_per_ptr] + base;
  MT* m = (MT*)M.p[mat / mats_per_ptr] + base;
  float s = 0.f;
  if (c < cols) {
    for (int r = ry; r < rows; r += 4) {
      const int64_t i = (int64_t)r * cols + c;
      const float v = st_round<MT>(__fadd_rn(st_load<MT>(m, i), g_load<GT>(g, i)));
      st_store<MT>(m, i, v);
      s += fabsf(v);
    }
  }
  red[ry][threadIdx.x & 63] = s;
  __syncthreads();
  if (ry == 0 && c < cols)
    norms[(int64_t)mat * cols + c] = (red[0][threadIdx.x] + red[1][threadIdx.x]) +
                                     (red[2][threadIdx.x] + red[3][threadIdx.x]);
}

// 4 columns per thread (8- / 16-byte accesses): each block owns 256 columns, four row lanes.
// With gridDim.z row slabs the block writes its slab's partial sums to out[(slab*n_mat + mat)*cols]
// (n_mat = gridDim.y); dion2_sum_slabs_kernel adds the slabs in a fixed order.
template <typename GT, typename MT>
__global__ __launch_bounds__(256) void dion2_acc_cols_vec_kernel(PtrTab G, PtrTab M, int mats_per_ptr,
                                                                 int rows, int cols, int slab_rows,
                                                                 float* __restrict__ norms) {
  __shared__ float4 red[4][64];
  const int mat = blockIdx.y;
  const int r0 = blockIdx.z * slab_rows;
  const int r1 = (r0 + slab_rows) < rows ? (r0 + slab_rows) : rows;
  norms += (int64_t)blockIdx.z * gridDim.y * cols;
  const int c = (blockIdx.x * 64 + (threadIdx.x & 63)) * 4;
  const int ry = threadIdx.x >> 6;
  const int64_t base = (int64_t)(mat % mats_per_ptr) * rows * cols;
  const GT* g = (const GT*)G.p[mat / mats_per_ptr] + base;
  MT* m = (MT*)M.p[mat / mats_per_ptr] + base;
  float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
  if (c < cols) {
#pragma unroll 4
    for (int r = r0 + ry; r < r1; r += 4) {
      const int64_t i4 = ((int64_t)r * cols + c) >> 2;  // cols % 4 == 0 on this path
      float gv[4], mv[4];
      st_load4<GT>(g, i4, gv);
      st_load4<MT>(m, i4, mv);
#pragma unroll
      for (int e = 0; e < 4; ++e) mv[e] = st_round<MT>(__fadd_rn(mv[e], gv[e]));
      st_store4<MT>(m, i4, mv);
      s.x += fabsf(mv[0]);
      s.y += fabsf(mv[1]);
      s.z += fabsf(mv[2]);
      s.w += fabsf(mv[3]);
    }
  }
  red[ry][threadIdx.x & 63] = s;
  __syncthreads();
  if (ry == 0 && c < cols) {
    const int t = threadIdx.x;
    float4 o;
    o.x = (red[0][t].x + red[1][t].x) + (red[2][t].x + red[3][t].x);
    o.y = (red[0][t].y + red[1][t].y) + (red[2][t].y + red[3][t].y);
    o.z = (red[0][t].z + red[1][t].z) + (red[2][t].z + red[3][t].z);
    o.w = (red[0][t].w + red[1][t].w) + (red[2][t].w + red[3][t].w);
    *(float4*)(norms + (int64_t)mat * cols + c) = o;
  }
}

__global__ __launch_bounds__(256) void dion2_sum_slabs_kernel(const float* __restrict__ part,
                                                             int64_t n, int slabs,
                                                             float* __restrict__ out) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  float s = part[i];
  for (int z = 1; z < slabs; ++z) s += part[(int64_t)z * n + i];
  out[i] = s;
}

int dion2_acc_slabs(int n_mat, int rows, int cols) {
  const int64_t blocks = (int64_t)((cols / 4 + 63) / 64) * n_mat;
  int64_t s = (2048 + blocks - 1) / blocks;
  const int64_t s_max = rows / 64 > 0 ? rows / 64 : 1;
  if (s > s_max) s = s_max;
  if (s > 32) s = 32;
  return s < 1 ? 1 : (int)s;
}

hipError_t launch_dion2_accumulate(const PtrTab& G, int g_dtype, const PtrTab& M, int m_dtype, int n_mat,
                                   int mats_per_ptr, int rows, int cols, int select_rows,
                                   float* norms, bool vec4, float* slab_scratch, int slabs,
                                   hipStream_t st) {
  // DISPATCH(kernel, grid, args...): the four (gradient, momentum) dtype pairs
#define ACC_LAUNCH(K, GRID, ...)                                                                        \
  do {                                                                                                  \
    if (g_dtype == 0 && m_dtype == 0)                                                                   \
      hipLaunchKernelGGL((K<bf16_t, bf16_t>), GRID, dim3(256), 0, st, __VA_ARGS__);                      \
    else if (g_dtype == 0)                                                                              \
      hipLaunchKernelGGL((K<bf16_t, float>), GRID, dim3(256), 0, st, __VA_ARGS__);                       \
    else if (m_dtype == 0)                                                                              \
      hipLaunchKernelGGL((K<float, bf16_t>), GRID, dim3(256), 0, st, __VA_ARGS__);                       \
    else                                                                                                \
      hipLaunchKernelGGL((K<float, float>), GRID, dim3(256), 0, st, __VA_ARGS__);                        \
  } while (0)
  if (select_rows) {
    dim3 grid((rows + 3) / 4, n_mat);
    ACC_LAUNCH(dion2_acc_rows_kernel, grid, G, M, mats_per_ptr, rows, cols, norms);
  } else if (vec4) {
    if (!slab_scratch) slabs = 1;
    const int slab_rows = ((rows + slabs - 1) / slabs + 3) / 4 * 4;
    slabs = (rows + slab_rows - 1) / slab_rows;
    float* dst = slabs > 1 ? slab_scratch : norms;
    dim3 grid((cols / 4 + 63) / 64, n_mat, slabs);
    ACC_LAUNCH(dion2_acc_cols_vec_kernel, grid, G, M, mats_per_ptr, rows, cols, slab_rows, dst);
    if (slabs > 1) {
      const int64_t n = (int64_t)n_mat * cols;
      hipLaunchKernelGGL(dion2_sum_slabs_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st,
                         slab_scratch, n, slabs, norms);
    }
  } else {
    dim3 grid((cols + 63) / 64, n_mat);
    ACC_LAUNCH(dion2_acc_cols_kernel, grid, G, M, mats_per_ptr, rows, cols, norms);
  }
#undef ACC_LAUNCH
  return hipGetLastError();
}

// Top-k by rank counting.  Stage 1 (block = 256 candidates of one matrix): the rank of a candidate is
// the number of entries that beat it (larger value, or equal value at a lower index); it is selected
// iff rank < k, and the flag goes to map (0 / -1).  NaN counts as +inf.  The row passes through LDS in
// chunks of kRankChunk entries (one chunk for every dimension a weight matrix has in practice) and is
// compared four entries per LDS read; entries before / after the block's own range need one
// comparison each (>= / >).  Stage 2 (one block per matrix) turns the flags into ascending positions.
constexpr int kRankChunk = 32768;  // floats per LDS chunk (128 KB); a multiple of the 256 candidates

__global__ __launch_bounds__(256) void dion2_rank_kernel(const float* __restrict__ norms, int dim,
                                                         int k, int32_t* __restrict__ map) {
  extern __shared__ float4 vals4[];  // chunk rounded up to 4 floats; padding -1 (never beats anything)
  float* vals = (float*)vals4;
  const int mat = blockIdx.y;
  const float* v = norms + (int64_t)mat * dim;
  const int b0 = blockIdx.x * 256;  // multiple of 4
  const int i = b0 + threadIdx.x;
  float x = i < dim ? v[i] : 0.f;
  if (x != x) x = INFINITY;
  int rank = 0;
  for (int c0 = 0; c0 < dim; c0 += kRankChunk) {
    const int cn = (dim - c0) < kRankChunk ? (dim - c0) : kRankChunk;
    const int cn4 = (cn + 3) / 4;
    __syncthreads();  // the previous chunk has been consumed
    for (int t = threadIdx.x; t < cn4 * 4; t += 256) {
      float y = t < cn ? v[c0 + t] : -1.0f;
      if (y != y) y = INFINITY;
      vals[t] = y;
    }
    __syncthreads();
    if (i < dim) {
      // the block's own candidates occupy [lo4, hi4) of this chunk (in float4 units), if at all
      int lo4 = (b0 > c0 ? b0 - c0 : 0) / 4, hi4 = (b0 + 256 > c0 ? b0 + 256 - c0 : 0) / 4;
      lo4 = lo4 < cn4 ? lo4 : cn4;
      hi4 = hi4 < cn4 ? hi4 : cn4;
      for (int j4 = 0; j4 < lo4; ++j4) {
        const float4 y = vals4[j4];
        rank += (y.x >= x) + (y.y >= x) + (y.z >= x) + (y.w >= x);
      }
      for (int j4 = lo4; j4 < hi4; ++j4) {
        const float4 y = vals4[j4];
        const int j = c0 + j4 * 4;
        rank += ((y.x > x) || (y.x == x && j < i)) + ((y.y > x) || (y.y == x && j + 1 < i)) +
                ((y.z > x) || (y.z == x && j + 2 < i)) + ((y.w > x) || (y.w == x && j + 3 < i));
      }
      for (int j4 = hi4; j4 < cn4; ++j4) {
        const float4 y = vals4[j4];
        rank += (y.x > x) + (y.y > x) + (y.z > x) + (y.w > x);
      }
    }
  }
  if (i < dim) map[(int64_t)mat * dim + i] = rank < k ? 0 : -1;
}

__global__ __launch_bounds__(1024) void dion2_compact_kernel(int dim, int k, int32_t* __restrict__ idx,
                                                             int32_t* __restrict__ map) {
  __shared__ int wave_tot[16];
  const int mat = blockIdx.x;
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  int running = 0;  // selected entries before the current chunk (same in every thread)
  for (int base = 0; base < dim; base += 1024) {
    const int i = base + threadIdx.x;
    const int sel = (i < dim) ? (map[(int64_t)mat * dim + i] == 0) : 0;
    const unsigned long long ball = __ballot(sel);
    const int in_wave = __popcll(ball & ((1ull << lane) - 1ull));
    __syncthreads();
    if (lane == 0) wave_tot[w] = __popcll(ball);
    __syncthreads();
    int before = 0, total = 0;
    for (int q = 0; q < 16; ++q) {
      const int tq = wave_tot[q];
      if (q < w) before += tq;
      total += tq;
    }
    if (sel) {
      const int pos = running + before + in_wave;
      idx[(int64_t)mat * k + pos] = i;
      map[(int64_t)mat * dim + i] = pos;
    }
    running += total;
  }
}

hipError_t launch_dion2_topk(const float* norms, int n_mat, int dim, int k, int32_t* idx,
                             int32_t* map, hipStream_t st) {
  const int chunk = dim < kRankChunk ? dim : kRankChunk;
  const size_t shmem = (size_t)((chunk + 3) / 4) * 16;
  static std::atomic<uint64_t> attr_done{0};
  if (hipError_t e = set_max_dynamic_lds_once((const void*)dion2_rank_kernel, 160 * 1024 - 256, attr_done))
    return e;
  hipLaunchKernelGGL(dion2_rank_kernel, dim3((dim + 255) / 256, n_mat), dim3(256), shmem, st, norms,
                     dim, k, map);
  hipLaunchKernelGGL(dion2_compact_kernel, dim3(n_mat), dim3(1024), 0, st, dim, k, idx, map);
  return hipGetLastError();
}

// U_sel = bf16(M[sel]); M[sel] *= ef_decay.
// rows selected: block (j, mat) copies row idx[j]; columns selected: block (row, mat) gathers the k
// selected columns (ascending, so the reads walk the row forwards).
// SUMSQ: the block also writes the sum of squares of the bf16 values of its slice of U, sumsq[mat * gridDim.x +
// blockIdx.x] -- one partial sum of ||U_mat||_F^2 per selected row (rows selected) or per row (columns).
template <typename MT, bool VEC, bool SUMSQ = false>
__global__ __launch_bounds__(256) void dion2_gather_kernel(PtrTab M, int mats_per_ptr, int rows,
                                                           int cols, int select_rows,
                                                           const int32_t* __restrict__ idx, int k,
                                                           float ef_decay, bf16_t* __restrict__ U,
                                                           float* __restrict__ sumsq = nullptr) {
  __shared__ float red[16];
  float ss = 0.f;
  const int mat = blockIdx.y;
  MT* m = (MT*)M.p[mat / mats_per_ptr] + (int64_t)(mat % mats_per_ptr) * rows * cols;
  const int32_t* id = idx + (int64_t)mat * k;
  if (select_rows) {
    const int j = blockIdx.x;
    MT* src = m + (int64_t)id[j] * cols;
    bf16_t* u = U + ((int64_t)mat * k + j) * cols;
    if (VEC) {
      for (int c4 = threadIdx.x; c4 < cols / 4; c4 += 256) {
        float v[4];
        st_load4<MT>(src, c4, v);
        st_store4<bf16_t>(u, c4, v);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          if (SUMSQ) {
            const float r = st_round<bf16_t>(v[e]);
            ss += r * r;
          }
          v[e] = __fmul_rn(v[e], ef_decay);
        }
        st_store4<MT>(src, c4, v);
      }
    } else {
      for (int c = threadIdx.x; c < cols; c += 256) {
        const float v = st_load<MT>(src, c);
        u[c] = f32_to_bf16(v);
        if (SUMSQ) {
          const float r = st_round<bf16_t>(v);
          ss += r * r;
        }
        st_store<MT>(src, c, __fmul_rn(v, ef_decay));
      }
    }
  } else {
    const int r = blockIdx.x;
    MT* src = m + (int64_t)r * cols;
    bf16_t* u = U + ((int64_t)mat * rows + r) * k;
    for (int j = threadIdx.x; j < k; j += 256) {
      const int c = id[j];
      const float v = st_load<MT>(src, c);
      u[j] = f32_to_bf16(v);
      if (SUMSQ) {
        const float q = st_round<bf16_t>(v);
        ss += q * q;
      }
      st_store<MT>(src, c, __fmul_rn(v, ef_decay));
    }
  }
  if (SUMSQ) {
    ss = block_sum(ss, red);
    if (threadIdx.x == 0) sumsq[(int64_t)mat * gridDim.x + blockIdx.x] = ss;
  }
}

// Columns selected from tall matrices, U written transposed ([k][rows]: the short side along rows, the
// layout the orthogonalization carries): one tile of 64 rows x 64 selected columns per workgroup, staged
// through LDS so that U^T rows leave as whole 128-byte runs.  sumsq[(mat * row_tiles + row tile) * (k / 64) +
// column tile]: sum of squares of the tile's bf16 values.  rows % 64 == 0, k % 64 == 0.
template <typename MT>
__global__ __launch_bounds__(256) void dion2_gather_cols_transposed_kernel(PtrTab M, int mats_per_ptr, int rows,
                                                                           int cols,
                                                                           const int32_t* __restrict__ idx, int k,
                                                                           float ef_decay, bf16_t* __restrict__ U,
                                                                           float* __restrict__ sumsq) {
  __shared__ __attribute__((aligned(16))) bf16_t tile[64][72];
  __shared__ float red[16];
  const int mat = blockIdx.z;
  MT* m = (MT*)M.p[mat / mats_per_ptr] + (int64_t)(mat % mats_per_ptr) * rows * cols;
  const int r0 = blockIdx.y * 64, j0 = blockIdx.x * 64;
  const int j = threadIdx.x & 63, rsub = threadIdx.x >> 6;
  const int c = idx[(int64_t)mat * k + j0 + j];
  float ss = 0.f;
  float v[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) v[i] = st_load<MT>(m, (int64_t)(r0 + rsub + 4 * i) * cols + c);
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const bf16_t b = f32_to_bf16(v[i]);
    tile[rsub + 4 * i][j] = b;
    const float q = bf16_to_f32(b);
    ss += q * q;
    st_store<MT>(m, (int64_t)(r0 + rsub + 4 * i) * cols + c, __fmul_rn(v[i], ef_decay));
  }
  ss = block_sum(ss, red);  // (its barriers also order the tile writes before the reads below)
  if (threadIdx.x == 0)
    sumsq[((int64_t)mat * gridDim.y + blockIdx.y) * gridDim.x + blockIdx.x] = ss;
  bf16_t* ut = U + (int64_t)mat * k * rows;
  const int chunk = threadIdx.x & 7, rr = threadIdx.x >> 3;
#pragma unroll
  for (int pass = 0; pass < 2; ++pass) {
    const int col = rr + pass * 32;
    uint32_t w[4];
#pragma unroll
    for (int e = 0; e < 4; ++e)
      w[e] = (uint32_t)tile[chunk * 8 + 2 * e][col] | ((uint32_t)tile[chunk * 8 + 2 * e + 1][col] << 16);
    *(uint4*)(ut + (int64_t)(j0 + col) * rows + r0 + chunk * 8) = make_uint4(w[0], w[1], w[2], w[3]);
  }
}

hipError_t launch_dion2_gather(const PtrTab& M, int m_dtype, int n_mat, int mats_per_ptr, int rows, int cols,
                               int select_rows, const int32_t* idx, int k, float ef_decay, bf16_t* U,
                               bool vec4, hipStream_t st) {
  dim3 grid(select_rows ? k : rows, n_mat);
#define GATHER_LAUNCH(MT, V)                                                                          \
  hipLaunchKernelGGL((dion2_gather_kernel<MT, V>), grid, dim3(256), 0, st, M, mats_per_ptr, rows, cols, \
                     select_rows, idx, k, ef_decay, U)
  if (m_dtype == 0) {
    if (vec4) GATHER_LAUNCH(bf16_t, true); else GATHER_LAUNCH(bf16_t, false);
  } else {
    if (vec4) GATHER_LAUNCH(float, true); else GATHER_LAUNCH(float, false);
  }
#undef GATHER_LAUNCH
  return hipGetLastError();
}

hipError_t launch_dion2_gather_prepared(const PtrTab& M, int m_dtype, int n_mat, int mats_per_ptr, int rows,
                                        int cols, int select_rows, const int32_t* idx, int k, float ef_decay,
                                        bf16_t* U, float* sumsq, bool vec4, hipStream_t st) {
  if (!select_rows && rows > k) {
    dim3 grid(k / 64, rows / 64, n_mat);
    if (m_dtype == 0)
      hipLaunchKernelGGL(dion2_gather_cols_transposed_kernel<bf16_t>, grid, dim3(256), 0, st, M, mats_per_ptr, rows,
                         cols, idx, k, ef_decay, U, sumsq);
    else
      hipLaunchKernelGGL(dion2_gather_cols_transposed_kernel<float>, grid, dim3(256), 0, st, M, mats_per_ptr, rows,
                         cols, idx, k, ef_decay, U, sumsq);
    return hipGetLastError();
  }
  dim3 grid(select_rows ? k : rows, n_mat);
#define GATHERS_LAUNCH(MT, V)                                                                               \
  hipLaunchKernelGGL((dion2_gather_kernel<MT, V, true>), grid, dim3(256), 0, st, M, mats_per_ptr, rows, cols, \
                     select_rows, idx, k, ef_decay, U, sumsq)
  if (m_dtype == 0) {
    if (vec4) GATHERS_LAUNCH(bf16_t, true); else GATHERS_LAUNCH(bf16_t, false);
  } else {
    if (vec4) GATHERS_LAUNCH(float, true); else GATHERS_LAUNCH(float, false);
  }
#undef GATHERS_LAUNCH
  return hipGetLastError();
}

// x = a*x - b*u[map] on selected slices, x = a*x elsewhere; one rounding of the sum.
// Block (row group of 8, mat); 4 columns per thread on the vector path.  u is bf16 or fp32 (UT).
template <typename UT>
static __device__ __forceinline__ float u_load(const UT* u, int64_t i) {
  return sizeof(UT) == 2 ? bf16_to_f32(((const bf16_t*)u)[i]) : ((const float*)u)[i];
}
template <typename UT>
static __device__ __forceinline__ float4 u_load4(const UT* u, int64_t i) {
  if (sizeof(UT) == 2) {
    const uint2 raw = *(const uint2*)((const bf16_t*)u + i);
    return make_float4(__uint_as_float(raw.x << 16), __uint_as_float(raw.x & 0xffff0000u),
                       __uint_as_float(raw.y << 16), __uint_as_float(raw.y & 0xffff0000u));
  }
  return *(const float4*)((const float*)u + i);
}

template <bool VEC, typename UT, typename XT>
__global__ __launch_bounds__(256) void dion2_post_kernel(PtrTab X, int mats_per_ptr, int rows,
                                                         int cols, int select_rows,
                                                         const UT* __restrict__ U, int k,
                                                         const int32_t* __restrict__ map,
                                                         const float* __restrict__ row_scale,
                                                         const float* __restrict__ lr_dev,
                                                         const float* __restrict__ adj_lr_dev,
                                                         float adj_ratio,
                                                         const float* __restrict__ wd_dev,
                                                         float wd_host) {
  const int mat = blockIdx.y;
  XT* x = (XT*)X.p[mat / mats_per_ptr] + (int64_t)(mat % mats_per_ptr) * rows * cols;
  const float lr = *lr_dev;
  const float wd = wd_dev ? *wd_dev : wd_host;
  const float a = __fsub_rn(1.0f, __fmul_rn(lr, wd));
  const float b0 = __fmul_rn(adj_lr_dev ? *adj_lr_dev : lr, adj_ratio);
  float b = b0;
  const int dim = select_rows ? rows : cols;
  const int32_t* mp = map + (int64_t)mat * dim;
  const UT* u = U + (int64_t)mat * (select_rows ? (int64_t)k * cols : (int64_t)rows * k);
  const int r_end = (blockIdx.x * 8 + 8) < rows ? (blockIdx.x * 8 + 8) : rows;
  for (int r = blockIdx.x * 8; r < r_end; ++r) {
    XT* xr = x + (int64_t)r * cols;
    if (select_rows) {
      const int j = mp[r];
      const UT* ur = u + (int64_t)(j < 0 ? 0 : j) * cols;
      // per-row scale of the selected slice (rows selected only): u is multiplied by it first
      if (row_scale && j >= 0) b = __fmul_rn(b0, row_scale[(int64_t)mat * k + j]);
      if (VEC) {
        for (int c4 = threadIdx.x; c4 < cols / 4; c4 += 256) {
          float v[4];
          st_load4<XT>(xr, c4, v);
          float4 uv = make_float4(0.f, 0.f, 0.f, 0.f);
          if (j >= 0) uv = u_load4<UT>(ur, c4 * 4);
          v[0] = fmaf(a, v[0], -(b * uv.x));
          v[1] = fmaf(a, v[1], -(b * uv.y));
          v[2] = fmaf(a, v[2], -(b * uv.z));
          v[3] = fmaf(a, v[3], -(b * uv.w));
          st_store4<XT>(xr, c4, v);
        }
      } else {
        for (int c = threadIdx.x; c < cols; c += 256) {
          const float uv = j >= 0 ? u_load<UT>(ur, c) : 0.f;
          st_store<XT>(xr, c, fmaf(a, st_load<XT>(xr, c), -(b * uv)));
        }
      }
    } else {
      const UT* ur = u + (int64_t)r * k;
      if (VEC) {
        for (int c4 = threadIdx.x; c4 < cols / 4; c4 += 256) {
          float v[4];
          st_load4<XT>(xr, c4, v);
          const int4 j4 = *(const int4*)(mp + c4 * 4);
          const float u0 = j4.x >= 0 ? u_load<UT>(ur, j4.x) : 0.f;
          const float u1 = j4.y >= 0 ? u_load<UT>(ur, j4.y) : 0.f;
          const float u2 = j4.z >= 0 ? u_load<UT>(ur, j4.z) : 0.f;
          const float u3 = j4.w >= 0 ? u_load<UT>(ur, j4.w) : 0.f;
          v[0] = fmaf(a, v[0], -(b * u0));
          v[1] = fmaf(a, v[1], -(b * u1));
          v[2] = fmaf(a, v[2], -(b * u2));
          v[3] = fmaf(a, v[3], -(b * u3));
          st_store4<XT>(xr, c4, v);
        }
      } else {
        for (int c = threadIdx.x; c < cols; c += 256) {
          const int j = mp[c];
          const float uv = j >= 0 ? u_load<UT>(ur, j) : 0.f;
          st_store<XT>(xr, c, fmaf(a, st_load<XT>(xr, c), -(b * uv)));
        }
      }
    }
  }
}

hipError_t launch_dion2_post(const PtrTab& X, int x_dtype, int n_mat, int mats_per_ptr, int rows, int cols,
                             int select_rows, const void* U, int u_dtype, int k, const int32_t* map,
                             const float* row_scale, const float* lr_dev, const float* adj_lr_dev,
                             float adj_ratio, const float* wd_dev, float wd_host, bool vec4,
                             hipStream_t st) {
  dim3 grid((rows + 7) / 8, n_mat);
#define D2POST_LAUNCH(V, UT, XT)                                                                          \
  hipLaunchKernelGGL((dion2_post_kernel<V, UT, XT>), grid, dim3(256), 0, st, X, mats_per_ptr, rows, cols, \
                     select_rows, (const UT*)U, k, map, row_scale, lr_dev, adj_lr_dev, adj_ratio,           \
                     wd_dev, wd_host)
#define D2POST_LAUNCH_X(V, UT) \
  do { if (x_dtype == 0) D2POST_LAUNCH(V, UT, bf16_t); else D2POST_LAUNCH(V, UT, float); } while (0)
  if (u_dtype == 0) {
    if (vec4) D2POST_LAUNCH_X(true, bf16_t); else D2POST_LAUNCH_X(false, bf16_t);
  } else {
    if (vec4) D2POST_LAUNCH_X(true, float); else D2POST_LAUNCH_X(false, float);
  }
#undef D2POST_LAUNCH_X
#undef D2POST_LAUNCH
  return hipGetLastError();
}

// map[m][idx[m][j]] = j for the k (distinct, unordered) int64 indices of every matrix, -1 elsewhere.
// One block per matrix: the fill and the scatter are separated by a block barrier.
__global__ __launch_bounds__(256) void dion2_index_map_kernel(const int64_t* __restrict__ idx, int k,
                                                              int dim, int32_t* __restrict__ map) {
  const int mat = blockIdx.x;
  int32_t* mp = map + (int64_t)mat * dim;
  for (int i = threadIdx.x; i < dim; i += 256) mp[i] = -1;
  __syncthreads();
  const int64_t* id = idx + (int64_t)mat * k;
  for (int j = threadIdx.x; j < k; j += 256) {
    const int64_t i = id[j];
    if (i >= 0 && i < dim) mp[i] = j;
  }
}

hipError_t launch_dion2_index_map(const int64_t* idx, int n_mat, int k, int dim, int32_t* map,
                                  hipStream_t st) {
  hipLaunchKernelGGL(dion2_index_map_kernel, dim3(n_mat), dim3(256), 0, st, idx, k, dim, map);
  return hipGetLastError();
}

}  // namespace dion
