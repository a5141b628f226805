// Kernels of the whole-matrix ("global" selection scope) Dion2 / NorDion2 sequence for gfx950: the
// selection happens on assembled bf16 matrices inside the orthogonalization call
// (dion/dion2.py:565-620) and the update afterwards only sees a full-size tensor that is zero outside
// the selected slices (dion/dion2.py:623-659, dion/nordion2.py:448-500).  All kernels are single-pass,
// reduce in a fixed order and use no float atomics.
#include "elementwise.h"

namespace dion {

static __device__ __forceinline__ float wave_sum64(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

template <typename T>
static __device__ __forceinline__ float abs_f32(const T* p, int64_t i) {
  return sizeof(T) == 2 ? fabsf(bf16_to_f32(((const bf16_t*)p)[i])) : fabsf(((const float*)p)[i]);
}

static __device__ __forceinline__ float through_bf16(float v) { return bf16_to_f32(f32_to_bf16(v)); }

// ------------------------------------------------------------------------------------------
// Slice L1 norms of a stacked [n_mat, rows, cols] tensor.
// ------------------------------------------------------------------------------------------
// Rows: one wavefront per row.
template <typename T>
__global__ __launch_bounds__(256) void slice_l1_rows_kernel(const T* __restrict__ U, int rows, int cols,
                                                            int round_bf16, float* __restrict__ norms) {
  const int mat = blockIdx.y;
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const int lane = threadIdx.x & 63;
  const T* u = U + ((int64_t)mat * rows + row) * cols;
  float s = 0.f;
  if (sizeof(T) == 2 && (cols & 7) == 0 && (((uintptr_t)u) & 15) == 0) {
    for (int c = lane * 8; c < cols; c += 512) {
      const uint4 raw = *(const uint4*)((const bf16_t*)u + c);
      const uint32_t wv[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        s += fabsf(__uint_as_float(wv[e] << 16));
        s += fabsf(__uint_as_float(wv[e] & 0xffff0000u));
      }
    }
  } else {
    for (int c = lane; c < cols; c += 64) s += abs_f32<T>(u, c);
  }
  s = wave_sum64(s);
  if (lane == 0) norms[(int64_t)mat * rows + row] = round_bf16 ? through_bf16(s) : s;
}

// Columns: a block owns 64*W columns (W consecutive ones per thread) and walks all rows, RL row
// lanes (wavefronts) at a time; the lanes' partial sums are added in lane order.
template <typename T, int W, int RL>
__global__ __launch_bounds__(64 * RL) void slice_l1_cols_kernel(const T* __restrict__ U, int rows, int cols,
                                                                int round_bf16, float* __restrict__ norms) {
  __shared__ float red[RL][64 * W];
  const int mat = blockIdx.y;
  const int t = threadIdx.x & 63, ry = threadIdx.x >> 6;
  const int c = (blockIdx.x * 64 + t) * W;
  const T* u = U + (int64_t)mat * rows * cols;
  float s[W];
#pragma unroll
  for (int e = 0; e < W; ++e) s[e] = 0.f;
  if (c < cols) {
#pragma unroll 4
    for (int r = ry; r < rows; r += RL) {
      const int64_t i = (int64_t)r * cols + c;
      if (W == 4 && sizeof(T) == 2) {
        const uint2 raw = *(const uint2*)((const bf16_t*)u + i);
        s[0] += fabsf(__uint_as_float(raw.x << 16));
        s[1] += fabsf(__uint_as_float(raw.x & 0xffff0000u));
        s[2] += fabsf(__uint_as_float(raw.y << 16));
        s[3] += fabsf(__uint_as_float(raw.y & 0xffff0000u));
      } else if (W == 4) {
        const float4 v = *(const float4*)((const float*)u + i);
        s[0] += fabsf(v.x);
        s[1] += fabsf(v.y);
        s[2] += fabsf(v.z);
        s[3] += fabsf(v.w);
      } else {
#pragma unroll
        for (int e = 0; e < W; ++e) s[e] += abs_f32<T>(u, i + e);
      }
    }
  }
#pragma unroll
  for (int e = 0; e < W; ++e) red[ry][t * W + e] = s[e];
  __syncthreads();
  if (ry == 0 && c < cols) {
#pragma unroll
    for (int e = 0; e < W; ++e) {
      const int q = t * W + e;
      float v = red[0][q];
#pragma unroll
      for (int l = 1; l < RL; ++l) v += red[l][q];
      norms[(int64_t)mat * cols + c + e] = round_bf16 ? through_bf16(v) : v;
    }
  }
}

template <typename T>
static void launch_slice_l1_cols(const T* U, int n_mat, int rows, int cols, int round_bf16, float* norms,
                                 bool vec, hipStream_t st) {
  if (vec) {
    dim3 grid((cols / 4 + 63) / 64, n_mat);
    // few column blocks and many rows: 16 wavefronts per block keep enough loads in flight
    if ((int64_t)grid.x * grid.y < 1024 && rows >= 256)
      hipLaunchKernelGGL((slice_l1_cols_kernel<T, 4, 16>), grid, dim3(1024), 0, st, U, rows, cols,
                         round_bf16, norms);
    else
      hipLaunchKernelGGL((slice_l1_cols_kernel<T, 4, 4>), grid, dim3(256), 0, st, U, rows, cols, round_bf16,
                         norms);
  } else {
    dim3 grid((cols + 63) / 64, n_mat);
    hipLaunchKernelGGL((slice_l1_cols_kernel<T, 1, 4>), grid, dim3(256), 0, st, U, rows, cols, round_bf16,
                       norms);
  }
}

hipError_t launch_slice_l1(const void* U, int dtype, int n_mat, int rows, int cols, int select_rows,
                           int round_bf16, float* norms, hipStream_t st) {
  if (select_rows) {
    dim3 grid((rows + 3) / 4, n_mat);
    if (dtype == 0)
      hipLaunchKernelGGL(slice_l1_rows_kernel<bf16_t>, grid, dim3(256), 0, st, (const bf16_t*)U, rows,
                         cols, round_bf16, norms);
    else
      hipLaunchKernelGGL(slice_l1_rows_kernel<float>, grid, dim3(256), 0, st, (const float*)U, rows,
                         cols, round_bf16, norms);
  } else {
    const int es = dtype == 0 ? 2 : 4;
    const bool vec = (cols % 4) == 0 && (((uintptr_t)U) % (4 * es)) == 0;
    if (dtype == 0)
      launch_slice_l1_cols<bf16_t>((const bf16_t*)U, n_mat, rows, cols, round_bf16, norms, vec, st);
    else
      launch_slice_l1_cols<float>((const float*)U, n_mat, rows, cols, round_bf16, norms, vec, st);
  }
  return hipGetLastError();
}

// ------------------------------------------------------------------------------------------
// Gather the selected slices into a dense block / scatter a dense block back into a full-size
// tensor that is zero elsewhere.  Pure data movement on 2- or 4-byte elements (E).
// ------------------------------------------------------------------------------------------
// Rows: block (j, mat) copies row idx[j] of the source to row j of the block.
// Columns: block (row group of 8, mat) gathers the k selected columns of each of its rows.
template <typename E>
__global__ __launch_bounds__(256) void gather_slices_kernel(const E* __restrict__ U, int rows, int cols,
                                                            int select_rows,
                                                            const int32_t* __restrict__ idx, int k,
                                                            E* __restrict__ sub, int vec16) {
  const int mat = blockIdx.y;
  const E* u = U + (int64_t)mat * rows * cols;
  const int32_t* id = idx + (int64_t)mat * k;
  if (select_rows) {
    const int j = blockIdx.x;
    const E* src = u + (int64_t)id[j] * cols;
    E* dst = sub + ((int64_t)mat * k + j) * cols;
    if (vec16) {
      const int n16 = cols * (int)sizeof(E) / 16;
      for (int c = threadIdx.x; c < n16; c += 256) ((uint4*)dst)[c] = ((const uint4*)src)[c];
    } else {
      for (int c = threadIdx.x; c < cols; c += 256) dst[c] = src[c];
    }
  } else {
    const int r_end = (blockIdx.x * 8 + 8) < rows ? (blockIdx.x * 8 + 8) : rows;
    for (int r = blockIdx.x * 8; r < r_end; ++r) {
      const E* src = u + (int64_t)r * cols;
      E* dst = sub + ((int64_t)mat * rows + r) * k;
      for (int j = threadIdx.x; j < k; j += 256) dst[j] = src[id[j]];
    }
  }
}

// Rows selected: block (row, mat) writes one full row of the output, the block's row map[row] or zeros.
// Columns selected: block (row group of 8, mat); per row, entry c is the block's entry map[c] where the
// map is >= 0, zero elsewhere.
template <typename E>
__global__ __launch_bounds__(256) void scatter_slices_kernel(const E* __restrict__ sub, int rows, int cols,
                                                             int select_rows,
                                                             const int32_t* __restrict__ map, int k,
                                                             E* __restrict__ out, int vec16) {
  const int mat = blockIdx.y;
  if (select_rows) {
    const int r = blockIdx.x;
    E* dst = out + ((int64_t)mat * rows + r) * cols;
    const int j = map[(int64_t)mat * rows + r];
    const E* src = sub + ((int64_t)mat * k + (j < 0 ? 0 : j)) * cols;
    if (vec16) {
      const int n16 = cols * (int)sizeof(E) / 16;
      const uint4 z = make_uint4(0u, 0u, 0u, 0u);
      for (int c = threadIdx.x; c < n16; c += 256) ((uint4*)dst)[c] = j >= 0 ? ((const uint4*)src)[c] : z;
    } else {
      for (int c = threadIdx.x; c < cols; c += 256) dst[c] = j >= 0 ? src[c] : (E)0;
    }
    return;
  }
  const int32_t* mp = map + (int64_t)mat * cols;
  const int r_end = (blockIdx.x * 8 + 8) < rows ? (blockIdx.x * 8 + 8) : rows;
  if (vec16) {
    // V columns per thread: V map entries in (kept across the block's rows), one 16-byte store out
    constexpr int V = 16 / (int)sizeof(E);
    for (int c = threadIdx.x * V; c < cols; c += 256 * V) {
      int j[V];
#pragma unroll
      for (int q = 0; q < V / 4; ++q) {
        const int4 m4 = *(const int4*)(mp + c + 4 * q);
        j[4 * q] = m4.x;
        j[4 * q + 1] = m4.y;
        j[4 * q + 2] = m4.z;
        j[4 * q + 3] = m4.w;
      }
      for (int r = blockIdx.x * 8; r < r_end; ++r) {
        const E* src = sub + ((int64_t)mat * rows + r) * k;
        uint32_t w[4];
        if (sizeof(E) == 2) {
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const uint32_t lo = j[2 * q] >= 0 ? (uint32_t)src[j[2 * q]] : 0u;
            const uint32_t hi = j[2 * q + 1] >= 0 ? (uint32_t)src[j[2 * q + 1]] : 0u;
            w[q] = lo | (hi << 16);
          }
        } else {
#pragma unroll
          for (int q = 0; q < 4; ++q) w[q] = j[q] >= 0 ? (uint32_t)src[j[q]] : 0u;
        }
        *(uint4*)(out + ((int64_t)mat * rows + r) * cols + c) = make_uint4(w[0], w[1], w[2], w[3]);
      }
    }
  } else {
    for (int r = blockIdx.x * 8; r < r_end; ++r) {
      const E* src = sub + ((int64_t)mat * rows + r) * k;
      E* dst = out + ((int64_t)mat * rows + r) * cols;
      for (int c = threadIdx.x; c < cols; c += 256) {
        const int j = mp[c];
        dst[c] = j >= 0 ? src[j] : (E)0;
      }
    }
  }
}

static bool rows_vec16(const void* a, const void* b, int cols, int es) {
  return ((int64_t)cols * es) % 16 == 0 && (((uintptr_t)a) & 15) == 0 && (((uintptr_t)b) & 15) == 0;
}

hipError_t launch_gather_slices(const void* U, int dtype, int n_mat, int rows, int cols, int select_rows,
                                const int32_t* idx, int k, void* sub, hipStream_t st) {
  const int es = dtype == 0 ? 2 : 4;
  const int vec16 = select_rows && rows_vec16(U, sub, cols, es);
  dim3 grid(select_rows ? k : (rows + 7) / 8, n_mat);
  if (es == 2)
    hipLaunchKernelGGL(gather_slices_kernel<uint16_t>, grid, dim3(256), 0, st, (const uint16_t*)U, rows,
                       cols, select_rows, idx, k, (uint16_t*)sub, vec16);
  else
    hipLaunchKernelGGL(gather_slices_kernel<uint32_t>, grid, dim3(256), 0, st, (const uint32_t*)U, rows,
                       cols, select_rows, idx, k, (uint32_t*)sub, vec16);
  return hipGetLastError();
}

hipError_t launch_scatter_slices(const void* sub, int dtype, int n_mat, int rows, int cols,
                                 int select_rows, const int32_t* map, int k, void* out, hipStream_t st) {
  const int es = dtype == 0 ? 2 : 4;
  // rows: both sides move whole 16-byte chunks; columns: the output row and the map do
  const int vec16 = select_rows ? rows_vec16(sub, out, cols, es)
                                : (rows_vec16(out, out, cols, es) && (cols % 8) == 0 &&
                                   (((uintptr_t)map) & 15) == 0);
  dim3 grid(select_rows ? rows : (rows + 7) / 8, n_mat);
  if (es == 2)
    hipLaunchKernelGGL(scatter_slices_kernel<uint16_t>, grid, dim3(256), 0, st, (const uint16_t*)sub,
                       rows, cols, select_rows, map, k, (uint16_t*)out, vec16);
  else
    hipLaunchKernelGGL(scatter_slices_kernel<uint32_t>, grid, dim3(256), 0, st, (const uint32_t*)sub,
                       rows, cols, select_rows, map, k, (uint32_t*)out, vec16);
  return hipGetLastError();
}

// ------------------------------------------------------------------------------------------
// Masked update: the selected slices are the ones whose L1 norm in U is > 0.
// ------------------------------------------------------------------------------------------
// gate[i] = i % dim where norms[i] > 0, else -1 (the row index form the per-row statistics take).
__global__ __launch_bounds__(256) void mask_index_kernel(const float* __restrict__ norms, int64_t n,
                                                         int dim, int32_t* __restrict__ gate) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) gate[i] = norms[i] > 0.f ? (int32_t)(i % dim) : -1;
}

hipError_t launch_mask_index(const float* norms, int n_mat, int dim, int32_t* gate, hipStream_t st) {
  const int64_t n = (int64_t)n_mat * dim;
  hipLaunchKernelGGL(mask_index_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, norms, n,
                     dim, gate);
  return hipGetLastError();
}

// x = a*x - b*u (one rounding of the sum; b carries the per-row scale when given) everywhere -- u is
// zero off the selected slices -- and m *= ef_decay on the selected slices.  Block = 8 rows of one
// matrix.  X and M share their dtype ST (fp32 or bf16).
template <bool VEC, typename ST>
__global__ __launch_bounds__(256) void dion2_post_masked_kernel(PtrTab X, PtrTab M, int mats_per_ptr,
                                                                int rows, int cols, int select_rows,
                                                                const bf16_t* __restrict__ U,
                                                                const float* __restrict__ norms,
                                                                const float* __restrict__ row_scale,
                                                                const float* __restrict__ lr_dev,
                                                                const float* __restrict__ adj_lr_dev,
                                                                float adj_ratio,
                                                                const float* __restrict__ wd_dev,
                                                                float wd_host, float ef_decay) {
  const int mat = blockIdx.y;
  const int64_t moff = (int64_t)(mat % mats_per_ptr) * rows * cols;
  ST* x = (ST*)X.p[mat / mats_per_ptr] + moff;
  ST* m = (ST*)M.p[mat / mats_per_ptr] + moff;
  const bf16_t* u = U + (int64_t)mat * rows * cols;
  const float lr = *lr_dev;
  const float wd = wd_dev ? *wd_dev : wd_host;
  const float a = __fsub_rn(1.0f, __fmul_rn(lr, wd));
  const float b0 = __fmul_rn(adj_lr_dev ? *adj_lr_dev : lr, adj_ratio);
  const int dim = select_rows ? rows : cols;
  const float* nm = norms + (int64_t)mat * dim;
  const int r_end = (blockIdx.x * 8 + 8) < rows ? (blockIdx.x * 8 + 8) : rows;
  for (int r = blockIdx.x * 8; r < r_end; ++r) {
    ST* xr = x + (int64_t)r * cols;
    ST* mr = m + (int64_t)r * cols;
    const bf16_t* ur = u + (int64_t)r * cols;
    const bool row_sel = select_rows && nm[r] > 0.f;
    const float b = (row_scale && select_rows) ? __fmul_rn(b0, row_scale[(int64_t)mat * rows + r]) : b0;
    if (select_rows && !row_sel) {
      // unselected row: u is zero, m stays
      if (VEC) {
        for (int c4 = threadIdx.x; c4 < cols / 4; c4 += 256) {
          float v[4];
          st_load4<ST>(xr, c4, v);
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] = __fmul_rn(a, v[e]);
          st_store4<ST>(xr, c4, v);
        }
      } else {
        for (int c = threadIdx.x; c < cols; c += 256) st_store<ST>(xr, c, __fmul_rn(a, st_load<ST>(xr, c)));
      }
      continue;
    }
    if (VEC) {
      for (int c4 = threadIdx.x; c4 < cols / 4; c4 += 256) {
        float v[4], uv[4];
        st_load4<ST>(xr, c4, v);
        st_load4<bf16_t>(ur, c4, uv);
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = fmaf(a, v[e], -(b * uv[e]));
        st_store4<ST>(xr, c4, v);
        if (select_rows) {
          float mv[4];
          st_load4<ST>(mr, c4, mv);
#pragma unroll
          for (int e = 0; e < 4; ++e) mv[e] = __fmul_rn(mv[e], ef_decay);
          st_store4<ST>(mr, c4, mv);
        } else {
          const float4 n4 = *(const float4*)(nm + c4 * 4);
          if (n4.x > 0.f || n4.y > 0.f || n4.z > 0.f || n4.w > 0.f) {
            float mv[4];
            st_load4<ST>(mr, c4, mv);
            if (n4.x > 0.f) mv[0] = __fmul_rn(mv[0], ef_decay);
            if (n4.y > 0.f) mv[1] = __fmul_rn(mv[1], ef_decay);
            if (n4.z > 0.f) mv[2] = __fmul_rn(mv[2], ef_decay);
            if (n4.w > 0.f) mv[3] = __fmul_rn(mv[3], ef_decay);
            st_store4<ST>(mr, c4, mv);
          }
        }
      }
    } else {
      for (int c = threadIdx.x; c < cols; c += 256) {
        st_store<ST>(xr, c, fmaf(a, st_load<ST>(xr, c), -(b * bf16_to_f32(ur[c]))));
        if (select_rows || nm[c] > 0.f) st_store<ST>(mr, c, __fmul_rn(st_load<ST>(mr, c), ef_decay));
      }
    }
  }
}

hipError_t launch_dion2_post_masked(const PtrTab& X, const PtrTab& M, int s_dtype, int n_mat, int mats_per_ptr,
                                    int rows, int cols, int select_rows, const bf16_t* U,
                                    const float* norms, const float* row_scale, const float* lr_dev,
                                    const float* adj_lr_dev, float adj_ratio, const float* wd_dev,
                                    float wd_host, float ef_decay, bool vec4, hipStream_t st) {
  dim3 grid((rows + 7) / 8, n_mat);
#define MASKED_LAUNCH(V, ST)                                                                              \
  hipLaunchKernelGGL((dion2_post_masked_kernel<V, ST>), grid, dim3(256), 0, st, X, M, mats_per_ptr, rows,  \
                     cols, select_rows, U, norms, row_scale, lr_dev, adj_lr_dev, adj_ratio, wd_dev,        \
                     wd_host, ef_decay)
  if (s_dtype == 0) {
    if (vec4) MASKED_LAUNCH(true, bf16_t); else MASKED_LAUNCH(false, bf16_t);
  } else {
    if (vec4) MASKED_LAUNCH(true, float); else MASKED_LAUNCH(false, float);
  }
#undef MASKED_LAUNCH
  return hipGetLastError();
}

}  // namespace dion
