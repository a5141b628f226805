// Shared declarations for the gfx950 kernels behind the C-ABI in include/dion_hip.h.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

namespace dion {

typedef uint16_t bf16_t;  // raw bfloat16 bits in memory

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;

__device__ __forceinline__ float bf16_to_f32(bf16_t v) {
  return __uint_as_float(((uint32_t)v) << 16);
}

// Round-to-nearest-even float -> bf16 (hardware v_cvt_pk_bf16_f32 on gfx950).
__device__ __forceinline__ bf16_t f32_to_bf16(float f) {
  __bf16 b = (__bf16)f;
  return __builtin_bit_cast(bf16_t, b);
}

__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  bf16x2 v;
  v[0] = (__bf16)lo;
  v[1] = (__bf16)hi;
  return __builtin_bit_cast(uint32_t, v);
}

// Optimizer state (parameters, momentum, second moments) lives in memory as fp32 or bf16.  All
// arithmetic on it is fp32; a bf16 value is rounded once, when it is stored.  i4 / i8 index groups
// of 4 / 8 consecutive elements (8- / 16-byte accesses for bf16, 16-byte pairs for fp32).
template <typename T>
__device__ __forceinline__ float st_load(const T* p, int64_t i) {
  if constexpr (sizeof(T) == 2) return bf16_to_f32(p[i]);
  else return p[i];
}
template <typename T>
__device__ __forceinline__ void st_store(T* p, int64_t i, float v) {
  if constexpr (sizeof(T) == 2) p[i] = f32_to_bf16(v);
  else p[i] = v;
}
// The value a later load of the stored element returns.
template <typename T>
__device__ __forceinline__ float st_round(float v) {
  if constexpr (sizeof(T) == 2) return bf16_to_f32(f32_to_bf16(v));
  else return v;
}
template <typename T>
__device__ __forceinline__ void st_load4(const T* p, int64_t i4, float v[4]) {
  if constexpr (sizeof(T) == 2) {
    const uint2 raw = ((const uint2*)p)[i4];
    v[0] = __uint_as_float(raw.x << 16);
    v[1] = __uint_as_float(raw.x & 0xffff0000u);
    v[2] = __uint_as_float(raw.y << 16);
    v[3] = __uint_as_float(raw.y & 0xffff0000u);
  } else {
    const float4 q = ((const float4*)p)[i4];
    v[0] = q.x; v[1] = q.y; v[2] = q.z; v[3] = q.w;
  }
}
template <typename T>
__device__ __forceinline__ void st_store4(T* p, int64_t i4, const float v[4]) {
  if constexpr (sizeof(T) == 2) {
    uint2 o;
    o.x = pack_bf16x2(v[0], v[1]);
    o.y = pack_bf16x2(v[2], v[3]);
    ((uint2*)p)[i4] = o;
  } else {
    ((float4*)p)[i4] = make_float4(v[0], v[1], v[2], v[3]);
  }
}
template <typename T>
__device__ __forceinline__ void st_load8(const T* p, int64_t i8, float v[8]) {
  if constexpr (sizeof(T) == 2) {
    const uint4 raw = ((const uint4*)p)[i8];
    const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      v[2 * e] = __uint_as_float(w[e] << 16);
      v[2 * e + 1] = __uint_as_float(w[e] & 0xffff0000u);
    }
  } else {
    st_load4<T>(p, 2 * i8, v);
    st_load4<T>(p, 2 * i8 + 1, v + 4);
  }
}
template <typename T>
__device__ __forceinline__ void st_store8(T* p, int64_t i8, const float v[8]) {
  if constexpr (sizeof(T) == 2) {
    uint4 o;
    o.x = pack_bf16x2(v[0], v[1]);
    o.y = pack_bf16x2(v[2], v[3]);
    o.z = pack_bf16x2(v[4], v[5]);
    o.w = pack_bf16x2(v[6], v[7]);
    ((uint4*)p)[i8] = o;
  } else {
    st_store4<T>(p, 2 * i8, v);
    st_store4<T>(p, 2 * i8 + 1, v + 4);
  }
}

// Muon's decoupled weight decay (plain or cautious) + scaled update of one element
// (dion/muon.py:315-347): a = 1 - lr*wd, coeff = lr*wd, b = lr*adj_ratio.  Every operation is
// rounded on its own, in the order of the eager reference, in every translation unit that uses it.
__device__ __forceinline__ float muon_post_one(float x, float u, float a, float coeff, float b, int cautious) {
  // Plain operators under this pragma: no fused multiply-add, whatever the translation unit's default
  // (the __fmul_rn / __fsub_rn wrappers carry the default of the header that defines them).
#pragma clang fp contract(off)
  if (cautious) {
    // mask = min(sign(x*u) + 1, 1): 0 only where x*u < 0  (dion/muon.py:333-340)
    const float mask = (x * u < 0.f) ? 0.f : 1.f;
    x = x - (x * mask) * coeff;
  } else {
    x = x * a;
  }
  return x - u * b;
}

// coeff = lr*wd, a = 1 - coeff, b = lr*adj_ratio, each rounded on its own.
__device__ __forceinline__ void muon_post_coeffs(float lr, float wd, float adj_ratio, float& a, float& coeff,
                                                 float& b) {
#pragma clang fp contract(off)
  coeff = lr * wd;
  a = 1.0f - coeff;
  b = lr * adj_ratio;
}

// Up to kMaxPtrs device pointers passed by value in the kernel-argument segment: the
// list-of-parameters of one shape group reaches the GPU without a host->device copy.
constexpr int kMaxPtrs = 64;
struct PtrTab {
  uint64_t p[kMaxPtrs];
};

// The Muon update applied by the epilogue of the last GEMM of an orthogonalization instead of
// storing the product: matrix b of the launch updates the parameter matrix
// X.p[b / mats_per_ptr] + (b % mats_per_ptr) * strideC (strideCt), leading dimension ldc (ldct),
// with the product element rounded to bf16 first (what a separate update pass would read back).
struct FusedPost {
  PtrTab X;
  int mats_per_ptr;
  int vec_ok;  // every pointer is 16-byte aligned: the transposed form may use 16-byte accesses
  const float* lr_dev;
  const float* wd_dev;  // optional; wd_host otherwise
  float wd_host;
  float adj_ratio;
  int cautious;
};
struct NoPost {
  int unused;
};

// Raises a kernel's dynamic-LDS limit once per device: the attribute belongs to the device that is
// current when it is set, so `done` keeps one bit per device ordinal.
static inline hipError_t set_max_dynamic_lds_once(const void* fn, int bytes, std::atomic<uint64_t>& done) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  const uint64_t bit = 1ull << (dev & 63);
  if (done.load(std::memory_order_acquire) & bit) return hipSuccess;
  e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (e != hipSuccess) return e;
  done.fetch_or(bit, std::memory_order_release);
  return hipSuccess;
}

// One batched C = alpha * P * Q^T + beta * D problem, all operands row-major bf16 with the
// reduction dimension contiguous ("NT" GEMM).  M, N, K are the computed extents and must be
// multiples of the tile the launcher picks; whole tiles are stored, so destinations are padded
// to the tile as well.
struct GemmParams {
  const bf16_t* P;   // [batch][M][K], leading dimension ldp
  const bf16_t* Q;   // [batch][N][K], leading dimension ldq (== P when tri); [batch][K][N] if q_kmajor
  const bf16_t* D;   // optional [batch][M][N] addend, leading dimension ldd
  bf16_t* C;         // optional [batch][M][N]
  bf16_t* Ct;        // optional [batch][N][M] (transposed copy; == C when tri -> mirror)
  int64_t strideP, strideQ, strideD, strideC, strideCt;  // batch strides in elements
  int ldp, ldq, ldd, ldc, ldct;
  int M, N, K;
  int batch;
  int tri;           // 1: Q == P, only tiles with tile_row <= tile_col are computed, Ct mirrors
  int q_kmajor;      // 1: Q is stored [K][N] (reduction index along rows); not with tri
  int xcd_interleave;  // set by the launcher: tile list dealt to the XCDs in interleaved 32-tile chunks
  float alpha, beta;
  float diag;        // added to C[i][i] (global diagonal); used with tri to fold a*I into B
  // Optional per-matrix factor of the product, read on the device: matrix b is scaled by
  // alpha * scale_vec[b] (scale_pow == 1) or alpha * scale_vec[b]^2 (scale_pow == 2).  This is how the
  // Frobenius normalisation of an orthogonalization input is folded into its first two GEMMs
  // (A = s^2 U U^T, X' = s B U) instead of being a pass over U.
  const float* scale_vec;
  int scale_pow;
};

// alpha of matrix b of a launch (see GemmParams::scale_vec)
__device__ __forceinline__ float gemm_alpha(const GemmParams& p, int b) {
  if (!p.scale_vec) return p.alpha;
  const float s = p.scale_vec[b];
  return p.alpha * (p.scale_pow == 2 ? s * s : s);
}

// Returns hipSuccess or the launch error; the tile configuration is picked by shape.
hipError_t launch_gemm_nt(const GemmParams& p, hipStream_t stream);
// Tile edge (128 or 256) launch_gemm_nt / launch_gemm_nt_post use for this problem: M and N must be
// multiples of it, K of 128.
int gemm_tile_edge(const GemmParams& p);
// C = P * Q with Q K-major (p.q_kmajor, no tri, no D), the product consumed by the fused Muon update
// instead of being stored: `transposed` false updates X[row][col] (ldc / strideC describe X),
// true updates X[col][row] (ldct / strideCt).  x_dtype 0 = bf16, 1 = fp32.  p.batch <= kMaxPtrs *
// post.mats_per_ptr.
hipError_t launch_gemm_nt_post(const GemmParams& p, const FusedPost& post, int x_dtype, bool transposed,
                               hipStream_t stream);
// Tile edge (128 or 256) launch_gemm_nt would use for a problem whose padded short/long
// dims are given; workspaces are padded to this.
int gemm_pad_granule(int m, int n, int batch);

}  // namespace dion
