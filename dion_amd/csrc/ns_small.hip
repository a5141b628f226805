// Whole Newton-Schulz / Polar-Express orthogonalization of one small matrix per workgroup, resident
// in LDS from the Frobenius normalisation to the last iteration: the per-head regime (e.g. 64 x 768
// attention heads), where the general path is 15 launches of GEMMs too small to fill a CU.
//
// Follows the same arithmetic as the batched driver (dion/newton_schulz_triton.py:508-522,
// dion/polar_express.py:30-50): X = bf16(G) / (||.||_F * s + eps); A = X X^T; B = c A A + b A + a I;
// X = B X, with A, B and X rounded to bf16 once per iteration and fp32 MFMA accumulation.
//
// Layout: X [64][n_pad] bf16 in LDS (row pitch + 16 B so that 16 consecutive rows hit 16 distinct
// 16-byte bank slots), A and B [64][64].  X' = B X needs X with the reduction index along rows:
// those fragments come from ds_read_b64_tr_b16 (a 4 x 16 block of 16-bit elements transposed
// across a 16-lane group), so no transposed copy of X is kept.
#include "elementwise.h"

namespace dion {

typedef __attribute__((ext_vector_type(4))) short s16x4;
constexpr int kThreads = 512;    // eight wavefronts: two per SIMD, so LDS and MFMA latencies of one hide behind the other
constexpr int kMaxChunks = 18;  // 16-byte chunks a thread may hold while loading (n_pad <= 1152)
constexpr int kPartialBytes = 4 * 3 * 64 * 16;  // A = X X^T: f32x4 per lane, three tiles, four wavefront groups
constexpr int kMaxLds = 160 * 1024 - 1024;      // dynamic LDS of one workgroup: the static part (reduction scratch) takes the first KB
#define LDS3(p) ((__attribute__((address_space(3))) s16x4*)(p))

static __device__ __forceinline__ bf16x8 join_tr(s16x4 lo, s16x4 hi) {
  typedef __attribute__((ext_vector_type(8))) short s16x8;
  s16x8 v = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
  return __builtin_bit_cast(bf16x8, v);
}

// One workgroup per CU walks matrices blockIdx.x, blockIdx.x + gridDim.x, ...: while the iterations of one
// matrix run out of LDS, the next matrix is already on its way into registers (it is read from memory once,
// the registers hold it until the norm is known), and the stores of the last iteration are left in flight.
// CH: 16-byte chunks of a matrix a thread holds (12 for n_pad <= 768, else kMaxChunks).  Only the small form
// has the registers to keep the next matrix next to the live values of an iteration; the large one fetches
// each matrix when its turn comes.
template <typename T, int CH>
__global__ __launch_bounds__(kThreads) void ns_small_kernel(const T* __restrict__ in, bf16_t* __restrict__ out,
                                                       int batch, int rows, int cols, int n_pad, NsCoeffs co,
                                                       float norm_scale, float eps) {
  constexpr bool kPrefetch = CH <= 12;
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  __shared__ float red[16];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const bool tall = rows > cols;
  const int m = tall ? cols : rows, n = tall ? rows : cols;  // m <= 64
  const int xp = n_pad * 2 + 16;                              // X row pitch in bytes
  constexpr int ap = 64 * 2 + 16;                             // A / B row pitch in bytes
  char* Xs = lds;
  char* As = lds + 64 * xp;
  char* Bs = As + 64 * ap;
  const int64_t mat_elems = (int64_t)rows * cols;
  // Each thread keeps its 16-byte chunks of a matrix in registers between the load, the reduction and the
  // scaled store to LDS, so a matrix is read from HBM once and LDS is written once.  Matrices are whole
  // numbers of chunks and all equally aligned, so the choice holds for every matrix of the batch.
  const bool vec = (cols % 8 == 0) && ((((uintptr_t)in) & 15) == 0) && n_pad * 8 <= CH * kThreads;
  const int cpr = tall ? 8 : n_pad / 8;  // chunks per 64-wide (tall) or n_pad-wide (wide) input row
  const int nchunks = 8 * n_pad;         // 64 * n_pad / 8
  uint4 raw[CH];
  auto fetch = [&](int64_t mat) {
    const T* src = in + mat * mat_elems;
    // (the chunk coordinates are recomputed per matrix from a value the compiler cannot see through: hoisted out of
    // the matrix loop they would sit in registers through every iteration phase)
    int tid_l = tid;
    asm volatile("" : "+v"(tid_l));
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      const int idx = tid_l + c * kThreads;
      raw[c] = make_uint4(0, 0, 0, 0);
      if (idx < nchunks) {
        const int r = idx / cpr, c0 = (idx - r * cpr) * 8;  // input row, first input column
        if (r < rows && c0 < cols) {
          if (sizeof(T) == 2) {
            raw[c] = *(const uint4*)((const bf16_t*)src + (int64_t)r * cols + c0);
          } else {
            const float4 f0 = *(const float4*)((const float*)src + (int64_t)r * cols + c0);
            const float4 f1 = *(const float4*)((const float*)src + (int64_t)r * cols + c0 + 4);
            raw[c].x = pack_bf16x2(f0.x, f0.y);
            raw[c].y = pack_bf16x2(f0.z, f0.w);
            raw[c].z = pack_bf16x2(f1.x, f1.y);
            raw[c].w = pack_bf16x2(f1.z, f1.w);
          }
        }
      }
    }
  };
  if (kPrefetch && vec && (int64_t)blockIdx.x < batch) fetch(blockIdx.x);

  for (int64_t mat = blockIdx.x; mat < batch; mat += gridDim.x) {
  const T* src = in + mat * mat_elems;
  bf16_t* dst = out + mat * mat_elems;

  // ---- (raw bf16 values in registers), sum of squares, scale, store to LDS
  float ss = 0.f;
  if (vec) {
    if (!kPrefetch) fetch(mat);
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      const uint32_t w[4] = {raw[c].x, raw[c].y, raw[c].z, raw[c].w};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float lo = __uint_as_float(w[e] << 16), hi = __uint_as_float(w[e] & 0xffff0000u);
        ss += lo * lo;
        ss += hi * hi;
      }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) ss += __shfl_xor(ss, o, 64);
    if (lane == 0) red[wave] = ss;
    __syncthreads();
    const float total = ((red[0] + red[1]) + (red[2] + red[3])) + ((red[4] + red[5]) + (red[6] + red[7]));
    const float sc = 1.0f / (sqrtf(total) * norm_scale + eps);
    int tid_l = tid;
    asm volatile("" : "+v"(tid_l));
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      const int idx = tid_l + c * kThreads;
      if (idx < nchunks) {
        const int r = idx / cpr, c0 = (idx - r * cpr) * 8;
        const uint32_t w[4] = {raw[c].x, raw[c].y, raw[c].z, raw[c].w};
        float v[8];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          v[2 * e] = __uint_as_float(w[e] << 16) * sc;
          v[2 * e + 1] = __uint_as_float(w[e] & 0xffff0000u) * sc;
        }
        if (!tall) {  // X[r][c0..c0+7]
          uint4 o;
          o.x = pack_bf16x2(v[0], v[1]);
          o.y = pack_bf16x2(v[2], v[3]);
          o.z = pack_bf16x2(v[4], v[5]);
          o.w = pack_bf16x2(v[6], v[7]);
          *(uint4*)(Xs + r * xp + c0 * 2) = o;
        } else {  // X[c0+e][r]
#pragma unroll
          for (int e = 0; e < 8; ++e) *(bf16_t*)(Xs + (c0 + e) * xp + r * 2) = f32_to_bf16(v[e]);
        }
      }
    }
    // the registers are free again: the next matrix of this workgroup travels while this one is iterated
    if (kPrefetch && mat + gridDim.x < batch) fetch(mat + gridDim.x);
  } else {
    for (int idx = tid; idx < 64 * n_pad; idx += kThreads) {
      const int i = idx / n_pad, j = idx - i * n_pad;  // X[i][j]
      float v = 0.f;
      if (i < m && j < n) {
        const int64_t g = tall ? (int64_t)j * cols + i : (int64_t)i * cols + j;
        v = sizeof(T) == 2 ? bf16_to_f32(((const bf16_t*)src)[g])
                           : bf16_to_f32(f32_to_bf16(((const float*)src)[g]));
      }
      ss += v * v;
      *(bf16_t*)(Xs + i * xp + j * 2) = f32_to_bf16(v);
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) ss += __shfl_xor(ss, o, 64);
    if (lane == 0) red[wave] = ss;
    __syncthreads();
    const float total = ((red[0] + red[1]) + (red[2] + red[3])) + ((red[4] + red[5]) + (red[6] + red[7]));
    const float sc = 1.0f / (sqrtf(total) * norm_scale + eps);
    for (int idx = tid; idx < 64 * n_pad; idx += kThreads) {
      const int i = idx / n_pad, j = idx - i * n_pad;
      bf16_t* p = (bf16_t*)(Xs + i * xp + j * 2);
      *p = f32_to_bf16(bf16_to_f32(*p) * sc);
    }
  }
  __syncthreads();

  const int frow = lane & 31, fhalf = lane >> 5;
  // A and B (64 x 64) are computed as 16x16 tiles with v_mfma_f32_16x16x32_bf16: lane l holds row / column
  // l % 16 and the eight k values 8 * (l / 16) .. + 7 of a 32-deep step; accumulator element r is row
  // 4 * (l / 16) + r, column l % 16.
  const int r16 = lane & 15, kq = lane >> 4;
  const int ti = wave >> 1, tj0 = (wave & 1) * 2;  // B = poly(A): two neighbouring tiles of one tile row
  const int nstep = n_pad / 32;
  // A = X X^T is symmetric: ten of its sixteen tiles are computed, the others are their mirror images.
  // Four groups of wavefronts take the tiles (row block, column block)
  //   (0,0) (0,1) (0,2) | (3,3) (3,0) (3,1) | (1,1) (1,2) | (2,2) (2,3)
  // -- always the group's first row block against itself and its one or two other row blocks, so a k step
  // costs a group three (two) fragment reads for three (two) MFMAs, the same fragments serving as both
  // operands -- and the two wavefronts of a group split the k steps, even and odd.  (One tile row per
  // wavefront pair over the full k range, the previous form, read 2.4 times as many fragment bytes and
  // computed all sixteen tiles; this phase was LDS-bound.)
  const int ag = wave >> 1, akh = wave & 1;
  const int rb0 = ag == 0 ? 0 : ag == 1 ? 3 : ag == 2 ? 1 : 2;
  const int rb1 = ag == 0 ? 1 : ag == 1 ? 0 : ag == 2 ? 2 : 3;
  const int rb2 = ag == 0 ? 2 : 1;
  const bool three = ag < 2;
  float* Ps = (float*)(Bs + 64 * ap);  // partial sums of the odd-k wavefronts: [group][tile][lane] f32x4

  // wide result with 16-byte aligned rows: written out from LDS as whole rows after the last iteration
  const bool out_rows = !tall && (cols % 8 == 0) && ((((uintptr_t)out) & 15) == 0);
  auto last_it = [&](int it) { return it == co.n - 1; };
  for (int it = 0; it < co.n; ++it) {
    const float a = co.c[it][0], b = co.c[it][1], c = co.c[it][2];
    // ---- A = X X^T
    {
      f32x4 acc[3];
#pragma unroll
      for (int t = 0; t < 3; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
      const char* p0 = Xs + (rb0 * 16 + r16) * xp + kq * 16;
      const char* p1 = Xs + (rb1 * 16 + r16) * xp + kq * 16;
      const char* p2 = Xs + (rb2 * 16 + r16) * xp + kq * 16;
      // fragments of the step after next are requested before the MFMAs of this one (two register sets)
      if (three) {
        bf16x8 f[2][3];
        f[0][0] = *(const bf16x8*)(p0 + akh * 64);
        f[0][1] = *(const bf16x8*)(p1 + akh * 64);
        f[0][2] = *(const bf16x8*)(p2 + akh * 64);
        int s = akh;
        for (; s + 2 < nstep; s += 4) {
          f[1][0] = *(const bf16x8*)(p0 + (s + 2) * 64);
          f[1][1] = *(const bf16x8*)(p1 + (s + 2) * 64);
          f[1][2] = *(const bf16x8*)(p2 + (s + 2) * 64);
          acc[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f[0][0], f[0][0], acc[0], 0, 0, 0);
          acc[1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f[0][0], f[0][1], acc[1], 0, 0, 0);
          acc[2] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f[0][0], f[0][2], acc[2], 0, 0, 0);
          if (s + 4 < nstep) {
            f[0][0] = *(const bf16x8*)(p0 + (s + 4) * 64);
            f[0][1] = *(const bf16x8*)(p1 + (s + 4) * 64);
            f[0][2] = *(const bf16x8*)(p2 + (s + 4) * 64);
          }
          acc[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f[1][0], f[1][0], acc[0], 0, 0, 0);
          acc[1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f[1][0], f[1][1], acc[1], 0, 0, 0);
          acc[2] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f[1][0], f[1][2], acc[2], 0, 0, 0);
        }
        if (s < nstep) {  // an odd number of steps for this wavefront: the last one sits in set 0
          acc[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f[0][0], f[0][0], acc[0], 0, 0, 0);
          acc[1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f[0][0], f[0][1], acc[1], 0, 0, 0);
          acc[2] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f[0][0], f[0][2], acc[2], 0, 0, 0);
        }
      } else {
        bf16x8 f[2][2];
        f[0][0] = *(const bf16x8*)(p0 + akh * 64);
        f[0][1] = *(const bf16x8*)(p1 + akh * 64);
        int s = akh;
        for (; s + 2 < nstep; s += 4) {
          f[1][0] = *(const bf16x8*)(p0 + (s + 2) * 64);
          f[1][1] = *(const bf16x8*)(p1 + (s + 2) * 64);
          acc[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f[0][0], f[0][0], acc[0], 0, 0, 0);
          acc[1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f[0][0], f[0][1], acc[1], 0, 0, 0);
          if (s + 4 < nstep) {
            f[0][0] = *(const bf16x8*)(p0 + (s + 4) * 64);
            f[0][1] = *(const bf16x8*)(p1 + (s + 4) * 64);
          }
          acc[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f[1][0], f[1][0], acc[0], 0, 0, 0);
          acc[1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f[1][0], f[1][1], acc[1], 0, 0, 0);
        }
        if (s < nstep) {
          acc[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f[0][0], f[0][0], acc[0], 0, 0, 0);
          acc[1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f[0][0], f[0][1], acc[1], 0, 0, 0);
        }
      }
      float* pp = Ps + ((ag * 3) * 64 + lane) * 4;
      if (akh == 1) {
#pragma unroll
        for (int t = 0; t < 3; ++t) *(f32x4*)(pp + t * 256) = acc[t];
      }
      __syncthreads();
      if (akh == 0) {
#pragma unroll
        for (int t = 0; t < 3; ++t) {
          if (t == 2 && !three) break;
          const f32x4 o = *(const f32x4*)(pp + t * 256);
          const int cb = t == 0 ? rb0 : t == 1 ? rb1 : rb2;
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int row = rb0 * 16 + kq * 4 + r, col = cb * 16 + r16;
            const bf16_t v = f32_to_bf16(acc[t][r] + o[r]);
            *(bf16_t*)(As + row * ap + col * 2) = v;
            if (t > 0) *(bf16_t*)(As + col * ap + row * 2) = v;
          }
        }
      }
    }
    __syncthreads();
    // ---- B = c A A + b A + a I  (A symmetric: rows of A serve both operands)
    {
      f32x4 acc[2];
      acc[0] = acc[1] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        const bf16x8 fa = *(const bf16x8*)(As + (ti * 16 + r16) * ap + s * 64 + kq * 16);
        const bf16x8 f0 = *(const bf16x8*)(As + (tj0 * 16 + r16) * ap + s * 64 + kq * 16);
        const bf16x8 f1 = *(const bf16x8*)(As + ((tj0 + 1) * 16 + r16) * ap + s * 64 + kq * 16);
        acc[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa, f0, acc[0], 0, 0, 0);
        acc[1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa, f1, acc[1], 0, 0, 0);
      }
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int row = ti * 16 + kq * 4 + r;
          const int col = (tj0 + j) * 16 + r16;
          float v = c * acc[j][r] + b * bf16_to_f32(*(const bf16_t*)(As + row * ap + col * 2));
          if (row == col) v += a;
          *(bf16_t*)(Bs + row * ap + col * 2) = f32_to_bf16(v);
        }
    }
    __syncthreads();
    // ---- X = B X: wavefront w owns column tiles w, w+8, ...; both row tiles per column tile, so
    // the whole 64 x 32 column block is read before it is overwritten.
    {
      bf16x8 fB[2][4];
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int s = 0; s < 4; ++s)
          fB[i][s] = *(const bf16x8*)(Bs + (i * 32 + frow) * ap + s * 32 + fhalf * 16);
      // transposed-read addressing: 16-lane group g covers columns (g&1)*16.., k rows 8*(g>>1)..;
      // lane t of the group points at row t/4, 4-element column chunk t%4.
      const int g16 = lane >> 4, t16 = lane & 15;
      const int trow = 8 * (g16 >> 1) + (t16 >> 2);
      const int tcol = (g16 & 1) * 16 + (t16 & 3) * 4;
      const bool last = (it == co.n - 1);
      // The MFMA operands are swapped (X fragment first): the accumulators then hold (B X)^T tiles, i.e.
      // lane l owns output row i*32 + l%32 and, per group of four accumulator elements, four consecutive
      // output columns -- one 8-byte store per group instead of four 2-byte ones.
      const int ntile = n_pad / 32;
      auto load_tile = [&](int jt, s16x4 (&lo)[4], s16x4 (&hi)[4]) {
        const char* px = Xs + trow * xp + (jt * 32 + tcol) * 2;
#pragma unroll
        for (int s = 0; s < 4; ++s) {
          lo[s] = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS3(px + (s * 16) * xp));
          hi[s] = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS3(px + (s * 16 + 4) * xp));
        }
      };
      auto do_tile = [&](int jt, s16x4 (&clo)[4], s16x4 (&chi)[4], s16x4 (&nlo)[4], s16x4 (&nhi)[4]) {
        f32x16 acc[2];
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
          for (int r = 0; r < 16; ++r) acc[i][r] = 0.f;
        // the next column tile's fragments are requested before this tile's MFMAs and stores
        if (jt + 8 < ntile) load_tile(jt + 8, nlo, nhi);
#pragma unroll
        for (int s = 0; s < 4; ++s) {
          const bf16x8 fx = join_tr(clo[s], chi[s]);
          acc[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fx, fB[0][s], acc[0], 0, 0, 0);
          acc[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fx, fB[1][s], acc[1], 0, 0, 0);
        }
        const int col0 = jt * 32 + 4 * fhalf;  // + 8 * g: first of four consecutive columns
        // The last X' of a wide matrix goes through LDS like the others and leaves as whole rows below (16 bytes
        // per lane): stored from the accumulators it would be 8-byte pieces 1.5 KB apart.
        if (!last || out_rows) {
#pragma unroll
          for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
              uint2 o;
              o.x = pack_bf16x2(acc[i][4 * g], acc[i][4 * g + 1]);
              o.y = pack_bf16x2(acc[i][4 * g + 2], acc[i][4 * g + 3]);
              *(uint2*)(Xs + (i * 32 + frow) * xp + (col0 + 8 * g) * 2) = o;
            }
        } else if (!tall) {
          const bool vec4 = (cols % 4 == 0) && ((((uintptr_t)dst) & 7) == 0);
#pragma unroll
          for (int i = 0; i < 2; ++i) {
            const int row = i * 32 + frow;
            if (row >= m) continue;
#pragma unroll
            for (int g = 0; g < 4; ++g) {
              const int col = col0 + 8 * g;
              bf16_t* q = dst + row * cols + col;
              if (vec4 && col + 3 < n) {
                uint2 o;
                o.x = pack_bf16x2(acc[i][4 * g], acc[i][4 * g + 1]);
                o.y = pack_bf16x2(acc[i][4 * g + 2], acc[i][4 * g + 3]);
                *(uint2*)q = o;
              } else {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                  if (col + e < n) q[e] = f32_to_bf16(acc[i][4 * g + e]);
              }
            }
          }
        } else {
          // tall input: X holds the transpose, output element (col, row); lanes run along `row`
#pragma unroll
          for (int i = 0; i < 2; ++i) {
            const int row = i * 32 + frow;
            if (row >= m) continue;
#pragma unroll
            for (int g = 0; g < 4; ++g)
#pragma unroll
              for (int e = 0; e < 4; ++e) {
                const int col = col0 + 8 * g + e;
                if (col < n) dst[col * cols + row] = f32_to_bf16(acc[i][4 * g + e]);
              }
          }
        }
      };
      s16x4 lo0[4], hi0[4], lo1[4], hi1[4];
      if (wave < ntile) load_tile(wave, lo0, hi0);
      for (int jt = wave; jt < ntile; jt += 16) {
        do_tile(jt, lo0, hi0, lo1, hi1);
        if (jt + 8 < ntile) do_tile(jt + 8, lo1, hi1, lo0, hi0);
      }
    }
    __syncthreads();
    if (last_it(it) && out_rows) {
      // X [m][n] in LDS -> dst [rows][cols], 16 bytes per lane, lanes side by side along a row
      const int cpr8 = cols / 8;
      for (int idx = tid; idx < m * cpr8; idx += kThreads) {
        const int r = idx / cpr8, c8 = idx - r * cpr8;
        *(uint4*)(dst + (int64_t)r * cols + c8 * 8) = *(const uint4*)(Xs + r * xp + c8 * 16);
      }
      __syncthreads();  // X is rewritten by the next matrix
    }
  }
  if (co.n == 0) {  // normalisation only
    for (int idx = tid; idx < m * n; idx += kThreads) {
      const int i = idx / n, j = idx - i * n;
      const int64_t g = tall ? (int64_t)j * cols + i : (int64_t)i * cols + j;
      dst[g] = *(const bf16_t*)(Xs + i * xp + j * 2);
    }
    __syncthreads();  // X is rewritten by the next matrix
  }
  }  // matrices of this workgroup
}

bool ns_small_fits(int rows, int cols) {
  const int m = rows < cols ? rows : cols, n = rows < cols ? cols : rows;
  if (m > 64) return false;
  const int n_pad = (n + 63) / 64 * 64;
  const size_t bytes = (size_t)64 * (n_pad * 2 + 16) + 2 * 64 * (64 * 2 + 16) + kPartialBytes;
  return bytes <= kMaxLds;
}

hipError_t launch_ns_small(const void* in, int in_dtype, bf16_t* out, int batch, int rows, int cols,
                           const NsCoeffs& co, float norm_scale, float eps, hipStream_t st) {
  const int n = rows < cols ? cols : rows;
  const int n_pad = (n + 63) / 64 * 64;
  const size_t bytes = (size_t)64 * (n_pad * 2 + 16) + 2 * 64 * (64 * 2 + 16) + kPartialBytes;
  static std::atomic<uint64_t> done[4];
  const bool small = n_pad * 8 <= 12 * kThreads;
  const void* kern = in_dtype == 0 ? (small ? (const void*)ns_small_kernel<bf16_t, 12> : (const void*)ns_small_kernel<bf16_t, kMaxChunks>)
                                   : (small ? (const void*)ns_small_kernel<float, 12> : (const void*)ns_small_kernel<float, kMaxChunks>);
  if (hipError_t e = set_max_dynamic_lds_once(kern, kMaxLds, done[(in_dtype == 0 ? 0 : 2) + (small ? 0 : 1)])) return e;
  // one workgroup per CU (the LDS footprint admits no second one), each walking its share of the batch
  static std::atomic<int> cu_count[64];
  int dev = 0;
  if (hipError_t e = hipGetDevice(&dev)) return e;
  int cus = cu_count[dev & 63].load(std::memory_order_relaxed);
  if (cus == 0) {
    if (hipError_t e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev)) return e;
    if (cus <= 0) return hipErrorInvalidValue;
    cu_count[dev & 63].store(cus, std::memory_order_relaxed);
  }
  const int grid = batch < cus ? batch : cus;
#define SMALL_LAUNCH(T, CHN)                                                                                   \
  hipLaunchKernelGGL((ns_small_kernel<T, CHN>), dim3(grid), dim3(kThreads), bytes, st, (const T*)in, out, batch, \
                     rows, cols, n_pad, co, norm_scale, eps)
  if (in_dtype == 0) {
    if (small) SMALL_LAUNCH(bf16_t, 12); else SMALL_LAUNCH(bf16_t, kMaxChunks);
  } else {
    if (small) SMALL_LAUNCH(float, 12); else SMALL_LAUNCH(float, kMaxChunks);
  }
#undef SMALL_LAUNCH
  return hipGetLastError();
}

}  // namespace dion
