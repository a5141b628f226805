// Batched bf16 GEMM for gfx950 (CDNA4):  C = alpha * P * Q^T + beta * D (+ diag * I), fp32 accumulate.
//
// Every GEMM of the Newton-Schulz / Polar-Express iteration is an instance of this one kernel:
//   A  = X X^T                     P = Q = X            (tri: upper tiles + mirrored store)
//   B  = c A A + b A + a I         P = Q = A (A = A^T)  (tri, D = A, a on the diagonal)
//   X' = B X  (= a X + (B - aI) X)  P = B, Q = X
// P is always read with the reduction index contiguous ("K-contiguous" rows).  Q comes in two forms:
// K-contiguous rows [N][K] like P (Q^T is then what multiplies P: the Gram products above, or
// X' = B X given X^T, which also stores (X')^T for the next round), or -- QK -- stored with the
// reduction index along rows, [K][N]: X' = B X then reads X as it lies, its MFMA fragments come from
// ds_read_b64_tr_b16 (transposing LDS read), and no X^T has to be kept or written.  QK is the form
// the orthogonalization driver uses.
// This replaces the reference's ns_line_1 / ns_line_2 / ns_line_3
// (dion/newton_schulz_triton.py:88-157, :206-287, :384-447) and the baddbmm of
// dion/newton_schulz_triton.py:557-563.
//
// Kernel structure: one workgroup per BM x BN output tile, WM x WN wavefronts (64 lanes) each
// owning a (BM/WM) x (BN/WN) sub-tile as 16x16 MFMA accumulators (v_mfma_f32_16x16x32_bf16: per
// FLOP half the accumulator register traffic of the 32x32x16 form, which on this power-limited part is
// worth 5 % of clock).  Operand tiles reach a two-slot LDS ring through direct-to-LDS
// loads (global_load_lds_dwordx4, no VGPR staging); XOR swizzles keep the LDS writes and the
// fragment reads bank-conflict free.
#include <type_traits>

#include "common.h"

namespace dion {

#define LDS_PTR(p) ((__attribute__((address_space(3))) void*)(p))
#define GLB_PTR(p) ((const __attribute__((address_space(1))) void*)(p))

template <int BM_, int BN_, int BK_, int WM_, int WN_, int NSTAGE_>
struct TileCfg {
  static constexpr int BM = BM_, BN = BN_, BK = BK_, WM = WM_, WN = WN_, NSTAGE = NSTAGE_;
  static_assert(NSTAGE_ == 2, "the pipeline below is written for a two-slot ring");
  static constexpr int NT = WM * WN * 64;
  static constexpr int CPR = BK / 8;            // 16-byte chunks per tile row
  static constexpr int ROWS_PER_LOAD = NT / CPR; // tile rows covered by one load instruction
  static constexpr int P_BYTES = BM * BK * 2;
  static constexpr int Q_BYTES = BN * BK * 2;
  static constexpr int STAGE_BYTES = P_BYTES + Q_BYTES;
  // Epilogue staging of the transposed tile: per wavefront WTN rows of WTM bf16 (+16 B pad).
  static constexpr int STG_PITCH = (BM / WM_) * 2 + 16;
  static constexpr int STG_BYTES = (BN / WN_) * STG_PITCH;
  static constexpr int RING_BYTES = STAGE_BYTES * NSTAGE;
  static constexpr int LDS_BYTES =
      RING_BYTES > STG_BYTES * WM_ * WN_ ? RING_BYTES : STG_BYTES * WM_ * WN_;
  static constexpr int P_LOADS = BM / ROWS_PER_LOAD;
  static constexpr int Q_LOADS = BN / ROWS_PER_LOAD;
  static constexpr int LOADS_PER_STAGE = P_LOADS + Q_LOADS;
  static constexpr int WTM = BM / WM, WTN = BN / WN;
  static constexpr int TM = WTM / 16, TN = WTN / 16;  // 16 x 16 accumulator tiles of a wavefront tile
  static constexpr int ST = BK / 32;                  // 32-deep MFMA steps per slab
  // The MFMAs of a step run in halves of sixteen: four A fragments against the four B fragments.
  static constexpr int HALVES = TM / 4;
  static_assert(TN == 4 && (TM == 4 || TM == 8) && ST == 2, "wavefront tiles of 64 or 128 rows by 64 columns, 64-deep slabs");
  // gfx950 LDS: 64 banks x 4 B = 256-byte bank rows, and a ds_read_b128 is served 16 lanes at a
  // time.  16 consecutive tile rows must therefore land in 16 distinct 16-byte slots of a bank
  // row: the 256/(2*BK) tile rows that share a bank row take one swizzle value.
  static constexpr int SWZ_DIV = 256 / (BK * 2);
  static_assert(BM % ROWS_PER_LOAD == 0 && BN % ROWS_PER_LOAD == 0, "tile/threads mismatch");
  static_assert(CPR == 8 || CPR == 4, "BK must be 64 or 32");
};

// s_waitcnt with only vmcnt constrained (gfx9 encoding: vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8]
// | vmcnt_hi[15:14]).
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  static_assert(N >= 0 && N < 64, "vmcnt range");
  __builtin_amdgcn_s_waitcnt((N & 0xF) | ((N >> 4) << 14) | 0x0F70);
}

// Compile-time loop: f(std::integral_constant<int, I>()) for I in [I0, N).
template <int I, int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>());
    static_for<I + 1, N>(f);
  }
}

// Issue order of the fragment reads.  A 32-deep step of a wavefront tile is HALVES halves of sixteen MFMAs
// (A fragment i = q / 4 against B fragment j = q % 4); a slab is ST steps, i.e. P = HALVES * ST halves.  While
// the MFMAs of one half issue, the fragments of the next half are requested behind them:
//   next half starts a step:   A0 B0 B1 B2 B3 A1 A2 A3 of that step, read r behind MFMA r, the order in
//                              which the MFMAs first need them;
//   next half is a second half: its A fragments 4..7, read r behind MFMA 4 r + 1 (B stays).
// Every fragment is requested fifteen or more MFMAs before its first use.  Every read is an assembly
// statement and so is every wait: the LDS returns in order, so "all but the newest N LDS instructions have
// returned" is exactly "the fragments MFMA q needs are in their registers", with N counted here from the
// issue order -- the LDS instructions issued after the later of the two fragments q needs.  Every MFMA
// carries its wait, also where an earlier one already covers its fragments: dropping those nine of sixteen
// measured 0.5-1.5 % slower on the polynomial and K-major launches.  (Left to the
// compiler, every group of MFMAs starts with a wait for all outstanding reads, the last of which was
// issued two MFMAs earlier.)  A K-major B fragment is two transposing reads.
template <int HALVES, int ST, bool QK>
struct FragSched {
  static constexpr int P = HALVES * ST, NM = 16;
  static constexpr bool issues_full(int hp) { return (hp + 1) % HALVES == 0; }
  static constexpr int read_behind(int hp, int q) {
    if (issues_full(hp)) return q < 8 ? q : -1;
    return (q % 4 == 1) ? q / 4 : -1;
  }
  static constexpr int instrs_full(int r) { return (QK && r >= 1 && r <= 4) ? 2 : 1; }
  static constexpr int lds_behind(int hp, int q) {
    const int r = read_behind(hp, q);
    if (r < 0) return 0;
    return issues_full(hp) ? instrs_full(r) : 1;
  }
  // LDS instructions that may still be outstanding when MFMA q of half hp issues
  static constexpr int allowed(int hp, int q) {
    const int i = q / 4, j = q % 4;
    const int prev = (hp + P - 1) % P;
    int need_q = 0;  // MFMA of the half before behind which the later of q's two fragments was requested
    if (hp % HALVES == 0) {
      const int ra = i == 0 ? 0 : 4 + i, rb = 1 + j;
      need_q = ra > rb ? ra : rb;
    } else {
      need_q = 4 * i + 1;  // A fragment 4 + i; the B fragments arrived a half earlier
    }
    int n = 0;
    for (int qq = need_q + 1; qq < NM; ++qq) n += lds_behind(prev, qq);
    for (int qq = 0; qq < q; ++qq) n += lds_behind(hp, qq);
    return n < 15 ? n : 15;  // lgkmcnt is a four-bit field; waiting for more than needed is harmless
  }
};

// Fragment wait: an asm statement that takes the fragments it guards as read-write operands, so that to
// the compiler they are (re)defined here and no use of them can be scheduled ahead of the wait.
template <int N>
__device__ __forceinline__ void frag_wait(bf16x8& a, bf16x8& b) {
  asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(a), "+v"(b) : "n"(N));
}
// 16-byte LDS read at addr + OFF, issued from assembly (the compiler does not know it is in flight: the
// matching frag_wait is what its consumers wait on).
template <int OFF>
__device__ __forceinline__ void lds_read16(bf16x8& dst, uint32_t addr) {
  static_assert(OFF >= 0 && OFF < 65536, "ds offset field");
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(OFF));
}
// K-major fragment: two transposing reads, rows k..k+3 and k+4..k+7 of the tile (HI bytes apart)
template <int OFF, int HI>
__device__ __forceinline__ void lds_read_tr(bf16x8& dst, uint32_t addr) {
  static_assert(OFF >= 0 && OFF + HI < 65536, "ds offset field");
  typedef __attribute__((ext_vector_type(2))) unsigned u32x2;
  typedef __attribute__((ext_vector_type(4))) unsigned u32x4f;
  u32x2 lo, hi;
  asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(lo) : "v"(addr), "n"(OFF));
  asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(hi) : "v"(addr), "n"(OFF + HI));
  const u32x4f v = {lo[0], lo[1], hi[0], hi[1]};
  dst = __builtin_bit_cast(bf16x8, v);
}

// Enumeration of the upper triangle (ti <= tj) of a T x T tile grid in super-blocks of SB x SB
// tiles, so that the ~32 workgroups an XCD runs side by side touch as few distinct operand row
// blocks as possible (their L2 is what feeds the LDS): a diagonal super-block has SB(SB+1)/2
// tiles over only SB row blocks; an off-diagonal one is walked in SB x 4 column groups.
__device__ __forceinline__ void tri_tile(int t, int T, int& ti, int& tj) {
  constexpr int SB = 8;
  const int nb = (T + SB - 1) / SB;
  for (int I = 0; I < nb; ++I) {
    const int r = (T - I * SB) < SB ? (T - I * SB) : SB;  // tile rows in super-row I
    const int diag = r * (r + 1) / 2;
    if (t < diag) {
      // row-major triangle of side r
      int i = 0, rem = t;
      while (rem >= r - i) {
        rem -= r - i;
        ++i;
      }
      ti = I * SB + i;
      tj = I * SB + i + rem;
      return;
    }
    t -= diag;
    for (int J = I + 1; J < nb; ++J) {
      const int c = (T - J * SB) < SB ? (T - J * SB) : SB;
      const int cnt = r * c;
      if (t < cnt) {
        const int per_group = r * 4;
        const int g = t / per_group;
        const int gw = (c - g * 4) < 4 ? (c - g * 4) : 4;  // columns in this group
        const int tg = t - g * per_group;
        ti = I * SB + tg / gw;
        tj = J * SB + g * 4 + tg % gw;
        return;
      }
      t -= cnt;
    }
  }
  ti = tj = 0;  // unreachable for t < T(T+1)/2
}

// Workgroup barrier preceded by the counter waits the software pipeline needs: every LDS read
// this wave issued has returned (the ring slot they read is about to be refilled) and all but the
// newest VM_LEFT direct-to-LDS loads of this wave have landed.  The "memory" clobber keeps the
// compiler from moving LDS accesses across it.
template <int VM_LEFT>
__device__ __forceinline__ void pipeline_barrier() {
  static_assert(VM_LEFT >= 0 && VM_LEFT < 64, "vmcnt range");
  __builtin_amdgcn_sched_barrier(0);
  asm volatile("" ::: "memory");
  // vmcnt = VM_LEFT, lgkmcnt = 0, expcnt unconstrained (gfx9 s_waitcnt encoding).
  __builtin_amdgcn_s_waitcnt((VM_LEFT & 0xF) | ((VM_LEFT >> 4) << 14) | 0x0070);
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
  __builtin_amdgcn_sched_barrier(0);
}

typedef __attribute__((ext_vector_type(4))) short s16x4;

// A pointer every lane holds the same value of, moved to scalar registers (where the compiler cannot
// prove uniformity it wraps each buffer access in a loop over the distinct values).
template <typename T>
__device__ __forceinline__ T* uniform_ptr(T* p) {
  const uint64_t v = (uint64_t)p;
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
  const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
  return (T*)(((uint64_t)hi << 32) | lo);
}

// Parameter accesses of the fused update go through buffer instructions: a descriptor based at the
// wavefront's tile of X (wave-uniform, scalar registers), a wave-uniform byte offset per instruction
// (scalar) and one per-lane byte offset shared by all accesses -- no 64-bit address per row in vector
// registers.  Offsets are 32-bit: the launcher checks that a wavefront tile spans less than 2 GiB.
typedef __attribute__((ext_vector_type(4))) unsigned bx_u32x4;
template <typename T>
__device__ __forceinline__ __amdgpu_buffer_rsrc_t bx_resource(T* base) {
  return __builtin_amdgcn_make_buffer_rsrc((void*)base, 0, (int)0xffffffffu, 0x00020000);
}
template <typename T>
__device__ __forceinline__ float bx_load(__amdgpu_buffer_rsrc_t rs, int lane_bytes, int uni_bytes) {
  if constexpr (sizeof(T) == 2)
    return bf16_to_f32((bf16_t)__builtin_amdgcn_raw_buffer_load_b16(rs, lane_bytes, uni_bytes, 0));
  else return __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(rs, lane_bytes, uni_bytes, 0));
}
template <typename T>
__device__ __forceinline__ void bx_store(__amdgpu_buffer_rsrc_t rs, int lane_bytes, int uni_bytes, float v) {
  if constexpr (sizeof(T) == 2)
    __builtin_amdgcn_raw_buffer_store_b16((unsigned short)f32_to_bf16(v), rs, lane_bytes, uni_bytes, 0);
  else __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(v), rs, lane_bytes, uni_bytes, 0);
}
// 16 bytes per lane: eight bf16 or four fp32 elements
template <typename T>
__device__ __forceinline__ void bx_load16(__amdgpu_buffer_rsrc_t rs, int lane_bytes, int uni_bytes, float* v) {
  const bx_u32x4 w = __builtin_amdgcn_raw_buffer_load_b128(rs, lane_bytes, uni_bytes, 0);
  if constexpr (sizeof(T) == 2) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      v[2 * e] = __uint_as_float(w[e] << 16);
      v[2 * e + 1] = __uint_as_float(w[e] & 0xffff0000u);
    }
  } else {
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] = __uint_as_float(w[e]);
  }
}
template <typename T>
__device__ __forceinline__ void bx_store16(__amdgpu_buffer_rsrc_t rs, int lane_bytes, int uni_bytes,
                                           const float* v) {
  bx_u32x4 o;
  if constexpr (sizeof(T) == 2) {
#pragma unroll
    for (int e = 0; e < 4; ++e) o[e] = pack_bf16x2(v[2 * e], v[2 * e + 1]);
  } else {
#pragma unroll
    for (int e = 0; e < 4; ++e) o[e] = __float_as_uint(v[e]);
  }
  __builtin_amdgcn_raw_buffer_store_b128(o, rs, lane_bytes, uni_bytes, 0);
}

// POST: 0 stores the product; 1 / 2 feed it to the fused Muon update of fp32 / bf16 parameters
// (HAS_C then means "update X[row][col]", HAS_CT "update X[col][row]"; nothing else is stored).
template <int POST>
struct PostSel {
  typedef NoPost arg;
  typedef float xt;
};
template <>
struct PostSel<1> {
  typedef FusedPost arg;
  typedef float xt;
};
template <>
struct PostSel<2> {
  typedef FusedPost arg;
  typedef bf16_t xt;
};

template <class Cfg, bool HAS_D, bool HAS_C, bool HAS_CT, bool QK = false, int POST = 0>
__global__ __launch_bounds__(Cfg::NT) void gemm_nt_kernel(const GemmParams p, const typename PostSel<POST>::arg post) {
  constexpr int BM = Cfg::BM, BN = Cfg::BN, BK = Cfg::BK;
  constexpr int TM = Cfg::TM, TN = Cfg::TN, ST = Cfg::ST, HALVES = Cfg::HALVES, NSTAGE = Cfg::NSTAGE;
  constexpr int HP = HALVES * ST;  // halves (sixteen MFMAs each) per slab
  constexpr int NM = 16;
  constexpr int LPS = Cfg::LOADS_PER_STAGE;
  static_assert(LPS <= NM / 2, "one refill load behind every second MFMA of a slab's last half");
  // Refill of the slot a slab occupied: all of it during the slab's last half, or -- the plain product of two
  // K-contiguous operands on 256-wide tiles, i.e. X X^T -- half then and half during the next slab's first half.
  // Measured: X X^T 2-3 % faster that way; the polynomial GEMM (addend loads in the epilogue) 1 % slower, the
  // K-major form (two-instruction fragment reads in the same half) 3 % slower, 128-wide tiles 10 % slower.
  constexpr bool SPREAD = !QK && !HAS_D && BM == 256;
  extern __shared__ __attribute__((aligned(1024))) char lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / Cfg::WN, wn = wave % Cfg::WN;

  // ---- workgroup -> (batch, tile) map.  Hardware deals workgroups round-robin over the 8 XCDs;
  // give each XCD (own L2) one contiguous run of the tile list so neighbours share operands.
  const int tilesM = p.M / BM, tilesN = p.N / BN;
  const int tiles_per_mat = p.tri ? (tilesM * (tilesM + 1)) / 2 : tilesM * tilesN;
  const int total = gridDim.x;
  int lt;
  {
    const int pid = blockIdx.x;
    if (p.xcd_interleave && pid < (total & ~255)) {
      // 256 consecutive workgroups = 32 per XCD: each XCD takes 32 consecutive tiles of the same 256-tile
      // stretch, so the 8 XCDs work on neighbouring tile groups (same matrix, same operand row panels)
      // at the same time, and what one of them fetches from memory the others find in the memory-side
      // cache.  Pays when a matrix's operands are much larger than an XCD's L2.
      const int j = pid & 255;
      lt = (pid & ~255) + (j & 7) * 32 + (j >> 3);
    } else if (p.xcd_interleave) {
      lt = pid;
    } else {
      // one contiguous run of the tile list per XCD: a small matrix stays in one L2
      const int xcd = pid & 7, loc = pid >> 3;
      const int q = total >> 3, r = total & 7;
      lt = xcd * q + (xcd < r ? xcd : r) + loc;
    }
  }
  const int b = lt / tiles_per_mat;
  const int t = lt - b * tiles_per_mat;
  int ti, tj;
  if (p.tri) {
    tri_tile(t, tilesM, ti, tj);
  } else {
    constexpr int GM = 8;
    const int per_group = GM * tilesN;
    const int g = t / per_group;
    const int first = g * GM;
    const int gsz = (tilesM - first) < GM ? (tilesM - first) : GM;
    const int tg = t - g * per_group;
    ti = first + tg % gsz;
    tj = tg / gsz;
  }

  // ---- global -> LDS addressing.  Chunk q = j*NT + tid of a tile lands at LDS byte q*16; it holds
  // logical 16-byte chunk (q % CPR) ^ swz(row) of tile row q / CPR.
  const int ld_row = tid / Cfg::CPR;
  const int ld_phys = tid % Cfg::CPR;
  const int ld_chunk = ld_phys ^ ((ld_row / Cfg::SWZ_DIV) % Cfg::CPR);
  const char* gP = (const char*)(p.P + (int64_t)b * p.strideP + (int64_t)(ti * BM) * p.ldp);
  // QK: the Q tile is BK rows (reduction index) of BN bf16; chunk q lands at LDS byte q*16 and holds
  // logical chunk ((c >> 2) ^ (row & 3)) << 2 | ((c & 3) ^ 2 * ((row >> 3) & 1)), c = q % QCPR, of tile row
  // q / QCPR: the four rows one transposing read gathers land in four distinct 64-byte bank groups, and
  // the rows 8 apart that neighbouring 16-lane groups read in the two 32-byte halves of a group.
  constexpr int QCPR = BN / 8;               // 16-byte chunks per K-major tile row
  constexpr int QROWS_PER_LOAD = Cfg::NT / QCPR;
  static_assert(!QK || (BK % QROWS_PER_LOAD == 0 && QROWS_PER_LOAD % 16 == 0), "K-major tile/threads");
  const int qk_row = tid / QCPR;
  const int qk_chunk = ((((tid % QCPR) >> 2) ^ (qk_row & 3)) << 2) | ((tid & 3) ^ (((qk_row >> 3) & 1) << 1));
  const char* gQ = QK ? (const char*)(p.Q + (int64_t)b * p.strideQ + tj * BN)
                      : (const char*)(p.Q + (int64_t)b * p.strideQ + (int64_t)(tj * BN) * p.ldq);
  uint32_t offP = (uint32_t)(ld_row * p.ldp + ld_chunk * 8) * 2u;
  uint32_t offQ = QK ? (uint32_t)(qk_row * p.ldq + qk_chunk * 8) * 2u
                           : (uint32_t)(ld_row * p.ldq + ld_chunk * 8) * 2u;
  const uint32_t stepP = (uint32_t)(Cfg::ROWS_PER_LOAD * p.ldp) * 2u;
  const uint32_t stepQ = (uint32_t)((QK ? QROWS_PER_LOAD : Cfg::ROWS_PER_LOAD) * p.ldq) * 2u;
  const int64_t slabQ = QK ? (int64_t)BK * p.ldq * 2 : (int64_t)BK * 2;  // bytes between k-slabs of Q
  const int KT = p.K / BK;

  // One direct-to-LDS load (index j of the LPS that make up a stage) of k-slab kt into ring
  // slot buf.  kt past the end re-fetches the last slab (never read): the refill count per stage
  // stays fixed, which is what the vmcnt bookkeeping in pipeline_barrier relies on.
  // A diagonal tile of a symmetric product of one matrix with itself (A = X X^T, A A) needs one operand
  // tile, not two: Q's loads are skipped and its fragments are read from P's half of the slot.  (With a
  // two-slot ring the barrier waits for every outstanding load, so the load count per slab is free to vary.)
  const bool one_operand = !QK && p.tri && ti == tj && p.P == p.Q && p.ldp == p.ldq && p.strideP == p.strideQ;
  // LDS layout of the ring: [P slot 0][P slot 1][Q slot 0][Q slot 1].  With the two slots of an operand
  // side by side, slot, wavefront-tile row block and k step all fit the offset field of the LDS read
  // instructions: the per-lane address registers below are all the address arithmetic the loop needs.
  static_assert(Cfg::P_BYTES == Cfg::Q_BYTES, "square tiles: a one-operand tile reads Q's fragments from P's slots");
  auto issue_load = [&](int kt, int buf, int j) {
    if (one_operand && j >= Cfg::P_LOADS) return;
    const int k = kt < KT ? kt : KT - 1;
    char* l = lds + buf * Cfg::P_BYTES + wave * (64 * 16);
    // Address = wave-uniform 64-bit base (scalar registers; slab and load index folded in) + one 32-bit
    // per-lane offset per operand.  The empty asm (re)defines both right at the load, so that the
    // instruction is selected in its scalar-base form: left to the compiler, base and offset are
    // folded and hoisted out of the loop as a 64-bit address in vector registers per load.
    if (j < Cfg::P_LOADS) {
      const char* src = gP + (int64_t)k * (BK * 2) + (uint64_t)j * stepP;
      asm volatile("" : "+s"(src), "+v"(offP));
      __builtin_amdgcn_global_load_lds(GLB_PTR(src + offP), LDS_PTR(l + j * (Cfg::NT * 16)), 16, 0, 0);
    } else {
      const int jq = j - Cfg::P_LOADS;
      const char* src = gQ + k * slabQ + (uint64_t)jq * stepQ;
      asm volatile("" : "+s"(src), "+v"(offQ));
      __builtin_amdgcn_global_load_lds(GLB_PTR(src + offQ), LDS_PTR(l + NSTAGE * Cfg::P_BYTES + jq * (Cfg::NT * 16)),
                                       16, 0, 0);
    }
  };

  // ---- LDS -> register fragment addressing.  A fragment of v_mfma_f32_16x16x32_bf16: lane l holds row (or
  // column) l % 16 and the eight reduction indices 8 * (l / 16) .. + 7 of a 32-deep step -- one 16-byte chunk.
  const uint32_t lds_base = (uint32_t)(size_t)(__attribute__((address_space(3))) char*)lds;
  const int l16 = lane & 15, quad = lane >> 4;
  const int fswz = (l16 / Cfg::SWZ_DIV) % Cfg::CPR;  // (every fragment's first row is a multiple of 16)
  uint32_t aoff[ST], boff[ST];
#pragma unroll
  for (int st = 0; st < ST; ++st) {
    const int chunk = ((st * 4 + quad) ^ fswz) * 16;
    aoff[st] = lds_base + (uint32_t)((wm * Cfg::WTM + l16) * (BK * 2) + chunk);
    boff[st] = lds_base + (uint32_t)((one_operand ? 0 : NSTAGE * Cfg::P_BYTES) + (wn * Cfg::WTN + l16) * (BK * 2) + chunk);
  }

  // QK fragments: a transposing read hands each 16-lane group a 4 (reduction index) x 16 (column) block, lane i
  // its column i; within the group, lane 4r+q addresses row r / 4-element piece q of the block.  Group g takes
  // reduction indices 8 g .. 8 g + 7 of the step (two reads of 4 rows); the 16 columns of fragment j are half
  // of a 64-byte group of the tile row; the swizzle keys the group on the row's index modulo 4 and the half
  // on bit 3 of the row (= g & 1), so the 32 lanes served together cover all 64 banks once.
  uint32_t qoff[TN];
  if (QK) {
    const int t16 = lane & 15;
#pragma unroll
    for (int j = 0; j < TN; ++j)
      qoff[j] = lds_base + (uint32_t)(NSTAGE * Cfg::P_BYTES + (8 * quad + (t16 >> 2)) * (BN * 2) +
                                      ((((wn * Cfg::WTN + j * 16) >> 5) ^ (t16 >> 2)) << 6) + ((j ^ quad) & 1) * 32 +
                                      (t16 & 3) * 8);
  }

  typedef FragSched<HALVES, ST, QK> FS;
  // A fragments: two sets of four, alternating by half; B fragments: two sets of TN, alternating by step
  bf16x8 fa[2][4], fb[2][TN];
  // Read r of the fragments half hn (0..HP-1) of ring slot buf needs: the first half of a step takes
  // A0 B0 B1 B2 B3 A1 A2 A3 (r = 0..7), a second half its A fragments 4..7 (r = 0..3).  All compile-time
  // constants, which end up in the instruction's offset field.
  auto read_frag = [&](auto bufc, auto hnc, auto rc) {
    constexpr int buf = decltype(bufc)::value, hn = decltype(hnc)::value, r = decltype(rc)::value;
    constexpr int st = hn / HALVES, part = hn % HALVES, fs = hn & 1, bs = st & 1;
    if constexpr (part != 0) {
      lds_read16<buf * Cfg::P_BYTES + (4 + r) * (16 * BK * 2)>(fa[fs][r], aoff[st]);
    } else if constexpr (r == 0 || r > 4) {
      constexpr int i = r == 0 ? 0 : r - 4;
      lds_read16<buf * Cfg::P_BYTES + i * (16 * BK * 2)>(fa[fs][i], aoff[st]);
    } else if constexpr (QK) {
      constexpr int j = r - 1;
      lds_read_tr<buf * Cfg::Q_BYTES + st * (32 * BN * 2), 4 * BN * 2>(fb[bs][j], qoff[j]);
    } else {
      constexpr int j = r - 1;
      lds_read16<buf * Cfg::Q_BYTES + j * (16 * BK * 2)>(fb[bs][j], boff[st]);
    }
  };
  typedef std::integral_constant<int, 0> ic0;

  f32x4 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

  // ---- prologue: fill NSTAGE-1 ring slots, wait for slab 0, read its first fragments, start the
  // last free slot.
#pragma unroll
  for (int s = 0; s < NSTAGE - 1; ++s)
#pragma unroll
    for (int j = 0; j < LPS; ++j) issue_load(s, s, j);
  pipeline_barrier<(NSTAGE - 2) * LPS>();
  static_for<0, 8>([&](auto rc) { read_frag(ic0(), ic0(), rc); });
#pragma unroll
  for (int j = 0; j < (SPREAD ? LPS / 2 : LPS); ++j) issue_load(NSTAGE - 1, NSTAGE - 1, j);
  __builtin_amdgcn_sched_barrier(0);

  // ---- main loop.  Halves run back to back across slab boundaries: while the MFMAs of one half issue, the
  // fragment reads of the next half (and, from the last half of a slab on, the refill of the slot that slab
  // occupied) are slotted behind them.  sched_barrier pins that order.  KT is a multiple of NSTAGE
  // (launcher checks) so ring slots are compile-time constants.
  for (int kt0 = 0; kt0 < KT; kt0 += NSTAGE) {
    static_for<0, NSTAGE * HP>([&](auto shc) {
      constexpr int s = decltype(shc)::value / HP, hp = decltype(shc)::value % HP;
      constexpr int st = hp / HALVES, part = hp % HALVES, fs = hp & 1, bs = st & 1;
      constexpr bool last = (hp == HP - 1);
      // slab kt+1 landed, slab kt fully read
      if constexpr (last) pipeline_barrier<(NSTAGE - 2) * LPS>();
      static_for<0, NM>([&](auto qc) {
        constexpr int q = decltype(qc)::value, i = q / 4, j = q % 4;
        frag_wait<FS::allowed(hp, q)>(fa[fs][i], fb[bs][j]);
        acc[part * 4 + i][j] =
            __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa[fs][i], fb[bs][j], acc[part * 4 + i][j], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (FS::read_behind(hp, q) >= 0) {
          typedef std::integral_constant<int, FS::read_behind(hp, q)> rc;
          if constexpr (last) read_frag(std::integral_constant<int, (s + 1) % NSTAGE>(), ic0(), rc());
          else read_frag(std::integral_constant<int, s>(), std::integral_constant<int, hp + 1>(), rc());
        }
        if constexpr (SPREAD) {
          if constexpr (last && q % 4 == 3 && q / 4 < LPS / 2) issue_load(kt0 + s + NSTAGE, s, q / 4);
          if constexpr (hp == 0 && q % 4 == 3 && LPS / 2 + q / 4 < LPS)
            issue_load(kt0 + s - 1 + NSTAGE, (s + NSTAGE - 1) % NSTAGE, LPS / 2 + q / 4);
        } else {
          if constexpr (last && (q & 1) && q / 2 < LPS) issue_load(kt0 + s + NSTAGE, s, q / 2);
        }
        __builtin_amdgcn_sched_barrier(0);
      });
    });
  }
  wait_vmcnt<0>();  // drain the redundant tail refills before LDS is reused / the wave exits
  // The read-ahead of the last half issued reads whose results nobody uses.  The compiler does not know
  // they are in flight; were their destination registers dead here, it would hand them to whatever comes
  // next (the lane index, store addresses) and a read landing late would overwrite that.  So: wait for the
  // LDS queue to drain, and only then let go of the fragment registers -- the empty asm statements below
  // are their last use and sit behind the wait.
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
  for (int f = 0; f < 2; ++f) {
#pragma unroll
    for (int i = 0; i < 4; ++i) asm volatile("" ::"v"(fa[f][i]));
#pragma unroll
    for (int j = 0; j < TN; ++j) asm volatile("" ::"v"(fb[f][j]));
  }

  // ---- epilogue.  Accumulator element e of lane l holds row 4 * (l / 16) + e, column l % 16 of its 16 x 16
  // tile.  Whole tiles are stored: destinations are padded to the tile.  C goes out straight from registers
  // (16 lanes x 2 B = one 32-byte run per row and instruction, neighbouring tiles completing the lines).
  // The transposed copy would be 8-byte pieces scattered over 16 rows per instruction, so it is staged
  // through LDS ([column][row], this wavefront's private slice) and stored as 16 bytes per lane with
  // 256-byte runs per row.
  const float alpha = gemm_alpha(p, b), beta = p.beta;
  const int row_base = ti * BM + wm * Cfg::WTM;
  const int col_base = tj * BN + wn * Cfg::WTN;
  const bool mirror = HAS_CT && !(p.tri && ti == tj);  // a diagonal tile is its own mirror
  const bf16_t* Dp = HAS_D ? p.D + (int64_t)b * p.strideD + (int64_t)(row_base + 4 * quad) * p.ldd +
                                 col_base + l16
                           : nullptr;
  bf16_t* Cp = (HAS_C && POST == 0) ? p.C + (int64_t)b * p.strideC +
                                           (int64_t)(row_base + 4 * quad) * p.ldc + col_base + l16
                                     : nullptr;
  const int ldd = p.ldd, ldc = p.ldc, ldct = p.ldct;
  typedef typename PostSel<POST>::xt XT;
  float pa = 0.f, pcoeff = 0.f, pb = 0.f;
  int pcautious = 0, pvec = 0;
  XT* xmat = nullptr;
  if constexpr (POST != 0) {
    const float lr = *post.lr_dev;
    const float wd = post.wd_dev ? *post.wd_dev : post.wd_host;
    muon_post_coeffs(lr, wd, post.adj_ratio, pa, pcoeff, pb);
    pcautious = post.cautious;
    pvec = post.vec_ok;
    const int pi = b / post.mats_per_ptr;
    xmat = (XT*)post.X.p[pi] + (int64_t)(b - pi * post.mats_per_ptr) * (HAS_C ? p.strideC : p.strideCt);
  }
  char* stg = lds + wave * Cfg::STG_BYTES;
  const bool on_diag = p.tri && ti == tj && p.diag != 0.0f;
  if (HAS_CT) __syncthreads();  // every wavefront is done with the operand ring

  if constexpr (POST != 0 && HAS_C) {
    // Update X[row][col] from registers.  The products are rounded to bf16 first, two per register,
    // which frees half of the accumulator registers: the parameter values of half a wavefront tile
    // are then loaded in one go (one round trip to memory per half, not one per tile).
    // 16 lanes x one element: a 64-byte (fp32) or 32-byte (bf16) run of X per row.
    uint32_t pk[TM][TN][2];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int q = 0; q < 2; ++q)
          pk[i][j][q] = pack_bf16x2(alpha * acc[i][j][2 * q], alpha * acc[i][j][2 * q + 1]);
    const __amdgpu_buffer_rsrc_t xr = bx_resource(uniform_ptr(xmat + (int64_t)row_base * ldc + col_base));
    const int xl = (4 * quad * ldc + l16) * (int)sizeof(XT);  // per lane
    constexpr int HM = TM / 2;
    auto run = [&](auto caut) {
      constexpr int CAUT = decltype(caut)::value;
#pragma unroll
      for (int i0 = 0; i0 < TM; i0 += HM) {
        float xv[HM][TN][4];
#pragma unroll
        for (int ii = 0; ii < HM; ++ii)
#pragma unroll
          for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int e = 0; e < 4; ++e)
              xv[ii][j][e] = bx_load<XT>(xr, xl, (((i0 + ii) * 16 + e) * ldc + j * 16) * (int)sizeof(XT));
#pragma unroll
        for (int ii = 0; ii < HM; ++ii)
#pragma unroll
          for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const uint32_t w = pk[i0 + ii][j][e >> 1];
              const float u = __uint_as_float((e & 1) ? (w & 0xffff0000u) : (w << 16));
              bx_store<XT>(xr, xl, (((i0 + ii) * 16 + e) * ldc + j * 16) * (int)sizeof(XT),
                           muon_post_one(xv[ii][j][e], u, pa, pcoeff, pb, CAUT));
            }
        asm volatile("" ::: "memory");  // the next batch of loads stays behind these stores
      }
    };
    if (pcautious) run(std::integral_constant<int, 1>());
    else run(std::integral_constant<int, 0>());
    return;
  }

  // The addend is loaded one row of tiles (TN tiles) at a time, one row ahead: the loads of a row are issued
  // before the stores of the row before it, so they neither wait for those stores (the memory counter retires
  // in order) nor cost a round trip to memory per tile.
  bf16_t dreg[HAS_D ? 2 : 1][TN][4];
  auto load_addend = [&](int i) {
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int e = 0; e < 4; ++e) dreg[i & 1][j][e] = Dp[(int64_t)(i * 16 + e) * ldd + j * 16];
  };
  if (HAS_D) load_addend(0);

#pragma unroll
  for (int i = 0; i < TM; ++i) {
    if (HAS_D && i + 1 < TM) load_addend(i + 1);
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      float v[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = alpha * acc[i][j][e];
      if (HAS_D) {
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] += beta * bf16_to_f32(dreg[i & 1][j][e]);
      }
      if (on_diag) {
        // element (row, col) of this tile sits on the global diagonal
        const int dcol = col_base + j * 16 + l16 - (row_base + i * 16 + 4 * quad);
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (dcol == e) v[e] += p.diag;
      }
      if (HAS_C && POST == 0) {
#pragma unroll
        for (int e = 0; e < 4; ++e) Cp[(int64_t)(i * 16 + e) * ldc + j * 16] = f32_to_bf16(v[e]);
      }
      if (HAS_CT) {
        // four consecutive rows of column j * 16 + l16: 8 bytes of the staged [column][row] tile
        uint2 pk;
        pk.x = pack_bf16x2(v[0], v[1]);
        pk.y = pack_bf16x2(v[2], v[3]);
        *(uint2*)(stg + (j * 16 + l16) * Cfg::STG_PITCH + (i * 16 + 4 * quad) * 2) = pk;
      }
    }
  }
  if (HAS_CT) {
    if (mirror) {
      constexpr int CH = Cfg::WTM / 8;  // 16-byte chunks per staged row
      constexpr int RPI = 64 / CH;      // staged rows per store instruction
      const int srow = lane / CH, schunk = lane % CH;
      const char* sp = stg + srow * Cfg::STG_PITCH + schunk * 16;
      if constexpr (POST != 0) {
        // The staged bf16 tile is the update.  One 16-byte access of X per lane and step (4 fp32 or 8 bf16
        // elements), lanes side by side along the row: every instruction covers whole contiguous runs.
        constexpr int EPL = 16 / (int)sizeof(XT);   // elements per lane
        constexpr int PCH = Cfg::WTM / EPL;          // lanes per staged row
        constexpr int PRPI = 64 / PCH;               // staged rows per instruction
        constexpr int NIT = Cfg::WTN / PRPI;
        constexpr int BI = NIT < (EPL == 4 ? 16 : 8) ? NIT : (EPL == 4 ? 16 : 8);
        static_assert(64 % PCH == 0 && Cfg::WTN % PRPI == 0 && NIT % BI == 0, "staged rows per wavefront");
        const int prow = lane / PCH, pchunk = lane % PCH;
        const char* pp = stg + prow * Cfg::STG_PITCH + pchunk * (EPL * 2);
        const __amdgpu_buffer_rsrc_t xr = bx_resource(uniform_ptr(xmat + (int64_t)col_base * ldct + row_base));
        const int xl = (prow * ldct + pchunk * EPL) * (int)sizeof(XT);  // per lane
        auto run = [&](auto caut) {
          constexpr int CAUT = decltype(caut)::value;
#pragma unroll
          for (int it0 = 0; it0 < NIT; it0 += BI) {
            float uv[BI][EPL], xv[BI][EPL];
#pragma unroll
            for (int k = 0; k < BI; ++k) {
              const char* q = pp + (it0 + k) * PRPI * Cfg::STG_PITCH;
              if constexpr (EPL == 8) st_load8<bf16_t>((const bf16_t*)q, 0, uv[k]);
              else st_load4<bf16_t>((const bf16_t*)q, 0, uv[k]);
            }
            if (pvec) {
#pragma unroll
              for (int k = 0; k < BI; ++k)
                bx_load16<XT>(xr, xl, (it0 + k) * PRPI * ldct * (int)sizeof(XT), xv[k]);
            } else {
#pragma unroll
              for (int k = 0; k < BI; ++k)
#pragma unroll
                for (int e = 0; e < EPL; ++e)
                  xv[k][e] = bx_load<XT>(xr, xl, ((it0 + k) * PRPI * ldct + e) * (int)sizeof(XT));
            }
#pragma unroll
            for (int k = 0; k < BI; ++k)
#pragma unroll
              for (int e = 0; e < EPL; ++e) xv[k][e] = muon_post_one(xv[k][e], uv[k][e], pa, pcoeff, pb, CAUT);
            if (pvec) {
#pragma unroll
              for (int k = 0; k < BI; ++k)
                bx_store16<XT>(xr, xl, (it0 + k) * PRPI * ldct * (int)sizeof(XT), xv[k]);
            } else {
#pragma unroll
              for (int k = 0; k < BI; ++k)
#pragma unroll
                for (int e = 0; e < EPL; ++e)
                  bx_store<XT>(xr, xl, ((it0 + k) * PRPI * ldct + e) * (int)sizeof(XT), xv[k][e]);
            }
          }
        };
        if (pcautious) run(std::integral_constant<int, 1>());
        else run(std::integral_constant<int, 0>());
      } else {
        bf16_t* Ctp =
            p.Ct + (int64_t)b * p.strideCt + (int64_t)(col_base + srow) * ldct + row_base + schunk * 8;
#pragma unroll 8
        for (int it = 0; it < Cfg::WTN / RPI; ++it) {
          const uint4 q = *(const uint4*)(sp + it * RPI * Cfg::STG_PITCH);
          *(uint4*)(Ctp + (int64_t)(it * RPI) * ldct) = q;
        }
      }
    }
  }
}

// ---------------------------------------------------------------------------------------------
// X' = P Q with Q stored [K][N] (the dominant launch of the iteration), one workgroup per CU walking a
// list of output tiles.  What the one-tile-per-workgroup kernel above pays at every tile boundary --
// the store acknowledgements a wavefront waits for before it may end, the dispatch of the next
// workgroup, and the latency of its first operand loads, together 5-8 us per 256x256 tile with the
// MFMA pipes idle -- is overlapped here:
//   * the operand ring runs on across tiles: the refills issued during the last two slabs of a tile
//     fetch the first two slabs of the workgroup's next tile, so the next tile's first MFMAs issue right
//     after this tile's epilogue;
//   * the epilogue goes through a private 4 KB LDS slice per wavefront next to the ring (not over
//     it: the ring is already receiving the next tile) and leaves as sixteen 16-byte stores per
//     lane, each instruction writing whole 128-byte lines.  Sixteen outstanding stores also stay countable
//     next to the ring's loads (the wait counter has six bits), and their acknowledgements come back
//     under the next tile's first slab.
// OUT_T false stores C[row][col]: the MFMA operands are swapped, so that a lane's four accumulator
// elements are four consecutive columns of one output row (8 bytes of a C row).
// OUT_T true stores Ct[col][row] (the product of a tall input, kept in the wide layout): operands
// in the usual order, the four elements are four consecutive rows = 8 bytes of a Ct row.
// Either way a staged chunk is 32 lines x 128 bytes from eight 16x16 accumulator tiles.
template <class Cfg, bool OUT_T>
__global__ __launch_bounds__(Cfg::NT) void gemm_qk_walk_kernel(const GemmParams p, const int total_tiles) {
  constexpr int BM = Cfg::BM, BN = Cfg::BN, BK = Cfg::BK;
  constexpr int TM = Cfg::TM, TN = Cfg::TN, ST = Cfg::ST, HALVES = Cfg::HALVES, NSTAGE = Cfg::NSTAGE;
  constexpr int HP = HALVES * ST, NM = 16, LPS = Cfg::LOADS_PER_STAGE;
  static_assert(NSTAGE == 2 && TM == 8 && TN == 4 && LPS <= NM / 2, "written for 128x64 wavefront tiles, two-slot ring");
  constexpr int STG_WAVE = 32 * 128;  // staging bytes per wavefront: 32 lines of 128 bytes
  extern __shared__ __attribute__((aligned(1024))) char lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / Cfg::WN, wn = wave % Cfg::WN;
  const int tilesM = p.M / BM, tilesN = p.N / BN;
  const int tiles_per_mat = tilesM * tilesN;
  const int KT = p.K / BK;

  // Tile number `pid` of the launch -> (batch, tile row, tile column): the same map as the kernel above
  // uses for its workgroup index, so consecutive workgroups (= XCDs) share operand panels the same way.
  auto tile_of = [&](int pid, int& b, int& ti, int& tj) {
    int lt;
    if (p.xcd_interleave && pid < (total_tiles & ~255)) {
      const int j = pid & 255;
      lt = (pid & ~255) + (j & 7) * 32 + (j >> 3);
    } else if (p.xcd_interleave) {
      lt = pid;
    } else {
      const int xcd = pid & 7, loc = pid >> 3;
      const int q = total_tiles >> 3, r = total_tiles & 7;
      lt = xcd * q + (xcd < r ? xcd : r) + loc;
    }
    b = lt / tiles_per_mat;
    const int t = lt - b * tiles_per_mat;
    constexpr int GM = 8;
    const int per_group = GM * tilesN;
    const int g = t / per_group;
    const int first = g * GM;
    const int gsz = (tilesM - first) < GM ? (tilesM - first) : GM;
    const int tg = t - g * per_group;
    ti = first + tg % gsz;
    tj = tg / gsz;
  };

  // ---- global -> LDS addressing (see the kernel above): per-lane offsets are the same for every tile,
  // the tile only moves the wave-uniform base pointers.
  const int ld_row = tid / Cfg::CPR;
  const int ld_phys = tid % Cfg::CPR;
  const int ld_chunk = ld_phys ^ ((ld_row / Cfg::SWZ_DIV) % Cfg::CPR);
  constexpr int QCPR = BN / 8;
  constexpr int QROWS_PER_LOAD = Cfg::NT / QCPR;
  static_assert(BK % QROWS_PER_LOAD == 0 && QROWS_PER_LOAD % 16 == 0, "K-major tile/threads");
  const int qk_row = tid / QCPR;
  const int qk_chunk = ((((tid % QCPR) >> 2) ^ (qk_row & 3)) << 2) | ((tid & 3) ^ (((qk_row >> 3) & 1) << 1));
  uint32_t offP = (uint32_t)(ld_row * p.ldp + ld_chunk * 8) * 2u;
  uint32_t offQ = (uint32_t)(qk_row * p.ldq + qk_chunk * 8) * 2u;
  const uint32_t stepP = (uint32_t)(Cfg::ROWS_PER_LOAD * p.ldp) * 2u;
  const uint32_t stepQ = (uint32_t)(QROWS_PER_LOAD * p.ldq) * 2u;
  const int64_t slabQ = (int64_t)BK * p.ldq * 2;

  int b_c, ti_c, tj_c, b_n, ti_n, tj_n;
  int pid = blockIdx.x;
  tile_of(pid, b_c, ti_c, tj_c);
  auto base_p = [&](int b, int ti) { return (const char*)(p.P + (int64_t)b * p.strideP + (int64_t)(ti * BM) * p.ldp); };
  auto base_q = [&](int b, int tj) { return (const char*)(p.Q + (int64_t)b * p.strideQ + tj * BN); };
  const char* gP_c = base_p(b_c, ti_c);
  const char* gQ_c = base_q(b_c, tj_c);
  const char *gP_n = gP_c, *gQ_n = gQ_c;
  auto look_ahead = [&]() {
    // the tile after the current one; past the end of the list the current tile stands in (its slabs are
    // fetched again and never read, which keeps the load count per slab fixed)
    const int np = pid + (int)gridDim.x;
    if (np < total_tiles) {
      tile_of(np, b_n, ti_n, tj_n);
      gP_n = base_p(b_n, ti_n);
      gQ_n = base_q(b_n, tj_n);
    } else {
      b_n = b_c; ti_n = ti_c; tj_n = tj_c;
      gP_n = gP_c; gQ_n = gQ_c;
    }
  };
  look_ahead();

  // slab kt of the current tile, or slab kt - KT of the next one, into ring slot buf (load j of LPS);
  // ring layout [P slot 0][P slot 1][Q slot 0][Q slot 1] as in the kernel above
  auto issue_load = [&](int kt, int buf, int j) {
    const bool nx = kt >= KT;
    const int k = nx ? kt - KT : kt;
    char* l = lds + buf * Cfg::P_BYTES + wave * (64 * 16);
    // wave-uniform base in scalar registers + one per-lane offset per operand (see the kernel above)
    if (j < Cfg::P_LOADS) {
      const char* src = (nx ? gP_n : gP_c) + (int64_t)k * (BK * 2) + (uint64_t)j * stepP;
      asm volatile("" : "+s"(src), "+v"(offP));
      __builtin_amdgcn_global_load_lds(GLB_PTR(src + offP), LDS_PTR(l + j * (Cfg::NT * 16)), 16, 0, 0);
    } else {
      const int jq = j - Cfg::P_LOADS;
      const char* src = (nx ? gQ_n : gQ_c) + k * slabQ + (uint64_t)jq * stepQ;
      asm volatile("" : "+s"(src), "+v"(offQ));
      __builtin_amdgcn_global_load_lds(GLB_PTR(src + offQ), LDS_PTR(l + NSTAGE * Cfg::P_BYTES + jq * (Cfg::NT * 16)), 16, 0, 0);
    }
  };

  // ---- LDS -> register fragments (see the kernel above)
  const uint32_t lds_base = (uint32_t)(size_t)(__attribute__((address_space(3))) char*)lds;
  const int l16 = lane & 15, quad = lane >> 4;
  const int fswz = (l16 / Cfg::SWZ_DIV) % Cfg::CPR;
  uint32_t aoff[ST];
#pragma unroll
  for (int st = 0; st < ST; ++st)
    aoff[st] = lds_base + (uint32_t)((wm * Cfg::WTM + l16) * (BK * 2) + ((st * 4 + quad) ^ fswz) * 16);
  uint32_t qoff[TN];
#pragma unroll
  for (int j = 0; j < TN; ++j)
    qoff[j] = lds_base + (uint32_t)(NSTAGE * Cfg::P_BYTES + (8 * quad + (l16 >> 2)) * (BN * 2) +
                                    ((((wn * Cfg::WTN + j * 16) >> 5) ^ (l16 >> 2)) << 6) + ((j ^ quad) & 1) * 32 +
                                    (l16 & 3) * 8);
  typedef FragSched<HALVES, ST, true> FS;
  bf16x8 fa[2][4], fb[2][TN];
  auto read_frag = [&](auto bufc, auto hnc, auto rc) {
    constexpr int buf = decltype(bufc)::value, hn = decltype(hnc)::value, r = decltype(rc)::value;
    constexpr int st = hn / HALVES, part = hn % HALVES, fs = hn & 1, bs = st & 1;
    if constexpr (part != 0) {
      lds_read16<buf * Cfg::P_BYTES + (4 + r) * (16 * BK * 2)>(fa[fs][r], aoff[st]);
    } else if constexpr (r == 0 || r > 4) {
      constexpr int i = r == 0 ? 0 : r - 4;
      lds_read16<buf * Cfg::P_BYTES + i * (16 * BK * 2)>(fa[fs][i], aoff[st]);
    } else {
      constexpr int j = r - 1;
      lds_read_tr<buf * Cfg::Q_BYTES + st * (32 * BN * 2), 4 * BN * 2>(fb[bs][j], qoff[j]);
    }
  };
  typedef std::integral_constant<int, 0> ic0;

  f32x4 acc[TM][TN];
  auto clear_acc = [&]() {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
  };
  clear_acc();

  // ---- epilogue addressing: lane = (line l16 of a tile, 8-byte piece quad) when staging, (line rl, 16-byte
  // piece rq) when storing
  char* stg = lds + Cfg::RING_BYTES + wave * STG_WAVE;
  const int rl = lane >> 3, rq = lane & 7;
  const int ld_out = OUT_T ? p.ldct : p.ldc;

  auto store_tile = [&](int b, int ti, int tj) {
    const int row_base = ti * BM + wm * Cfg::WTM;
    const int col_base = tj * BN + wn * Cfg::WTN;
    bf16_t* out = OUT_T ? p.Ct + (int64_t)b * p.strideCt + (int64_t)col_base * ld_out + row_base
                        : p.C + (int64_t)b * p.strideC + (int64_t)row_base * ld_out + col_base;
    const __amdgpu_buffer_rsrc_t rs = bx_resource(uniform_ptr(out));
    const int lane_bytes = (rl * ld_out + rq * 8) * 2;
    const float alpha = gemm_alpha(p, b);  // 1 unless a per-matrix factor rides on this launch
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      // chunk c: 32 output lines of 128 bytes.  OUT_T false: C rows 32 c .. 32 c + 31 of the wavefront tile
      // (accumulator tiles i = 2 c, 2 c + 1, all j); OUT_T true: Ct lines = C columns 32 (c / 2) .. + 31
      // (j = 2 (c / 2), + 1) by C rows 64 (c % 2) .. + 63 (i = 4 (c % 2) .. + 3).
      const int line0 = OUT_T ? (c >> 1) * 32 : c * 32;   // first output line of the chunk (relative)
      const int run0 = OUT_T ? (c & 1) * 64 : 0;          // first element of the chunk within a line
#pragma unroll
      for (int t = 0; t < 8; ++t) {
        const f32x4& a = OUT_T ? acc[4 * (c & 1) + (t & 3)][2 * (c >> 1) + (t >> 2)] : acc[2 * c + (t >> 2)][t & 3];
        uint2 pk;
        pk.x = pack_bf16x2(alpha * a[0], alpha * a[1]);
        pk.y = pack_bf16x2(alpha * a[2], alpha * a[3]);
        // 8-byte piece 4 (t % 4) + quad of line 16 (t / 4) + l16; XOR with twice the line pair number spreads
        // the 16 lines of half a wavefront over all 64 banks and keeps 16-byte pairs together
        const int line = 16 * (t >> 2) + l16;
        *(uint2*)(stg + line * 128 + (((4 * (t & 3) + quad) ^ (((line >> 1) & 7) << 1)) << 3)) = pk;
      }
      asm volatile("" ::: "memory");
      uint4 v[4];
#pragma unroll
      for (int it = 0; it < 4; ++it) {
        const int line = rl + 8 * it;
        v[it] = *(const uint4*)(stg + line * 128 + (((2 * rq) ^ (((line >> 1) & 7) << 1)) << 3));
      }
      asm volatile("" ::: "memory");
#pragma unroll
      for (int it = 0; it < 4; ++it) {
        const bx_u32x4 o = {v[it].x, v[it].y, v[it].z, v[it].w};
        __builtin_amdgcn_raw_buffer_store_b128(o, rs, lane_bytes, ((line0 + 8 * it) * ld_out + run0) * 2, 0);
      }
    }
  };

  // ---- prologue: slab 0 of the first tile, its first fragments, slab 1
#pragma unroll
  for (int j = 0; j < LPS; ++j) issue_load(0, 0, j);
  pipeline_barrier<0>();
  static_for<0, 8>([&](auto rc) { read_frag(ic0(), ic0(), rc); });
#pragma unroll
  for (int j = 0; j < LPS; ++j) issue_load(1, 1, j);
  __builtin_amdgcn_sched_barrier(0);

  for (;;) {
    // ---- one tile: the main loop of the kernel above; refills past the tile's last slab fetch the next tile
    for (int kt0 = 0; kt0 < KT; kt0 += NSTAGE) {
      static_for<0, NSTAGE * HP>([&](auto shc) {
        constexpr int s = decltype(shc)::value / HP, hp = decltype(shc)::value % HP;
        constexpr int st = hp / HALVES, part = hp % HALVES, fs = hp & 1, bs = st & 1;
        constexpr bool last = (hp == HP - 1);
        if constexpr (last) pipeline_barrier<0>();
        static_for<0, NM>([&](auto qc) {
          constexpr int q = decltype(qc)::value, i = q / 4, j = q % 4;
          frag_wait<FS::allowed(hp, q)>(fa[fs][i], fb[bs][j]);
          if constexpr (OUT_T)
            acc[part * 4 + i][j] =
                __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa[fs][i], fb[bs][j], acc[part * 4 + i][j], 0, 0, 0);
          else
            acc[part * 4 + i][j] =
                __builtin_amdgcn_mfma_f32_16x16x32_bf16(fb[bs][j], fa[fs][i], acc[part * 4 + i][j], 0, 0, 0);
          __builtin_amdgcn_sched_barrier(0);
          if constexpr (FS::read_behind(hp, q) >= 0) {
            typedef std::integral_constant<int, FS::read_behind(hp, q)> rc;
            if constexpr (last) read_frag(std::integral_constant<int, (s + 1) % NSTAGE>(), ic0(), rc());
            else read_frag(std::integral_constant<int, s>(), std::integral_constant<int, hp + 1>(), rc());
          }
          if constexpr (last && (q & 1) && q / 2 < LPS) issue_load(kt0 + s + NSTAGE, s, q / 2);
          __builtin_amdgcn_sched_barrier(0);
        });
      });
    }
    // The first fragments of the next tile are on their way into set 0.  Let them land before the epilogue:
    // its register traffic must not meet a transposing read still in flight.
    asm volatile("s_waitcnt lgkmcnt(0)"
                 : "+v"(fa[0][0]), "+v"(fa[0][1]), "+v"(fa[0][2]), "+v"(fa[0][3]), "+v"(fb[0][0]), "+v"(fb[0][1]),
                   "+v"(fb[0][2]), "+v"(fb[0][3]));
    store_tile(b_c, ti_c, tj_c);
    pid += (int)gridDim.x;
    if (pid >= total_tiles) break;
    clear_acc();
    b_c = b_n; ti_c = ti_n; tj_c = tj_n;
    gP_c = gP_n; gQ_c = gQ_n;
    look_ahead();
    __builtin_amdgcn_sched_barrier(0);
  }
  wait_vmcnt<0>();  // the stand-in refills of the last tile must land before the LDS is given back
}

// ---------------------------------------------------------------------------------------------
typedef TileCfg<128, 128, 64, 2, 2, 2> Cfg128;     // 4 wavefronts, 64x64 each; two workgroups per CU
typedef TileCfg<256, 256, 64, 2, 4, 2> Cfg256w8;   // 8 wavefronts, 128x64 each: two per SIMD, one workgroup per CU
constexpr int kWalkMaxK = 2048;                    // longest reduction the tile-walking kernel is used for

// Tile list dealt to the XCDs in interleaved 32-tile chunks (see the kernel) when the first operand of
// one matrix is at least 16 MB; below that a contiguous run per XCD keeps whole matrices in one L2.
static bool xcd_interleave_pays(const GemmParams& p) { return (int64_t)p.M * p.K * 2 >= (16L << 20); }

template <class Cfg, bool HAS_D, bool HAS_C, bool HAS_CT, bool QK = false, int POST = 0>
static hipError_t launch_epi(const GemmParams& p, hipStream_t stream,
                             const typename PostSel<POST>::arg& post = typename PostSel<POST>::arg()) {
  static std::atomic<uint64_t> attr_done{0};
  auto kern = gemm_nt_kernel<Cfg, HAS_D, HAS_C, HAS_CT, QK, POST>;
  if (hipError_t e = set_max_dynamic_lds_once((const void*)kern, Cfg::LDS_BYTES, attr_done)) return e;
  const int tilesM = p.M / Cfg::BM, tilesN = p.N / Cfg::BN;
  const int64_t per_mat = p.tri ? (int64_t)tilesM * (tilesM + 1) / 2 : (int64_t)tilesM * tilesN;
  const int64_t total = per_mat * p.batch;
  if (total <= 0) return hipSuccess;
  if (total > 0x7fffffff) return hipErrorInvalidValue;
  GemmParams pp = p;
  pp.xcd_interleave = xcd_interleave_pays(p) ? 1 : 0;
  hipLaunchKernelGGL(kern, dim3((unsigned)total), dim3(Cfg::NT), Cfg::LDS_BYTES, stream, pp, post);
  return hipGetLastError();
}

// One workgroup per CU, each walking its share of the tile list.
template <class Cfg, bool OUT_T>
static hipError_t launch_walk(const GemmParams& p, hipStream_t stream) {
  static std::atomic<uint64_t> attr_done{0};
  constexpr int kLds = Cfg::RING_BYTES + Cfg::WM * Cfg::WN * 32 * 128;
  auto kern = gemm_qk_walk_kernel<Cfg, OUT_T>;
  if (hipError_t e = set_max_dynamic_lds_once((const void*)kern, kLds, attr_done)) return e;
  const int64_t total = (int64_t)(p.M / Cfg::BM) * (p.N / Cfg::BN) * p.batch;
  if (total <= 0) return hipSuccess;
  if (total > 0x7fffffff) return hipErrorInvalidValue;
  // a wavefront's output tile is addressed with 32-bit byte offsets from its first element
  if ((int64_t)(OUT_T ? p.ldct : p.ldc) * 129 * 2 > 0x7fffffffLL) return hipErrorInvalidValue;
  static std::atomic<int> cu_count[64];
  int dev = 0;
  if (hipError_t e = hipGetDevice(&dev)) return e;
  int cus = cu_count[dev & 63].load(std::memory_order_relaxed);
  if (cus == 0) {
    if (hipError_t e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev)) return e;
    if (cus <= 0) return hipErrorInvalidValue;
    cu_count[dev & 63].store(cus, std::memory_order_relaxed);
  }
  GemmParams pp = p;
  pp.xcd_interleave = xcd_interleave_pays(p) ? 1 : 0;
  const unsigned grid = (unsigned)(total < cus ? total : cus);
  hipLaunchKernelGGL(kern, dim3(grid), dim3(Cfg::NT), kLds, stream, pp, (int)total);
  return hipGetLastError();
}

// The operand / result combinations the Newton-Schulz drivers use.
template <class Cfg>
static hipError_t launch_cfg(const GemmParams& p, hipStream_t stream) {
  if (p.M % Cfg::BM || p.N % Cfg::BN || p.K % (Cfg::BK * Cfg::NSTAGE)) return hipErrorInvalidValue;
  const bool d = p.D != nullptr, c = p.C != nullptr, ct = p.Ct != nullptr;
  if (p.q_kmajor) {
    if (p.tri) return hipErrorInvalidValue;
    if constexpr (Cfg::BM == 256) {
      // Short reductions go to the tile-walking kernel: what it saves is a fixed cost per tile, 13 % of the
      // launch at 32 slabs and nothing at 64 (where its static tile order costs as much as it saves).
      if (p.K <= kWalkMaxK && p.alpha == 1.0f) {  // (the drivers' X' products are unscaled)
        if (!d && c && !ct) return launch_walk<Cfg, false>(p, stream);  // X' = B X
        if (!d && !c && ct) return launch_walk<Cfg, true>(p, stream);   // (B X)^T only
      }
    }
    if (!d && c && !ct) return launch_epi<Cfg, false, true, false, true>(p, stream);  // X' = B X
    if (!d && !c && ct) return launch_epi<Cfg, false, false, true, true>(p, stream);  // (B X)^T only
    if (d && c && !ct) return launch_epi<Cfg, true, true, false, true>(p, stream);    // a X + B X
    return hipErrorInvalidValue;
  }
  if (p.tri && !d && c && ct) return launch_epi<Cfg, false, true, true>(p, stream);   // A = X X^T, R = T Z
  if (p.tri && d && c && ct) return launch_epi<Cfg, true, true, true>(p, stream);     // B = c A A + b A (+ a I)
  if (!p.tri && !d && c && !ct) return launch_epi<Cfg, false, true, false>(p, stream); // full product of two symmetric matrices
  return hipErrorInvalidValue;
}

int gemm_pad_granule(int m, int n, int batch) {
  // 256-wide tiles need enough of them to fill 256 CUs; small problems use 128-wide tiles.
  const int64_t m256 = (m + 255) / 256;
  const int64_t syrk_tiles = m256 * (m256 + 1) / 2 * batch;
  (void)n;
  return syrk_tiles >= 256 ? 256 : 128;
}

// 256-wide tiles when there are enough of them: a full product from 384 tiles (one and a half rounds of the
// 256 CUs; 432 tiles of 12 x (768 x 3072) run 14 % faster than the 1728 128-wide ones, 108 tiles of
// 12 x (768 x 768) 20 % slower), a symmetric one from 160 (16 x 1024-wide: 5 % faster; 72 tiles of
// 12 x 768-wide: 70 % slower).  Rounds that are not full cost less than their geometry says: the part is
// power-limited, and the CUs that are busy run faster while others idle.  Below the thresholds the 128-wide
// tiles (two workgroups per CU) win.
static bool wants_256_tiles(const GemmParams& p) {
  const long T = p.M / 256;
  const long t256 = (p.tri ? T * (T + 1) / 2 : T * (p.N / 256)) * p.batch;
  return p.M % 256 == 0 && p.N % 256 == 0 && t256 >= (p.tri ? 160L : 384L);
}

int gemm_tile_edge(const GemmParams& p) { return wants_256_tiles(p) ? 256 : 128; }

template <class Cfg>
static hipError_t launch_post_cfg(const GemmParams& p, const FusedPost& post, int x_dtype, bool transposed,
                                  hipStream_t stream) {
  if (p.M % Cfg::BM || p.N % Cfg::BN || p.K % (Cfg::BK * Cfg::NSTAGE)) return hipErrorInvalidValue;
  if (x_dtype == 1) {
    return transposed ? launch_epi<Cfg, false, false, true, true, 1>(p, stream, post)
                      : launch_epi<Cfg, false, true, false, true, 1>(p, stream, post);
  }
  return transposed ? launch_epi<Cfg, false, false, true, true, 2>(p, stream, post)
                    : launch_epi<Cfg, false, true, false, true, 2>(p, stream, post);
}

hipError_t launch_gemm_nt_post(const GemmParams& p, const FusedPost& post, int x_dtype, bool transposed,
                               hipStream_t stream) {
  if (p.M <= 0 || p.N <= 0 || p.K <= 0 || p.batch <= 0) return hipSuccess;
  // the epilogue addresses a wavefront tile of X (at most 128 rows) with 32-bit byte offsets
  if ((int64_t)(transposed ? p.ldct : p.ldc) * 129 * 4 > 0x7fffffffLL) return hipErrorInvalidValue;
  if (!p.q_kmajor || p.tri || p.D || post.mats_per_ptr <= 0 || !post.lr_dev ||
      p.batch > (int64_t)kMaxPtrs * post.mats_per_ptr || (x_dtype != 0 && x_dtype != 1))
    return hipErrorInvalidValue;
  return wants_256_tiles(p) ? launch_post_cfg<Cfg256w8>(p, post, x_dtype, transposed, stream)
                            : launch_post_cfg<Cfg128>(p, post, x_dtype, transposed, stream);
}

hipError_t launch_gemm_nt(const GemmParams& p, hipStream_t stream) {
  if (p.M <= 0 || p.N <= 0 || p.K <= 0 || p.batch <= 0) return hipSuccess;
  if (p.tri && (p.M != p.N)) return hipErrorInvalidValue;
  return wants_256_tiles(p) ? launch_cfg<Cfg256w8>(p, stream) : launch_cfg<Cfg128>(p, stream);
}

}  // namespace dion
