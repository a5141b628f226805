// extern "C" surface of libdion_hip.so (declared in include/dion_hip.h) and the host-side
// Newton-Schulz driver that strings the GEMM launches together.
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <vector>

#include "../../include/dion_hip.h"
#include "elementwise.h"

using namespace dion;

static thread_local char g_err[512] = "";

static int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

static int hip_fail(hipError_t e, const char* what) {
  return fail(DION_E_HIP, "%s: %s", what, hipGetErrorString(e));
}

#define HIP_TRY(expr, what)                     \
  do {                                          \
    hipError_t _e = (expr);                     \
    if (_e != hipSuccess) return hip_fail(_e, what); \
  } while (0)

static inline int round_up(int v, int g) { return (v + g - 1) / g * g; }
static inline size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }
static inline bool aligned16(uint64_t p) { return (p & 15) == 0; }

extern "C" const char* dion_last_error(void) { return g_err; }
extern "C" int dion_abi_version(void) { return 12; }

// ---------------------------------------------------------------------------------------------
// Kernel-level GEMMs
// ---------------------------------------------------------------------------------------------
static int check_gemm_dims(const char* who, int batch, int m, int n) {
  if (batch < 0 || m < 0 || n < 0) return fail(DION_E_INVALID, "%s: negative extent", who);
  if (m % 128 || n % 128)
    return fail(DION_E_INVALID, "%s: extents (%d, %d) must be multiples of 128", who, m, n);
  return DION_OK;
}

// The GEMM kernels move operands with 16-byte direct-to-LDS loads and store 16 bytes per lane.
static int check_gemm_ptr(const char* who, const char* arg, const void* ptr) {
  if (ptr && !aligned16((uint64_t)(uintptr_t)ptr))
    return fail(DION_E_INVALID, "%s: %s is not 16-byte aligned", who, arg);
  return DION_OK;
}

extern "C" int dion_ns_line_1(const void* X, void* A, int batch, int m, int k, void* stream) {
  if (int rc = check_gemm_dims("dion_ns_line_1", batch, m, k)) return rc;
  if (batch == 0 || m == 0) return DION_OK;
  if (k == 0) return fail(DION_E_INVALID, "dion_ns_line_1: k == 0");
  if (!X || !A) return fail(DION_E_INVALID, "dion_ns_line_1: null argument");
  if (int rc = check_gemm_ptr("dion_ns_line_1", "X", X)) return rc;
  if (int rc = check_gemm_ptr("dion_ns_line_1", "A", A)) return rc;
  GemmParams p;
  memset(&p, 0, sizeof(p));
  p.P = p.Q = (const bf16_t*)X;
  p.C = p.Ct = (bf16_t*)A;
  p.strideP = p.strideQ = (int64_t)m * k;
  p.strideC = p.strideCt = (int64_t)m * m;
  p.ldp = p.ldq = k;
  p.ldc = p.ldct = m;
  p.M = p.N = m;
  p.K = k;
  p.batch = batch;
  p.tri = 1;
  p.alpha = 1.0f;
  HIP_TRY(launch_gemm_nt(p, (hipStream_t)stream), "dion_ns_line_1");
  return DION_OK;
}

extern "C" int dion_ns_line_2(const void* A, void* B, int batch, int m, float alpha, float beta,
                              void* stream) {
  if (int rc = check_gemm_dims("dion_ns_line_2", batch, m, m)) return rc;
  if (batch == 0 || m == 0) return DION_OK;
  if (!A || !B) return fail(DION_E_INVALID, "dion_ns_line_2: null argument");
  if (A == B) return fail(DION_E_INVALID, "dion_ns_line_2: in-place not supported");
  if (int rc = check_gemm_ptr("dion_ns_line_2", "A", A)) return rc;
  if (int rc = check_gemm_ptr("dion_ns_line_2", "B", B)) return rc;
  GemmParams p;
  memset(&p, 0, sizeof(p));
  p.P = p.Q = p.D = (const bf16_t*)A;
  p.C = p.Ct = (bf16_t*)B;
  p.strideP = p.strideQ = p.strideD = p.strideC = p.strideCt = (int64_t)m * m;
  p.ldp = p.ldq = p.ldd = p.ldc = p.ldct = m;
  p.M = p.N = p.K = m;
  p.batch = batch;
  p.tri = 1;
  p.alpha = alpha;
  p.beta = beta;
  HIP_TRY(launch_gemm_nt(p, (hipStream_t)stream), "dion_ns_line_2");
  return DION_OK;
}

extern "C" int dion_ns_line_3(const void* B, const void* X, void* C, int batch, int m, int n, float a,
                              void* stream) {
  if (int rc = check_gemm_dims("dion_ns_line_3", batch, m, n)) return rc;
  if (batch == 0 || m == 0 || n == 0) return DION_OK;
  if (!B || !X || !C) return fail(DION_E_INVALID, "dion_ns_line_3: null argument");
  if (C == X) return fail(DION_E_INVALID, "dion_ns_line_3: in-place not supported");
  if (int rc = check_gemm_ptr("dion_ns_line_3", "B", B)) return rc;
  if (int rc = check_gemm_ptr("dion_ns_line_3", "X", X)) return rc;
  if (int rc = check_gemm_ptr("dion_ns_line_3", "C", C)) return rc;
  GemmParams p;
  memset(&p, 0, sizeof(p));
  p.P = (const bf16_t*)B;
  p.Q = (const bf16_t*)X;  // read as it lies: reduction index along rows
  p.q_kmajor = 1;
  p.D = a != 0.0f ? (const bf16_t*)X : nullptr;  // a == 0: pure product, X is not read a second time
  p.C = (bf16_t*)C;
  p.strideP = (int64_t)m * m;
  p.strideQ = p.strideD = p.strideC = (int64_t)m * n;
  p.ldp = m;
  p.ldq = p.ldd = p.ldc = n;
  p.M = m;
  p.N = n;
  p.K = m;
  p.batch = batch;
  p.alpha = 1.0f;
  p.beta = a;
  HIP_TRY(launch_gemm_nt(p, (hipStream_t)stream), "dion_ns_line_3");
  return DION_OK;
}

// ---------------------------------------------------------------------------------------------
// Whole orthogonalization.  A call is planned first -- buffer layout in the workspace and the full
// list of kernel launches with their operands -- then the list is checked on the host against the
// buffers the call owns, and only then launched.
// ---------------------------------------------------------------------------------------------
static bool table_aligned(const uint64_t* t, int n);
static int check_state_dtype(const char* who, const char* arg, int dtype) {
  if (dtype != DION_BF16 && dtype != DION_F32)
    return fail(DION_E_INVALID, "%s: %s %d (DION_BF16 or DION_F32)", who, arg, dtype);
  return DION_OK;
}
static inline int dt(int dtype) { return dtype == DION_BF16 ? 0 : 1; }

namespace {
struct NsPlan {
  int m, n, mp, np, tall, nblk;
  bool gram;  // the Gram-matrix recurrence is used (requested and worth it for this aspect ratio)
  size_t x_bytes, a_bytes, partial_bytes, inv_bytes, total;
};

// The Gram recurrence trades rectangular GEMMs for m x m ones: 6 m^2 n + 20 m^3 executed FLOP
// against 15 m^2 n + 5 m^3 for the standard iteration (five iterations, one restart), so it only
// pays for n > 5/3 m; it also squares the condition number between restarts, which costs accuracy
// on inputs that are not long (measured: 2.4e-2 from the exact result at n = 2.5 m, under 1e-2
// from n = 3 m).  Both forms apply the same polynomial: below n = 3 m the standard iteration is
// run whatever the flag says.
bool gram_pays(int m, int n) { return (int64_t)n >= 3 * (int64_t)m; }

NsPlan make_plan(int batch, int rows, int cols, int flags) {
  NsPlan pl;
  pl.tall = rows > cols;
  pl.m = pl.tall ? cols : rows;
  pl.n = pl.tall ? rows : cols;
  pl.gram = (flags & DION_NS_GRAM) && gram_pays(pl.m, pl.n);
  const int g = gemm_pad_granule(pl.m, pl.n, batch);
  pl.mp = round_up(pl.m, g);
  pl.np = round_up(pl.n, g);
  const int64_t numel = (int64_t)rows * cols;
  int64_t nb = numel / (256 * 32);
  if (nb < 1) nb = 1;
  if (nb > 1024) nb = 1024;
  pl.nblk = (int)nb;
  pl.x_bytes = align256((size_t)batch * pl.mp * pl.np * 2);
  pl.a_bytes = align256((size_t)batch * pl.mp * pl.mp * 2);
  pl.partial_bytes = align256((size_t)batch * pl.nblk * 4);
  pl.inv_bytes = align256((size_t)batch * 4);
  // X ping-pong pair + one X^T (the last product of a padded tall input); A, B (six m x m buffers
  // for the Gram recurrence); norm partials and reciprocal norms
  pl.total = 3 * pl.x_bytes + (pl.gram ? 6 : 2) * pl.a_bytes + pl.partial_bytes + pl.inv_bytes;
  return pl;
}

// The Muon update that consumes the orthogonalized matrices (dion_ns_orthogonalize_update).
struct PostSpec {
  const uint64_t* X_ptrs;
  int x_dtype, n_ptrs, mats_per_ptr;
  const float* lr_dev;
  float adj_ratio;
  const float* wd_dev;
  float wd_host;
  int cautious;
};

// per-head regime: whole iteration resident in LDS, one workgroup per matrix, no workspace.  The Gram
// flag changes nothing here: the recurrence saves memory traffic of rectangular GEMMs, and a matrix
// that never leaves LDS has none; the standard iteration applies the same polynomial.
bool ns_small_path(int rows, int cols, int flags, int n_iters) {
  (void)flags;
  return n_iters <= kMaxSmallIters && ns_small_fits(rows, cols);
}

// The update rides on the last GEMM when that GEMM produces the caller's tensor directly: at least
// one iteration, no padding between the matrices and the tiles, not the LDS-resident kernel.
bool ns_update_fuses(int batch, int rows, int cols, int flags, int n_iters) {
  if (n_iters <= 0 || ns_small_path(rows, cols, flags, n_iters)) return false;
  const NsPlan pl = make_plan(batch, rows, cols, flags);
  return pl.mp == pl.m && pl.np == pl.n;
}

// A prepared input (short side along rows, unnormalised, with partial sums of squares) is taken when
// the matrices fill whole tiles -- no padding, so the input can be the first GEMMs' operand as it lies --
// outside the LDS-resident kernel and with at least one iteration to carry the normalisation.
bool ns_accepts_prepared(int batch, int rows, int cols, int flags, int n_iters) {
  if (batch <= 0 || batch > 65535 || rows <= 0 || cols <= 0 || n_iters <= 0) return false;
  if (ns_small_path(rows, cols, flags, n_iters)) return false;
  if (((int64_t)rows * cols) % 4096) return false;
  const NsPlan pl = make_plan(batch, rows, cols, flags);
  return pl.mp == pl.m && pl.np == pl.n;
}

// One kernel launch of a planned call.
struct NsStep {
  enum Kind { kNorm, kNormFinalize, kPrepare, kGemm, kGemmUpdate, kUnpad, kSmall } kind;
  const char* what;
  GemmParams g;    // kGemm, kGemmUpdate
  // kGemmUpdate: the launch updates parameters ptr0 .. ptr0 + n_ptr - 1 of the call's table
  int ptr0, n_ptr;
  int x_code;      // kGemmUpdate: 0 bf16, 1 fp32 parameters
  bool transposed; // kGemmUpdate: the product updates X[col][row]
  // kNorm, kPrepare, kSmall: the caller's input; kNormFinalize: `partial` is read, not written
  const void* in;
  int in_dtype, batch, R, C;
  float norm_scale, eps;
  float* partial;
  int nblk;
  float* inv;
  // kPrepare: X (same orientation as the input) and / or its transpose, padded to Rp x Cp
  bf16_t* same;
  int Rp, Cp, ld_same;
  int64_t stride_same;
  bf16_t* trans;
  int ld_trans;
  int64_t stride_trans;
  // kUnpad: padded source -> dense destination;  kSmall: dst = the caller's output
  const bf16_t* src;
  int64_t src_stride;
  int ld;
  bf16_t* dst;
  NsCoeffs co;  // kSmall
};

// The launch list of one call.  Fixed capacity and no heap: planning a call allocates nothing, on
// the host or on the device.  A standard iteration is three launches, a Gram iteration at most five.
constexpr int kMaxSteps = 160;
struct NsCall {
  NsStep steps[kMaxSteps];
  int n_steps;
  bool overflow;
  void push(const NsStep& s) {
    if (n_steps < kMaxSteps) steps[n_steps++] = s;
    else overflow = true;
  }
  const PostSpec* post;  // the update a kGemmUpdate step applies
  // what the call may read and write: [lo, hi) byte ranges (sq: the caller's norm partials, read only)
  const char *in_lo, *in_hi, *out_lo, *out_hi, *ws_lo, *ws_hi, *sq_lo, *sq_hi;
  // parameters updated in place by a fused update: n_ptrs ranges of x_bytes each
  const uint64_t* X_ptrs;
  int n_ptrs;
  size_t x_bytes;
};

NsStep blank_step(NsStep::Kind kind, const char* what) {
  NsStep s;
  memset((void*)&s, 0, sizeof(s));
  s.kind = kind;
  s.what = what;
  return s;
}

// Builds the launch list of one orthogonalization (no HIP call is made).  With `post` (only when
// ns_update_fuses) the last GEMM applies the update to the parameters and `out` is not written.
// With `sumsq` the input is "prepared": bf16 [batch, m, n] with the short side along rows (the transpose
// of a tall caller matrix), not normalised, and sumsq [batch, sumsq_blocks] holds partial sums of its
// squares per matrix.  The normalisation is then folded into the first two GEMMs as a per-matrix factor
// and neither the norm pass nor the prepare pass runs (only when ns_accepts_prepared).
int ns_build(const void* in, int in_dtype, void* out, int batch, int rows, int cols, const float* coeffs,
             int n_iters, float norm_scale, float eps, int flags, int gram_reset, void* workspace,
             size_t workspace_bytes, const PostSpec* post, NsCall& call, const float* sumsq = nullptr,
             int sumsq_blocks = 0) {
  call.n_steps = 0;
  call.overflow = false;
  call.post = post;
  call.in_lo = call.in_hi = call.out_lo = call.out_hi = call.ws_lo = call.ws_hi = call.sq_lo = call.sq_hi = nullptr;
  call.X_ptrs = nullptr;
  call.n_ptrs = 0;
  call.x_bytes = 0;
  if (batch < 0 || rows < 0 || cols < 0 || n_iters < 0)
    return fail(DION_E_INVALID, "dion_ns_orthogonalize: negative extent");
  if (in_dtype != DION_BF16 && in_dtype != DION_F32)
    return fail(DION_E_INVALID, "dion_ns_orthogonalize: in_dtype %d", in_dtype);
  if (batch == 0 || rows == 0 || cols == 0) return DION_OK;
  if (!in || (!out && !post) || (n_iters > 0 && !coeffs))
    return fail(DION_E_INVALID, "dion_ns_orthogonalize: null argument");
  if (flags & ~DION_NS_GRAM) return fail(DION_E_INVALID, "dion_ns_orthogonalize: flags 0x%x", flags);
  const size_t mat_elems = (size_t)rows * cols;
  call.in_lo = (const char*)in;
  call.in_hi = call.in_lo + (size_t)batch * mat_elems * (in_dtype == DION_BF16 ? 2 : 4);
  if (out) {
    call.out_lo = (const char*)out;
    call.out_hi = call.out_lo + (size_t)batch * mat_elems * 2;
  }
  if (post) {
    call.X_ptrs = post->X_ptrs;
    call.n_ptrs = post->n_ptrs;
    call.x_bytes = (size_t)post->mats_per_ptr * mat_elems * (post->x_dtype == DION_BF16 ? 2 : 4);
  }
  if (sumsq) {
    if (!ns_accepts_prepared(batch, rows, cols, flags, n_iters) || in_dtype != DION_BF16 || sumsq_blocks <= 0)
      return fail(DION_E_INVALID,
                  "dion_ns_orthogonalize_prepared: %d x (%d x %d), %d iterations does not take a prepared input "
                  "(see dion_ns_accepts_prepared)", batch, rows, cols, n_iters);
    if (!aligned16((uint64_t)(uintptr_t)in))
      return fail(DION_E_INVALID, "dion_ns_orthogonalize_prepared: in is not 16-byte aligned");
    call.sq_lo = (const char*)sumsq;
    call.sq_hi = call.sq_lo + (size_t)batch * sumsq_blocks * 4;
  }
  if (ns_small_path(rows, cols, flags, n_iters)) {
    NsStep s = blank_step(NsStep::kSmall, "small-matrix Newton-Schulz");
    s.in = in;
    s.in_dtype = in_dtype;
    s.dst = (bf16_t*)out;
    s.batch = batch;
    s.R = rows;
    s.C = cols;
    s.norm_scale = norm_scale;
    s.eps = eps;
    s.co.n = n_iters;
    for (int i = 0; i < n_iters * 3; ++i) s.co.c[i / 3][i % 3] = coeffs[i];
    call.push(s);
    return DION_OK;
  }
  // the last GEMM stores into the caller's buffer 16 bytes per lane
  if (out && !aligned16((uint64_t)(uintptr_t)out))
    return fail(DION_E_INVALID, "dion_ns_orthogonalize: out is not 16-byte aligned");
  if (batch > 65535)
    return fail(DION_E_INVALID,
                "dion_ns_orthogonalize: %d matrices in one call (at most 65535 outside the small-matrix "
                "kernel): split the batch",
                batch);
  const NsPlan pl = make_plan(batch, rows, cols, flags);
  if (!workspace || workspace_bytes < pl.total)
    return fail(DION_E_WORKSPACE, "dion_ns_orthogonalize: workspace %zu < %zu bytes", workspace_bytes,
                pl.total);
  if (((uintptr_t)workspace & 255) != 0)
    return fail(DION_E_INVALID, "dion_ns_orthogonalize: workspace not 256-byte aligned");
  call.ws_lo = (const char*)workspace;
  call.ws_hi = call.ws_lo + workspace_bytes;

  char* w = (char*)workspace;
  bf16_t* X[2];
  X[0] = (bf16_t*)w; w += pl.x_bytes;
  X[1] = (bf16_t*)w; w += pl.x_bytes;
  bf16_t* Xt = (bf16_t*)w; w += pl.x_bytes;
  bf16_t* sq[6] = {nullptr, nullptr, nullptr, nullptr, nullptr, nullptr};  // m x m scratch
  for (int i = 0; i < (pl.gram ? 6 : 2); ++i) {
    sq[i] = (bf16_t*)w;
    w += pl.a_bytes;
  }
  float* partial = (float*)w; w += pl.partial_bytes;
  float* inv = (float*)w; w += pl.inv_bytes;

  const int mp = pl.mp, np = pl.np;
  const int64_t sX = (int64_t)mp * np, sA = (int64_t)mp * mp;
  // An input that fills whole tiles is not scaled on its way in either: a wide bf16 one is read by the first
  // GEMMs where it lies, any other is copied (rounded to bf16, transposed if tall) value for value, and the
  // normalisation rides on the first two GEMMs as for a prepared input -- one pass over a wide bf16 input instead
  // of two, and the same arithmetic whichever way (orientation, fp32 or bf16) a matrix is handed over.
  const bool self_prep = !sumsq && aligned16((uint64_t)(uintptr_t)in) &&
                         ns_accepts_prepared(batch, rows, cols, flags, n_iters);
  // (not when `out` overlaps `in`: the copy is then what keeps a caller's in-place call working)
  const bool aliased = out && call.out_lo < call.in_hi && call.in_lo < call.out_hi;
  const bool in_place = self_prep && !pl.tall && in_dtype == DION_BF16 && !aliased;
  const bool copy_first = self_prep && pl.tall;
  auto plan_norm = [&]() {
    if (sumsq) {
      NsStep s = blank_step(NsStep::kNormFinalize, "frobenius norm from the caller's partial sums");
      s.batch = batch;
      s.norm_scale = norm_scale;
      s.eps = eps;
      s.partial = const_cast<float*>(sumsq);
      s.nblk = sumsq_blocks;
      s.inv = inv;
      call.push(s);
    } else {
      // (over the transposed copy of a tall input that is copied unscaled: the sum then runs in the order it
      // runs in for the same matrix handed over wide, and the two calls agree bit for bit)
      NsStep s = blank_step(NsStep::kNorm, "frobenius norm");
      s.in = copy_first ? (const void*)X[0] : in;
      s.in_dtype = copy_first ? DION_BF16 : in_dtype;
      s.batch = batch;
      s.R = copy_first ? mp : rows;
      s.C = copy_first ? np : cols;
      s.norm_scale = norm_scale;
      s.eps = eps;
      s.partial = partial;
      s.nblk = pl.nblk;
      s.inv = inv;
      call.push(s);
    }
  };
  auto plan_prepare = [&]() {
    if (!sumsq && !in_place) {
      // Only X (short side along rows) is carried between iterations: X' = B X reads X with the
      // reduction index along rows.  With no iteration at all the result is the prepared input, and
      // the output copy of a tall input reads X^T: prepare that layout instead.
      NsStep s = blank_step(NsStep::kPrepare, "prepare");
      s.in = in;
      s.in_dtype = in_dtype;
      s.batch = batch;
      s.R = rows;
      s.C = cols;
      s.inv = self_prep ? nullptr : inv;  // null: plain copy
      if (pl.tall) {
        s.Rp = np;
        s.Cp = mp;
        s.same = n_iters > 0 ? nullptr : Xt;
        s.ld_same = mp;
        s.stride_same = sX;
        s.trans = n_iters > 0 ? X[0] : nullptr;
        s.ld_trans = np;
        s.stride_trans = sX;
      } else {
        s.Rp = mp;
        s.Cp = np;
        s.same = X[0];
        s.ld_same = np;
        s.stride_same = sX;
      }
      call.push(s);
    }
  };
  if (copy_first) {
    plan_prepare();
    plan_norm();
  } else {
    plan_norm();
    plan_prepare();
  }

  const bool direct = (mp == pl.m && np == pl.n);

  // ---- the GEMM shapes of the iteration
  // sym(P, Q -> C): C = alpha P Q^T + beta D + diag I for symmetric m x m operands whose product
  // is symmetric; upper tiles computed, mirrored on store.
  // With tri == false the whole product is computed: needed when symmetry of the result rests on
  // the (bf16-rounded, hence only approximate) commutation of P and Q -- mirroring such a product
  // plants a commutator-sized error.
  auto sym = [&](const char* what, const bf16_t* P, const bf16_t* Q, const bf16_t* D, bf16_t* C, float alpha,
                 float beta, float diag, bool tri = true) {
    NsStep s = blank_step(NsStep::kGemm, what);
    GemmParams& p = s.g;
    p.P = P;
    p.Q = Q;
    p.D = D;
    p.C = C;
    p.Ct = tri ? C : nullptr;
    p.strideP = p.strideQ = p.strideD = p.strideC = p.strideCt = sA;
    p.ldp = p.ldq = p.ldd = p.ldc = p.ldct = mp;
    p.M = p.N = p.K = mp;
    p.batch = batch;
    p.tri = tri ? 1 : 0;
    p.alpha = alpha;
    p.beta = beta;
    p.diag = diag;
    call.push(s);
  };
  // A prepared input is the unnormalised X_0: every GEMM that reads it carries the factor 1/(||X_0|| s + eps)
  // (squared for X_0 X_0^T); products of these GEMMs are normalised, and so is every later X.
  const bf16_t* const x_raw = (sumsq || in_place) ? (const bf16_t*)in : self_prep ? X[0] : nullptr;
  bool x_written = false;  // an X' has been written: from then on every X is normalised
  auto scaled = [&](GemmParams& p, const bf16_t* Xc, int pow) {
    if (x_raw && Xc == x_raw && !x_written) {
      p.scale_vec = inv;
      p.scale_pow = pow;
    }
  };
  // gram(Xc -> R): R = Xc Xc^T
  auto gram = [&](const char* what, const bf16_t* Xc, bf16_t* R) {
    NsStep s = blank_step(NsStep::kGemm, what);
    GemmParams& p = s.g;
    scaled(p, Xc, 2);
    p.P = p.Q = Xc;
    p.C = p.Ct = R;
    p.strideP = p.strideQ = sX;
    p.strideC = p.strideCt = sA;
    p.ldp = p.ldq = np;
    p.ldc = p.ldct = mp;
    p.M = p.N = mp;
    p.K = np;
    p.batch = batch;
    p.tri = 1;
    p.alpha = 1.0f;
    call.push(s);
  };
  // apply(S, Xc -> Xn | Xt | out | parameters): X' = S X (S symmetric m x m).  The last product of a
  // tall input is written transposed (the caller's orientation); when no padding is in the way
  // (`final_direct`) it goes straight into the caller's tensor, or into the update of the parameters.
  auto apply = [&](const char* what, const bf16_t* S, const bf16_t* Xc, bf16_t* Xn, bool last, bool final_direct) {
    GemmParams p;
    memset(&p, 0, sizeof(p));
    p.P = S;
    p.strideP = sA;
    p.ldp = mp;
    p.Q = Xc;
    p.strideQ = sX;
    p.ldq = np;
    p.q_kmajor = 1;
    p.M = mp;
    p.N = np;
    p.K = mp;
    p.batch = batch;
    p.alpha = 1.0f;
    scaled(p, Xc, 1);
    if (final_direct && post) {
      // the product is consumed by the update: one launch per kMaxPtrs parameters
      const int mpp = post->mats_per_ptr;
      if (pl.tall) {
        p.strideCt = sX;
        p.ldct = mp;
      } else {
        p.strideC = sX;
        p.ldc = np;
      }
      for (int c0 = 0; c0 < post->n_ptrs; c0 += kMaxPtrs) {
        const int c = (post->n_ptrs - c0) < kMaxPtrs ? (post->n_ptrs - c0) : kMaxPtrs;
        const int64_t b0 = (int64_t)c0 * mpp;
        NsStep s = blank_step(NsStep::kGemmUpdate, what);
        s.g = p;
        s.g.P = p.P + b0 * p.strideP;
        s.g.Q = p.Q + b0 * p.strideQ;
        if (s.g.scale_vec) s.g.scale_vec += b0;
        s.g.batch = c * mpp;
        s.ptr0 = c0;
        s.n_ptr = c;
        s.x_code = dt(post->x_dtype);
        s.transposed = pl.tall != 0;
        call.push(s);
      }
      return;
    }
    if (final_direct) {
      if (pl.tall) {
        p.Ct = (bf16_t*)out;
        p.strideCt = sX;
        p.ldct = mp;
      } else {
        p.C = (bf16_t*)out;
        p.strideC = sX;
        p.ldc = np;
      }
    } else if (last && pl.tall) {
      p.Ct = Xt;
      p.strideCt = sX;
      p.ldct = mp;
    } else {
      p.C = Xn;
      p.strideC = sX;
      p.ldc = np;
    }
    NsStep s = blank_step(NsStep::kGemm, what);
    s.g = p;
    call.push(s);
  };

  int cur = 0;
  bool wrote_out = false;
  // the matrix the next GEMM reads as X: the unnormalised input until the first X' is written
  auto xc = [&]() -> const bf16_t* { return (x_raw && !x_written) ? x_raw : X[cur]; };
  if (!pl.gram) {
    for (int it = 0; it < n_iters; ++it) {
      const float a = coeffs[3 * it], b = coeffs[3 * it + 1], c = coeffs[3 * it + 2];
      gram("A = X X^T", xc(), sq[0]);
      // a*I folded into B: the next GEMM needs no addend (one fewer pass over X)
      sym("B = c A A + b A + a I", sq[0], sq[0], sq[0], sq[1], c, b, a);
      const bool fin = (it == n_iters - 1) && direct;
      apply("X = B X", sq[1], xc(), X[cur ^ 1], it == n_iters - 1, fin);
      wrote_out = fin;
      cur ^= 1;
      x_written = true;
    }
  } else {
    // Gram recurrence: R = X X^T and Q with X_t = Q X_0 live in m x m; per iteration
    // Z = a I + b R + c R^2, Q <- Z Q, R <- Z R Z (all symmetric and commuting).  At the restart
    // iteration X is materialised, R recomputed from it and Q reset, which bounds the bf16 drift
    // of the R recurrence.  The rectangular work drops from 10 GEMMs to 2 Gram + 2 apply.
    bool used[6] = {false, false, false, false, false, false};
    auto take = [&]() -> int {
      for (int i = 0; i < 6; ++i)
        if (!used[i]) {
          used[i] = true;
          return i;
        }
      return -1;
    };
    int r = take(), q = -1;
    gram("R = X X^T", xc(), sq[r]);
    for (int it = 0; it < n_iters; ++it) {
      const float a = coeffs[3 * it], b = coeffs[3 * it + 1], c = coeffs[3 * it + 2];
      if (it == gram_reset && it > 0 && q >= 0) {
        apply("X = Q X (restart)", sq[q], xc(), X[cur ^ 1], false, false);
        cur ^= 1;
        x_written = true;
        used[q] = false;
        q = -1;
        gram("R = X X^T (restart)", xc(), sq[r]);
      }
      const int z = take();
      sym("Z = a I + b R + c R R", sq[r], sq[r], sq[r], sq[z], c, b, a);
      const bool need_r = !(it == n_iters - 1 || (it + 1 == gram_reset));
      if (need_r) {
        const int t = take();
        sym("T = Z R", sq[z], sq[r], nullptr, sq[t], 1.0f, 0.0f, 0.0f, false);
        const int rn = take();
        sym("R = T Z", sq[t], sq[z], nullptr, sq[rn], 1.0f, 0.0f, 0.0f);
        used[t] = false;
        used[r] = false;
        r = rn;
      }
      if (q < 0) {
        q = z;  // Q = Z (Q was the identity)
      } else {
        const int qn = take();
        sym("Q = Z Q", sq[z], sq[q], nullptr, sq[qn], 1.0f, 0.0f, 0.0f, false);
        used[q] = false;
        used[z] = false;
        q = qn;
      }
    }
    if (q >= 0) {
      apply("X = Q X", sq[q], xc(), X[cur ^ 1], true, direct);
      wrote_out = direct;
      cur ^= 1;
      x_written = true;
    }
  }
  if (!wrote_out) {
    if (post) return fail(DION_E_INVALID, "dion_ns_orthogonalize_update: update not applied (internal)");
    NsStep s = blank_step(NsStep::kUnpad, "unpad");
    // a tall result lies transposed-back in Xt: written there by the last product, or by the
    // prepare step when there was no iteration
    s.src = pl.tall ? Xt : X[cur];
    s.src_stride = sX;
    s.ld = pl.tall ? mp : np;
    s.dst = (bf16_t*)out;
    s.batch = batch;
    s.R = rows;
    s.C = cols;
    call.push(s);
  }
  if (call.overflow)
    return fail(DION_E_INVALID, "dion_ns_orthogonalize: more than %d kernel launches in one call (%d iterations, %d "
                "parameters): split the call", kMaxSteps, n_iters, post ? post->n_ptrs : 0);
  return DION_OK;
}

// ---- host-side bounds check of a planned call: every byte a launch reads lies inside the caller's
// input or the workspace, every byte it writes inside the workspace, the caller's output or (fused
// update) one parameter; tile shapes divide the padded extents.
bool inside(const void* lo, size_t bytes, const char* r_lo, const char* r_hi) {
  const char* p = (const char*)lo;
  return r_lo && p >= r_lo && p <= r_hi && bytes <= (size_t)(r_hi - p);
}

// bytes spanned by `batch` matrices of `rows` x `cols` elements of `es` bytes, row pitch ld, batch stride
size_t span_bytes(int batch, int64_t stride, int rows, int ld, int cols, int es) {
  if (batch <= 0 || rows <= 0 || cols <= 0) return 0;
  return ((size_t)(batch - 1) * (size_t)stride + (size_t)(rows - 1) * (size_t)ld + (size_t)cols) * (size_t)es;
}

int ns_audit(const NsCall& call) {
  auto rd = [&](const void* p, size_t bytes) {
    return inside(p, bytes, call.in_lo, call.in_hi) || inside(p, bytes, call.ws_lo, call.ws_hi);
  };
  auto wr = [&](const void* p, size_t bytes) {
    return inside(p, bytes, call.ws_lo, call.ws_hi) || inside(p, bytes, call.out_lo, call.out_hi);
  };
  for (int idx = 0; idx < call.n_steps; ++idx) {
    const NsStep& s = call.steps[idx];
    const char* bad = nullptr;
    switch (s.kind) {
      case NsStep::kNormFinalize:
        if (s.nblk <= 0 || !inside(s.partial, (size_t)s.batch * s.nblk * 4, call.sq_lo, call.sq_hi)) bad = "norm partials";
        else if (!wr(s.inv, (size_t)s.batch * 4)) bad = "reciprocal norms";
        break;
      case NsStep::kNorm: {
        const size_t es = s.in_dtype == DION_BF16 ? 2 : 4;
        if (!rd(s.in, (size_t)s.batch * s.R * s.C * es)) bad = "input";
        else if (!wr(s.partial, (size_t)s.batch * s.nblk * 4)) bad = "norm partials";
        else if (!wr(s.inv, (size_t)s.batch * 4)) bad = "reciprocal norms";
        break;
      }
      case NsStep::kPrepare: {
        const size_t es = s.in_dtype == DION_BF16 ? 2 : 4;
        if (s.Rp % 64 || s.Cp % 64 || s.Rp < s.R || s.Cp < s.C) bad = "padded extents";
        else if (!rd(s.in, (size_t)s.batch * s.R * s.C * es)) bad = "input";
        else if (s.inv && !rd(s.inv, (size_t)s.batch * 4)) bad = "reciprocal norms";
        else if (s.same && !wr(s.same, span_bytes(s.batch, s.stride_same, s.Rp, s.ld_same, s.Cp, 2))) bad = "X";
        else if (s.trans && !wr(s.trans, span_bytes(s.batch, s.stride_trans, s.Cp, s.ld_trans, s.Rp, 2)))
          bad = "X^T";
        else if (!s.same && !s.trans) bad = "no destination";
        break;
      }
      case NsStep::kGemm:
      case NsStep::kGemmUpdate: {
        const GemmParams& p = s.g;
        const int tile = gemm_tile_edge(p);
        if (p.M % tile || p.N % tile || p.K % 128 || (p.tri && p.M != p.N)) bad = "tile does not divide the extents";
        else if (!rd(p.P, span_bytes(p.batch, p.strideP, p.M, p.ldp, p.K, 2))) bad = "first operand";
        else if (!(p.q_kmajor ? rd(p.Q, span_bytes(p.batch, p.strideQ, p.K, p.ldq, p.N, 2))
                              : rd(p.Q, span_bytes(p.batch, p.strideQ, p.N, p.ldq, p.K, 2))))
          bad = "second operand";
        else if (p.D && !rd(p.D, span_bytes(p.batch, p.strideD, p.M, p.ldd, p.N, 2))) bad = "addend";
        else if (p.scale_vec && (!inside(p.scale_vec, (size_t)p.batch * 4, call.ws_lo, call.ws_hi) ||
                                 (p.scale_pow != 1 && p.scale_pow != 2)))
          bad = "per-matrix factors";
        else if (p.C && !wr(p.C, span_bytes(p.batch, p.strideC, p.M, p.ldc, p.N, 2))) bad = "product";
        else if (p.Ct && !wr(p.Ct, span_bytes(p.batch, p.strideCt, p.N, p.ldct, p.M, 2))) bad = "transposed product";
        else if (s.kind == NsStep::kGemm && !p.C && !p.Ct) bad = "no destination";
        else if (s.kind == NsStep::kGemmUpdate) {
          // matrix b updates parameter b / mats_per_ptr at matrix offset b % mats_per_ptr
          const int es = s.x_code == 0 ? 2 : 4;
          const int mpp = call.post ? call.post->mats_per_ptr : 0;
          const size_t one = s.transposed ? span_bytes(1, 0, p.N, p.ldct, p.M, es) : span_bytes(1, 0, p.M, p.ldc, p.N, es);
          const size_t stride = (size_t)(s.transposed ? p.strideCt : p.strideC) * es;
          if (mpp <= 0 || s.n_ptr <= 0 || s.n_ptr > kMaxPtrs || p.batch != s.n_ptr * mpp || s.ptr0 < 0 ||
              s.ptr0 + s.n_ptr > call.n_ptrs || p.C || p.Ct)
            bad = "update batch";
          else if ((size_t)(mpp - 1) * stride + one > call.x_bytes) bad = "parameter extent";
          else
            for (int i = 0; i < s.n_ptr && !bad; ++i)
              if (!call.X_ptrs[s.ptr0 + i]) bad = "null parameter";
        }
        break;
      }
      case NsStep::kUnpad:
        if (!rd(s.src, span_bytes(s.batch, s.src_stride, s.R, s.ld, s.C, 2))) bad = "padded source";
        else if (!wr(s.dst, (size_t)s.batch * s.R * s.C * 2)) bad = "output";
        break;
      case NsStep::kSmall: {
        const size_t es = s.in_dtype == DION_BF16 ? 2 : 4;
        if (!rd(s.in, (size_t)s.batch * s.R * s.C * es)) bad = "input";
        else if (!wr(s.dst, (size_t)s.batch * s.R * s.C * 2)) bad = "output";
        break;
      }
    }
    if (bad)
      return fail(DION_E_INVALID, "dion_ns_orthogonalize: launch %d (%s) would access its %s outside the call's buffers",
                  idx, s.what, bad);
  }
  return DION_OK;
}

int ns_execute(const NsCall& call, hipStream_t st) {
  for (int idx = 0; idx < call.n_steps; ++idx) {
    const NsStep& s = call.steps[idx];
    hipError_t e = hipSuccess;
    switch (s.kind) {
      case NsStep::kNormFinalize:
        e = launch_norm_finalize(s.partial, s.nblk, s.batch, s.norm_scale, s.eps, s.inv, st);
        break;
      case NsStep::kNorm:
        e = launch_frobenius_inv(s.in, s.in_dtype, s.batch, (int64_t)s.R * s.C, s.norm_scale, s.eps, s.partial,
                                 s.nblk, s.inv, st);
        break;
      case NsStep::kPrepare:
        e = launch_ns_prepare(s.in, s.in_dtype, s.batch, s.R, s.C, s.inv, s.same, s.Rp, s.Cp, s.ld_same,
                              s.stride_same, s.trans, s.ld_trans, s.stride_trans, st);
        break;
      case NsStep::kGemm:
        e = launch_gemm_nt(s.g, st);
        break;
      case NsStep::kGemmUpdate: {
        const PostSpec& ps = *call.post;
        FusedPost fp;
        memset((void*)&fp, 0, sizeof(fp));
        memcpy(fp.X.p, ps.X_ptrs + s.ptr0, (size_t)s.n_ptr * sizeof(uint64_t));
        fp.mats_per_ptr = ps.mats_per_ptr;
        fp.vec_ok = table_aligned(ps.X_ptrs + s.ptr0, s.n_ptr) ? 1 : 0;
        fp.lr_dev = ps.lr_dev;
        fp.wd_dev = ps.wd_dev;
        fp.wd_host = ps.wd_host;
        fp.adj_ratio = ps.adj_ratio;
        fp.cautious = ps.cautious;
        e = launch_gemm_nt_post(s.g, fp, s.x_code, s.transposed, st);
        break;
      }
      case NsStep::kUnpad:
        e = launch_unpad(s.src, s.src_stride, s.ld, s.dst, s.batch, s.R, s.C, st);
        break;
      case NsStep::kSmall:
        e = launch_ns_small(s.in, s.in_dtype, s.dst, s.batch, s.R, s.C, s.co, s.norm_scale, s.eps, st);
        break;
    }
    if (e != hipSuccess) return hip_fail(e, s.what);
  }
  return DION_OK;
}

int ns_run(const void* in, int in_dtype, void* out, int batch, int rows, int cols, const float* coeffs,
           int n_iters, float norm_scale, float eps, int flags, int gram_reset, void* workspace,
           size_t workspace_bytes, void* stream, const PostSpec* post, const float* sumsq = nullptr,
           int sumsq_blocks = 0) {
  NsCall call;  // on the stack: planning allocates nothing
  if (int rc = ns_build(in, in_dtype, out, batch, rows, cols, coeffs, n_iters, norm_scale, eps, flags, gram_reset,
                        workspace, workspace_bytes, post, call, sumsq, sumsq_blocks))
    return rc;
  if (int rc = ns_audit(call)) return rc;
  return ns_execute(call, (hipStream_t)stream);
}
}  // namespace

extern "C" size_t dion_ns_workspace_bytes(int batch, int rows, int cols, int flags) {
  if (batch <= 0 || rows <= 0 || cols <= 0) return 0;
  return make_plan(batch, rows, cols, flags).total;
}

extern "C" int dion_ns_orthogonalize(const void* in, int in_dtype, void* out, int batch, int rows,
                                     int cols, const float* coeffs, int n_iters, float norm_scale,
                                     float eps, int flags, int gram_reset, void* workspace,
                                     size_t workspace_bytes, void* stream) {
  return ns_run(in, in_dtype, out, batch, rows, cols, coeffs, n_iters, norm_scale, eps, flags, gram_reset,
                workspace, workspace_bytes, stream, nullptr);
}

// ---------------------------------------------------------------------------------------------
// dion_ns_orthogonalize for callers that cannot provide (or allocate) a workspace: the same driver
// and kernels over a fixed device array that is part of the library's code object.  Each GPU holds
// its own copy of the array at its own address, resolved once per device; host code never uses the
// array's name as an address, only the resolved pointer.
// ---------------------------------------------------------------------------------------------
static __device__ __align__(256) unsigned char scratch[DION_NS_STATIC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
std::atomic<void*> g_scratch_ptr[kMaxDevices];

// Device address of `scratch` on the current device (looked up on the first call per device).
int static_scratch(void** ptr) {
  int dev = 0;
  HIP_TRY(hipGetDevice(&dev), "hipGetDevice");
  if (dev < 0 || dev >= kMaxDevices)
    return fail(DION_E_INVALID, "dion_ns_orthogonalize_static: device ordinal %d (at most %d devices)", dev,
                kMaxDevices);
  void* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (!p) {
    // Racing first calls resolve the same address; the lookup allocates nothing.
    HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)), "hipGetSymbolAddress(scratch)");
    if (!p || ((uintptr_t)p & 255) != 0)
      return fail(DION_E_HIP, "dion_ns_orthogonalize_static: scratch array resolved to %p", p);
    g_scratch_ptr[dev].store(p, std::memory_order_release);
  }
  *ptr = p;
  return DION_OK;
}
}  // namespace

extern "C" int dion_ns_orthogonalize_static(const void* in, int in_dtype, void* out, int batch, int rows,
                                            int cols, const float* coeffs, int n_iters, float norm_scale,
                                            float eps, int flags, int gram_reset, void* stream) {
  size_t need = 0;
  if (batch > 0 && rows > 0 && cols > 0 && !(flags & ~DION_NS_GRAM) && n_iters >= 0 &&
      !ns_small_path(rows, cols, flags, n_iters))
    need = make_plan(batch, rows, cols, flags).total;
  if (need > (size_t)DION_NS_STATIC_SCRATCH_BYTES)
    return fail(DION_E_WORKSPACE,
                "dion_ns_orthogonalize_static: %d x (%d x %d) needs %zu bytes of scratch, the library's fixed "
                "array holds %zu: use dion_ns_orthogonalize with a caller workspace",
                batch, rows, cols, need, (size_t)DION_NS_STATIC_SCRATCH_BYTES);
  void* ws = nullptr;
  if (need > 0)
    if (int rc = static_scratch(&ws)) return rc;
  // Nothing in the workspace has to start at zero: the prepare kernel writes every element of the
  // padded X (zero padding included) and every later buffer is fully written before it is read.
  return ns_run(in, in_dtype, out, batch, rows, cols, coeffs, n_iters, norm_scale, eps, flags, gram_reset, ws,
                need, stream, nullptr);
}

extern "C" size_t dion_ns_update_workspace_bytes(int batch, int rows, int cols, int flags, int n_iters) {
  if (batch <= 0 || rows <= 0 || cols <= 0) return 0;
  const size_t ns = ns_small_path(rows, cols, flags, n_iters) ? 0 : align256(make_plan(batch, rows, cols, flags).total);
  if (ns_update_fuses(batch, rows, cols, flags, n_iters)) return ns;
  return ns + align256((size_t)batch * rows * cols * 2);
}

extern "C" int dion_ns_orthogonalize_update(const void* in, int in_dtype, const uint64_t* X_ptrs, int x_dtype,
                                            int n_ptrs, int mats_per_ptr, int rows, int cols,
                                            const float* coeffs, int n_iters, float norm_scale, float eps,
                                            int flags, int gram_reset, const float* lr_dev, float adj_ratio,
                                            const float* wd_dev, float wd_host, int cautious,
                                            void* workspace, size_t workspace_bytes, void* stream) {
  if (int rc = check_state_dtype("dion_ns_orthogonalize_update", "x_dtype", x_dtype)) return rc;
  if (n_ptrs < 0 || mats_per_ptr <= 0 || rows < 0 || cols < 0 || n_iters < 0)
    return fail(DION_E_INVALID, "dion_ns_orthogonalize_update: bad size");
  if ((int64_t)n_ptrs * mats_per_ptr > 0x7fffffff)
    return fail(DION_E_INVALID, "dion_ns_orthogonalize_update: too many matrices");
  const int batch = n_ptrs * mats_per_ptr;
  if (batch == 0 || rows == 0 || cols == 0) return DION_OK;
  if (!X_ptrs || !lr_dev) return fail(DION_E_INVALID, "dion_ns_orthogonalize_update: null argument");
  for (int i = 0; i < n_ptrs; ++i)
    if (!X_ptrs[i]) return fail(DION_E_INVALID, "dion_ns_orthogonalize_update: parameter %d is null", i);
  const size_t need = dion_ns_update_workspace_bytes(batch, rows, cols, flags, n_iters);
  if (workspace_bytes < need)
    return fail(DION_E_WORKSPACE, "dion_ns_orthogonalize_update: workspace %zu < %zu bytes", workspace_bytes, need);
  if (ns_update_fuses(batch, rows, cols, flags, n_iters)) {
    const PostSpec ps = {X_ptrs, x_dtype, n_ptrs, mats_per_ptr, lr_dev, adj_ratio, wd_dev, wd_host, cautious};
    return ns_run(in, in_dtype, nullptr, batch, rows, cols, coeffs, n_iters, norm_scale, eps, flags, gram_reset,
                  workspace, workspace_bytes, stream, &ps);
  }
  // padded shapes and the LDS-resident kernel: orthogonalize into the tail of the workspace (the
  // last align256(batch * rows * cols * 2) bytes of what dion_ns_update_workspace_bytes reports),
  // then the plain update pass
  const size_t tail = align256((size_t)batch * rows * cols * 2);
  const size_t ns = need - tail;
  if (!workspace) return fail(DION_E_WORKSPACE, "dion_ns_orthogonalize_update: workspace is null");
  if (((uintptr_t)workspace & 255) != 0)
    return fail(DION_E_INVALID, "dion_ns_orthogonalize_update: workspace not 256-byte aligned");
  void* tmp = (char*)workspace + ns;
  if (int rc = ns_run(in, in_dtype, tmp, batch, rows, cols, coeffs, n_iters, norm_scale, eps, flags, gram_reset,
                      workspace, ns, stream, nullptr))
    return rc;
  return dion_muon_post(X_ptrs, x_dtype, tmp, DION_BF16, n_ptrs, (int64_t)mats_per_ptr * rows * cols, cols,
                        nullptr, lr_dev, nullptr, adj_ratio, wd_dev, wd_host, cautious, stream);
}

extern "C" int dion_ns_accepts_prepared(int batch, int rows, int cols, int flags, int n_iters) {
  if (flags & ~DION_NS_GRAM) return 0;
  return ns_accepts_prepared(batch, rows, cols, flags, n_iters) ? 1 : 0;
}

extern "C" int dion_ns_orthogonalize_prepared(const void* in, const float* sumsq, int sumsq_blocks, void* out,
                                              int batch, int rows, int cols, const float* coeffs, int n_iters,
                                              float norm_scale, float eps, int flags, int gram_reset,
                                              void* workspace, size_t workspace_bytes, void* stream) {
  if (batch == 0 || rows == 0 || cols == 0) return DION_OK;
  if (!sumsq) return fail(DION_E_INVALID, "dion_ns_orthogonalize_prepared: sumsq is null");
  return ns_run(in, DION_BF16, out, batch, rows, cols, coeffs, n_iters, norm_scale, eps, flags, gram_reset,
                workspace, workspace_bytes, stream, nullptr, sumsq, sumsq_blocks);
}

extern "C" int dion_ns_orthogonalize_update_prepared(const void* in, const float* sumsq, int sumsq_blocks,
                                                     const uint64_t* X_ptrs, int x_dtype, int n_ptrs,
                                                     int mats_per_ptr, int rows, int cols, const float* coeffs,
                                                     int n_iters, float norm_scale, float eps, int flags,
                                                     int gram_reset, const float* lr_dev, float adj_ratio,
                                                     const float* wd_dev, float wd_host, int cautious,
                                                     void* workspace, size_t workspace_bytes, void* stream) {
  if (int rc = check_state_dtype("dion_ns_orthogonalize_update_prepared", "x_dtype", x_dtype)) return rc;
  if (n_ptrs < 0 || mats_per_ptr <= 0 || rows < 0 || cols < 0 || n_iters < 0)
    return fail(DION_E_INVALID, "dion_ns_orthogonalize_update_prepared: bad size");
  if ((int64_t)n_ptrs * mats_per_ptr > 0x7fffffff)
    return fail(DION_E_INVALID, "dion_ns_orthogonalize_update_prepared: too many matrices");
  const int batch = n_ptrs * mats_per_ptr;
  if (batch == 0 || rows == 0 || cols == 0) return DION_OK;
  if (!X_ptrs || !lr_dev || !sumsq)
    return fail(DION_E_INVALID, "dion_ns_orthogonalize_update_prepared: null argument");
  for (int i = 0; i < n_ptrs; ++i)
    if (!X_ptrs[i]) return fail(DION_E_INVALID, "dion_ns_orthogonalize_update_prepared: parameter %d is null", i);
  if (!ns_update_fuses(batch, rows, cols, flags, n_iters))
    return fail(DION_E_INVALID, "dion_ns_orthogonalize_update_prepared: %d x (%d x %d) does not take a prepared input "
                "(see dion_ns_accepts_prepared)", batch, rows, cols);
  const PostSpec ps = {X_ptrs, x_dtype, n_ptrs, mats_per_ptr, lr_dev, adj_ratio, wd_dev, wd_host, cautious};
  return ns_run(in, DION_BF16, nullptr, batch, rows, cols, coeffs, n_iters, norm_scale, eps, flags, gram_reset,
                workspace, workspace_bytes, stream, &ps, sumsq, sumsq_blocks);
}

extern "C" int dion_gemm_tile_edge(int batch, int m, int n, int symmetric) {
  GemmParams p;
  memset(&p, 0, sizeof(p));
  p.M = m;
  p.N = symmetric ? m : n;
  p.batch = batch;
  p.tri = symmetric ? 1 : 0;
  return gemm_tile_edge(p);
}

// Host-only check of the planning code: builds the launch list of dion_ns_orthogonalize
// (with_update == 0) or of the fused form of dion_ns_orthogonalize_update (with_update != 0, when
// the shape fuses) over synthetic, never dereferenced addresses and checks it as every real call
// is checked before its first launch.  audit_ws_bytes > 0 checks against a workspace of that size
// instead of the size the plan was laid out for.
static int plan_audit(int batch, int rows, int cols, int in_dtype, int n_iters, int flags, int gram_reset,
                      int with_update, int x_dtype, int mats_per_ptr, size_t audit_ws_bytes, bool prepared) {
  if (batch <= 0 || rows <= 0 || cols <= 0 || n_iters < 0 || n_iters > 16 || mats_per_ptr <= 0)
    return fail(DION_E_INVALID, "dion_ns_plan_audit: bad size");
  if (int rc = check_state_dtype("dion_ns_plan_audit", "x_dtype", x_dtype)) return rc;
  float coeffs[48];
  for (int i = 0; i < 48; ++i) coeffs[i] = 1.0f;
  const bool small = ns_small_path(rows, cols, flags, n_iters);
  const size_t ws_bytes = small ? 0 : make_plan(batch, rows, cols, flags).total;
  // disjoint synthetic regions, 1 TiB apart
  char* const base = (char*)(uintptr_t)0x100000000000ull;
  const size_t gap = (size_t)1 << 40;
  void* in = base;
  void* out = base + gap;
  void* ws = base + 2 * gap;
  const float* sumsq = prepared ? (const float*)(base + 3 * gap + (gap >> 1)) : nullptr;
  const int sumsq_blocks = prepared ? (int)((int64_t)rows * cols / 4096) : 0;
  NsCall call;
  std::vector<uint64_t> xp;
  PostSpec ps;
  const bool fused = with_update && ns_update_fuses(batch, rows, cols, flags, n_iters);
  if (with_update && !fused)
    return fail(DION_E_INVALID, "dion_ns_plan_audit: this shape does not take the fused update");
  if (fused) {
    if (batch % mats_per_ptr) return fail(DION_E_INVALID, "dion_ns_plan_audit: batch %% mats_per_ptr != 0");
    const int n_ptrs = batch / mats_per_ptr;
    for (int i = 0; i < n_ptrs; ++i) xp.push_back((uint64_t)(uintptr_t)(base + (size_t)(4 + i) * gap));
    ps = {xp.data(), x_dtype, n_ptrs, mats_per_ptr, (const float*)(base + 3 * gap), 1.0f, nullptr, 0.0f, 0};
  }
  if (int rc = ns_build(in, in_dtype, fused ? nullptr : out, batch, rows, cols, coeffs, n_iters, 1.0f, 0.0f, flags,
                        gram_reset, small ? nullptr : ws, ws_bytes, fused ? &ps : nullptr, call, sumsq,
                        sumsq_blocks))
    return rc;
  if (audit_ws_bytes > 0 && call.ws_lo) call.ws_hi = call.ws_lo + audit_ws_bytes;
  if (int rc = ns_audit(call)) return rc;
  return call.n_steps;
}

extern "C" int dion_ns_plan_audit(int batch, int rows, int cols, int in_dtype, int n_iters, int flags,
                                  int gram_reset, int with_update, int x_dtype, int mats_per_ptr,
                                  size_t audit_ws_bytes) {
  return plan_audit(batch, rows, cols, in_dtype, n_iters, flags, gram_reset, with_update, x_dtype, mats_per_ptr,
                    audit_ws_bytes, false);
}

extern "C" int dion_ns_plan_audit_prepared(int batch, int rows, int cols, int n_iters, int flags, int gram_reset,
                                           int with_update, int x_dtype, int mats_per_ptr,
                                           size_t audit_ws_bytes) {
  return plan_audit(batch, rows, cols, DION_BF16, n_iters, flags, gram_reset, with_update, x_dtype, mats_per_ptr,
                    audit_ws_bytes, true);
}

// ---------------------------------------------------------------------------------------------
// Memory-bound kernels
// ---------------------------------------------------------------------------------------------
static bool table_aligned(const uint64_t* t, int n) {
  for (int i = 0; i < n; ++i)
    if (!aligned16(t[i])) return false;
  return true;
}

// Pointers per launch when every pointer covers mats_per_ptr matrices and the launch puts one
// matrix on each gridDim.y slot (at most 65535); 0 if even one pointer is too many.
static int ptr_chunk(int mats_per_ptr) {
  const int c = 65535 / mats_per_ptr;
  return c < kMaxPtrs ? c : kMaxPtrs;
}


static void fill_tab(PtrTab& tab, const uint64_t* src, int n) {
  memset(&tab, 0, sizeof(tab));
  memcpy(tab.p, src, (size_t)n * sizeof(uint64_t));
}

extern "C" int dion_muon_pre(const uint64_t* G_ptrs, int g_dtype, const uint64_t* M_ptrs, int m_dtype,
                             void* U, int n, int64_t numel, float mu, int nesterov, void* stream) {
  if (n < 0 || numel < 0) return fail(DION_E_INVALID, "dion_muon_pre: negative size");
  if (int rc = check_state_dtype("dion_muon_pre", "m_dtype", m_dtype)) return rc;
  if (g_dtype != DION_BF16 && g_dtype != DION_F32) return fail(DION_E_INVALID, "dion_muon_pre: g_dtype");
  if (n == 0 || numel == 0) return DION_OK;
  if (!G_ptrs || !M_ptrs || !U) return fail(DION_E_INVALID, "dion_muon_pre: null argument");
  const bool vec = (numel % 8 == 0) && table_aligned(G_ptrs, n) && table_aligned(M_ptrs, n) &&
                   aligned16((uint64_t)U);
  for (int i0 = 0; i0 < n; i0 += kMaxPtrs) {
    const int c = (n - i0) < kMaxPtrs ? (n - i0) : kMaxPtrs;
    PtrTab g, m;
    fill_tab(g, G_ptrs + i0, c);
    fill_tab(m, M_ptrs + i0, c);
    HIP_TRY(launch_muon_pre(g, dt(g_dtype), m, dt(m_dtype), (bf16_t*)U + (int64_t)i0 * numel, c, numel, mu,
                            nesterov, vec, (hipStream_t)stream),
            "dion_muon_pre");
  }
  return DION_OK;
}

extern "C" int dion_muon_pre_sumsq_blocks(int rows, int cols) {
  if (rows <= 0 || cols <= 0 || ((int64_t)rows * cols) % 4096 || rows % 64 || cols % 64) return 0;
  const int64_t b = (int64_t)rows * cols / 4096;
  return b > 0x7fffffff ? 0 : (int)b;
}

extern "C" int dion_muon_pre_prepared(const uint64_t* G_ptrs, int g_dtype, const uint64_t* M_ptrs, int m_dtype,
                                      void* U, float* sumsq, int n, int mats_per_ptr, int rows, int cols, float mu,
                                      int nesterov, void* stream) {
  if (n < 0 || mats_per_ptr <= 0 || rows < 0 || cols < 0)
    return fail(DION_E_INVALID, "dion_muon_pre_prepared: bad size");
  if (int rc = check_state_dtype("dion_muon_pre_prepared", "m_dtype", m_dtype)) return rc;
  if (g_dtype != DION_BF16 && g_dtype != DION_F32) return fail(DION_E_INVALID, "dion_muon_pre_prepared: g_dtype");
  if (n == 0 || rows == 0 || cols == 0) return DION_OK;
  if (!G_ptrs || !M_ptrs || !U || !sumsq) return fail(DION_E_INVALID, "dion_muon_pre_prepared: null argument");
  const int blocks = dion_muon_pre_sumsq_blocks(rows, cols);
  if (blocks == 0)
    return fail(DION_E_INVALID, "dion_muon_pre_prepared: rows and cols (%d, %d) must be multiples of 64", rows, cols);
  const int64_t mat = (int64_t)rows * cols;
  if ((int64_t)mats_per_ptr * blocks > 0x7fffffff || (int64_t)n * mats_per_ptr > 0x7fffffff)
    return fail(DION_E_INVALID, "dion_muon_pre_prepared: too many matrices per parameter");
  if (!table_aligned(G_ptrs, n) || !table_aligned(M_ptrs, n) || !aligned16((uint64_t)U))
    return fail(DION_E_INVALID, "dion_muon_pre_prepared: pointers must be 16-byte aligned");
  const int chunk = ptr_chunk(mats_per_ptr);
  if (chunk == 0) return fail(DION_E_INVALID, "dion_muon_pre_prepared: mats_per_ptr %d > 65535", mats_per_ptr);
  for (int c0 = 0; c0 < n; c0 += chunk) {
    const int c = (n - c0) < chunk ? (n - c0) : chunk;
    PtrTab G, M;
    fill_tab(G, G_ptrs + c0, c);
    fill_tab(M, M_ptrs + c0, c);
    const int64_t first = (int64_t)c0 * mats_per_ptr;
    HIP_TRY(launch_muon_pre_prepared(G, dt(g_dtype), M, dt(m_dtype), (bf16_t*)U + first * mat,
                                     sumsq + first * blocks, c, mats_per_ptr, rows, cols, mu, nesterov,
                                     (hipStream_t)stream),
            "dion_muon_pre_prepared");
  }
  return DION_OK;
}

extern "C" int dion_muon_post(const uint64_t* X_ptrs, int x_dtype, const void* U, int u_dtype, int n,
                              int64_t numel, int cols, const float* row_scale, const float* lr_dev,
                              const float* adj_lr_dev, float adj_ratio, const float* wd_dev, float wd_host,
                              int cautious, void* stream) {
  if (n < 0 || numel < 0 || cols <= 0) return fail(DION_E_INVALID, "dion_muon_post: bad size");
  if (int rc = check_state_dtype("dion_muon_post", "x_dtype", x_dtype)) return rc;
  if (u_dtype != DION_BF16 && u_dtype != DION_F32) return fail(DION_E_INVALID, "dion_muon_post: u_dtype");
  if (n == 0 || numel == 0) return DION_OK;
  if (numel % cols) return fail(DION_E_INVALID, "dion_muon_post: numel %% cols != 0");
  if (!X_ptrs || !U || !lr_dev) return fail(DION_E_INVALID, "dion_muon_post: null argument");
  const size_t usz = u_dtype == DION_BF16 ? 2 : 4;
  const bool vec = (numel % 8 == 0) && (cols % 8 == 0) && table_aligned(X_ptrs, n) &&
                   aligned16((uint64_t)U);
  const int64_t rows = numel / cols;
  for (int i0 = 0; i0 < n; i0 += kMaxPtrs) {
    const int c = (n - i0) < kMaxPtrs ? (n - i0) : kMaxPtrs;
    PtrTab x;
    fill_tab(x, X_ptrs + i0, c);
    HIP_TRY(launch_muon_post(x, dt(x_dtype), (const char*)U + (size_t)i0 * numel * usz, dt(u_dtype), c, numel,
                             cols,
                             row_scale ? row_scale + (int64_t)i0 * rows : nullptr, lr_dev, adj_lr_dev,
                             adj_ratio, wd_dev, wd_host, cautious, vec, (hipStream_t)stream),
            "dion_muon_post");
  }
  return DION_OK;
}

extern "C" int dion_scale_rows(const void* U, const float* scale, void* out, int out_dtype, int64_t n_rows,
                               int cols, void* stream) {
  if (int rc = check_state_dtype("dion_scale_rows", "out_dtype", out_dtype)) return rc;
  if (n_rows < 0 || cols < 0 || n_rows > 0x7fffffff) return fail(DION_E_INVALID, "dion_scale_rows: bad size");
  if (n_rows == 0 || cols == 0) return DION_OK;
  if (!U || !scale || !out) return fail(DION_E_INVALID, "dion_scale_rows: null argument");
  HIP_TRY(launch_scale_rows((const bf16_t*)U, scale, out, dt(out_dtype), n_rows, cols, (hipStream_t)stream),
          "dion_scale_rows");
  return DION_OK;
}

static int normuon_stats_impl(const char* who, const void* U, const uint64_t* V_ptrs, int v_dtype, int n,
                              int mats_per_ptr, int rows, int cols, const int32_t* row_idx, int v_rows,
                              float beta2, float* row_scale, void* stream) {
  if (int rc = check_state_dtype(who, "v_dtype", v_dtype)) return rc;
  if (n < 0 || mats_per_ptr <= 0 || rows < 0 || cols < 0 || v_rows < rows)
    return fail(DION_E_INVALID, "%s: bad size", who);
  if (n == 0 || rows == 0 || cols == 0) return DION_OK;
  if (!U || !V_ptrs || !row_scale) return fail(DION_E_INVALID, "%s: null argument", who);
  const float w = 1.0f - beta2;
  const int cmax = ptr_chunk(mats_per_ptr);  // matrices of one launch sit on gridDim.y
  if (cmax == 0) return fail(DION_E_INVALID, "more than 65535 matrices behind one pointer");
  for (int i0 = 0; i0 < n; i0 += cmax) {
    const int c = (n - i0) < cmax ? (n - i0) : cmax;
    PtrTab v;
    fill_tab(v, V_ptrs + i0, c);
    const int64_t mat0 = (int64_t)i0 * mats_per_ptr;
    HIP_TRY(launch_normuon_stats((const bf16_t*)U + mat0 * rows * cols, v, dt(v_dtype), c * mats_per_ptr,
                                 mats_per_ptr, rows, cols, row_idx ? row_idx + mat0 * rows : nullptr,
                                 v_rows, w, row_scale + mat0 * rows, (hipStream_t)stream),
            who);
  }
  return DION_OK;
}

extern "C" int dion_normuon_stats(const void* U, const uint64_t* V_ptrs, int v_dtype, int n,
                                  int mats_per_ptr, int rows, int cols, float beta2, float* row_scale,
                                  void* stream) {
  return normuon_stats_impl("dion_normuon_stats", U, V_ptrs, v_dtype, n, mats_per_ptr, rows, cols, nullptr, rows,
                            beta2, row_scale, stream);
}

extern "C" int dion_normuon_stats_selected(const void* U, const uint64_t* V_ptrs, int v_dtype, int n,
                                           int mats_per_ptr, int k, int cols, const int32_t* row_idx,
                                           int v_rows, float beta2, float* row_scale, void* stream) {
  if (!row_idx) return fail(DION_E_INVALID, "dion_normuon_stats_selected: null row_idx");
  return normuon_stats_impl("dion_normuon_stats_selected", U, V_ptrs, v_dtype, n, mats_per_ptr, k, cols, row_idx,
                            v_rows, beta2, row_scale, stream);
}

static int check_select_dim(const char* who, int select_dim) {
  if (select_dim != -2 && select_dim != -1)
    return fail(DION_E_INVALID, "%s: select_dim must be -2 or -1, got %d", who, select_dim);
  return DION_OK;
}

extern "C" size_t dion_dion2_accumulate_scratch_bytes(int n_mat, int rows, int cols, int select_dim) {
  if (select_dim != -1 || n_mat <= 0 || rows <= 0 || cols <= 0 || cols % 4 != 0) return 0;
  const int slabs = dion2_acc_slabs(n_mat, rows, cols);
  return slabs > 1 ? (size_t)slabs * n_mat * cols * sizeof(float) : 0;
}

extern "C" int dion_dion2_accumulate(const uint64_t* G_ptrs, int g_dtype, const uint64_t* M_ptrs,
                                     int m_dtype, int n, int mats_per_ptr, int rows, int cols, int select_dim,
                                     float* norms, void* scratch, size_t scratch_bytes,
                                     void* stream) {
  if (int rc = check_select_dim("dion_dion2_accumulate", select_dim)) return rc;
  if (int rc = check_state_dtype("dion_dion2_accumulate", "m_dtype", m_dtype)) return rc;
  if (n < 0 || mats_per_ptr <= 0 || rows < 0 || cols < 0)
    return fail(DION_E_INVALID, "dion_dion2_accumulate: bad size");
  if (g_dtype != DION_BF16 && g_dtype != DION_F32)
    return fail(DION_E_INVALID, "dion_dion2_accumulate: g_dtype");
  if (n == 0 || rows == 0 || cols == 0) return DION_OK;
  if (!G_ptrs || !M_ptrs || !norms) return fail(DION_E_INVALID, "dion_dion2_accumulate: null argument");
  const int dim = select_dim == -2 ? rows : cols;
  // 16-byte accesses need 4-column alignment of every row of every matrix
  const bool vec4 = (cols % 4 == 0) && table_aligned(G_ptrs, n) && table_aligned(M_ptrs, n) &&
                    aligned16((uint64_t)norms);
  // Row slabs (column sums only): sized for the whole group, used if the scratch holds them.
  int slabs = 1;
  if (select_dim == -1 && vec4 && scratch && aligned16((uint64_t)scratch)) {
    const int64_t n_mat = (int64_t)n * mats_per_ptr;
    slabs = dion2_acc_slabs((int)n_mat, rows, cols);
    if ((size_t)slabs * n_mat * cols * sizeof(float) > scratch_bytes) slabs = 1;
  }
  const int cmax = ptr_chunk(mats_per_ptr);  // matrices of one launch sit on gridDim.y
  if (cmax == 0) return fail(DION_E_INVALID, "more than 65535 matrices behind one pointer");
  for (int i0 = 0; i0 < n; i0 += cmax) {
    const int c = (n - i0) < cmax ? (n - i0) : cmax;
    PtrTab g, m;
    fill_tab(g, G_ptrs + i0, c);
    fill_tab(m, M_ptrs + i0, c);
    HIP_TRY(launch_dion2_accumulate(g, dt(g_dtype), m, dt(m_dtype), c * mats_per_ptr, mats_per_ptr, rows, cols,
                                    select_dim == -2, norms + (int64_t)i0 * mats_per_ptr * dim, vec4,
                                    slabs > 1 ? (float*)scratch : nullptr, slabs,
                                    (hipStream_t)stream),
            "dion_dion2_accumulate");
  }
  return DION_OK;
}

extern "C" int dion_dion2_topk(const float* norms, int n_mat, int dim, int k, int32_t* idx,
                               int32_t* map, void* stream) {
  if (n_mat < 0 || dim < 0 || k < 0 || k > dim) return fail(DION_E_INVALID, "dion_dion2_topk: bad size");
  if (n_mat == 0 || dim == 0) return DION_OK;
  if (!norms || !idx || !map) return fail(DION_E_INVALID, "dion_dion2_topk: null argument");
  for (int m0 = 0; m0 < n_mat; m0 += 65535) {  // one matrix per gridDim.y slot
    const int c = (n_mat - m0) < 65535 ? (n_mat - m0) : 65535;
    HIP_TRY(launch_dion2_topk(norms + (int64_t)m0 * dim, c, dim, k, idx + (int64_t)m0 * k,
                              map + (int64_t)m0 * dim, (hipStream_t)stream),
            "dion_dion2_topk");
  }
  return DION_OK;
}

extern "C" int dion_dion2_gather(const uint64_t* M_ptrs, int m_dtype, int n, int mats_per_ptr, int rows, int cols,
                                 int select_dim, const int32_t* idx, int k, float ef_decay,
                                 void* U_sel, void* stream) {
  if (int rc = check_select_dim("dion_dion2_gather", select_dim)) return rc;
  if (int rc = check_state_dtype("dion_dion2_gather", "m_dtype", m_dtype)) return rc;
  if (n < 0 || mats_per_ptr <= 0 || rows < 0 || cols < 0 || k < 0)
    return fail(DION_E_INVALID, "dion_dion2_gather: bad size");
  if (n == 0 || rows == 0 || cols == 0 || k == 0) return DION_OK;
  if (!M_ptrs || !idx || !U_sel) return fail(DION_E_INVALID, "dion_dion2_gather: null argument");
  const int64_t sel_numel = select_dim == -2 ? (int64_t)k * cols : (int64_t)rows * k;
  const bool vec4 = (cols % 4 == 0) && table_aligned(M_ptrs, n) && aligned16((uint64_t)U_sel);
  const int cmax = ptr_chunk(mats_per_ptr);  // matrices of one launch sit on gridDim.y
  if (cmax == 0) return fail(DION_E_INVALID, "more than 65535 matrices behind one pointer");
  for (int i0 = 0; i0 < n; i0 += cmax) {
    const int c = (n - i0) < cmax ? (n - i0) : cmax;
    PtrTab m;
    fill_tab(m, M_ptrs + i0, c);
    const int64_t mat0 = (int64_t)i0 * mats_per_ptr;
    HIP_TRY(launch_dion2_gather(m, dt(m_dtype), c * mats_per_ptr, mats_per_ptr, rows, cols, select_dim == -2,
                                idx + mat0 * k, k, ef_decay, (bf16_t*)U_sel + mat0 * sel_numel, vec4,
                                (hipStream_t)stream),
            "dion_dion2_gather");
  }
  return DION_OK;
}

extern "C" int dion_dion2_gather_sumsq_blocks(int rows, int cols, int select_dim, int k) {
  if (rows <= 0 || cols <= 0 || k <= 0 || (select_dim != -2 && select_dim != -1)) return 0;
  if (select_dim == -2) return (k <= rows && k <= cols) ? k : 0;  // [k, cols] as it lies; a tall block is not taken
  if (k > cols) return 0;
  if (rows <= k) return rows;                                      // [rows, k] as it lies
  if (rows % 64 || k % 64) return 0;
  const int64_t b = (int64_t)(rows / 64) * (k / 64);              // [k, rows], transposed through 64 x 64 tiles
  return b > 0x7fffffff ? 0 : (int)b;
}

extern "C" int dion_dion2_gather_prepared(const uint64_t* M_ptrs, int m_dtype, int n, int mats_per_ptr, int rows,
                                          int cols, int select_dim, const int32_t* idx, int k, float ef_decay,
                                          void* U_sel, float* sumsq, void* stream) {
  if (int rc = check_select_dim("dion_dion2_gather_prepared", select_dim)) return rc;
  if (int rc = check_state_dtype("dion_dion2_gather_prepared", "m_dtype", m_dtype)) return rc;
  if (n < 0 || mats_per_ptr <= 0 || rows < 0 || cols < 0 || k < 0)
    return fail(DION_E_INVALID, "dion_dion2_gather_prepared: bad size");
  if (n == 0 || rows == 0 || cols == 0 || k == 0) return DION_OK;
  if (!M_ptrs || !idx || !U_sel || !sumsq) return fail(DION_E_INVALID, "dion_dion2_gather_prepared: null argument");
  const int blocks = dion_dion2_gather_sumsq_blocks(rows, cols, select_dim, k);
  if (blocks == 0)
    return fail(DION_E_INVALID, "dion_dion2_gather_prepared: %d of %d x %d along dim %d has no prepared form "
                "(see dion_dion2_gather_sumsq_blocks)", k, rows, cols, select_dim);
  if (!aligned16((uint64_t)U_sel))
    return fail(DION_E_INVALID, "dion_dion2_gather_prepared: U_sel is not 16-byte aligned");
  const int64_t sel_numel = select_dim == -2 ? (int64_t)k * cols : (int64_t)rows * k;
  const bool vec4 = (cols % 4 == 0) && table_aligned(M_ptrs, n);
  const int cmax = ptr_chunk(mats_per_ptr);
  if (cmax == 0) return fail(DION_E_INVALID, "more than 65535 matrices behind one pointer");
  for (int i0 = 0; i0 < n; i0 += cmax) {
    const int c = (n - i0) < cmax ? (n - i0) : cmax;
    PtrTab m;
    fill_tab(m, M_ptrs + i0, c);
    const int64_t mat0 = (int64_t)i0 * mats_per_ptr;
    HIP_TRY(launch_dion2_gather_prepared(m, dt(m_dtype), c * mats_per_ptr, mats_per_ptr, rows, cols,
                                         select_dim == -2, idx + mat0 * k, k, ef_decay,
                                         (bf16_t*)U_sel + mat0 * sel_numel, sumsq + mat0 * blocks, vec4,
                                         (hipStream_t)stream),
            "dion_dion2_gather_prepared");
  }
  return DION_OK;
}

extern "C" int dion_dion2_post(const uint64_t* X_ptrs, int x_dtype, int n, int mats_per_ptr, int rows, int cols,
                               int select_dim, const void* U_sel, int u_dtype, int k, const int32_t* map,
                               const float* row_scale, const float* lr_dev, const float* adj_lr_dev,
                               float adj_ratio, const float* wd_dev, float wd_host, void* stream) {
  if (int rc = check_select_dim("dion_dion2_post", select_dim)) return rc;
  if (int rc = check_state_dtype("dion_dion2_post", "x_dtype", x_dtype)) return rc;
  if (u_dtype != DION_BF16 && u_dtype != DION_F32) return fail(DION_E_INVALID, "dion_dion2_post: u_dtype");
  if (row_scale && select_dim != -2)
    return fail(DION_E_INVALID, "dion_dion2_post: row_scale needs select_dim == -2");
  if (n < 0 || mats_per_ptr <= 0 || rows < 0 || cols < 0 || k < 0)
    return fail(DION_E_INVALID, "dion_dion2_post: bad size");
  if (n == 0 || rows == 0 || cols == 0) return DION_OK;
  if (!X_ptrs || !map || !lr_dev || (k > 0 && !U_sel))
    return fail(DION_E_INVALID, "dion_dion2_post: null argument");
  const int dim = select_dim == -2 ? rows : cols;
  const int64_t sel_numel = select_dim == -2 ? (int64_t)k * cols : (int64_t)rows * k;
  const int es = u_dtype == DION_BF16 ? 2 : 4;
  const bool vec4 = (cols % 4 == 0) && table_aligned(X_ptrs, n) && aligned16((uint64_t)U_sel) &&
                    aligned16((uint64_t)map);
  const int cmax = ptr_chunk(mats_per_ptr);  // matrices of one launch sit on gridDim.y
  if (cmax == 0) return fail(DION_E_INVALID, "more than 65535 matrices behind one pointer");
  for (int i0 = 0; i0 < n; i0 += cmax) {
    const int c = (n - i0) < cmax ? (n - i0) : cmax;
    PtrTab x;
    fill_tab(x, X_ptrs + i0, c);
    const int64_t mat0 = (int64_t)i0 * mats_per_ptr;
    HIP_TRY(launch_dion2_post(x, dt(x_dtype), c * mats_per_ptr, mats_per_ptr, rows, cols, select_dim == -2,
                              (const char*)U_sel + mat0 * sel_numel * es, u_dtype == DION_BF16 ? 0 : 1, k,
                              map + mat0 * dim, row_scale ? row_scale + mat0 * k : nullptr, lr_dev,
                              adj_lr_dev, adj_ratio, wd_dev, wd_host, vec4, (hipStream_t)stream),
            "dion_dion2_post");
  }
  return DION_OK;
}

extern "C" int dion_dion2_index_map(const int64_t* idx, int n_mat, int k, int dim, int32_t* map,
                                    void* stream) {
  if (n_mat < 0 || k < 0 || dim < 0 || k > dim) return fail(DION_E_INVALID, "dion_dion2_index_map: bad size");
  if (n_mat == 0 || dim == 0) return DION_OK;
  if (!map || (k > 0 && !idx)) return fail(DION_E_INVALID, "dion_dion2_index_map: null argument");
  HIP_TRY(launch_dion2_index_map(idx, n_mat, k, dim, map, (hipStream_t)stream), "dion_dion2_index_map");
  return DION_OK;
}

// ---------------------------------------------------------------------------------------------
// Whole-matrix selection: the sequence a rank runs on assembled matrices under
// selection_scope="global" (dion/dion2.py:301-343, 565-659; dion/nordion2.py:291-335, 448-500)
// ---------------------------------------------------------------------------------------------
static int check_stacked(const char* who, int dtype, int n_mat, int rows, int cols, int select_dim) {
  if (int rc = check_select_dim(who, select_dim)) return rc;
  if (dtype != DION_BF16 && dtype != DION_F32) return fail(DION_E_INVALID, "%s: dtype", who);
  if (n_mat < 0 || rows < 0 || cols < 0) return fail(DION_E_INVALID, "%s: bad size", who);
  if (n_mat > 65535) return fail(DION_E_INVALID, "%s: more than 65535 matrices in one call", who);
  return DION_OK;
}

extern "C" int dion_slice_l1(const void* U, int dtype, int n_mat, int rows, int cols, int select_dim,
                             int round_bf16, float* norms, void* stream) {
  if (int rc = check_stacked("dion_slice_l1", dtype, n_mat, rows, cols, select_dim)) return rc;
  const int dim = select_dim == -2 ? rows : cols;
  if (n_mat == 0 || dim == 0) return DION_OK;
  if (!norms) return fail(DION_E_INVALID, "dion_slice_l1: null argument");
  // empty slices (rows or cols == 0 on the other side) still launch: every norm comes out 0
  if (!U && rows > 0 && cols > 0) return fail(DION_E_INVALID, "dion_slice_l1: null argument");
  HIP_TRY(launch_slice_l1(U, dtype, n_mat, rows, cols, select_dim == -2, round_bf16, norms,
                          (hipStream_t)stream),
          "dion_slice_l1");
  return DION_OK;
}

extern "C" int dion_gather_slices(const void* U, int dtype, int n_mat, int rows, int cols, int select_dim,
                                  const int32_t* idx, int k, void* sub, void* stream) {
  if (int rc = check_stacked("dion_gather_slices", dtype, n_mat, rows, cols, select_dim)) return rc;
  const int dim = select_dim == -2 ? rows : cols;
  if (k < 0 || k > dim) return fail(DION_E_INVALID, "dion_gather_slices: k outside [0, dim]");
  if (n_mat == 0 || rows == 0 || cols == 0 || k == 0) return DION_OK;
  if (!U || !idx || !sub) return fail(DION_E_INVALID, "dion_gather_slices: null argument");
  HIP_TRY(launch_gather_slices(U, dtype, n_mat, rows, cols, select_dim == -2, idx, k, sub,
                               (hipStream_t)stream),
          "dion_gather_slices");
  return DION_OK;
}

extern "C" int dion_scatter_slices(const void* sub, int dtype, int n_mat, int rows, int cols,
                                   int select_dim, const int32_t* map, int k, void* out, void* stream) {
  if (int rc = check_stacked("dion_scatter_slices", dtype, n_mat, rows, cols, select_dim)) return rc;
  const int dim = select_dim == -2 ? rows : cols;
  if (k < 0 || k > dim) return fail(DION_E_INVALID, "dion_scatter_slices: k outside [0, dim]");
  if (n_mat == 0 || rows == 0 || cols == 0) return DION_OK;
  if (!map || !out || (k > 0 && !sub)) return fail(DION_E_INVALID, "dion_scatter_slices: null argument");
  HIP_TRY(launch_scatter_slices(sub, dtype, n_mat, rows, cols, select_dim == -2, map, k, out,
                                (hipStream_t)stream),
          "dion_scatter_slices");
  return DION_OK;
}

extern "C" int dion_mask_index(const float* norms, int n_mat, int dim, int32_t* gate, void* stream) {
  if (n_mat < 0 || dim < 0) return fail(DION_E_INVALID, "dion_mask_index: bad size");
  if (n_mat == 0 || dim == 0) return DION_OK;
  if (!norms || !gate) return fail(DION_E_INVALID, "dion_mask_index: null argument");
  HIP_TRY(launch_mask_index(norms, n_mat, dim, gate, (hipStream_t)stream), "dion_mask_index");
  return DION_OK;
}

extern "C" int dion_dion2_post_masked(const uint64_t* X_ptrs, const uint64_t* M_ptrs, int s_dtype, int n,
                                      int mats_per_ptr, int rows, int cols, int select_dim,
                                      const void* U, const float* norms, const float* row_scale,
                                      const float* lr_dev, const float* adj_lr_dev, float adj_ratio,
                                      const float* wd_dev, float wd_host, float ef_decay, void* stream) {
  if (int rc = check_select_dim("dion_dion2_post_masked", select_dim)) return rc;
  if (int rc = check_state_dtype("dion_dion2_post_masked", "s_dtype", s_dtype)) return rc;
  if (row_scale && select_dim != -2)
    return fail(DION_E_INVALID, "dion_dion2_post_masked: row_scale needs select_dim == -2");
  if (n < 0 || mats_per_ptr <= 0 || rows < 0 || cols < 0)
    return fail(DION_E_INVALID, "dion_dion2_post_masked: bad size");
  if (n == 0 || rows == 0 || cols == 0) return DION_OK;
  if (!X_ptrs || !M_ptrs || !U || !norms || !lr_dev)
    return fail(DION_E_INVALID, "dion_dion2_post_masked: null argument");
  for (int i = 0; i < n; ++i)
    if (!X_ptrs[i] || !M_ptrs[i])
      return fail(DION_E_INVALID, "dion_dion2_post_masked: tensor %d has a null pointer", i);
  const int dim = select_dim == -2 ? rows : cols;
  const bool vec4 = (cols % 4 == 0) && table_aligned(X_ptrs, n) && table_aligned(M_ptrs, n) &&
                    aligned16((uint64_t)U) && aligned16((uint64_t)norms);
  const int cmax = ptr_chunk(mats_per_ptr);  // matrices of one launch sit on gridDim.y
  if (cmax == 0) return fail(DION_E_INVALID, "more than 65535 matrices behind one pointer");
  for (int i0 = 0; i0 < n; i0 += cmax) {
    const int c = (n - i0) < cmax ? (n - i0) : cmax;
    PtrTab x, m;
    fill_tab(x, X_ptrs + i0, c);
    fill_tab(m, M_ptrs + i0, c);
    const int64_t mat0 = (int64_t)i0 * mats_per_ptr;
    HIP_TRY(launch_dion2_post_masked(x, m, dt(s_dtype), c * mats_per_ptr, mats_per_ptr, rows, cols,
                                     select_dim == -2,
                                     (const bf16_t*)U + mat0 * rows * cols, norms + mat0 * dim,
                                     row_scale ? row_scale + mat0 * rows : nullptr, lr_dev, adj_lr_dev,
                                     adj_ratio, wd_dev, wd_host, ef_decay, vec4, (hipStream_t)stream),
            "dion_dion2_post_masked");
  }
  return DION_OK;
}

// ---------------------------------------------------------------------------------------------
// Multi-tensor AdamW / Lion for the non-matrix parameter groups
// ---------------------------------------------------------------------------------------------
static int check_mta(const char* who, const uint64_t* X, const uint64_t* G, int g_dtype, const uint64_t* M,
                     const int64_t* numels, int n, const float* lr_dev) {
  if (n < 0) return fail(DION_E_INVALID, "%s: negative count", who);
  if (g_dtype != DION_BF16 && g_dtype != DION_F32) return fail(DION_E_INVALID, "%s: g_dtype", who);
  if (n == 0) return DION_OK;
  if (!X || !G || !M || !numels || !lr_dev) return fail(DION_E_INVALID, "%s: null argument", who);
  for (int i = 0; i < n; ++i)
    if (numels[i] < 0 || (numels[i] > 0 && (!X[i] || !G[i] || !M[i])))
      return fail(DION_E_INVALID, "%s: tensor %d has a null pointer or a negative size", who, i);
  return DION_OK;
}

extern "C" int dion_adamw_step(const uint64_t* X_ptrs, const uint64_t* G_ptrs, int g_dtype,
                               const uint64_t* M_ptrs, const uint64_t* V_ptrs, int s_dtype,
                               const uint64_t* step_ptrs, const int64_t* numels, int n,
                               const float* lr_dev, float beta1, float beta2, float eps,
                               const float* wd_dev, float wd_host, int cautious, void* stream) {
  if (int rc = check_state_dtype("dion_adamw_step", "s_dtype", s_dtype)) return rc;
  if (int rc = check_mta("dion_adamw_step", X_ptrs, G_ptrs, g_dtype, M_ptrs, numels, n, lr_dev)) return rc;
  if (n == 0) return DION_OK;
  if (!V_ptrs || !step_ptrs) return fail(DION_E_INVALID, "dion_adamw_step: null argument");
  for (int i = 0; i < n; ++i)
    if (!step_ptrs[i] || (numels[i] > 0 && !V_ptrs[i]))
      return fail(DION_E_INVALID, "dion_adamw_step: tensor %d has a null state pointer", i);
  // One step counter may serve several tensors; a counter shared ACROSS launch chunks would be
  // advanced once per chunk, so every chunk must own its counters.
  for (int i0 = 0; i0 < n; i0 += kMtaTensors) {
    const int c = (n - i0) < kMtaTensors ? (n - i0) : kMtaTensors;
    for (int i = i0; i < i0 + c; ++i)
      for (int j = 0; j < i0; ++j)
        if (step_ptrs[i] == step_ptrs[j])
          return fail(DION_E_INVALID,
                      "dion_adamw_step: step counter of tensor %d is shared with tensor %d of an earlier "
                      "chunk of %d tensors",
                      i, j, kMtaTensors);
    HIP_TRY(launch_adamw_mt(X_ptrs + i0, G_ptrs + i0, dt(g_dtype), M_ptrs + i0, V_ptrs + i0, dt(s_dtype),
                            step_ptrs + i0,
                            numels + i0, c, lr_dev, beta1, beta2, eps, wd_dev, wd_host, cautious,
                            (hipStream_t)stream),
            "dion_adamw_step");
  }
  return DION_OK;
}

extern "C" int dion_lion_step(const uint64_t* X_ptrs, const uint64_t* G_ptrs, int g_dtype,
                              const uint64_t* M_ptrs, int s_dtype, const int64_t* numels, int n,
                              const float* lr_dev,
                              float beta1, float beta2, const float* wd_dev, float wd_host, int cautious,
                              void* stream) {
  if (int rc = check_state_dtype("dion_lion_step", "s_dtype", s_dtype)) return rc;
  if (int rc = check_mta("dion_lion_step", X_ptrs, G_ptrs, g_dtype, M_ptrs, numels, n, lr_dev)) return rc;
  for (int i0 = 0; i0 < n; i0 += kMtaTensors) {
    const int c = (n - i0) < kMtaTensors ? (n - i0) : kMtaTensors;
    HIP_TRY(launch_lion_mt(X_ptrs + i0, G_ptrs + i0, dt(g_dtype), M_ptrs + i0, dt(s_dtype), numels + i0, c,
                           lr_dev, beta1,
                           beta2, wd_dev, wd_host, cautious, (hipStream_t)stream),
            "dion_lion_step");
  }
  return DION_OK;
}
