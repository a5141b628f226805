/*
 * dion_hip.h -- C ABI of libdion_hip.so: the MI355X (gfx950) kernels behind the Muon / NorMuon /
 * Dion2 optimizer-step hot path of microsoft/dion.
 *
 * Conventions
 *   - Every pointer named *_dev / X / U / ... is a DEVICE pointer unless the comment says host.
 *   - bf16 data is passed as `const void*` / `void*` to raw bfloat16 bits; fp32 as float*.
 *   - `stream` is a hipStream_t passed as void* (NULL = default stream).  All work is enqueued on
 *     it; no entry point synchronises the host or allocates device memory.
 *   - Return value: 0 on success, otherwise a negative DION_E_* code; dion_last_error() returns a
 *     thread-local message for the last failure.
 *   - "ptr table": host array of `n` device pointers (uint64), one per parameter of a shape
 *     group, in the reference's List[Tensor] order.
 *
 * Each entry point cites the reference interface (file:line under the reference tree) it
 * replaces.
 */
#ifndef DION_HIP_H
#define DION_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define DION_OK 0
#define DION_E_INVALID (-1)   /* bad shape / size / flag */
#define DION_E_WORKSPACE (-2) /* workspace too small */
#define DION_E_HIP (-3)       /* HIP runtime error, see dion_last_error() */

/* dtype codes for inputs that may arrive in either precision */
#define DION_BF16 0
#define DION_F32 1

const char* dion_last_error(void);
/* Library ABI version (bumped when a signature changes). */
int dion_abi_version(void);

/* --------------------------------------------------------------------------------------------
 * Symmetric / polynomial GEMMs of one Newton-Schulz iteration (kernel-level API).
 * Operands are dense row-major bf16 batches; leading dimension == last extent.
 * Extents must be multiples of 128 (the Python layer pads; the full driver below pads itself),
 * operand and result pointers 16-byte aligned (DION_E_INVALID otherwise).
 * ------------------------------------------------------------------------------------------ */

/* A[b] = X[b] X[b]^T.  X [batch,m,k] -> A [batch,m,m]; only tiles on/above the diagonal are
 * computed, each also stored mirrored.  Replaces ns_line_1 (dion/newton_schulz_triton.py:160-203,
 * kernel :88-157). */
int dion_ns_line_1(const void* X, void* A, int batch, int m, int k, void* stream);

/* B[b] = alpha A[b] A[b]^T + beta A[b], A symmetric [batch,m,m].  Replaces ns_line_2
 * (dion/newton_schulz_triton.py:290-333, kernel :206-287). */
int dion_ns_line_2(const void* A, void* B, int batch, int m, float alpha, float beta, void* stream);

/* C[b] = a X[b] + B[b] X[b]: B [batch,m,m] symmetric, X and C [batch,m,n] (C != X).  X is read as
 * it lies (reduction index along rows; transposing LDS reads in the kernel), so no X^T is needed.
 * With a == 0 the addend is skipped altogether (X is read once).
 * Replaces ns_line_3 (dion/newton_schulz_triton.py:450-491) and the baddbmm at :557-563. */
int dion_ns_line_3(const void* B, const void* X, void* C, int batch, int m, int n, float a, void* stream);

/* --------------------------------------------------------------------------------------------
 * Whole orthogonalization: the operator behind `newton_schulz_func(input, epsilon)`
 * (dion/muon.py:47-48; implementations dion/newton_schulz_triton.py:494-522 and
 * dion/polar_express.py:20-50).
 *
 *   in   [batch, rows, cols]  bf16 or fp32 (in_dtype), dense
 *   out  [batch, rows, cols]  bf16, dense, 16-byte aligned (DION_E_INVALID otherwise; batches that take
 *        the LDS-resident small-matrix kernel are exempt)
 *   coeffs  host array of n_iters*3 floats (a,b,c per iteration)
 *   X0 = bf16(in) / (||bf16(in)||_F * norm_scale + eps)  per matrix, then n_iters times
 *   A = X X^T; B = b A + c A A; X = a X + B X   on the orientation with rows <= cols.
 *   (For matrices that fill whole GEMM tiles the division is not a pass of its own: the factor is applied
 *   in the fp32 epilogue of the first two GEMMs, and a wide bf16 `in` is read where it lies.)
 *   flags: DION_NS_GRAM selects the Gram-matrix recurrence (call site
 *   dion/megabatch_base.py:77-94) with a restart at iteration `gram_reset` (<=0: none).  Both forms
 *   apply the same polynomial; the recurrence only saves work for long matrices, so it is used
 *   when max(rows, cols) >= 3 min(rows, cols) and the standard iteration otherwise.
 * workspace: device scratch of at least dion_ns_workspace_bytes() bytes, 256-byte aligned.
 * Every launch of a call is checked on the host against the buffers the call owns (in, out,
 * workspace) before the first one is issued.
 * ------------------------------------------------------------------------------------------ */
#define DION_NS_GRAM 1
size_t dion_ns_workspace_bytes(int batch, int rows, int cols, int flags);
int dion_ns_orthogonalize(const void* in, int in_dtype, void* out, int batch, int rows, int cols,
                          const float* coeffs, int n_iters, float norm_scale, float eps, int flags,
                          int gram_reset, void* workspace, size_t workspace_bytes, void* stream);

/* dion_ns_orthogonalize without a workspace argument and without any allocation: the library's own
 * fixed device array (DION_NS_STATIC_SCRATCH_BYTES, part of the code object; every GPU the library
 * runs on holds one copy until the process ends) takes the workspace's place.  No counterpart in
 * the reference: it exists for callers that cannot allocate device memory or pass a workspace --
 * code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  Same
 * arguments, same kernels and bit-identical results as dion_ns_orthogonalize.  A problem whose
 * dion_ns_workspace_bytes() exceeds DION_NS_STATIC_SCRATCH_BYTES is refused with DION_E_WORKSPACE
 * (dion_last_error() names both sizes).  The array's device address is looked up on the first call
 * per device (hipGetSymbolAddress; make that first call outside a graph capture).  All calls on one
 * GPU share the array: calls that overlap in time on the same GPU (different streams or threads)
 * race; calls ordered on one stream are safe.  Nothing in the array needs to start at zero. */
#define DION_NS_STATIC_SCRATCH_BYTES (64u << 20)
int dion_ns_orthogonalize_static(const void* in, int in_dtype, void* out, int batch, int rows, int cols,
                                 const float* coeffs, int n_iters, float norm_scale, float eps, int flags,
                                 int gram_reset, void* stream);

/* Host-only self-check of the planning code (no device work, usable without a GPU): builds the launch
 * list of dion_ns_orthogonalize (with_update == 0) or of the fused form of
 * dion_ns_orthogonalize_update (with_update != 0; DION_E_INVALID if the shape does not fuse) over
 * synthetic, never dereferenced addresses and runs the bounds check every real call runs before
 * its first launch: each launch's reads inside the input or the workspace, its writes inside the
 * workspace, the output or one parameter, tile shapes dividing the padded extents.  Returns the
 * number of kernel launches, or a negative DION_E_* code (dion_last_error() names the launch and
 * the operand).  audit_ws_bytes > 0 checks against a workspace of that many bytes instead of the
 * size the plan was laid out for.  No counterpart in the reference. */
int dion_ns_plan_audit(int batch, int rows, int cols, int in_dtype, int n_iters, int flags, int gram_reset,
                       int with_update, int x_dtype, int mats_per_ptr, size_t audit_ws_bytes);

/* Orthogonalization and Muon update in one call: what dion_ns_orthogonalize followed by dion_muon_post
 * (bf16 update, no row_scale) does to the parameters, bit for bit, without the pass that writes the
 * orthogonalized matrices and the pass that reads them back.  Replaces the pair
 * `muon_update_newton_schulz` + `muon_update_post_orthogonalize`, dion/muon.py:249-277.
 * in: [n_ptrs * mats_per_ptr, rows, cols] as for dion_ns_orthogonalize; X_ptrs: host array of n_ptrs
 * device pointers, each to mats_per_ptr contiguous [rows, cols] matrices of x_dtype, updated in place.
 * When the matrices fill whole tiles (rows, cols multiples of 128; more than 64 rows or
 * columns on the short side) the last GEMM applies the update in its epilogue; otherwise the library
 * runs the two passes itself, through the tail of the workspace.  Workspace size from
 * dion_ns_update_workspace_bytes (same flags and n_iters).  lr / weight decay as for dion_muon_post. */
size_t dion_ns_update_workspace_bytes(int batch, int rows, int cols, int flags, int n_iters);
int dion_ns_orthogonalize_update(const void* in, int in_dtype, const uint64_t* X_ptrs, int x_dtype, int n_ptrs,
                                 int mats_per_ptr, int rows, int cols, const float* coeffs, int n_iters,
                                 float norm_scale, float eps, int flags, int gram_reset, const float* lr_dev,
                                 float adj_ratio, const float* wd_dev, float wd_host, int cautious,
                                 void* workspace, size_t workspace_bytes, void* stream);

/* --------------------------------------------------------------------------------------------
 * Orthogonalization of a "prepared" input: the producer of the input (dion_muon_pre_prepared) has
 * already written it in the layout the iteration carries -- bf16 [batch, min(rows, cols),
 * max(rows, cols)], short side along rows, i.e. a tall matrix transposed -- and has left partial
 * sums of its squares per matrix.  The Frobenius normalisation X0 = in / (||in||_F * norm_scale + eps)
 * (dion/polar_express.py:30-35, dion/newton_schulz_triton.py:508-513) then needs no pass over the
 * input: the factor rides on the first two GEMMs (A = s^2 in in^T, X' = s B in), computed on the
 * device from the partial sums.  rows / cols describe the caller's matrices (`out`, the
 * parameters), as in dion_ns_orthogonalize; all other arguments as there.
 *   in     bf16 [batch, m, n], m = min(rows, cols), n = max(rows, cols), 16-byte aligned
 *   sumsq  fp32 [batch, sumsq_blocks]; the sum of row b is ||in[b]||_F^2
 * Taken only when dion_ns_accepts_prepared() returns 1: rows and cols multiples of the GEMM tile
 * (no padding), rows * cols a multiple of 4096, at least one iteration, more than 64 rows or columns
 * on the short side, at most 65535 matrices; DION_E_INVALID otherwise (use dion_ns_orthogonalize).
 * Results differ from dion_ns_orthogonalize in the last bf16 bit (X0 is not rounded to bf16 once
 * more before the first products).
 * ------------------------------------------------------------------------------------------ */
int dion_ns_accepts_prepared(int batch, int rows, int cols, int flags, int n_iters);
int dion_ns_orthogonalize_prepared(const void* in, const float* sumsq, int sumsq_blocks, void* out, int batch,
                                   int rows, int cols, const float* coeffs, int n_iters, float norm_scale,
                                   float eps, int flags, int gram_reset, void* workspace,
                                   size_t workspace_bytes, void* stream);
/* dion_ns_orthogonalize_update on a prepared input (the update always rides on the last GEMM:
 * every shape that takes a prepared input fuses).  Workspace from dion_ns_update_workspace_bytes. */
int dion_ns_orthogonalize_update_prepared(const void* in, const float* sumsq, int sumsq_blocks,
                                          const uint64_t* X_ptrs, int x_dtype, int n_ptrs, int mats_per_ptr,
                                          int rows, int cols, const float* coeffs, int n_iters,
                                          float norm_scale, float eps, int flags, int gram_reset,
                                          const float* lr_dev, float adj_ratio, const float* wd_dev,
                                          float wd_host, int cautious, void* workspace,
                                          size_t workspace_bytes, void* stream);
/* dion_ns_plan_audit for the prepared form (host only, no device work). */
int dion_ns_plan_audit_prepared(int batch, int rows, int cols, int n_iters, int flags, int gram_reset,
                                int with_update, int x_dtype, int mats_per_ptr, size_t audit_ws_bytes);

/* Tile edge (128 or 256) the GEMM launcher picks for `batch` products of an m x n result
 * (symmetric != 0: an m x m symmetric product, upper tiles only).  Lets a benchmark count executed
 * FLOP with the library's own rule.  No counterpart in the reference. */
int dion_gemm_tile_edge(int batch, int m, int n, int symmetric);

/* --------------------------------------------------------------------------------------------
 * Memory-bound fused kernels of the optimizer step.
 * Optimizer state -- parameters X, momentum M, second moments V -- is fp32 or bf16 in memory, as the
 * reference keeps it in the parameter's dtype (dion/megabatch_base.py:198-203, dion/normuon.py:122):
 * every entry point that touches state takes its dtype (x_dtype / m_dtype / v_dtype / s_dtype,
 * DION_F32 or DION_BF16).  Arithmetic is fp32; a bf16 state value is rounded once, on store.
 * ------------------------------------------------------------------------------------------ */

/* Momentum update + orthogonalization input for one shape group.
 *   M_i = mu M_i + G_i;  U[i] = bf16(nesterov ? mu M_i + G_i : M_i)
 * G_ptrs / M_ptrs: host ptr tables of n device pointers, each to `numel` dense elements
 * (G bf16 or fp32 per g_dtype; M per m_dtype).  U: one dense [n, numel] bf16 arena.
 * Replaces muon_update_pre_orthogonalize (dion/muon.py:284-311) plus the torch.stack of
 * dion/megabatch_base.py:872. */
int dion_muon_pre(const uint64_t* G_ptrs, int g_dtype, const uint64_t* M_ptrs, int m_dtype, void* U,
                  int n, int64_t numel, float mu, int nesterov, void* stream);

/* dion_muon_pre for matrices that take a prepared orthogonalization input: same momentum update,
 * but U is written in the layout the iteration carries and the Frobenius norm's partial sums come
 * out of the same pass (they are in registers anyway).
 *   G_ptrs / M_ptrs: n pointers, each to mats_per_ptr dense [rows, cols] matrices
 *   U      bf16 [n * mats_per_ptr, min(rows, cols), max(rows, cols)]: matrix as it lies when
 *          rows <= cols, transposed when rows > cols
 *   sumsq  fp32 [n * mats_per_ptr, dion_muon_pre_sumsq_blocks(rows, cols)]: sums of squares of the bf16
 *          values written, over 4096-element pieces of each matrix, in a fixed order
 * rows and cols multiples of 64, all pointers 16-byte aligned (DION_E_INVALID otherwise).
 * M is bit-identical to dion_muon_pre's, U holds the same values.
 * Replaces muon_update_pre_orthogonalize (dion/muon.py:284-311), the torch.stack of
 * dion/megabatch_base.py:872, the transposition of tall inputs and the norm of
 * dion/newton_schulz_triton.py:508-513 / dion/polar_express.py:30-35. */
int dion_muon_pre_sumsq_blocks(int rows, int cols);
int dion_muon_pre_prepared(const uint64_t* G_ptrs, int g_dtype, const uint64_t* M_ptrs, int m_dtype, void* U,
                           float* sumsq, int n, int mats_per_ptr, int rows, int cols, float mu, int nesterov,
                           void* stream);

/* Weight decay + update for one shape group.
 *   X_i = (1 - lr wd) X_i - lr adj_ratio U[i]            (cautious == 0)
 *   X_i = X_i - X_i [X_i U[i] >= 0] lr wd - lr adj_ratio U[i]   (cautious != 0)
 * lr_dev: device float (the reference's live 0-d lr tensor); wd_dev: device float or NULL, in
 * which case wd_host is used.  U is the [n, numel] arena, bf16 or fp32 per u_dtype.
 * row_scale (nullable): device [n, rows] fp32; U[i][r][:] is multiplied by row_scale[i][r]
 * first, rows = numel / cols (used by NorMuon).  X per x_dtype.
 * adj_lr_dev (nullable): device float that replaces lr * adj_ratio in the update term (the
 * reference's `adjusted_lr` tensor).
 * Replaces muon_update_post_orthogonalize (dion/muon.py:315-347). */
int dion_muon_post(const uint64_t* X_ptrs, int x_dtype, const void* U, int u_dtype, int n, int64_t numel,
                   int cols, const float* row_scale, const float* lr_dev, const float* adj_lr_dev,
                   float adj_ratio, const float* wd_dev, float wd_host, int cautious, void* stream);

/* out[r][:] = U[r][:] * scale[r] for n_rows rows of cols bf16 elements; out fp32 or bf16 per out_dtype.
 * With the scales of dion_normuon_stats this is the `normalized_U` that
 * normuon_normalization_stacked returns (dion/normuon.py:344-399); the optimizers never materialise
 * it (the scale is folded into dion_muon_post / dion_dion2_post). */
int dion_scale_rows(const void* U, const float* scale, void* out, int out_dtype, int64_t n_rows, int cols,
                    void* stream);

/* NorMuon neuron-wise normalization statistics for one shape group.
 *   r = mean(U^2, dim=-1); V = lerp(V, r, 1-beta2); d = sqrt(V)+1e-8;
 *   row_scale[i][r] = (1/d) * ||U_i||_F / max(||U_i / d||_F, 1e-8)
 * U [n_mat, rows, cols] bf16 (orthogonalized); V_ptrs: host ptr table of n device pointers, each
 * to mats_per_ptr*rows elements of v_dtype (n*mats_per_ptr == n_mat); row_scale out [n_mat, rows]
 * fp32.  The
 * scaled update is applied by dion_muon_post(row_scale=...).
 * Replaces normuon_normalization_stacked (dion/normuon.py:345-399) and the V write-back of
 * dion/normuon.py:320. */
int dion_normuon_stats(const void* U, const uint64_t* V_ptrs, int v_dtype, int n, int mats_per_ptr,
                       int rows, int cols, float beta2, float* row_scale, void* stream);

/* NorMuon statistics for an update made of k selected rows per matrix (NorDion2): U [n_mat, k,
 * cols] bf16, row_idx [n_mat, k] int32 gives the row of the parameter each update row belongs to
 * (a negative entry: that update row is not part of the update, its second moment stays and its
 * scale is 0);
 * V_ptrs entries each point to mats_per_ptr * v_rows elements of v_dtype (the full per-row buffers); only the
 * selected entries of V are read and written.  row_scale out [n_mat, k].
 * Replaces nordion2_normalize_selected_stacked (dion/nordion2.py:430-447). */
int dion_normuon_stats_selected(const void* U, const uint64_t* V_ptrs, int v_dtype, int n, int mats_per_ptr,
                                int k, int cols, const int32_t* row_idx, int v_rows, float beta2,
                                float* row_scale, void* stream);

/* Dion2 momentum accumulate + slice L1 norms for one shape group.
 *   M_i += G_i;  norms[i][s] = sum |M_i| over the other dim, for each slice s along select_dim
 * select_dim: -2 (rows) or -1 (columns).  norms out [n_mat, dim] fp32 (dim = rows or cols).
 * M_ptrs entries each cover mats_per_ptr consecutive matrices.
 * scratch (nullable): device memory of dion_dion2_accumulate_scratch_bytes() bytes, 16-byte
 * aligned; with it the column sums (select_dim -1) of tall matrices are split over row slabs so
 * that the launch fills the chip, and added in a fixed order.  Without it one workgroup walks
 * all rows of its columns.
 * Replaces the first half of dion2_pre_orthogonalize (dion/dion2.py:487-509). */
size_t dion_dion2_accumulate_scratch_bytes(int n_mat, int rows, int cols, int select_dim);
int dion_dion2_accumulate(const uint64_t* G_ptrs, int g_dtype, const uint64_t* M_ptrs, int m_dtype, int n,
                          int mats_per_ptr, int rows, int cols, int select_dim, float* norms,
                          void* scratch, size_t scratch_bytes, void* stream);

/* Dion2 top-k selection: for each of n_mat rows of norms [n_mat, dim] pick the k largest
 * (ties: lower index first), write their indices ascending to idx [n_mat, k] (int32) and the
 * dense inverse map [n_mat, dim] (int32, position in idx or -1).
 * Replaces torch.topk(..., sorted=False) at dion/dion2.py:513 and _build_index_map
 * (dion/dion2_triton.py:30-47). */
int dion_dion2_topk(const float* norms, int n_mat, int dim, int k, int32_t* idx, int32_t* map,
                    void* stream);

/* Dion2 gather + error-feedback decay.
 *   U_sel[i] = bf16(M_i[selected slices]);  M_i[selected slices] *= ef_decay
 * U_sel [n_mat, k, cols] (select_dim -2) or [n_mat, rows, k] (select_dim -1) bf16.
 * Replaces dion/dion2.py:519-545. */
int dion_dion2_gather(const uint64_t* M_ptrs, int m_dtype, int n, int mats_per_ptr, int rows, int cols,
                      int select_dim, const int32_t* idx, int k, float ef_decay, void* U_sel,
                      void* stream);

/* dion_dion2_gather writing U_sel as a prepared orthogonalization input (see
 * dion_ns_orthogonalize_prepared): the selected block with its short side along rows, plus partial sums
 * of squares of each block.  dion_dion2_gather_sumsq_blocks gives the partial sums per matrix, or 0 when
 * the block has no prepared form (then use dion_dion2_gather):
 *   select_dim -2, k <= cols:          U_sel [n_mat, k, cols] as dion_dion2_gather writes it, k sums
 *   select_dim -1, rows <= k:          U_sel [n_mat, rows, k] likewise, `rows` sums
 *   select_dim -1, rows > k:           U_sel [n_mat, k, rows], the block transposed; rows and k multiples
 *                                      of 64, (rows / 64) * (k / 64) sums
 * M is updated exactly as by dion_dion2_gather.  U_sel 16-byte aligned.
 * Replaces dion/dion2.py:519-545 together with the transposition and norm of
 * dion/newton_schulz_triton.py:508-513 / dion/polar_express.py:30-35. */
int dion_dion2_gather_sumsq_blocks(int rows, int cols, int select_dim, int k);
int dion_dion2_gather_prepared(const uint64_t* M_ptrs, int m_dtype, int n, int mats_per_ptr, int rows, int cols,
                               int select_dim, const int32_t* idx, int k, float ef_decay, void* U_sel,
                               float* sumsq, void* stream);

/* Dion2 fused weight decay + selective update, single rounding:
 *   x = (1 - lr wd) x - b u[map]   on selected slices,  x = (1 - lr wd) x elsewhere
 *   b = lr * adj_ratio, or (*adj_lr_dev) * adj_ratio when adj_lr_dev (nullable, device fp32 scalar:
 *   the reference's `adjusted_lr` tensor) is given
 * U_sel [n_mat, k, cols] / [n_mat, rows, k] in u_dtype (DION_BF16 or DION_F32).
 * row_scale (nullable, select_dim -2 only): device [n_mat, k] fp32; selected row j of U_sel is
 * multiplied by row_scale[i][j] first (NorDion2's normalised update).
 * Replaces dion2_post_orthogonalize_triton (dion/dion2_triton.py:147-242, kernel :57-144),
 * dion2_post_orthogonalize (dion/dion2.py:666-697) and its use at dion/nordion2.py:403-425. */
int dion_dion2_post(const uint64_t* X_ptrs, int x_dtype, int n, int mats_per_ptr, int rows, int cols,
                    int select_dim, const void* U_sel, int u_dtype, int k, const int32_t* map,
                    const float* row_scale, const float* lr_dev, const float* adj_lr_dev,
                    float adj_ratio, const float* wd_dev, float wd_host, void* stream);

/* Dense inverse map of k distinct (unordered) int64 slice indices per matrix: map[i][idx[i][j]] = j,
 * -1 elsewhere.  idx [n_mat, k] int64, map out [n_mat, dim] int32.
 * Replaces _build_index_map (dion/dion2_triton.py:30-47). */
int dion_dion2_index_map(const int64_t* idx, int n_mat, int k, int dim, int32_t* map, void* stream);

/* --------------------------------------------------------------------------------------------
 * Whole-matrix selection: what a rank runs on assembled matrices when the top-k is taken inside
 * the orthogonalization call and the update only sees a full-size tensor that is zero outside the
 * selected slices (selection_scope="global").  Stacked tensors are contiguous [n_mat, rows, cols];
 * dtype is DION_BF16 or DION_F32; n_mat <= 65535.
 * ------------------------------------------------------------------------------------------ */

/* norms[i][s] = sum |U_i[slice s]| (fp32 accumulate; round_bf16 != 0 rounds the result to bf16,
 * which is what a bf16 input gets from Tensor.norm).  norms out [n_mat, dim] fp32.
 * Replaces X.norm(p=1, dim=norm_dim) at dion/dion2.py:602 and the non-zero test
 * u.abs().sum(dim) > 0 at dion/dion2.py:648, dion/nordion2.py:487. */
int dion_slice_l1(const void* U, int dtype, int n_mat, int rows, int cols, int select_dim,
                  int round_bf16, float* norms, void* stream);

/* sub_i = U_i[selected slices], idx [n_mat, k] int32 as written by dion_dion2_topk;
 * sub [n_mat, k, cols] (select_dim -2) or [n_mat, rows, k] (select_dim -1), same dtype as U.
 * Replaces torch.gather at dion/dion2.py:604-610. */
int dion_gather_slices(const void* U, int dtype, int n_mat, int rows, int cols, int select_dim,
                       const int32_t* idx, int k, void* sub, void* stream);

/* out_i = zeros;  out_i[selected slices] = sub_i.  map [n_mat, dim] int32 is the dense inverse map
 * of dion_dion2_topk; every element of out is written (no prior clear needed).
 * Replaces zeros_like + scatter_ at dion/dion2.py:612-613. */
int dion_scatter_slices(const void* sub, int dtype, int n_mat, int rows, int cols, int select_dim,
                        const int32_t* map, int k, void* out, void* stream);

/* gate[i][s] = s where norms[i][s] > 0, else -1: the row_idx form dion_normuon_stats_selected takes,
 * in which a negative entry leaves that row's second moment untouched and gives it scale 0
 * (torch.where(sel, v_new, v) at dion/nordion2.py:494). */
int dion_mask_index(const float* norms, int n_mat, int dim, int32_t* gate, void* stream);

/* Masked Dion2 / NorDion2 update, single rounding of the sum:
 *   x = (1 - lr wd) x - b u   everywhere (u [n_mat, rows, cols] bf16, zero off the selected
 *   slices; b as in dion_dion2_post);   m *= ef_decay   on slices with norms[i][s] > 0
 * norms as written by dion_slice_l1 on U.  row_scale (nullable, select_dim -2 only): device
 * [n_mat, rows] fp32, row r of u is multiplied by row_scale[i][r] first.
 * Replaces dion2_post_orthogonalize_masked (dion/dion2.py:623-659) and, with row_scale, the update
 * half of nordion2_post_orthogonalize_masked (dion/nordion2.py:448-500). */
int dion_dion2_post_masked(const uint64_t* X_ptrs, const uint64_t* M_ptrs, int s_dtype, int n, int mats_per_ptr,
                           int rows, int cols, int select_dim, const void* U, const float* norms,
                           const float* row_scale, const float* lr_dev, const float* adj_lr_dev,
                           float adj_ratio, const float* wd_dev, float wd_host, float ef_decay,
                           void* stream);

/* --------------------------------------------------------------------------------------------
 * Multi-tensor AdamW / Lion for the non-matrix parameter groups (algorithm "adamw" / "lion").
 * X_ptrs, G_ptrs, M_ptrs, V_ptrs: host ptr tables of n device pointers; tensor i has numels[i]
 * elements (host array); X, M, V share s_dtype, G bf16 or fp32 per g_dtype (one dtype each per call).
 * lr_dev / wd_dev as in dion_muon_post.  Any number of tensors per call, any sizes.
 * ------------------------------------------------------------------------------------------ */

/* AdamW with bias correction and decoupled (optionally cautious) weight decay:
 *   step_i += 1 (device float counters, step_ptrs; a counter may be shared by tensors of one call
 *   if they lie within the same run of 48 consecutive tensors)
 *   M = lerp(M, G, 1-beta1); V = beta2 V + (1-beta2) G^2; d = sqrt(V)/sqrt(1-beta2^step) + eps
 *   X = X (1 - lr wd)   [cautious: X -= X [M/d * X >= 0] lr wd];   X -= lr/(1-beta1^step) M/d
 * Replaces adamw_update / adamw_update_foreach (dion/scalar_opts.py:7-65, :121-268; capturable
 * form: counters advance on the device, lr is read on the device). */
int dion_adamw_step(const uint64_t* X_ptrs, const uint64_t* G_ptrs, int g_dtype, const uint64_t* M_ptrs,
                    const uint64_t* V_ptrs, int s_dtype, const uint64_t* step_ptrs, const int64_t* numels, int n,
                    const float* lr_dev, float beta1, float beta2, float eps, const float* wd_dev,
                    float wd_host, int cautious, void* stream);

/* Lion:  U = sign(lerp(M, G, 1-beta1)); M = lerp(M, G, 1-beta2);
 *   X = X (1 - lr wd)   [cautious: X -= X [U X >= 0] lr wd];   X -= lr U
 * Replaces lion_update / lion_update_foreach (dion/scalar_opts.py:68-118, :271-325). */
int dion_lion_step(const uint64_t* X_ptrs, const uint64_t* G_ptrs, int g_dtype, const uint64_t* M_ptrs,
                   int s_dtype, const int64_t* numels, int n, const float* lr_dev, float beta1, float beta2,
                   const float* wd_dev, float wd_host, int cautious, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* DION_HIP_H */
