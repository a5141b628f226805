// Launchers for the memory-bound kernels in elementwise.hip (internal; the public surface is
// include/dion_hip.h).
#pragma once
#include "common.h"

namespace dion {


// Coefficient schedule passed by value to the LDS-resident small-matrix kernel.
constexpr int kMaxSmallIters = 8;
struct NsCoeffs {
  int n;
  float c[kMaxSmallIters][3];
};
// True when a rows x cols matrix (short side <= 64) fits the one-workgroup-per-matrix kernel.
bool ns_small_fits(int rows, int cols);
hipError_t launch_ns_small(const void* in, int in_dtype, bf16_t* out, int batch, int rows, int cols,
                           const NsCoeffs& co, float norm_scale, float eps, hipStream_t st);

hipError_t launch_frobenius_inv(const void* in, int in_dtype, int batch, int64_t numel,
                                float norm_scale, float eps, float* partial, int nblk,
                                float* inv_norm, hipStream_t st);
// inv_norm[b] = 1 / (sqrt(sum of partial[b][0..nblk)) * norm_scale + eps), fixed summation order.
hipError_t launch_norm_finalize(const float* partial, int nblk, int batch, float norm_scale, float eps,
                                float* inv_norm, hipStream_t st);
hipError_t launch_ns_prepare(const void* in, int in_dtype, int batch, int R, int C,
                             const float* inv_norm, bf16_t* same, int Rp, int Cp, int ld_same,
                             int64_t stride_same, bf16_t* trans, int ld_trans, int64_t stride_trans,
                             hipStream_t st);
hipError_t launch_unpad(const bf16_t* src, int64_t src_stride, int ld, bf16_t* dst, int batch, int R,
                        int C, hipStream_t st);
// State tensors (parameters X, momentum M, second moments V) are fp32 or bf16: *_dtype 0 = bf16,
// 1 = fp32, like the gradient / update dtypes.
hipError_t launch_muon_pre(const PtrTab& G, int g_dtype, const PtrTab& M, int m_dtype, bf16_t* U, int n,
                           int64_t numel, float mu, int nesterov, bool vec, hipStream_t st);
// muon_pre for matrices that go to the orthogonalization as they are written: U [n * mats][min][max] with
// the short side along rows (a tall matrix is written transposed) plus sumsq [n * mats][rows * cols / 4096]
// partial sums of squares.  rows, cols multiples of 64, rows * cols of 4096, all pointers 16-byte aligned,
// numel / 4096 <= 2^31 - 1 and n * mats <= 65535 (checked by the caller).
hipError_t launch_muon_pre_prepared(const PtrTab& G, int g_dtype, const PtrTab& M, int m_dtype, bf16_t* U,
                                    float* sumsq, int n, int mats, int rows, int cols, float mu,
                                    int nesterov, hipStream_t st);
hipError_t launch_muon_post(const PtrTab& X, int x_dtype, const void* U, int u_dtype, int n, int64_t numel,
                            int cols, const float* row_scale, const float* lr_dev, const float* adj_lr_dev,
                            float adj_ratio, const float* wd_dev, float wd_host, int cautious, bool vec,
                            hipStream_t st);
hipError_t launch_scale_rows(const bf16_t* U, const float* scale, void* out, int out_dtype, int64_t n_rows,
                             int cols, hipStream_t st);
hipError_t launch_normuon_stats(const bf16_t* U, const PtrTab& V, int v_dtype, int n_mat, int mats_per_ptr,
                                int rows, int cols, const int32_t* row_idx, int v_rows, float w,
                                float* row_scale, hipStream_t st);
hipError_t launch_dion2_accumulate(const PtrTab& G, int g_dtype, const PtrTab& M, int m_dtype, int n_mat,
                                   int mats_per_ptr, int rows, int cols, int select_rows,
                                   float* norms, bool vec4, float* slab_scratch, int slabs,
                                   hipStream_t st);
// Row slabs the column-sum path of launch_dion2_accumulate wants for this shape (1 = no scratch).
int dion2_acc_slabs(int n_mat, int rows, int cols);
hipError_t launch_dion2_topk(const float* norms, int n_mat, int dim, int k, int32_t* idx,
                             int32_t* map, hipStream_t st);
hipError_t launch_dion2_gather(const PtrTab& M, int m_dtype, int n_mat, int mats_per_ptr, int rows, int cols,
                               int select_rows, const int32_t* idx, int k, float ef_decay, bf16_t* U,
                               bool vec4, hipStream_t st);
// dion2 gather writing the orthogonalization input in the iteration's layout plus partial sums of squares:
// rows selected (k <= cols): U [n_mat, k, cols], one partial per selected row; columns selected: U [n_mat, rows, k]
// with one partial per row when rows <= k, else U^T [n_mat, k, rows] with one partial per 64 x 64 tile
// (rows % 64 == 0 and k % 64 == 0).
hipError_t launch_dion2_gather_prepared(const PtrTab& M, int m_dtype, int n_mat, int mats_per_ptr, int rows,
                                        int cols, int select_rows, const int32_t* idx, int k, float ef_decay,
                                        bf16_t* U, float* sumsq, bool vec4, hipStream_t st);
hipError_t launch_dion2_post(const PtrTab& X, int x_dtype, int n_mat, int mats_per_ptr, int rows, int cols,
                             int select_rows, const void* U, int u_dtype, int k, const int32_t* map,
                             const float* row_scale, const float* lr_dev, const float* adj_lr_dev,
                             float adj_ratio, const float* wd_dev, float wd_host, bool vec4,
                             hipStream_t st);
hipError_t launch_dion2_index_map(const int64_t* idx, int n_mat, int k, int dim, int32_t* map,
                                  hipStream_t st);

// Whole-matrix selection (select_scope.hip): slice L1 norms of a stacked tensor, dense gather /
// zero-filled scatter of the selected slices, and the update keyed off the non-zero slices.
// dtype 0 = bf16, 1 = fp32.
hipError_t launch_slice_l1(const void* U, int dtype, int n_mat, int rows, int cols, int select_rows,
                           int round_bf16, float* norms, hipStream_t st);
hipError_t launch_gather_slices(const void* U, int dtype, int n_mat, int rows, int cols, int select_rows,
                                const int32_t* idx, int k, void* sub, hipStream_t st);
hipError_t launch_scatter_slices(const void* sub, int dtype, int n_mat, int rows, int cols,
                                 int select_rows, const int32_t* map, int k, void* out, hipStream_t st);
hipError_t launch_mask_index(const float* norms, int n_mat, int dim, int32_t* gate, hipStream_t st);
hipError_t launch_dion2_post_masked(const PtrTab& X, const PtrTab& M, int s_dtype, int n_mat, int mats_per_ptr,
                                    int rows, int cols, int select_rows, const bf16_t* U,
                                    const float* norms, const float* row_scale, const float* lr_dev,
                                    const float* adj_lr_dev, float adj_ratio, const float* wd_dev,
                                    float wd_host, float ef_decay, bool vec4, hipStream_t st);

// Multi-tensor AdamW / Lion (scalar_opts.hip): n <= kMtaTensors tensors per launch, host arrays of
// device pointers and element counts.
constexpr int kMtaTensors = 48;
hipError_t launch_adamw_mt(const uint64_t* X, const uint64_t* G, int g_dtype, const uint64_t* M,
                           const uint64_t* V, int s_dtype, const uint64_t* steps, const int64_t* numel, int n,
                           const float* lr_dev, float beta1, float beta2, float eps, const float* wd_dev,
                           float wd_host, int cautious, hipStream_t st);
hipError_t launch_lion_mt(const uint64_t* X, const uint64_t* G, int g_dtype, const uint64_t* M, int s_dtype,
                          const int64_t* numel, int n, const float* lr_dev, float beta1, float beta2,
                          const float* wd_dev, float wd_host, int cautious, hipStream_t st);

}  // namespace dion
