// Multi-tensor AdamW and Lion steps for the non-matrix parameter groups (embeddings, heads, norms,
// biases) of a model whose matrices are updated by Muon / NorMuon / Dion2 / NorDion2.
//
// One launch updates up to kMtaTensors tensors of different sizes: their pointers and element
// counts travel by value in the kernel-argument segment, blockIdx.y picks the tensor and the
// blocks of a row walk it with a grid stride.  All traffic is HBM streaming: AdamW reads X, G, M, V
// and writes X, M, V (28 B/element with fp32 state and gradients, 26 with bf16 gradients), Lion 20 / 18
// B/element.  The state tensors X, M, V of one launch share a dtype, fp32 or bf16 (half the bytes);
// arithmetic is fp32 either way.
//
// Arithmetic follows dion/scalar_opts.py:7-65 (adamw_update) and :68-118 (lion_update); the step
// counters are device scalars advanced on the device, like the capturable form of
// adamw_update_foreach (dion/scalar_opts.py:196-213), and lr / weight decay are read from device
// scalars, so a captured step sees live values.
#include "elementwise.h"

namespace dion {

struct MtaTensors {
  uint64_t x[kMtaTensors], g[kMtaTensors], m[kMtaTensors], v[kMtaTensors], step[kMtaTensors];
  int64_t numel[kMtaTensors];
};

// step[t] += 1 for every tensor of the launch (before the update kernel reads them).
__global__ void mta_advance_steps_kernel(MtaTensors a, int n) {
  const int t = threadIdx.x;
  if (t < n) {
    float* s = (float*)a.step[t];
    // the same counter may serve several tensors: advance each distinct one once
    bool first = true;
    for (int u = 0; u < t; ++u) first = first && (a.step[u] != a.step[t]);
    if (first) *s = *s + 1.0f;
  }
}

struct AdamwScalars {
  float beta1, beta2, eps, wd_host;
  int cautious;
};

template <typename GT>
static __device__ __forceinline__ void adamw_one(float& x, float g, float& m, float& v, float w1,
                                                 float beta2, float w2, float inv_bc2_sqrt, float eps,
                                                 float adj_lr, float a, float coeff, int cautious) {
  m = m + w1 * (g - m);                 // lerp(M, G, 1 - beta1)
  v = v * beta2 + w2 * (g * g);         // V * beta2 + (1 - beta2) * G * G
  const float denom = sqrtf(v) * inv_bc2_sqrt + eps;
  const float upd = m / denom;
  if (cautious) {
    if (upd * x >= 0.0f) x = x - x * coeff;
  } else {
    x = x * a;
  }
  x = x - adj_lr * upd;
}

template <typename GT, typename ST>
__global__ __launch_bounds__(256) void adamw_mt_kernel(MtaTensors a, const float* __restrict__ lr_dev,
                                                       const float* __restrict__ wd_dev,
                                                       AdamwScalars sc) {
  const int t = blockIdx.y;
  const int64_t numel = a.numel[t];
  ST* __restrict__ x = (ST*)a.x[t];
  const GT* __restrict__ g = (const GT*)a.g[t];
  ST* __restrict__ m = (ST*)a.m[t];
  ST* __restrict__ v = (ST*)a.v[t];
  const float step = *(const float*)a.step[t];
  const float lr = *lr_dev;
  const float wd = wd_dev ? *wd_dev : sc.wd_host;
  const float bc1 = 1.0f - powf(sc.beta1, step);
  const float bc2 = 1.0f - powf(sc.beta2, step);
  const float inv_bc2_sqrt = 1.0f / sqrtf(bc2);
  const float adj_lr = lr / bc1;
  const float coeff = lr * wd;
  const float aa = 1.0f - coeff;
  const float w1 = 1.0f - sc.beta1, w2 = 1.0f - sc.beta2;
  const int64_t stride = (int64_t)gridDim.x * 256;
  const int64_t tid = (int64_t)blockIdx.x * 256 + threadIdx.x;
  // groups of 4 elements: 16-byte accesses to fp32 tensors, 8-byte accesses to bf16 ones
  const bool vec = (((a.x[t] | a.m[t] | a.v[t]) & (sizeof(ST) == 2 ? 7 : 15)) == 0) &&
                   ((a.g[t] & (sizeof(GT) == 2 ? 7 : 15)) == 0);
  const int64_t n4 = vec ? numel / 4 : 0;
  for (int64_t q = tid; q < n4; q += stride) {
    float xv[4], mv[4], vv[4], gv[4];
    st_load4<ST>(x, q, xv);
    st_load4<ST>(m, q, mv);
    st_load4<ST>(v, q, vv);
    st_load4<GT>(g, q, gv);
#pragma unroll
    for (int e = 0; e < 4; ++e)
      adamw_one<GT>(xv[e], gv[e], mv[e], vv[e], w1, sc.beta2, w2, inv_bc2_sqrt, sc.eps, adj_lr, aa, coeff,
                    sc.cautious);
    st_store4<ST>(x, q, xv);
    st_store4<ST>(m, q, mv);
    st_store4<ST>(v, q, vv);
  }
  for (int64_t i = n4 * 4 + tid; i < numel; i += stride) {
    float xs = st_load<ST>(x, i), ms = st_load<ST>(m, i), vs = st_load<ST>(v, i);
    adamw_one<GT>(xs, st_load<GT>(g, i), ms, vs, w1, sc.beta2, w2, inv_bc2_sqrt, sc.eps, adj_lr, aa, coeff,
                  sc.cautious);
    st_store<ST>(x, i, xs);
    st_store<ST>(m, i, ms);
    st_store<ST>(v, i, vs);
  }
}

static __device__ __forceinline__ void lion_one(float& x, float g, float& m, float w1, float w2, float lr,
                                                float a, float coeff, int cautious) {
  const float c = m + w1 * (g - m);  // lerp(M, G, 1 - beta1)
  const float u = c > 0.0f ? 1.0f : (c < 0.0f ? -1.0f : 0.0f);
  m = m + w2 * (g - m);              // lerp(M, G, 1 - beta2)
  if (cautious) {
    if (u * x >= 0.0f) x = x - x * coeff;
  } else {
    x = x * a;
  }
  x = x - lr * u;
}

template <typename GT, typename ST>
__global__ __launch_bounds__(256) void lion_mt_kernel(MtaTensors a, const float* __restrict__ lr_dev,
                                                      const float* __restrict__ wd_dev, float beta1,
                                                      float beta2, float wd_host, int cautious) {
  const int t = blockIdx.y;
  const int64_t numel = a.numel[t];
  ST* __restrict__ x = (ST*)a.x[t];
  const GT* __restrict__ g = (const GT*)a.g[t];
  ST* __restrict__ m = (ST*)a.m[t];
  const float lr = *lr_dev;
  const float wd = wd_dev ? *wd_dev : wd_host;
  const float coeff = lr * wd;
  const float aa = 1.0f - coeff;
  const float w1 = 1.0f - beta1, w2 = 1.0f - beta2;
  const int64_t stride = (int64_t)gridDim.x * 256;
  const int64_t tid = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const bool vec = (((a.x[t] | a.m[t]) & (sizeof(ST) == 2 ? 7 : 15)) == 0) &&
                   ((a.g[t] & (sizeof(GT) == 2 ? 7 : 15)) == 0);
  const int64_t n4 = vec ? numel / 4 : 0;
  for (int64_t q = tid; q < n4; q += stride) {
    float xv[4], mv[4], gv[4];
    st_load4<ST>(x, q, xv);
    st_load4<ST>(m, q, mv);
    st_load4<GT>(g, q, gv);
#pragma unroll
    for (int e = 0; e < 4; ++e) lion_one(xv[e], gv[e], mv[e], w1, w2, lr, aa, coeff, cautious);
    st_store4<ST>(x, q, xv);
    st_store4<ST>(m, q, mv);
  }
  for (int64_t i = n4 * 4 + tid; i < numel; i += stride) {
    float xs = st_load<ST>(x, i), ms = st_load<ST>(m, i);
    lion_one(xs, st_load<GT>(g, i), ms, w1, w2, lr, aa, coeff, cautious);
    st_store<ST>(x, i, xs);
    st_store<ST>(m, i, ms);
  }
}

// Blocks per tensor row: enough for the largest tensor of the launch at 8 elements per thread,
// capped so that a launch of many small tensors does not carry thousands of idle blocks.
static unsigned mta_blocks(const int64_t* numel, int n) {
  int64_t mx = 0;
  for (int i = 0; i < n; ++i) mx = numel[i] > mx ? numel[i] : mx;
  int64_t b = (mx + 2047) / 2048;
  if (b < 1) b = 1;
  if (b > 4096) b = 4096;
  return (unsigned)b;
}

static void fill(MtaTensors& a, const uint64_t* X, const uint64_t* G, const uint64_t* M, const uint64_t* V,
                 const uint64_t* S, const int64_t* numel, int n) {
  for (int i = 0; i < kMtaTensors; ++i) {
    const int j = i < n ? i : 0;
    a.x[i] = X[j];
    a.g[i] = G[j];
    a.m[i] = M[j];
    a.v[i] = V ? V[j] : 0;
    a.step[i] = S ? S[j] : 0;
    a.numel[i] = i < n ? numel[j] : 0;
  }
}

hipError_t launch_adamw_mt(const uint64_t* X, const uint64_t* G, int g_dtype, const uint64_t* M,
                           const uint64_t* V, int s_dtype, const uint64_t* steps, const int64_t* numel, int n,
                           const float* lr_dev, float beta1, float beta2, float eps, const float* wd_dev,
                           float wd_host, int cautious, hipStream_t st) {
  MtaTensors a;
  fill(a, X, G, M, V, steps, numel, n);
  hipLaunchKernelGGL(mta_advance_steps_kernel, dim3(1), dim3(64), 0, st, a, n);
  AdamwScalars sc{beta1, beta2, eps, wd_host, cautious};
  dim3 grid(mta_blocks(numel, n), n);
#define ADAMW_LAUNCH(GT, ST) \
  hipLaunchKernelGGL((adamw_mt_kernel<GT, ST>), grid, dim3(256), 0, st, a, lr_dev, wd_dev, sc)
  if (g_dtype == 0) {
    if (s_dtype == 0) ADAMW_LAUNCH(bf16_t, bf16_t); else ADAMW_LAUNCH(bf16_t, float);
  } else {
    if (s_dtype == 0) ADAMW_LAUNCH(float, bf16_t); else ADAMW_LAUNCH(float, float);
  }
#undef ADAMW_LAUNCH
  return hipGetLastError();
}

hipError_t launch_lion_mt(const uint64_t* X, const uint64_t* G, int g_dtype, const uint64_t* M, int s_dtype,
                          const int64_t* numel, int n, const float* lr_dev, float beta1, float beta2,
                          const float* wd_dev, float wd_host, int cautious, hipStream_t st) {
  MtaTensors a;
  fill(a, X, G, M, nullptr, nullptr, numel, n);
  dim3 grid(mta_blocks(numel, n), n);
#define LION_LAUNCH(GT, ST)                                                                             \
  hipLaunchKernelGGL((lion_mt_kernel<GT, ST>), grid, dim3(256), 0, st, a, lr_dev, wd_dev, beta1, beta2, \
                     wd_host, cautious)
  if (g_dtype == 0) {
    if (s_dtype == 0) LION_LAUNCH(bf16_t, bf16_t); else LION_LAUNCH(bf16_t, float);
  } else {
    if (s_dtype == 0) LION_LAUNCH(float, bf16_t); else LION_LAUNCH(float, float);
  }
#undef LION_LAUNCH
  return hipGetLastError();
}

}  // namespace dion
