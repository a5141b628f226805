/* A caller of libdion_hip.so written in C: no Python, no torch, no C++.  It orthogonalizes three 96 x 160
 * matrices with the Polar-Express schedule (dion/polar_express.py:10-16, the reference's default) through
 * dion_ns_orthogonalize and through the entry point that allocates nothing, compares the two bit for bit,
 * and checks the result against what the iteration is for: rows of unit length that are orthogonal to each
 * other, to the accuracy five iterations of that schedule reach.  Exit status 0 when everything holds.
 *
 *   gcc -std=c11 -D__HIP_PLATFORM_AMD__ -I/opt/rocm/include -Iinclude tests/c_caller/ns_caller.c \
 *       -o tests/c_caller/ns_caller -Ldion_amd -ldion_hip -L/opt/rocm/lib -lamdhip64 -lm \
 *       -Wl,-rpath,'$ORIGIN/../../dion_amd' -Wl,-rpath,/opt/rocm/lib
 */
#include <hip/hip_runtime_api.h>
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "dion_hip.h"

#define CHECK_HIP(x)                                                                      \
  do {                                                                                    \
    hipError_t e_ = (x);                                                                  \
    if (e_ != hipSuccess) {                                                               \
      fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_));                             \
      return 2;                                                                           \
    }                                                                                     \
  } while (0)
#define CHECK_DION(x)                                                                     \
  do {                                                                                    \
    int rc_ = (x);                                                                        \
    if (rc_ != DION_OK) {                                                                 \
      fprintf(stderr, "%s: %d (%s)\n", #x, rc_, dion_last_error());                       \
      return 3;                                                                           \
    }                                                                                     \
  } while (0)

static uint16_t to_bf16(float f) { /* round to nearest even */
  uint32_t u;
  memcpy(&u, &f, 4);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}
static float from_bf16(uint16_t h) {
  uint32_t u = (uint32_t)h << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

int main(void) {
  enum { BATCH = 3, ROWS = 96, COLS = 160, N = BATCH * ROWS * COLS };
  /* dion/polar_express.py:10-16 */
  static const float pe[15] = {8.156554524902461f,  -22.48329292557795f, 15.878769915207462f,
                               4.042929935166739f,  -2.808917465908714f, 0.5000178451051316f,
                               3.8916678022926607f, -2.772484153217685f, 0.5060648178503393f,
                               3.285753657755655f,  -2.3681294933425376f, 0.46449024233003106f,
                               2.3465413258596377f, -1.7097828382687081f, 0.42323551169305323f};
  printf("libdion_hip ABI version %d\n", dion_abi_version());
  uint16_t* h_in = (uint16_t*)malloc(N * 2);
  uint16_t* h_out = (uint16_t*)malloc(N * 2);
  uint16_t* h_out2 = (uint16_t*)malloc(N * 2);
  uint32_t s = 12345u;
  for (int i = 0; i < N; ++i) { /* sum of four uniforms: bell-shaped, zero mean */
    float v = 0.f;
    for (int k = 0; k < 4; ++k) {
      s = s * 1664525u + 1013904223u;
      v += (float)(s >> 8) / 16777216.0f - 0.5f;
    }
    h_in[i] = to_bf16(0.02f * v);
  }
  void *d_in, *d_out, *d_ws;
  const size_t ws_bytes = dion_ns_workspace_bytes(BATCH, ROWS, COLS, 0);
  CHECK_HIP(hipMalloc(&d_in, N * 2));
  CHECK_HIP(hipMalloc(&d_out, N * 2));
  CHECK_HIP(hipMalloc(&d_ws, ws_bytes ? ws_bytes : 16));
  CHECK_HIP(hipMemcpy(d_in, h_in, N * 2, hipMemcpyHostToDevice));
  CHECK_DION(dion_ns_orthogonalize(d_in, DION_BF16, d_out, BATCH, ROWS, COLS, pe, 5, 1.02f, 1e-6f, 0, 0, d_ws,
                                   ws_bytes, NULL));
  CHECK_HIP(hipDeviceSynchronize());
  CHECK_HIP(hipMemcpy(h_out, d_out, N * 2, hipMemcpyDeviceToHost));
  CHECK_HIP(hipMemset(d_out, 0xff, N * 2));
  CHECK_DION(dion_ns_orthogonalize_static(d_in, DION_BF16, d_out, BATCH, ROWS, COLS, pe, 5, 1.02f, 1e-6f, 0, 0, NULL));
  CHECK_HIP(hipDeviceSynchronize());
  CHECK_HIP(hipMemcpy(h_out2, d_out, N * 2, hipMemcpyDeviceToHost));
  if (memcmp(h_out, h_out2, N * 2) != 0) {
    fprintf(stderr, "dion_ns_orthogonalize_static differs from dion_ns_orthogonalize\n");
    return 4;
  }
  double worst_diag = 0.0, worst_off = 0.0;
  for (int b = 0; b < BATCH; ++b) {
    const uint16_t* o = h_out + (size_t)b * ROWS * COLS;
    for (int i = 0; i < ROWS; ++i)
      for (int j = i; j < ROWS; ++j) {
        double g = 0.0;
        for (int k = 0; k < COLS; ++k) g += (double)from_bf16(o[i * COLS + k]) * (double)from_bf16(o[j * COLS + k]);
        if (i == j) {
          if (fabs(g - 1.0) > worst_diag) worst_diag = fabs(g - 1.0);
        } else if (fabs(g) > worst_off) {
          worst_off = fabs(g);
        }
      }
  }
  printf("O O^T - I: worst diagonal %.3e, worst off-diagonal %.3e\n", worst_diag, worst_off);
  CHECK_HIP(hipFree(d_in));
  CHECK_HIP(hipFree(d_out));
  CHECK_HIP(hipFree(d_ws));
  free(h_in);
  free(h_out);
  free(h_out2);
  /* five Polar-Express iterations leave the singular values within about [0.85, 1.15] of one: O O^T = U S^2 U^T
   * then differs from the identity by up to 0.3 on the diagonal and half of that band off it */
  return (worst_diag < 0.3 && worst_off < 0.2) ? 0 : 1;
}
