/*
 * A caller of libslowrun_ce.so that knows nothing but include/slowrun_ce.h and the HIP
 * runtime: what a binding for FusedSoftcappedCrossEntropy (tiny/cuda_kernels.py:336-414)
 * does underneath, written out in C.  It runs forward and backward on a small ragged
 * problem and checks loss, dX and dW against the formulas of the eager head
 * (tiny/train.py:741-743) evaluated in double precision right here.
 *
 * The inputs are chosen so that the fp8 cast is exact (every X / x_s and W / w_s is an
 * e4m3 value), which keeps a quantiser out of this file.
 *
 * Built by slowrun_amd/build.py into tests/bin/abi_example; run by tests/test_c_abi.py.
 */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <hip/hip_runtime_api.h>

#include "slowrun_ce.h"

#define CHECK_HIP(call)                                                                   \
  do {                                                                                    \
    hipError_t e_ = (call);                                                               \
    if (e_ != hipSuccess) {                                                               \
      fprintf(stderr, "%s:%d: %s: %s\n", __FILE__, __LINE__, #call, hipGetErrorString(e_)); \
      return 2;                                                                           \
    }                                                                                     \
  } while (0)
#define CHECK_SCE(call)                                                                   \
  do {                                                                                    \
    int rc_ = (call);                                                                     \
    if (rc_ != SCE_OK) {                                                                  \
      fprintf(stderr, "%s:%d: %s -> %d: %s\n", __FILE__, __LINE__, #call, rc_, sce_last_error()); \
      return 3;                                                                           \
    }                                                                                     \
  } while (0)

enum { N = 1201, D = 64, V = 500 };
static const float kTable[16] = {0.f, 0.25f, -0.25f, 0.5f, -0.5f, 0.75f, -0.75f, 1.f, -1.f, 1.5f, -1.5f, 2.f, -2.f, 3.f, -3.f, 0.f};

static uint32_t mix(uint32_t a) {
  a ^= a >> 16; a *= 0x7feb352du; a ^= a >> 15; a *= 0x846ca68bu; a ^= a >> 16;
  return a;
}

static void* dev_alloc(size_t bytes) {
  void* p = NULL;
  if (hipMalloc(&p, bytes ? bytes : 256) != hipSuccess) return NULL;
  return p;
}

int main(void) {
  const float x_s = 1.0f, w_s = 0.125f, cap = 15.0f;
  static float X[N][D], W[D][V], dX[N][D], dW[D][V];
  static double rdX[N][D], rdW[D][V], u[V], du[V];
  static int64_t y[N];
  for (int i = 0; i < N; ++i)
    for (int j = 0; j < D; ++j) X[i][j] = kTable[mix((uint32_t)(i * D + j)) & 15];
  for (int j = 0; j < D; ++j)
    for (int v = 0; v < V; ++v) W[j][v] = 0.125f * kTable[mix(0x9e3779b9u + (uint32_t)(j * V + v)) & 15];
  int n_valid = 0;
  for (int i = 0; i < N; ++i) {
    y[i] = (i % 11 == 5) ? -1 : (int64_t)((i * 7 + 3) % V);
    n_valid += y[i] >= 0;
  }

  /* reference: F.cross_entropy(cap * tanh(X W / cap), y, ignore_index = -1, reduction = 'mean') and its gradients */
  double ref_loss = 0.0;
  memset(rdX, 0, sizeof rdX);
  memset(rdW, 0, sizeof rdW);
  for (int i = 0; i < N; ++i) {
    if (y[i] < 0) continue;
    double zmax = -1e300, sum = 0.0;
    for (int v = 0; v < V; ++v) {
      double acc = 0.0;
      for (int j = 0; j < D; ++j) acc += (double)X[i][j] * (double)W[j][v];
      u[v] = acc;
      const double z = cap * tanh(acc / cap);
      if (z > zmax) zmax = z;
    }
    for (int v = 0; v < V; ++v) sum += exp(cap * tanh(u[v] / cap) - zmax);
    const double lse = zmax + log(sum);
    ref_loss += lse - cap * tanh(u[y[i]] / cap);
    for (int v = 0; v < V; ++v) {
      const double t = tanh(u[v] / cap), p = exp(cap * t - lse);
      du[v] = (p - (v == y[i] ? 1.0 : 0.0)) * (1.0 - t * t) / n_valid;
    }
    for (int j = 0; j < D; ++j) {
      double a = 0.0;
      for (int v = 0; v < V; ++v) {
        a += du[v] * (double)W[j][v];
        rdW[j][v] += (double)X[i][j] * du[v];
      }
      rdX[i][j] = a;
    }
  }
  ref_loss /= n_valid;

  /* the call sequence of a binding */
  CHECK_HIP(hipSetDevice(0));
  sce_shape shape = {N, D, V, 1, 0};
  sce_sizes sz;
  CHECK_SCE(sce_sizes_for(&shape, &sz));
  void *d_x = dev_alloc(sizeof X), *d_w = dev_alloc(sizeof W), *d_y = dev_alloc(sizeof y);
  void *d_dx = dev_alloc(sizeof dX), *d_dw = dev_alloc(sizeof dW);
  void *d_saved = dev_alloc(sz.saved_bytes), *d_ws_f = dev_alloc(sz.fwd_workspace_bytes), *d_ws_b = dev_alloc(sz.bwd_workspace_bytes);
  float* d_small = (float*)dev_alloc(1024);      /* loss, grad_output, n_valid */
  float* d_losses = (float*)dev_alloc(sizeof(float) * N);
  if (!d_x || !d_w || !d_y || !d_dx || !d_dw || !d_saved || !d_ws_f || !d_ws_b || !d_small || !d_losses) {
    fprintf(stderr, "hipMalloc failed\n");
    return 2;
  }
  CHECK_HIP(hipMemcpy(d_x, X, sizeof X, hipMemcpyHostToDevice));
  CHECK_HIP(hipMemcpy(d_w, W, sizeof W, hipMemcpyHostToDevice));
  CHECK_HIP(hipMemcpy(d_y, y, sizeof y, hipMemcpyHostToDevice));
  const float one = 1.0f;
  CHECK_HIP(hipMemcpy(d_small + 1, &one, sizeof one, hipMemcpyHostToDevice));

  sce_args a;
  memset(&a, 0, sizeof a);
  a.struct_size = sizeof a;
  a.device = 0;
  a.stream = NULL;
  a.shape = shape;
  a.x = d_x; a.x_dtype = SCE_F32; a.x_ld = D;
  a.w = d_w; a.w_dtype = SCE_F32; a.w_ld = V;
  a.targets = (const int64_t*)d_y;
  a.x_s = x_s; a.w_s = w_s; a.cap = cap; a.grad_scale = 1.0f;
  a.ignore_index = -1;
  a.reduction = SCE_REDUCE_MEAN;
  a.loss = d_small; a.losses = d_losses; a.n_valid = (int32_t*)(d_small + 8);
  a.saved = d_saved; a.saved_bytes = sz.saved_bytes;
  a.workspace = d_ws_f; a.workspace_bytes = sz.fwd_workspace_bytes;
  CHECK_SCE(sce_forward(&a));
  a.workspace = d_ws_b; a.workspace_bytes = sz.bwd_workspace_bytes;
  a.grad_output = d_small + 1;
  a.dx = d_dx; a.dx_dtype = SCE_F32; a.dx_ld = D;
  a.dw = d_dw; a.dw_dtype = SCE_F32; a.dw_ld = V;
  CHECK_SCE(sce_backward(&a));
  CHECK_HIP(hipDeviceSynchronize());

  float loss = 0.f;
  int32_t counts[2] = {0, 0};
  CHECK_HIP(hipMemcpy(&loss, d_small, sizeof loss, hipMemcpyDeviceToHost));
  CHECK_HIP(hipMemcpy(counts, d_small + 8, sizeof counts, hipMemcpyDeviceToHost));
  CHECK_HIP(hipMemcpy(dX, d_dx, sizeof dX, hipMemcpyDeviceToHost));
  CHECK_HIP(hipMemcpy(dW, d_dw, sizeof dW, hipMemcpyDeviceToHost));

  /* an error path: a workspace that is too small must be refused with a message, not written to */
  a.workspace_bytes = 1024;
  const int rc_small = sce_backward(&a);

  double num = 0, na = 0, nb = 0, maxd = 0, maxr = 0;
  for (int i = 0; i < N; ++i)
    for (int j = 0; j < D; ++j) {
      const double g = dX[i][j], r = rdX[i][j];
      num += g * r; na += g * g; nb += r * r;
      if (fabs(g - r) > maxd) maxd = fabs(g - r);
      if (fabs(r) > maxr) maxr = fabs(r);
    }
  const double cos_dx = num / sqrt(na * nb), rel_dx = maxd / maxr;
  num = na = nb = maxd = maxr = 0;
  for (int j = 0; j < D; ++j)
    for (int v = 0; v < V; ++v) {
      const double g = dW[j][v], r = rdW[j][v];
      num += g * r; na += g * g; nb += r * r;
      if (fabs(g - r) > maxd) maxd = fabs(g - r);
      if (fabs(r) > maxr) maxr = fabs(r);
    }
  const double cos_dw = num / sqrt(na * nb), rel_dw = maxd / maxr;
  const double rel_loss = fabs(loss - ref_loss) / fabs(ref_loss);
  int ignored_rows_zero = 1;
  for (int i = 0; i < N; ++i)
    if (y[i] < 0)
      for (int j = 0; j < D; ++j) ignored_rows_zero &= dX[i][j] == 0.0f;
  printf("abi_example: version %d loss %.7f ref %.7f rel %.2e | dX maxrel %.2e cos %.7f | dW maxrel %.2e cos %.7f | n_valid %d/%d | "
         "small workspace -> %d (%s)\n",
         sce_version(), loss, ref_loss, rel_loss, rel_dx, cos_dx, rel_dw, cos_dw, counts[0], n_valid, rc_small, sce_last_error());
  const int ok = rel_loss <= 1e-3 && rel_dx <= 2e-2 && rel_dw <= 2e-2 && cos_dx > 0.9995 && cos_dw > 0.9995 &&
                 counts[0] == n_valid && counts[1] == 0 && ignored_rows_zero && rc_small == SCE_EINVAL;
  hipFree(d_x); hipFree(d_w); hipFree(d_y); hipFree(d_dx); hipFree(d_dw); hipFree(d_saved); hipFree(d_ws_f); hipFree(d_ws_b);
  hipFree(d_small); hipFree(d_losses);
  puts(ok ? "abi_example: ok" : "abi_example: FAILED");
  return ok ? 0 : 1;
}
