/* A host program in plain C that uses libsiirl_hip.so through include/siirl_hip.h alone -- no Python, no torch:
 * device buffers from the HIP runtime, log-prob / entropy forward and backward of fp32 logits [T, V], checked
 * against a double-precision loop written here, and the top-k pick of the KL-Cov loss over the same values.  Exit status 0 and a line starting with "OK" on success. */
#include <hip/hip_runtime_api.h>
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>

#include "siirl_hip.h"

#define CK(x)                                                              \
  do {                                                                     \
    hipError_t e_ = (x);                                                   \
    if (e_ != hipSuccess) {                                                \
      printf("FAIL %s: %s\n", #x, hipGetErrorString(e_));                  \
      return 2;                                                            \
    }                                                                      \
  } while (0)
#define CALL(x)                                                            \
  do {                                                                     \
    int rc_ = (x);                                                         \
    if (rc_ != SIIRL_OK) {                                                 \
      printf("FAIL %s -> %d: %s\n", #x, rc_, siirl_hip_last_error());      \
      return 3;                                                            \
    }                                                                      \
  } while (0)

int main(void) {
  enum { T = 96, V = 1003 };
  const float inv_temperature = 1.0f / 0.9f;
  float* x = (float*)malloc(sizeof(float) * T * V);
  int64_t* y = (int64_t*)malloc(sizeof(int64_t) * T);
  float *g_lp = (float*)malloc(sizeof(float) * T), *g_h = (float*)malloc(sizeof(float) * T);
  uint32_t s = 12345u;
  for (int i = 0; i < T * V; ++i) {
    s = s * 1664525u + 1013904223u;
    x[i] = ((float)(s >> 8) / 16777216.0f - 0.5f) * 8.0f;
  }
  for (int t = 0; t < T; ++t) {
    y[t] = (int64_t)((t * 7919) % V);
    g_lp[t] = 0.01f * (float)(t % 11 - 5);
    g_h[t] = 0.02f * (float)(t % 7 - 3);
  }
  float *d_x, *d_dx, *d_lp, *d_ent, *d_lse, *d_ex, *d_glp, *d_gh;
  int64_t* d_y;
  CK(hipMalloc((void**)&d_x, sizeof(float) * T * V));
  CK(hipMalloc((void**)&d_dx, sizeof(float) * T * V));
  CK(hipMalloc((void**)&d_y, sizeof(int64_t) * T));
  CK(hipMalloc((void**)&d_lp, sizeof(float) * T));
  CK(hipMalloc((void**)&d_ent, sizeof(float) * T));
  CK(hipMalloc((void**)&d_lse, sizeof(float) * T));
  CK(hipMalloc((void**)&d_ex, sizeof(float) * T));
  CK(hipMalloc((void**)&d_glp, sizeof(float) * T));
  CK(hipMalloc((void**)&d_gh, sizeof(float) * T));
  CK(hipMemcpy(d_x, x, sizeof(float) * T * V, hipMemcpyHostToDevice));
  CK(hipMemcpy(d_y, y, sizeof(int64_t) * T, hipMemcpyHostToDevice));
  CK(hipMemcpy(d_glp, g_lp, sizeof(float) * T, hipMemcpyHostToDevice));
  CK(hipMemcpy(d_gh, g_h, sizeof(float) * T, hipMemcpyHostToDevice));
  hipStream_t stream;
  CK(hipStreamCreate(&stream));

  if (siirl_hip_abi_version() != SIIRL_HIP_ABI_VERSION) {
    printf("FAIL abi version %d\n", siirl_hip_abi_version());
    return 4;
  }
  CALL(siirl_logprob_entropy_fwd(d_x, SIIRL_F32, T, V, V, d_y, inv_temperature, d_lp, d_ent, d_lse, d_ex, stream));
  CALL(siirl_logprob_entropy_bwd(d_x, SIIRL_F32, T, V, V, d_y, inv_temperature, d_lse, d_ex, d_glp, d_gh, d_dx, V, 0,
                                 stream));
  CK(hipStreamSynchronize(stream));
  /* an invalid call must come back as an error code with a message, not as a crash */
  if (siirl_logprob_entropy_fwd(d_x, SIIRL_F32, T, 0, 0, d_y, inv_temperature, d_lp, d_ent, d_lse, d_ex, stream) !=
      SIIRL_ERR_INVALID_ARGUMENT) {
    printf("FAIL V = 0 was accepted\n");
    return 5;
  }

  float *lp = (float*)malloc(sizeof(float) * T), *ent = (float*)malloc(sizeof(float) * T);
  float* dx = (float*)malloc(sizeof(float) * T * V);
  CK(hipMemcpy(lp, d_lp, sizeof(float) * T, hipMemcpyDeviceToHost));
  CK(hipMemcpy(ent, d_ent, sizeof(float) * T, hipMemcpyDeviceToHost));
  CK(hipMemcpy(dx, d_dx, sizeof(float) * T * V, hipMemcpyDeviceToHost));

  double e_lp = 0, e_ent = 0, e_dx = 0;
  for (int t = 0; t < T; ++t) {
    const float* r = x + (size_t)t * V;
    double mx = -1e300, sum = 0, ex = 0;
    for (int v = 0; v < V; ++v) mx = fmax(mx, (double)r[v] * inv_temperature);
    for (int v = 0; v < V; ++v) sum += exp((double)r[v] * inv_temperature - mx);
    const double lse = mx + log(sum);
    for (int v = 0; v < V; ++v) {
      const double z = (double)r[v] * inv_temperature;
      ex += exp(z - lse) * z;
    }
    e_lp = fmax(e_lp, fabs((double)lp[t] - ((double)r[y[t]] * inv_temperature - lse)));
    e_ent = fmax(e_ent, fabs((double)ent[t] - (lse - ex)));
    for (int v = 0; v < V; ++v) {
      const double z = (double)r[v] * inv_temperature, p = exp(z - lse);
      const double want = inv_temperature * (g_lp[t] * ((v == y[t] ? 1.0 : 0.0) - p) - g_h[t] * p * (z - ex));
      e_dx = fmax(e_dx, fabs((double)dx[(size_t)t * V + v] - want));
    }
  }
  /* the k largest of the T * V logits, marked by the selection step of the KL-Cov loss: exactly k marks, none of
   * them below an unmarked value */
  enum { K = 777 };
  float* d_marks;
  void* d_ws;
  const size_t ws_bytes = siirl_topk_mark_workspace_bytes();
  CK(hipMalloc((void**)&d_marks, sizeof(float) * T * V));
  CK(hipMalloc(&d_ws, ws_bytes));
  CALL(siirl_topk_mark(d_x, (int64_t)T * V, K, 1.0f, d_marks, d_ws, ws_bytes, stream));
  CK(hipStreamSynchronize(stream));
  if (siirl_topk_mark(d_x, (int64_t)T * V, (int64_t)T * V + 1, 1.0f, d_marks, d_ws, ws_bytes, stream) !=
      SIIRL_ERR_INVALID_ARGUMENT) {
    printf("FAIL k > n was accepted\n");
    return 6;
  }
  float* marks = (float*)malloc(sizeof(float) * T * V);
  CK(hipMemcpy(marks, d_marks, sizeof(float) * T * V, hipMemcpyDeviceToHost));
  int n_marked = 0;
  float lowest_marked = INFINITY, highest_unmarked = -INFINITY;
  for (int i = 0; i < T * V; ++i) {
    if (marks[i] != 0.0f) {
      ++n_marked;
      lowest_marked = fminf(lowest_marked, x[i]);
    } else {
      highest_unmarked = fmaxf(highest_unmarked, x[i]);
    }
  }
  const int ok_sel = n_marked == K && lowest_marked >= highest_unmarked;

  const int ok = e_lp < 1e-4 && e_ent < 1e-4 && e_dx < 1e-6 && ok_sel;
  printf("%s C ABI consumer: T=%d V=%d max |err| logprob %.2e entropy %.2e dlogits %.2e; top-%d pick: %d marked, "
         "lowest marked %.6f, highest unmarked %.6f\n", ok ? "OK" : "FAIL", T, V, e_lp, e_ent, e_dx, K, n_marked,
         (double)lowest_marked, (double)highest_unmarked);
  return ok ? 0 : 1;
}
