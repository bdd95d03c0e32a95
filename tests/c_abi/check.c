/* A caller of libfcr.so that knows nothing of Python or torch: plain HIP runtime calls and the C ABI of
 * include/fcr.h.  With all-zero queries every visible key of a row gets the same weight, so the results
 * have closed forms (the ones tests/golden/closed_forms.json holds as rationals):
 *   without the mask  sum[j] = M / N, max[j] = 1 / N
 *   with the mask     sum[j] = H(N) - H(max(j, c)), max[j] = 1 / (max(j, c) + 1), c = max(N - M, 0),
 *                     H(n) = 1 + 1/2 + .. + 1/n, H(0) = 0   (row i sees i + c + 1 keys)
 * Prints "ok" and returns 0 when every value agrees to 2e-5 relative. */
#include <hip/hip_runtime_api.h>
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>

#include "fcr.h"

#define CHECK_HIP(x)                                                        \
  do {                                                                      \
    hipError_t e_ = (x);                                                    \
    if (e_ != hipSuccess) {                                                 \
      fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_));               \
      return 2;                                                             \
    }                                                                       \
  } while (0)

/* the closed form of column j */
static double closed_form(int red, int causal, int M, int N, int j) {
  const int c = N > M ? N - M : 0;
  if (!causal) return red == FCR_REDUCE_SUM ? (double)M / N : 1.0 / N;
  const int first = j > c ? j : c;   /* the first row that sees key j is row first - c, with first + 1 keys */
  if (red != FCR_REDUCE_SUM) return 1.0 / (first + 1);
  double want = 0.0;
  for (int n = first + 1; n <= (M <= N ? N : M + c); ++n) want += (n <= N) ? 1.0 / n : 1.0 / N;
  return want;
}

static int run_case(int B, int H, int M, int N, int D, int causal) {
  const size_t qn = (size_t)B * H * M * D, kn = (size_t)B * H * N * D, on = (size_t)B * H * N;
  uint16_t* hk = (uint16_t*)malloc(kn * 2);
  float* ho = (float*)malloc(on * 4);
  for (size_t i = 0; i < kn; ++i) hk[i] = (uint16_t)(0x3c00 + (i * 2654435761u) % 512);  /* fp16 values in [1, 1.5) */
  void *q, *k;
  float *out, *lse;
  CHECK_HIP(hipMalloc(&q, qn * 2));
  CHECK_HIP(hipMalloc(&k, kn * 2));
  CHECK_HIP(hipMalloc((void**)&out, on * 4));
  CHECK_HIP(hipMalloc((void**)&lse, fcr_lse_bytes(B, H, M, N, D)));
  CHECK_HIP(hipMemset(q, 0, qn * 2));
  CHECK_HIP(hipMemcpy(k, hk, kn * 2, hipMemcpyHostToDevice));
  const int64_t qs[4] = {(int64_t)H * M * D, (int64_t)M * D, D, 1}, ks[4] = {(int64_t)H * N * D, (int64_t)N * D, D, 1};
  int bad = 0;
  for (int red = FCR_REDUCE_SUM; red <= FCR_REDUCE_MAX; ++red) {
    const int rc = fcr_colreduce(q, k, out, lse, FCR_DTYPE_F16, B, H, M, N, D, qs, ks, 0.125f, red, causal, NULL);
    if (rc != 0) {
      fprintf(stderr, "fcr_colreduce: %d %s\n", rc, fcr_last_error());
      return 3;
    }
    CHECK_HIP(hipDeviceSynchronize());
    CHECK_HIP(hipMemcpy(ho, out, on * 4, hipMemcpyDeviceToHost));
    for (int j = 0; j < N; ++j) {
      const double want = closed_form(red, causal, M, N, j);
      for (int bh = 0; bh < B * H; ++bh) {
        const double got = ho[(size_t)bh * N + j];
        if (!(fabs(got - want) <= 2e-5 * want)) {
          if (bad++ < 5) fprintf(stderr, "B%d H%d M%d N%d causal%d red%d bh%d j%d: got %.9g want %.9g\n", B, H, M, N, causal, red, bh, j, got, want);
        }
      }
    }
  }
  /* sums and maxima from one call, and the word that says whether every workgroup of a single sweep met its team */
  {
    float* out2;
    CHECK_HIP(hipMalloc((void**)&out2, on * 4));
    const int rc = fcr_colreduce_sum_max(q, k, out, out2, lse, FCR_DTYPE_F16, B, H, M, N, D, qs, ks, 0.125f, causal, NULL);
    if (rc != 0) {
      fprintf(stderr, "fcr_colreduce_sum_max: %d %s\n", rc, fcr_last_error());
      return 3;
    }
    const int st = fcr_colreduce_status(lse, FCR_DTYPE_F16, B, H, M, N, D, NULL);
    if (st != 0) {
      fprintf(stderr, "fcr_colreduce_status: %d %s\n", st, fcr_last_error());
      return 3;
    }
    for (int red = FCR_REDUCE_SUM; red <= FCR_REDUCE_MAX; ++red) {
      CHECK_HIP(hipMemcpy(ho, red == FCR_REDUCE_SUM ? out : out2, on * 4, hipMemcpyDeviceToHost));
      for (int j = 0; j < N; j += (N > 7 ? N / 7 : 1)) {
        const double want = closed_form(red, causal, M, N, j), got = ho[(size_t)(B * H - 1) * N + j];
        if (!(fabs(got - want) <= 2e-5 * want)) {
          if (bad++ < 5) fprintf(stderr, "sum_max B%d H%d M%d N%d causal%d red%d j%d: got %.9g want %.9g\n", B, H, M, N, causal, red, j, got, want);
        }
      }
    }
    CHECK_HIP(hipFree(out2));
  }
  CHECK_HIP(hipFree(q));
  CHECK_HIP(hipFree(k));
  CHECK_HIP(hipFree(out));
  CHECK_HIP(hipFree(lse));
  free(hk);
  free(ho);
  return bad ? 1 : 0;
}

int main(void) {
  if (fcr_version() != FCR_VERSION) {
    fprintf(stderr, "header %d, library %d\n", FCR_VERSION, fcr_version());
    return 4;
  }
  int rc = 0;
  rc |= run_case(1, 2, 96, 160, 64, 0);
  rc |= run_case(2, 3, 96, 160, 64, 1);
  rc |= run_case(1, 2, 300, 300, 128, 1);
  rc |= run_case(1, 4, 64, 5000, 128, 1);
  rc |= run_case(1, 1, 200, 120, 32, 1);   /* more queries than keys: c = 0, rows beyond N see all keys */
  if (rc == 0) printf("ok\n");
  return rc;
}
