/*
 * A caller of libave_fp4.so written in plain C: no Python, no torch.  It allocates device buffers with the HIP
 * runtime, runs a small MXFP4 GEMM with unit scales through the C ABI and compares every bf16 result with the
 * integer-exact value computed here on the host (with unit scales all products are multiples of 0.25 and the sum
 * is exact in fp32, so the only rounding is the final one to bf16).  Exit status 0 and the line "abi_check: ok" on
 * success.  It stands for the binding a compiled-language host would use, which sees nothing but include/ave_fp4.h.
 */
#include <hip/hip_runtime_api.h>
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "../../../include/ave_fp4.h"

#define CHECK_HIP(x)                                                                        \
  do {                                                                                      \
    hipError_t e_ = (x);                                                                    \
    if (e_ != hipSuccess) {                                                                 \
      fprintf(stderr, "abi_check: HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__); \
      return 2;                                                                             \
    }                                                                                       \
  } while (0)

static const float kE2M1[8] = {0.0f, 0.5f, 1.0f, 1.5f, 2.0f, 3.0f, 4.0f, 6.0f};

static float decode_fp4(unsigned code) { return (code & 8) ? -kE2M1[code & 7] : kE2M1[code & 7]; }

/* fp32 -> bf16 bits, round to nearest even (finite inputs only) */
static uint16_t to_bf16(float x) {
  uint32_t u;
  memcpy(&u, &x, 4);
  u += 0x7FFFu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

int main(void) {
  enum { M = 96, N = 160, K = 512 };
  if (ave_fp4_abi_version() < 1) {
    fprintf(stderr, "abi_check: unexpected ABI version %d\n", ave_fp4_abi_version());
    return 1;
  }
  const size_t a_bytes = (size_t)M * K / 2, b_bytes = (size_t)N * K / 2;
  const size_t as_bytes = (size_t)M * K / 32, bs_bytes = (size_t)N * K / 32;
  uint8_t* a = (uint8_t*)malloc(a_bytes);
  uint8_t* b = (uint8_t*)malloc(b_bytes);
  uint16_t* c = (uint16_t*)malloc((size_t)M * N * 2);
  if (!a || !b || !c) return 1;
  uint32_t x = 2463534242u;
  for (size_t i = 0; i < a_bytes; ++i) { x ^= x << 13; x ^= x >> 17; x ^= x << 5; a[i] = (uint8_t)(x >> 11); }
  for (size_t i = 0; i < b_bytes; ++i) { x ^= x << 13; x ^= x >> 17; x ^= x << 5; b[i] = (uint8_t)(x >> 11); }

  uint8_t *dA, *dB, *dAs, *dBs;
  uint16_t* dC;
  CHECK_HIP(hipMalloc((void**)&dA, a_bytes));
  CHECK_HIP(hipMalloc((void**)&dB, b_bytes));
  CHECK_HIP(hipMalloc((void**)&dAs, as_bytes));
  CHECK_HIP(hipMalloc((void**)&dBs, bs_bytes));
  CHECK_HIP(hipMalloc((void**)&dC, (size_t)M * N * 2));
  CHECK_HIP(hipMemcpy(dA, a, a_bytes, hipMemcpyHostToDevice));
  CHECK_HIP(hipMemcpy(dB, b, b_bytes, hipMemcpyHostToDevice));
  CHECK_HIP(hipMemset(dAs, 127, as_bytes)); /* E8M0 127 = 2^0 */
  CHECK_HIP(hipMemset(dBs, 127, bs_bytes));

  /* a rejected argument is reported through the return value and ave_fp4_last_error() */
  if (ave_fp4_gemm_mxfp4(dA, dAs, dB, dBs, dC, M, N, 33, NULL) != AVE_FP4_EINVAL || !strstr(ave_fp4_last_error(), "multiple of 32")) {
    fprintf(stderr, "abi_check: K = 33 was not rejected as expected (\"%s\")\n", ave_fp4_last_error());
    return 1;
  }
  const int variants[3] = {AVE_FP4_AUTO, AVE_FP4_GENERIC, AVE_FP4_TILE};
  for (int v = 0; v < 3; ++v) {
    CHECK_HIP(hipMemset(dC, 0xFF, (size_t)M * N * 2));
    const int rc = ave_fp4_gemm_mxfp4_ex(dA, dAs, dB, dBs, dC, M, N, K, NULL /* default stream */, variants[v]);
    if (rc != 0) {
      fprintf(stderr, "abi_check: variant %d returned %d: %s\n", variants[v], rc, ave_fp4_last_error());
      return 1;
    }
    CHECK_HIP(hipDeviceSynchronize());
    CHECK_HIP(hipMemcpy(c, dC, (size_t)M * N * 2, hipMemcpyDeviceToHost));
    for (int m = 0; m < M; ++m)
      for (int n = 0; n < N; ++n) {
        float sum = 0.0f; /* exact: every term is a multiple of 0.25 below 36, K = 512 terms */
        for (int k = 0; k < K; ++k) {
          const unsigned ca = (a[(size_t)m * K / 2 + k / 2] >> (4 * (k & 1))) & 15u;
          const unsigned cb = (b[(size_t)n * K / 2 + k / 2] >> (4 * (k & 1))) & 15u;
          sum += decode_fp4(ca) * decode_fp4(cb);
        }
        if (c[(size_t)m * N + n] != to_bf16(sum)) {
          fprintf(stderr, "abi_check: variant %d, C[%d,%d] = 0x%04x, expected 0x%04x\n", variants[v], m, n,
                  c[(size_t)m * N + n], to_bf16(sum));
          return 1;
        }
      }
  }
  CHECK_HIP(hipFree(dA));
  CHECK_HIP(hipFree(dB));
  CHECK_HIP(hipFree(dAs));
  CHECK_HIP(hipFree(dBs));
  CHECK_HIP(hipFree(dC));
  free(a);
  free(b);
  free(c);
  printf("abi_check: ok\n");
  return 0;
}
