/*
 * swiglu_oracle.c — CPU restatement of the reference's SwiGLU formulation. TEST INFRASTRUCTURE ONLY:
 * nothing in the shipped library or its bindings links, loads or calls this file; it is the checker the
 * tests, the smoke run and the benchmark's cpu_baseline leg compare the HIP path against.
 *
 * What it restates (bit-ml/Fused-SwiGLU):
 *   numeric_tests.py:41-43   C = A @ B.T ; gated = C[:, ::2] * silu(C[:, 1::2])
 *   swiglu.cu:380-381        same pairing in the kernel: even column = linear operand, odd column = SiLU operand,
 *                            product and SiLU in fp32, one rounding afterwards
 *   swiglu.cu:96             silu(x) = x / (1 + exp(-x))
 *   swiglu.cu:538-553        shapes: X [M,K], W1W3 [N,K], out [M,N/2]
 *   swiglu.cu:73-75          fp32 -> bf16 is round-to-nearest-even
 * and the `@ Wd` step the reference lacks: Y = H @ W2.T with W2 [D, FF].
 *
 * Arithmetic: inputs are the 16-bit encodings the GPU sees, decoded exactly; dot products accumulate in
 * double (so the result is the correctly rounded value of the real-number formula to far below the test
 * tolerances); outputs are double, unrounded. Rounding helpers are provided separately.
 *
 * Parity pinning: the reference ships no golden vectors for this path (numeric_tests.py asserts nothing), so
 * these functions are pinned by tests/test_oracle.py against brute-force Python loops on tiny shapes, closed
 * forms of SiLU, one-hot probes of the even/odd convention, and torch fp64 matmul.
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

#define ORACLE_BF16 0
#define ORACLE_FP16 1

float oracle_bf16_to_f32(uint16_t h) {
  uint32_t u = ((uint32_t)h) << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

float oracle_f16_to_f32(uint16_t h) {
  const uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
  const uint32_t exp = (h >> 10) & 0x1f;
  const uint32_t man = h & 0x3ff;
  uint32_t u;
  if (exp == 0) {
    if (man == 0) {
      u = sign;
    } else { /* subnormal: value = man * 2^-24 */
      float f = (float)man * 5.9604644775390625e-08f;
      memcpy(&u, &f, 4);
      u |= sign;
    }
  } else if (exp == 31) {
    u = sign | 0x7f800000u | (man << 13);
  } else {
    u = sign | ((exp + 112) << 23) | (man << 13);
  }
  float f;
  memcpy(&f, &u, 4);
  return f;
}

/* round-to-nearest-even, NaN kept quiet (the behaviour of cute::bfloat16_t(float), swiglu.cu:73-75) */
uint16_t oracle_f32_to_bf16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

/* round-to-nearest-even fp32 -> fp16 with subnormals and overflow to infinity */
uint16_t oracle_f32_to_f16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  const uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
  const uint32_t a = u & 0x7fffffffu;
  if (a > 0x7f800000u) return (uint16_t)(sign | 0x7e00u);
  if (a >= 0x47800000u) return (uint16_t)(sign | 0x7c00u); /* >= 65536 -> inf (65520 rounds up below) */
  if (a < 0x33000000u) return sign;                        /* < 2^-25 -> 0 */
  int32_t e = (int32_t)(a >> 23) - 127;
  uint32_t m = (a & 0x7fffffu) | 0x800000u; /* 24-bit significand */
  int shift;                                 /* bits dropped from m */
  uint32_t base;
  if (e < -14) { /* subnormal result: value = m * 2^(e-23), unit 2^-24 */
    shift = -e - 1; /* 13 + (-14 - e) */
    base = 0;
  } else {
    shift = 13;
    base = (uint32_t)(e + 15) << 10;
    m &= 0x7fffffu;
  }
  uint32_t q = m >> shift;
  const uint32_t rem = m & ((1u << shift) - 1u);
  const uint32_t half = 1u << (shift - 1);
  if (rem > half || (rem == half && (q & 1u))) q++;
  return (uint16_t)(sign | (base + q)); /* carries ripple into the exponent, reaching 0x7c00 = inf at the top */
}

static double decode(int dtype, uint16_t v) {
  return dtype == ORACLE_BF16 ? (double)oracle_bf16_to_f32(v) : (double)oracle_f16_to_f32(v);
}

double oracle_silu(double x) { return x / (1.0 + exp(-x)); } /* swiglu.cu:96 */

/* H[m, j] = (X[m,:] . W13[2j,:]) * silu(X[m,:] . W13[2j+1,:]); N = number of W13 rows (even). Returns 0, or -1
 * on a bad argument. */
int oracle_gateup(int dtype, int64_t M, int64_t N, int64_t K, const uint16_t* X, int64_t ldx, const uint16_t* W13,
                  int64_t ldw, double* H, int64_t ldh) {
  if ((dtype != ORACLE_BF16 && dtype != ORACLE_FP16) || M < 0 || N < 0 || (N & 1) || K < 0) return -1;
  for (int64_t m = 0; m < M; ++m) {
    for (int64_t j = 0; j < N / 2; ++j) {
      double up = 0.0, gate = 0.0;
      const uint16_t* x = X + m * ldx;
      const uint16_t* wu = W13 + (2 * j) * ldw;
      const uint16_t* wg = W13 + (2 * j + 1) * ldw;
      for (int64_t k = 0; k < K; ++k) {
        const double xv = decode(dtype, x[k]);
        up += xv * decode(dtype, wu[k]);
        gate += xv * decode(dtype, wg[k]);
      }
      H[m * ldh + j] = up * oracle_silu(gate);
    }
  }
  return 0;
}

/* Y[m, n] = H[m,:] . W2[n,:] with H given in double (the unrounded intermediate of the fp32 formulation). */
int oracle_down_f64(int dtype, int64_t M, int64_t D, int64_t FF, const double* H, int64_t ldh, const uint16_t* W2,
                    int64_t ldw2, double* Y, int64_t ldy) {
  if ((dtype != ORACLE_BF16 && dtype != ORACLE_FP16) || M < 0 || D < 0 || FF < 0) return -1;
  for (int64_t m = 0; m < M; ++m)
    for (int64_t n = 0; n < D; ++n) {
      double acc = 0.0;
      for (int64_t k = 0; k < FF; ++k) acc += H[m * ldh + k] * decode(dtype, W2[n * ldw2 + k]);
      Y[m * ldy + n] = acc;
    }
  return 0;
}

/* Same with H given as 16-bit elements (the down projection on its own, as fsw_down sees it). */
int oracle_down(int dtype, int64_t M, int64_t D, int64_t FF, const uint16_t* H, int64_t ldh, const uint16_t* W2,
                int64_t ldw2, double* Y, int64_t ldy) {
  if ((dtype != ORACLE_BF16 && dtype != ORACLE_FP16) || M < 0 || D < 0 || FF < 0) return -1;
  for (int64_t m = 0; m < M; ++m)
    for (int64_t n = 0; n < D; ++n) {
      double acc = 0.0;
      for (int64_t k = 0; k < FF; ++k) acc += decode(dtype, H[m * ldh + k]) * decode(dtype, W2[n * ldw2 + k]);
      Y[m * ldy + n] = acc;
    }
  return 0;
}
