/*
 * TEST INFRASTRUCTURE ONLY - plain C restatement of the reference's FP8 block-scaled GEMM, independent of torch.
 *
 * Follows fp8_gemm_kernel, dlblas/kernels/fp8_gemm.py:49-60: for every 128-wide K block the e4m3 products are
 * summed in fp32, the block sum is multiplied by a_s[m, kb] and then by b_s[n / 128, kb] (the order of :55) and
 * added to the fp32 accumulator; one conversion at the end.  The decode is the OCP E4M3 "fn" format definition
 * (bias 7, subnormals m/8 * 2^-6, S.1111.111 = NaN, no infinities).
 *
 * Built by oracle/build_oracle.py into oracle/_build/libfp8_gemm_oracle.so and used by tests/ only.
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

float dlb_oracle_e4m3fn_to_f32(uint8_t code) {
  const int sign = code >> 7;
  const int exp = (code >> 3) & 0xF;
  const int man = code & 0x7;
  float mag;
  if (exp == 0xF && man == 0x7) return NAN;
  if (exp == 0)
    mag = ldexpf((float)man, -9);
  else
    mag = ldexpf((float)(8 + man), exp - 10);
  return sign ? -mag : mag;
}

/* c[M, N] (fp32) = block-scaled product of a[M, K], b[N, K] (e4m3fn bytes), a_s[M, KB], b_s[NB, KB]. */
void dlb_oracle_fp8_gemm(const uint8_t* a, const uint8_t* b, const float* a_s, const float* b_s, float* c,
                         int64_t M, int64_t N, int64_t K) {
  const int64_t kblocks = (K + 127) / 128;
  float table[256];
  for (int i = 0; i < 256; ++i) table[i] = dlb_oracle_e4m3fn_to_f32((uint8_t)i);
  for (int64_t m = 0; m < M; ++m) {
    for (int64_t n = 0; n < N; ++n) {
      float acc = 0.0f;
      for (int64_t kb = 0; kb < kblocks; ++kb) {
        const int64_t k1 = (kb + 1) * 128 < K ? (kb + 1) * 128 : K;
        float dot = 0.0f;
        for (int64_t k = kb * 128; k < k1; ++k) dot += table[a[m * K + k]] * table[b[n * K + k]];
        acc += dot * a_s[m * kblocks + kb] * b_s[(n / 128) * kblocks + kb];
      }
      c[m * N + n] = acc;
    }
  }
}

/* fp32 -> bf16 bits, round to nearest even (NaN stays NaN); used to restate the final cast. */
uint16_t dlb_oracle_f32_to_bf16(float x) {
  uint32_t u;
  memcpy(&u, &x, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}
