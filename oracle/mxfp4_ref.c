/* C restatement of the OCP MXFP4 decode and the dequantise-then-multiply GEMM.
 * TEST INFRASTRUCTURE ONLY: built by oracle/build_oracle.py into oracle/_build/libmxfp4_ref.so and
 * loaded only by tests and by the CPU-baseline leg of the benchmark.
 *
 * Format (OCP Microscaling Formats v1.0; type names f4e2m1fn / f8e8m0fnu as in
 * iree/turbine/kernel/_support/dtype.py:117,119): a code is sign(1) exponent(2, bias 1) mantissa(1);
 * a scale byte b means 2^(b-127), 0xFF = NaN; one scale per 32 consecutive k; two codes per byte,
 * even k in the low nibble. */
#include <math.h>
#include <stdint.h>
#include <string.h>

static float e2m1(unsigned c) {
  unsigned s = (c >> 3) & 1u, e = (c >> 1) & 3u, m = c & 1u;
  float mag = e == 0 ? 0.5f * (float)m : ldexpf(1.0f + 0.5f * (float)m, (int)e - 1);
  return s ? -mag : mag;
}

static float e8m0(unsigned b) { return b == 255u ? NAN : ldexpf(1.0f, (int)b - 127); }

void mxfp4_dequant_c(const uint8_t* codes, const uint8_t* scales, float* out, int64_t rows, int64_t K) {
  for (int64_t r = 0; r < rows; r++)
    for (int64_t k = 0; k < K; k++) {
      unsigned byte = codes[r * (K / 2) + k / 2];
      unsigned c = (k & 1) ? (byte >> 4) : (byte & 15u);
      out[r * K + k] = e2m1(c) * e8m0(scales[r * (K / 32) + k / 32]);
    }
}

/* C[M,N] = dq(A) . dq(B)^T, double accumulation, float result.  Scalar, single thread. */
void mxfp4_gemm_c(const uint8_t* a, const uint8_t* as, const uint8_t* b, const uint8_t* bs, float* c, int64_t M, int64_t N,
                  int64_t K) {
  for (int64_t i = 0; i < M; i++)
    for (int64_t j = 0; j < N; j++) {
      double acc = 0.0;
      for (int64_t kb = 0; kb < K / 32; kb++) {
        double part = 0.0;
        for (int64_t k = kb * 32; k < kb * 32 + 32; k++) {
          unsigned ba = a[i * (K / 2) + k / 2], bb = b[j * (K / 2) + k / 2];
          unsigned ca = (k & 1) ? (ba >> 4) : (ba & 15u), cb = (k & 1) ? (bb >> 4) : (bb & 15u);
          part += (double)e2m1(ca) * (double)e2m1(cb);
        }
        acc += part * (double)e8m0(as[i * (K / 32) + kb]) * (double)e8m0(bs[j * (K / 32) + kb]);
      }
      c[i * N + j] = (float)acc;
    }
}
