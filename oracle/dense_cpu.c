/* TEST INFRASTRUCTURE (oracle) -- not part of the product path.
 *
 * Plain C restatement, in single precision, of the elementwise and row-wise parts of the two dense programs of the
 * benchmark (the modules reactant.jl_amd/programs.py:mlp and :fp8_linear write):
 *   bias + gelu (tanh form) after a matrix product, with the result rounded to bfloat16 where the module stores a
 *   bf16 tensor (reference ext/ReactantNNlibExt/Implementations.jl:11-26 for the dense layer, src/Ops.jl:1932-1961 for
 *   the conversions);
 *   softmax over the minor dimension (reference src/Ops.jl:4537-4546: max, subtract, exponential, sum, divide);
 *   the dequantizing scale of the FP8 product followed by the row-wise RMSNorm (x * rsqrt(mean(x^2) + eps)).
 * The matrix products themselves are numpy's sgemm (OpenBLAS) on operands decoded to float32.  Together they are the
 * CPU baseline of bench.py for these two programs on all host cores (OpenMP); tests/test_oracle_golden.py pins every
 * function here against the numpy interpreter on seeded data and against closed forms. */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <string.h>

/* float32 rounded to the nearest bfloat16 (ties to even), as a float32 */
static inline float round_bf16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return f; /* NaN */
  u += 0x7fffu + ((u >> 16) & 1u);
  u &= 0xffff0000u;
  memcpy(&f, &u, 4);
  return f;
}

/* h[r][c] = bf16(gelu_tanh(h[r][c] + b[c])): 0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3))) */
void rx_oracle_bias_gelu_bf16(float* h, const float* b, long long rows, long long cols) {
#pragma omp parallel for schedule(static)
  for (long long r = 0; r < rows; ++r) {
    float* p = h + r * cols;
    for (long long c = 0; c < cols; ++c) {
      const float x = p[c] + b[c];
      const float t = tanhf(0.7978845608028654f * (x + 0.044715f * (x * x * x)));
      p[c] = round_bf16(0.5f * x * (1.0f + t));
    }
  }
}

/* every row replaced by bf16(softmax(row)) */
void rx_oracle_softmax_rows_bf16(float* h, long long rows, long long cols) {
#pragma omp parallel for schedule(static)
  for (long long r = 0; r < rows; ++r) {
    float* p = h + r * cols;
    float m = p[0];
    for (long long c = 1; c < cols; ++c) m = p[c] > m ? p[c] : m;
    float s = 0.0f;
    for (long long c = 0; c < cols; ++c) {
      p[c] = expf(p[c] - m);
      s += p[c];
    }
    for (long long c = 0; c < cols; ++c) p[c] = round_bf16(p[c] / s);
  }
}

/* y = bf16(scale * acc), then every row y * rsqrt(mean(y^2) + eps), rounded to bf16 */
void rx_oracle_scale_rmsnorm_bf16(float* h, float scale, float eps, long long rows, long long cols) {
#pragma omp parallel for schedule(static)
  for (long long r = 0; r < rows; ++r) {
    float* p = h + r * cols;
    float s = 0.0f;
    for (long long c = 0; c < cols; ++c) {
      p[c] = round_bf16(scale * p[c]);
      s += p[c] * p[c];
    }
    const float k = 1.0f / sqrtf(s * (1.0f / (float)cols) + eps);
    for (long long c = 0; c < cols; ++c) p[c] = round_bf16(p[c] * k);
  }
}
