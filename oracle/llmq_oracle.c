/*
 * CPU restatement in C of the arithmetic on llm-quant's kernel path -- TEST INFRASTRUCTURE.
 * Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may load this
 * library; the shipped package never links or calls it.
 *
 * It exists for two things: a second, independently written statement of the numpy oracle
 * (oracle/llmq_oracle.py; tests compare the two bit for bit), and a CPU baseline that can be
 * timed on the GPU box's host cores. Each function names the reference source it follows.
 * bfloat16 tensors are passed as uint16 bit patterns.
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

static inline float bf16_to_f32(uint16_t b) {
  uint32_t u = (uint32_t)b << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

static inline uint16_t f32_to_bf16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return 0x7fc0;
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

int llmq_oracle_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

/* fake_quantize on contiguous groups (llmquant/core/quant_ops.py:26-37 with
 * llmquant/core/observers.py:74-98): fp32 in, fp32 out, optional scales. */
void llmq_oracle_fake_quant_f32(const float* x, float* out, float* scale_or_null, int64_t n_groups,
                                int group_size, int num_bits) {
  const float qmax = (float)((1 << (num_bits - 1)) - 1);
  const float qmin = -qmax - 1.0f;
#pragma omp parallel for schedule(static)
  for (int64_t g = 0; g < n_groups; ++g) {
    const float* xs = x + g * group_size;
    float amax = 0.0f;
    for (int i = 0; i < group_size; ++i) amax = fmaxf(amax, fabsf(xs[i]));
    const float scale = fmaxf(amax / qmax, 1e-8f);
    if (scale_or_null) scale_or_null[g] = scale;
    for (int i = 0; i < group_size; ++i) {
      const float q = fminf(fmaxf(rintf(xs[i] / scale), qmin), qmax);
      out[g * group_size + i] = q * scale;
    }
  }
}

/* Same, bfloat16 storage. */
void llmq_oracle_fake_quant_bf16(const uint16_t* x, uint16_t* out, float* scale_or_null,
                                 int64_t n_groups, int group_size, int num_bits) {
  const float qmax = (float)((1 << (num_bits - 1)) - 1);
  const float qmin = -qmax - 1.0f;
#pragma omp parallel for schedule(static)
  for (int64_t g = 0; g < n_groups; ++g) {
    const uint16_t* xs = x + g * group_size;
    float amax = 0.0f;
    for (int i = 0; i < group_size; ++i) amax = fmaxf(amax, fabsf(bf16_to_f32(xs[i])));
    const float scale = fmaxf(amax / qmax, 1e-8f);
    if (scale_or_null) scale_or_null[g] = scale;
    for (int i = 0; i < group_size; ++i) {
      const float q = fminf(fmaxf(rintf(bf16_to_f32(xs[i]) / scale), qmin), qmax);
      out[g * group_size + i] = f32_to_bf16(q * scale);
    }
  }
}

static inline int code_at(const uint8_t* qw, int64_t idx, int packed) {
  if (!packed) return (int8_t)qw[idx];
  const uint8_t byte = qw[idx >> 1];
  return (int)((idx & 1) ? (byte >> 4) : (byte & 0xf)) - 8; /* llmquant/packing/packing.py:20-33 */
}

/* RealQuantLinear.forward without activation quant (llmquant/quantizers/real.py:76-103):
 * for each group in order, partial = sum_k x[k]*q[k] in fp32 (k ascending), * scale, out += partial.
 * x bf16 [M, G*gs]; qw int8 [N, G, gs] or packed [N, G, gs/2]; ws fp32 [scale_rows, G];
 * out fp32 [M, N]. */
void llmq_oracle_real_gemv_bf16(const uint16_t* x, const uint8_t* qw, const float* ws, float* out,
                                int M, int N, int G, int gs, int out_group, int packed) {
  const int64_t K = (int64_t)G * gs;
#pragma omp parallel for schedule(static)
  for (int n = 0; n < N; ++n) {
    const int srow = out_group > 0 ? n / out_group : n;
    for (int m = 0; m < M; ++m) {
      float acc = 0.0f;
      for (int g = 0; g < G; ++g) {
        float partial = 0.0f;
        for (int k = 0; k < gs; ++k) {
          const int64_t idx = (int64_t)n * K + (int64_t)g * gs + k;
          partial += bf16_to_f32(x[(int64_t)m * K + (int64_t)g * gs + k]) * (float)code_at(qw, idx, packed);
        }
        partial = partial * ws[(int64_t)srow * G + g];
        acc = acc + partial;
      }
      out[(int64_t)m * N + n] = acc;
    }
  }
}

/* The A8 branch of the same forward: integer group sums (exact), then
 * float(sum) * s_w * s_x, each product rounded to fp32, added in group order.
 * a int8 [M, G*gs]; sx fp32 [M, G]. */
void llmq_oracle_real_gemm_a8(const int8_t* a, const float* sx, const uint8_t* qw, const float* ws,
                              float* out, int M, int N, int G, int gs, int out_group, int packed) {
  const int64_t K = (int64_t)G * gs;
#pragma omp parallel for schedule(static)
  for (int n = 0; n < N; ++n) {
    const int srow = out_group > 0 ? n / out_group : n;
    for (int m = 0; m < M; ++m) {
      float acc = 0.0f;
      for (int g = 0; g < G; ++g) {
        int32_t isum = 0;
        for (int k = 0; k < gs; ++k) {
          const int64_t idx = (int64_t)n * K + (int64_t)g * gs + k;
          isum += (int32_t)a[(int64_t)m * K + (int64_t)g * gs + k] * code_at(qw, idx, packed);
        }
        float partial = (float)isum;
        partial = partial * ws[(int64_t)srow * G + g];
        partial = partial * sx[(int64_t)m * G + g];
        acc = acc + partial;
      }
      out[(int64_t)m * N + n] = acc;
    }
  }
}
