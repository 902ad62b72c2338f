/*
 * jitllm_oracle.h -- CPU restatement of jitLLM's Java CPU quantized matmul.
 *
 * TEST INFRASTRUCTURE ONLY.  This library is the checker the HIP path is held
 * against.  Nothing in the shipped package links, loads or calls it; only the
 * test-suite, the smoke check and the benchmark's cpu_baseline leg do.
 *
 * Every function names the reference source (paths relative to the reference
 * checkout, J = src/main/java/org/beehive/jitllm) it restates.
 */
#ifndef JITLLM_ORACLE_H
#define JITLLM_ORACLE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ggml type ids, the numbering GGUF files carry (J/format/GGMLType.java:7,13,18 by ordinal). */
enum { JO_Q4_0 = 2, JO_Q4_1 = 3, JO_Q5_0 = 6, JO_Q8_0 = 8, JO_Q4_K = 12, JO_Q5_K = 13, JO_Q6_K = 14, JO_IQ4_XS = 23 };

/* dot flavours: which branch of Q8_0FloatTensor.dot / Q4_0FloatTensor.dot runs.  JO_DOT_Q8ACT is
 * Q8_0FloatTensor's -Djitllm.quantizeActivation=true branch (activations quantized per block of 32,
 * integer sums); the other types have no such branch and read it as JO_DOT_SCALAR. */
enum { JO_DOT_SCALAR = 0, JO_DOT_Q8ACT = 8, JO_DOT_VEC128 = 128, JO_DOT_VEC256 = 256 };

int jo_block_elems(int type);  /* 32 / 32 / 256 / 256 */
int jo_block_bytes(int type);  /* 18 / 34 / 144 / 210 */

float    jo_f16_to_f32(uint16_t bits);
uint16_t jo_f32_to_f16(float value);

float jo_get_float(int type, const uint8_t *w, int64_t index);
void  jo_dequant(int type, const uint8_t *w, int64_t n, float *out);

/* second, independently worded decoders (the device-side statements in the reference) */
float jo_get_float_alt(int type, const uint8_t *w, int64_t index);

float jo_dot(int type, int flavour, const uint8_t *w, int64_t this_offset,
             const float *x, int64_t that_offset, int64_t size);

/* out[i] = dot(i*dim1, x, 0, dim1), i in [0, dim0); rows spread over nthreads. */
void jo_matmul(int type, int flavour, const uint8_t *w, const float *x, float *out,
               int dim0, int dim1, int nthreads);

/* out[b*dim0 + i] = dot(i*dim1, X + b*dim1, 0, dim1), flat index spread over nthreads. */
void jo_matmul_batch(int type, int flavour, const uint8_t *w, const float *X, float *out,
                     int context, int dim0, int dim1, int nthreads);

/* gate[i] = gate[i] / (float)(1.0 + exp(-gate[i])) * up[i] */
void jo_swiglu(float *gate, const float *up, int64_t n);

/* RMS normalisation as the host path computes it, and the first maximum of a vector */
float   jo_rms_scale(const float *x, int64_t n, float eps);
void    jo_rmsnorm(float *out, const float *x, const float *weight, int64_t n, float eps);
int64_t jo_argmax(const float *x, int64_t n);
/* the batched prefill's RMS reduction (parallel order, local size 256) and fp16 apply */
void    jo_batched_rms_apply_f16(float *x, const float *delta, const float *weight, float eps, int64_t rows,
                                 int64_t n, float *scales, uint16_t *out);

/* per-32-block int8 quantisation of activations and the block-scaled int8 GEMM arithmetic */
void jo_quantize_q8(const float *x, int8_t *q, float *scales, int64_t rows, int64_t k);
void jo_gemm_int8_block_scaled(int type, const int8_t *aq, const float *ascale, const uint8_t *w,
                               float *out, int m, int n, int k, int nthreads);

/* The packed-integer decode path: activation quantiser and the projections over it. */
void jo_quantize_q8_blocks(const float *x, int64_t n, int8_t *q, float *scales, int32_t *sums);
void jo_matmul_q8x(int type, const uint8_t *w, const int8_t *q, const float *scales, const int32_t *sums,
                   float *out, int dim0, int dim1, int nthreads);

/* java.util.Random */
typedef struct { int64_t seed; double next_next_gaussian; int have_next_next_gaussian; } jo_jrandom;
void    jo_jrandom_init(jo_jrandom *r, int64_t seed);
int32_t jo_jrandom_next_int(jo_jrandom *r);
int32_t jo_jrandom_next_int_bound(jo_jrandom *r, int32_t bound);
int     jo_jrandom_next_boolean(jo_jrandom *r);
double  jo_jrandom_next_gaussian(jo_jrandom *r);
void    jo_jrandom_next_bytes(jo_jrandom *r, uint8_t *out, int64_t n);
int32_t jo_java_string_hash(const char *s);

int jo_max_threads(void);

#ifdef __cplusplus
}
#endif
#endif
