/*
 * CPU oracle for the quantized-weight matmul path. TEST INFRASTRUCTURE ONLY.
 *
 * This is a plain-C restatement of the reference's CPU algorithms (and of the integer block
 * dots its device primitives define). It exists so the HIP kernels have something exact to
 * be compared with. Nothing in the shipped library links, loads or calls it: only tests,
 * the smoke check and the benchmark's cpu_baseline leg do, and only as the checker.
 *
 * Pinning status of each function (what fixes its answers independently of this file):
 *   yvo_f16_decode / yvo_f16_encode / yvo_bf16_*   exhaustive 65 536-code round trips, RNE tie
 *                                                  cases (tests/unit/quant_numeric.c:188-259),
 *                                                  and the compiled reference (oracle/_ref).
 *   yvo_decode_block Q8_0 / Q2_K / IQ2_XXS / MXFP4 golden bytes (quant_numeric.c:502-609),
 *                                                  the compiled reference on random blocks.
 *   yvo_decode_block Q4_K                          PARITY UNPINNED by the reference (it has no
 *                                                  Q4_K codec). Pinned only by the public ggml
 *                                                  block_q4_K definition restated here, closed
 *                                                  forms and brute force in the tests.
 *   yvo_cpu_dot                                    compiled reference yvex_quant_cpu_dot,
 *                                                  numpy float64 brute force.
 *   yvo_q8k_quantize                               closed forms (zero block, spike, sign tie);
 *                                                  the reference has no CPU entry point for it.
 *   yvo_block_dot_*                                exact integer definitions, numpy int64 brute
 *                                                  force.
 *   yvo_block_dot_float                            float32 re-evaluation of the device primitive's
 *                                                  expression step by step (an exact-rational fused
 *                                                  multiply-add for Q8_0), against which other
 *                                                  orders of the same operations are shown to differ.
 *   yvo_q8_row_dot / yvo_q8_matvec                 block floats added in double in block order
 *                                                  (recomputed in the test; a float accumulator is
 *                                                  told apart), and the reference's own bound for
 *                                                  its Q8_K-activation kernels: 1e-5 (1 + |x|) of
 *                                                  yvo_cpu_dot on the dequantised activations
 *                                                  (tests/unit/cuda/quant_qtype.c:402,419-421).
 *   yvo_moe_route (sqrt_softplus)                  compiled reference yvex_moe_route_cpu and the
 *                                                  expectations of tests/unit/runtime_moe.c:105-150.
 *   yvo_moe_route (sigmoid)                        PARITY UNPINNED by the reference (not in it);
 *                                                  closed form only.
 *   yvo_moe_expert / yvo_moe_layer                 compiled reference yvex_moe_expert_cpu, the
 *                                                  exact-equality case runtime_moe.c:178-212; with
 *                                                  Q8_K activations the composition of the pinned
 *                                                  pieces rebuilt in the test (quantize, row dots,
 *                                                  double SwiGLU with the clamp active, bfloat16
 *                                                  roundings, route, float sum over the ranks,
 *                                                  shared expert), with plausible slips shown to
 *                                                  give other bits.
 *   yvo_worklist_build                             properties (stable sort, sums) and the cases of
 *                                                  tests/unit/expert_worklist.c.
 *   yvo_argmax_f32                                 brute force over small rows (largest value, its
 *                                                  first position, its multiplicity) and rows built
 *                                                  with known ties; the reference holds no fixture
 *                                                  for its selection kernel.
 */
#ifndef YVEX_ORACLE_H
#define YVEX_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Status values, equal to the reference's yvex_status (include/yvex/core.h:13-26). */
enum {
    YVO_OK = 0,
    YVO_ERR = -1,
    YVO_ERR_NOMEM = -2,
    YVO_ERR_IO = -3,
    YVO_ERR_FORMAT = -4,
    YVO_ERR_UNSUPPORTED = -5,
    YVO_ERR_BACKEND = -6,
    YVO_ERR_BOUNDS = -7,
    YVO_ERR_STATE = -8,
    YVO_ERR_CANCELLED = -9,
    YVO_ERR_INVALID_ARG = -10,
    YVO_ERR_TIMEOUT = -11
};

/* GGUF qtype IDs used on this path (include/yvex/qtype.h:19-63). */
enum {
    YVO_QTYPE_F32 = 0,
    YVO_QTYPE_F16 = 1,
    YVO_QTYPE_Q8_0 = 8,
    YVO_QTYPE_Q2_K = 10,
    YVO_QTYPE_Q4_K = 12,
    YVO_QTYPE_Q8_K = 15,
    YVO_QTYPE_IQ2_XXS = 16,
    YVO_QTYPE_I32 = 26,
    YVO_QTYPE_BF16 = 30,
    YVO_QTYPE_MXFP4 = 39,
    YVO_QTYPE_COUNT = 43
};

enum { YVO_SCORING_SQRT_SOFTPLUS = 0, YVO_SCORING_SIGMOID = 1 };

/* Scalar rules: src/gguf/quant_scalar.c:40-143. */
float yvo_f16_decode(uint16_t bits);
uint16_t yvo_f16_encode(float value);
float yvo_bf16_decode(uint16_t bits);
uint16_t yvo_bf16_encode(float value);
float yvo_bf16_round(float value);
float yvo_e8m0_decode(uint8_t bits);

/* Geometry: src/gguf/qtype.c:15-104. Returns 0 for an unknown ID. */
int yvo_qtype_geometry(unsigned int qtype, unsigned int *block_size, unsigned int *block_bytes);
/* 1 when the reference's CPU row dot admits the qtype (src/gguf/quant_registry.c:50-103). */
int yvo_qtype_reference_cpu_compute(unsigned int qtype);
/* 1 when this build admits the qtype: the reference's set plus the Q4_K extension row. */
int yvo_qtype_admitted(unsigned int qtype);

/* Block codecs: src/gguf/quant_block.c:160-186 (Q8_0 encode), :715-881 (decode). */
int yvo_q8_0_encode_block(const float *source, uint8_t *encoded);
int yvo_decode_block(unsigned int qtype, const uint8_t *encoded, float *out);

/* Row dot: src/gguf/quant_compute.c:116-181. */
int yvo_cpu_dot(unsigned int qtype, const uint8_t *encoded, size_t encoded_bytes,
                const float *vector, uint64_t elements, float *out);
/* out[input_row * row_count + row]; rows walked exactly like src/graph/moe.c:430-444. */
int yvo_matvec(unsigned int qtype, const uint8_t *encoded, uint64_t row_count,
               uint64_t row_width, const float *input, uint64_t input_rows, float *out);
/* Same, rows split over `threads` pthreads with identical per-row arithmetic. */
int yvo_matvec_threads(unsigned int qtype, const uint8_t *encoded, uint64_t row_count,
                       uint64_t row_width, const float *input, uint64_t input_rows,
                       float *out, unsigned int threads);
/* Decode whole rows to float (gather / row decode: kernels.cu:784-830). */
int yvo_decode_rows(unsigned int qtype, const uint8_t *encoded, uint64_t row_width,
                    const uint32_t *row_ids, uint64_t selected, float *out);

/* Q8_K activation quantizer: src/backend/cuda/kernels.cu:436-489 and the host twin
 * tests/unit/cuda/quant_qtype.c:161-186. `values` holds rows*width floats, width % 256 == 0.
 * Returns YVO_ERR_FORMAT when a value is not finite. */
int yvo_q8k_quantize(const float *values, uint64_t rows, uint64_t width, uint8_t *encoded);
void yvo_q8k_dequantize(const uint8_t *encoded, uint64_t blocks, float *out);

/* Integer block dots: src/backend/cuda/kernel_primitives.h:287-313 (IQ2_XXS), :342-359
 * (Q8_0), :314-341 (Q2_K); Q4_K follows the same shape over the ggml block_q4_K layout. */
int32_t yvo_block_dot_iq2xxs_q8k(const uint8_t *weight66, const uint8_t *act292);
void yvo_block_dot_q8_0_q8k(const uint8_t *weight8x34, const uint8_t *act292, int32_t dots[8]);
void yvo_block_dot_q4k_q8k(const uint8_t *weight144, const uint8_t *act292, int32_t *dot,
                           int32_t *minimum);
void yvo_block_dot_q2k_q8k(const uint8_t *weight84, const uint8_t *act292, int32_t *dot,
                           int32_t *minimum);
/* One weight superblock (or eight Q8_0 blocks) times one Q8_K block, float result with the
 * float operations in the order the reference's device primitive uses. */
float yvo_block_dot_float(unsigned int qtype, const uint8_t *weight, const uint8_t *act292);
/* Row result on Q8_K activations: per-block floats summed in double in block order. */
int yvo_q8_row_dot(unsigned int qtype, const uint8_t *encoded_row, uint64_t row_width,
                   const uint8_t *act_row, float *out);
int yvo_q8_matvec(unsigned int qtype, const uint8_t *encoded, uint64_t row_count,
                  uint64_t row_width, const uint8_t *act, uint64_t input_rows, float *out);

/* Router: src/graph/moe.c:497-585. logits has `experts` floats; bias may be NULL (zeros). */
int yvo_moe_route(const float *logits, const float *bias, uint64_t experts, uint64_t topk,
                  int scoring, int normalize, double scaling, float *scores,
                  uint64_t *selected, float *weights);
/* Hash router (moe.c:539-559): the token's row of the I32 table names the experts; an ordinal
 * outside the expert range or a repeated one is FORMAT, a token outside the table is BOUNDS.
 * Pinned by tests/unit/runtime_moe.c:152-170 and a fixture from the compiled reference. */
int yvo_moe_route_hash(const float *logits, const int32_t *table, uint64_t table_rows,
                       uint64_t table_row_bytes, uint64_t token, uint64_t experts, uint64_t topk,
                       int scoring, int normalize, double scaling, float *scores_out,
                       uint64_t *selected, float *weights);

/* Expert FFN: src/graph/moe.c:587-622. Weight matrices are encoded rows; gate/up are
 * [intermediate x hidden], down is [hidden x intermediate]. `intermediate_out` (may be NULL)
 * receives the bf16-rounded SwiGLU vector; `unrounded_out` (may be NULL) receives the down
 * projection before its bf16 round. act_q8 = 1 routes both projections through Q8_K
 * quantization of their inputs and yvo_q8_matvec (device contract); 0 is the reference's
 * CPU path. */
int yvo_moe_expert(unsigned int gate_qtype, const uint8_t *gate, unsigned int up_qtype,
                   const uint8_t *up, unsigned int down_qtype, const uint8_t *down,
                   uint64_t hidden, uint64_t intermediate, const float *input,
                   float route_weight, double activation_limit, int act_q8, float *output,
                   float *intermediate_out, float *unrounded_out);

/* Expert-major worklist: src/graph/worklist.c:369-441. Arrays sized pair_count (pairs) and
 * expert_count (+1 for offsets). Returns the bucket count through *bucket_count. */
int yvo_worklist_build(const uint64_t *selected_experts, const float *route_weights,
                       uint64_t pair_count, uint64_t experts_per_row, uint64_t expert_count,
                       uint64_t *expert_ids, uint64_t *bucket_offsets,
                       uint64_t *bucket_populations, uint64_t *source_pairs,
                       uint64_t *source_rows, uint64_t *destination_rows,
                       float *ordered_weights, uint64_t *bucket_count);

/* Greedy selection per row: src/backend/cuda/kernels.cu:59-110 (yvex_argmax_f32). The reference
 * scans a row with 128 strided threads and merges them in a tree; "larger wins, equal keeps the
 * lower index and adds the counts" is associative and commutative, so one serial pass gives the
 * same three numbers. Returns 1 (and leaves that row's outputs untouched) when a row holds a
 * non-finite value, as the kernel raises status 1. */
int yvo_argmax_f32(const float *values, uint64_t row_count, uint64_t row_width,
                   uint32_t *selected_tokens, float *selected_values, uint64_t *tie_counts);

/* Residual-stream envelope around the expert math (dense strides; tokens x streams x width).
 * yvo_rms_norm: src/graph/numeric.c:630-666. yvo_mhc_pre: numeric.c:691-826 (sigmoid, Sinkhorn,
 * ingress; collapsed is bf16-rounded as the compute contract asks). yvo_mhc_post:
 * numeric.c:828-877. yvo_moe_ffn_prepare: src/graph/moe.c:446-495 (mixes through the CPU row
 * dot, ingress, weighted RMS norm, bf16 publication) with scale, base and norm already decoded.
 * Pinned by the reference's own vectors (tests/unit/deepseek_attention.c:2255-2266,2302-2309 and
 * tests/reference/deepseek_attention.c:2725-2730), by float64 closed forms (doubly-stochastic
 * combination, einsum egress, sigmoid limits) and by a fixture written from the compiled
 * reference's yvex_moe_ffn_prepare_cpu. */
int yvo_rms_norm(float *values, uint64_t count, const float *weights, double epsilon);
int yvo_mhc_pre(const float *residual, const float *mixes, const float *scale, const float *base,
                uint64_t tokens, uint64_t streams, uint64_t width, uint64_t iterations,
                double rms_epsilon, double mhc_epsilon, double post_multiplier, float *collapsed,
                float *post, float *combination);
int yvo_mhc_post(const float *core, const float *residual, const float *post,
                 const float *combination, uint64_t tokens, uint64_t streams, uint64_t width,
                 float *output);
int yvo_moe_ffn_prepare(unsigned int function_qtype, const uint8_t *function,
                        const float *expanded, const float *scale, const float *base,
                        const float *norm, uint64_t tokens, uint64_t streams, uint64_t width,
                        uint64_t iterations, double rms_epsilon, double mhc_epsilon,
                        double post_multiplier, float *normalized, float *post, float *combination);

/* MoE layer over a row batch: routing given logits, routed experts in rank order, one shared
 * expert, combined = bf16(routed + shared) (src/runtime/moe.c:596-632).
 * Weights: routed gate/up/down are expert-major ([experts][rows][row_bytes]).
 * Outputs may be NULL except combined. */
typedef struct {
    uint64_t hidden, intermediate, experts, topk, rows;
    unsigned int gate_qtype, up_qtype, down_qtype;
    const uint8_t *routed_gate, *routed_up, *routed_down;
    const uint8_t *shared_gate, *shared_up, *shared_down; /* NULL: no shared expert */
    const float *router_bias;                             /* NULL: zeros */
    int scoring, normalize, act_q8;
    double scaling, activation_limit;
    unsigned int threads;
    const int32_t *hash_selected;   /* [rows][topk] expert ordinals of the hash router, or NULL */
} yvo_moe_layer_args;
int yvo_moe_layer(const yvo_moe_layer_args *args, const float *inputs, const float *logits,
                  uint64_t *selected, float *weights, float *routed, float *shared,
                  float *combined);

/* Synthetic-data generator shared by tests and the benchmark: splitmix64-seeded
 * xoshiro256**, Box-Muller normals computed in double then cast. */
typedef struct { uint64_t s[4]; } yvo_rng;
void yvo_rng_seed(yvo_rng *rng, uint64_t seed, const char *tensor_name);
uint64_t yvo_rng_next(yvo_rng *rng);
double yvo_rng_uniform(yvo_rng *rng);
void yvo_rng_normal_f32(yvo_rng *rng, float *out, uint64_t count, double sigma);
void yvo_rng_bytes(yvo_rng *rng, uint8_t *out, uint64_t count);
/* Random packed rows as BASELINE's configs describe them. */
void yvo_fill_iq2xxs(yvo_rng *rng, uint8_t *encoded, uint64_t blocks, double scale_sigma);
void yvo_fill_q4k(yvo_rng *rng, uint8_t *encoded, uint64_t blocks, double scale_sigma);
void yvo_fill_q8_0_from_normal(yvo_rng *rng, uint8_t *encoded, uint64_t blocks, double sigma);

#ifdef __cplusplus
}
#endif
#endif
