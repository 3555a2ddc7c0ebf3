/*
 * Launch-level C ABI of the gfx950 kernels: plain device pointers, sizes and a stream.
 *
 * This is the thin layer the C11 backend (include/yvex_rocm.h) sits on; every entry point
 * enqueues work on `stream` (a hipStream_t passed as void *, NULL = the default stream) and
 * returns without synchronising. Return value: 0 or a negative yvex_status
 * (INVALID_ARG -10 / BOUNDS -7 / UNSUPPORTED -5 for a refused shape, BACKEND -6 when the launch
 * itself fails). Numerical trouble is reported through the device `status` word the caller
 * owns: 0 ok, 1 non-finite value met, 2 contract violation seen on device - the convention of
 * the reference's kernels (src/backend/cuda/kernels.cu:555-564,623).
 *
 * All pointers are device pointers unless a comment says "host".
 */
#ifndef YVEX_ROCM_KERNELS_H
#define YVEX_ROCM_KERNELS_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void *yvex_hip_stream;

/* Router scoring policies. 0 is the reference's only policy (include/yvex/internal/moe.h:35);
 * 1 is the sigmoid scoring the benchmark configuration asks for. */
#define YVEX_HIP_SCORING_SQRT_SOFTPLUS 0
#define YVEX_HIP_SCORING_SIGMOID 1

/* Replaces yvex_q8_quantize (src/backend/cuda/kernels.cu:436-489): F32 rows -> Q8_K blocks
 * {f32 d; i8 q[256]; i16 bsums[16]}. width % 256 == 0, input_stride >= width (in floats).
 * Among equal |x| the lowest index provides the sign of d. */
int yvex_hip_q8k_quantize(const float *values, uint64_t rows, uint64_t width,
                          uint64_t input_stride, uint8_t *encoded, int *status,
                          yvex_hip_stream stream);

/* Replaces yvex_qtype_matvec / yvex_qtype_tensorcore_rows (kernels.cu:529-626,
 * tensorcore.cu:248-374): out[in * out_stride + row] = dot(encoded row, input row in)
 * (+ additive[in * out_stride + row]) (optionally bf16-rounded).
 * input is F32 rows of stride input_stride when input_q8 == 0, else Q8_K rows of
 * (row_width / 256) * 292 bytes. */
int yvex_hip_matvec(const uint8_t *encoded, unsigned int qtype, uint64_t row_count,
                    uint64_t row_width, uint64_t row_bytes, const void *input, int input_q8,
                    uint64_t input_rows, uint64_t input_stride, const float *additive,
                    float *out, uint64_t out_stride, int output_bf16, int *status,
                    yvex_hip_stream stream);


/* Verification twin of the integer hot loop (kernel_primitives.h:287-359): writes the int32
 * block sums the Q8_K matvec accumulates, before any float scaling.
 *   IQ2_XXS: sums[((in * row_count + row) * blocks + b) * 2 + 0] = T,            slot 1 = 0
 *   Q4_K / Q2_K:                                       slot 0 = dot, slot 1 = min-sum
 *   Q8_0:    sums[(in * row_count + row) * blocks * 8 + 8 * b + k] = D_k (eight per 256 block) */
int yvex_hip_block_dots_i32(const uint8_t *encoded, unsigned int qtype, uint64_t row_count,
                            uint64_t row_width, uint64_t row_bytes, const uint8_t *input_q8,
                            uint64_t input_rows, int32_t *sums, int *status,
                            yvex_hip_stream stream);

/* Replaces yvex_qtype_row_dot (kernels.cu:112-124): out[0] = float(sum over i in order of
 * double(decode(i)) * double(vector[i])), one thread. */
int yvex_hip_row_dot(const uint8_t *encoded, unsigned int qtype, const float *vector,
                     uint64_t elements, float *out, yvex_hip_stream stream);

/* The activation side of yvex_qtype_split_matvec (kernels.cu:736-782): out[row] = bf16 values of
 * head[row, 0..head_width) followed by tail[row, 0..tail_width), so that the split projection is
 * the ordinary F32-activation projection over out. Non-finite values raise status 1. */
int yvex_hip_concat_rows_bf16(const float *head, const float *tail, uint64_t rows,
                              uint64_t head_width, uint64_t tail_width, float *out, int *status,
                              yvex_hip_stream stream);

/* yvex_hip_matvec for F32 weight rows and a decode-width batch of F32 input rows (8 to 255: the
 * router projection of the MoE row batch, src/backend/cuda/moe.c:1259-1284), given scratch memory
 * (8-byte aligned): the row width is split between workgroups so that the whole device takes
 * part, the partial sums (doubles) go to scratch and a second launch adds them in split order
 * (deterministic). With NULL or too little scratch (yvex_hip_matvec_f32_scratch_bytes, 0 when
 * the shape is not split) or operands that are not 16-byte aligned it is yvex_hip_matvec;
 * yvex_hip_matvec_f32_rows_launches says which of the two it will be for given operands (2 or 1
 * kernel launches). Products and sums run in double and the result is rounded to float once, as
 * the CPU row dot does (src/gguf/quant_compute.c:152-172). */
uint64_t yvex_hip_matvec_f32_scratch_bytes(uint64_t row_count, uint64_t row_width, uint64_t input_rows);
unsigned int yvex_hip_matvec_f32_rows_launches(const float *weights, uint64_t row_count, uint64_t row_width,
                                               const float *input, uint64_t input_rows,
                                               uint64_t input_stride, const void *scratch,
                                               uint64_t scratch_bytes);
int yvex_hip_matvec_f32_rows(const float *weights, uint64_t row_count, uint64_t row_width,
                             const float *input, uint64_t input_rows, uint64_t input_stride,
                             const float *additive, float *out, uint64_t out_stride, int output_bf16,
                             void *scratch, uint64_t scratch_bytes, int *status, yvex_hip_stream stream);
/* The split form of yvex_hip_matvec_f32_rows for the router's logits, which also publishes the
 * router's score of every logit (scores, dense [input row][weight row]; the float that the
 * double-precision score of src/graph/moe.c:497-537 rounds to, as yvex_hip_moe_route_scores
 * publishes it): the second launch's many workgroups compute them, so that the routing launch
 * that follows (yvex_hip_moe_prepare_scored) has none left. UNSUPPORTED where
 * yvex_hip_matvec_f32_rows_launches says 1 for the operands. A logit whose score is not finite
 * raises status 1. */
int yvex_hip_matvec_f32_rows_scored(const float *weights, uint64_t row_count, uint64_t row_width,
                                    const float *input, uint64_t input_rows, uint64_t input_stride,
                                    float *out, uint64_t out_stride, float *scores, int scoring,
                                    void *scratch, uint64_t scratch_bytes, int *status,
                                    yvex_hip_stream stream);

/* Replaces yvex_argmax_f32 (kernels.cu:59-110): for each of row_count (<= 65535) rows of
 * row_width (< 2^32) F32 values the largest value, the lowest index holding it and the number of
 * elements holding it. A non-finite element raises status 1 and its row publishes nothing.
 * scratch (8-byte aligned device memory, may be NULL) lets a long row be split over several
 * workgroups: with at least yvex_hip_argmax_scratch_bytes(row_count, row_width) bytes two
 * launches share the row among the chip's compute units, without it one workgroup scans a row. */
uint64_t yvex_hip_argmax_scratch_bytes(uint64_t row_count, uint64_t row_width);
int yvex_hip_argmax_f32(const float *values, uint64_t row_count, uint64_t row_width,
                        uint32_t *selected_tokens, float *selected_values, uint64_t *tie_counts,
                        void *scratch, uint64_t scratch_bytes, int *status, yvex_hip_stream stream);

/* yvex_hip_argmax_f32 for callers that cannot allocate device memory (code under graph capture,
 * serving loops and harnesses that forbid it); it has no counterpart in the reference. The span
 * results live in a static device array of yvex_hip_argmax_static_capacity() bytes (256 KiB:
 * 16 384 span results, one per 8192 values of a row) that each device holds until the process
 * ends, so the call allocates nothing; a batch needing more is refused with BOUNDS and an error
 * text. Every call on a device shares that device's array: calls that overlap on one device
 * (different streams or threads) race and must be ordered by the caller. Results are those of
 * yvex_hip_argmax_f32 given a workspace. */
uint64_t yvex_hip_argmax_static_capacity(void);
int yvex_hip_argmax_f32_static(const float *values, uint64_t row_count, uint64_t row_width,
                               uint32_t *selected_tokens, float *selected_values, uint64_t *tie_counts,
                               int *status, yvex_hip_stream stream);

/* Replaces yvex_qtype_gather / yvex_encoded_row_decode (kernels.cu:784-830): decode selected
 * rows to F32. row_ids may be NULL (rows 0..selected-1). */
int yvex_hip_gather(const uint8_t *encoded, unsigned int qtype, uint64_t row_count,
                    uint64_t row_width, uint64_t row_bytes, const uint32_t *row_ids,
                    uint64_t selected, float *out, int *status, yvex_hip_stream stream);

/* Replaces yvex_moe_route_rows (src/backend/cuda/moe_kernels.cu:180-291): per row, scores in
 * fp64 from the logits, top-k of score + bias with ties to the lowest expert, weights
 * normalised over the selection and scaled. selected is [rows, topk] u64, weights [rows, topk]. */
int yvex_hip_moe_route_rows(const float *logits, const float *bias, uint64_t rows,
                            uint64_t experts, uint64_t topk, int scoring, int normalize,
                            double scaling, uint64_t *selected, float *weights, int *status,
                            yvex_hip_stream stream);

/* Hash router of yvex_moe_route_rows (moe_kernels.cu:222-245; CPU rule src/graph/moe.c:539-582):
 * row r takes the first topk ordinals of row token_ids[r] of an I32 table (table_row_bytes per
 * row, 4-byte aligned; single_row != 0: the table holds one row that serves every token, as
 * moe.c:547-549 reads it) and weighs them like the learned router. token_ids[r] >= table_rows,
 * an ordinal outside [0, experts) or a repeated one raise status 2. */
int yvex_hip_moe_route_hash_rows(const float *logits, const uint8_t *table,
                                 const uint32_t *token_ids, uint64_t rows, uint64_t experts,
                                 uint64_t topk, uint64_t table_rows, uint64_t table_row_bytes,
                                 int single_row, int scoring, int normalize, double scaling,
                                 uint64_t *selected, float *weights, int *status,
                                 yvex_hip_stream stream);

/* scores[i] = score(logits[i]) under the layer's scoring policy, as float: what the token-local
 * operation publishes beside the logits (src/backend/cuda/moe_kernels.cu:29-55,
 * src/graph/moe.c:497-501). */
int yvex_hip_moe_route_scores(const float *logits, uint64_t count, int scoring, float *scores,
                              int *status, yvex_hip_stream stream);

/* Replaces yvex_expert_worklist_build_cuda (moe_kernels.cu:294-402): stable counting sort of
 * the pairs = rows*topk (row, rank) pairs by expert; rows <= 4096 per call. Outputs, all
 * device memory:
 *   order[pairs]            source pair of each ordered position
 *   expert_ids[experts], bucket_offsets[experts + 1], bucket_populations[experts]
 *   sweep_offsets[experts + 1]  running count of weight sweeps (two pairs per sweep) before each
 *                           bucket: the generic grouped kernels spread sweeps, not buckets, over
 *                           the chip (the IQ2_XXS sweeps number theirs, four pairs each, on device)
 *   counts[4]               {bucket_count, maximum_population, pair_count, sweep_count} */
int yvex_hip_worklist_build(const uint64_t *selected, uint64_t pairs, uint64_t topk,
                            uint64_t experts, uint64_t *order, uint64_t *expert_ids,
                            uint64_t *bucket_offsets, uint64_t *bucket_populations,
                            uint64_t *sweep_offsets, uint64_t *counts, int *status,
                            yvex_hip_stream stream);

/* A decode batch's preparation in one launch: yvex_hip_moe_route_rows, yvex_hip_worklist_build and
 * (when values is not NULL) yvex_hip_q8k_quantize of the rows x width input, with the same outputs
 * bit for bit. One workgroup routes and sorts while the others quantize, so the three launches'
 * latencies are paid once. For rows <= 128, experts <= 256, topk <= 16
 * (yvex_hip_moe_prepare_supported), else UNSUPPORTED. The reference launches these steps one by
 * one (src/backend/cuda/moe.c:1286-1345, 1363-1376). */
int yvex_hip_moe_prepare_supported(uint64_t rows, uint64_t experts, uint64_t topk);
int yvex_hip_moe_prepare(const float *logits, const float *bias, uint64_t rows, uint64_t experts,
                         uint64_t topk, int scoring, int normalize, double scaling, uint64_t *selected,
                         float *weights, uint64_t *order, uint64_t *expert_ids, uint64_t *bucket_offsets,
                         uint64_t *bucket_populations, uint64_t *sweep_offsets, uint64_t *counts,
                         const float *values, uint64_t width, uint64_t input_stride, uint8_t *encoded,
                         int *status, yvex_hip_stream stream);
/* yvex_hip_moe_prepare over scores that yvex_hip_matvec_f32_rows_scored has published
 * (rows x experts floats) in place of the logits: same outputs bit for bit. */
int yvex_hip_moe_prepare_scored(const float *scores, const float *bias, uint64_t rows, uint64_t experts,
                                uint64_t topk, int normalize, double scaling, uint64_t *selected,
                                float *weights, uint64_t *order, uint64_t *expert_ids,
                                uint64_t *bucket_offsets, uint64_t *bucket_populations,
                                uint64_t *sweep_offsets, uint64_t *counts, const float *values,
                                uint64_t width, uint64_t input_stride, uint8_t *encoded, int *status,
                                yvex_hip_stream stream);

/* Expert matrices of one MoE layer. routed_* are expert-major: expert e starts at
 * base + e * expert_bytes and holds rows * row_bytes canonical GGUF bytes. gate_up_image /
 * down_image say that those IQ2_XXS matrices are given as the sweep image of
 * yvex_hip_iq2_sweep_image_build (72 bytes a superblock, row_bytes and expert_bytes counted in
 * image bytes); only the decode sweeps with Q8_K activations read it. */
typedef struct {
    const uint8_t *gate, *up, *down;
    unsigned int gate_qtype, up_qtype, down_qtype;
    uint64_t hidden, intermediate;
    uint64_t gate_row_bytes, up_row_bytes, down_row_bytes;
    uint64_t gate_expert_bytes, up_expert_bytes, down_expert_bytes;
    int gate_up_image, down_image;
} yvex_hip_expert_weights;

/* The sweep image of IQ2_XXS weights: the backend's own re-packing for the decode sweeps, built
 * on the device from canonical bytes (`blocks` superblocks of 66 bytes, any alignment) into
 * `image` (yvex_hip_iq2_sweep_image_bytes(blocks) bytes, dword-aligned), block order kept. Per
 * superblock two records of nine dwords, one per half: {f16 d | the half's four 4-bit group
 * scales << 16}, then per group the four codebook bytes and the four 7-bit sign fields one to a
 * byte. The counterpart of the reference's derived layout (src/backend/cuda/layout.c:95-167) for
 * this backend's kernels; the canonical bytes stay the authority. */
uint64_t yvex_hip_iq2_sweep_image_bytes(uint64_t blocks);
int yvex_hip_iq2_sweep_image_build(const uint8_t *canonical, uint64_t blocks, void *image,
                                   yvex_hip_stream stream);

/* Replaces yvex_moe_grouped_up_rows (+ _up_tensorcore) (moe_kernels.cu:431-516,
 * tensorcore.cu:527-626): for every ordered pair p of every bucket,
 *   intermediate[p, i] = bf16(silu(min(g,L)) * clamp(u,+-L) * route_weight), g/u = gate/up row i
 * dotted with the pair's source row (source pair / topk). An expert's bytes are read once per
 * two pairs of its bucket.
 * activations: Q8_K rows [rows][hidden/256 * 292] when act_q8, else F32 rows [rows][hidden].
 * With expert_ids == NULL the call is the single-expert form: one bucket holding pairs
 * 0..pairs-1 of expert 0, pair p reading activation row p / topk, weight 1 when
 * route_weights == NULL.
 * shared != NULL folds the layer's shared expert into the same launch: it must have the same
 * qtypes and shapes as the routed experts (else UNSUPPORTED: launch it separately), is applied
 * to activation rows 0..shared_rows-1 with weight 1 and writes shared_intermediate[row, i]. */
int yvex_hip_moe_up(const yvex_hip_expert_weights *weights, const void *activations, int act_q8,
                    const float *route_weights, const uint64_t *order,
                    const uint64_t *expert_ids, const uint64_t *bucket_offsets,
                    const uint64_t *bucket_populations, const uint64_t *sweep_offsets,
                    const uint64_t *counts, uint64_t pairs, uint64_t topk, uint64_t experts,
                    double limit,
                    float *intermediate, const yvex_hip_expert_weights *shared,
                    uint64_t shared_rows, float *shared_intermediate, int *status,
                    yvex_hip_stream stream);

/* Replaces yvex_moe_grouped_down_rows (+ _down_tensorcore) (moe_kernels.cu:518-582,
 * tensorcore.cu:628-702): pair_outputs[source_pair, c] = bf16(dot(down row c, intermediate of
 * the ordered pair)). intermediate is Q8_K [pairs][intermediate/256*292] when act_q8 else F32,
 * indexed by ordered position. shared != NULL folds the shared expert in as for the up sweep:
 * shared_outputs[row, c] = bf16(dot(shared down row c, shared_intermediate row)). */
int yvex_hip_moe_down(const yvex_hip_expert_weights *weights, const void *intermediate,
                      int act_q8, const uint64_t *order, const uint64_t *expert_ids,
                      const uint64_t *bucket_offsets, const uint64_t *bucket_populations,
                      const uint64_t *sweep_offsets, const uint64_t *counts, uint64_t pairs,
                      uint64_t experts,
                      float *pair_outputs, const yvex_hip_expert_weights *shared,
                      uint64_t shared_rows, const void *shared_intermediate,
                      float *shared_outputs, int *status, yvex_hip_stream stream);

/* Row-batch (prefill-width) forms of the two sweeps above on the int8 matrix cores; they replace
 * yvex_moe_grouped_up_tensorcore / _down_tensorcore (tensorcore.cu:378-702). Same inputs,
 * outputs and rounding points as yvex_hip_moe_up / yvex_hip_moe_down with act_q8 = 1; weights
 * must be IQ2_XXS. A work item is 64 ordered pairs of one bucket times a tile of 256 weight rows,
 * so buckets of any population are served; expert_ids == NULL is the single-bucket form
 * (shared expert: every pair uses expert 0, order may be NULL for the identity). */
int yvex_hip_moe_up_rows(const yvex_hip_expert_weights *weights, const void *act_q8k,
                         const float *route_weights, const uint64_t *order,
                         const uint64_t *expert_ids, const uint64_t *bucket_offsets,
                         const uint64_t *bucket_populations, const uint64_t *counts,
                         uint64_t pairs, uint64_t topk, uint64_t experts, double limit,
                         float *intermediate, int *status, yvex_hip_stream stream);
int yvex_hip_moe_down_rows(const yvex_hip_expert_weights *weights, const void *intermediate_q8k,
                           const uint64_t *order, const uint64_t *expert_ids,
                           const uint64_t *bucket_offsets, const uint64_t *bucket_populations,
                           const uint64_t *counts, uint64_t pairs, uint64_t experts,
                           float *pair_outputs, int *status, yvex_hip_stream stream);

/* The SwiGLU stage of an expert whose gate and up projections ran as dense projections (a shared
 * expert of a format the expert kernels do not take): out[i] = bf16(silu(min(gate[i], limit)) *
 * clamp(up[i], -limit, limit)), the value yvex_moe_grouped_up_rows forms with a route weight of
 * one (moe_kernels.cu:431-516, src/graph/moe.c:605-611). out may be gate or up. A product that is
 * not finite raises status 1 and is not stored. */
int yvex_hip_moe_swiglu_rows(const float *gate, const float *up, uint64_t count, double limit,
                             float *out, int *status, yvex_hip_stream stream);

/* Replaces yvex_moe_reduce_rows + yvex_moe_combine_rows (moe_kernels.cu:584-616):
 * routed[row, c] = sum over rank (in rank order, fp32) of pair_outputs[row*topk+rank, c];
 * combined[row, c] = bf16(routed + shared) when shared != NULL and combined != NULL. */
int yvex_hip_moe_reduce_combine(const float *pair_outputs, uint64_t rows, uint64_t topk,
                                uint64_t hidden, const float *shared, float *routed,
                                float *combined, int *status, yvex_hip_stream stream);

/* Residual-stream envelope around the expert math (row_count rows of streams x width F32 values,
 * streams <= 7 so that (streams + 2) * streams <= 64 mixing rows, width <= 16384).
 *
 * yvex_hip_mhc_ingress replaces yvex_residual_mhc_pre followed by yvex_attention_weighted_norm
 * (src/backend/cuda/kernels.cu:1243-1387 and :867-910; launched from
 * src/backend/cuda/moe.c:1210-1254) with the arithmetic of src/graph/numeric.c:630-826: the
 * residual is rounded to bf16 as it is read (the rows themselves are left untouched), gates and
 * the mixing matrix are formed in double precision from mixes[row, (streams + 2) * streams]
 * (= function . row), scale[3] and base[(streams + 2) * streams], the collapsed row is
 * bf16-rounded, normalised with norm[width] and published as bf16 in normalized[row, width];
 * post[row, streams] and combination[row, streams, streams] are kept for the egress.
 *
 * yvex_hip_mhc_egress replaces yvex_residual_mhc_post (kernels.cu:1389-1428,
 * numeric.c:828-877): output[row, target, lane] = bf16(post[target] * core[row, lane] +
 * sum over source of combination[source, target] * bf16(rows[row, source, lane])), accumulated
 * in double in source order. Non-finite values raise status 1 in both. */
int yvex_hip_mhc_ingress(const float *rows, const float *mixes, const float *scale,
                         const float *base, const float *norm, uint64_t row_count,
                         uint64_t streams, uint64_t width, uint64_t iterations,
                         double rms_epsilon, double mhc_epsilon, double post_multiplier,
                         float *normalized, float *post, float *combination, int *status,
                         yvex_hip_stream stream);
/* yvex_hip_mhc_ingress with scale, base and norm as the layer stores them (F32 or BF16 values;
 * UNSUPPORTED for anything else), decoded inside the launch: the reference decodes each
 * into an F32 buffer with a launch of its own first (src/backend/cuda/moe.c:1226-1240). Same
 * outputs and status. */
int yvex_hip_mhc_ingress_encoded(const float *rows, const float *mixes, const void *scale,
                                 unsigned int scale_qtype, const void *base, unsigned int base_qtype,
                                 const void *norm, unsigned int norm_qtype, uint64_t row_count,
                                 uint64_t streams, uint64_t width, uint64_t iterations, double rms_epsilon,
                                 double mhc_epsilon, double post_multiplier, float *normalized, float *post,
                                 float *combination, int *status, yvex_hip_stream stream);
int yvex_hip_mhc_egress(const float *core, const float *rows, const float *post,
                        const float *combination, uint64_t row_count, uint64_t streams,
                        uint64_t width, float *output, int *status, yvex_hip_stream stream);

/* Bandwidth probe (the reference publishes the same fact at backend start,
 * src/backend/cuda/backend.c:1550): streams `bytes` of device memory through 16-byte loads.
 * Time it with events; `sink` is a 4-byte device word that is practically never written. */
int yvex_hip_stream_read(const void *data, uint64_t bytes, uint32_t *sink, yvex_hip_stream stream);

/* One timed sample of the bandwidth probe: `iterations` streaming reads of `bytes` (destination
 * NULL; `sink` as for yvex_hip_stream_read) or `iterations` device-to-device copies of `bytes`,
 * bracketed by events on the stream; the call waits for the second event. */
int yvex_hip_bandwidth_sample(const void *source, void *destination, uint64_t bytes, uint64_t iterations,
                              uint32_t *sink, uint64_t *elapsed_ns, yvex_hip_stream stream);

/* Clock probe, the companion of the bandwidth probe: every SIMD of the device runs `chain` (a
 * multiple of 4) 32x32x32 int8 matrix instructions on four accumulators in turn, each taking the
 * matrix pipe for 32 shader cycles, so the launch lasts chain * 32 cycles; timed with events it
 * gives the clock under matrix-core load, the figure a fraction of the matrix-core peak has to
 * be read with. `sink` is a device word that is practically never written. */
int yvex_hip_clock_probe(uint64_t chain, int *sink, yvex_hip_stream stream);

/* Device-side fill, usable where a captured graph must not hold a memset node. */
int yvex_hip_fill_u32(void *dst, uint32_t value, uint64_t count, yvex_hip_stream stream);

/* ---- plumbing for the C11 host layer (no HIP headers needed there) ---- */
int yvex_hip_device_count(void);
int yvex_hip_device_info(int device, char *name, unsigned long name_cap, char *arch,
                         unsigned long arch_cap, uint64_t *total_bytes, uint64_t *free_bytes,
                         int *compute_units);
/* Peak engine and memory clocks the device reports, in kHz. */
int yvex_hip_device_clocks(int device, int *engine_khz, int *memory_khz);
int yvex_hip_malloc(void **out, uint64_t bytes);
int yvex_hip_free(void *ptr);
int yvex_hip_host_alloc(void **out, uint64_t bytes);
int yvex_hip_host_free(void *ptr);
int yvex_hip_memcpy_h2d(void *dst, const void *src, uint64_t bytes, yvex_hip_stream stream);
/* The same copy queued on the stream without waiting for it: `src` is pinned host memory
 * (yvex_hip_host_alloc) that stays untouched until the stream has passed the copy. */
int yvex_hip_memcpy_h2d_queued(void *dst, const void *src, uint64_t bytes, yvex_hip_stream stream);
int yvex_hip_memcpy_d2h(void *dst, const void *src, uint64_t bytes, yvex_hip_stream stream);
int yvex_hip_memcpy_d2d(void *dst, const void *src, uint64_t bytes, yvex_hip_stream stream);
int yvex_hip_stream_create(yvex_hip_stream *out);
int yvex_hip_stream_destroy(yvex_hip_stream stream);
int yvex_hip_stream_sync(yvex_hip_stream stream);
/* Launch graphs, the counterpart of yvex_cuda_graph_execute (src/backend/cuda/moe.c:1665-1681):
 * capture_begin puts the stream in capture mode, the launch wrappers above then record instead
 * of running, capture_end instantiates the recording (refusing one that holds anything but
 * kernel nodes, and reporting how many it holds) and capture_abort discards it. A graph is
 * launched on a stream like a kernel and stays valid while every address it recorded does. */
typedef void *yvex_hip_graph;
int yvex_hip_capture_begin(yvex_hip_stream stream);
int yvex_hip_capture_end(yvex_hip_stream stream, yvex_hip_graph *out, uint64_t *kernel_nodes);
int yvex_hip_capture_abort(yvex_hip_stream stream);
int yvex_hip_graph_launch(yvex_hip_graph graph, yvex_hip_stream stream);
int yvex_hip_graph_destroy(yvex_hip_graph graph);
/* 1 when the gfx950 code object for the kernels is loadable on the current device. */
int yvex_hip_kernels_loadable(void);
const char *yvex_hip_last_error(void);

#ifdef __cplusplus
}
#endif
#endif
