// Problem description shared by the grouped expert kernels (decode-width sweeps and the MFMA
// row-batch kernel): one set of expert matrices, the activation rows and the expert-major worklist.
#pragma once

#include "common.hpp"
#include "launch.hpp"

namespace yvex {

constexpr int kPass = 2;          // pairs of one bucket handled per sweep over the expert's bytes
constexpr int kUnitsPerLane = 4;  // a sweep lane owns half a superblock: 128 columns

// One set of expert matrices plus the pairs that use it.
struct GroupedProblem {
    const unsigned char *gate, *up;          // up == nullptr: plain projection (down)
    unsigned long long row_bytes, expert_bytes, up_row_bytes, up_expert_bytes;
    const void *activations;                 // Q8_K rows or F32 rows
    unsigned long long act_stride;           // bytes between activation rows
    int act_by_ordered_pair;                 // 1: activation row = ordered position (down)
    const unsigned long long *order, *expert_ids, *bucket_offsets, *bucket_populations;
    const unsigned long long *sweep_offsets, *counts;
    const float *route_weights;
    unsigned pairs, topk, experts;
    float *out;                              // [ordered or source pair][out_rows]
    int out_by_source_pair;
    unsigned sweeps;                         // single known bucket: ceil(pairs / kPass), else 0
};

struct GroupedArgs {
    GroupedProblem problem[2];               // [0] routed experts, [1] optional shared expert
    unsigned problems;
    unsigned width;                          // reduction width (activation row length)
    unsigned out_rows;                       // rows of the weight matrix per expert
    unsigned item_rows;                      // weight rows (row pairs when fused) per work item
    double limit;
    int *status;
    int image;                               // weights are the IQ2_XXS sweep image (72 B a superblock)
};

// The same value from fp32 arithmetic when that provably rounds to the same bfloat16. For
// |gate| <= 16 the fp32 result is within about 24 units in the last place of the exact one (the
// rounded product gate * log2(e) and the rounded constant contribute up to 19 of them, exp2,
// reciprocal, 1 + t and the multiplications the rest), so unless its low 16 bits sit within 64
// of the rounding midpoint the two roundings agree. Otherwise, and for non-finite or vanishing
// values, the double path decides.
__device__ __forceinline__ float swiglu_bf16(float g, float u, float route_weight, double limit);
__device__ __forceinline__ float swiglu_bf16_fast(float g, float u, float route_weight,
                                                  double limit, float limit_f32)
{
    const float gv = fminf(g, limit_f32);
    const float uv = fmaxf(-limit_f32, fminf(u, limit_f32));
    const float t = __builtin_amdgcn_exp2f(-fabsf(gv) * 1.44269504088896340736f);
    const float r = __builtin_amdgcn_rcpf(1.0f + t);
    const float silu = gv >= 0.0f ? gv * r : gv * t * r;
    const float v = silu * uv * route_weight;
    const unsigned bits = __float_as_uint(v), low = bits & 0xffffu;
    // (one branch: the tests are combined without short circuits)
    const bool finite = finite_f32(v), large = fabsf(v) > 1.0e-30f, inside = fabsf(gv) <= 16.0f;
    const bool clear = (low < 0x8000u - 64u) | (low > 0x8000u + 64u);
    const bool safe = ((double)limit_f32 == limit) & finite & large & inside & clear;
    if (safe) return bf16_round_number(v);
    return swiglu_bf16(g, u, route_weight, limit);
}

// SiLU-gated product in double, as src/graph/moe.c:605-611 orders it.
__device__ __forceinline__ float swiglu_bf16(float g, float u, float route_weight, double limit)
{
    const double gv = fmin((double)g, limit);
    const double uv = fmax(-limit, fmin((double)u, limit));
    const double t = exp(-fabs(gv));
    const double silu = gv >= 0.0 ? gv / (1.0 + t) : gv * t / (1.0 + t);
    return bf16_round((float)(silu * uv * (double)route_weight));
}

// Geometry of a matrix given as the IQ2_XXS sweep image.
static inline int check_image_matrix(unsigned qtype, uint64_t width, uint64_t row_bytes, const void *base,
                                     uint64_t expert_bytes)
{
    if (qtype != QT_IQ2_XXS) return ST_UNSUPPORTED;
    if (!width || width % 256u || width / 256u * 72u != row_bytes) return ST_BOUNDS;
    if (((uintptr_t)base & 3u) || (expert_bytes & 3u)) return ST_INVALID_ARG;
    return ST_OK;
}

static inline int check_matrix(unsigned qtype, uint64_t width, uint64_t row_bytes)
{
    unsigned block, bytes;
    if (!qtype_geometry(qtype, block, bytes) || block < 32u) return ST_UNSUPPORTED;
    if (!width || width % 256u || width / block * bytes != row_bytes) return ST_BOUNDS;
    if (width / 32u > 64u * kUnitsPerLane) return ST_UNSUPPORTED;   // one wave spans a row
    return ST_OK;
}

struct WorklistView {
    const uint64_t *order, *expert_ids, *bucket_offsets, *bucket_populations, *sweep_offsets, *counts;
};

static inline void fill_up_problem(GroupedProblem &p, const yvex_hip_expert_weights *w,
                            const void *activations, int act_q8, const float *route_weights,
                            const WorklistView &wl, uint64_t pairs, uint64_t topk, uint64_t experts,
                            float *out)
{
    p.gate = w->gate;
    p.up = w->up;
    p.row_bytes = w->gate_row_bytes;
    p.expert_bytes = w->gate_expert_bytes;
    p.up_row_bytes = w->up_row_bytes;
    p.up_expert_bytes = w->up_expert_bytes;
    p.activations = activations;
    p.act_stride = act_q8 ? w->hidden / 256u * kQ8KBytes : w->hidden * sizeof(float);
    p.act_by_ordered_pair = 0;
    p.order = (const unsigned long long *)wl.order;
    p.expert_ids = (const unsigned long long *)wl.expert_ids;
    p.bucket_offsets = (const unsigned long long *)wl.bucket_offsets;
    p.bucket_populations = (const unsigned long long *)wl.bucket_populations;
    p.sweep_offsets = (const unsigned long long *)wl.sweep_offsets;
    p.counts = (const unsigned long long *)wl.counts;
    p.route_weights = route_weights;
    p.pairs = (unsigned)pairs;
    p.topk = (unsigned)topk;
    p.experts = (unsigned)experts;
    p.out = out;
    p.out_by_source_pair = 0;
    p.sweeps = wl.expert_ids ? 0u : (unsigned)((pairs + kPass - 1u) / kPass);
}

static inline void fill_down_problem(GroupedProblem &p, const yvex_hip_expert_weights *w,
                              const void *intermediate, int act_q8, const WorklistView &wl,
                              uint64_t pairs, uint64_t experts, float *out)
{
    p.gate = w->down;
    p.up = nullptr;
    p.row_bytes = w->down_row_bytes;
    p.expert_bytes = w->down_expert_bytes;
    p.up_row_bytes = p.up_expert_bytes = 0;
    p.activations = intermediate;
    p.act_stride = act_q8 ? w->intermediate / 256u * kQ8KBytes : w->intermediate * sizeof(float);
    p.act_by_ordered_pair = 1;
    p.order = (const unsigned long long *)wl.order;
    p.expert_ids = (const unsigned long long *)wl.expert_ids;
    p.bucket_offsets = (const unsigned long long *)wl.bucket_offsets;
    p.bucket_populations = (const unsigned long long *)wl.bucket_populations;
    p.sweep_offsets = (const unsigned long long *)wl.sweep_offsets;
    p.counts = (const unsigned long long *)wl.counts;
    p.route_weights = nullptr;
    p.pairs = (unsigned)pairs;
    p.topk = 1u;
    p.experts = (unsigned)experts;
    p.out = out;
    p.out_by_source_pair = 1;
    p.sweeps = wl.expert_ids ? 0u : (unsigned)((pairs + kPass - 1u) / kPass);
}

// Specialised IQ2_XXS x Q8_K decode sweeps (sweep_iq2.hip): reduction widths whose rows span 16
// to 64 lanes of 128 columns each.
bool iq2_sweep_supported(unsigned qtype, unsigned width, unsigned out_rows, unsigned long long pairs, bool image);
int launch_iq2_sweep(const GroupedArgs &a, unsigned qtype, bool fused, bool image, hipStream_t stream);

// Row-batch expert kernels on the int8 matrix cores (rows_q4k.hip): Q4_K weights, fused gate/up
// or a plain projection; Q2_K weights, a plain projection (the down experts).
int launch_q4k_rows_grouped(const GroupedProblem &problem, unsigned qtype, bool fused, uint64_t width,
                            uint64_t out_rows, double limit, int *status, hipStream_t stream);

static inline bool same_shape(const yvex_hip_expert_weights *a, const yvex_hip_expert_weights *b)
{
    return a->gate_qtype == b->gate_qtype && a->up_qtype == b->up_qtype &&
           a->down_qtype == b->down_qtype && a->hidden == b->hidden &&
           a->intermediate == b->intermediate;
}


}  // namespace yvex
