/*
 * Status names, structured errors, and the qtype geometry / capability registry of the ROCm
 * backend. Restates include/yvex/core.h:13-48, src/core/status.c, src/gguf/qtype.c:15-124 and
 * src/gguf/quant_registry.c:50-117. The registry is fail-closed: an ID without a row, or a row
 * without device compute, is refused before anything is launched.
 */
#include <stdio.h>
#include <string.h>

#include "yvex_rocm.h"

const char *yvex_rocm_status_name(yvex_status status)
{
    switch (status) {
    case YVEX_OK: return "ok";
    case YVEX_ERR: return "error";
    case YVEX_ERR_NOMEM: return "nomem";
    case YVEX_ERR_IO: return "io";
    case YVEX_ERR_FORMAT: return "format";
    case YVEX_ERR_UNSUPPORTED: return "unsupported";
    case YVEX_ERR_BACKEND: return "backend";
    case YVEX_ERR_BOUNDS: return "bounds";
    case YVEX_ERR_STATE: return "state";
    case YVEX_ERR_CANCELLED: return "cancelled";
    case YVEX_ERR_INVALID_ARG: return "invalid-arg";
    case YVEX_ERR_TIMEOUT: return "timeout";
    default: return "unknown";
    }
}

void yvex_rocm_error_clear(yvex_error *err)
{
    if (err) memset(err, 0, sizeof(*err));
}

void yvex_rocm_error_set(yvex_error *err, yvex_status code, const char *where, const char *message)
{
    if (!err) return;
    err->code = code;
    snprintf(err->where, sizeof(err->where), "%s", where ? where : "");
    snprintf(err->message, sizeof(err->message), "%s", message ? message : "");
}

int yvex_rocm_error_is_set(const yvex_error *err) { return err && err->code != YVEX_OK; }
yvex_status yvex_rocm_error_code(const yvex_error *err) { return err ? err->code : YVEX_OK; }

#define ADMIT YVEX_GGUF_QTYPE_IDENTITY_ADMITTED
#define GONE YVEX_GGUF_QTYPE_IDENTITY_REMOVED
#define LATER YVEX_GGUF_QTYPE_IDENTITY_OUTSIDE_BASELINE

static const yvex_rocm_qtype_geometry geometry_table[] = {
    {0, "F32", ADMIT, 1, 4},        {1, "F16", ADMIT, 1, 2},         {2, "Q4_0", ADMIT, 32, 18},
    {3, "Q4_1", ADMIT, 32, 20},     {4, "Q4_2", GONE, 0, 0},         {5, "Q4_3", GONE, 0, 0},
    {6, "Q5_0", ADMIT, 32, 22},     {7, "Q5_1", ADMIT, 32, 24},      {8, "Q8_0", ADMIT, 32, 34},
    {9, "Q8_1", ADMIT, 32, 36},     {10, "Q2_K", ADMIT, 256, 84},    {11, "Q3_K", ADMIT, 256, 110},
    {12, "Q4_K", ADMIT, 256, 144},  {13, "Q5_K", ADMIT, 256, 176},   {14, "Q6_K", ADMIT, 256, 210},
    {15, "Q8_K", ADMIT, 256, 292},  {16, "IQ2_XXS", ADMIT, 256, 66}, {17, "IQ2_XS", ADMIT, 256, 74},
    {18, "IQ3_XXS", ADMIT, 256, 98}, {19, "IQ1_S", ADMIT, 256, 50},  {20, "IQ4_NL", ADMIT, 32, 18},
    {21, "IQ3_S", ADMIT, 256, 110}, {22, "IQ2_S", ADMIT, 256, 82},   {23, "IQ4_XS", ADMIT, 256, 136},
    {24, "I8", ADMIT, 1, 1},        {25, "I16", ADMIT, 1, 2},        {26, "I32", ADMIT, 1, 4},
    {27, "I64", ADMIT, 1, 8},       {28, "F64", ADMIT, 1, 8},        {29, "IQ1_M", ADMIT, 256, 56},
    {30, "BF16", ADMIT, 1, 2},      {31, "Q4_0_4_4", GONE, 0, 0},    {32, "Q4_0_4_8", GONE, 0, 0},
    {33, "Q4_0_8_8", GONE, 0, 0},   {34, "TQ1_0", ADMIT, 256, 54},   {35, "TQ2_0", ADMIT, 256, 66},
    {36, "IQ4_NL_4_4", GONE, 0, 0}, {37, "IQ4_NL_4_8", GONE, 0, 0},  {38, "IQ4_NL_8_8", GONE, 0, 0},
    {39, "MXFP4", ADMIT, 32, 17},   {40, "NVFP4", LATER, 64, 36},    {41, "Q1_0", LATER, 128, 18},
    {42, "Q2_0", LATER, 64, 18},
};

const yvex_rocm_qtype_geometry *yvex_rocm_gguf_qtype_geometry_find(unsigned int qtype)
{
    if (qtype > YVEX_GGUF_QTYPE_ABI_UPSTREAM_MAX_ID) return NULL;
    return &geometry_table[qtype];
}

/* {known, storage, decoder, cpu, device, extension, refusal} per ID. */
#define FULL(q) {q, 1, 1, 1, 1, 1, 0, YVEX_ROCM_QUANT_REFUSAL_NONE}
#define CPU_ONLY(q) {q, 1, 1, 1, 1, 0, 0, YVEX_ROCM_QUANT_REFUSAL_NONE}
#define EXTENDED(q) {q, 1, 1, 1, 1, 1, 1, YVEX_ROCM_QUANT_REFUSAL_NONE}
#define NO_CODEC(q) {q, 1, 1, 0, 0, 0, 0, YVEX_ROCM_QUANT_REFUSAL_ENCODER_UNAVAILABLE}
#define REMOVED(q) {q, 1, 0, 0, 0, 0, 0, YVEX_ROCM_QUANT_REFUSAL_REMOVED_IDENTITY}
#define OUTSIDE(q) {q, 1, 0, 0, 0, 0, 0, YVEX_ROCM_QUANT_REFUSAL_OUTSIDE_PINNED_BASELINE}

static const yvex_rocm_numeric_capability capability_table[] = {
    FULL(0),      FULL(1),      NO_CODEC(2),  NO_CODEC(3),  REMOVED(4),   REMOVED(5),
    NO_CODEC(6),  NO_CODEC(7),  FULL(8),      NO_CODEC(9),  FULL(10),     NO_CODEC(11),
    EXTENDED(12), NO_CODEC(13), NO_CODEC(14), NO_CODEC(15), FULL(16),     NO_CODEC(17),
    NO_CODEC(18), NO_CODEC(19), NO_CODEC(20), NO_CODEC(21), NO_CODEC(22), NO_CODEC(23),
    NO_CODEC(24), NO_CODEC(25), FULL(26),     NO_CODEC(27), NO_CODEC(28), NO_CODEC(29),
    FULL(30),     REMOVED(31),  REMOVED(32),  REMOVED(33),  NO_CODEC(34), NO_CODEC(35),
    REMOVED(36),  REMOVED(37),  REMOVED(38),  CPU_ONLY(39), OUTSIDE(40),  OUTSIDE(41),
    OUTSIDE(42),
};

_Static_assert(sizeof(geometry_table) / sizeof(geometry_table[0]) == 43u, "IDs 0 through 42");
_Static_assert(sizeof(capability_table) / sizeof(capability_table[0]) == 43u, "IDs 0 through 42");

const yvex_rocm_numeric_capability *yvex_rocm_quant_numeric_capability_at(unsigned int qtype)
{
    if (qtype >= sizeof(capability_table) / sizeof(capability_table[0])) return NULL;
    return &capability_table[qtype];
}
