// Plumbing the C11 host layer needs from the HIP runtime: memory, copies, streams, device facts.
// Kept behind plain C entry points so the host sources compile with a C11 compiler alone.
#include <stdio.h>
#include <string.h>

#include <mutex>
#include <vector>

#include "launch.hpp"

namespace yvex {

static thread_local char g_last_error[256] = "";

void set_last_error(const char *where, hipError_t code)
{
    snprintf(g_last_error, sizeof(g_last_error), "%s: %s", where, hipGetErrorString(code));
}
void set_last_error_text(const char *text)
{
    snprintf(g_last_error, sizeof(g_last_error), "%s", text);
}

// Compute units of the current device, read once: persistent kernels size their grids with it.
int compute_units()
{
    static std::once_flag once;
    static int units = 256;
    std::call_once(once, [] {
        int device = 0;
        hipDeviceProp_t prop;
        if (hipGetDevice(&device) == hipSuccess && hipGetDeviceProperties(&prop, device) == hipSuccess &&
            prop.multiProcessorCount > 0)
            units = prop.multiProcessorCount;
        else
            (void)hipGetLastError();
    });
    return units;
}

static int wrap(const char *where, hipError_t code)
{
    if (code == hipSuccess) return ST_OK;
    set_last_error(where, code);
    (void)hipGetLastError();
    return code == hipErrorOutOfMemory ? ST_NOMEM : ST_BACKEND;
}

__global__ void fill_u32_kernel(uint32_t *dst, uint32_t value, uint64_t count)
{
    uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < count) dst[i] = value;
}

// Streaming read of a buffer with 16-byte loads; every lane folds what it read into one word so
// the loads cannot be dropped. Used to measure the sustainable read bandwidth of the device.
__global__ __launch_bounds__(256) void stream_read_kernel(const uint4 *__restrict__ data,
                                                          uint64_t count, uint32_t *sink)
{
    uint32_t fold = 0u;
    const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
    uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    for (; i + 3u * stride < count; i += 4u * stride) {
        const uint4 a = data[i], b = data[i + stride], c = data[i + 2u * stride],
                    d = data[i + 3u * stride];
        fold ^= a.x ^ a.y ^ a.z ^ a.w ^ b.x ^ b.y ^ b.z ^ b.w ^ c.x ^ c.y ^ c.z ^ c.w ^ d.x ^ d.y ^
                d.z ^ d.w;
    }
    for (; i < count; i += stride) {
        const uint4 a = data[i];
        fold ^= a.x ^ a.y ^ a.z ^ a.w;
    }
    if (fold == 0x9e3779b9u) *sink = fold;   // practically never true; keeps the loads alive
}

// Back-to-back 32x32x32 int8 matrix instructions on four independent accumulators, one wave per
// SIMD on every compute unit: the matrix pipe takes 8 passes of 4 cycles for each, and with four
// accumulators in turn no instruction waits for the one before it, so a launch lasts
// chain * 32 shader cycles and its duration gives the clock the matrix cores run at under load.
// (A single accumulator would measure the 56-cycle dependent latency instead.)
__global__ __launch_bounds__(256) void clock_probe_kernel(uint64_t chain, int *sink)
{
    typedef int v4i __attribute__((ext_vector_type(4)));
    typedef int v16i __attribute__((ext_vector_type(16)));
    v4i a = {(int)threadIdx.x, 1, 2, 3}, b = {3, 2, 1, (int)blockIdx.x};
    v16i acc0 = {0}, acc1 = {0}, acc2 = {0}, acc3 = {0};
    for (uint64_t i = 0; i < chain; i += 4u) {
        acc0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, acc0, 0, 0, 0);
        acc1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, acc1, 0, 0, 0);
        acc2 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, acc2, 0, 0, 0);
        acc3 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, acc3, 0, 0, 0);
    }
    const int folded = acc0[0] ^ acc1[1] ^ acc2[2] ^ acc3[3];
    if (folded == 0x7fffffff && acc0[5] == 0x7ffffffe) *sink = folded;   // practically never
}

__global__ void probe_kernel(int *out)
{
    if (out) *out = 950;
}

}  // namespace yvex

using namespace yvex;

extern "C" {

const char *yvex_hip_last_error(void) { return g_last_error; }

int yvex_hip_device_count(void)
{
    int count = 0;
    if (hipGetDeviceCount(&count) != hipSuccess) {
        (void)hipGetLastError();
        return 0;
    }
    return count;
}

int yvex_hip_device_info(int device, char *name, unsigned long name_cap, char *arch,
                         unsigned long arch_cap, uint64_t *total_bytes, uint64_t *free_bytes,
                         int *compute_units)
{
    hipDeviceProp_t prop;
    size_t free_b = 0, total_b = 0;
    int rc = wrap("hipGetDeviceProperties", hipGetDeviceProperties(&prop, device));
    if (rc) return rc;
    if (name && name_cap) snprintf(name, name_cap, "%s", prop.name);
    if (arch && arch_cap) snprintf(arch, arch_cap, "%s", prop.gcnArchName);
    if (compute_units) *compute_units = prop.multiProcessorCount;
    rc = wrap("hipSetDevice", hipSetDevice(device));
    if (rc) return rc;
    rc = wrap("hipMemGetInfo", hipMemGetInfo(&free_b, &total_b));
    if (rc) return rc;
    if (total_bytes) *total_bytes = total_b;
    if (free_bytes) *free_bytes = free_b;
    return ST_OK;
}

int yvex_hip_device_clocks(int device, int *engine_khz, int *memory_khz)
{
    int engine = 0, memory = 0;
    int rc = wrap("hipDeviceGetAttribute", hipDeviceGetAttribute(&engine, hipDeviceAttributeClockRate, device));
    if (!rc) rc = wrap("hipDeviceGetAttribute",
                       hipDeviceGetAttribute(&memory, hipDeviceAttributeMemoryClockRate, device));
    if (rc) return rc;
    if (engine_khz) *engine_khz = engine;
    if (memory_khz) *memory_khz = memory;
    return ST_OK;
}

int yvex_hip_kernels_loadable(void)
{
    // Fail closed: the code object counts as present only if a kernel from it really launches.
    int *flag = nullptr, host = 0;
    if (yvex_hip_device_count() <= 0) return 0;
    if (hipMalloc(&flag, sizeof(int)) != hipSuccess) {
        (void)hipGetLastError();
        return 0;
    }
    (void)hipMemset(flag, 0, sizeof(int));
    probe_kernel<<<1, 1>>>(flag);
    bool ok = hipGetLastError() == hipSuccess && hipDeviceSynchronize() == hipSuccess &&
              hipMemcpy(&host, flag, sizeof(int), hipMemcpyDeviceToHost) == hipSuccess;
    (void)hipFree(flag);
    (void)hipGetLastError();
    return ok && host == 950;
}

int yvex_hip_malloc(void **out, uint64_t bytes)
{
    if (!out) return ST_INVALID_ARG;
    *out = nullptr;
    return wrap("hipMalloc", hipMalloc(out, bytes ? bytes : 1));
}
int yvex_hip_free(void *ptr) { return ptr ? wrap("hipFree", hipFree(ptr)) : ST_OK; }

int yvex_hip_host_alloc(void **out, uint64_t bytes)
{
    if (!out) return ST_INVALID_ARG;
    *out = nullptr;
    return wrap("hipHostMalloc", hipHostMalloc(out, bytes ? bytes : 1, hipHostMallocDefault));
}
int yvex_hip_host_free(void *ptr) { return ptr ? wrap("hipHostFree", hipHostFree(ptr)) : ST_OK; }

int yvex_hip_memcpy_h2d(void *dst, const void *src, uint64_t bytes, yvex_hip_stream stream)
{
    if (!bytes) return ST_OK;
    int rc = wrap("hipMemcpyAsync(h2d)",
                  hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, as_stream(stream)));
    return rc ? rc : wrap("hipStreamSynchronize", hipStreamSynchronize(as_stream(stream)));
}
int yvex_hip_memcpy_h2d_queued(void *dst, const void *src, uint64_t bytes, yvex_hip_stream stream)
{
    if (!bytes) return ST_OK;
    return wrap("hipMemcpyAsync(h2d)",
                hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, as_stream(stream)));
}
int yvex_hip_memcpy_d2h(void *dst, const void *src, uint64_t bytes, yvex_hip_stream stream)
{
    if (!bytes) return ST_OK;
    int rc = wrap("hipMemcpyAsync(d2h)",
                  hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, as_stream(stream)));
    return rc ? rc : wrap("hipStreamSynchronize", hipStreamSynchronize(as_stream(stream)));
}
int yvex_hip_memcpy_d2d(void *dst, const void *src, uint64_t bytes, yvex_hip_stream stream)
{
    if (!bytes) return ST_OK;
    return wrap("hipMemcpyAsync(d2d)",
                hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, as_stream(stream)));
}

int yvex_hip_stream_create(yvex_hip_stream *out)
{
    hipStream_t s = nullptr;
    if (!out) return ST_INVALID_ARG;
    int rc = wrap("hipStreamCreate", hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
    *out = rc ? nullptr : reinterpret_cast<yvex_hip_stream>(s);
    return rc;
}
int yvex_hip_stream_destroy(yvex_hip_stream stream)
{
    return stream ? wrap("hipStreamDestroy", hipStreamDestroy(as_stream(stream))) : ST_OK;
}
int yvex_hip_stream_sync(yvex_hip_stream stream)
{
    return wrap("hipStreamSynchronize", hipStreamSynchronize(as_stream(stream)));
}

int yvex_hip_stream_read(const void *data, uint64_t bytes, uint32_t *sink, yvex_hip_stream stream)
{
    if (!data || !sink || bytes < 16u || ((uintptr_t)data & 15u)) return ST_INVALID_ARG;
    stream_read_kernel<<<256 * 16, 256, 0, as_stream(stream)>>>((const uint4 *)data, bytes / 16u, sink);
    return check_launch("stream_read");
}

int yvex_hip_bandwidth_sample(const void *source, void *destination, uint64_t bytes, uint64_t iterations,
                              uint32_t *sink, uint64_t *elapsed_ns, yvex_hip_stream stream)
{
    if (!source || !elapsed_ns || !iterations || bytes < 16u || ((uintptr_t)source & 15u) ||
        (!destination && !sink))
        return ST_INVALID_ARG;
    hipStream_t s = as_stream(stream);
    hipEvent_t begin = nullptr, end = nullptr;
    int rc = wrap("hipEventCreate", hipEventCreate(&begin));
    if (!rc) rc = wrap("hipEventCreate", hipEventCreate(&end));
    if (!rc) rc = wrap("hipEventRecord", hipEventRecord(begin, s));
    for (uint64_t i = 0; !rc && i < iterations; ++i) {
        if (destination) {
            rc = wrap("hipMemcpyAsync(d2d)", hipMemcpyAsync(destination, source, bytes, hipMemcpyDeviceToDevice, s));
        } else {
            stream_read_kernel<<<256 * 16, 256, 0, s>>>((const uint4 *)source, bytes / 16u, sink);
            rc = check_launch("stream_read");
        }
    }
    if (!rc) rc = wrap("hipEventRecord", hipEventRecord(end, s));
    if (!rc) rc = wrap("hipEventSynchronize", hipEventSynchronize(end));
    float ms = 0.0f;
    if (!rc) rc = wrap("hipEventElapsedTime", hipEventElapsedTime(&ms, begin, end));
    if (begin) (void)hipEventDestroy(begin);
    if (end) (void)hipEventDestroy(end);
    if (rc) return rc;
    *elapsed_ns = (uint64_t)((double)ms * 1.0e6);
    return ST_OK;
}

int yvex_hip_clock_probe(uint64_t chain, int *sink, yvex_hip_stream stream)
{
    if (!chain || (chain & 3u) || !sink) return ST_INVALID_ARG;
    clock_probe_kernel<<<compute_units(), 256, 0, as_stream(stream)>>>(chain, sink);
    return check_launch("clock_probe");
}

int yvex_hip_fill_u32(void *dst, uint32_t value, uint64_t count, yvex_hip_stream stream)
{
    if (!count) return ST_OK;
    if (!dst || ((uintptr_t)dst & 3u)) return ST_INVALID_ARG;
    uint64_t blocks = (count + 255u) / 256u;
    if (blocks > 0x7fffffffull) return ST_BOUNDS;
    fill_u32_kernel<<<(unsigned)blocks, 256, 0, as_stream(stream)>>>((uint32_t *)dst, value, count);
    return check_launch("fill_u32");
}

// ---- launch graphs: a captured kernel sequence replayed with one submission ----

int yvex_hip_capture_begin(yvex_hip_stream stream)
{
    return wrap("hipStreamBeginCapture",
                hipStreamBeginCapture(as_stream(stream), hipStreamCaptureModeThreadLocal));
}

int yvex_hip_capture_abort(yvex_hip_stream stream)
{
    hipGraph_t graph = nullptr;
    hipError_t code = hipStreamEndCapture(as_stream(stream), &graph);
    if (graph) (void)hipGraphDestroy(graph);
    (void)hipGetLastError();
    return code == hipSuccess ? ST_OK : ST_BACKEND;
}

int yvex_hip_capture_end(yvex_hip_stream stream, yvex_hip_graph *out, uint64_t *kernel_nodes)
{
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    size_t count = 0;
    if (!out) return ST_INVALID_ARG;
    *out = nullptr;
    if (kernel_nodes) *kernel_nodes = 0;
    int rc = wrap("hipStreamEndCapture", hipStreamEndCapture(as_stream(stream), &graph));
    if (rc || !graph) return rc ? rc : ST_BACKEND;
    // Only kernel nodes are replayed: a memset or copy node would mean a launch wrapper did
    // something a replay cannot be trusted to repeat.
    rc = wrap("hipGraphGetNodes", hipGraphGetNodes(graph, nullptr, &count));
    if (!rc && count) {
        std::vector<hipGraphNode_t> nodes(count);
        rc = wrap("hipGraphGetNodes", hipGraphGetNodes(graph, nodes.data(), &count));
        for (size_t i = 0; !rc && i < count; ++i) {
            hipGraphNodeType type;
            rc = wrap("hipGraphNodeGetType", hipGraphNodeGetType(nodes[i], &type));
            if (!rc && type != hipGraphNodeTypeKernel) {
                set_last_error_text("launch graph holds a node that is not a kernel");
                rc = ST_UNSUPPORTED;
            }
        }
    }
    if (!rc && !count) {
        set_last_error_text("launch graph is empty");
        rc = ST_UNSUPPORTED;
    }
    if (!rc) rc = wrap("hipGraphInstantiate", hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0));
    (void)hipGraphDestroy(graph);
    if (rc) return rc;
    if (kernel_nodes) *kernel_nodes = count;
    *out = reinterpret_cast<yvex_hip_graph>(exec);
    return ST_OK;
}

int yvex_hip_graph_launch(yvex_hip_graph graph, yvex_hip_stream stream)
{
    if (!graph) return ST_INVALID_ARG;
    return wrap("hipGraphLaunch",
                hipGraphLaunch(reinterpret_cast<hipGraphExec_t>(graph), as_stream(stream)));
}

int yvex_hip_graph_destroy(yvex_hip_graph graph)
{
    return graph ? wrap("hipGraphExecDestroy", hipGraphExecDestroy(reinterpret_cast<hipGraphExec_t>(graph)))
                 : ST_OK;
}

}  // extern "C"
