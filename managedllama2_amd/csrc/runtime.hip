// Runtime half of the C ABI: device context, memory, stream, events, errors.
// Replaces what the reference gets from ManagedCuda (CudaContext,
// CudaDeviceVariable<T>; src/Module.cs:7-26, src/RunState.cs:27-53).
#include "common.hpp"

#include <cstdio>
#include <cstdlib>
#include <cstring>

namespace l2 {

static Context g_ctx;
// 32 heads x 64 blocks x (128 partial outputs + block max + block sum) floats
constexpr size_t kAttnPartialsFloor = sizeof(float) * 32 * 64 * 130;
static thread_local char g_err[512] = "";

Context& ctx() { return g_ctx; }

int fail(int code, const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

int hip_fail(hipError_t e, const char* what)
{
    snprintf(g_err, sizeof(g_err), "%s: %s (%d)", what, hipGetErrorString(e), static_cast<int>(e));
    return static_cast<int>(e);
}

int ensure_attn_partials(size_t bytes)
{
    Context& c = ctx();
    if (bytes <= c.attn_partials_bytes)
        return LLAMA2_OK;
    if (c.capturing)
        return fail(LLAMA2_ERR_INVALID_ARGUMENT,
                    "scratch of %zu bytes must exist before graph capture starts (run the call once eagerly first)", bytes);
    // The old buffer is never freed here: kernels already on the stream may still use it, and a
    // graph the caller captured earlier keeps its address in its kernel arguments.  It is retired
    // and released at llama2_shutdown.  Sizes at least double, so a handful of buffers covers any
    // growth; the first request is rounded up to what a 32-head, 8192-row context needs.
    size_t want = bytes < kAttnPartialsFloor ? kAttnPartialsFloor : bytes;
    if (want < 2 * c.attn_partials_bytes)
        want = 2 * c.attn_partials_bytes;
    if (c.attn_partials && c.n_retired_partials >= kMaxRetiredPartials)
        return fail(LLAMA2_ERR_UNSUPPORTED, "attention scratch grew more than %d times", kMaxRetiredPartials);
    float* fresh = nullptr;
    L2_HIP(hipMalloc(reinterpret_cast<void**>(&fresh), want));
    if (c.attn_partials)
        c.retired_partials[c.n_retired_partials++] = c.attn_partials;
    c.attn_partials = fresh;
    c.attn_partials_bytes = want;
    return LLAMA2_OK;
}

std::recursive_mutex& api_mutex()
{
    static std::recursive_mutex m;
    return m;
}

int bind_thread()
{
    static thread_local int bound_device = -1;
    const int device = ctx().device;
    if (bound_device != device) {
        L2_HIP(hipSetDevice(device));
        bound_device = device;
    }
    return LLAMA2_OK;
}

} // namespace l2

using namespace l2;

extern "C" {

const char* llama2_last_error(void) { return g_err; }

int llama2_init(int device)
{
    std::lock_guard<std::recursive_mutex> lock(api_mutex());
    Context& c = ctx();
    if (c.ready && c.device == device)
        return LLAMA2_OK;
    if (c.ready)
        return fail(LLAMA2_ERR_INVALID_ARGUMENT, "llama2_init: already bound to device %d", c.device);
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess || count <= 0)
        return fail(LLAMA2_ERR_NO_DEVICE, "llama2_init: no HIP device (%s)", hipGetErrorString(e));
    if (device < 0 || device >= count)
        return fail(LLAMA2_ERR_INVALID_ARGUMENT, "llama2_init: device %d out of range [0,%d)", device, count);
    L2_HIP(hipSetDevice(device));
    hipDeviceProp_t prop;
    L2_HIP(hipGetDeviceProperties(&prop, device));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return fail(LLAMA2_ERR_NO_DEVICE, "llama2_init: device %d is %s, this library is built for gfx950 only",
                    device, prop.gcnArchName);
    c.num_cus = prop.multiProcessorCount;
    L2_HIP(hipStreamCreateWithFlags(&c.stream, hipStreamNonBlocking));
    L2_HIP(hipMalloc(reinterpret_cast<void**>(&c.attn_counters), kMaxAttnHeads * sizeof(unsigned)));
    L2_HIP(hipMemset(c.attn_counters, 0, kMaxAttnHeads * sizeof(unsigned)));
    L2_HIP(hipMalloc(reinterpret_cast<void**>(&c.sort_keys), LLAMA2_MAX_SAMPLER_SIZE * sizeof(uint16_t)));
    L2_HIP(hipMalloc(reinterpret_cast<void**>(&c.sort_values), LLAMA2_MAX_SAMPLER_SIZE * sizeof(int)));
    c.device = device;
    if (int rc = resolve_vec_mat_static_scratch(device)) {
        c.device = -1;
        return rc;
    }
    c.int4_narrow = getenv("LLAMA2_INT4_NARROW") != nullptr;
    c.int4_blocks = getenv("LLAMA2_INT4_BLOCKS") != nullptr;
    c.int4_no_span = getenv("LLAMA2_INT4_NO_SPAN") != nullptr;
    c.attn_waves = getenv("LLAMA2_ATTN_WAVES") ? atoi(getenv("LLAMA2_ATTN_WAVES")) : 0;
    c.ready = true;
    g_err[0] = 0;
    return LLAMA2_OK;
}

int llama2_shutdown(void)
{
    std::lock_guard<std::recursive_mutex> lock(api_mutex());
    Context& c = ctx();
    if (!c.ready)
        return LLAMA2_OK;
    L2_HIP(hipStreamSynchronize(c.stream));
    if (c.attn_partials)
        L2_HIP(hipFree(c.attn_partials));
    c.attn_partials = nullptr;
    c.attn_partials_bytes = 0;
    for (int i = 0; i < c.n_retired_partials; ++i)
        L2_HIP(hipFree(c.retired_partials[i]));
    c.n_retired_partials = 0;
    if (c.attn_counters)
        L2_HIP(hipFree(c.attn_counters));
    c.attn_counters = nullptr;
    if (c.sort_keys)
        L2_HIP(hipFree(c.sort_keys));
    c.sort_keys = nullptr;
    if (c.sort_values)
        L2_HIP(hipFree(c.sort_values));
    c.sort_values = nullptr;
    L2_HIP(hipStreamDestroy(c.stream));
    c.stream = nullptr;
    c.ready = false;
    c.device = -1;
    return LLAMA2_OK;
}

int llama2_malloc(void** ptr, size_t bytes)
{
    L2_REQUIRE_INIT();
    if (ctx().capturing)
        return fail(LLAMA2_ERR_INVALID_ARGUMENT, "llama2_malloc: not allowed during graph capture");
    L2_CHECK(ptr != nullptr, "llama2_malloc: ptr is null");
    *ptr = nullptr;
    L2_CHECK(bytes > 0, "llama2_malloc: zero-sized allocation");
    L2_HIP(hipMalloc(ptr, bytes));
    return LLAMA2_OK;
}

int llama2_free(void* ptr)
{
    L2_REQUIRE_INIT();
    if (ctx().capturing)
        return fail(LLAMA2_ERR_INVALID_ARGUMENT, "llama2_free: not allowed during graph capture");
    if (!ptr)
        return LLAMA2_OK;
    L2_HIP(hipStreamSynchronize(ctx().stream));
    L2_HIP(hipFree(ptr));
    return LLAMA2_OK;
}

int llama2_memcpy_h2d(void* dst, size_t dst_offset_bytes, const void* src, size_t bytes)
{
    L2_REQUIRE_INIT();
    if (ctx().capturing)
        return fail(LLAMA2_ERR_INVALID_ARGUMENT, "llama2_memcpy_h2d: not allowed during graph capture");
    if (bytes == 0)
        return LLAMA2_OK;
    L2_CHECK(dst && src, "llama2_memcpy_h2d: null pointer");
    // Pageable source: hipMemcpyAsync stages it before returning, so the host
    // buffer may be reused at once, and the copy is ordered on the stream.
    L2_HIP(hipMemcpyAsync(static_cast<char*>(dst) + dst_offset_bytes, src, bytes, hipMemcpyHostToDevice,
                          ctx().stream));
    L2_HIP(hipStreamSynchronize(ctx().stream));
    return LLAMA2_OK;
}

int llama2_memcpy_d2h(void* dst, const void* src, size_t src_offset_bytes, size_t bytes)
{
    L2_REQUIRE_INIT();
    if (ctx().capturing)
        return fail(LLAMA2_ERR_INVALID_ARGUMENT, "llama2_memcpy_d2h: not allowed during graph capture");
    if (bytes == 0)
        return LLAMA2_OK;
    L2_CHECK(dst && src, "llama2_memcpy_d2h: null pointer");
    L2_HIP(hipMemcpyAsync(dst, static_cast<const char*>(src) + src_offset_bytes, bytes,
                          hipMemcpyDeviceToHost, ctx().stream));
    L2_HIP(hipStreamSynchronize(ctx().stream));
    return LLAMA2_OK;
}

__global__ void fill_bytes_kernel(uint8_t* dst, uint8_t v, size_t n)
{
    size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
    for (; i < n; i += stride)
        dst[i] = v;
}

int llama2_memset(void* dst, int byte_value, size_t bytes)
{
    L2_REQUIRE_INIT();
    if (bytes == 0)
        return LLAMA2_OK;
    L2_CHECK(dst, "llama2_memset: null pointer");
    // A fill kernel rather than hipMemsetAsync, so the call stays safe to
    // record into a captured graph.
    size_t blocks = (bytes + 255) / 256;
    if (blocks > 4096)
        blocks = 4096;
    hipLaunchKernelGGL(fill_bytes_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, ctx().stream,
                       static_cast<uint8_t*>(dst), static_cast<uint8_t>(byte_value), bytes);
    L2_LAUNCH_CHECK("fill_bytes_kernel");
    return LLAMA2_OK;
}

// Plain 16-byte-per-lane copy: every byte is read once and written once.
__global__ __launch_bounds__(256) void copy_bytes_kernel(u32x4* dst, const u32x4* src, size_t n16)
{
    size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    const size_t stride = static_cast<size_t>(gridDim.x) * 256;
    for (; i < n16; i += stride)
        dst[i] = src[i];
}

int llama2_memcpy_d2d(void* dst, const void* src, size_t bytes)
{
    L2_REQUIRE_INIT();
    if (bytes == 0)
        return LLAMA2_OK;
    L2_CHECK(dst && src, "llama2_memcpy_d2d: null pointer");
    L2_CHECK(aligned(dst, 16) && aligned(src, 16) && bytes % 16 == 0,
             "llama2_memcpy_d2d: pointers and size must be multiples of 16 bytes");
    L2_CHECK(!overlap(dst, bytes, src, bytes), "llama2_memcpy_d2d: ranges overlap");
    size_t blocks = (bytes / 16 + 1023) / 1024;
    if (blocks > 65536)
        blocks = 65536;
    hipLaunchKernelGGL(copy_bytes_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, ctx().stream,
                       static_cast<u32x4*>(dst), static_cast<const u32x4*>(src), bytes / 16);
    L2_LAUNCH_CHECK("copy_bytes_kernel");
    return LLAMA2_OK;
}

int llama2_mem_info(size_t* free_bytes, size_t* total_bytes)
{
    L2_REQUIRE_INIT();
    size_t f = 0, t = 0;
    L2_HIP(hipMemGetInfo(&f, &t));
    if (free_bytes)
        *free_bytes = f;
    if (total_bytes)
        *total_bytes = t;
    return LLAMA2_OK;
}

int llama2_sync(void)
{
    L2_REQUIRE_INIT();
    if (ctx().capturing)
        return fail(LLAMA2_ERR_INVALID_ARGUMENT, "llama2_sync: not allowed during graph capture");
    L2_HIP(hipStreamSynchronize(ctx().stream));
    return LLAMA2_OK;
}

void* llama2_stream(void) { return ctx().ready ? static_cast<void*>(ctx().stream) : nullptr; }

#define L2_NOT_CAPTURING(fn)                                                                  \
    do {                                                                                      \
        if (ctx().capturing)                                                                  \
            return fail(LLAMA2_ERR_INVALID_ARGUMENT, fn ": not allowed during graph capture"); \
    } while (0)

int llama2_graph_begin_capture(void)
{
    L2_REQUIRE_INIT();
    L2_NOT_CAPTURING("llama2_graph_begin_capture");
    L2_HIP(hipStreamBeginCapture(ctx().stream, hipStreamCaptureModeThreadLocal));
    ctx().capturing = true;
    api_mutex().lock(); // released by llama2_graph_end_capture: no other thread may launch into the capture
    return LLAMA2_OK;
}

int llama2_graph_end_capture(void** graph)
{
    L2_REQUIRE_INIT();
    L2_CHECK(graph, "llama2_graph_end_capture: null pointer");
    *graph = nullptr;
    if (!ctx().capturing)
        return fail(LLAMA2_ERR_INVALID_ARGUMENT, "llama2_graph_end_capture: no capture in progress");
    ctx().capturing = false;
    hipGraph_t g = nullptr;
    const hipError_t ended = hipStreamEndCapture(ctx().stream, &g);
    api_mutex().unlock(); // taken by llama2_graph_begin_capture (this call still holds its own)
    if (ended != hipSuccess)
        return hip_fail(ended, "hipStreamEndCapture");
    hipGraphExec_t exec = nullptr;
    hipError_t e = hipGraphInstantiate(&exec, g, nullptr, nullptr, 0);
    (void)hipGraphDestroy(g);
    if (e != hipSuccess)
        return hip_fail(e, "hipGraphInstantiate");
    *graph = exec;
    return LLAMA2_OK;
}

int llama2_graph_launch(void* graph)
{
    L2_REQUIRE_INIT();
    L2_CHECK(graph, "llama2_graph_launch: null graph");
    L2_NOT_CAPTURING("llama2_graph_launch");
    L2_HIP(hipGraphLaunch(static_cast<hipGraphExec_t>(graph), ctx().stream));
    return LLAMA2_OK;
}

int llama2_graph_destroy(void* graph)
{
    L2_REQUIRE_INIT();
    if (!graph)
        return LLAMA2_OK;
    L2_HIP(hipStreamSynchronize(ctx().stream));
    L2_HIP(hipGraphExecDestroy(static_cast<hipGraphExec_t>(graph)));
    return LLAMA2_OK;
}

int llama2_event_create(void** event)
{
    L2_REQUIRE_INIT();
    L2_CHECK(event, "llama2_event_create: null pointer");
    hipEvent_t ev;
    L2_HIP(hipEventCreate(&ev));
    *event = ev;
    return LLAMA2_OK;
}

int llama2_event_record(void* event)
{
    L2_REQUIRE_INIT();
    L2_CHECK(event, "llama2_event_record: null event");
    L2_HIP(hipEventRecord(static_cast<hipEvent_t>(event), ctx().stream));
    return LLAMA2_OK;
}

int llama2_event_elapsed_ms(void* start, void* stop, float* ms)
{
    L2_REQUIRE_INIT();
    L2_CHECK(start && stop && ms, "llama2_event_elapsed_ms: null pointer");
    L2_HIP(hipEventSynchronize(static_cast<hipEvent_t>(stop)));
    L2_HIP(hipEventElapsedTime(ms, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(stop)));
    return LLAMA2_OK;
}

int llama2_event_destroy(void* event)
{
    L2_REQUIRE_INIT();
    if (event)
        L2_HIP(hipEventDestroy(static_cast<hipEvent_t>(event)));
    return LLAMA2_OK;
}

} // extern "C"
