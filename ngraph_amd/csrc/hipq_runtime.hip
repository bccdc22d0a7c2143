// Device plumbing of libhipq.so: errors, memory, streams, events, workspace, byte fill.
#include "hipq_common.h"

#include <mutex>

namespace hipq
{
    static thread_local char t_error[512] = "";
    static thread_local const char* t_kernel = "none";

    int fail(int code, const char* fmt, ...)
    {
        va_list ap;
        va_start(ap, fmt);
        vsnprintf(t_error, sizeof(t_error), fmt, ap);
        va_end(ap);
        return code;
    }

    void set_last_kernel(const char* name) { t_kernel = name; }

    int check_launch(const char* kernel)
    {
        hipError_t e = hipGetLastError();
        if (e != hipSuccess)
            return fail(HIPQ_ERR_HIP, "launch of %s failed: %s", kernel, hipGetErrorString(e));
        set_last_kernel(kernel);
        return HIPQ_OK;
    }

    static const int kMaxDevices = 16;
    static std::mutex g_ws_mutex;
    static void* g_ws_ptr[kMaxDevices] = {};
    static size_t g_ws_bytes[kMaxDevices] = {};
    static uint64_t g_ws_epoch[kMaxDevices] = {};

    int workspace(size_t bytes, void** ptr)
    {
        int dev = 0;
        HIPQ_HIP(hipGetDevice(&dev));
        if (dev < 0 || dev >= kMaxDevices)
            return fail(HIPQ_ERR_LIMIT, "device ordinal %d beyond %d", dev, kMaxDevices);
        std::lock_guard<std::mutex> lock(g_ws_mutex);
        if (g_ws_bytes[dev] < bytes)
        {
            if (g_ws_ptr[dev])
            {
                // earlier launches may still read the old block
                HIPQ_HIP(hipDeviceSynchronize());
                HIPQ_HIP(hipFree(g_ws_ptr[dev]));
                g_ws_ptr[dev] = nullptr;
                g_ws_bytes[dev] = 0;
            }
            size_t want = align_up(bytes + bytes / 4, 1 << 20);
            HIPQ_HIP(hipMalloc(&g_ws_ptr[dev], want));
            g_ws_bytes[dev] = want;
            ++g_ws_epoch[dev];
        }
        *ptr = g_ws_ptr[dev];
        return HIPQ_OK;
    }

    // Second grow-only block: partial sums of reductions split over workgroups, with a counter per
    // output tile at its head.  The counters are zeroed when the block is (re)allocated and every
    // kernel that uses them leaves them at zero.
    static void* g_split_ptr[kMaxDevices] = {};
    static size_t g_split_bytes[kMaxDevices] = {};
    int split_workspace(size_t partial_bytes, uint32_t** counters, void** partials)
    {
        int dev = 0;
        HIPQ_HIP(hipGetDevice(&dev));
        if (dev < 0 || dev >= kMaxDevices)
            return fail(HIPQ_ERR_LIMIT, "device ordinal %d beyond %d", dev, kMaxDevices);
        std::lock_guard<std::mutex> lock(g_ws_mutex);
        const size_t need = kSplitCounterBytes + partial_bytes;
        if (g_split_bytes[dev] < need)
        {
            if (g_split_ptr[dev])
            {
                HIPQ_HIP(hipDeviceSynchronize());
                HIPQ_HIP(hipFree(g_split_ptr[dev]));
                g_split_ptr[dev] = nullptr;
                g_split_bytes[dev] = 0;
            }
            size_t want = align_up(need + need / 4, 1 << 20);
            HIPQ_HIP(hipMalloc(&g_split_ptr[dev], want));
            HIPQ_HIP(hipMemset(g_split_ptr[dev], 0, kSplitCounterBytes));
            HIPQ_HIP(hipDeviceSynchronize());
            g_split_bytes[dev] = want;
            ++g_ws_epoch[dev];
        }
        *counters = static_cast<uint32_t*>(g_split_ptr[dev]);
        *partials = static_cast<uint8_t*>(g_split_ptr[dev]) + kSplitCounterBytes;
        return HIPQ_OK;
    }

    __global__ void fill_bytes_kernel(uint8_t* dst, uint32_t pattern, size_t bytes)
    {
        size_t i = (static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x) * 16;
        size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x * 16;
        for (; i < bytes; i += stride)
        {
            if (i + 16 <= bytes && (reinterpret_cast<uintptr_t>(dst + i) & 15) == 0)
            {
                *reinterpret_cast<uint4*>(dst + i) = make_uint4(pattern, pattern, pattern, pattern);
            }
            else
            {
                for (size_t j = i; j < bytes && j < i + 16; ++j)
                    dst[j] = static_cast<uint8_t>(pattern);
            }
        }
    }
}

using namespace hipq;

extern "C" {

const char* hipq_last_error(void)
{
    return t_error;
}

const char* hipq_last_kernel(void)
{
    return t_kernel;
}

int hipq_version(void)
{
    return 100;
}

int hipq_device_count(int* count)
{
    HIPQ_REQUIRE(count, "count is null");
    *count = 0;
    HIPQ_HIP(hipGetDeviceCount(count));
    return HIPQ_OK;
}

int hipq_set_device(int ordinal)
{
    int n = 0;
    HIPQ_HIP(hipGetDeviceCount(&n));
    if (ordinal < 0 || ordinal >= n)
        return fail(HIPQ_ERR_INVALID, "device ordinal %d out of range (%d devices)", ordinal, n);
    HIPQ_HIP(hipSetDevice(ordinal));
    return HIPQ_OK;
}

int hipq_get_device_info(hipq_device_info_t* info)
{
    HIPQ_REQUIRE(info, "info is null");
    int dev = 0;
    HIPQ_HIP(hipGetDevice(&dev));
    hipDeviceProp_t p;
    HIPQ_HIP(hipGetDeviceProperties(&p, dev));
    memset(info, 0, sizeof(*info));
    strncpy(info->name, p.name, sizeof(info->name) - 1);
    strncpy(info->arch, p.gcnArchName, sizeof(info->arch) - 1);
    info->compute_units = p.multiProcessorCount;
    info->clock_mhz = p.clockRate / 1000;
    info->lds_bytes_per_cu = static_cast<int32_t>(p.maxSharedMemoryPerMultiProcessor);
    info->hbm_bytes = p.totalGlobalMem;
    return HIPQ_OK;
}

int hipq_malloc(void** dptr, size_t bytes)
{
    HIPQ_REQUIRE(dptr, "dptr is null");
    *dptr = nullptr;
    HIPQ_HIP(hipMalloc(dptr, bytes ? bytes : 1));
    return HIPQ_OK;
}

int hipq_free(void* dptr)
{
    if (dptr)
        HIPQ_HIP(hipFree(dptr));
    return HIPQ_OK;
}

int hipq_memcpy_h2d(void* dst, const void* src, size_t bytes, void* stream)
{
    if (bytes == 0)
        return HIPQ_OK;
    HIPQ_REQUIRE(dst && src, "null pointer in memcpy_h2d");
    HIPQ_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, as_stream(stream)));
    HIPQ_HIP(hipStreamSynchronize(as_stream(stream)));
    return HIPQ_OK;
}

int hipq_memcpy_d2h(void* dst, const void* src, size_t bytes, void* stream)
{
    if (bytes == 0)
        return HIPQ_OK;
    HIPQ_REQUIRE(dst && src, "null pointer in memcpy_d2h");
    HIPQ_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, as_stream(stream)));
    HIPQ_HIP(hipStreamSynchronize(as_stream(stream)));
    return HIPQ_OK;
}

int hipq_memcpy_d2d(void* dst, const void* src, size_t bytes, void* stream)
{
    if (bytes == 0)
        return HIPQ_OK;
    HIPQ_REQUIRE(dst && src, "null pointer in memcpy_d2d");
    HIPQ_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, as_stream(stream)));
    return HIPQ_OK;
}

int hipq_fill_bytes(void* dst, int value, size_t bytes, void* stream)
{
    if (bytes == 0)
        return HIPQ_OK;
    HIPQ_REQUIRE(dst, "dst is null");
    uint32_t b = static_cast<uint32_t>(value) & 0xFF;
    uint32_t pattern = b | (b << 8) | (b << 16) | (b << 24);
    size_t chunks = (bytes + 15) / 16;
    unsigned blocks = static_cast<unsigned>(chunks / 256 + 1);
    if (blocks > 4096)
        blocks = 4096;
    fill_bytes_kernel<<<blocks, 256, 0, as_stream(stream)>>>(static_cast<uint8_t*>(dst), pattern, bytes);
    return check_launch("fill_bytes");
}

int hipq_stream_create(void** stream)
{
    HIPQ_REQUIRE(stream, "stream is null");
    hipStream_t s;
    HIPQ_HIP(hipStreamCreate(&s));
    *stream = s;
    return HIPQ_OK;
}

int hipq_stream_destroy(void* stream)
{
    if (stream)
        HIPQ_HIP(hipStreamDestroy(as_stream(stream)));
    return HIPQ_OK;
}

int hipq_stream_sync(void* stream)
{
    HIPQ_HIP(hipStreamSynchronize(as_stream(stream)));
    return HIPQ_OK;
}

int hipq_capture_begin(void* stream)
{
    HIPQ_REQUIRE(stream, "capture needs a stream of its own, not the null stream");
    HIPQ_HIP(hipStreamBeginCapture(as_stream(stream), hipStreamCaptureModeRelaxed));
    return HIPQ_OK;
}

int hipq_capture_end(void* stream, void** graph_exec)
{
    HIPQ_REQUIRE(stream && graph_exec, "null argument");
    *graph_exec = nullptr;
    hipGraph_t graph = nullptr;
    HIPQ_HIP(hipStreamEndCapture(as_stream(stream), &graph));
    hipGraphExec_t exec = nullptr;
    hipError_t e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
    (void)hipGraphDestroy(graph); // the executable graph keeps what it needs
    if (e != hipSuccess)
        return fail(HIPQ_ERR_HIP, "hipGraphInstantiate: %s", hipGetErrorString(e));
    *graph_exec = exec;
    return HIPQ_OK;
}

int hipq_graph_launch(void* graph_exec, void* stream)
{
    HIPQ_REQUIRE(graph_exec, "graph is null");
    HIPQ_HIP(hipGraphLaunch(reinterpret_cast<hipGraphExec_t>(graph_exec), as_stream(stream)));
    return HIPQ_OK;
}

int hipq_graph_destroy(void* graph_exec)
{
    if (graph_exec)
        HIPQ_HIP(hipGraphExecDestroy(reinterpret_cast<hipGraphExec_t>(graph_exec)));
    return HIPQ_OK;
}

uint64_t hipq_workspace_epoch(void)
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices)
        return 0;
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    return g_ws_epoch[dev];
}

int hipq_event_create(void** event)
{
    HIPQ_REQUIRE(event, "event is null");
    hipEvent_t e;
    HIPQ_HIP(hipEventCreate(&e));
    *event = e;
    return HIPQ_OK;
}

int hipq_event_destroy(void* event)
{
    if (event)
        HIPQ_HIP(hipEventDestroy(reinterpret_cast<hipEvent_t>(event)));
    return HIPQ_OK;
}

int hipq_event_record(void* event, void* stream)
{
    HIPQ_REQUIRE(event, "event is null");
    HIPQ_HIP(hipEventRecord(reinterpret_cast<hipEvent_t>(event), as_stream(stream)));
    return HIPQ_OK;
}

int hipq_event_sync(void* event)
{
    HIPQ_REQUIRE(event, "event is null");
    HIPQ_HIP(hipEventSynchronize(reinterpret_cast<hipEvent_t>(event)));
    return HIPQ_OK;
}

int hipq_event_elapsed_ms(void* start, void* stop, float* ms)
{
    HIPQ_REQUIRE(start && stop && ms, "null argument");
    HIPQ_HIP(hipEventElapsedTime(ms, reinterpret_cast<hipEvent_t>(start), reinterpret_cast<hipEvent_t>(stop)));
    return HIPQ_OK;
}
}
