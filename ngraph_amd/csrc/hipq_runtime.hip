// Device plumbing of libhipq.so: errors, memory, streams, events, workspace, byte fill.
#include "hipq_common.h"

#include <map>
#include <mutex>
#include <utility>

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

    int device_compute_units()
    {
        static int cus[16] = {};
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 16)
            return 256;
        if (cus[dev] == 0)
        {
            hipDeviceProp_t prop;
            cus[dev] = hipGetDeviceProperties(&prop, dev) == hipSuccess && prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
        }
        return cus[dev];
    }

    __global__ void fill_bytes_kernel(uint8_t* dst, uint32_t pattern, size_t bytes);

    static const int kMaxDevices = 16;
    static std::mutex g_ws_mutex;
    static uint64_t g_ws_epoch[kMaxDevices] = {};

    struct Block
    {
        void* ptr = nullptr;
        size_t bytes = 0;
    };
    struct StreamBlocks
    {
        Block ws;    // layout copies
        Block split; // tile counters + partial sums
    };
    static std::map<std::pair<int, hipStream_t>, StreamBlocks> g_blocks;

    // Scratch of the entry point that allocates nothing: one array per device, resident from the
    // moment the library's code is loaded until the process ends.  Host code never uses the name
    // as an address; g_scratch_ptr[dev] is what hipGetSymbolAddress gave on that device.
    static __device__ __align__(256) unsigned char scratch[kScratchBytes];
    static unsigned char* g_scratch_ptr[kMaxDevices] = {};
    static thread_local int t_noalloc = 0;

    static int current_device(int* dev)
    {
        HIPQ_HIP(hipGetDevice(dev));
        if (*dev < 0 || *dev >= kMaxDevices)
            return fail(HIPQ_ERR_LIMIT, "device ordinal %d beyond %d", *dev, kMaxDevices);
        return HIPQ_OK;
    }

    // resolves the scratch array's address on the current device (once per device)
    static int resolve_scratch(int dev)
    {
        std::lock_guard<std::mutex> lock(g_ws_mutex);
        if (!g_scratch_ptr[dev])
        {
            void* p = nullptr;
            HIPQ_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
            if (!p)
                return fail(HIPQ_ERR_HIP, "the scratch array has no address on device %d", dev);
            g_scratch_ptr[dev] = static_cast<unsigned char*>(p);
        }
        return HIPQ_OK;
    }

    // hipq_set_device resolves the address, so a caller that selected its device through the library
    // never meets this step inside a graph capture; the check here serves callers that did not.
    int noalloc_begin()
    {
        int dev = 0;
        int rc = current_device(&dev);
        if (rc)
            return rc;
        rc = resolve_scratch(dev);
        if (rc)
            return rc;
        ++t_noalloc;
        return HIPQ_OK;
    }

    void noalloc_end()
    {
        if (t_noalloc > 0)
            --t_noalloc;
    }

    static int grow(Block& b, size_t need, hipStream_t stream, int dev, size_t zero_head)
    {
        if (b.bytes >= need)
            return HIPQ_OK;
        if (b.ptr)
        {
            // earlier launches on this stream may still use the old block
            HIPQ_HIP(hipStreamSynchronize(stream));
            HIPQ_HIP(hipFree(b.ptr));
            b.ptr = nullptr;
            b.bytes = 0;
        }
        const size_t want = align_up(need + need / 4, 1 << 20);
        HIPQ_HIP(hipMalloc(&b.ptr, want));
        if (zero_head)
        {
            HIPQ_HIP(hipMemset(b.ptr, 0, zero_head));
            HIPQ_HIP(hipDeviceSynchronize());
        }
        b.bytes = want;
        ++g_ws_epoch[dev];
        return HIPQ_OK;
    }

    int workspace(size_t bytes, hipStream_t stream, void** ptr)
    {
        int dev = 0;
        int rc = current_device(&dev);
        if (rc)
            return rc;
        if (t_noalloc)
        {
            if (bytes > kScratchWorkspaceBytes)
                return fail(HIPQ_ERR_LIMIT,
                            "this call needs a %zu-byte layout copy of its input; the entry point that allocates nothing holds %zu bytes for it",
                            bytes,
                            kScratchWorkspaceBytes);
            *ptr = g_scratch_ptr[dev];
            return HIPQ_OK;
        }
        std::lock_guard<std::mutex> lock(g_ws_mutex);
        Block& b = g_blocks[std::make_pair(dev, stream)].ws;
        rc = grow(b, bytes, stream, dev, 0);
        if (rc)
            return rc;
        *ptr = b.ptr;
        return HIPQ_OK;
    }

    // The counters are zeroed when the block is (re)allocated and every kernel that uses them
    // leaves them at zero.  The fixed array of the entry point that allocates nothing keeps whatever
    // its last call left, so there the counters are cleared (by a kernel: a caller may be capturing
    // a graph) ahead of every launch that uses them.
    int split_workspace(size_t partial_bytes, hipStream_t stream, uint32_t** counters, void** partials)
    {
        int dev = 0;
        int rc = current_device(&dev);
        if (rc)
            return rc;
        const size_t need = kSplitCounterBytes + partial_bytes;
        if (t_noalloc)
        {
            if (need > kScratchSplitBytes)
                return fail(HIPQ_ERR_LIMIT,
                            "this call needs %zu bytes of partial sums; the entry point that allocates nothing holds %zu bytes for them",
                            partial_bytes,
                            kScratchSplitBytes - kSplitCounterBytes);
            unsigned char* base = g_scratch_ptr[dev] + kScratchWorkspaceBytes;
            fill_bytes_kernel<<<static_cast<unsigned>(kSplitCounterBytes / 16 / 256), 256, 0, stream>>>(base, 0u, kSplitCounterBytes);
            rc = check_launch("fill_bytes");
            if (rc)
                return rc;
            *counters = reinterpret_cast<uint32_t*>(base);
            *partials = base + kSplitCounterBytes;
            return HIPQ_OK;
        }
        std::lock_guard<std::mutex> lock(g_ws_mutex);
        Block& b = g_blocks[std::make_pair(dev, stream)].split;
        rc = grow(b, need, stream, dev, kSplitCounterBytes);
        if (rc)
            return rc;
        *counters = static_cast<uint32_t*>(b.ptr);
        *partials = static_cast<uint8_t*>(b.ptr) + kSplitCounterBytes;
        return HIPQ_OK;
    }

    int release_stream_workspace(hipStream_t stream)
    {
        int dev = 0;
        int rc = current_device(&dev);
        if (rc)
            return rc;
        std::lock_guard<std::mutex> lock(g_ws_mutex);
        auto it = g_blocks.find(std::make_pair(dev, stream));
        if (it == g_blocks.end())
            return HIPQ_OK;
        const StreamBlocks blocks = it->second;
        g_blocks.erase(it);
        ++g_ws_epoch[dev];
        if (blocks.ws.ptr)
            HIPQ_HIP(hipFree(blocks.ws.ptr));
        if (blocks.split.ptr)
            HIPQ_HIP(hipFree(blocks.split.ptr));
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
    // set-up of the entry point that allocates nothing: the scratch array's address on this device
    return ordinal < kMaxDevices ? resolve_scratch(ordinal) : HIPQ_OK;
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
    {
        HIPQ_HIP(hipStreamSynchronize(as_stream(stream)));
        int rc = release_stream_workspace(as_stream(stream));
        if (rc)
            return rc;
        HIPQ_HIP(hipStreamDestroy(as_stream(stream)));
    }
    return HIPQ_OK;
}

int hipq_stream_release_scratch(void* stream)
{
    HIPQ_HIP(hipStreamSynchronize(as_stream(stream)));
    return release_stream_workspace(as_stream(stream));
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
    hipError_t d = hipGraphDestroy(graph); // the executable graph keeps what it needs
    if (e != hipSuccess)
        return fail(HIPQ_ERR_HIP, "hipGraphInstantiate: %s", hipGetErrorString(e));
    if (d != hipSuccess)
    {
        // a template graph that cannot be destroyed says the runtime's graph state is damaged:
        // hand back no executable rather than one that may replay wrongly
        (void)hipGraphExecDestroy(exec);
        return fail(HIPQ_ERR_HIP, "hipGraphDestroy after instantiation: %s", hipGetErrorString(d));
    }
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
