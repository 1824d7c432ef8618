// Device, memory, stream and event entry points of the C ABI.
//
// The reference keeps one cuBLAS handle per (device, thread) and relies on the
// per-thread default stream (Sources/Sapphire/compute/dense/cuda/Gemm.cu:24-30,
// CMake/CompileOptions.cmake:227).  Here the same slot holds a HIP stream:
// every thread gets its own non-blocking stream per device, created on first
// use at the default priority and handed back to a free list when the thread
// ends, so no stream is destroyed while the runtime may be shutting down.
#include "sph_internal.h"

#include <atomic>

#include <cstring>
#include <mutex>
#include <vector>

namespace
{
constexpr int kMaxDevices = 16;

thread_local std::string tlsLastError;

std::mutex gPoolMutex;
std::vector<hipStream_t> gIdleStreams[kMaxDevices];
int gComputeUnits[kMaxDevices] = {};
bool gPoolRetains[kMaxDevices] = {};

struct ThreadSlots
{
    int device = 0;
    hipStream_t own[kMaxDevices] = {};
    hipStream_t borrowed[kMaxDevices] = {};
    hipStream_t capturing = nullptr;  // stream under capture, if any

    ~ThreadSlots()
    {
        std::lock_guard<std::mutex> lock(gPoolMutex);
        for (int d = 0; d < kMaxDevices; ++d)
            if (own[d] != nullptr)
                gIdleStreams[d].push_back(own[d]);
    }
};

thread_local ThreadSlots tlsSlots;
}  // namespace

namespace
{
std::atomic<uint64_t> gAllocations{0};
}

namespace sph
{
void CountAllocation()
{
    gAllocations.fetch_add(1, std::memory_order_relaxed);
}

int Fail(int status, const std::string& msg)
{
    tlsLastError = msg;
    return status;
}

int CurrentDevice()
{
    return tlsSlots.device;
}

hipStream_t CurrentStream()
{
    const int d = tlsSlots.device;
    if (tlsSlots.borrowed[d] != nullptr)
        return tlsSlots.borrowed[d];
    if (tlsSlots.own[d] == nullptr)
    {
        {
            std::lock_guard<std::mutex> lock(gPoolMutex);
            if (!gIdleStreams[d].empty())
            {
                tlsSlots.own[d] = gIdleStreams[d].back();
                gIdleStreams[d].pop_back();
            }
        }
        if (tlsSlots.own[d] == nullptr)
        {
            hipStream_t s = nullptr;
            hipError_t err = hipSetDevice(d);
            if (err == hipSuccess)
                err = hipStreamCreateWithFlags(&s, hipStreamNonBlocking);
            if (err != hipSuccess)
            {
                Fail(SPH_ERR_DEVICE, std::string("stream creation failed with ") +
                                         hipGetErrorString(err));
                return nullptr;
            }
            tlsSlots.own[d] = s;
        }
    }
    return tlsSlots.own[d];
}

bool Capturing()
{
    return tlsSlots.capturing != nullptr;
}

int ComputeUnits()
{
    const int d = tlsSlots.device;
    if (gComputeUnits[d] == 0)
    {
        int cu = 0;
        if (hipDeviceGetAttribute(&cu, hipDeviceAttributeMultiprocessorCount, d) !=
                hipSuccess ||
            cu <= 0)
            cu = 256;
        gComputeUnits[d] = cu;
    }
    return gComputeUnits[d];
}
}  // namespace sph

#define SPH_STREAM_OR_FAIL(var)                                                \
    hipStream_t var = ::sph::CurrentStream();                                  \
    if (var == nullptr)                                                        \
    return SPH_ERR_DEVICE

extern "C" {

const char* sph_last_error(void)
{
    return tlsLastError.c_str();
}

int sph_device_count(int* count)
{
    SPH_REQUIRE(count != nullptr, "count is null");
    int n = 0;
    const hipError_t err = hipGetDeviceCount(&n);
    if (err != hipSuccess)
    {
        *count = 0;
        return sph::Fail(SPH_ERR_DEVICE, std::string("hipGetDeviceCount failed with ") +
                                             hipGetErrorString(err));
    }
    *count = n;
    return SPH_OK;
}

int sph_set_device(int deviceId)
{
    SPH_REFUSE_WHILE_CAPTURING();
    int n = 0;
    const int rc = sph_device_count(&n);
    if (rc != SPH_OK)
        return rc;
    // Memory.cpp:14-28: an id at or beyond the device count is refused
    if (deviceId < 0 || deviceId >= n || deviceId >= kMaxDevices)
        return sph::Fail(SPH_ERR_INVALID,
                         "sph_set_device - deviceId exceeds number of available devices");
    SPH_HIP_TRY(hipSetDevice(deviceId));
    tlsSlots.device = deviceId;
    return SPH_OK;
}

int sph_get_device(int* deviceId)
{
    SPH_REQUIRE(deviceId != nullptr, "deviceId is null");
    *deviceId = tlsSlots.device;
    return SPH_OK;
}

int sph_device_info(int deviceId, SphDeviceInfo* info)
{
    SPH_REQUIRE(info != nullptr, "info is null");
    hipDeviceProp_t prop;
    SPH_HIP_TRY(hipGetDeviceProperties(&prop, deviceId));
    std::memset(info, 0, sizeof(*info));
    std::strncpy(info->name, prop.name, sizeof(info->name) - 1);
    std::strncpy(info->arch, prop.gcnArchName, sizeof(info->arch) - 1);
    info->computeUnits = prop.multiProcessorCount;
    info->clockMHz = prop.clockRate / 1000;
    info->memoryClockMHz = prop.memoryClockRate / 1000;
    info->memoryBusWidthBits = prop.memoryBusWidth;
    info->ldsBytesPerBlock = static_cast<int>(prop.sharedMemPerBlock);
    info->l2Bytes = prop.l2CacheSize;
    info->totalMemoryBytes = prop.totalGlobalMem;
    info->wavefrontSize = prop.warpSize;
    return SPH_OK;
}

int sph_malloc(void** ptr, size_t bytes)
{
    SPH_REFUSE_WHILE_CAPTURING();
    SPH_REQUIRE(ptr != nullptr, "ptr is null");
    SPH_HIP_TRY(hipSetDevice(tlsSlots.device));
    ::sph::CountAllocation();
    SPH_HIP_TRY(hipMalloc(ptr, bytes));
    return SPH_OK;
}

int sph_free(void* ptr)
{
    SPH_REFUSE_WHILE_CAPTURING();
    SPH_HIP_TRY(hipFree(ptr));
    return SPH_OK;
}

int sph_malloc_async(void** ptr, size_t bytes)
{
    SPH_REFUSE_WHILE_CAPTURING();
    SPH_REQUIRE(ptr != nullptr, "ptr is null");
    SPH_STREAM_OR_FAIL(stream);
    const int d = tlsSlots.device;
    {
        // freed blocks stay in the device's pool instead of going back to the driver
        std::lock_guard<std::mutex> lock(gPoolMutex);
        if (!gPoolRetains[d])
        {
            hipMemPool_t pool = nullptr;
            SPH_HIP_TRY(hipDeviceGetDefaultMemPool(&pool, d));
            uint64_t keep = ~0ull;
            SPH_HIP_TRY(hipMemPoolSetAttribute(pool, hipMemPoolAttrReleaseThreshold, &keep));
            gPoolRetains[d] = true;
        }
    }
    ::sph::CountAllocation();
    SPH_HIP_TRY(hipMallocAsync(ptr, bytes != 0 ? bytes : 1, stream));
    return SPH_OK;
}

int sph_free_async(void* ptr)
{
    SPH_REFUSE_WHILE_CAPTURING();
    if (ptr == nullptr)
        return SPH_OK;
    SPH_STREAM_OR_FAIL(stream);
    SPH_HIP_TRY(hipFreeAsync(ptr, stream));
    return SPH_OK;
}

int sph_allocation_count(uint64_t* count)
{
    SPH_REQUIRE(count != nullptr, "count is null");
    *count = gAllocations.load(std::memory_order_relaxed);
    return SPH_OK;
}

int sph_mem_pool_trim(void)
{
    SPH_REFUSE_WHILE_CAPTURING();
    hipMemPool_t pool = nullptr;
    SPH_HIP_TRY(hipDeviceGetDefaultMemPool(&pool, tlsSlots.device));
    SPH_HIP_TRY(hipMemPoolTrimTo(pool, 0));
    return SPH_OK;
}

int sph_host_malloc(void** ptr, size_t bytes)
{
    SPH_REFUSE_WHILE_CAPTURING();
    SPH_REQUIRE(ptr != nullptr, "ptr is null");
    ::sph::CountAllocation();
    SPH_HIP_TRY(hipHostMalloc(ptr, bytes, hipHostMallocDefault));
    return SPH_OK;
}

int sph_host_free(void* ptr)
{
    SPH_REFUSE_WHILE_CAPTURING();
    SPH_HIP_TRY(hipHostFree(ptr));
    return SPH_OK;
}

int sph_memcpy_h2d(void* dev, const void* host, size_t bytes)
{
    SPH_REFUSE_WHILE_CAPTURING();
    if (bytes == 0)
        return SPH_OK;
    SPH_REQUIRE(dev != nullptr && host != nullptr, "null pointer");
    SPH_STREAM_OR_FAIL(stream);
    SPH_HIP_TRY(hipMemcpyAsync(dev, host, bytes, hipMemcpyHostToDevice, stream));
    SPH_HIP_TRY(hipStreamSynchronize(stream));
    return SPH_OK;
}

int sph_memcpy_d2h(void* host, const void* dev, size_t bytes)
{
    SPH_REFUSE_WHILE_CAPTURING();
    if (bytes == 0)
        return SPH_OK;
    SPH_REQUIRE(dev != nullptr && host != nullptr, "null pointer");
    SPH_STREAM_OR_FAIL(stream);
    SPH_HIP_TRY(hipMemcpyAsync(host, dev, bytes, hipMemcpyDeviceToHost, stream));
    SPH_HIP_TRY(hipStreamSynchronize(stream));
    return SPH_OK;
}

int sph_memcpy_d2d(void* dst, const void* src, size_t bytes)
{
    SPH_REFUSE_WHILE_CAPTURING();
    if (bytes == 0)
        return SPH_OK;
    SPH_REQUIRE(dst != nullptr && src != nullptr, "null pointer");
    SPH_STREAM_OR_FAIL(stream);
    SPH_HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, stream));
    SPH_HIP_TRY(hipStreamSynchronize(stream));
    return SPH_OK;
}

int sph_memcpy_d2d_async(void* dst, const void* src, size_t bytes)
{
    if (bytes == 0)
        return SPH_OK;
    SPH_REQUIRE(dst != nullptr && src != nullptr, "null pointer");
    SPH_STREAM_OR_FAIL(stream);
    SPH_HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, stream));
    return SPH_OK;
}

int sph_stream_sync(void)
{
    SPH_REFUSE_WHILE_CAPTURING();
    SPH_STREAM_OR_FAIL(stream);
    SPH_HIP_TRY(hipStreamSynchronize(stream));
    return SPH_OK;
}

int sph_device_sync(void)
{
    SPH_REFUSE_WHILE_CAPTURING();
    SPH_HIP_TRY(hipSetDevice(tlsSlots.device));
    SPH_HIP_TRY(hipDeviceSynchronize());
    return SPH_OK;
}

int sph_stream_wait_stream(void* hipStream)
{
    SPH_REFUSE_WHILE_CAPTURING();
    SPH_STREAM_OR_FAIL(stream);
    hipStream_t other = static_cast<hipStream_t>(hipStream);
    if (other == nullptr || other == stream)
        return SPH_OK;
    hipEvent_t marker = nullptr;
    SPH_HIP_TRY(hipEventCreateWithFlags(&marker, hipEventDisableTiming));
    hipError_t err = hipEventRecord(marker, other);
    if (err == hipSuccess)
        err = hipStreamWaitEvent(stream, marker, 0);
    // the event's resources are released once the wait has been satisfied
    const hipError_t destroyed = hipEventDestroy(marker);
    if (err == hipSuccess)
        err = destroyed;
    if (err != hipSuccess)
        return sph::Fail(SPH_ERR_DEVICE, std::string("sph_stream_wait_stream failed with ") +
                                             hipGetErrorString(err));
    return SPH_OK;
}

int sph_get_stream(void** hipStream)
{
    SPH_REQUIRE(hipStream != nullptr, "hipStream is null");
    SPH_STREAM_OR_FAIL(stream);
    *hipStream = stream;
    return SPH_OK;
}

int sph_set_stream(void* hipStream)
{
    SPH_REFUSE_WHILE_CAPTURING();
    tlsSlots.borrowed[tlsSlots.device] = static_cast<hipStream_t>(hipStream);
    return SPH_OK;
}

int sph_event_create(void** event)
{
    SPH_REQUIRE(event != nullptr, "event is null");
    hipEvent_t ev = nullptr;
    SPH_HIP_TRY(hipEventCreate(&ev));
    *event = ev;
    return SPH_OK;
}

int sph_event_record(void* event)
{
    SPH_REQUIRE(event != nullptr, "event is null");
    SPH_STREAM_OR_FAIL(stream);
    SPH_HIP_TRY(hipEventRecord(static_cast<hipEvent_t>(event), stream));
    return SPH_OK;
}

int sph_event_elapsed_ms(void* start, void* stop, float* ms)
{
    SPH_REFUSE_WHILE_CAPTURING();
    SPH_REQUIRE(start != nullptr && stop != nullptr && ms != nullptr, "null argument");
    SPH_HIP_TRY(hipEventSynchronize(static_cast<hipEvent_t>(stop)));
    SPH_HIP_TRY(hipEventElapsedTime(ms, static_cast<hipEvent_t>(start),
                                    static_cast<hipEvent_t>(stop)));
    return SPH_OK;
}

int sph_event_destroy(void* event)
{
    SPH_REQUIRE(event != nullptr, "event is null");
    SPH_HIP_TRY(hipEventDestroy(static_cast<hipEvent_t>(event)));
    return SPH_OK;
}

int sph_graph_begin_capture(void)
{
    SPH_REQUIRE(!sph::Capturing(), "a capture is already in progress on this thread");
    // resolve everything that queries the device before the stream goes into capture
    (void)sph::ComputeUnits();
    {
        const int rc = sph::ResolveCsrScratch(nullptr);
        if (rc != SPH_OK)
            return rc;
    }
    SPH_STREAM_OR_FAIL(stream);
    SPH_HIP_TRY(hipStreamBeginCapture(stream, hipStreamCaptureModeThreadLocal));
    tlsSlots.capturing = stream;
    return SPH_OK;
}

int sph_graph_end_capture(void** graph)
{
    SPH_REQUIRE(graph != nullptr, "graph is null");
    SPH_REQUIRE(sph::Capturing(), "no capture in progress on this thread");
    hipStream_t stream = tlsSlots.capturing;
    tlsSlots.capturing = nullptr;
    *graph = nullptr;
    hipGraph_t recorded = nullptr;
    SPH_HIP_TRY(hipStreamEndCapture(stream, &recorded));
    if (recorded == nullptr)
        return sph::Fail(SPH_ERR_DEVICE, "sph_graph_end_capture - the capture was invalidated");
    hipGraphExec_t exec = nullptr;
    const hipError_t err = hipGraphInstantiate(&exec, recorded, nullptr, nullptr, 0);
    (void)hipGraphDestroy(recorded);
    if (err != hipSuccess)
        return sph::Fail(SPH_ERR_DEVICE, std::string("hipGraphInstantiate failed with ") +
                                             hipGetErrorString(err));
    *graph = exec;
    return SPH_OK;
}

int sph_graph_launch(void* graph)
{
    SPH_REQUIRE(graph != nullptr, "graph is null");
    SPH_REFUSE_WHILE_CAPTURING();
    SPH_STREAM_OR_FAIL(stream);
    SPH_HIP_TRY(hipGraphLaunch(static_cast<hipGraphExec_t>(graph), stream));
    return SPH_OK;
}

int sph_graph_destroy(void* graph)
{
    SPH_REQUIRE(graph != nullptr, "graph is null");
    SPH_HIP_TRY(hipGraphExecDestroy(static_cast<hipGraphExec_t>(graph)));
    return SPH_OK;
}

}  // extern "C"
