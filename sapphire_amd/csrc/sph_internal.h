// Internal helpers shared by the translation units of libsapphire_hip.so.
#ifndef SPH_INTERNAL_H
#define SPH_INTERNAL_H

#include <hip/hip_runtime.h>

#include <cstdint>
#include <string>

#include "sapphire_hip.h"

namespace sph
{
// Records `msg` as this thread's last error and returns `status`.
int Fail(int status, const std::string& msg);

// Stream that this thread's work on the current device is enqueued on.
// Returns nullptr (and records the error) when it cannot be created.
hipStream_t CurrentStream();

// Device the calling thread last selected through sph_set_device (0 at start).
int CurrentDevice();

// Number of compute units of the current device (cached).
int ComputeUnits();

// Exclusive prefix sum of n 32-bit counts in place on `stream` (data[i] = sum of data[0..i)).
// With lastHost the last element (the total, when the last count is 0) is copied to the host
// and the stream is drained.
// Scans of more than ScanSingleLimit() values need one 32-bit total per 4096 values: taken from
// `sums` when that is not null (device memory, at least ScanBlocks(n) entries, contents
// irrelevant), from a stream-ordered allocation otherwise.
int ExclusiveScanInPlace(uint32_t* data, uint32_t n, uint32_t* lastHost, hipStream_t stream,
                         uint32_t* sums = nullptr);

// True when ExclusiveScanInPlace(data, n, lastHost, stream) would read back or allocate, which
// a stream under capture cannot record.  Entry points ask before they enqueue anything.
bool ScanWaitsOrAllocates(uint32_t n, const uint32_t* lastHost);

// Resolves, once per device, the address of the scratch array behind
// sph_csr_row_offsets_noalloc_f32 on the calling thread's device.
int ResolveCsrScratch(uint32_t** scratch);

// Counts one device or pinned-host allocation made by the library (read back through
// sph_allocation_count); called next to every hipMalloc / hipMallocAsync / hipHostMalloc.
void CountAllocation();

// True between sph_graph_begin_capture and sph_graph_end_capture on this thread.  Entry
// points that must wait for the device or allocate refuse to run while it is set.
bool Capturing();
}  // namespace sph

#define SPH_HIP_TRY(expr)                                                      \
    do                                                                         \
    {                                                                          \
        const hipError_t sphErr__ = (expr);                                    \
        if (sphErr__ != hipSuccess)                                            \
            return ::sph::Fail(SPH_ERR_DEVICE, std::string(#expr) +            \
                                                   " failed with " +           \
                                                   hipGetErrorString(sphErr__)); \
    } while (0)

#define SPH_REQUIRE(cond, what)                                                \
    do                                                                         \
    {                                                                          \
        if (!(cond))                                                           \
            return ::sph::Fail(SPH_ERR_INVALID, std::string(__func__) +        \
                                                    " - " + (what));           \
    } while (0)

// For entry points that synchronise, allocate or read back: not recordable into a graph.
#define SPH_REFUSE_WHILE_CAPTURING()                                           \
    do                                                                         \
    {                                                                          \
        if (::sph::Capturing())                                                \
            return ::sph::Fail(SPH_ERR_UNSUPPORTED,                            \
                               std::string(__func__) +                         \
                                   " - not available while a graph is being captured"); \
    } while (0)

// Checks the launch that was just issued.
#define SPH_CHECK_LAUNCH()                                                     \
    do                                                                         \
    {                                                                          \
        const hipError_t sphErr__ = hipGetLastError();                         \
        if (sphErr__ != hipSuccess)                                            \
            return ::sph::Fail(SPH_ERR_DEVICE, std::string(__func__) +         \
                                                   " launch failed with " +    \
                                                   hipGetErrorString(sphErr__)); \
    } while (0)

#endif
