// The library's file-scope device scratch and the one entry point that uses it.
//
// smelt_hip_encode_prefill_record_static_scratch is smelt_hip_encode_prefill_record for callers
// that may not allocate device memory: the split-K kernels it launches keep their partial sums and
// arrival counters in the array below instead of the workspace a context allocates.  Every GPU the
// library runs on holds its own copy of the array at its own address until the process ends; the
// host-side name `scratch` is only a handle for hipGetSymbolAddress and is never passed to a
// kernel, a fill or a copy.
#include <hip/hip_runtime.h>

#include <atomic>
#include <mutex>
#include <string>

#include "../../include/smelt_hip.h"
#include "runtime_internal.hpp"

namespace {

constexpr size_t kCounterBytes = (size_t)64 << 10;    // 16384 tile counters
constexpr size_t kPartialBytes = SMELT_HIP_STATIC_SCRATCH_BYTES;   // 4096 workgroup partials of 4 KB
constexpr size_t kScratchBytes = kCounterBytes + kPartialBytes;
constexpr int kMaxDevices = 64;

static __device__ __align__(256) unsigned char scratch[kScratchBytes];

// device address of `scratch` on each device, filled by static_scratch_prepare
std::atomic<void*> g_scratch_ptr[kMaxDevices] = {};
std::mutex g_scratch_mutex;

__global__ __launch_bounds__(256) void smelt_static_scratch_fill(uint32_t* words, uint32_t count, uint32_t value) {
    for (uint32_t i = blockIdx.x * blockDim.x + threadIdx.x; i < count; i += gridDim.x * blockDim.x) words[i] = value;
}

// zero `count` counters with a fill kernel (a memset node must not end up in a caller's graph)
hipError_t clear_counters(void* base, size_t count, hipStream_t stream) {
    if (count == 0) return hipSuccess;
    const unsigned blocks = (unsigned)((count + 255) / 256 < 64 ? (count + 255) / 256 : 64);
    (void)hipGetLastError();   // the launch's own status is wanted, not an earlier call's
    hipLaunchKernelGGL(smelt_static_scratch_fill, dim3(blocks), dim3(256), 0, stream,
                       static_cast<uint32_t*>(base), (uint32_t)count, 0u);
    return hipGetLastError();
}

}  // namespace

namespace smelt_host {

int static_scratch_prepare(int device, hipStream_t stream, std::string* why) {
    if (device < 0 || device >= kMaxDevices) {
        *why = "static scratch: device index out of range";
        return SMELT_HIP_ERR_INVALID_ARGUMENT;
    }
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_ptr[device].load(std::memory_order_acquire)) return SMELT_HIP_OK;
    // the caller has made `device` current
    void* ptr = nullptr;
    hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr) {
        *why = std::string("hipGetSymbolAddress(static scratch): ") + hipGetErrorString(e);
        return SMELT_HIP_ERR_HIP;
    }
    e = clear_counters(ptr, kCounterBytes / 4, stream);
    if (e == hipSuccess) e = hipStreamSynchronize(stream);
    if (e != hipSuccess) {
        *why = std::string("clearing the static scratch: ") + hipGetErrorString(e);
        return SMELT_HIP_ERR_HIP;
    }
    g_scratch_ptr[device].store(ptr, std::memory_order_release);
    return SMELT_HIP_OK;
}

}  // namespace smelt_host

extern "C" {

int smelt_hip_encode_prefill_record_static_scratch(smelt_hip_context* ctx, const SmeltDispatchRecord* rec, int cur,
                                                   int alt, int32_t seq_len, int32_t start_pos) {
    using namespace smelt_host;
    if (!ctx || !rec) return context_fail(ctx, SMELT_HIP_ERR_INVALID_ARGUMENT, "null context or record");
    const int device = context_device(ctx);
    void* base = device >= 0 && device < kMaxDevices ? g_scratch_ptr[device].load(std::memory_order_acquire) : nullptr;
    if (!base) return context_fail(ctx, SMELT_HIP_ERR_HIP, "the static scratch was not set up on this device");
    {
        const hipError_t e = hipSetDevice(device);   // the array's address belongs to this device
        if (e != hipSuccess) return context_fail(ctx, SMELT_HIP_ERR_HIP, std::string("hipSetDevice: ") + hipGetErrorString(e));
    }
    SplitKWorkspace ws;
    ws.counters = base;
    ws.counter_bytes = kCounterBytes;
    ws.partial = static_cast<unsigned char*>(base) + kCounterBytes;
    ws.partial_bytes = kPartialBytes;
    // The counters must be zero when a split-K launch starts.  They are cleared once per device at set-up and
    // every split-K kernel leaves the counters it used at zero when it finishes, so a call launches nothing
    // but the record's own kernel (records that do not split K never touch them).  Calls that overlap on one
    // GPU share the array and race; that is the caller's to avoid.
    return encode_prefill_with_workspace(ctx, rec, cur, alt, seq_len, start_pos, ws);
}

}  // extern "C"
