// Internal seams of the runtime shared between its translation units (not part of the C ABI).
#pragma once
#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>
#include <string>

#include "../../include/smelt_hip.h"

namespace smelt_host {

// Split-K scratch a launch may use: partial sums and per-tile arrival counters.  The counters are
// zero whenever no launch is in flight (the last workgroup of a tile resets its own).
struct SplitKWorkspace {
    void* partial = nullptr;
    void* counters = nullptr;
    size_t partial_bytes = 0;
    size_t counter_bytes = 0;
};

// emitDispatchRecord with the split-K scratch taken from `ws` instead of the context's own
// allocation.  Returns 1 launched, 0 skipped, negative status on error.
int encode_prefill_with_workspace(smelt_hip_context* ctx, const SmeltDispatchRecord* rec, int cur, int alt,
                                  int32_t seq_len, int32_t start_pos, const SplitKWorkspace& ws);

int context_device(const smelt_hip_context* ctx);
hipStream_t context_stream(const smelt_hip_context* ctx);
int context_fail(const smelt_hip_context* ctx, int code, const std::string& message);

// The library's file-scope device scratch: looked up once per device when a context is created on
// it (defined next to the array).  Returns a SMELT_HIP status; on failure `why` names the HIP error.
int static_scratch_prepare(int device, hipStream_t stream, std::string* why);

}  // namespace smelt_host
