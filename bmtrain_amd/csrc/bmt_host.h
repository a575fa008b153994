// Host-side helpers shared by the launchers: per-thread error text, device properties.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace bmt {

// Records `what` (plus the HIP error string when `e` is given) as the calling
// thread's last error and returns `code`.
int fail(int code, const char *what, hipError_t e = hipSuccess);
// Same for code that does not see the HIP headers.
int fail_message(int code, const char *what);

// Number of compute units of the current device (cached per device).
int device_cu_count();

// Ticket counters for one launch of a resident kernel on `stream`: a slot of the per-device table that
// cross_entropy.hip keeps (one slot per stream; launches on one stream follow each other, so a slot is never used by
// two running launches).  False when the launch has to do without: a stream under graph capture, the per-thread
// default stream, a stream of another device than the current one, or a full table with nothing to hand on.
// `counted` says whether the call shows in bmt_hip_flat_stream_stats (the in-place cross-entropy kernels do).
struct StreamSlot {
    uint32_t *tickets;      // device: the slot's first word
    uint32_t *done_word;    // pinned host memory: the last workgroup of the launch writes `number` here
    uint32_t number;        // this launch's number on the slot
};
bool stream_slot_for(hipStream_t stream, StreamSlot *slot, bool counted);

}  // namespace bmt
