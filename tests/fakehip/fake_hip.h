// A host-only stand-in for the HIP runtime, for running the backend's own host code (zyx_amd/csrc/*.cpp) on a
// machine without a GPU and under sanitizers. It executes nothing on a device: device memory is host memory,
// copies are memcpy, kernel launches only record which allocations they read and write.
//
// What it checks is ordering. Every stream carries a vector clock; an event copies the clock of the stream that
// records it, a wait merges it, host synchronisation merges into the host's clock, and work enqueued after the host
// has synchronised inherits the host's clock. Each allocation remembers its last writer and the readers since. An
// operation that touches an allocation whose last conflicting access is not ordered before it is a hazard
// (read-after-write, write-after-write, write-after-read): exactly the bugs a missing event wait causes on the GPU,
// where they show up as rare wrong results. The hazards found so far are read with fakehip_hazards().
#pragma once
#include <cstddef>
#include <string>
#include <vector>

typedef struct ihipStream_t *hipStream_t;

struct FakeAccess {
    const void *ptr; // any address inside a live allocation; null is ignored
    bool write;
};
// A kernel launch (called by the recording stand-ins of the kernel launchers). Returns false when a non-null pointer
// belongs to no live allocation (use after free, stale workspace).
bool fakehip_launch(hipStream_t stream, const char *name, const std::vector<FakeAccess> &accesses);

// Messages of the hazards and misuse seen since the last call (cleared by the call).
std::vector<std::string> fakehip_hazards();
// How many times an API function was called since the process started ("hipMalloc", "hipFree", "hipEventCreate", ...).
unsigned long fakehip_calls(const char *api);
// Kernel launches recorded so far, in issue order: "name@stream".
std::vector<std::string> fakehip_launch_log();
// Live device allocations (count, bytes).
void fakehip_live(size_t *count, size_t *bytes);
