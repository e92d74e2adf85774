// Host-pointer path of the package functions (host_path.hip): pageable arrays of the caller <-> device buffers through
// pinned staging, the kernel in between.
#pragma once
#include <hip/hip_runtime.h>
#include <atomic>
#include <functional>
#include <stddef.h>

namespace acc950 {

struct HostOperands {
    const void* A;
    const void* B;
    void* C;
    size_t a_bytes, b_bytes, c_bytes; // extent of each operand in the caller's memory (gaps of strided views included)
    bool send_c;                      // C travels to the device first (it is read, or its extent has gaps the copy back must keep)
};

// launches the kernel(s) on device copies of A, B, C on `stream`; returns the library's status code (0: ok)
typedef std::function<int(void* dA, void* dB, void* dC, hipStream_t stream)> HostLaunchFn;

// Copies in, launches, copies C back, and returns when C is in the caller's memory.  The HIP error of a copy or an
// allocation comes back as the return value, the launcher's status in *launch_status.  Calls from different host threads
// run side by side, each on a context of its own.
hipError_t host_path_run(const HostOperands& h, const HostLaunchFn& launch, int* launch_status);

// Frees the contexts of `device` that no call is using (their device buffers, pinned staging slots, events and streams);
// the next call on a host pointer makes a new one.
hipError_t host_path_release_idle(int device);

// device allocations of the path's contexts are added to this counter
void host_path_count_allocations(std::atomic<unsigned long long>* counter);

} // namespace acc950
