// Host-pointer path of the package functions: what `functions[name](A, B, C)` of a HAT package runs
// (/root/reference/README.md:118-136, /root/reference/accera/python/accera/Package.py:776-784: a function of a HOST
// package takes NumPy arrays, i.e. pageable host memory).
//
// The caller's arrays are pageable, and this system does not let existing memory be pinned after the fact, so every
// byte goes through pinned staging buffers that the library allocates itself (hipHostMalloc):
//   * one context per call in flight -- device buffers for A, B, C, a ring of pinned staging slots, a stream and one
//     event per slot -- taken from a pool for the duration of the call, so calls from different host threads do not
//     wait for each other (each brings or reuses its own context);
//   * host to device: the caller's bytes are copied into a staging slot by a few worker threads, the slot is sent with
//     an asynchronous copy, and the next slot is filled meanwhile (a slot is reused once its copy's event has passed);
//   * the kernel runs on the context's stream behind the copies;
//   * device to host: the same ring the other way round -- the copies of the first slots are queued at once, each slot is
//     copied out to the caller's array when its event has passed and then queued again for a later piece.
#include "host_path.h"

#include <atomic>
#include <condition_variable>
#include <cstring>
#include <mutex>
#include <thread>
#include <vector>

namespace acc950 {

namespace {

constexpr size_t kSlotBytes = (size_t)4 << 20; // one staging slot
constexpr int kSlots = 4;
constexpr int kCopyThreads = 6;               // workers that move bytes between the caller's arrays and the staging slots
constexpr size_t kParallelFrom = (size_t)256 << 10; // smaller pieces are copied by the calling thread alone

// ---- worker threads for the copies on the host ------------------------------------------------
// A fixed set of threads, started at the first large copy.  One copy at a time is dealt out (callers take turns);
// the calling thread takes a share itself.  The threads live until the process ends.
class CopyPool {
public:
    void copy(char* dst, const char* src, size_t bytes)
    {
        if (bytes < kParallelFrom) { std::memcpy(dst, src, bytes); return; }
        std::lock_guard<std::mutex> turn(turn_);
        start_workers();
        const size_t parts = kCopyThreads + 1;
        const size_t per = ((bytes + parts - 1) / parts + 4095) & ~(size_t)4095;
        {
            std::lock_guard<std::mutex> lock(m_);
            dst_ = dst; src_ = src; bytes_ = bytes; per_ = per;
            next_part_ = 0; parts_left_ = 0;
            for (size_t off = 0; off < bytes; off += per) ++parts_left_;
            ++generation_;
        }
        wake_.notify_all();
        work(); // the caller's share
        std::unique_lock<std::mutex> lock(m_);
        done_.wait(lock, [&] { return parts_left_ == 0; });
    }

private:
    void start_workers()
    {
        if (started_) return;
        started_ = true;
        for (int i = 0; i < kCopyThreads; ++i) std::thread([this] { loop(); }).detach();
    }
    // takes pieces of the current copy until none is left
    void work()
    {
        for (;;) {
            size_t off;
            {
                std::lock_guard<std::mutex> lock(m_);
                off = next_part_ * per_;
                if (off >= bytes_) return;
                ++next_part_;
            }
            const size_t n = bytes_ - off < per_ ? bytes_ - off : per_;
            std::memcpy(dst_ + off, src_ + off, n);
            std::lock_guard<std::mutex> lock(m_);
            if (--parts_left_ == 0) done_.notify_all();
        }
    }
    void loop()
    {
        unsigned long long seen = 0;
        for (;;) {
            {
                std::unique_lock<std::mutex> lock(m_);
                wake_.wait(lock, [&] { return generation_ != seen; });
                seen = generation_;
            }
            work();
        }
    }
    std::mutex turn_, m_;
    std::condition_variable wake_, done_;
    bool started_ = false;
    char* dst_ = nullptr;
    const char* src_ = nullptr;
    size_t bytes_ = 0, per_ = 1, next_part_ = 0, parts_left_ = 0;
    unsigned long long generation_ = 0;
};

CopyPool& copy_pool()
{
    static CopyPool* pool = new CopyPool; // (never destroyed: its threads may still be parked when the process ends)
    return *pool;
}

// ---- contexts ------------------------------------------------------------------------------
struct DevBuf {
    void* p = nullptr;
    size_t bytes = 0;
};

struct HostContext {
    int device = 0;
    hipStream_t stream = nullptr;
    DevBuf a, b, c;
    char* slot[kSlots] = {};
    hipEvent_t event[kSlots] = {};
};

std::mutex g_pool_mutex;
std::vector<HostContext*> g_idle; // contexts not in use, any device
std::atomic<unsigned long long>* g_allocations = nullptr;

hipError_t make_context(int device, HostContext** out)
{
    HostContext* c = new HostContext;
    c->device = device;
    hipError_t e = hipStreamCreateWithFlags(&c->stream, hipStreamNonBlocking);
    for (int i = 0; i < kSlots && e == hipSuccess; ++i) {
        e = hipHostMalloc((void**)&c->slot[i], kSlotBytes, hipHostMallocDefault);
        if (e == hipSuccess) e = hipEventCreateWithFlags(&c->event[i], hipEventDisableTiming);
    }
    if (e != hipSuccess) {
        for (int i = 0; i < kSlots; ++i) {
            if (c->event[i]) (void)hipEventDestroy(c->event[i]);
            if (c->slot[i]) (void)hipHostFree(c->slot[i]);
        }
        if (c->stream) (void)hipStreamDestroy(c->stream);
        delete c;
        return e;
    }
    *out = c;
    return hipSuccess;
}

hipError_t acquire(HostContext** out)
{
    int device = 0;
    hipError_t e = hipGetDevice(&device);
    if (e != hipSuccess) return e;
    {
        std::lock_guard<std::mutex> lock(g_pool_mutex);
        for (size_t i = 0; i < g_idle.size(); ++i)
            if (g_idle[i]->device == device) {
                *out = g_idle[i];
                g_idle.erase(g_idle.begin() + (long)i);
                return hipSuccess;
            }
    }
    return make_context(device, out);
}

void release(HostContext* c)
{
    std::lock_guard<std::mutex> lock(g_pool_mutex);
    g_idle.push_back(c);
}

hipError_t reserve(DevBuf& b, size_t bytes)
{
    if (bytes <= b.bytes) return hipSuccess;
    if (b.p) {
        hipError_t e = hipFree(b.p);
        if (e != hipSuccess) return e;
        b.p = nullptr;
        b.bytes = 0;
    }
    hipError_t e = hipMalloc(&b.p, bytes);
    if (e == hipSuccess) {
        b.bytes = bytes;
        if (g_allocations) ++*g_allocations;
    }
    return e;
}

// caller's array -> device buffer, through the staging ring
hipError_t upload(HostContext& c, void* dev, const void* host, size_t bytes)
{
    const char* src = (const char*)host;
    size_t piece = 0;
    for (size_t off = 0; off < bytes; off += kSlotBytes, ++piece) {
        const int s = (int)(piece % kSlots);
        const size_t n = bytes - off < kSlotBytes ? bytes - off : kSlotBytes;
        // (the slot's last copy to the device -- of this call or an earlier one -- has read it)
        hipError_t e = hipEventSynchronize(c.event[s]);
        if (e != hipSuccess) return e;
        copy_pool().copy(c.slot[s], src + off, n);
        e = hipMemcpyAsync((char*)dev + off, c.slot[s], n, hipMemcpyHostToDevice, c.stream);
        if (e == hipSuccess) e = hipEventRecord(c.event[s], c.stream);
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

// device buffer -> caller's array
hipError_t download(HostContext& c, void* host, const void* dev, size_t bytes)
{
    char* dst = (char*)host;
    const size_t pieces = (bytes + kSlotBytes - 1) / kSlotBytes;
    auto queue = [&](size_t piece) {
        const size_t off = piece * kSlotBytes, n = bytes - off < kSlotBytes ? bytes - off : kSlotBytes;
        const int s = (int)(piece % kSlots);
        hipError_t e = hipMemcpyAsync(c.slot[s], (const char*)dev + off, n, hipMemcpyDeviceToHost, c.stream);
        if (e == hipSuccess) e = hipEventRecord(c.event[s], c.stream);
        return e;
    };
    // (stream order puts these behind the kernel, and behind the uploads that last read the slots)
    for (size_t piece = 0; piece < pieces && piece < (size_t)kSlots; ++piece)
        if (hipError_t e = queue(piece); e != hipSuccess) return e;
    for (size_t piece = 0; piece < pieces; ++piece) {
        const size_t off = piece * kSlotBytes, n = bytes - off < kSlotBytes ? bytes - off : kSlotBytes;
        const int s = (int)(piece % kSlots);
        hipError_t e = hipEventSynchronize(c.event[s]);
        if (e != hipSuccess) return e;
        copy_pool().copy(dst + off, c.slot[s], n);
        if (piece + kSlots < pieces)
            if (e = queue(piece + kSlots); e != hipSuccess) return e;
    }
    return hipSuccess;
}

} // namespace

void host_path_count_allocations(std::atomic<unsigned long long>* counter) { g_allocations = counter; }

hipError_t host_path_release_idle(int device)
{
    std::vector<HostContext*> mine;
    {
        std::lock_guard<std::mutex> lock(g_pool_mutex);
        for (size_t i = 0; i < g_idle.size();) {
            if (g_idle[i]->device != device) { ++i; continue; }
            mine.push_back(g_idle[i]);
            g_idle.erase(g_idle.begin() + (long)i);
        }
    }
    // (a context goes back to the pool with its stream idle: nothing of it is in use any more)
    hipError_t first = hipSuccess;
    auto note = [&](hipError_t e) { if (e != hipSuccess && first == hipSuccess) first = e; };
    for (HostContext* c : mine) {
        for (DevBuf* b : {&c->a, &c->b, &c->c})
            if (b->p) note(hipFree(b->p));
        for (int i = 0; i < kSlots; ++i) {
            if (c->event[i]) note(hipEventDestroy(c->event[i]));
            if (c->slot[i]) note(hipHostFree(c->slot[i]));
        }
        if (c->stream) note(hipStreamDestroy(c->stream));
        delete c;
    }
    return first;
}

hipError_t host_path_run(const HostOperands& h, const HostLaunchFn& launch, int* launch_status)
{
    HostContext* c = nullptr;
    hipError_t e = acquire(&c);
    if (e != hipSuccess) return e;
    *launch_status = 0;
    do {
        if ((e = reserve(c->a, h.a_bytes ? h.a_bytes : 16)) != hipSuccess) break;
        if ((e = reserve(c->b, h.b_bytes ? h.b_bytes : 16)) != hipSuccess) break;
        if ((e = reserve(c->c, h.c_bytes ? h.c_bytes : 16)) != hipSuccess) break;
        if ((e = upload(*c, c->a.p, h.A, h.a_bytes)) != hipSuccess) break;
        if ((e = upload(*c, c->b.p, h.B, h.b_bytes)) != hipSuccess) break;
        if (h.send_c && (e = upload(*c, c->c.p, h.C, h.c_bytes)) != hipSuccess) break;
        *launch_status = launch(c->a.p, c->b.p, c->c.p, c->stream);
        if (*launch_status != 0) break;
        if ((e = download(*c, h.C, c->c.p, h.c_bytes)) != hipSuccess) break;
    } while (false);
    // whatever happened, the stream is idle and the slots are free when the context goes back
    hipError_t e2 = hipStreamSynchronize(c->stream);
    release(c);
    return e != hipSuccess ? e : e2;
}

} // namespace acc950
