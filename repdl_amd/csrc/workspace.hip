// Scratch memory of the entry points that need some: a small cache per device and stream.
//
// The stream-ordered allocator would be the natural source, but on this runtime a
// hipMallocAsync / hipFreeAsync pair around a kernel holds the HOST until the kernel has run
// (measured: 17 KiB allocated, a 0.9 ms kernel, freed -- 0.96 ms of host time per iteration
// against 19 us for the launch alone): every operator with a workspace then runs in lockstep
// with the GPU, and the side streams of a backward pass overlap nothing.  So the library keeps
// what it has allocated: a list of buffers per (device, stream), handed out to the calls on
// that stream and taken back when the call returns.  A buffer goes from one call to the next on
// the SAME stream only, whose work is ordered, so the next call's kernels cannot touch it before
// the previous call's are done; calls that nest (an entry point that calls another while it
// holds a buffer) get different buffers of the list.  Buffers grow to the largest size asked
// for and stay until the process ends.  A request beyond CACHE_LIMIT is not worth keeping and
// goes to the stream-ordered allocator.
#include <map>
#include <mutex>
#include <utility>
#include <vector>

#include "common.h"

namespace
{
constexpr size_t CACHE_LIMIT = (size_t)4 << 30;
struct Slot
{
    void *ptr;
    size_t bytes;
    bool busy;
};
std::mutex g_lock;
std::map<std::pair<int, hipStream_t>, std::vector<Slot>> g_slots;
} // namespace

hipError_t repdl_ws_acquire(void **p, size_t bytes, hipStream_t s)
{
    *p = nullptr;
    if (bytes == 0)
        return hipSuccess;
    if (bytes > CACHE_LIMIT)
        return hipMallocAsync(p, bytes, s);
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess)
        return e;
    std::lock_guard<std::mutex> guard(g_lock);
    std::vector<Slot> &v = g_slots[std::make_pair(dev, s)];
    Slot *best = nullptr, *spare = nullptr; // the smallest free buffer that is large enough; else any free one
    for (Slot &c : v)
    {
        if (c.busy)
            continue;
        if (c.bytes >= bytes && (best == nullptr || c.bytes < best->bytes))
            best = &c;
        if (spare == nullptr || c.bytes > spare->bytes)
            spare = &c;
    }
    if (best == nullptr)
    {
        // grow the largest free buffer, or add one (sizes in MiB steps from 64 KiB on, a quarter more than asked)
        size_t want = bytes <= ((size_t)64 << 10) ? ((bytes + 4095) & ~(size_t)4095) : (((bytes + bytes / 4) + ((size_t)1 << 20) - 1) & ~(((size_t)1 << 20) - 1));
        void *q = nullptr;
        if (spare != nullptr)
        {
            (void)hipFree(spare->ptr); // (waits for the device: the buffer's last kernels are done)
            spare->ptr = nullptr;
            spare->bytes = 0;
        }
        e = hipMalloc(&q, want);
        if (e != hipSuccess && want > bytes)
        {
            want = bytes;
            e = hipMalloc(&q, want);
        }
        if (e != hipSuccess)
        {
            if (spare != nullptr)
                v.erase(v.begin() + (spare - v.data()));
            return e;
        }
        if (spare != nullptr)
        {
            spare->ptr = q;
            spare->bytes = want;
            best = spare;
        }
        else
        {
            v.push_back(Slot{q, want, false});
            best = &v.back();
        }
    }
    best->busy = true;
    *p = best->ptr;
    return hipSuccess;
}

hipError_t repdl_ws_release(void *p, hipStream_t s)
{
    if (p == nullptr)
        return hipSuccess;
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess)
        return e;
    {
        std::lock_guard<std::mutex> guard(g_lock);
        auto it = g_slots.find(std::make_pair(dev, s));
        if (it != g_slots.end())
            for (Slot &c : it->second)
                if (c.ptr == p)
                {
                    c.busy = false;
                    return hipSuccess;
                }
    }
    return hipFreeAsync(p, s); // not one of the cache's: a request beyond CACHE_LIMIT
}
