// Scratch memory of the entry points that need some.
//
// Two sources, chosen per call on the calling thread:
//
//  * The caller's workspace.  The *_ws entry points install the buffer they were given
//    (RepdlWorkspace) and run the plain entry point under it: every request, nested calls included,
//    is carved from that buffer in call order and given back in reverse order, so one buffer of
//    repdl_hip_<op>_workspace_bytes() serves the whole call.  Nothing is allocated, freed or kept;
//    such calls can be captured into a graph.  The same object in "dry" mode answers the size
//    queries: it runs the entry point's own host logic (route choice included) with the launches
//    switched off and records the peak.
//
//  * The library's cache, for the plain entry points.  The stream-ordered allocator would be the
//    natural source, but on this runtime a hipMallocAsync / hipFreeAsync pair around a kernel holds
//    the HOST until the kernel has run (measured: 17 KiB allocated, a 0.9 ms kernel, freed -- 0.96 ms
//    of host time per iteration against 19 us for the launch alone): every operator with a workspace
//    then runs in lockstep with the GPU, and the side streams of a backward pass overlap nothing.  So
//    the library keeps what it has allocated: a list of buffers per (device, stream), handed out to
//    the calls on that stream and taken back when the call returns.  A buffer goes from one call to
//    the next on the SAME stream only, whose work is ordered, so the next call's kernels cannot touch
//    it before the previous call's are done; calls that nest get different buffers of the list.
//    Buffers grow to the largest size asked for and stay until repdl_hip_scratch_trim() or the end
//    of the process.  A request beyond CACHE_LIMIT is not worth keeping and goes to the
//    stream-ordered allocator.
//    While the stream is being captured into a graph the cache neither allocates nor frees: a request
//    is served from a buffer that is already there (which is then never freed or moved again -- the
//    graph holds its address) or fails with hipErrorStreamCaptureUnsupported.
#include <map>
#include <mutex>
#include <thread>
#include <tuple>
#include <utility>
#include <vector>

#include "common.h"

// ---------------------------------------------------------------------------------------------
// the caller's workspace
// ---------------------------------------------------------------------------------------------
struct RepdlWorkspace::State
{
    char *base;
    size_t size, top, peak;
    bool dry, matrix_path;
    std::vector<size_t> marks; // offsets of the pieces handed out, in order
};

namespace
{
constexpr size_t PIECE_ALIGN = 256;
thread_local RepdlWorkspace::State *t_ws = nullptr;
// where the pieces of a dry run "lie": never dereferenced, 256-byte aligned like the real ones
char *const DRY_BASE = reinterpret_cast<char *>((uintptr_t)1 << 40);
inline size_t round_up(size_t v) { return (v + PIECE_ALIGN - 1) / PIECE_ALIGN * PIECE_ALIGN; }
} // namespace

RepdlWorkspace::RepdlWorkspace(void *base, size_t bytes, bool dry, bool matrix_path) : state_(new State()), previous_(t_ws)
{
    // the caller's buffer may start anywhere: the pieces start at its first 256-byte boundary
    const uintptr_t b = reinterpret_cast<uintptr_t>(base);
    const size_t skip = dry || base == nullptr ? 0 : (size_t)((PIECE_ALIGN - b % PIECE_ALIGN) % PIECE_ALIGN);
    state_->base = dry ? DRY_BASE : (base == nullptr ? nullptr : static_cast<char *>(base) + skip);
    state_->size = dry ? ~(size_t)0 >> 1 : (bytes > skip && base != nullptr ? bytes - skip : 0);
    state_->top = state_->peak = 0;
    state_->dry = dry;
    state_->matrix_path = matrix_path;
    t_ws = state_;
}

RepdlWorkspace::~RepdlWorkspace()
{
    t_ws = previous_;
    delete state_;
}

// (+ PIECE_ALIGN: what the constructor may skip at the start of a buffer that is not aligned)
size_t RepdlWorkspace::peak() const { return state_->peak == 0 ? 0 : state_->peak + PIECE_ALIGN; }

bool repdl_ws_dry() { return t_ws != nullptr && t_ws->dry; }
int repdl_ws_dry_matrix_path() { return repdl_ws_dry() ? (t_ws->matrix_path ? 1 : 0) : -1; }

// ---------------------------------------------------------------------------------------------
// the cache
// ---------------------------------------------------------------------------------------------
namespace
{
constexpr size_t CACHE_LIMIT = (size_t)4 << 30;
struct Slot
{
    void *ptr;
    size_t bytes;
    bool busy;
    bool pinned; // handed out during a stream capture: a graph holds its address
};
// hipStreamPerThread is one handle that names a different stream in every thread: the thread is part
// of its key (0 for every other stream, which two threads may well share)
typedef std::tuple<int, hipStream_t, size_t> Key;
std::mutex g_lock;
std::map<Key, std::vector<Slot>> g_slots;

Key key_of(int dev, hipStream_t s)
{
    const size_t thread = s == hipStreamPerThread ? std::hash<std::thread::id>()(std::this_thread::get_id()) | 1 : 0;
    return Key(dev, s, thread);
}

bool capturing(hipStream_t s)
{
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    const hipError_t e = hipStreamIsCapturing(s, &st);
    if (e != hipSuccess)
    {
        // (the legacy null stream while another stream captures in global mode: no allocation is allowed then either)
        (void)hipGetLastError();
        return true;
    }
    return st != hipStreamCaptureStatusNone;
}
} // namespace

hipError_t repdl_ws_acquire(void **p, size_t bytes, hipStream_t s)
{
    *p = nullptr;
    if (bytes == 0)
        return hipSuccess;
    if (t_ws != nullptr)
    {
        RepdlWorkspace::State &w = *t_ws;
        const size_t need = round_up(bytes);
        if (need > w.size - w.top)
            return static_cast<hipError_t>(REPDL_E_WORKSPACE);
        *p = w.base + w.top;
        w.marks.push_back(w.top);
        w.top += need;
        w.peak = w.top > w.peak ? w.top : w.peak;
        return hipSuccess;
    }
    if (bytes > CACHE_LIMIT)
        return hipMallocAsync(p, bytes, s);
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess)
        return e;
    const bool in_capture = capturing(s);
    std::lock_guard<std::mutex> guard(g_lock);
    std::vector<Slot> &v = g_slots[key_of(dev, s)];
    Slot *best = nullptr, *spare = nullptr; // the smallest free buffer that is large enough; else the largest free one that may go
    for (Slot &c : v)
    {
        if (c.busy)
            continue;
        if (c.bytes >= bytes && (best == nullptr || c.bytes < best->bytes))
            best = &c;
        if (!c.pinned && (spare == nullptr || c.bytes > spare->bytes))
            spare = &c;
    }
    if (best == nullptr)
    {
        if (in_capture)
            return hipErrorStreamCaptureUnsupported; // (run the entry point once before the capture, or use its _ws form)
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
            (void)hipGetLastError();
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
            v.push_back(Slot{q, want, false, false});
            best = &v.back();
        }
    }
    best->busy = true;
    best->pinned = best->pinned || in_capture;
    *p = best->ptr;
    return hipSuccess;
}

hipError_t repdl_ws_release(void *p, hipStream_t s)
{
    if (p == nullptr)
        return hipSuccess;
    if (t_ws != nullptr)
    {
        RepdlWorkspace::State &w = *t_ws;
        if (w.marks.empty() || w.base + w.marks.back() != static_cast<char *>(p))
            return static_cast<hipError_t>(REPDL_E_WORKSPACE); // (pieces go back in reverse order)
        w.top = w.marks.back();
        w.marks.pop_back();
        return hipSuccess;
    }
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess)
        return e;
    {
        std::lock_guard<std::mutex> guard(g_lock);
        auto it = g_slots.find(key_of(dev, s));
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

REPDL_API size_t repdl_hip_scratch_bytes(void)
{
    std::lock_guard<std::mutex> guard(g_lock);
    size_t total = 0;
    for (const auto &kv : g_slots)
        for (const Slot &c : kv.second)
            total += c.bytes;
    return total;
}

REPDL_API int repdl_hip_scratch_trim(void)
{
    std::lock_guard<std::mutex> guard(g_lock);
    hipError_t first = hipSuccess;
    for (auto it = g_slots.begin(); it != g_slots.end();)
    {
        std::vector<Slot> &v = it->second;
        for (size_t i = 0; i < v.size();)
        {
            if (v[i].busy || v[i].pinned)
            {
                i++;
                continue;
            }
            const hipError_t e = hipFree(v[i].ptr); // (waits for the device)
            if (e != hipSuccess && first == hipSuccess)
                first = e;
            v.erase(v.begin() + i);
        }
        it = v.empty() ? g_slots.erase(it) : std::next(it);
    }
    return first == hipSuccess ? REPDL_OK : (int)first;
}
