// Per-(device, stream) scratch arenas.  See workspace.h for the rules they implement.
#include "workspace.h"

#include "capture_lanes.h"

#include <vector>

namespace fp8bs {

namespace {

std::mutex g_mutex; // held by WorkspaceLock: covers the table below and a call's launch sequence

struct Block
{
    void*  ptr   = nullptr;
    size_t bytes = 0;
};

// Blocks for eager work on one stream, or (capture = true: `lane` of the device's graph scratch) for
// work recorded into graphs.
struct Arena
{
    int         device   = -1;
    hipStream_t stream   = nullptr;
    bool        capture  = false;
    int         lane     = 0;
    uint64_t    last_use = 0; // eager arenas: g_use_clock at the latest request
    Block       block[(int)WsKind::kinds];
};

// a few streams per device in practice (torch hands out 32 per device at most); searched linearly
std::vector<Arena> g_arenas;
// blocks that a larger one has replaced; kept until the process ends (captured graphs may use them)
std::vector<Block> g_retired;

constexpr size_t kMaxArenas = 1024;
uint64_t         g_use_clock = 0;
// per device: which stream of which capture sequence records into which lane of the graph scratch
constexpr int    kMaxDevices = 64;
CaptureLaneTable g_lanes[kMaxDevices];
// per kind: smallest block worth allocating, and the largest request served
constexpr size_t kMinBytes[(int)WsKind::kinds] = {(size_t)1 << 20, (size_t)16 << 10, (size_t)64 << 10, (size_t)1 << 20};
constexpr size_t kMaxBytes[(int)WsKind::kinds] = {(size_t)2 << 30, (size_t)64 << 20, (size_t)1 << 30, (size_t)64 << 30};
// largest eager request for which the capture arena is kept in step (graphs record decode-sized
// calls; a prefill-sized expert layer would pin gigabytes twice)
constexpr size_t kMaxCaptureBytes[(int)WsKind::kinds] = {(size_t)256 << 20, (size_t)64 << 20, (size_t)64 << 20,
                                                         (size_t)1 << 30};

__global__ void __launch_bounds__(256) workspace_fill_zero_kernel(uint4* dst, size_t vecs)
{
    for(size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < vecs; i += (size_t)gridDim.x * blockDim.x)
        dst[i] = uint4{0u, 0u, 0u, 0u};
}

// The static buffer: [partial tiles | tickets].  In host code the array's name is only a handle
// for hipGetSymbolAddress; g_static_base holds each device's own address of it.
constexpr size_t kStaticBytes = kStaticPartialBytes + kStaticTickets * sizeof(uint32_t);
static __device__ __align__(256) unsigned char scratch[kStaticBytes];
unsigned char* g_static_base[kMaxDevices]; // guarded by g_mutex

void say(const LaunchCtx& ctx, const char* msg)
{
    if(ctx.why)
        *ctx.why = msg;
}

} // namespace

WorkspaceLock::WorkspaceLock(bool engage) : engaged_(engage)
{
    if(engaged_)
        g_mutex.lock();
}
WorkspaceLock::~WorkspaceLock()
{
    if(engaged_)
        g_mutex.unlock();
}

namespace {

// The block of one kind in one arena, at least `bytes` large; allocates (never on a capturing
// stream: the callers see to that) when there is none or it is too small.  A fresh block that must
// start at zero is cleared with a fill kernel on ctx.stream; with `wait`, for a block that work on
// other streams (graph replays) will use, the call also waits for that fill.
// Another host thread may be capturing a graph in the mode that forbids allocation to every thread
// (hipStreamCaptureModeGlobal, the default of most frameworks): the allocation is made with this
// thread's mode set to relaxed, which leaves that capture valid.  Should the runtime refuse the
// allocation all the same, the call fails with a message and the foreign capture is not touched
// any further.
hipError_t block_for(const LaunchCtx& ctx, Arena& arena, int k, size_t bytes, bool zeroed, bool wait)
{
    Block& b = arena.block[k];
    if(b.bytes >= bytes)
        return hipSuccess;
    // at least double, so that everything retired along the way stays below the live block's size
    size_t want = bytes + bytes / 4;
    if(want < 2 * b.bytes)
        want = 2 * b.bytes;
    if(want < kMinBytes[k])
        want = kMinBytes[k];
    want                      = (want + 255) & ~(size_t)255;
    void*                fresh = nullptr;
    hipStreamCaptureMode mode  = hipStreamCaptureModeRelaxed;
    const bool           swapped = hipThreadExchangeStreamCaptureMode(&mode) == hipSuccess;
    hipError_t           e       = hipMalloc(&fresh, want);
    if(swapped)
        (void)hipThreadExchangeStreamCaptureMode(&mode);
    if(e != hipSuccess)
    {
        (void)hipGetLastError();
        say(ctx, e == hipErrorStreamCaptureUnsupported || e == hipErrorStreamCaptureInvalidated
                     ? "a scratch buffer must grow, and the runtime refuses to allocate while another thread captures "
                       "a graph: run this call once before that capture begins"
                     : "hipMalloc of a scratch buffer failed");
        return e;
    }
    if(zeroed)
    {
        const size_t vecs   = want / 16;
        const size_t groups = (vecs + 255) / 256;
        hipLaunchKernelGGL(workspace_fill_zero_kernel, dim3((unsigned)(groups > 1024 ? 1024 : groups)), dim3(256), 0,
                           ctx.stream, (uint4*)fresh, vecs);
        e = hipGetLastError();
        if(e == hipSuccess && wait)
            e = hipStreamSynchronize(ctx.stream);
        if(e != hipSuccess)
        {
            // (the fill may be in flight: the block is leaked rather than freed under it)
            say(ctx, "clearing a fresh scratch buffer failed");
            return e;
        }
    }
    if(b.ptr != nullptr)
        g_retired.push_back(b);
    b.ptr   = fresh;
    b.bytes = want;
    return hipSuccess;
}

// This device's copy of the static buffer (the device must be current).  The array is zero when
// the code object is loaded and the kernels leave the tickets zero: nothing is cleared here.
hipError_t static_base(const LaunchCtx& ctx, unsigned char** base)
{
    if(ctx.device_id < 0 || ctx.device_id >= kMaxDevices)
    {
        say(ctx, "device ordinal outside 0..63");
        return hipErrorInvalidDevice;
    }
    if(g_static_base[ctx.device_id] == nullptr)
    {
        void*      ptr = nullptr;
        hipError_t e   = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if(e != hipSuccess || ptr == nullptr)
        {
            say(ctx, "hipGetSymbolAddress of the static scratch buffer failed");
            return e != hipSuccess ? e : hipErrorInvalidSymbol;
        }
        g_static_base[ctx.device_id] = (unsigned char*)ptr;
    }
    *base = g_static_base[ctx.device_id];
    return hipSuccess;
}

Arena* find_arena(int device, hipStream_t stream)
{
    for(Arena& a : g_arenas)
        if(!a.capture && a.device == device && a.stream == stream)
            return &a;
    return nullptr;
}

Arena* find_lane(int device, int lane)
{
    for(Arena& a : g_arenas)
        if(a.capture && a.device == device && a.lane == lane)
            return &a;
    return nullptr;
}

int eager_streams_of(int device)
{
    int n = 0;
    for(const Arena& a : g_arenas)
        n += (!a.capture && a.device == device) ? 1 : 0;
    return n;
}

// A new arena; when the table is full, the eager arena of this device that was used longest ago
// changes hands (its stream is most likely gone: a process that creates and destroys streams).  The
// device is brought to rest first, so that nothing still works in the blocks that change hands.
Arena* add_arena(const LaunchCtx& ctx, bool capture, int lane)
{
    if(g_arenas.size() >= kMaxArenas)
    {
        Arena* oldest = nullptr;
        for(Arena& a : g_arenas)
            if(!a.capture && a.device == ctx.device_id && (oldest == nullptr || a.last_use < oldest->last_use))
                oldest = &a;
        if(capture || oldest == nullptr)
        {
            say(ctx, "too many (device, stream) pairs hold scratch buffers");
            return nullptr;
        }
        hipStreamCaptureMode mode    = hipStreamCaptureModeRelaxed;
        const bool           swapped = hipThreadExchangeStreamCaptureMode(&mode) == hipSuccess;
        const hipError_t     e       = hipDeviceSynchronize();
        if(swapped)
            (void)hipThreadExchangeStreamCaptureMode(&mode);
        if(e != hipSuccess)
        {
            (void)hipGetLastError();
            say(ctx, "too many (device, stream) pairs hold scratch buffers, and the device could not be brought to rest "
                     "to hand the oldest ones on");
            return nullptr;
        }
        oldest->stream = ctx.stream;
        return oldest;
    }
    g_arenas.push_back(Arena{});
    Arena& a  = g_arenas.back();
    a.device  = ctx.device_id;
    a.stream  = capture ? nullptr : ctx.stream;
    a.capture = capture;
    a.lane    = lane;
    return &a;
}

} // namespace

hipError_t workspace_acquire(const LaunchCtx& ctx, const WorkspaceLock& held, WsKind kind, size_t bytes, bool zeroed,
                             void** out)
{
    const int k = (int)kind;
    *out        = nullptr;
    if(!held.engaged())
        return hipErrorInvalidValue;
    if(ctx.static_only)
    {
        const bool partial = kind == WsKind::split_partial, tickets = kind == WsKind::split_tickets;
        if(!partial && !tickets)
        {
            say(ctx, "this kind of scratch memory is not served from the static buffer");
            return hipErrorInvalidValue;
        }
        if(bytes > (partial ? kStaticPartialBytes : kStaticTickets * sizeof(uint32_t)))
        {
            say(ctx, partial ? "the kernel for this problem needs more than the 32 MiB of split-K partial tiles that "
                               "the static scratch buffer holds: use the allocating entry point, or ask for fewer K "
                               "ranges (kernelName / splitK)"
                             : "the kernel for this problem needs more than the 4 MiB of split-K counters and exchange "
                               "slots that the static scratch buffer holds: use the allocating entry point");
            return hipErrorInvalidValue;
        }
        unsigned char* base = nullptr;
        hipError_t     e    = static_base(ctx, &base);
        if(e != hipSuccess)
            return e;
        *out = partial ? base : base + kStaticPartialBytes;
        return hipSuccess;
    }
    if(bytes > kMaxBytes[k])
    {
        say(ctx, "the call needs more scratch memory than the library serves for this kind of buffer");
        return hipErrorInvalidValue;
    }
    if(ctx.device_id < 0 || ctx.device_id >= kMaxDevices)
    {
        say(ctx, "device ordinal outside 0..63");
        return hipErrorInvalidDevice;
    }
    hipStreamCaptureStatus status     = hipStreamCaptureStatusNone;
    unsigned long long     capture_id = 0;
    hipError_t             e          = hipStreamGetCaptureInfo(ctx.stream, &status, &capture_id);
    if(e != hipSuccess)
        return e;
    if(status != hipStreamCaptureStatusNone)
    {
        // Work recorded into a graph uses the device's graph scratch, which only eager calls size:
        // one lane per stream of the capture sequence that records scratch-using calls.
        int lanes_ready = 0;
        while(lanes_ready < kCaptureLanes)
        {
            const Arena* l = find_lane(ctx.device_id, lanes_ready);
            if(l == nullptr || l->block[k].bytes < bytes)
                break;
            ++lanes_ready;
        }
        if(lanes_ready == 0)
        {
            say(ctx, "this call needs scratch memory that has not been allocated, and its stream is capturing: "
                     "nothing is allocated under capture -- run the same call once (on any stream of this device) "
                     "before the capture");
            return hipErrorStreamCaptureUnsupported;
        }
        const int lane = g_lanes[ctx.device_id].lane_of((uint64_t)capture_id, (const void*)ctx.stream, lanes_ready);
        if(lane < 0)
        {
            say(ctx, "this capture records scratch-using calls on more streams than ran such calls before it (each "
                     "such stream of a capture needs scratch of its own, up to four, and nothing is allocated under "
                     "capture): run the calls once on as many streams as the capture forks, or record them on one");
            return hipErrorStreamCaptureUnsupported;
        }
        *out = find_lane(ctx.device_id, lane)->block[k].ptr;
        return hipSuccess;
    }
    Arena* arena = find_arena(ctx.device_id, ctx.stream);
    if(arena == nullptr && (arena = add_arena(ctx, false, 0)) == nullptr)
        return hipErrorOutOfMemory;
    arena->last_use = ++g_use_clock;
    if((e = block_for(ctx, *arena, k, bytes, zeroed, false)) != hipSuccess)
        return e;
    void* const mine = arena->block[k].ptr; // (add_arena below may move the table)
    // Keep the graph scratch large enough for this call to be recorded later (the usual order: an
    // eager warm-up, then the capture on a stream of the framework's choosing): as many lanes as
    // streams of this device have run scratch-using calls, so that a warm-up which forks side
    // streams as the capture will prepares a lane for each of them.
    if(bytes <= kMaxCaptureBytes[k])
    {
        int lanes = eager_streams_of(ctx.device_id);
        lanes     = lanes < 1 ? 1 : (lanes > kCaptureLanes ? kCaptureLanes : lanes);
        for(int lane = 0; lane < lanes; ++lane)
        {
            Arena* cap = find_lane(ctx.device_id, lane);
            if(cap == nullptr && (cap = add_arena(ctx, true, lane)) == nullptr)
                return hipErrorOutOfMemory;
            // every kind this device has used so far, so that a new lane is as large as lane 0
            for(int kk = 0; kk < (int)WsKind::kinds; ++kk)
            {
                const Arena* first = find_lane(ctx.device_id, 0);
                size_t       need  = kk == k ? bytes : 0;
                if(first != nullptr && first != cap && first->block[kk].bytes > need)
                    need = first->block[kk].bytes;
                if(need == 0)
                    continue;
                const bool clear = kk == (int)WsKind::split_tickets || (kk == k && zeroed);
                if((e = block_for(ctx, *cap, kk, need, clear, true)) != hipSuccess)
                    return e;
            }
        }
    }
    *out = mine;
    return hipSuccess;
}

hipError_t split_workspace(const LaunchCtx& ctx, const WorkspaceLock& held, size_t partial_bytes, size_t n_tickets,
                           float** partial, uint32_t** tickets)
{
    void*      p = nullptr;
    void*      t = nullptr;
    hipError_t e = workspace_acquire(ctx, held, WsKind::split_partial, partial_bytes, false, &p);
    if(e != hipSuccess)
        return e;
    if((e = workspace_acquire(ctx, held, WsKind::split_tickets, n_tickets * sizeof(uint32_t), true, &t)) != hipSuccess)
        return e;
    *partial = (float*)p;
    *tickets = (uint32_t*)t;
    return hipSuccess;
}

} // namespace fp8bs
