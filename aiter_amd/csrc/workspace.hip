// Per-(device, stream) scratch arenas.  See workspace.h for the rules they implement.
#include "workspace.h"

#include <vector>

namespace fp8bs {

namespace {

std::mutex g_mutex; // held by WorkspaceLock: covers the table below and a call's launch sequence

struct Block
{
    void*  ptr   = nullptr;
    size_t bytes = 0;
};

// Blocks for eager work on one stream, or (capture = true, one per device) for work recorded into
// graphs on any stream of the device.
struct Arena
{
    int         device  = -1;
    hipStream_t stream  = nullptr;
    bool        capture = false;
    Block       block[(int)WsKind::kinds];
};

// a few streams per device in practice (torch hands out 32 per device at most); searched linearly
std::vector<Arena> g_arenas;
// blocks that a larger one has replaced; kept until the process ends (captured graphs may use them)
std::vector<Block> g_retired;

constexpr size_t kMaxArenas = 1024;
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
constexpr int  kMaxDevices = 64;
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

// The block of one kind in one arena, at least `bytes` large; allocates (never under capture: the
// callers see to that) when there is none or it is too small.  A fresh block that must start at
// zero is cleared with a fill kernel on `fill_stream`, or, when the work that will use it may run
// on another stream, with a synchronous hipMemset.
hipError_t block_for(const LaunchCtx& ctx, Arena& arena, int k, size_t bytes, bool zeroed, bool fill_in_stream)
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
    want         = (want + 255) & ~(size_t)255;
    void*      fresh = nullptr;
    hipError_t e     = hipMalloc(&fresh, want);
    if(e != hipSuccess)
    {
        say(ctx, "hipMalloc of a scratch buffer failed");
        return e;
    }
    if(zeroed)
    {
        if(fill_in_stream)
        {
            const size_t vecs   = want / 16;
            const size_t groups = (vecs + 255) / 256;
            hipLaunchKernelGGL(workspace_fill_zero_kernel, dim3((unsigned)(groups > 1024 ? 1024 : groups)), dim3(256),
                               0, ctx.stream, (uint4*)fresh, vecs);
            e = hipGetLastError();
        }
        else
            e = hipMemset(fresh, 0, want);
        if(e != hipSuccess)
        {
            (void)hipFree(fresh); // never handed out
            return e;
        }
    }
    if(b.ptr != nullptr)
        g_retired.push_back(b);
    b.ptr   = fresh;
    b.bytes = want;
    return hipSuccess;
}

// This device's copy of the static buffer.  First use on a device (which must be current): look
// the address up and clear the tickets with a fill kernel on the caller's stream.
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
        unsigned char* const tickets = (unsigned char*)ptr + kStaticPartialBytes;
        const size_t         vecs    = kStaticTickets * sizeof(uint32_t) / 16;
        hipLaunchKernelGGL(workspace_fill_zero_kernel, dim3((unsigned)((vecs + 255) / 256)), dim3(256), 0, ctx.stream,
                           (uint4*)tickets, vecs);
        if((e = hipGetLastError()) != hipSuccess)
            return e;
        g_static_base[ctx.device_id] = (unsigned char*)ptr;
    }
    *base = g_static_base[ctx.device_id];
    return hipSuccess;
}

Arena* find_arena(int device, hipStream_t stream, bool capture)
{
    for(Arena& a : g_arenas)
        if(a.device == device && a.capture == capture && (capture || a.stream == stream))
            return &a;
    return nullptr;
}

Arena* add_arena(const LaunchCtx& ctx, bool capture)
{
    if(g_arenas.size() >= kMaxArenas)
    {
        say(ctx, "too many (device, stream) pairs hold scratch buffers");
        return nullptr;
    }
    g_arenas.push_back(Arena{});
    Arena& a  = g_arenas.back();
    a.device  = ctx.device_id;
    a.stream  = capture ? nullptr : ctx.stream;
    a.capture = capture;
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
                             : "the kernel for this problem needs more than the 16384 split-K tickets that the static "
                               "scratch buffer holds: use the allocating entry point");
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
    hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
    hipError_t             e      = hipStreamIsCapturing(ctx.stream, &status);
    if(e != hipSuccess)
        return e;
    if(status != hipStreamCaptureStatusNone)
    {
        // Work recorded into a graph uses the device's capture arena, which only eager calls size.
        Arena* cap = find_arena(ctx.device_id, nullptr, true);
        if(cap == nullptr || cap->block[k].bytes < bytes)
        {
            say(ctx, "this call needs scratch memory that has not been allocated, and its stream is capturing: "
                     "nothing is allocated under capture -- run the same call once (on any stream of this device) "
                     "before the capture");
            return hipErrorStreamCaptureUnsupported;
        }
        *out = cap->block[k].ptr;
        return hipSuccess;
    }
    Arena* arena = find_arena(ctx.device_id, ctx.stream, false);
    if(arena == nullptr && (arena = add_arena(ctx, false)) == nullptr)
        return hipErrorOutOfMemory;
    if((e = block_for(ctx, *arena, k, bytes, zeroed, true)) != hipSuccess)
        return e;
    void* const mine = arena->block[k].ptr; // (add_arena below may move the table)
    // Keep the capture arena large enough for this call to be recorded later (the usual order: an
    // eager warm-up, then the capture on a stream of the framework's choosing).
    if(bytes <= kMaxCaptureBytes[k])
    {
        Arena* cap = find_arena(ctx.device_id, nullptr, true);
        if(cap == nullptr && (cap = add_arena(ctx, true)) == nullptr)
            return hipErrorOutOfMemory;
        if((e = block_for(ctx, *cap, k, bytes, zeroed, false)) != hipSuccess)
            return e;
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
