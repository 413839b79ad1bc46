// Scratch memory of the entry points whose kernels need more than their operands: split-K
// partial tiles and tickets of the GEMM kernels, the intermediates of the expert layer.
//
// Eager calls take it from arenas: one set of blocks per (device, stream), allocated on first use
// and grown on demand.  Work on different streams never shares a block, so calls on different
// streams cannot touch each other's partial results.  A block that has been handed out is never
// freed: HIP graphs captured earlier may hold its address.
// A call whose stream is capturing allocates, clears and synchronises nothing.  It takes its
// scratch from the device's graph scratch, which every eager call keeps at least as large as its
// own request (up to a cap per kind of buffer): after one eager run of a call, on any stream, the
// same call can be recorded on any stream; otherwise it fails with a message.  The graph scratch
// has up to four lanes, as many as streams of the device have run scratch-using calls eagerly:
// inside one capture sequence every stream that records such a call keeps a lane to itself
// (capture_lanes.h), so calls recorded on forked streams, which may run side by side on replay,
// never share partial results; a capture that forks wider than the warm-up did is refused with a
// message.  Graphs of one device share the lanes with each other (not with eager work): replay
// them one at a time.
// An eager call that must allocate while ANOTHER host thread is capturing does so with its
// thread's capture mode set to relaxed, which leaves that capture valid; if the runtime refuses
// all the same, the call fails with a message.
//
// Callers that cannot allocate at all have the static buffer instead: a fixed array in device
// memory, one copy per GPU, shared by every call on that GPU that asks for it (LaunchCtx::
// static_only).  It serves the split-K buffers up to kStaticPartialBytes / kStaticTickets; a
// larger request fails.  Calls that use it and overlap on one GPU race.
//
// A WorkspaceLock must be held from the first request of a call to its last launch: it keeps two
// host threads that use one stream from interleaving the launches of their calls.
#pragma once

#include <hip/hip_runtime.h>
#include <mutex>
#include <stddef.h>
#include <stdint.h>

namespace fp8bs {

enum class WsKind : int
{
    split_partial = 0, // fp32 partial tiles of K split across workgroups
    split_tickets,     // arrival counters and exchange slots: all zero between launches (their users put the zeros back)
    moe_sort,          // histograms and expert offsets of the sorting kernels
    moe_layer,         // intermediates of the expert layer
    kinds
};

// what the static buffer holds: partial tiles, then tickets
constexpr size_t kStaticPartialBytes = (size_t)32 << 20;
constexpr size_t kStaticTickets      = (size_t)1 << 20; // 32-bit words: 4 MiB

// What a launcher needs to know about the call it serves besides the operands.
struct LaunchCtx
{
    int          device_id     = 0;
    hipStream_t  stream        = nullptr;
    bool         static_only   = false;   // scratch from the static buffer only: nothing is allocated
    const char** why           = nullptr; // receives a static message when a request fails
};

class WorkspaceLock
{
  public:
    explicit WorkspaceLock(bool engage = true); // engage = false: a call that needs no scratch
    ~WorkspaceLock();
    WorkspaceLock(const WorkspaceLock&)            = delete;
    WorkspaceLock& operator=(const WorkspaceLock&) = delete;
    bool engaged() const { return engaged_; }

  private:
    bool engaged_;
};

// `bytes` of scratch of one kind for work on ctx.stream, 256-byte aligned.  With `zeroed`, a
// freshly allocated block is cleared by a fill kernel on that stream before it is handed out
// (the kernels that use tickets leave them zero).  The caller holds a WorkspaceLock.
hipError_t workspace_acquire(const LaunchCtx& ctx, const WorkspaceLock& held, WsKind kind, size_t bytes, bool zeroed,
                             void** out);

// Both split-K buffers at once.
hipError_t split_workspace(const LaunchCtx& ctx, const WorkspaceLock& held, size_t partial_bytes, size_t n_tickets,
                           float** partial, uint32_t** tickets);

} // namespace fp8bs
