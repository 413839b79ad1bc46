// Which part of a device's graph scratch a call gets while its stream is capturing.  Plain C++
// (no HIP), so that the bookkeeping can be compiled and tested on the host.
//
// The graph scratch of a device is cut into lanes of equal standing.  Inside one capture sequence
// (one capture id: the stream that began the capture and every stream forked from it) each stream
// that records a scratch-using call keeps one lane to itself: calls recorded on one stream are
// ordered by that stream and may share their lane, calls recorded on two forked streams may run at
// the same time when the graph is replayed and never share one.  Different capture sequences start
// again at lane 0 (graphs of one device are replayed one at a time).
#pragma once

#include <stdint.h>

namespace fp8bs {

constexpr int kCaptureLanes = 4;

class CaptureLaneTable
{
  public:
    // Lane (0 .. lanes_ready - 1) of `stream` inside capture sequence `capture_id`; -1 when the
    // sequence already uses `lanes_ready` other streams (lanes_ready <= kCaptureLanes).
    int lane_of(uint64_t capture_id, const void* stream, int lanes_ready)
    {
        Sequence* seq = nullptr;
        for(Sequence& s : seq_)
            if(s.used && s.id == capture_id)
                seq = &s;
        if(seq == nullptr)
        {
            // a new capture sequence takes the slot that was touched longest ago
            seq = &seq_[0];
            for(Sequence& s : seq_)
                if(!s.used || s.touched < seq->touched)
                {
                    seq = &s;
                    if(!s.used)
                        break;
                }
            seq->used    = true;
            seq->id      = capture_id;
            seq->streams = 0;
        }
        seq->touched = ++clock_;
        for(int i = 0; i < seq->streams; ++i)
            if(seq->stream[i] == stream)
                return i < lanes_ready ? i : -1;
        if(seq->streams >= lanes_ready || seq->streams >= kCaptureLanes)
            return -1;
        seq->stream[seq->streams] = stream;
        return seq->streams++;
    }

  private:
    struct Sequence
    {
        bool        used    = false;
        uint64_t    id      = 0;
        uint64_t    touched = 0;
        int         streams = 0;
        const void* stream[kCaptureLanes] = {};
    };
    // capture sequences that are being recorded side by side (by different host threads); a sequence
    // that falls out of the table and comes back starts again at lane 0
    Sequence seq_[8];
    uint64_t clock_ = 0;
};

} // namespace fp8bs
