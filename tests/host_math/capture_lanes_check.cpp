// Host check of the bookkeeping that hands out lanes of the graph scratch to the streams of a
// capture sequence (aiter_amd/csrc/capture_lanes.h).  Prints OK or the first failed expectation.
#include "../../aiter_amd/csrc/capture_lanes.h"

#include <cstdio>
#include <cstdlib>

#define EXPECT(cond)                                             \
    do                                                           \
    {                                                            \
        if(!(cond))                                              \
        {                                                        \
            std::printf("FAILED line %d: %s\n", __LINE__, #cond); \
            return 1;                                            \
        }                                                        \
    } while(0)

int main()
{
    using fp8bs::CaptureLaneTable;
    int         s[8];
    const void *A = &s[0], *B = &s[1], *C = &s[2], *D = &s[3], *E = &s[4];
    {
        CaptureLaneTable t;
        // two streams of one capture get two lanes; each keeps its own on later calls
        EXPECT(t.lane_of(7, A, 2) == 0);
        EXPECT(t.lane_of(7, B, 2) == 1);
        EXPECT(t.lane_of(7, A, 2) == 0);
        EXPECT(t.lane_of(7, B, 2) == 1);
        // a third stream finds no lane while only two are ready, and gets one when a third is
        EXPECT(t.lane_of(7, C, 2) == -1);
        EXPECT(t.lane_of(7, C, 3) == 2);
        EXPECT(t.lane_of(7, D, 4) == 3);
        EXPECT(t.lane_of(7, E, 4) == -1); // never more than kCaptureLanes
        // a stream whose lane lies beyond what is ready for this request is refused, not moved
        EXPECT(t.lane_of(7, D, 2) == -1);
        EXPECT(t.lane_of(7, D, 4) == 3);
    }
    {
        CaptureLaneTable t;
        // another capture sequence starts again at lane 0, whatever its stream was before
        EXPECT(t.lane_of(1, A, 2) == 0);
        EXPECT(t.lane_of(1, B, 2) == 1);
        EXPECT(t.lane_of(2, B, 2) == 0);
        EXPECT(t.lane_of(2, A, 2) == 1);
        // two sequences recorded side by side keep their own assignments
        EXPECT(t.lane_of(1, B, 2) == 1);
        EXPECT(t.lane_of(2, B, 2) == 0);
        EXPECT(t.lane_of(1, A, 1) == 0);
        EXPECT(t.lane_of(1, B, 1) == -1); // only one lane is large enough for this request
    }
    {
        CaptureLaneTable t;
        // more sequences than the table remembers: the one touched longest ago is forgotten,
        // the others keep their lanes
        for(unsigned long long id = 100; id < 108; ++id)
        {
            EXPECT(t.lane_of(id, A, 2) == 0);
            EXPECT(t.lane_of(id, B, 2) == 1);
        }
        EXPECT(t.lane_of(107, B, 2) == 1);
        EXPECT(t.lane_of(200, C, 2) == 0); // evicts sequence 100
        EXPECT(t.lane_of(101, B, 2) == 1);
        EXPECT(t.lane_of(107, A, 2) == 0);
        EXPECT(t.lane_of(100, B, 2) == 0); // forgotten: starts again (and evicts the oldest)
    }
    std::printf("OK\n");
    return 0;
}
