// TEST INFRASTRUCTURE: a kernel with the mistake that the emulation must refuse -- a lane exchange on the right of
// `&&`, which only the lanes with a true left side reach.  argv[1] = "bad" runs it, "good" runs the same kernel with
// the exchange made by every lane.  tests/test_emu_engine.py::test_emulation_refuses_exchange_in_divergent_branch
#include "hip_emu.h"
#include "f3m_rt.h"
#include <cstdio>
#include <cstring>
#include <vector>

using namespace f3m;

static void kernel(bool bad, int *out)
{
    const int lane = (int)lane_id();
    const bool odd = lane & 1;
    bool same;
    if (bad) {
        same = odd && wave_shfl_i(lane, (lane + 63) & 63) + 1 == lane;
    } else {
        const int prev = wave_shfl_i(lane, (lane + 63) & 63);
        same = odd && prev + 1 == lane;
    }
    const unsigned long long m = wave_ballot(same);
    if (lane == 0) out[0] = (int)__builtin_popcountll(m);
}

int main(int argc, char **argv)
{
    const bool bad = argc > 1 && !strcmp(argv[1], "bad");
    int out = -1;
    emu::launch(1, 64, 0, [&] { kernel(bad, &out); });
    printf("%d\n", out);
    return out == 32 ? 0 : 1;
}
