// The library's tuning switches, read from the environment once at load time (see mts_tuning.h).
#include "mts_tuning.h"

#include <stdlib.h>

namespace {

bool flag(const char* name) {
    const char* s = getenv(name);
    return s && atoi(s) != 0;
}

MtsTuning read_environment() {
    static const char* const kTileEnv[MTS_K_COUNT] = {"MTS_TILE_GATEUP", "MTS_TILE_DOWN", "MTS_TILE_DY1",
                                                      "MTS_TILE_DX",     "MTS_TILE_DW2",  "MTS_TILE_DW1"};
    MtsTuning t;
    for (int k = 0; k < MTS_K_COUNT; ++k) {
        const char* s = getenv(kTileEnv[k]);
        const int c = s && *s ? atoi(s) : -1;
        t.tile[k] = (c >= 0 && c <= 4) ? c : -1;
    }
    const char* ranges = getenv("MTS_XCD_RANGES");
    t.xcd_ranges = ranges && *ranges ? (atoi(ranges) != 0) : -1;
    const char* pick = getenv("MTS_TILE_ORDER");
    t.tile_order_mask = flag("MTS_NO_TILE_ORDER") ? 0 : (pick && *pick ? atoi(pick) & 15 : 15);
    t.tail_split = !flag("MTS_NO_TAIL_SPLIT");
    t.mfma_router = !flag("MTS_NO_MFMA_ROUTER");
    t.joint_schedule = !flag("MTS_NO_JOINT_SCHEDULE");
    const char* tail = getenv("MTS_FWD_JOINT_TAIL");
    t.fwd_joint_tail = tail && *tail && atoi(tail) >= 0 ? atoi(tail) : -1;
    const char* spin = getenv("MTS_FWD_JOINT_SPIN_US");
    t.fwd_joint_spin_us = spin && *spin && atoll(spin) >= 0 ? atoll(spin) : 200000;
    return t;
}

// initialised by the dynamic loader before any entry point can be called; never written afterwards
const MtsTuning g_tuning = read_environment();

}  // namespace

const MtsTuning& mts_tuning() { return g_tuning; }
