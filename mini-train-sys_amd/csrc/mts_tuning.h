// Tuning switches of the library.  They exist for comparison runs (a tile shape or a block order against the
// default) and are read from the environment ONCE, when the library is loaded, into one immutable struct that
// every launcher reads: no launcher looks at the environment, and nothing is written after load, so calls from
// several host threads see the same values without synchronisation.
//
//   MTS_TILE_GATEUP / _DOWN / _DY1 / _DX / _DW1 / _DW2 = 0..4   tile family of that GEMM instead of the default
//   MTS_XCD_RANGES = 0 | 1        round-robin deal of the m-tiles | contiguous ranges per XCD, whatever the weights' size
//   MTS_NO_TILE_ORDER = 1         no n-tile groups, no reversed walks of an XCD's range
//   MTS_TILE_ORDER = mask         those one by one (bit 0 groups, 1 down reversed, 2 dY1 reversed, 3 dX reversed)
//   MTS_NO_TAIL_SPLIT = 1         every tile whole (the tiles behind an XCD's last whole round are not cut in two)
//   MTS_NO_MFMA_ROUTER = 1        router projection on the vector pipe for every shape
//   MTS_NO_JOINT_SCHEDULE = 1     units and dX tiles of the joint backward launch are dealt round-robin / in equal ranges
//   MTS_FWD_JOINT_TAIL = n        gate/up + down as one launch: the last n m-tiles of every XCD's down part are cut in two
//   MTS_FWD_JOINT_SPIN_US = n     ... and a down block gives up waiting for its rows after n microseconds (0: at once)
// A switch is on when its value parses to a non-zero integer ("0" and the empty string leave it off).
#pragma once

enum MtsGemmKind { MTS_K_GATEUP = 0, MTS_K_DOWN, MTS_K_DY1, MTS_K_DX, MTS_K_DW2, MTS_K_DW1, MTS_K_COUNT };

struct MtsTuning {
    int tile[MTS_K_COUNT];      // forced tile family per GEMM, -1: the launcher's own choice
    int xcd_ranges;             // -1: by the size of one expert's weights
    int tile_order_mask;        // ORDER_* bits
    bool tail_split;
    bool mfma_router;
    bool joint_schedule;
    int fwd_joint_tail;         // -1: the launcher's own choice
    long long fwd_joint_spin_us;
};

const MtsTuning& mts_tuning();
