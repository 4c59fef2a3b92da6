// Launch-heuristic overrides for experiments (host side only).  Every knob defaults to 0 = "use
// the built-in heuristic"; mhc_tuning_set (exported, but not part of the public header) changes
// one for the whole process.  Not thread-safe and not meant for production callers: the public
// entry points behave identically with all knobs at 0.
#pragma once

namespace mhc {

enum TuneKey {
    kTuneOnepassOff = 0,    // one-launch forward: 0 = by cost model, 1 = never, 2 = whenever the shape allows
    kTuneOnepassG = 1,      // samples per workgroup of the one-launch forward
    kTuneGramFused = 2,     // n <= 8 channel sums and coefficient backward: 1 = two launches, 2 = one launch
    kTuneSlabSplits = 3,    // batch splits of the slab backward
    kTuneSeparateFinalize = 4,  // 1 = batch sums always as a launch of their own, never inside the dphi launch
    kTuneProjApart = 5,     // n <= 18 projection backward: 1 = both products in one launch, 2 = two launches
    kTuneStaticSpg = 6,     // static backward: samples per workgroup of the dx kernel (n <= 8)
    kTuneSpare3 = 7,
    kTuneCount = 8
};

extern int g_tuning[kTuneCount];
inline int tuning_get(int key) { return g_tuning[key]; }

}  // namespace mhc
