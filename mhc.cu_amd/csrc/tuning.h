// Launch-heuristic overrides for experiments and for tests that must reach a path the heuristics
// would not pick at the test's shape (host side only).  They exist only in a build with -DMHC_TUNING
// (libmhc_hip_tuning.so, `build.py --tuning`): there, mhc_tuning_set changes a knob for the whole
// process, unsynchronised.  In the product library tuning_get() is the constant 0 = "use the built-in
// heuristic", no knob and no setter exist, and the dispatch code reads no global state.
#pragma once

namespace mhc {

enum TuneKey {
    kTuneOnepassOff = 0,    // one-launch forward: 0 = by cost model, 1 = never, 2 = whenever the shape allows
    kTuneOnepassG = 1,      // samples per workgroup of the one-launch forward
    kTuneGramFused = 2,     // n <= 8 channel sums and coefficient backward: 1 = two launches, 2 = one launch
    kTuneSlabSplits = 3,    // batch splits of the slab backward (n <= 4) and of the projection backward (n = 5 .. 18)
    kTuneSeparateFinalize = 4,  // 1 = batch sums always as a launch of their own, never inside the dphi launch
    kTuneProjApart = 5,     // n <= 18 projection backward: 1 = both products in one launch, 2 = two launches
    kTuneStaticSpg = 6,     // static backward: samples per workgroup of the dx kernel (n <= 8)
    kTuneResident = 7,      // n <= 8 sample-resident backward: 0 = by heuristic, 1 = never, 2 = whenever the shape allows
    kTuneWideDxBeside = 8,  // wide projections (n > 18): dx workgroups beside the coefficient launch: 1 = never, 2 = always
    kTuneSpareB = 9,        // projection forward (matrix-core kernels): K splits, 0 = by heuristic
    kTuneCount = 10
};

#ifdef MHC_TUNING
extern int g_tuning[kTuneCount];
inline int tuning_get(int key) { return g_tuning[key]; }
#else
constexpr int tuning_get(int) { return 0; }
#endif

}  // namespace mhc
