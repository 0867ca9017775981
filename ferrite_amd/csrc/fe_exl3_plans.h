// Tuned launch plans of the EXL3 decode GEMV: the measured choice of programs per CU (occ) and of the fewest
// 128-channel x 128-column units a program takes (min_units) per (k, n, bits, CU count). Written from the output of
// `python -m ferrite_amd.exl3 tune` on the GPU it is for (the table of crates/fe-exl3/src/plans.rs:8-131 plays this role
// in the reference, keyed by SM count). fe_exl3_plan_for consults it; FE_EXL3_UNTUNED=1 skips it.
#pragma once
#include <cstdint>

struct FeTunedPlan {
    uint32_t k, n, bits, cus, occ, min_units;
};

// clang-format off
static const FeTunedPlan kFeTunedPlans[] = {
    // MI355X, 256 CUs: us at 1 row / 16 rows of the best candidates (graph-replayed, weights cycled past the caches)
    {5120, 17408, 3, 256, 4, 2},  // occ 4 wk 2: 17.3 / 24.0; occ 3 wk 8: 18.0 / 23.2; occ 4 wk 8: 18.0 / 23.2
    {17408, 5120, 3, 256, 3, 8},  // occ 3..5 wk 8 (680 programs, 17 a column block): 18.9 / 26.3; occ 3 wk 2: 19.1 / 26.0
    {5120, 17408, 4, 256, 4, 2},  // occ 4 wk 2: 17.7 / 24.6; occ 4 wk 8: 18.3 / 23.6; occ 3 wk 8: 18.4 / 23.6
    {17408, 5120, 4, 256, 3, 8},  // occ 3..5 wk 8: 19.1 / 26.7; occ 3 wk 2: 19.5 / 26.7
    {5120, 17408, 5, 256, 3, 8},  // occ 3 wk 8: 20.1 / 25.8; occ 4 wk 8: 20.3 / 25.9; occ 4 wk 2: 20.1 / 27.4
    {17408, 5120, 5, 256, 3, 8},  // occ 3..5 wk 8: 21.1 / 29.0; occ 3 wk 2: 21.3 / 28.7
    {5120, 5120, 4, 256, 4, 4},   // occ 2..5 wk 4 (400 programs): 10.7 / 14.6
    {5120, 1024, 4, 256, 4, 4},   // occ 2..5 wk 4 (80 programs): 8.1 / 11.9
};
// clang-format on
