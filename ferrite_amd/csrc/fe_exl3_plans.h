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
    {5120, 17408, 3, 256, 4, 2},  // occ 4 wk 2: 17.7 / 24.9; occ 3 wk 8: 18.2 / 23.8; occ 4 wk 8: 18.2 / 23.7
    {17408, 5120, 3, 256, 3, 2},  // occ 3 wk 2: 19.3 / 26.7; occ 3 wk 8: 19.6 / 27.2; occ 4 wk 8: 19.6 / 27.2
    {5120, 17408, 4, 256, 4, 2},  // occ 4 wk 2: 18.0 / 25.4; occ 5 wk 8: 18.5 / 24.2; occ 4 wk 8: 18.5 / 24.2
    {17408, 5120, 4, 256, 3, 2},  // occ 3 wk 2: 19.7 / 27.1; occ 4 wk 8: 20.0 / 27.9; occ 5 wk 8: 20.0 / 28.0
    {5120, 17408, 5, 256, 3, 8},  // occ 3 wk 8: 23.8 / 30.5; occ 2 wk 2: 24.0 / 29.9; occ 5 wk 8: 23.9 / 30.5
    {17408, 5120, 5, 256, 2, 2},  // occ 2 wk 2: 24.0 / 30.5; occ 5 wk 8: 24.7 / 34.0; occ 3 wk 8: 24.7 / 33.9
    {5120, 5120, 4, 256, 4, 4},   // occ 4 wk 4: 10.9 / 14.9; occ 5 wk 4: 10.9 / 15.0; occ 3 wk 4: 10.9 / 14.9
    {5120, 1024, 4, 256, 4, 4},   // occ 3 wk 4: 8.2 / 12.1; occ 4 wk 4: 8.2 / 12.2; occ 2 wk 4: 8.2 / 12.2
};
// clang-format on
