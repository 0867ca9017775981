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
    // MI355X, 256 CUs: us at 1 row / 16 rows of the best candidates (graph-replayed after 40 ms of the same replays, weights
    // cycled past the caches)
    {5120, 17408, 3, 256, 4, 2},  // occ 4 wk 2: 17.6 / 24.2; occ 3..5 wk 8: 18.2 / 23.5
    {17408, 5120, 3, 256, 3, 8},  // occ 3..5 wk 8 (680 programs, 17 a column block): 19.1 / 26.4; occ 3 wk 2: 19.4 / 26.3
    // (gate + up in one launch: occ 4 wk 2 30.7 us at 1 row, 33.5 at 4, 36.0 at 8, 42.3 at 16; occ 3..5 wk 8 32.5 / 35.5 /
    // 35.8 / 39.9: the plan is the one of few rows, and one plan for all row counts keeps a row's bits)
    {5120, 17408, 4, 256, 4, 2},  // occ 4 wk 2: 18.5 / 24.9; occ 3..5 wk 8: 18.5 / 23.9
    {17408, 5120, 4, 256, 3, 8},  // occ 3 wk 8: 19.3 / 26.8; occ 4, 5 wk 8: 19.6 / 26.8; occ 3 wk 2: 19.8 / 26.7
    {5120, 17408, 5, 256, 3, 8},  // occ 3 wk 8: 20.5 / 26.3; occ 5 wk 8: 20.6 / 26.3; occ 4 wk 2: 20.9 / 27.7
    {17408, 5120, 5, 256, 2, 2},  // occ 2 wk 2: 21.1 / 27.6; occ 3..5 wk 8: 21.4 / 29.4
    {5120, 5120, 4, 256, 4, 4},   // occ 2..5 wk 4 (400 programs): 10.8 / 14.8
    {5120, 1024, 4, 256, 4, 4},   // occ 2..5 wk 4 (80 programs): 8.2 / 12.1
};
// clang-format on
