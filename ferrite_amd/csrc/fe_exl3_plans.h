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
    // MI355X, 256 CUs
    {5120, 17408, 4, 256, 4, 4},
};
// clang-format on
