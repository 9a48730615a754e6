// Host-side planning shared by the runtime and the kernel launchers: how a world's selections are cut
// into units, what the count kernel needs of LDS, how many work items the cast-back kernel's list can
// hold.  Plain C++ (no device code), so that the runtime's bookkeeping can also be built and exercised on
// a machine without a GPU.
#include "ep_kernels.h"

namespace mcep {

size_t count_lds_bytes(const Dims& d) {
    // per wave of the unit and per expert: a 64-bit lane mask and a 16-bit prefix
    return (size_t)(d.plan.selections() / 64) * d.E * (8 + 2) + 64;
}

void plan_units(Dims& d, const Tuning& t) {
    const long long per_rank_sel = (long long)d.max_tokens * d.K;
    const long long big = (per_rank_sel + kBigUnitSelections - 1) / kBigUnitSelections;
    const size_t big_lds = (size_t)(kBigUnitSelections / 64) * d.E * (8 + 2) + 64;
    UnitPlan p;
    if (t.routing_sum != 0 && d.Tgrid > 0 && big * d.R <= kMaxSummedUnits && big_lds <= kMaxCountLdsBytes) {
        p.per_rank = (int)big;
        p.shift = 10;
        p.summed = 1;
        p.carried = t.routing_sum == 1 ? 1 : 0;
    } else {
        p.per_rank = (int)((per_rank_sel + kUnitSelections - 1) / kUnitSelections);
        p.shift = 8;
        p.summed = 0;
    }
    p.total = d.R * p.per_rank;
    d.plan = p;
}

long long cast_back_chunks(long long max_rows, int num_experts) {
    // every row is in one chunk, and each expert has at most one partly filled chunk
    return (max_rows + kCastRows - 1) / kCastRows + num_experts;
}

}  // namespace mcep
