// Test infrastructure only.  Exposes two host-only, header-only functions of the reference with
// C linkage so the CPU checker can be validated against the real thing where the reference tree
// is mounted: onecycle_point (optim.h:18-44) and hash_u64 (utils.h:13-18).  The headers are
// included from the reference tree where they lie; nothing of theirs is copied here.
#include "optim.h"
#include "utils.h"
#include <cstdint>

extern "C" int tgref_onecycle_point(int total_steps, double warmup_fraction,
                                    double initial_lr_fraction, double final_lr_fraction,
                                    double low_momentum, double high_momentum, int step,
                                    float *multiplier, float *momentum) {
    try {
        OneCycle schedule{total_steps, warmup_fraction, initial_lr_fraction, final_lr_fraction,
                          low_momentum, high_momentum};
        StepRates rates = onecycle_point(schedule, step);
        *multiplier = rates.multiplier;
        *momentum = rates.momentum;
        return 0;
    } catch (...) {
        return -1;
    }
}
extern "C" uint64_t tgref_hash_u64(uint64_t x) {
    return hash_u64(x);
}
