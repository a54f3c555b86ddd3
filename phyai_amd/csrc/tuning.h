// Tuning and test overrides of the kernel selection.
//
// The PHYAI_FP8_* variables (PHYAI_FP8_BIG, _BIG_DEPTH, _BIG_SPLITS, _BAND, _BY_ROWS, _SKINNY_MAXM,
// _SKINNY_PLAN, _SKINNY_STAGED, _TILE) force tile shapes, split counts and tile orders for
// experiments and for the tests that exercise every kernel variant.  They are looked at only when
// PHYAI_FP8_TUNING was set to a non-zero value when the library made its first call; that switch is
// read once.  Without it no launch reads the environment, and a stray variable cannot change which
// kernel a production process runs.
#pragma once
#include <stdlib.h>

namespace phyai {

inline bool tuning_enabled() {
    static const bool on = []() {
        const char* e = getenv("PHYAI_FP8_TUNING");
        return e != nullptr && atoi(e) != 0;
    }();
    return on;
}

// Value of a tuning variable, or null when tuning is off or the variable is unset.
inline const char* tuning_env(const char* name) { return tuning_enabled() ? getenv(name) : nullptr; }

}  // namespace phyai
