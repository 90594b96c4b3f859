// Optional per-launch timing of the library's own kernels.
//
// When switched on (fmoe_profile_enable), every kernel launch of a profiled class
// is bracketed by two HIP events recorded on the stream the kernel is launched
// on, and the amount of algorithmic work of that launch (flop or bytes) is noted.
// fmoe_profile_collect synchronises the device and returns, per class, the number
// of launches, their summed duration and summed work.  Off by default: the
// brackets cost two event records per launch.
#pragma once
#include "common.hpp"

namespace fmoe {

enum ProfileClass {
    kProfGemmFwd = 0,
    kProfGemmDgrad = 1,
    kProfGemmWgrad = 2,
    kProfBiasGrad = 3,
    kProfGatherRows = 4,
    kProfScatterRows = 5,
    kProfReduceSlots = 6,
    kProfIndexAdd = 7,
    kProfCombine = 8,
    kProfClasses = 9
};

bool profile_enabled();
// Records the opening event; returns a token (or -1 when profiling is off).
int profile_begin(int cls, double work, hipStream_t stream);
void profile_end(int token, hipStream_t stream);

struct ProfileScope {
    int token;
    hipStream_t stream;
    ProfileScope(int cls, double work, hipStream_t s) : token(-1), stream(s) {
        if (profile_enabled()) token = profile_begin(cls, work, s);
    }
    ~ProfileScope() {
        if (token >= 0) profile_end(token, stream);
    }
};

}  // namespace fmoe
