// machine.hpp — the two numbers of the device that the launch planners size their work by.
//
// A 256 x 256 output tile occupies a CU, so tiles run in rounds of `cus` workgroups, and workgroup
// ids are dealt round-robin to `xcds` dies, each with its own L2.  Both are asked of the device
// once (a full MI355X: 256 and 8; a partition of it or a part with fewer active CUs reports less)
// instead of being written into the planners.
#pragma once
#include <stdint.h>

namespace t2sp {
struct Machine {
    int cus;    // compute units of the device the library runs on
    int xcds;   // dies the workgroup ids are dealt to
};
// The current device's values (queried on first use; 256 / 8 when no device is present), or what
// t2sp_set_machine() stated.
Machine machine();
// Dies of a device with `cus` compute units: the largest of 8, 4, 2, 1 that leaves 20 to 40 CUs per
// die (MI355X: 32 per die, MI300X: 38), else 1.
int xcds_for(int cus);
// A stride or leading dimension the entry points accept (see T2SP_MAX_STRIDE in t2sp_hip.h): with
// extents of at most 2^30, every extent x stride product and every sum of a few of them stays
// inside 64 bits.
inline bool stride_in_range(int64_t s) { return s >= -((int64_t)1 << 31) && s <= ((int64_t)1 << 31); }
template <class... S>
inline bool strides_in_range(S... s) { return (stride_in_range((int64_t)s) && ...); }
}  // namespace t2sp

// States the machine the planners plan for (cus <= 0: ask the device again on next use; xcds <= 0:
// derive it from cus).  For partitioned devices whose properties mislead, and for tests of the
// planners that run without a device.
extern "C" void t2sp_set_machine(int cus, int xcds);
