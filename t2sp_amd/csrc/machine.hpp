// machine.hpp — the two numbers of the device that the launch planners size their work by.
//
// A 256 x 256 output tile occupies a CU, so tiles run in rounds of `cus` workgroups, and workgroup
// ids are dealt round-robin to `xcds` dies, each with its own L2.  Both are asked of the device
// once (a full MI355X: 256 and 8; a partition of it or a part with fewer active CUs reports less)
// instead of being written into the planners.
#pragma once
#include <stddef.h>
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
// Workgroups of a four-wave LDS-tile kernel (three fit a CU) that should share a CU in a launch of `groups`
// of them, 0 for as many as fit.  The dispatcher fills every free slot of a CU at once, so when the
// groups per CU are not a multiple of the slots, some CUs take a whole extra set of the last groups and the
// others none (measured, 128 x 128 SGEMM tiles, 1024 = 4 per CU: 359 us as launched, 295 with two slots,
// 300 with one; 1280 = 5 per CU: 411 / 417 / 381; 768 = 3 per CU: 225 / 274 / 237).  The largest slot count
// that divides the groups per CU keeps the CUs level; beyond 8 per CU the uneven end no longer shows.
inline int resident_cap(int64_t groups) {
    const int cus = machine().cus;
    const int64_t per_cu = (groups + cus - 1) / cus;
    if (per_cu <= 3 || per_cu > 8 || per_cu % 3 == 0) return 0;
    return per_cu % 2 == 0 ? 2 : 1;
}
// Dynamic LDS to ask for so that at most `cap` workgroups share a CU's 160 KB (cap 0: just `need`).
inline size_t lds_request(size_t need, int cap) {
    if (cap <= 0) return need;
    const size_t want = (size_t)160 * 1024 / (size_t)(cap + 1) + 1024;
    return want > need ? want : need;
}
}  // namespace t2sp

// States the machine the planners plan for (cus <= 0: ask the device again on next use; xcds <= 0:
// derive it from cus).  For partitioned devices whose properties mislead, and for tests of the
// planners that run without a device.
extern "C" void t2sp_set_machine(int cus, int xcds);
