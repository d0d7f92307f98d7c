/* t2sp_runtime.h — the few runtime calls a driver may use next to the operator
 * entry points.  They stand in for pieces of t2s/src/AOT-OpenCL-Runtime.cpp. */
#ifndef T2SP_RUNTIME_H
#define T2SP_RUNTIME_H
/* The C headers (and <iostream> in C++) that the reference's generated <op>-interface.h brings in
 * through AOT-OpenCL-Runtime.h (t2s/src/AOT-OpenCL-Runtime.h:22-31, included by the generated
 * header: Halide/src/CodeGen_C.cpp:327).  The reference's drivers rely on them: conv-run-fpga.cpp
 * and capsule-run-fpga.cpp call fabs() and include no <math.h> of their own. */
#include <assert.h>
#include <float.h>
#include <limits.h>
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>
#ifdef __cplusplus
#include <iostream>
extern "C" {
#endif

/* GPU time, in nanoseconds, of the kernels of the most recent operator call made by the
 * calling thread (hipEvent bracket on the library stream); for a thread that has made none, of
 * the most recent call in the process.  Callers on several threads are serialised by the
 * library and each reads its own call's time.  Counterpart of the
 * "latest end - earliest start" figure the reference writes to exec_time.txt
 * (t2s/src/AOT-OpenCL-Runtime.cpp:358-396) and reads back with ExecTime()
 * (t2s/src/Roofline.cpp:113-140), and of the value the oneAPI-flavour entry
 * returns (t2s/src/CodeGen_OneAPI_Dev.cpp:3554-3617). */
double t2sp_last_kernel_ns(void);

/* Frees the cached device allocations the entry points keep between calls
 * (counterpart of halide_device_and_host_free, AOT-OpenCL-Runtime.cpp:280-295). */
void t2sp_release(void);

/* Host memory for operator arguments: page-locked when a device is present, so that the copies
 * the entry points make run at the full rate of the link, and 64-byte aligned in every case.
 * Counterpart of halide_malloc / halide_free (t2s/src/AOT-OpenCL-Runtime.cpp:56-72).
 * t2sp_host_free takes NULL or a pointer t2sp_host_malloc returned. */
void *t2sp_host_malloc(size_t bytes);
void t2sp_host_free(void *p);

/* The machine the launch planners size rounds of workgroups and the die-aware tile order for:
 * compute units and dies (XCDs) of the current device, asked of it on first use (256 and 8 on a
 * full MI355X; a partition reports less).  t2sp_set_machine states them instead (cus <= 0: ask the
 * device again; xcds <= 0: derive from cus).  No counterpart in the reference, whose designs are
 * sized at synthesis time. */
int t2sp_machine_cus(void);
int t2sp_machine_xcds(void);
void t2sp_set_machine(int cus, int xcds);

/* Number of HIP devices visible; 0 when there is none. */
int t2sp_device_count(void);

#ifdef __cplusplus
}
#endif
#endif
