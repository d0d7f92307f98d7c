// runtime.hpp — host-side plumbing shared by the operator entry points:
// argument checks with the reference's error codes, staging of halide_buffer_t
// contents to and from device memory, and a small cache of device allocations.
//
// This replaces t2s/src/AOT-OpenCL-Runtime.cpp for this path:
//   halide_device_and_host_malloc  (:119-277)  -> DevicePool::get
//   halide_copy_to_device          (:434-437)  -> Staged (inputs)
//   halide_copy_to_host            (:439-441)  -> Staged::finish (outputs)
//   halide_opencl_wait_for_kernels_finish (:312-397) -> KernelTimer + stream sync
//   halide_error_* helpers         (:443-731)  -> check_buffer's messages and codes
// Unlike the reference it never calls exit() on a device error
// (AOT-OpenCL-Runtime.h:2429-2433): every failure is a negative return code.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include <mutex>
#include <vector>

#include "t2sp_buffer.h"

namespace t2sp {

// One lock for the whole library: the entry points are synchronous and share
// the stream, the pool and the timer, like the reference's file-scope globals
// (Halide/src/CodeGen_C.cpp:1718-1727), but callers on several threads are
// serialised instead of racing.
std::mutex &api_mutex();
hipStream_t api_stream();

int report(int code, const char *op, const char *what);

// Logical shape of a buffer: product of extents and the dense span it covers.
struct Span {
    int64_t elements;  // product of extents
    int64_t span;      // 1 + sum (extent-1)*stride  (strides are >= 0 on this path)
};

// Checks that `b` is a float32 buffer with `dims` dimensions (or one of two
// allowed counts), non-negative extents, zero mins honoured through host
// addressing, innermost stride 1.  Returns 0 or the Halide error code the
// generated checks of the reference return for the same misuse
// (Halide/src/AddImageChecks.cpp:352-636).
int check_buffer(const halide_buffer_t *b, const char *op, const char *name, int dims_a,
                 int dims_b, Span *span);
// The same for another element type (halide_type_code_t and bits), e.g. the uint8 characters of PairHMM.
int check_buffer_typed(const halide_buffer_t *b, const char *op, const char *name, int dims_a,
                       int dims_b, Span *span, int type_code, int type_bits);

class DevicePool {
public:
    // Returns a device allocation of at least `bytes`, reusing a cached one.
    void *get(size_t bytes);
    void put(void *p);
    void release_all();

private:
    struct Block {
        void *p;
        size_t bytes;
        bool busy;
    };
    std::vector<Block> blocks_;
};
DevicePool &pool();

// A buffer made available on the device for one call.
class Staged {
public:
    Staged() = default;
    ~Staged();
    // Input: use b->device when the caller staged it (copying the host data up
    // first when host_dirty is set), else copy the host span into pool memory.
    int input(const halide_buffer_t *b, const Span &s, const char *op, int element_bytes = 4);
    // Output: use b->device when present, else pool memory (pre-filled from the
    // host when the buffer is not dense, so that gaps keep their contents).
    // `partial`: the kernels write only part of the buffer; the rest must keep what it holds.
    int output(halide_buffer_t *b, const Span &s, const char *op, bool partial = false);
    // After the kernels: copy a pool-backed output down to the host, or mark a
    // caller-staged one device_dirty.
    int finish(const char *op);
    float *ptr() const { return ptr_; }

private:
    float *ptr_ = nullptr;
    bool pooled_ = false;
    halide_buffer_t *out_ = nullptr;
    int64_t span_ = 0;
};

// hipEvent bracket around the kernels of one entry-point call, on the library
// stream; the elapsed time of the last call is what t2sp_last_kernel_ns returns
// (the counterpart of the "latest end - earliest start" figure the reference
// writes to exec_time.txt, AOT-OpenCL-Runtime.cpp:358-396).
// Records `ns` as the kernel time of the call that just ended (what t2sp_last_kernel_ns returns
// and, when $T2SP_EXEC_TIME_FILE names a file, what is written there in the reference's format).
void publish_kernel_ns(double ns, const char *op);

// Streams and events for operator entries that move large host buffers through the device in
// panels: copies in, kernels (the library stream), copies out, chained by events so that the upload
// of the next panel and the download of the previous one overlap with the kernels of the current
// one (the reference copies everything in, runs, copies everything out:
// AOT-OpenCL-Runtime.cpp:402-441).  Default priority, created on first use, kept for the process.
constexpr int MAX_PANELS = 8;
struct PanelStreams {
    hipStream_t in = nullptr, out = nullptr;
    hipEvent_t up[MAX_PANELS], k0[MAX_PANELS], k1[MAX_PANELS];
    bool ok = false;
    PanelStreams();
};
PanelStreams &panel_streams();

class KernelTimer {
public:
    KernelTimer();
    int stop_and_sync(const char *op);
};

}  // namespace t2sp
