// runtime.cpp — see runtime.hpp.
#include "runtime.hpp"
#include "machine.hpp"

#include <atomic>
#include <stdlib.h>

namespace t2sp {

std::mutex &api_mutex() {
    static std::mutex m;
    return m;
}

// The entry points run on the default stream: it orders against work the caller
// queued on it (for example a framework that filled a pre-staged device buffer).
hipStream_t api_stream() { return nullptr; }

// Kernel time of the last call: per calling thread (an entry point runs in its caller's thread and
// publishes while it holds the library lock, so a second thread's call cannot overwrite what the
// first is about to read), with the process-wide latest as the answer for a thread that has made
// no call itself.
static std::atomic<double> g_last_kernel_ns{0.0};
static thread_local double tl_last_kernel_ns = -1.0;
static hipEvent_t g_ev0 = nullptr, g_ev1 = nullptr;

int report(int code, const char *op, const char *what) {
    if (code != 0) fprintf(stderr, "t2sp: %s: %s (error %d)\n", op, what, code);
    return code;
}

int check_buffer(const halide_buffer_t *b, const char *op, const char *name, int dims_a,
                 int dims_b, Span *span) {
    return check_buffer_typed(b, op, name, dims_a, dims_b, span, halide_type_float, 32);
}

int check_buffer_typed(const halide_buffer_t *b, const char *op, const char *name, int dims_a,
                       int dims_b, Span *span, int type_code, int type_bits) {
    char msg[160];
    if (!b) {
        snprintf(msg, sizeof msg, "buffer argument %s is NULL", name);
        return report(halide_error_code_buffer_argument_is_null, op, msg);
    }
    if (b->type.code != type_code || b->type.bits != type_bits || b->type.lanes != 1) {
        snprintf(msg, sizeof msg, "%s has type code %d bits %d lanes %d, expected code %d bits %d", name,
                 (int)b->type.code, (int)b->type.bits, (int)b->type.lanes, type_code, type_bits);
        return report(halide_error_code_bad_type, op, msg);
    }
    if (b->dimensions != dims_a && b->dimensions != dims_b) {
        snprintf(msg, sizeof msg, "%s has %d dimensions, expected %d%s", name, b->dimensions, dims_a,
                 dims_b != dims_a ? " (or the tiled form)" : "");
        return report(halide_error_code_bad_dimensions, op, msg);
    }
    if (!b->dim) {
        snprintf(msg, sizeof msg, "%s has no dimension array", name);
        return report(halide_error_code_buffer_is_null, op, msg);
    }
    int64_t elements = 1, spn = 1;
    for (int d = 0; d < b->dimensions; d++) {
        if (b->dim[d].extent < 0) {
            snprintf(msg, sizeof msg, "%s dimension %d has negative extent %d", name, d,
                     b->dim[d].extent);
            return report(halide_error_code_buffer_extents_negative, op, msg);
        }
        if (b->dim[d].stride < 0) {
            snprintf(msg, sizeof msg, "%s dimension %d has negative stride", name, d);
            return report(halide_error_code_constraint_violated, op, msg);
        }
        // (a buffer of more than 2^40 elements, or one that spans more, is refused before the products
        // below could leave 64 bits: Halide's own limit is 2^31 - 1 bytes, halide_error_code_buffer_extents_too_large)
        constexpr int64_t LIMIT = (int64_t)1 << 40;
        const int64_t reach = (int64_t)(b->dim[d].extent > 0 ? b->dim[d].extent - 1 : 0) * b->dim[d].stride;
        if ((b->dim[d].extent > 0 && elements > LIMIT / b->dim[d].extent) || reach > LIMIT || spn + reach > LIMIT) {
            snprintf(msg, sizeof msg, "%s is larger than 2^40 elements at dimension %d", name, d);
            return report(halide_error_code_buffer_extents_too_large, op, msg);
        }
        elements *= b->dim[d].extent;
        spn += reach;
    }
    if (b->dimensions > 0 && b->dim[0].stride != 1) {
        snprintf(msg, sizeof msg, "%s.stride.0 is %d, must be 1", name, b->dim[0].stride);
        return report(halide_error_code_constraint_violated, op, msg);
    }
    if (!b->host && !b->device) {
        snprintf(msg, sizeof msg, "%s has neither host nor device memory", name);
        return report(halide_error_code_host_is_null, op, msg);
    }
    if ((b->flags & halide_buffer_flag_host_dirty) && (b->flags & halide_buffer_flag_device_dirty)) {
        snprintf(msg, sizeof msg, "%s is dirty on both host and device", name);
        return report(halide_error_code_host_and_device_dirty, op, msg);
    }
    if (span) {
        span->elements = elements;
        span->span = elements == 0 ? 0 : spn;
    }
    return 0;
}

void *DevicePool::get(size_t bytes) {
    if (bytes == 0) bytes = 16;
    Block *best = nullptr;
    for (auto &b : blocks_)
        if (!b.busy && b.bytes >= bytes && (!best || b.bytes < best->bytes)) best = &b;
    if (best && best->bytes <= 2 * bytes + (1u << 20)) {
        best->busy = true;
        return best->p;
    }
    void *p = nullptr;
    if (hipMalloc(&p, bytes) != hipSuccess) {
        // drop idle blocks and retry once
        for (size_t i = 0; i < blocks_.size();) {
            if (!blocks_[i].busy) {
                (void)hipFree(blocks_[i].p);
                blocks_.erase(blocks_.begin() + i);
            } else {
                i++;
            }
        }
        (void)hipGetLastError();
        if (hipMalloc(&p, bytes) != hipSuccess) {
            (void)hipGetLastError();
            return nullptr;
        }
    }
    blocks_.push_back({p, bytes, true});
    return p;
}

void DevicePool::put(void *p) {
    for (auto &b : blocks_)
        if (b.p == p) b.busy = false;
}

void DevicePool::release_all() {
    for (auto &b : blocks_) (void)hipFree(b.p);
    blocks_.clear();
}

DevicePool &pool() {
    static DevicePool p;
    return p;
}

Staged::~Staged() {
    if (pooled_ && ptr_) pool().put(ptr_);
}

int Staged::input(const halide_buffer_t *b, const Span &s, const char *op, int element_bytes) {
    span_ = s.span;
    const size_t bytes = (size_t)s.span * element_bytes;
    if (b->device) {
        ptr_ = reinterpret_cast<float *>(b->device);
        if ((b->flags & halide_buffer_flag_host_dirty) && b->host && bytes)
            if (hipMemcpyAsync(ptr_, b->host, bytes, hipMemcpyHostToDevice, api_stream()) != hipSuccess)
                return report(halide_error_code_copy_to_device_failed, op, "host to device copy failed");
        return 0;
    }
    ptr_ = static_cast<float *>(pool().get(bytes));
    if (!ptr_) return report(halide_error_code_device_malloc_failed, op, "device allocation failed");
    pooled_ = true;
    if (bytes && hipMemcpyAsync(ptr_, b->host, bytes, hipMemcpyHostToDevice, api_stream()) != hipSuccess)
        return report(halide_error_code_copy_to_device_failed, op, "host to device copy failed");
    return 0;
}

int Staged::output(halide_buffer_t *b, const Span &s, const char *op, bool partial) {
    span_ = s.span;
    out_ = b;
    const size_t bytes = (size_t)s.span * sizeof(float);
    if (b->device) {
        ptr_ = reinterpret_cast<float *>(b->device);
        return 0;
    }
    ptr_ = static_cast<float *>(pool().get(bytes));
    if (!ptr_) return report(halide_error_code_device_malloc_failed, op, "device allocation failed");
    pooled_ = true;
    if ((partial || s.span != s.elements) && bytes)
        if (hipMemcpyAsync(ptr_, b->host, bytes, hipMemcpyHostToDevice, api_stream()) != hipSuccess)
            return report(halide_error_code_copy_to_device_failed, op, "host to device copy failed");
    return 0;
}

int Staged::finish(const char *op) {
    if (!out_) return 0;
    if (!pooled_) {
        out_->flags |= halide_buffer_flag_device_dirty;
        out_->flags &= ~(uint64_t)halide_buffer_flag_host_dirty;
        return 0;
    }
    const size_t bytes = (size_t)span_ * sizeof(float);
    if (bytes && hipMemcpy(out_->host, ptr_, bytes, hipMemcpyDeviceToHost) != hipSuccess)
        return report(halide_error_code_copy_to_host_failed, op, "device to host copy failed");
    out_->flags &= ~(uint64_t)(halide_buffer_flag_device_dirty | halide_buffer_flag_host_dirty);
    return 0;
}

PanelStreams::PanelStreams() {
    ok = hipStreamCreateWithFlags(&in, hipStreamNonBlocking) == hipSuccess &&
         hipStreamCreateWithFlags(&out, hipStreamNonBlocking) == hipSuccess;
    for (int i = 0; i < MAX_PANELS && ok; i++)
        ok = hipEventCreate(&up[i]) == hipSuccess && hipEventCreate(&k0[i]) == hipSuccess &&
             hipEventCreate(&k1[i]) == hipSuccess;
    if (!ok) (void)hipGetLastError();
}

PanelStreams &panel_streams() {
    static PanelStreams s;
    return s;
}

KernelTimer::KernelTimer() {
    if (!g_ev0) {
        (void)hipEventCreate(&g_ev0);
        (void)hipEventCreate(&g_ev1);
    }
    (void)hipEventRecord(g_ev0, api_stream());
}

int KernelTimer::stop_and_sync(const char *op) {
    (void)hipEventRecord(g_ev1, api_stream());
    if (hipStreamSynchronize(api_stream()) != hipSuccess) {
        (void)hipGetLastError();
        return report(halide_error_code_device_run_failed, op, "kernel execution failed");
    }
    float ms = 0.f;
    if (hipEventElapsedTime(&ms, g_ev0, g_ev1) == hipSuccess) publish_kernel_ns((double)ms * 1e6, op);
    return 0;
}

void publish_kernel_ns(double ns, const char *op) {
    g_last_kernel_ns = ns;
    tl_last_kernel_ns = ns;
    // Optional file in the reference's exec_time.txt format (AOT-OpenCL-Runtime.cpp:380-394):
    // overall ns on the first line, then "<kernel_name> <ns>" lines.  The reference's drivers ask
    // for "kernel_unloader", the last kernel of its pipeline, so that name is written too.
    if (const char *file = getenv("T2SP_EXEC_TIME_FILE")) {
        if (*file) {
            if (FILE *fp = fopen(file, "w")) {
                fprintf(fp, "%f\nkernel_%s %lf\nkernel_unloader %lf\n", ns, op, ns, ns);
                fclose(fp);
            }
        }
    }
}

}  // namespace t2sp

namespace t2sp {
static std::atomic<int> g_machine_cus{0}, g_machine_xcds{0};

int xcds_for(int cus) {
    for (int x = 8; x > 1; x /= 2)
        if (cus % x == 0 && cus / x >= 20 && cus / x <= 40) return x;
    return 1;
}

Machine machine() {
    int cus = g_machine_cus.load(), xcds = g_machine_xcds.load();
    if (cus <= 0) {
        int dev = 0;
        hipDeviceProp_t prop;
        if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess && prop.multiProcessorCount > 0) {
            cus = prop.multiProcessorCount;
        } else {
            (void)hipGetLastError();
            cus = 256;                     // no device: plan for a full MI355X
        }
        xcds = xcds_for(cus);
        g_machine_cus = cus;
        g_machine_xcds = xcds;
    }
    return Machine{cus, xcds > 0 ? xcds : xcds_for(cus)};
}
}  // namespace t2sp

extern "C" void t2sp_set_machine(int cus, int xcds) {
    t2sp::g_machine_cus = cus > 0 ? cus : 0;
    t2sp::g_machine_xcds = cus > 0 ? (xcds > 0 ? xcds : t2sp::xcds_for(cus)) : 0;
}

extern "C" int t2sp_machine_cus(void) { return t2sp::machine().cus; }
extern "C" int t2sp_machine_xcds(void) { return t2sp::machine().xcds; }

extern "C" double t2sp_last_kernel_ns(void) {
    return t2sp::tl_last_kernel_ns >= 0.0 ? t2sp::tl_last_kernel_ns : t2sp::g_last_kernel_ns.load();
}

extern "C" void t2sp_release(void) {
    std::lock_guard<std::mutex> lock(t2sp::api_mutex());
    (void)hipDeviceSynchronize();
    t2sp::pool().release_all();
}

extern "C" int t2sp_device_count(void) {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) {
        (void)hipGetLastError();
        return 0;
    }
    return n;
}

// Host memory for operator arguments.  Pinned (page-locked) when a device is present, so the
// copies the entry points make run at the link's full rate (57 GB/s each way here, against 30 in
// and 18 out for pageable memory); plain 64-byte aligned memory otherwise.  Counterpart of
// halide_malloc / halide_free (t2s/src/AOT-OpenCL-Runtime.cpp:56-72), which align to 64 bytes for
// the same reason (DMA).  A small header in front of the block records how it was obtained.
namespace {
struct HostBlockHeader {
    uint64_t magic;
    uint64_t pinned;
    void *base;
    uint64_t pad[5];
};
static_assert(sizeof(HostBlockHeader) == 64, "keeps the payload 64-byte aligned");
constexpr uint64_t HOST_BLOCK_MAGIC = 0x7432737068626c6bull;
}  // namespace

extern "C" void *t2sp_host_malloc(size_t bytes) {
    const size_t total = bytes + sizeof(HostBlockHeader);
    void *base = nullptr;
    uint64_t pinned = 0;
    if (t2sp_device_count() > 0) {
        if (hipHostMalloc(&base, total, hipHostMallocDefault) == hipSuccess) pinned = 1;
        else { (void)hipGetLastError(); base = nullptr; }
    }
    if (!base) {
        if (posix_memalign(&base, 64, (total + 63) / 64 * 64) != 0) return nullptr;
    }
    HostBlockHeader *h = static_cast<HostBlockHeader *>(base);
    h->magic = HOST_BLOCK_MAGIC;
    h->pinned = pinned;
    h->base = base;
    return h + 1;
}

extern "C" void t2sp_host_free(void *p) {
    if (!p) return;
    HostBlockHeader *h = static_cast<HostBlockHeader *>(p) - 1;
    if (h->magic != HOST_BLOCK_MAGIC) return;      // freed twice, or not from t2sp_host_malloc: do nothing
    h->magic = 0;
    if (h->pinned) (void)hipHostFree(h->base);
    else free(h->base);
}
