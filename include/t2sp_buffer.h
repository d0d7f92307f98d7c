/* t2sp_buffer.h — the argument type of every operator entry point.
 *
 * A self-contained, ABI-identical restatement of the three structs that the
 * reference's generated host interface takes and of its error codes:
 *   halide_type_t       Halide/src/runtime/HalideRuntime.h:426-438
 *   halide_dimension_t  Halide/src/runtime/HalideRuntime.h:1356-1360
 *   halide_buffer_t     Halide/src/runtime/HalideRuntime.h:1392-1418
 *   buffer flags        Halide/src/runtime/HalideRuntime.h:1384-1385
 *   error codes         Halide/src/runtime/HalideRuntime.h:957-1143
 *   filter metadata     Halide/src/runtime/HalideRuntime.h:1603-1675
 * When the reference's own HalideRuntime.h is on the include path (a driver that
 * uses Halide::Runtime::Buffer from HalideBuffer.h has it there), that header is
 * included here instead and the definitions below are skipped, exactly as the
 * generated <op>-interface.h brings in the Halide types before it declares the
 * entry (Halide/src/CodeGen_C.cpp:327, t2s/src/AOT-OpenCL-Runtime.h:20-31).  This
 * happens by itself where the compiler has __has_include; defining
 * T2SP_USE_HALIDE_RUNTIME forces it, T2SP_NO_HALIDE_RUNTIME forbids it.
 *
 * Layout facts checked by the static asserts at the bottom:
 *   sizeof(halide_type_t) == 4, sizeof(halide_dimension_t) == 16,
 *   sizeof(halide_buffer_t) == 56 on LP64.
 * dim[0] is the innermost dimension; element (i0,i1,...) lives at
 *   host + sizeof(T) * sum_d (i_d - dim[d].min) * dim[d].stride.
 */
#ifndef T2SP_BUFFER_H
#define T2SP_BUFFER_H

#include <stddef.h>
#include <stdint.h>

#if !defined(T2SP_USE_HALIDE_RUNTIME) && !defined(T2SP_NO_HALIDE_RUNTIME) && defined(__has_include)
#if __has_include("HalideRuntime.h")
#define T2SP_USE_HALIDE_RUNTIME 1
#endif
#endif

#ifdef T2SP_USE_HALIDE_RUNTIME
#include "HalideRuntime.h"
#else

#ifdef __cplusplus
extern "C" {
#endif

enum halide_type_code_t {
    halide_type_int = 0,
    halide_type_uint = 1,
    halide_type_float = 2,
    halide_type_handle = 3
};

struct halide_type_t {
    uint8_t code;   /* halide_type_code_t */
    uint8_t bits;   /* bits of one scalar */
    uint16_t lanes; /* vector width, 1 for scalars */
};

typedef struct halide_dimension_t {
    int32_t min, extent, stride;
    uint32_t flags; /* reserved */
} halide_dimension_t;

typedef enum {
    halide_buffer_flag_host_dirty = 1,
    halide_buffer_flag_device_dirty = 2
} halide_buffer_flags;

struct halide_device_interface_t;

typedef struct halide_buffer_t {
    uint64_t device;                                         /* device handle, 0 = none */
    const struct halide_device_interface_t *device_interface;/* unused by this library */
    uint8_t *host;                                           /* address of the min coordinate */
    uint64_t flags;                                          /* halide_buffer_flags */
    struct halide_type_t type;
    int32_t dimensions;
    halide_dimension_t *dim;                                 /* caller-owned array */
    void *padding;
} halide_buffer_t;

enum halide_error_code_t {
    halide_error_code_success = 0,
    halide_error_code_generic_error = -1,
    halide_error_code_explicit_bounds_too_small = -2,
    halide_error_code_bad_type = -3,
    halide_error_code_access_out_of_bounds = -4,
    halide_error_code_buffer_allocation_too_large = -5,
    halide_error_code_buffer_extents_too_large = -6,
    halide_error_code_constraints_make_required_region_smaller = -7,
    halide_error_code_constraint_violated = -8,
    halide_error_code_param_too_small = -9,
    halide_error_code_param_too_large = -10,
    halide_error_code_out_of_memory = -11,
    halide_error_code_buffer_argument_is_null = -12,
    halide_error_code_copy_to_host_failed = -14,
    halide_error_code_copy_to_device_failed = -15,
    halide_error_code_device_malloc_failed = -16,
    halide_error_code_device_sync_failed = -17,
    halide_error_code_device_free_failed = -18,
    halide_error_code_internal_error = -22,
    halide_error_code_device_run_failed = -23,
    halide_error_code_buffer_extents_negative = -28,
    halide_error_code_host_is_null = -34,
    halide_error_code_host_and_device_dirty = -37,
    halide_error_code_buffer_is_null = -38,
    halide_error_code_bad_dimensions = -43
};

/* What <fn>_metadata() returns: one record per argument of the entry. */
enum halide_argument_kind_t {
    halide_argument_kind_input_scalar = 0,
    halide_argument_kind_input_buffer = 1,
    halide_argument_kind_output_buffer = 2
};

struct halide_scalar_value_t;

struct halide_filter_argument_t {
    const char *name;
    int32_t kind;       /* halide_argument_kind_t */
    int32_t dimensions; /* 0 for scalars */
    struct halide_type_t type;
    const struct halide_scalar_value_t *scalar_def, *scalar_min, *scalar_max, *scalar_estimate; /* NULL for buffers */
    int64_t const *const *buffer_estimates;                                                   /* may be NULL */
};

struct halide_filter_metadata_t {
    int32_t version; /* 1 */
    int32_t num_arguments;
    const struct halide_filter_argument_t *arguments;
    const char *target; /* what the entry was built for */
    const char *name;   /* the entry's name */
};

#ifdef __cplusplus
} /* extern "C" */
#endif

#endif /* !T2SP_USE_HALIDE_RUNTIME */

#ifdef __cplusplus
static_assert(sizeof(struct halide_type_t) == 4, "halide_type_t must be 32 bits");
static_assert(sizeof(halide_dimension_t) == 16, "halide_dimension_t must be 16 bytes");
static_assert(sizeof(halide_buffer_t) == 56, "halide_buffer_t must be 56 bytes");
static_assert(offsetof(halide_buffer_t, host) == 16, "host at 16");
static_assert(offsetof(halide_buffer_t, flags) == 24, "flags at 24");
static_assert(offsetof(halide_buffer_t, type) == 32, "type at 32");
static_assert(offsetof(halide_buffer_t, dimensions) == 36, "dimensions at 36");
static_assert(offsetof(halide_buffer_t, dim) == 40, "dim at 40");
static_assert(sizeof(struct halide_filter_argument_t) == 64, "halide_filter_argument_t must be 64 bytes");
static_assert(offsetof(struct halide_filter_argument_t, type) == 16, "argument type at 16");
static_assert(sizeof(struct halide_filter_metadata_t) == 32, "halide_filter_metadata_t must be 32 bytes");
#endif

#ifdef __cplusplus
/* A small fixed-capacity owner of a dense float32 buffer, for drivers written
 * in the style of the reference's *-run-*.cpp files: t2sp::Buffer<float>
 * a(TOTAL_K, TOTAL_I); a(k, i) = ...; gemm(a, b, c);  It plays the role of
 * Halide::Runtime::Buffer<float> (Halide/src/runtime/HalideBuffer.h:1050-1061:
 * raw_buffer() and the implicit conversion to halide_buffer_t*) for the subset
 * those drivers use: dense allocation, operator() element access, extents.
 * Element types: float, and unsigned char for the character buffers of pairhmm. */
#include <cstring>
#include <initializer_list>
#include <new>
#include <type_traits>
#include <vector>
extern "C" void *t2sp_host_malloc(size_t bytes);
extern "C" void t2sp_host_free(void *p);
namespace t2sp {
template <typename T>
class Buffer {
    static_assert(std::is_same<T, float>::value || std::is_same<T, uint8_t>::value,
                  "float (every operator) and unsigned char (the characters of pairhmm) are the element types of this path");
    T *storage_ = nullptr;           // from t2sp_host_malloc: page-locked when a device is present
    std::vector<halide_dimension_t> dims_;
    halide_buffer_t buf_;

    void init(const int *ext, int nd, T *external) {
        dims_.resize(nd);
        int64_t stride = 1;
        for (int d = 0; d < nd; d++) {
            dims_[d].min = 0;
            dims_[d].extent = ext[d];
            dims_[d].stride = (int32_t)stride;
            dims_[d].flags = 0;
            stride *= ext[d];
        }
        if (!external) {
            storage_ = static_cast<T *>(t2sp_host_malloc((size_t)stride * sizeof(T) + 1));
            if (!storage_) throw std::bad_alloc();
            std::memset(storage_, 0, (size_t)stride * sizeof(T));
        }
        buf_.device = 0;
        buf_.device_interface = nullptr;
        buf_.host = (uint8_t *)(external ? external : storage_);
        buf_.flags = 0;
        buf_.type.code = std::is_same<T, float>::value ? halide_type_float : halide_type_uint;
        buf_.type.bits = (uint8_t)(8 * sizeof(T));
        buf_.type.lanes = 1;
        buf_.dimensions = nd;
        buf_.dim = dims_.data();
        buf_.padding = nullptr;
    }

public:
    template <typename... Ints>
    explicit Buffer(int e0, Ints... rest) {
        const int ext[] = {e0, (int)rest...};
        init(ext, 1 + (int)sizeof...(rest), nullptr);
    }
    Buffer(T *data, const std::vector<int> &ext) { init(ext.data(), (int)ext.size(), data); }
    ~Buffer() { t2sp_host_free(storage_); }
    Buffer(const Buffer &) = delete;
    Buffer &operator=(const Buffer &) = delete;

    template <typename... Ints>
    T &operator()(Ints... idx) {
        const int64_t ix[] = {(int64_t)idx...};
        int64_t off = 0;
        for (int d = 0; d < (int)sizeof...(idx); d++) off += ix[d] * dims_[d].stride;
        return ((T *)buf_.host)[off];
    }
    int dimensions() const { return buf_.dimensions; }
    int extent(int d) const { return dims_[d].extent; }
    size_t number_of_elements() const {
        size_t n = 1;
        for (auto &d : dims_) n *= (size_t)d.extent;
        return n;
    }
    T *data() { return (T *)buf_.host; }
    halide_buffer_t *raw_buffer() { return &buf_; }
    operator halide_buffer_t *() { return &buf_; }
};
}  // namespace t2sp
#endif

#endif /* T2SP_BUFFER_H */
