// metadata.cpp — <fn>_metadata() of every operator entry, and <fn>_argv() of the entries whose
// host file does not define it.
//
// Halide emits, next to every generated entry with the default ExternalPlusMetadata linkage, an
// argv form and a function that returns a static table of the entry's arguments
// (Halide/src/CodeGen_C.cpp:1828-1833 declares both; struct halide_filter_metadata_t and
// halide_filter_argument_t: Halide/src/runtime/HalideRuntime.h:1634-1675; a generated header the
// reference ships shows the three declarations side by side:
// t2s/peppers/blas/level3/syrk/release/s10/syrk-interface.h:11-18).  Tools built on Halide (RunGen,
// the registration mechanism of HalideRuntime.h:1677-1691) walk the table to build argument lists
// for <fn>_argv.  The tables here list the arguments in call order under the names the reference's
// specifications give them: the ImageParams and Params (gemm.cpp:53, conv.cpp:51, capsule.cpp:51,
// syrk.cpp:56-58, ger.cpp:53, gbmv3.cpp:50-51, symv.cpp:52-53, pairhmm.cpp:34-44, qrd.cpp:20) and
// the output "deserializer" (gemm.cpp:83, conv.cpp:89, capsule.cpp:88, syrk.cpp:98, ger.cpp:95,
// gbmv3.cpp:92, symv.cpp:91, pairhmm.cpp:112; QDeserializer and RDeserializer, qrd.cpp:107).  MTTKRP
// has no specification in the reference and uses the names of mttkrp-interface.h.  Ranks are those
// of the FPGA flow's buffers; the entries also accept the other forms their headers list.
#include "gbmv3-interface.h"
#include "ger-interface.h"
#include "pairhmm-interface.h"
#include "qrd-interface.h"
#include "symv-interface.h"
#include "syrk-interface.h"
#include "t2sp_buffer.h"

namespace {

enum Elem { F32, I32, U8 };

struct ArgSpec {
    const char *name;
    int kind, dimensions;
    Elem elem;
};

constexpr int SCALAR = halide_argument_kind_input_scalar, IN = halide_argument_kind_input_buffer,
              OUT = halide_argument_kind_output_buffer;
constexpr int MAX_ARGS = 10;

// halide_type_t has constructors when it comes from Halide's header and none in the restatement of
// t2sp_buffer.h, so a table is filled at first use instead of brace-initialised.
struct Table {
    halide_filter_argument_t args[MAX_ARGS];
    halide_filter_metadata_t meta;
    Table(const char *fn, std::initializer_list<ArgSpec> specs) {
        int n = 0;
        for (const ArgSpec &s : specs) {
            halide_filter_argument_t &a = args[n++];
            a.name = s.name;
            a.kind = s.kind;
            a.dimensions = s.dimensions;
            a.type.code = s.elem == F32 ? halide_type_float : s.elem == I32 ? halide_type_int : halide_type_uint;
            a.type.bits = s.elem == U8 ? 8 : 32;
            a.type.lanes = 1;
            a.scalar_def = a.scalar_min = a.scalar_max = a.scalar_estimate = nullptr;
            a.buffer_estimates = nullptr;
        }
        meta.version = 1;
        meta.num_arguments = n;
        meta.arguments = args;
        meta.target = "hip-gfx950";
        meta.name = fn;
    }
};

inline halide_buffer_t *buf(void *p) { return static_cast<halide_buffer_t *>(p); }
inline float f32(void *p) { return *static_cast<float *>(p); }
inline int32_t i32(void *p) { return *static_cast<int32_t *>(p); }

}  // namespace

#define T2SP_METADATA(fn, ...)                                            \
    extern "C" const halide_filter_metadata_t *fn##_metadata(void) {      \
        static const Table t(#fn, {__VA_ARGS__});                         \
        return &t.meta;                                                   \
    }

T2SP_METADATA(gemm, {"A", IN, 2, F32}, {"B", IN, 2, F32}, {"deserializer", OUT, 6, F32})
// t2s/tests/correctness/aot/gemm-generate.cpp:43-44,176: ImageParams a and b, entry "GEMM".
T2SP_METADATA(GEMM, {"a", IN, 2, F32}, {"b", IN, 2, F32}, {"deserializer", OUT, 6, F32})
T2SP_METADATA(conv, {"I", IN, 2, F32}, {"K", IN, 2, F32}, {"deserializer", OUT, 10, F32})
T2SP_METADATA(capsule, {"P", IN, 2, F32}, {"W", IN, 2, F32}, {"deserializer", OUT, 10, F32})
T2SP_METADATA(mttkrp, {"B", IN, 3, F32}, {"C", IN, 2, F32}, {"D", IN, 2, F32}, {"A", OUT, 2, F32})
T2SP_METADATA(syrk, {"OpA", SCALAR, 0, I32}, {"Alpha", SCALAR, 0, F32}, {"Beta", SCALAR, 0, F32}, {"A", IN, 2, F32},
              {"C", IN, 2, F32}, {"deserializer", OUT, 6, F32})
T2SP_METADATA(ger, {"A", IN, 2, F32}, {"X", IN, 1, F32}, {"Y", IN, 1, F32}, {"deserializer", OUT, 6, F32})
T2SP_METADATA(gbmv3, {"Alpha", SCALAR, 0, F32}, {"Beta", SCALAR, 0, F32}, {"A", IN, 2, F32}, {"X", IN, 1, F32},
              {"Y", IN, 1, F32}, {"deserializer", OUT, 3, F32})
T2SP_METADATA(symv, {"Alpha", SCALAR, 0, F32}, {"Beta", SCALAR, 0, F32}, {"A", IN, 2, F32}, {"X", IN, 1, F32},
              {"Y", IN, 1, F32}, {"deserializer", OUT, 3, F32})
T2SP_METADATA(pairhmm, {"H", IN, 2, U8}, {"R", IN, 2, U8}, {"delta", IN, 2, F32}, {"zeta", IN, 2, F32},
              {"eta", IN, 2, F32}, {"alpha_match", IN, 2, F32}, {"alpha_gap", IN, 2, F32}, {"beta_match", IN, 2, F32},
              {"beta_gap", IN, 2, F32}, {"deserializer", OUT, 4, F32})
T2SP_METADATA(qrd, {"a", IN, 3, F32}, {"QDeserializer", OUT, 3, F32}, {"RDeserializer", OUT, 3, F32})

// The argv forms: args[i] points at the i-th scalar, or is the i-th halide_buffer_t* itself.
extern "C" int syrk_argv(void **a) {
    if (!a) return halide_error_code_buffer_argument_is_null;
    return syrk(i32(a[0]), f32(a[1]), f32(a[2]), buf(a[3]), buf(a[4]), buf(a[5]));
}
extern "C" int ger_argv(void **a) {
    if (!a) return halide_error_code_buffer_argument_is_null;
    return ger(buf(a[0]), buf(a[1]), buf(a[2]), buf(a[3]));
}
extern "C" int gbmv3_argv(void **a) {
    if (!a) return halide_error_code_buffer_argument_is_null;
    return gbmv3(f32(a[0]), f32(a[1]), buf(a[2]), buf(a[3]), buf(a[4]), buf(a[5]));
}
extern "C" int symv_argv(void **a) {
    if (!a) return halide_error_code_buffer_argument_is_null;
    return symv(f32(a[0]), f32(a[1]), buf(a[2]), buf(a[3]), buf(a[4]), buf(a[5]));
}
extern "C" int pairhmm_argv(void **a) {
    if (!a) return halide_error_code_buffer_argument_is_null;
    return pairhmm(buf(a[0]), buf(a[1]), buf(a[2]), buf(a[3]), buf(a[4]), buf(a[5]), buf(a[6]), buf(a[7]), buf(a[8]),
                   buf(a[9]));
}
extern "C" int qrd_argv(void **a) {
    if (!a) return halide_error_code_buffer_argument_is_null;
    return qrd(buf(a[0]), buf(a[1]), buf(a[2]));
}
