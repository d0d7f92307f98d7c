// blas_gemm_entry.cpp — libt2sp_blas_gemm.so: the 8-argument pipeline entry of the reference's BLAS
// release under its own C name.
//
// The reference generates two different pipelines that are both called `gemm` with C linkage: the
// 3-argument one of t2s/tests/performance/gemm (gemm-run-fpga.cpp:70) and the 8-argument one behind
// its BLAS wrapper, gemm(opa, opb, alpha, beta, A, B, C, O) (t2s/peppers/blas/level3/gemm/release/
// a10/blas-gemm.cpp:29).  They never meet in one program there; one library cannot export both, so
// the second lives in this small library of its own, which forwards to t2sp_gemm_ex of
// libt2sp_mi355x.so.  A program built like the reference's release (compile.txt: sgemm-run-fpga.cpp,
// blas-gemm.cpp and the generated gemm-interface.cpp) links -lt2sp_blas_gemm -lt2sp_mi355x in place
// of gemm-interface.cpp and the OpenCL runtime.  The scalar arguments are 32-bit integers, as
// Param<int> gives the SYRK pipeline of the same family (t2s/tests/performance/syrk/syrk.cpp:56).
#include <stdint.h>

#include "t2sp_buffer.h"

extern "C" int t2sp_gemm_ex(int opa, int opb, float alpha, float beta, struct halide_buffer_t *A, struct halide_buffer_t *B,
                            struct halide_buffer_t *C, struct halide_buffer_t *O);

extern "C" int gemm(int32_t opa, int32_t opb, float alpha, float beta, struct halide_buffer_t *A, struct halide_buffer_t *B,
                    struct halide_buffer_t *C, struct halide_buffer_t *O) {
    return t2sp_gemm_ex(opa, opb, alpha, beta, A, B, C, O);
}

extern "C" int gemm_argv(void **args) {
    if (!args) return halide_error_code_buffer_argument_is_null;
    return t2sp_gemm_ex(*static_cast<int32_t *>(args[0]), *static_cast<int32_t *>(args[1]), *static_cast<float *>(args[2]),
                        *static_cast<float *>(args[3]), static_cast<halide_buffer_t *>(args[4]),
                        static_cast<halide_buffer_t *>(args[5]), static_cast<halide_buffer_t *>(args[6]),
                        static_cast<halide_buffer_t *>(args[7]));
}

// The argument table of the 8-argument entry (Halide/src/CodeGen_C.cpp:1830-1833).  The release
// ships no specification for it; the scalar names are those of the SYRK pipeline of the same family
// (Param<int> OpA, Param<float> Alpha, Beta: t2s/tests/performance/syrk/syrk.cpp:56-57).
extern "C" const halide_filter_metadata_t *gemm_metadata(void) {
    static halide_filter_argument_t args[8];
    static halide_filter_metadata_t meta;
    static const bool once = [] {
        const char *names[8] = {"OpA", "OpB", "Alpha", "Beta", "A", "B", "C", "deserializer"};
        for (int i = 0; i < 8; i++) {
            args[i].name = names[i];
            args[i].kind = i < 4 ? halide_argument_kind_input_scalar
                                 : i < 7 ? halide_argument_kind_input_buffer : halide_argument_kind_output_buffer;
            args[i].dimensions = i < 4 ? 0 : i < 7 ? 2 : 6;
            args[i].type.code = i < 2 ? halide_type_int : halide_type_float;
            args[i].type.bits = 32;
            args[i].type.lanes = 1;
            args[i].scalar_def = args[i].scalar_min = args[i].scalar_max = args[i].scalar_estimate = nullptr;
            args[i].buffer_estimates = nullptr;
        }
        meta.version = 1;
        meta.num_arguments = 8;
        meta.arguments = args;
        meta.target = "hip-gfx950";
        meta.name = "gemm";
        return true;
    }();
    (void)once;
    return &meta;
}
