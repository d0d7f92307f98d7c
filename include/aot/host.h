/* host.h — the header name the reference's AOT boundary test generates:
 * mm.compile_to_host("host", args, "GEMM", target) (t2s/tests/correctness/aot/gemm-generate.cpp:176)
 * writes host.h declaring GEMM(a, b, result), and gemm-run.cpp:19,62 includes and calls it.  The
 * entry is declared by gemm-interface.h; this file only carries the generated name, in a directory
 * of its own so that the plain name does not sit on every user's include path (-I include/aot). */
#ifndef T2SP_AOT_HOST_H
#define T2SP_AOT_HOST_H
#include "../gemm-interface.h"
#endif
