// MTTKRP driver around the reference's only definition of the operator, the helper
// get_result_of_mttkrp<T, L, I, J, K>(a, b, c) -> d of t2s/tests/performance/util/util.h:498-515:
// a(l,i,k), c(l,j), b(k,j) -> d(i,j).  mttkrp(B, C, D, A) takes them as B = a, C = c, D = b, A = d.
#include "mttkrp-interface.h"
#include "driver_common.h"

#define L 32
#define I 48
#define J 40
#define K 24

int main() {
    t2sp::Buffer<float> a(L, I, K), c(L, J), b(K, J), d(I, J);
    drv::Rng ra(7), rc_(8), rb(9);
    for (int k = 0; k < K; k++)
        for (int i = 0; i < I; i++)
            for (int l = 0; l < L; l++) a(l, i, k) = ra.next();
    for (int j = 0; j < J; j++)
        for (int l = 0; l < L; l++) c(l, j) = rc_.next();
    for (int j = 0; j < J; j++)
        for (int k = 0; k < K; k++) b(k, j) = rb.next();
    const int rc = mttkrp(a, c, b, d);
    if (rc != 0) {
        std::printf("mttkrp returned %d\n", rc);
        return 2;
    }
    drv::Check chk;
    for (int i = 0; i < I; i++)
        for (int j = 0; j < J; j++) {
            float dij = 0.0f;
            for (int k = 0; k < K; k++) {
                float e = 0.0f;
                for (int l = 0; l < L; l++) e += a(l, i, k) * c(l, j);
                dij += e * b(k, j);
            }
            chk.one(dij, d(i, j));
        }
    return chk.report("mttkrp", t2sp_last_kernel_ns());
}
