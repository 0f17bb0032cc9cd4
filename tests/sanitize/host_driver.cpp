// Host-only run of the library's host code for AddressSanitizer / UBSan (tests/test_host.py builds
// and runs it): generate the five workloads at small scale, partition them at several tau, and lay
// out the CSR part's slice form and the whole host half of a plan under every flag.  No GPU call.
#include <cstdio>
#include <cstdlib>
#include <vector>
#include "matxtract_hip.h"
int main()
{
    const int cfgs[] = {1, 2, 3, 4, 5};
    const double scales[] = {1.0, 1.0 / 32, 1.0 / 64, 1.0 / 32, 1.0 / 128};
    const float taus[][2] = {{1.f, 1.f}, {0.75f, 0.5f}, {0.5f, 0.f}, {0.f, 0.f}};
    const int flags[] = {MX_PLAN_DEFAULT, MX_PLAN_KEEP_TILES, MX_PLAN_ALL_TILES, MX_PLAN_NO_TILES};
    for (int c = 0; c < 5; ++c) {
        mx_csr A;
        void *x = nullptr, *val = nullptr;
        int *rp = nullptr, *ci = nullptr;
        if (mx_gen_config(cfgs[c], 0, scales[c], &A.rows, &A.cols, &A.nnz, &A.dtype, &rp, &ci, &val, &x)) { printf("gen failed: %s\n", mx_last_error()); return 1; }
        A.rowPtr = rp; A.colInd = ci; A.val = val;
        printf("cfg %d rows %d nnz %d\n", cfgs[c], A.rows, A.nnz);
        mx_slice_layout_view sv;
        if (mx_slice_layout(&A, 8, nullptr, &sv)) { printf("slice layout: %s\n", mx_last_error()); return 1; }
        mx_slice_layout_free(&sv);
        // the layout of the one-launch form (refused for the power-law workloads, whose rows reach many slices)
        for (int nCU : {8, 32, 256}) {
            if (mx_slice_layout_fused(&A, nCU, &sv)) { printf("fused slice layout: %s\n", mx_last_error()); return 1; }
            printf("  fused layout on %d workgroups: %d\n", nCU, sv.fused);
            mx_slice_layout_free(&sv);
        }
        for (auto &t : taus) {
            mx_partition *P = nullptr;
            if (mx_partition_create(&A, t[0], t[1], &P)) { printf("partition: %s\n", mx_last_error()); return 1; }
            for (int f : flags) {
                mx_plan_layout_view v;
                if (mx_plan_layout(P, f, 8, &v)) { printf("plan layout: %s\n", mx_last_error()); return 1; }
                mx_plan_layout_free(&v);
            }
            mx_partition_destroy(P);
        }
        free(rp); free(ci); free(val); free(x);
    }
    printf("ok\n");
    return 0;
}
