// matxtract_perftest -- the reference's performance driver, on the HIP library.
//
//   matxtract_perftest [col_frac hot_frac] matrix.mtx            (reference form,
//                                                                  test/test_autotc_spmv.cpp:1052-1076)
//   matxtract_perftest [col_frac hot_frac] --config N [options]   (synthetic workload N = 1..5)
//
// Additive options: --scale S (shrink a synthetic workload), --seed S, --keep-values (do not
// overwrite the file's values with i%15 as the reference does at :1091), --warm W --iters K
// (default 200 / 4000), --no-tiles / --all-tiles (plan flags), --json (one JSON record on the
// last line), --tune (pick the two fractions from the 5x5 grid by timing each on the device,
// then run with them), --estimate-tau (pick them from counts over the same grid, nothing timed), --partition-cache FILE (read the partition from FILE when it was made for a
// matrix of this shape with these fractions, otherwise compute it and write FILE), --device-prep / --host-prep (the extraction runs on the GPU /
// on the host cores; same partition; without either the GPU takes matrices of two million entries or more), --device-plan (the matrix is uploaded as it is and everything after
// that -- extraction, the plan's decisions, its layouts -- happens on the GPU: mx_plan_create_device;
// same plan, no partition on the host, so no --partition-cache and no checksum in the JSON record).
// Precision is the build's: -Dfp64 -> FP64 binary, otherwise FP16.
//
// Lines other tools parse (ML/bayes_opt.py:64, script/duse.sh:35-38) keep their form:
//   cols_ratio = %f / TC_nnz_ratio = %lf / MatXtract time = %lf ms / Success! ... |
//   Error at index (... / MatXtract GFLOPS= %.2f
#include <chrono>
#include <cmath>
#include <iostream>
#include <string>

#include <hip/hip_runtime_api.h>

#include "MatXtract.h"

namespace {

// The driver's own CPU check (spmv_serial, test/test_autotc_spmv.cpp:300-316).  FP16 builds
// accumulate in float, the arithmetic the synthetic workloads specify.
void spmv_check_cpu(const valT *val, const indT *rowPtr, const indT *colInd, const valT *x, valT *y, int rows)
{
    for (int i = 0; i < rows; ++i) {
#ifdef fp64
        double t = 0.0;
        for (indT p = rowPtr[i]; p < rowPtr[i + 1]; ++p) t = t + val[p] * x[colInd[p]];
        y[i] = y[i] + t;
#else
        float t = 0.f;
        for (indT p = rowPtr[i]; p < rowPtr[i + 1]; ++p) t = t + (float)val[p] * (float)x[colInd[p]];
        y[i] = half(t);
#endif
    }
}

// eQcheck (test/test_autotc_spmv.cpp:257-293), same messages and tolerances.
int eQcheck(const valT *a, const valT *b, int n)
{
#ifdef fp64
    const double tol = 1e-8;
    for (int i = 0; i < n; ++i) {
        double v1 = a[i], v2 = b[i];
        if (std::fabs(v1 - v2) / std::fmax(std::fabs(v1), std::fabs(v2)) > tol) {
            printf("Error at index (%d), res(%4.15f), our(%4.15f), please check your code!\n", i, v1, v2);
            return -1;
        }
    }
#else
    const float tol = 1e-1f;
    for (int i = 0; i < n; ++i) {
        float v1 = (float)a[i], v2 = (float)b[i];
        if (std::fabs(v1 - v2) / std::fmax(std::fabs(v1), std::fabs(v2)) > tol) {
            printf("Error at index (%d), res(%4.3f), our(%4.3f), please check your code!\n", i, v1, v2);
            return -1;
        }
    }
#endif
    printf("Success! All values match within the tolerance for %d elements.\n", n);
    return 0;
}

double rel_l2(const valT *ref, const valT *got, int n)
{
    double num = 0.0, den = 0.0;
    for (int i = 0; i < n; ++i) {
        double r = (double)ref[i], g = (double)got[i];
        num += (r - g) * (r - g);
        den += r * r;
    }
    return den > 0 ? std::sqrt(num / den) : std::sqrt(num);
}

void usage()
{
    printf("Run the code by './matxtract_perftest (col_frac) (hot_frac) matrix.mtx'.\n");
    printf("col_frac and hot_frac are optional, defaulting to 0 if not provided.\n");
}

}  // namespace

int main(int argc, char **argv)
{
    std::vector<std::string> pos;
    int config = 0, warm = 200, iters = 4000, planFlags = MX_PLAN_DEFAULT;
    double scale = 1.0;
    unsigned long long seed = 0;
    bool keepValues = false, json = false, tune = false, estimate = false, devicePlan = false;
    int devicePrep = -1;  // -1: the GPU for a matrix of two million entries or more, the host otherwise
    std::string cachePath;
    for (int i = 1; i < argc; ++i) {
        std::string a = argv[i];
        auto next = [&](const char *name) -> const char * {
            if (i + 1 >= argc) {
                printf("Error: %s needs a value.\n", name);
                exit(1);
            }
            return argv[++i];
        };
        if (a == "--config") config = atoi(next("--config"));
        else if (a == "--scale") scale = atof(next("--scale"));
        else if (a == "--seed") seed = strtoull(next("--seed"), nullptr, 0);
        else if (a == "--warm") warm = atoi(next("--warm"));
        else if (a == "--iters") iters = atoi(next("--iters"));
        else if (a == "--keep-values") keepValues = true;
        else if (a == "--no-tiles") planFlags = MX_PLAN_NO_TILES;
        else if (a == "--all-tiles") planFlags = MX_PLAN_ALL_TILES;
        else if (a == "--keep-tiles") planFlags = MX_PLAN_KEEP_TILES;
        else if (a == "--json") json = true;
        else if (a == "--partition-cache") cachePath = next("--partition-cache");
        else if (a == "--tune") tune = true;
        else if (a == "--estimate-tau") estimate = true;
        else if (a == "--device-prep") devicePrep = 1;
        else if (a == "--host-prep") devicePrep = 0;
        else if (a == "--device-plan") devicePlan = true;
        else pos.push_back(a);
    }
    const size_t npos = pos.size() + (config ? 1 : 0);  // a --config stands for the file name
    if (npos < 1) {
        usage();
        return 1;
    }
    double col_frac = 0.0, hot_frac = 0.0;
    if (npos == 3) {
        col_frac = atof(pos[0].c_str());
        hot_frac = atof(pos[1].c_str());
        if (col_frac < hot_frac) {
            printf("Error: col_frac must be greater than hot_frac.\n");
            printf("Please run the program with valid parameters.\n");
            return 1;
        }
    } else if (npos > 3 || npos == 2) {
        printf("Error: Too many arguments provided.\n");
        usage();
        return 1;
    }

    int rowA = 0, colA = 0, isSymmetricA = 0;
    indT nnzA = 0;
    valT *csrVal = nullptr, *X_val = nullptr;
    indT *csrColInd = nullptr, *csrRowPtr = nullptr;
    std::string name;
    if (config) {
        name = "synthetic workload " + std::to_string(config);
        mx_dtype dt;
        int rc = mx_gen_config(config, seed, scale, &rowA, &colA, &nnzA, &dt, &csrRowPtr, &csrColInd, (void **)&csrVal,
                               (void **)&X_val);
        if (rc != MX_OK) {
            printf("Error: %s\n", mx_last_error());
            return 1;
        }
        if (dt != MX_VALT_DTYPE) {
            printf("Error: workload %d is %s; use the %s build of this program.\n", config, dt == MX_F64 ? "FP64" : "FP16",
                   dt == MX_F64 ? "FP64" : "FP16");
            return 1;
        }
    } else {
        name = pos.back();
    }
#ifdef fp64
    printf("\n Processing the %s graph in FP64\n\n", name.c_str());
#else
    printf("\n Processing the %s graph in FP16\n\n", name.c_str());
#endif
    if (!config) {
        if (mmio_allinone(&rowA, &colA, &nnzA, &isSymmetricA, &csrRowPtr, &csrColInd, &csrVal, (char *)name.c_str()) != 0) {
            printf("Error: %s\n", mx_last_error());
            return 1;
        }
        if (!keepValues) initVec(csrVal, nnzA);  // :1091
        X_val = (valT *)malloc(sizeof(valT) * (size_t)(colA > 0 ? colA : 1));
        initVec(X_val, colA);  // :1433-1434
    }

    if (tune) {
        // the two fractions chosen on the device instead of given (what ML/bayes_opt.py does around this program)
        mx_csr A{rowA, colA, (int)nnzA, MX_VALT_DTYPE, csrRowPtr, csrColInd, csrVal};
        mx_tau_point table[15];
        float tc = 0.f, tr = 0.f;
        int n = 0;
        if (mx_tune_tau(&A, 5, planFlags, 20, 200, &tc, &tr, table, 15, &n) != MX_OK) {
            printf("Error: %s\n", mx_last_error());
            return 1;
        }
        for (int i = 0; i < n && i < 15; ++i)
            printf("tune: col_frac = %.2f hot_frac = %.2f time = %lf ms tile_nnz = %d\n", table[i].tau_c, table[i].tau_r,
                   table[i].ms_total, table[i].tile_nnz);
        printf("tuned: col_frac = %.2f hot_frac = %.2f\n", tc, tr);
        col_frac = tc;
        hot_frac = tr;
    }
    if (estimate) {
        // the two fractions from counts over the grid (the plan's own estimate of what its tiles save), nothing timed
        mx_csr A{rowA, colA, (int)nnzA, MX_VALT_DTYPE, csrRowPtr, csrColInd, csrVal};
        mx_tau_estimate table[15];
        float tc = 0.f, tr = 0.f;
        int n = 0;
        if (mx_estimate_tau(&A, 5, &tc, &tr, table, 15, &n) != MX_OK) {
            printf("Error: %s\n", mx_last_error());
            return 1;
        }
        for (int i = 0; i < n && i < 15; ++i)
            printf("estimate: col_frac = %.2f hot_frac = %.2f saved = %lf us tile_nnz = %lld\n", table[i].tau_c, table[i].tau_r,
                   table[i].saved_us, table[i].tile_entries);
        printf("estimated: col_frac = %.2f hot_frac = %.2f\n", tc, tr);
        col_frac = tc;
        hot_frac = tr;
    }
    const float colProp = (float)col_frac, rowProp = (float)hot_frac;
    const bool extracting = !((rowProp == 0.0) && (colProp == 0.0));
    if (extracting) {
        std::cout << "---------------------------------------------------------" << std::endl;
        std::cout << "                     localRow: " << rowProp << std::endl;
        std::cout << "                     globalCol: " << colProp << std::endl;
        std::cout << "---------------------------------------------------------" << std::endl;
        std::cout << "---------------------Compression Info--------------------" << std::endl;
    }
    if (devicePrep < 0) devicePrep = nnzA >= (1 << 21) && extracting && mx_device_count() > 0;
    if (devicePrep || devicePlan) (void)hipFree(nullptr);  // the first use of the device is not part of the preprocessing time
    auto t0 = std::chrono::steady_clock::now();
    mx_partition *part = nullptr;
    mx_plan *plan = nullptr;
    mx_plan_info info;
    mx_partition_view pv{};
    double preprocess_ms = 0.0;
    if (devicePlan) {
        if (!cachePath.empty()) {
            printf("Error: --device-plan keeps no partition on the host; it cannot be combined with --partition-cache.\n");
            return 1;
        }
        // the matrix goes up as it is; extraction, decisions and layouts are made on the device
        void *dRowPtr = nullptr, *dColInd = nullptr, *dVal = nullptr;
        const size_t nz = (size_t)(nnzA > 0 ? nnzA : 1);
        if (hipMalloc(&dRowPtr, sizeof(indT) * ((size_t)rowA + 1)) != hipSuccess || hipMalloc(&dColInd, sizeof(indT) * nz) != hipSuccess ||
            hipMalloc(&dVal, sizeof(valT) * nz) != hipSuccess ||
            hipMemcpy(dRowPtr, csrRowPtr, sizeof(indT) * ((size_t)rowA + 1), hipMemcpyHostToDevice) != hipSuccess ||
            hipMemcpy(dColInd, csrColInd, sizeof(indT) * (size_t)nnzA, hipMemcpyHostToDevice) != hipSuccess ||
            hipMemcpy(dVal, csrVal, sizeof(valT) * (size_t)nnzA, hipMemcpyHostToDevice) != hipSuccess) {
            fprintf(stderr, "MatXtract HIP error: could not put the matrix on the device\n");
            return EXIT_FAILURE;
        }
        matxtract_detail::check(mx_plan_create_device(MX_VALT_DTYPE, rowA, colA, (int)nnzA, (const int *)dRowPtr, (const int *)dColInd, dVal,
                                                      colProp, rowProp, planFlags, &plan),
                                "mx_plan_create_device");
        (void)hipFree(dRowPtr);
        (void)hipFree(dColInd);
        (void)hipFree(dVal);
        preprocess_ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
        mx_plan_get_info(plan, &info);
        pv.dCols = info.ext_dCols;
        pv.dRows = info.ext_dRows;
        pv.cols_ratio = colA > 0 ? (float)info.ext_dCols / (float)colA : 0.0f;
        pv.tc_nnz_ratio = info.ext_frags > 0 ? (double)info.ext_nnzRowD / ((double)info.ext_frags * 8.0 * (MX_VALT_DTYPE == MX_F64 ? 4 : 8)) : 0.0;
    } else {
        bool fromCache = false;
        if (!cachePath.empty() && mx_partition_load(cachePath.c_str(), MX_VALT_DTYPE, &part) == MX_OK) {
            // The file is used only if it was made from a matrix of this shape with these fractions.
            mx_partition_view cv;
            mx_partition_get(part, &cv);
            fromCache = cv.rows == rowA && cv.cols == colA && cv.nnz == (long long)nnzA && cv.tau_c == colProp && cv.tau_r == rowProp;
            if (!fromCache) {
                mx_partition_destroy(part);
                part = nullptr;
            }
        }
        if (!part) part = matxtract_preprocess(csrVal, csrRowPtr, csrColInd, rowA, colA, nnzA, colProp, rowProp, devicePrep);
        auto t1 = std::chrono::steady_clock::now();
        if (!part) return 1;
        if (!cachePath.empty()) {
            if (fromCache) printf("partition read from %s\n", cachePath.c_str());
            else if (mx_partition_save(part, cachePath.c_str()) != MX_OK) printf("Warning: %s\n", mx_last_error());
            else printf("partition written to %s\n", cachePath.c_str());
        }
        preprocess_ms = std::chrono::duration<double, std::milli>(t1 - t0).count();
        mx_partition_counts(part, &pv);  // (the arrays of a partition made on the device stay there: the plan is made from them)
    }
    if (extracting) {
        printf("cols_ratio = %f \n", pv.cols_ratio);
        printf("TC_nnz_ratio = %lf\n", pv.tc_nnz_ratio);
        std::cout << "---------------------Performance Info--------------------" << std::endl;
    }
    if (!plan) {
        matxtract_detail::check(mx_plan_create(part, planFlags, &plan), "mx_plan_create");
        mx_plan_get_info(plan, &info);
    }

    valT *Y_val = (valT *)malloc(sizeof(valT) * (size_t)(rowA > 0 ? rowA : 1));
    valT *ourY_val = (valT *)malloc(sizeof(valT) * (size_t)(rowA > 0 ? rowA : 1));
    for (int i = 0; i < rowA; ++i) Y_val[i] = static_cast<valT>(0.0);
    spmv_check_cpu(csrVal, csrRowPtr, csrColInd, X_val, Y_val, rowA);

    void *dx = nullptr, *dy = nullptr;
    if (hipMalloc(&dx, sizeof(valT) * (size_t)(colA > 0 ? colA : 1)) != hipSuccess ||
        hipMalloc(&dy, sizeof(valT) * (size_t)(rowA > 0 ? rowA : 1)) != hipSuccess ||
        hipMemcpy(dx, X_val, sizeof(valT) * (size_t)colA, hipMemcpyHostToDevice) != hipSuccess) {
        fprintf(stderr, "MatXtract HIP error: could not stage x/y on the device\n");
        return EXIT_FAILURE;
    }
    double ms_total = 0.0, ms_tile = 0.0, ms_csr = 0.0;
    matxtract_detail::check(mx_time(plan, dx, dy, warm, iters, &ms_total, &ms_tile, &ms_csr), "mx_time");
    if (hipMemcpy(ourY_val, dy, sizeof(valT) * (size_t)rowA, hipMemcpyDeviceToHost) != hipSuccess) {
        fprintf(stderr, "MatXtract HIP error: could not fetch y\n");
        return EXIT_FAILURE;
    }

    // "MatXtract time" is the measured latency of the whole sequence; the reference adds two
    // separately timed halves (:1561-1572), printed alongside for comparison.
    printf("tile kernel = %lf ms, csr kernel = %lf ms (timed apart, sum %lf ms)\n", ms_tile, ms_csr, ms_tile + ms_csr);
    printf("MatXtract time = %lf ms\n\n", ms_total);
    int result = eQcheck(Y_val, ourY_val, rowA);
    const double gflops = (2.0 * (double)nnzA) / (ms_total * 1e-3) / 1e9;
    const double bytes = mx_algorithmic_bytes(MX_VALT_DTYPE, rowA, colA, nnzA);
    const double gbs = bytes / (ms_total * 1e-3) / 1e9;
    printf("rel_l2 = %.3e, algorithmic bytes = %.0f, %.1f GB/s = %.1f%% of 8 TB/s\n", rel_l2(Y_val, ourY_val, rowA), bytes,
           gbs, gbs / 80.0);
    printf("MatXtract GFLOPS= %.2f\n", gflops);
    if (json) {
        printf("{\"rows\": %d, \"cols\": %d, \"nnz\": %d, \"dtype\": \"%s\", \"tau_c\": %g, \"tau_r\": %g, "
               "\"dCols\": %d, \"dRows\": %d, \"tc_nnz_ratio\": %.6f, \"tile_chunks\": %d, \"tile_nnz\": %d, "
               "\"csr_nnz\": %d, \"preprocess_ms\": %.3f, \"ms_total\": %.6f, \"ms_tile\": %.6f, \"ms_csr\": %.6f, "
               "\"gflops\": %.3f, \"algorithmic_bytes\": %.0f, \"gbs\": %.3f, \"hbm_frac\": %.5f, \"rel_l2\": %.3e, "
               "\"pass\": %s, \"partition_hash\": \"%016llx\", \"prep_route\": %d}\n",
               rowA, colA, nnzA,
#ifdef fp64
               "f64",
#else
               "f16",
#endif
               col_frac, hot_frac, pv.dCols, pv.dRows, extracting ? pv.tc_nnz_ratio : 0.0, info.tile_chunks, info.tile_nnz,
               info.csr_nnz, preprocess_ms, ms_total, ms_tile, ms_csr, gflops, bytes, gbs, gbs / 8000.0,
               rel_l2(Y_val, ourY_val, rowA), result == 0 ? "true" : "false", part ? (unsigned long long)mx_partition_hash(part) : 0ull,
               info.prep_route);
    }
    (void)hipFree(dx);
    (void)hipFree(dy);
    mx_plan_destroy(plan);
    if (part) mx_partition_destroy(part);
    free(Y_val);
    free(ourY_val);
    free(X_val);
    free(csrColInd);
    free(csrRowPtr);
    free(csrVal);
    return 0;
}
