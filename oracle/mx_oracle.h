/*
 * mx_oracle.h -- declarations of the CPU oracle (TEST INFRASTRUCTURE ONLY).
 * See mx_oracle.c for what each function restates and how it is pinned.
 */
#ifndef MX_ORACLE_H
#define MX_ORACLE_H
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Everything the reference driver derives from (A, tau_c, tau_r); names are
 * the reference's own (test/test_autotc_spmv.cpp:1106-1492). */
typedef struct ora_partition {
    int elem;            /* 8 = binary64, 2 = binary16 */
    int rows, cols, nnz;
    int fragM, fragK;
    int dCols, sCols, nnzColD, nnzColS;
    int dRows, sRows, nnzRowD, nnzRowS;
    float cols_ratio;
    double tc_nnz_ratio;
    int *descColId;      /* [cols]  columns by count desc; first dCols are the dense ones */
    int *newArray;       /* [sCols] remaining columns ascending */
    int *rId;            /* [dRows] extracted rows in rank order */
    int *newArray_;      /* [sRows] remaining rows ascending */
    int *ddRowPtr;       /* A_dd as CSR: [dRows+1] */
    int *ddColInd;       /*              [nnzRowD] dense-column rank ids */
    void *ddVal;         /*              [nnzRowD] */
    int chunkNum, totalTcFrags, tcValCount;
    int *chunkPtr;           /* [chunkNum+1] */
    int *sparse_AToX_index;  /* [totalTcFrags*fragK] */
    int *fragPtr;            /* [totalTcFrags+1] */
    void *fragBit;           /* [totalTcFrags] uint32 (binary64) | uint64 (binary16) */
    void *tcVal;             /* [tcValCount] */
    int nnzCD;
    int *cdRowPtr;       /* residual A_CD: [rows+1] */
    int *cdColInd;       /*                [nnzCD], [0,dCols) dense space, then sparse space */
    void *cdVal;         /*                [nnzCD] */
} ora_partition;

float ora_h2f(uint16_t h);
uint16_t ora_f2h(float f);

void ora_spmv_f64(const double *val, const int *rowPtr, const int *colInd,
                  const double *x, double *y, int rows);
void ora_spmv_f16_f32acc(const uint16_t *val, const int *rowPtr, const int *colInd,
                         const uint16_t *x, float *y32, uint16_t *y16, int rows);
void ora_spmv_f16_halfacc(const uint16_t *val, const int *rowPtr, const int *colInd,
                          const uint16_t *x, uint16_t *y, int rows);
int ora_eqcheck_f64(const double *a, const double *b, int n, double tol);
int ora_eqcheck_f16(const uint16_t *a, const uint16_t *b, int n, float tol);

int ora_transpose(int elem, int outer, int inner, int nnz,
                  const int *ptr, const int *ind, const void *val,
                  int **tPtr, int **tInd, void **tVal);
int ora_threshold(int nnz, float frac);

ora_partition *ora_partition_create(int elem, int rows, int cols, int nnz,
                                    const int *rowPtr, const int *colInd, const void *val,
                                    float colProp, float rowProp);
void ora_partition_free(ora_partition *P);

void ora_tcspmv_f64(const double *x_d, double *y_d, const int *chunkPtr, const int *fragPtr,
                    const uint32_t *fragBit, const double *tcVal, const int *atox, int dRows);
void ora_tcspmv_f16(const uint16_t *x_d, float *y_d, const int *chunkPtr, const int *fragPtr,
                    const uint64_t *fragBit, const uint16_t *tcVal, const int *atox, int dRows);
void ora_hybrid_f64(const ora_partition *P, const double *x, double *y);
void ora_hybrid_f16(const ora_partition *P, const uint16_t *x, float *y);

uint64_t ora_hash(const void *p, size_t n, uint64_t h);
void ora_free(void *p);

#ifdef __cplusplus
}
#endif
#endif
