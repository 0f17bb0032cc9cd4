/*
 * matxtract_hip.h -- C ABI of libmatxtract_hip.so, the MI355X (gfx950) implementation of
 * MatXtract's hybrid SpMV path.
 *
 * Plain C: opaque handles, plain pointers and sizes, int status codes (0 = MX_OK), no C++
 * or torch types.  Every entry point names the reference interface it stands in for
 * (paths relative to the reference repository).  binary16 values cross this boundary as
 * their uint16_t bit pattern.
 *
 * Two groups:
 *   1. host-only: partition (the cascaded extraction), Matrix-Market ingest, transposes,
 *      synthetic workload generators.  Usable on a machine without a GPU.
 *   2. device: plans (persistent device copies of a partition) and the SpMV itself.
 *      These fail with MX_ERR_DEVICE when no HIP device is present; there is no CPU
 *      fallback.
 */
#ifndef MATXTRACT_HIP_H
#define MATXTRACT_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MX_OK 0
#define MX_ERR_ARG 1     /* bad argument (null pointer, negative size, tau_c < tau_r ...) */
#define MX_ERR_ALLOC 2   /* host or device allocation failed */
#define MX_ERR_DEVICE 3  /* HIP runtime error or no device */
#define MX_ERR_IO 4      /* file could not be opened / parsed */

typedef enum mx_dtype {
    MX_F64 = 0, /* binary64 values, binary64 accumulation, 8x4 tiles, 32-bit bitmaps */
    MX_F16 = 1  /* binary16 values, binary32 accumulation, 8x8 tiles, 64-bit bitmaps */
} mx_dtype;

/* The CSR triple of the reference (`valT *csrVal, indT *csrRowPtr, indT *csrColInd`,
 * include/common.h:53-79; produced by mmio_allinone, utilities/mmio.cpp:1547-1713). */
typedef struct mx_csr {
    int rows, cols, nnz;
    mx_dtype dtype;
    const int *rowPtr;  /* [rows+1] */
    const int *colInd;  /* [nnz], any order inside a row, duplicates allowed */
    const void *val;    /* [nnz] double | uint16_t(binary16) */
} mx_csr;

typedef struct mx_partition mx_partition; /* host result of the cascaded extraction */
typedef struct mx_plan mx_plan;           /* device-resident executable form */

/* Read-only view of the canonical partition arrays; names are the reference driver's
 * (test/test_autotc_spmv.cpp:1106-1492).  Pointers stay valid until the partition is
 * destroyed. */
typedef struct mx_partition_view {
    mx_dtype dtype;
    int rows, cols, nnz;
    int fragM, fragK;
    int dCols, sCols, nnzColD, nnzColS;
    int dRows, sRows, nnzRowD, nnzRowS;
    float cols_ratio;     /* dCols / cols, printed as "cols_ratio" (:1142) */
    double tc_nnz_ratio;  /* nnzRowD / (totalTcFrags*fragM*fragK), "TC_nnz_ratio" (:1376) */
    const int *descColId; /* [cols]  columns by nnz desc (ties: ascending id); NULL at tau=(0,0) */
    const int *newArray;  /* [sCols] columns not extracted, ascending */
    const int *rId;       /* [dRows] extracted rows, rank order */
    const int *newArray_; /* [sRows] rows not extracted, ascending */
    const int *ddRowPtr;  /* A_dd (dRows x dCols) as CSR */
    const int *ddColInd;
    const void *ddVal;
    int chunkNum, totalTcFrags, tcValCount;
    const int *chunkPtr;          /* [chunkNum+1] */
    const int *sparse_AToX_index; /* [totalTcFrags*fragK] */
    const int *fragPtr;           /* [totalTcFrags+1] */
    const void *fragBit;          /* [totalTcFrags] uint32_t (F64) | uint64_t (F16) */
    const void *tcVal;            /* [tcValCount] */
    int nnzCD;
    const int *cdRowPtr;  /* residual A_CD (rows x cols): columns [0,dCols) = dense-column */
    const int *cdColInd;  /* ranks, [dCols,cols) = dCols + index into newArray             */
    const void *cdVal;
    float tau_c, tau_r;   /* the fractions the partition was made with */
} mx_partition_view;

/* ---------------------------------------------------------------------------------- */
/* 1. host-only                                                                        */

/* Last error text of the calling thread ("" if none). */
const char *mx_last_error(void);

/* Cascaded compute-density extraction: column pass with tau_c (`global_col`), then row
 * pass with tau_r (`local_row`), tile format over A_dd, residual A_CD.  Stands in for the
 * code inlined in the reference driver's main(), test/test_autotc_spmv.cpp:1106-1427 and
 * merge2CSR_opt (:129-250), ecrPreprocess_opt1 (:502-585), generateFormat_opt[_fp16]
 * (:718-978).  tau_c < tau_r is rejected as the driver does (:1064-1069); tau=(0,0)
 * yields an empty tile part and A itself as residual (:1638-1658). */
int mx_partition_create(const mx_csr *A, float tau_c, float tau_r, mx_partition **out);
void mx_partition_destroy(mx_partition *p);
int mx_partition_get(const mx_partition *p, mx_partition_view *view);
/* 64-bit FNV-1a over the canonical arrays (dCols, dRows, descColId[0..dCols), newArray, rId,
 * newArray_, chunkPtr, sparse_AToX_index, fragPtr, fragBit, tcVal, cdRowPtr, cdColInd,
 * cdVal), little-endian, in that order. */
uint64_t mx_partition_hash(const mx_partition *p);

/* A partition on disk.  The file starts with the reference's "_preprocessed.dat" fields in its
 * own byte layout (written by test/tcpreprocess.cpp:1208-1255, read by test/tckernel.cpp:586-638:
 * chunkPtr, sparse_AToX_index, fragPtr, fragBit, tcVal -- so that tool reads the tile part of a
 * binary64 file unchanged) and goes on with what the reference does not store: sizes,
 * thresholds, the index maps, A_dd, the residual A_CD and a checksum.  mx_partition_load checks
 * the precision, every size and index range and the checksum; a file written by the reference
 * tool (tile part only) is refused with MX_ERR_IO and a message that says so. */
int mx_partition_save(const mx_partition *p, const char *path);
int mx_partition_load(const char *path, mx_dtype dtype, mx_partition **out);

/* csr2csc / csc2csr of utilities/csr2csc.cpp:4-203 as a host transpose: each output line
 * lists its entries by ascending source line, equal pairs in source order.  Outputs are
 * malloc()ed by the callee and released by the caller with free() or mx_free(), as in
 * the reference (csr2csc.cpp:15-17). `outer` = number of source lines (rows for csr2csc),
 * `inner` = number of output lines. */
int mx_transpose(mx_dtype dtype, int outer, int inner, int nnz, const int *ptr, const int *ind,
                 const void *val, int **tPtr, int **tInd, void **tVal);
void mx_free(void *p);

/* The same transpose on the device, as the reference runs it (csr2csc / csc2csr upload the
 * matrix, call cusparseCsr2cscEx2 and download the result, utilities/csr2csc.cpp:4-203) -- but
 * on arrays that already live in device memory and stay there.  Every pointer is a device
 * pointer; the caller provides tPtr_dev[inner + 1], tInd_dev[nnz] and tVal_dev[nnz].  The order
 * inside every output line is mx_transpose's (ascending source line, equal pairs in source
 * order), so both give the same arrays.  Scratch memory (about 16 bytes per entry plus the
 * sort's own) is allocated and released inside the call, which returns after `stream` (a
 * hipStream_t, or NULL) has finished the work.  MX_ERR_ARG when an index lies outside
 * [0, inner), MX_ERR_ALLOC / MX_ERR_DEVICE as elsewhere. */
int mx_transpose_device(mx_dtype dtype, int outer, int inner, int nnz, const int *ptr_dev, const int *ind_dev,
                        const void *val_dev, int *tPtr_dev, int *tInd_dev, void *tVal_dev, void *stream);

/* The two selections of the cascaded extraction, on a matrix that lives in device memory
 * (test/test_autotc_spmv.cpp:1122-1141 for the columns, :1240-1267 for the rows; the reference
 * counts through its transposes and sorts with qsort on the host):
 *   descColId_dev[cols] = the columns by entry count descending, ties by ascending column;
 *   dCols = the shortest prefix whose counts sum to >= (int)((float)nnz * tau_c), nnzColD its sum;
 *   descRowId_dev[rows] = the rows by their number of entries in those dCols columns, descending,
 *   ties by ascending row; dRows, nnzRowD likewise with tau_r (the first dRows are rId).
 * These are the values mx_partition_create derives on the host (a target out of reach selects
 * every line with a count above zero, as there).  rowPtr_dev, colInd_dev and both outputs are
 * device pointers; `out` is host memory.  Scratch is allocated and released inside; the call
 * returns after `stream` has finished. */
typedef struct mx_selection {
    int dCols, nnzColD, dRows, nnzRowD;
} mx_selection;
int mx_select_device(int rows, int cols, int nnz, const int *rowPtr_dev, const int *colInd_dev, float tau_c,
                     float tau_r, int *descColId_dev, int *descRowId_dev, mx_selection *out, void *stream);

/* The split that follows the selections (test/test_autotc_spmv.cpp:1286-1300 for A_dd,
 * :129-250 merge2CSR_opt for the residual), device arrays in and out.  With `sel`, descColId_dev
 * and descRowId_dev as mx_select_device left them:
 *   A_dd  = the dRows selected rows in rank order, their entries in selected columns, column =
 *           rank of the column, ascending (ddRowPtr_dev[dRows + 1], ddColInd_dev / ddVal_dev[nnzRowD]);
 *   A_CD  = every row in place: first its entries in unselected columns (column = dCols + position
 *           of the column among the unselected, ascending), then, for a row that was not selected,
 *           its entries in selected columns (cdRowPtr_dev[rows + 1], cdColInd_dev / cdVal_dev[nnz - nnzRowD]).
 * Entries that name the same row and column twice keep their source order.  The arrays equal
 * mx_partition_create's ddRowPtr .. cdVal.  The caller sizes the outputs from `sel`.  Everything
 * that is used as an address is looked at first: a rowPtr that does not rise from 0 to nnz, a
 * column id outside [0, cols), an entry of descColId[0, dCols) outside [0, cols) or of
 * descRowId[0, dRows) outside [0, rows), and a selection whose totals differ from the matrix's
 * are refused with MX_ERR_ARG.  Scratch (about 28 bytes per entry) is allocated and released inside. */
int mx_split_device(mx_dtype dtype, int rows, int cols, int nnz, const int *rowPtr_dev, const int *colInd_dev,
                    const void *val_dev, const mx_selection *sel, const int *descColId_dev, const int *descRowId_dev,
                    int *ddRowPtr_dev, int *ddColInd_dev, void *ddVal_dev, int *cdRowPtr_dev, int *cdColInd_dev,
                    void *cdVal_dev, void *stream);

/* The tile encoding of A_dd on the device (ecrPreprocess_opt1 test/test_autotc_spmv.cpp:502-585,
 * chunkPtr and sparse_AToX_index :1369-1404, generateFormat_opt :718-847 / _fp16 :849-978):
 * from A_dd as mx_split_device left it (rows sorted by column) to the arrays the tile kernels
 * read.  Per chunk of 8 rows: its distinct columns ascending (sparse_AToX_index, padded with
 * zeros to whole fragments of fragK = 4 (binary64) or 8 (binary16) columns); per fragment a
 * bitmap with bit r * fragK + c for an entry in local row r and compacted column c; tcVal in
 * ascending bit order, of entries naming the same place the last.  The arrays equal
 * mx_partition_create's.  A ddRowPtr that does not rise from 0 to nnzRowD or a column id outside
 * [0, dCols) is refused with MX_ERR_ARG before it is used.  The library allocates the outputs in
 * one block (device memory) and fills in `out`; mx_tiles_device_free releases the block. */
typedef struct mx_device_tiles {
    int chunkNum, totalTcFrags, fragK, tcValCount;
    int *chunkPtr;          /* [chunkNum + 1] */
    int *sparse_AToX_index; /* [totalTcFrags * fragK] */
    int *fragPtr;           /* [totalTcFrags + 1] */
    void *fragBit;          /* [totalTcFrags] uint32_t (binary64) or uint64_t (binary16) */
    void *tcVal;            /* [tcValCount] */
    void *base;             /* the block that holds them */
} mx_device_tiles;
int mx_tiles_device(mx_dtype dtype, int dRows, int dCols, int nnzRowD, const int *ddRowPtr_dev, const int *ddColInd_dev,
                    const void *ddVal_dev, mx_device_tiles *out, void *stream);
void mx_tiles_device_free(mx_device_tiles *t);

/* mx_partition_create by the device route: A (host arrays, as there) is uploaded and the three
 * steps above run on the device; the handle is the same kind of handle -- every array, count and
 * the checksum (mx_partition_hash) equal mx_partition_create's, so plans, files and callers cannot
 * tell the routes apart.  The arrays stay in device memory, held by the handle, until somebody asks
 * for them: mx_partition_get, mx_partition_hash and mx_partition_save copy them to the host first
 * (once); mx_plan_create makes its plan from them where they are and never asks, which is what
 * takes a caller of the reference's surface from the matrix to the first y in tens of milliseconds
 * instead of a second on the largest workload; mx_partition_counts gives the counts without the
 * arrays.  tau = (0, 0) extracts nothing and is handed to the host routine.  MX_ERR_DEVICE without a
 * HIP device: there is no silent fallback. */
int mx_partition_create_device(const mx_csr *A, float tau_c, float tau_r, mx_partition **out);
/* The counts of a partition (every field of the view that is not a pointer: the sizes, cols_ratio,
 * tc_nnz_ratio, the thresholds) without asking for its arrays; the pointers are filled in as well when the
 * arrays are in host memory already and are NULL otherwise. */
int mx_partition_counts(const mx_partition *p, mx_partition_view *view);

/* mmio_allinone (utilities/mmio.cpp:1547-1713): Matrix-Market coordinate file -> CSR with
 * entries kept in file order inside each row, symmetric/hermitian files expanded,
 * pattern files given value 1.  Outputs malloc()ed; returns MX_ERR_IO on failure. */
int mx_mmio_read(const char *path, mx_dtype dtype, int *rows, int *cols, int *nnz, int *isSymmetric,
                 int **rowPtr, int **colInd, void **val);

/* initVec (include/common.h:237-245): v[i] = (valT)(float)(i % 15). */
void mx_init_vec(mx_dtype dtype, void *v, int n);

/* binary16 <-> binary32, round to nearest even: the conversions behind CUDA's host-side
 * `half` that the reference's valT relies on (include/common.h:60). */
uint16_t mx_f32_to_f16(float f);
float mx_f16_to_f32(uint16_t h);

/* Synthetic workloads 1..5 (seeded; see mx_gen.cpp for the exact recipes).  `scale`
 * in (0,1] shrinks the row count (1 = full size).  Outputs malloc()ed: the matrix and
 * the input vector x.  The reference has no generators; these define the benchmark. */
int mx_gen_config(int config_id, uint64_t seed, double scale, int *rows, int *cols, int *nnz,
                  mx_dtype *dtype, int **rowPtr, int **colInd, void **val, void **x);
/* The same with variants of the recipes.  MX_GEN_UNALIGNED: the dense structure of workloads 2 and 5 off
 * the grid of eight columns -- a block of workload 2 starts at any column of its band, a strip of workload 5
 * at a column that is not a multiple of eight (the benchmark quotes the aligned form and reports this one
 * beside it).  gen_flags = 0 is mx_gen_config. */
#define MX_GEN_UNALIGNED 1
int mx_gen_config_ex(int config_id, uint64_t seed, double scale, int gen_flags, int *rows, int *cols, int *nnz,
                     mx_dtype *dtype, int **rowPtr, int **colInd, void **val, void **x);
/* Members of the families around workloads 2 and 5, for checking decisions away from the benchmark's own
 * matrices: dense_share is the share of the entries that sit in dense 8x8 blocks (workload 2; 0.4 in the
 * benchmark, up to 1) or the probability that a run of 128 rows is a strip (workload 5; 0.2 in the benchmark).
 * A negative share means the benchmark's; other workloads take no share. */
int mx_gen_config_family(int config_id, uint64_t seed, double scale, int gen_flags, double dense_share, int *rows, int *cols,
                         int *nnz, mx_dtype *dtype, int **rowPtr, int **colInd, void **val, void **x);

/* Algorithmic bytes of one SpMV: nnz*(sizeof(valT)+4) + (rows+1)*4 + cols*sizeof(valT) +
 * rows*sizeof(valT) (`data_origin1`, test/test_cdspmv.cpp:214). */
double mx_algorithmic_bytes(mx_dtype dtype, int rows, int cols, int nnz);

/* ---------------------------------------------------------------------------------- */
/* 2. device                                                                           */

/* Plan flags */
#define MX_PLAN_DEFAULT 0
#define MX_PLAN_NO_TILES 1   /* run the extracted block A_dd through the CSR kernel too */
#define MX_PLAN_ALL_TILES 2  /* run every extracted chunk through the MFMA tile kernel */
#define MX_PLAN_CSR_ROWS 4   /* CSR part: force the row-tile kernel (direct x gathers) */
#define MX_PLAN_CSR_SLICES 8 /* CSR part: prefer the column-slice kernel (x resident in LDS) when the matrix suits it */
#define MX_PLAN_KEEP_TILES 16 /* keep the tiles that the per-fragment fill gate selects.  Without this flag (and
                                 without MX_PLAN_ALL_TILES) a plan also asks whether the tiles pay for their
                                 own launch -- the entries they take off the CSR part against the bytes they
                                 stream themselves, at rates measured on MI355X -- and runs everything through
                                 the CSR part when they do not (the reference gates its tile kernel on matrix
                                 size and fill, test/test_autotc_spmv.cpp:1507,1518) */

#define MX_PLAN_NO_FUSE 32   /* CSR part in slice form: always two launches (csr_slice_kernel, then slice_combine_kernel).
                                 Without this flag a plan whose CSR part is the whole product takes the one-launch
                                 form (mx_plan_info.csr_fused) where the matrix suits it -- no row with more than eight
                                 virtual rows, at most 100 KB of sums under the busiest workgroup and at most eight slices of x
                                 (beyond that two launches are as fast or faster) -- and
                                 the device deals its workgroups round-robin to eight XCDs, which plan creation checks */
#define MX_PLAN_FUSE 64      /* the one-launch form wherever the matrix suits it, whatever its size */
#define MX_PLAN_KEEP 128     /* CSR part in slice form: read the entries with plain loads, so that a matrix that fits the L2s or the
                                 memory-side cache stays there from one product to the next (a solver that multiplies with the same
                                 matrix again and again).  Without this flag and MX_PLAN_STREAM the plan decides by size
                                 (mx_plan_info.csr_keep): plain loads where the entries fit the L2s, or fit the memory-side cache
                                 and the second launch moves enough to push streamed entries out of it */
#define MX_PLAN_STREAM 256   /* ... read them with streaming (non-temporal) loads whatever the size: 10-25 % faster when a
                                 product finds the caches cold, slower when the matrix could have stayed in them */

/* Uploads a partition once and keeps it on the device: the persistent counterpart of the
 * per-call cudaMalloc/cudaMemcpy blocks in cdspmv (src/spmv_kernel/cdSpMV.cu:407-418) and
 * du_tcspmv_fp64 (src/spmv_kernel/du_tcSpMV_fp64.cu:271-300), plus the x_d/x_s/x_CD
 * permutation of test/test_autotc_spmv.cpp:1454-1463 folded into the column indices so that
 * x and y are used in the caller's own ordering. */
int mx_plan_create(const mx_partition *p, int flags, mx_plan **out);
void mx_plan_destroy(mx_plan *plan);

/* A plan for y = A x from a CSR matrix that already lives in device memory (the counterpart of
 * mx_plan_create for the reference's tau = (0, 0) branch, test/test_autotc_spmv.cpp:1638-1658, where
 * the whole matrix is the CSR part; the reference always starts from host arrays and uploads them
 * on every call, src/spmv_kernel/cdSpMV.cu:407-418).  Every pointer is a device pointer; the arrays
 * are read during the call and may be released after it.  The layouts are built on the device from
 * the device arrays; of the matrix only the row pointers (row-tile form) or the lengths of its chunks
 * (slice form) cross to the host.  The form is chosen as in mx_plan_create, from the same counts taken
 * on the device: the plan, and with it every y, equals the one mx_plan_create makes from a partition
 * of the same matrix with tau = (0, 0).  rowPtr_dev and colInd_dev are checked on the device before
 * they are used as addresses (MX_ERR_ARG).  flags: MX_PLAN_CSR_ROWS, MX_PLAN_CSR_SLICES, MX_PLAN_NO_FUSE,
 * MX_PLAN_FUSE, MX_PLAN_KEEP, MX_PLAN_STREAM or 0.  For the one-launch form of the slices the records of the
 * virtual rows (slice and length of each) cross to the host as well, and its plan comes back; the entries stay.
 * Two things are laid out on the host, from a copy of the part that is brought down for it: the split form and
 * the timed choice that MX_CSR_KERNEL=split and MX_PLAN_AUTOTUNE=1 ask for. */
int mx_plan_create_device_csr(mx_dtype dtype, int rows, int cols, int nnz, const int *rowPtr_dev, const int *colInd_dev,
                              const void *val_dev, int flags, mx_plan **out);

/* The whole preparation of the reference's driver on the device, for a CSR matrix that lives in
 * device memory: the cascaded extraction with tau_c / tau_r (test/test_autotc_spmv.cpp:1099-1300),
 * the tile encoding (:1352-1421), and what mx_plan_create does with the result -- the fill gate of
 * the fragments, the search for rows of dense binary16 strips and their chunks, the question whether
 * the tiles pay, the CSR part in the caller's numbering with its layout, the strips' steps.  Nothing
 * of the matrix crosses to the host: decisions are made there from counts (fragments and entries
 * that pass the gate, blocks and entries per strip chunk, lengths of the slice layout's chunks).
 * The plan equals -- array for array, and so y bit for bit -- the one mx_plan_create makes from
 * mx_partition_create of the same matrix with the same fractions and flags, whatever tile forms it
 * keeps: the general form (the columns of a chunk's fragments sorted by the caller's ids with one radix
 * sort over all chunks, the values placed by the walk over A_dd that assembles the CSR part), the
 * binary16 strips, the binary64 8 x 8 blocks (one sort of (block row, block column) keys).  Every pointer is a
 * device pointer; the arrays are read during the call and may be released after it; rowPtr_dev and
 * colInd_dev are checked on the device before they are used as addresses (MX_ERR_ARG).
 * tau = (0, 0) is mx_plan_create_device_csr. */
int mx_plan_create_device(mx_dtype dtype, int rows, int cols, int nnz, const int *rowPtr_dev, const int *colInd_dev,
                          const void *val_dev, float tau_c, float tau_r, int flags, mx_plan **out);

/* The host's share of laying tiles out on the device, for inspection (no device needed): from the
 * number of blocks of every chunk alone, the steps of the layout -- a chunk of up to slots / 2 blocks
 * shares a step with the next such chunk, a larger one takes whole steps of its own -- and its waves,
 * exactly as mx_plan_layout lays the same chunks out.  stepDesc: 10 ints per step {chunk of half 0,
 * chunk of half 1 (-1 none, -2 the first goes on), flags, blocks in half 0, blocks in half 1, first
 * value, first value and blocks in half 0 of the step four further on, first block of half 0 inside
 * its chunk, 0}; chunkBlock0[nChunks]: first block of every chunk among the stored values; waveDesc: 8
 * ints per wave.  blockValues: values per block; perMin: fewest steps a wave takes.  No counterpart
 * in the reference, which walks its fragments in place. */
typedef struct mx_tile_steps_view {
    int steps, nWaves;
    long long totalBlocks;
    int *stepDesc, *chunkBlock0, *waveDesc;
} mx_tile_steps_view;
int mx_tile_steps(const int *chunkBlocks, int nChunks, int slots, int blockValues, int perMin, int nCU, mx_tile_steps_view *out);
void mx_tile_steps_free(mx_tile_steps_view *v);

/* Every device array of a plan copied to host memory, each with a name ("slices.ecol",
 * "strips.hdr", ...) and its size: for tests that hold two routes of making a plan against each
 * other.  `out` has room for `cap` entries (32 is enough); *n receives their number; the data
 * pointers are malloc()ed and mx_plan_arrays_free releases them.  No counterpart in the reference. */
typedef struct mx_plan_array {
    const char *name;
    size_t bytes;
    void *data;
} mx_plan_array;
int mx_plan_arrays(const mx_plan *plan, mx_plan_array *out, int cap, int *n);
void mx_plan_arrays_free(mx_plan_array *a, int n);

/* y = A*x on the device.  x [cols] and y [rows] are DEVICE pointers of the plan's value
 * type, x 16-byte aligned (the kernels copy it in 16-byte vectors; a plan whose CSR part keeps
 * x in LDS, or whose binary64 8 x 8 blocks read x in aligned pieces, returns MX_ERR_ARG otherwise,
 * before anything is launched, and reads the last 16-byte block of x whole when cols is
 * not a multiple of the vector -- the bytes past x[cols-1] in that block are read, never used);
 * `stream` is a hipStream_t (NULL = default stream).
 * Asynchronous.  The hybrid sequence of test/test_autotc_spmv.cpp:1507-1559 (tile part, scatter
 * through rId, residual accumulated on top) without host round trips.  A plan holds device
 * buffers of partial sums: calls on the same plan must not overlap in time. */
int mx_spmv(mx_plan *plan, const void *x_dev, void *y_dev, void *stream);

/* mx_spmv for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference, whose
 * compute calls allocate on every call (src/spmv_kernel/cdSpMV.cu:407-418).  Same arguments,
 * same kernels and bit-for-bit the same y as mx_spmv; the one buffer the kernels need beyond
 * the plan's arrays, x and y -- the sums of the virtual rows that csr_slice_kernel hands to
 * slice_combine_kernel -- lives in a fixed array of mx_static_scratch_bytes() (32 MiB) that is
 * part of the library's code object on every GPU it runs on (held until the process ends) and
 * is addressed through hipGetSymbolAddress once per device.  The call itself allocates
 * nothing, frees nothing and calls no allocating routine.  A plan whose sums need more than
 * the array holds is refused with MX_ERR_ARG and a message that says so (the largest benchmark
 * workload, the mixed one at full size, needs 27 MB and fits).  A plan in the one-launch form runs
 * its two-launch form here, whose sums are the ones that go to the array.  Every call on one GPU shares that GPU's array: calls that overlap in time
 * on one GPU -- also through different plans or streams -- race.  Nothing in the array has to
 * start at zero: every sum the second kernel reads is written by the first in the same call. */
int mx_spmv_static(mx_plan *plan, const void *x_dev, void *y_dev, void *stream);
int mx_static_scratch_bytes(void);

/* For tests of the one-launch form's way out (no counterpart in the reference).  A one-launch product
 * relies on the device dealing the workgroups of a launch round-robin to its eight XCDs (a workgroup takes
 * its share of the work by the XCD it runs on and its number / 8); every launch checks that no share is taken
 * twice, and a workgroup that finds its share taken sets a word in host memory.  The next product of any
 * one-launch plan then returns MX_ERR_DEVICE once (the products since the previous call may be wrong) and every
 * plan of the process takes the two-launch form from there on.  mx_debug_fused_misplaced(1) sets that word from
 * the host, as such a workgroup would; (0) clears it and lets new plans take the one-launch form again. */
int mx_debug_fused_misplaced(int set);

/* n back-to-back SpMVs y = A*x on `stream`, queued from C without returning to the caller in
 * between: the reference's timed loops (src/spmv_kernel/cdSpMV.cu:464-469) as an entry point,
 * for callers whose per-call overhead (an interpreter, an FFI hop) would otherwise sit
 * between launches.  Asynchronous. */
int mx_spmv_repeat(mx_plan *plan, const void *x_dev, void *y_dev, int n, void *stream);

/* Same as mx_spmv with HOST pointers (allocates nothing persistent; copies x in and y out). */
int mx_spmv_host(mx_plan *plan, const void *x_host, void *y_host);

/* The reference's timing protocol (200 warm-ups + 4000 timed back-to-back launches,
 * src/spmv_kernel/cdSpMV.cu:454-479, du_tcSpMV_fp64.cu:311-333) on the plan's own stream.
 * ms_total: mean per SpMV of the whole sequence (hipEvents around the loop);
 * ms_tile / ms_csr: the tile part and the CSR part timed on their own (the two numbers the reference adds
 * up, test/test_autotc_spmv.cpp:1561-1572).  Where strips or 8 x 8 blocks ride in the combine kernel's launch
 * there is no tile launch to time: ms_csr is then the CSR part's launches as the product runs them, riders
 * included, and ms_tile what the riders add (the same launches without them taken off); binary64 blocks in a
 * launch of their own are priced the same way, as the pair less the CSR part, so that y never grows.  Any
 * may be NULL.  MX_ERR_ARG for an x the plan cannot take (see mx_spmv), before anything is launched. */
int mx_time(mx_plan *plan, const void *x_dev, void *y_dev, int warm, int iters,
            double *ms_total, double *ms_tile, double *ms_csr);

/* The protocol of mx_time on a train of products that takes the `n` plans in turn (product k runs
 * plans[k % n] on x_dev[k % n] into y_dev[k % n], all on the first plan's stream): with n copies of one
 * plan whose arrays add up to several times the 256 MB memory-side cache, no product finds any of its
 * arrays in a cache, which is what a solver sees whose matrix is larger than that cache -- the
 * reference's loops (src/spmv_kernel/cdSpMV.cu:464-469) always re-run one matrix.  ms = mean per product. */
int mx_time_rotate(mx_plan *const *plans, const void *const *x_dev, void *const *y_dev, int n, int warm, int iters, double *ms);

/* Mean ms per launch of the CSR part's main kernel alone (csr_rows_kernel, or csr_slice_kernel
 * without its combine kernel), same protocol as mx_time: the figure a roofline is priced on. */
int mx_time_csr_main(mx_plan *plan, const void *x_dev, void *y_dev, int warm, int iters, double *ms);

/* Every kernel launch of one product, timed alone with the protocol of mx_time, in launch order,
 * each with its share of the algorithmic bytes (the shares add up to mx_algorithmic_bytes of the
 * matrix: entries go to the kernel that multiplies them, x to the first kernel that reads it, the
 * row structure and y to the kernel that writes y).  The reference times its two kernels apart
 * in the same way (test/test_autotc_spmv.cpp:1561-1572).  Up to `cap` records; *n_kernels = how many. */
typedef struct mx_kernel_time {
    char name[64];            /* e.g. "csr_slice_kernel<f16>", "slice_combine_kernel<f16,strips>" */
    double ms;                /* mean per launch */
    double algorithmic_bytes; /* this kernel's share */
    int nnz;                  /* matrix entries this kernel multiplies */
    int reserved;
} mx_kernel_time;
int mx_time_kernels(mx_plan *plan, const void *x_dev, void *y_dev, int warm, int iters, mx_kernel_time *out, int cap,
                    int *n_kernels);

/* Choice of (tau_c, tau_r) for a matrix on this device.  The reference tunes the two fractions
 * per matrix by running its CLI once per candidate and reading "MatXtract time" back
 * (ML/bayes_opt.py:22-84: candidates with hot_frac > col_frac are rejected, :37-38); here the
 * candidates are the `levels` x `levels` grid {0, 1/(levels-1), .. 1}^2 with tau_c >= tau_r, each
 * one partitioned, planned (with `flags`) and timed on the device with the protocol of mx_time
 * (`warm` untimed and `iters` timed back-to-back products of a seeded x).  Candidates that send
 * nothing to the tile kernel are one and the same plan and are timed once, as (0, 0).  A matrix of
 * two million entries or more is uploaded once and every candidate's extraction and plan are made
 * on the device (mx_plan_create_device: the same plans).
 * Returns the fastest in tau_c/tau_r; when `table` is given, up to `cap` candidates are written
 * to it in grid order (tau_c outer, ascending) and *n_points is set to their number. */
typedef struct mx_tau_point {
    float tau_c, tau_r;
    double ms_total;  /* mean ms per product */
    int tile_nnz;     /* entries the tile kernel holds at this point */
} mx_tau_point;
int mx_tune_tau(const mx_csr *A, int levels, int flags, int warm, int iters, float *tau_c, float *tau_r,
                mx_tau_point *table, int cap, int *n_points);

/* The same choice from counts alone, nothing planned or timed: for every point of that grid the
 * extraction runs on the device and the estimate a plan makes of its own tiles -- the entries they
 * take off the CSR part against their launch and their own stream, at rates measured on MI355X -- is
 * read off; the point whose tiles save most wins, (0, 0) when none saves anything.  The reference's
 * counterpart is the regression model of ML/train_*.py over the count features of
 * ML/extract_features.cpp:31-95, queried through ML/bayes_opt.py; here the features are the counts the
 * plan itself decides from (fragments and entries that pass the fill gate, strip chunks, 8 x 8
 * blocks).  A host matrix is uploaded once.  `table` as in mx_tune_tau. */
typedef struct mx_tau_estimate {
    float tau_c, tau_r;
    double saved_us;         /* estimated microseconds per product that the kept tile forms save (0: none kept) */
    long long tile_entries;  /* entries those forms would hold */
} mx_tau_estimate;
int mx_estimate_tau(const mx_csr *A, int levels, float *tau_c, float *tau_r, mx_tau_estimate *table, int cap, int *n_points);

/* Facts about a plan, for reporting. */
typedef struct mx_plan_info {
    mx_dtype dtype;
    int rows, cols, nnz;
    int tile_chunks;     /* chunks executed by the MFMA tile kernel */
    int tile_frags;      /* fragments executed by the MFMA tile kernel */
    int tile_nnz;        /* matrix entries held in those fragments */
    int csr_nnz;         /* entries executed by the CSR kernel */
    int csr_blocks;      /* workgroups of the CSR kernel */
    int csr_variant;     /* 0 = row tiles (csr_rows_kernel), 1 = column slices (csr_slice_kernel),
                            2 = row tiles for the short rows, then column slices for the long ones */
    double tile_bytes;   /* bytes the tile kernel must read+write per launch */
    double csr_bytes;    /* bytes the CSR kernel must read+write per launch */
    int csr_main_kernel; /* the CSR-part kernel that holds most entries (the one mx_time_csr_main times):
                            0 = csr_rows_kernel, 1 = csr_slice_kernel */
    int csr_main_nnz;    /* entries that kernel holds */
    int tile_variant;    /* 1 when part of the tiles runs through tile_dense_kernel: binary16 rows whose columns
                            fill at most 8 blocks of 8 consecutive columns at least half (a row of a dense strip in
                            the simplest case; the blocks start at multiples of eight or, where that takes fewer
                            blocks, at the row's own first column plus multiples of eight, so a strip may start at
                            any column), with nothing in the residual and no column named twice; the plan
                            groups rows with the same blocks, 8 at a time, into chunks of its own (at least 4
                            rows each) and takes them out of the reference's fragments.  MX_NO_STRIPS=1 in the
                            environment switches this off; with an x that is not 16-byte aligned these chunks
                            run through tile_kernel.
                            2: a binary64 plan whose tiles are aligned blocks of 8 x 8 (eight consecutive rows
                            from a multiple of eight, eight consecutive columns from a multiple of eight, in the
                            caller's numbering, at least three quarters full) found in the extracted block and
                            run through v_mfma_f64_16x16x4_f64 with x read in aligned 16-byte pieces; their rows
                            keep their other entries in the CSR part, and with the slice form of that part the
                            blocks ride in the combine kernel's launch (MX_NO_BLOCKS=1 switches the form off) */
    int tile_strip_nnz;  /* entries held by those chunks */
    int csr_value_dict;  /* > 0: the main kernel of the CSR part reads one byte per entry, an index into this many
                            distinct values (matrices with at most 255 of them: stencils, graphs); 0: values as
                            they are.  MX_CSR_DICT=0 switches the form off */
    double est_rows_us;  /* what the choice between row tiles and slices was made from: the estimated microseconds */
    double est_slices_us;/* per product through either form, from counts over the matrix and rates measured on
                            MI355X (both 0 when a flag, MX_CSR_KERNEL or the shape of the matrix left no choice).
                            Nothing is timed unless MX_PLAN_AUTOTUNE=1 is set, so a matrix gets the same plan on
                            every run */
    int prep_route;      /* where the plan's layouts were made: 0 = from host arrays (mx_plan_create), 1 = on the
                            device from device arrays (mx_plan_create_device, mx_plan_create_device_csr) */
    int ext_dCols, ext_dRows, ext_nnzRowD, ext_frags; /* what the extraction behind the plan selected (columns, rows,
                            entries of A_dd) and the fragments of its tile encoding -- cols_ratio and TC_nnz_ratio of
                            the reference's driver follow from them; 0 for plans without an extraction */
    int csr_fused;       /* 1: the CSR part in slice form runs as ONE launch (the reference's residual kernel is one
                            launch too, src/spmv_kernel/cdSpMV.cu:459): the workgroups that hold sums of the same rows
                            sit on one XCD, count themselves off on a counter in that XCD's L2, and the one that
                            completes the count adds the sums up and writes y; nobody waits.  0: two launches */
    int opt_flags;       /* MX_OPT_* bits: the switches of the environment that were set when the plan was made.  The
                            library reads the environment when a plan or layout is created and never while a plan
                            runs; a plan made under one setting keeps it whatever the environment says later */
    double opt_tile_gate;/* the fill a fragment needed for the tile kernels when the plan was made (MX_TILE_GATE;
                            one half unless set) */
    int csr_keep;        /* 1: the slice kernel reads the entries with plain loads (they may stay in the caches between
                            products), 0: it streams them (MX_PLAN_KEEP / MX_PLAN_STREAM, MX_CSR_KEEP, or the plan's own
                            choice by size) */
    double touched_bytes;/* what one product touches in device memory as the plan stores it (entries in their stored form,
                            sums, row tables, tile part, x, y): what has to fit a cache for the matrix to stay in it.  The
                            algorithmic bytes of the matrix count a value and a 4-byte column per entry whatever is stored */
} mx_plan_info;
/* mx_plan_info.opt_flags */
#define MX_OPT_NO_STRIPS 1     /* MX_NO_STRIPS=1: no binary16 strip chunks */
#define MX_OPT_NO_BLOCKS 2     /* MX_NO_BLOCKS=1: no binary64 8 x 8 blocks */
#define MX_OPT_NO_DICT 4       /* MX_CSR_DICT=0: values as they are, also where at most 255 distinct ones exist */
#define MX_OPT_STRIPS_APART 8  /* MX_STRIPS_APART=1: binary16 strips in a launch of their own */
#define MX_OPT_CSR_KERNEL 16   /* MX_CSR_KERNEL=rows|slices|split named the form of the CSR part */
#define MX_OPT_CSR_FUSED 32    /* MX_CSR_FUSED=0|1 decided about the one-launch form */
#define MX_OPT_AUTOTUNE 64     /* MX_PLAN_AUTOTUNE=1: forms were timed, not estimated (the plan may differ run to run) */
#define MX_OPT_LAYOUT_HOST 128 /* MX_LAYOUT=host: layouts made on the host where the device route exists (same arrays) */
#define MX_OPT_CSR_KEEP 512    /* MX_CSR_KEEP=0|1 decided how the slice kernel reads its entries */
#define MX_OPT_TUNING 256      /* one of the tuning knobs was set: MX_SLICE_CAP, MX_SPLIT_LEN, MX_CSR_NPT, MX_TILE_PER,
                                  MX_CSR_REDUCE, MX_CSR_COL16 */
int mx_plan_get_info(const mx_plan *plan, mx_plan_info *info);

/* The layout csr_slice_kernel runs on, built on the host for a machine with `nCU` compute units,
 * for inspection (tests walk it the way the kernel does; nothing here touches a device).  `sel`
 * marks the rows to include (NULL = all).  No counterpart in the reference, whose CSR kernel
 * (src/spmv_kernel/cdSpMV.cu:29-393) gathers x from global memory.
 *   wgDesc    [nWG][4]  {slice, first chunk, chunks, 0}
 *   waveDesc  [nWG*waves][4] {first batch, batches, first chunk inside the workgroup, chunks}
 *   chunkEnd  [chunks]  step, counted from the wave's first, at which the chunk ends
 *   ecol      [batches][64][batchEntries] column - slice*sliceCols
 *   eval      per batch: binary16 [64][batchEntries]; binary64 [batchEntries/2][64][2]
 *   a lane takes stepEntries (= 1) entries per step; chunkEnd counts steps
 *   virtual row v = 64*chunk + lane; matrix row r owns segIdx[segPtr[r] .. segPtr[r+1])
 *   rowInfo   [rows] the virtual row of a row that owns exactly one; -1 for none, -2 for several
 *   lightInfo [nLight][4] {row, segPtr[row], count, 0} of the rows with 2..lightSegs virtual rows
 *   heavyInfo [nHeavy][4] the same for the rows with more
 * Release with mx_slice_layout_free. */
typedef struct mx_slice_layout_view {
    int nWG, S, sliceCols, waves, stepEntries, batchEntries, cap, chunks, batches, vrows, nLight, nHeavy, lightSegs;
    long long nEcol;
    int *wgDesc, *waveDesc, *chunkEnd, *segPtr, *segIdx, *rowInfo, *lightInfo, *heavyInfo;
    unsigned short *ecol;
    unsigned char *eval;
    int nDict;            /* > 0: the value dictionary form exists beside the values (at most 255 distinct values) */
    unsigned char *ecode; /* [nEcol] one byte per entry, at the place of its column offset; 255 = the padding's zero */
    unsigned char *dict;  /* [256] values (binary64 or binary16), zeros beyond nDict */
    /* the one-launch form (mx_slice_layout_fused; all zero otherwise): rows in groups of groupRows, virtual rows
     * ordered by (slice, group, length), workgroup b (of nWG = nCU, in the numbering of wgDesc) belongs to XCD
     * b * 8 / nWG and bumps the counters of groups wgGroups[b] = {first, count}; groupNeed[g] = how many
     * workgroups bump group g; fusedTarget[64 * chunk + lane] = where that virtual row puts its sum: the k-th
     * virtual row of row r at ((r / groupRows) * placesPerRow + k) * groupRows + r % groupRows (padding lanes
     * at nGroups * placesPerRow * groupRows + lane); rowVrows[r] = virtual rows of row r */
    int fused, groupRows, nGroups, placesPerRow;
    int *wgGroups, *groupNeed, *fusedTarget;
    unsigned char *rowVrows;
} mx_slice_layout_view;
int mx_slice_layout(const mx_csr *A, int nCU, const unsigned char *sel, mx_slice_layout_view *out);
/* The layout of the one-launch form for the whole matrix (out->fused = 1), or the ordinary one
 * (out->fused = 0) when the matrix does not suit it: a row with more than eight virtual rows, more
 * slices with entries in an XCD's rows than the XCD has workgroups, or more chunks in a workgroup
 * than it can keep the targets of in LDS. */
int mx_slice_layout_fused(const mx_csr *A, int nCU, mx_slice_layout_view *out);
/* The same view by the route plans take for a whole matrix: A goes up, the layout is built on the
 * device from the device arrays (sorts, running sums and placement kernels; only the assignment of
 * chunks to workgroups and waves, a few values per thousand entries, is decided on the host, by the
 * routine both routes share) and comes down.  Every array equals mx_slice_layout's (sel = NULL) byte
 * for byte.  MX_ERR_DEVICE without a HIP device. */
int mx_slice_layout_device(const mx_csr *A, int nCU, mx_slice_layout_view *out);
void mx_slice_layout_free(mx_slice_layout_view *v);

/* The host half of a plan for a partition, for inspection and tests on a machine without a GPU
 * (no counterpart in the reference, where these decisions are inline in main(),
 * test/test_autotc_spmv.cpp:1486-1559): the CSR part in the caller's numbering (the residual plus
 * every entry of the extracted block that the tile kernels do not take; for a partition with
 * tau = (0,0) the matrix itself), and up to two tile layouts as the kernels read them -- [0] for
 * tile_kernel, [1] the plan's own chunks of 8-column blocks (binary16 strips for tile_dense_kernel,
 * binary64 8 x 8 blocks for tile_block_wave: four block slots per half, slot 4h+i, blocks 8 x 8).  Per step: hdr[32] ints (output rows
 * [0,16) of the two halves, -1 = none; [16] flags: 1 = the sums are stored after this step, 2 = the
 * halves belong to two chunks; [17],[18] blocks in half 0 and 1; [21,29) first column per slot in
 * the strip layout), atox[64] column ids (slot-major, -1 = unused; block i of half h sits in
 * slot 2i+h of a binary64 step and in slot 4h+i of a binary16 step), and the blocks' values in
 * `val` from valOffset[step] on (elements): the blocks of half 0, then of half 1, each
 * fragM x fragK row-major.  `nCU` sizes the waves (waveDesc[nWaves][8] = {first step, end step,
 * ...}).  Release with mx_plan_layout_free. */
typedef struct mx_tile_layout_view {
    int steps, nWaves, chunks, nnz, dense;
    long long nVal; /* elements in val */
    int *hdr, *atox, *waveDesc, *valOffset;
    unsigned char *val;
} mx_tile_layout_view;
typedef struct mx_plan_layout_view {
    int rows, cols, csr_nnz, fragM, fragK, slots; /* slots: block slots of a step (two halves of slots/2) */
    int *csrRowPtr, *csrColInd;
    unsigned char *csrVal;
    unsigned char *stripRows; /* [rows] 1 = the row is written by the strip layout alone (binary16); 2 = the row's sums from
                                 the CSR part and from the 8 x 8 blocks of tiles[1] are added (binary64) */
    mx_tile_layout_view tiles[2];
    int csr_variant;     /* the form mx_plan_create would give the CSR part on a device with nCU compute units:
                            0 row tiles, 1 slices, 2 split; -1 when MX_PLAN_AUTOTUNE=1 leaves it to a timed trial */
    double est_rows_us, est_slices_us; /* the estimates behind that choice (mx_plan_info) */
} mx_plan_layout_view;
int mx_plan_layout(const mx_partition *P, int flags, int nCU, mx_plan_layout_view *out);
void mx_plan_layout_free(mx_plan_layout_view *v);

/* Reference surface, host pointers in / host pointers out, one-shot (allocate, upload,
 * `warm` + `iters` timed launches into a scratch y, one real launch, download, free).
 * The C++ functions of include/MatXtract.h are inline wrappers over these.
 *
 * mx_cdspmv_*: cdspmv(), include/MatXtract.h:3-5, src/spmv_kernel/cdSpMV.cu:395-491.
 *   y is IN/OUT: y += A*x.  cdTime = mean ms per launch, cdPre = ms spent building the
 *   workgroup row map (the reference's pre_startRowPerBlock). */
int mx_cdspmv_f64(const double *csrVal, const int *csrRowPtr, const int *csrColInd, const double *x,
                  double *y, int rows, int cols, int nnz, int warm, int iters, double *cdTime,
                  double *cdPre);
int mx_cdspmv_f16(const uint16_t *csrVal, const int *csrRowPtr, const int *csrColInd,
                  const uint16_t *x, uint16_t *y, int rows, int cols, int nnz, int warm, int iters,
                  double *cdTime, double *cdPre);
/* mx_du_tcspmv_f64: du_tcspmv_fp64(), include/MatXtract.h:7-9,
 *   src/spmv_kernel/du_tcSpMV_fp64.cu:258-350.  y is IN/OUT (y += A_dd*x_d).
 * mx_du_tcspmv_f16: du_tcspmv_fp16_v2(), include/MatXtract.h:27-29,
 *   src/spmv_kernel/du_tcSpMV_fp16_v2.cu:112-203.  y is overwritten. */
int mx_du_tcspmv_f64(const int *chunkPtr, const int *fragPtr, const uint32_t *fragBit,
                     const double *tcVal, const int *sparse_AToX_index, const double *x_d, double *y_d,
                     int dRows, int dCols, int warm, int iters, double *tcTime);
int mx_du_tcspmv_f16(const int *chunkPtr, const int *fragPtr, const uint64_t *fragBit,
                     const uint16_t *tcVal, const int *sparse_AToX_index, const uint16_t *x_d,
                     uint16_t *y_d, int dRows, int dCols, int warm, int iters, double *tcTime);

/* Number of HIP devices visible (0 when none; never fails). */
int mx_device_count(void);

/* Diagnostics: one MFMA on one wave with raw per-lane operands, so a test can pin the
 * operand layout the tile kernels assume.  f64 (v_mfma_f64_16x16x4_f64): A[64], B[64] one
 * value per lane, D[64][4] the four accumulator registers of each lane.  f16
 * (v_mfma_f32_16x16x32_f16): A[64][8], B[64][8] binary16, D[64][4] binary32.  HOST arrays.
 * No counterpart in the reference. */
int mx_probe_mfma_f64(const double *A, const double *B, double *D);
int mx_probe_mfma_f16(const uint16_t *A, const uint16_t *B, float *D);

#ifdef __cplusplus
}
#endif
#endif /* MATXTRACT_HIP_H */
