// Internal declarations shared by the translation units of libmatxtract_hip.so.
#pragma once
#include <cstddef>
#include <cstdint>
#include <string>
#include <vector>

#include "matxtract_hip.h"

namespace mx {

inline int elem_size(mx_dtype d) { return d == MX_F64 ? 8 : 2; }
inline int frag_k(mx_dtype d) { return d == MX_F64 ? 4 : 8; }
constexpr int kFragM = 8;

void set_error(const std::string &msg);

// Every switch the library takes from the environment, read in one place (refresh_options, which the
// entry points that make plans and layouts call first) and looked at through opt() from there on; a plan
// keeps the ones that change what it computes or how (mx_plan_info.opt_flags, opt_tile_gate).
struct Options {
    double tile_gate = -1.0;  // MX_TILE_GATE=<fraction>: fill a fragment needs for the tile kernels; -1 = the default (one half)
    int csr_dict = 1;         // MX_CSR_DICT: 0 = never one byte per value; 1 = wherever at most 255 values exist; 2 = also against a timed choice
    bool no_strips = false;   // MX_NO_STRIPS=1: no binary16 strip chunks
    bool no_blocks = false;   // MX_NO_BLOCKS=1: no binary64 8 x 8 blocks
    bool strips_apart = false;// MX_STRIPS_APART=1: strips in a launch of their own instead of the combine kernel's
    int csr_kernel = 0;       // MX_CSR_KERNEL=rows|slices|split: 1 | 2 | 3; 0 = the plan decides
    int csr_fused = -1;       // MX_CSR_FUSED: 0 = never the one-launch form, 1 = wherever the matrix suits it; -1 = the plan decides
    int csr_keep = -1;        // MX_CSR_KEEP: 0 = the slice kernel streams its entries, 1 = it reads them with plain loads; -1 = the plan decides
    bool autotune = false;    // MX_PLAN_AUTOTUNE=1: the forms of the CSR part are timed on the spot instead of estimated
    bool layout_host = false; // MX_LAYOUT=host: layouts on the host also where the device route exists
    int slice_cap = 0;        // MX_SLICE_CAP=<entries>: longest virtual row (tuning runs); 0 = a lane's fair share
    int split_len = 0;        // MX_SPLIT_LEN=<entries>: shortest row the split form sends to the slices; 0 = 32
    int csr_npt = 0;          // MX_CSR_NPT: entries per lane and tile of the row kernel; 0 = the default
    int tile_per = 0;         // MX_TILE_PER: steps per wave of the tile kernels; 0 = by the size
    int csr_reduce = 0;       // MX_CSR_REDUCE=rows|scan: 1 | 2; 0 = by the spread of the row lengths
    bool csr_col16 = true;    // MX_CSR_COL16=0: never 16-bit column offsets in the row kernel
    bool plan_log = false;    // MX_PLAN_LOG=1: phase times of plan creation on stderr
};
const Options &opt();
void refresh_options();

// `int dColsNnz = nnzA * colProp;` (test/test_autotc_spmv.cpp:1131, :1249): int * float is a float
// product, truncated.
inline int threshold(int nnz, float frac)
{
    float t = (float)nnz * frac;
    if (t >= 2147483648.0f) return 2147483647;
    return (int)t;
}

// double -> binary16 bits, round to nearest even, straight from the double (no
// intermediate float rounding); binary16 bits -> float.
uint16_t f64_to_f16_bits(double v);
float f16_bits_to_f32(uint16_t h);

// Raw byte buffer holding matrix values of either type.
struct ValBuf {
    std::vector<unsigned char> bytes;
    void resize(size_t n, int elem) { bytes.assign(n * (size_t)elem, 0); }
    void *data() { return bytes.data(); }
    const void *data() const { return bytes.data(); }
};

}  // namespace mx

// Host result of the cascaded extraction; arrays named as in the reference driver.
struct mx_partition {
    mx_dtype dtype = MX_F64;
    int rows = 0, cols = 0, nnz = 0;
    int fragM = 8, fragK = 4;
    float tau_c = 0.f, tau_r = 0.f;
    int dCols = 0, sCols = 0, nnzColD = 0, nnzColS = 0;
    int dRows = 0, sRows = 0, nnzRowD = 0, nnzRowS = 0;
    float cols_ratio = 0.f;
    double tc_nnz_ratio = 0.0;
    bool extracted = false;  // false at tau = (0,0)
    std::vector<int> descColId, newArray, rId, newArray_;
    std::vector<int> ddRowPtr, ddColInd;
    mx::ValBuf ddVal;
    int chunkNum = 0, totalTcFrags = 0, tcValCount = 0;
    std::vector<int> chunkPtr, sparse_AToX_index, fragPtr;
    std::vector<uint64_t> fragBit64;  // F16
    std::vector<uint32_t> fragBit32;  // F64
    mx::ValBuf tcVal;
    int nnzCD = 0;
    std::vector<int> cdRowPtr, cdColInd;
    mx::ValBuf cdVal;
    // A partition made on the device (mx_partition_create_device) keeps its arrays there: `twin` owns them and is
    // released with the partition.  The vectors above are filled from them when somebody asks for the arrays
    // (mx::partition_host); until then only the counts are set and host_ready is false.  A plan made from such a
    // partition works on the device arrays and never asks.
    bool host_ready = true;
    void *twin = nullptr;
    int (*twin_download)(mx_partition *) = nullptr;
    void (*twin_free)(void *) = nullptr;
    mx_partition() = default;
    mx_partition(const mx_partition &) = delete;
    mx_partition &operator=(const mx_partition &) = delete;
    ~mx_partition()
    {
        if (twin && twin_free) twin_free(twin);
    }
};

namespace mx {
// The argument checks of mx_partition_create (null pointers, shape, tau range and order, rowPtr
// monotone over [0, nnz], column range); *out is cleared.
int check_partition_args(const mx_csr *A, float tau_c, float tau_r, mx_partition **out);
// The arrays of `p` in host memory: copies them down first when they still live on the device only.
int partition_host(const mx_partition *p);
}  // namespace mx
