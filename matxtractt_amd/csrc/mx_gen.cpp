// Seeded synthetic workloads.  The reference ships no generators (it reads SuiteSparse
// .mtx files and overwrites their values, test/test_autotc_spmv.cpp:1090-1091); these
// recipes define the five benchmark matrices.
//
// One generator everywhere: xoshiro256** seeded through splitmix64; the default seed of
// workload k is 0x9E3779B97F4A7C15 ^ k.  uniform[-1,1] = 2*(u53/2^53) - 1; binary16 values
// are that double rounded to nearest even.  Every row lists distinct columns in ascending
// order.  `scale` in (0,1] shrinks the number of rows (tests use small scales).
//
//  1  random            n = 4096*scale, 16 distinct uniform columns per row, f64.
//  2  block-clustered   n = 65536*scale, 64 entries per row.  floor(0.4*n) dense 8x8 blocks:
//                       block row uniform, block column uniform in the band
//                       [r/8-128, r/8+127] (clipped), no two blocks overlapping, at most 8 per
//                       block row.  Every row is then filled up to 64 entries with distinct
//                       uniform columns.  f64.
//  3  27-point stencil  g^3 grid, g = round(100*cbrt(scale)); row = x + g*(y + g*z); the 27
//                       neighbours inside the grid; centre 26, others -1; x uniform[0,1]. f64.
//  4  power-law         n = 1048576*scale.  Row length L = clip(floor(s*U^(-1/0.6)), 1, Lmax)
//                       (tail exponent of Zipf(1.6)), Lmax = min(4096, n/2), s solved so that the
//                       mean is 10.  Each row has a uniform locality centre; every entry is
//                       drawn, with probability 0.7, from centre +- 512 (clipped), otherwise
//                       uniformly; duplicates are redrawn (uniformly after 8 attempts). f16.
//  5  mixed             n = 4194304*scale.  Runs of 128 rows are "strips" with probability
//                       0.2: each 8-row block of a strip holds 32 consecutive columns starting
//                       at 8*(block + off), off uniform in [-32,32] per strip (clipped) -- a
//                       dense 8x32 block sliding along the diagonal.  All other rows are
//                       power-law rows as in 4. f16.
//
// MX_GEN_UNALIGNED (mx_gen_config_ex) takes the dense structure of workloads 2 and 5 off the grid of
// eight columns: a block of workload 2 starts at any column of the band [r - 1024, r + 1024 - 8]
// (its eight rows still start at a multiple of eight; blocks of one block row do not overlap), and a
// strip of workload 5 starts at 8*(block + off) + shift with shift uniform in [1, 7] per strip.
// Everything else is drawn as before.
//
// mx_gen_config_family varies how much of the matrix is dense structure: the share of the entries that
// sit in 8x8 blocks (workload 2, 0.4 in the benchmark) or the probability that a run of 128 rows is a
// strip (workload 5, 0.2 in the benchmark).
#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "mx_internal.h"

namespace {

struct Rng {
    uint64_t s[4];
    explicit Rng(uint64_t seed)
    {
        for (int i = 0; i < 4; ++i) {  // splitmix64
            uint64_t z = (seed += 0x9E3779B97F4A7C15ull);
            z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
            z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
            s[i] = z ^ (z >> 31);
        }
    }
    static uint64_t rotl(uint64_t x, int k) { return (x << k) | (x >> (64 - k)); }
    uint64_t next()
    {
        const uint64_t result = rotl(s[1] * 5, 7) * 9;
        const uint64_t t = s[1] << 17;
        s[2] ^= s[0];
        s[3] ^= s[1];
        s[1] ^= s[2];
        s[0] ^= s[3];
        s[2] ^= t;
        s[3] = rotl(s[3], 45);
        return result;
    }
    double u01() { return (double)(next() >> 11) * (1.0 / 9007199254740992.0); }
    double sym() { return 2.0 * u01() - 1.0; }
    int below(int n) { return (int)(((unsigned __int128)next() * (unsigned __int128)(uint64_t)n) >> 64); }
};

struct Builder {
    mx_dtype dtype;
    std::vector<int> rowPtr{0}, colInd;
    std::vector<double> v64;
    std::vector<uint16_t> v16;
    void push(int col, double v)
    {
        colInd.push_back(col);
        if (dtype == MX_F64)
            v64.push_back(v);
        else
            v16.push_back(mx::f64_to_f16_bits(v));
    }
    void end_row() { rowPtr.push_back((int)colInd.size()); }
};

// Scale parameter s of the row-length law so that E[L] = mean, with
// E[L] = sum_{k=1..Lmax} min(1, (s/k)^0.6).
double solve_length_scale(int Lmax, double mean)
{
    auto expect = [&](double s) {
        double e = 0.0;
        for (int k = 1; k <= Lmax; ++k) e += std::min(1.0, std::pow(s / k, 0.6));
        return e;
    };
    double lo = 1e-9, hi = (double)Lmax;
    for (int it = 0; it < 200; ++it) {
        double mid = 0.5 * (lo + hi);
        (expect(mid) < mean ? lo : hi) = mid;
    }
    return 0.5 * (lo + hi);
}

struct PowerLaw {
    int n, Lmax;
    double s;
    std::vector<int> stamp;  // stamp[col] == row+1 when col already used in this row
    std::vector<int> cols;
    PowerLaw(int n_) : n(n_), Lmax(std::max(1, std::min(4096, n_ / 2))), s(solve_length_scale(Lmax, std::min(10.0, (double)Lmax))), stamp(n_, 0) {}
    void row(Rng &g, int r, Builder &B)
    {
        double u = g.u01();
        double raw = (u <= 0.0) ? (double)Lmax : s * std::pow(u, -1.0 / 0.6);
        int L = raw >= (double)Lmax ? Lmax : std::max(1, (int)raw);
        int centre = g.below(n);
        cols.clear();
        for (int i = 0; i < L; ++i) {
            int c = -1;
            for (int attempt = 0;; ++attempt) {
                if (attempt < 8 && g.u01() < 0.7) {
                    c = centre + g.below(1025) - 512;
                    c = std::min(std::max(c, 0), n - 1);
                } else {
                    c = g.below(n);
                }
                if (stamp[c] != r + 1) break;
            }
            stamp[c] = r + 1;
            cols.push_back(c);
        }
        std::sort(cols.begin(), cols.end());
        for (int c : cols) B.push(c, g.sym());
        B.end_row();
    }
};

void gen_random(Rng &g, int n, int per_row, Builder &B)
{
    std::vector<int> cols;
    per_row = std::min(per_row, n);
    for (int r = 0; r < n; ++r) {
        cols.clear();
        while ((int)cols.size() < per_row) {
            int c = g.below(n);
            if (std::find(cols.begin(), cols.end(), c) == cols.end()) cols.push_back(c);
        }
        std::sort(cols.begin(), cols.end());
        for (int c : cols) B.push(c, g.sym());
        B.end_row();
    }
}

void gen_block_clustered(Rng &g, int n, Builder &B, bool unaligned, double share)
{
    const int per_row = std::min(64, n), nb = n / 8;
    const int max_blocks_per_row = per_row / 8;
    int want = (int)std::floor(share * (double)n * per_row / 64.0);
    std::vector<std::vector<int>> blocks(nb);  // first column of every block of each block row
    int placed = 0;
    for (long long attempts = 0; placed < want && attempts < 64LL * want + 1024; ++attempts) {
        int br = g.below(nb);
        int c0;
        if (unaligned) {
            c0 = 8 * br - 1024 + g.below(2048 - 8 + 1);
            c0 = std::min(std::max(c0, 0), n - 8);
        } else {
            int bc = br - 128 + g.below(256);
            c0 = 8 * std::min(std::max(bc, 0), nb - 1);
        }
        auto &v = blocks[br];
        if ((int)v.size() >= max_blocks_per_row) continue;
        bool overlaps = false;
        for (int o : v) overlaps = overlaps || std::abs(o - c0) < 8;
        if (overlaps) continue;
        v.push_back(c0);
        ++placed;
    }
    std::vector<int> cols;
    for (int r = 0; r < n; ++r) {
        cols.clear();
        if (r / 8 < nb)
            for (int c0 : blocks[r / 8])
                for (int j = 0; j < 8; ++j) cols.push_back(c0 + j);
        while ((int)cols.size() < per_row) {
            int c = g.below(n);
            if (std::find(cols.begin(), cols.end(), c) == cols.end()) cols.push_back(c);
        }
        std::sort(cols.begin(), cols.end());
        for (int c : cols) B.push(c, g.sym());
        B.end_row();
    }
}

void gen_stencil27(int g3, Builder &B)
{
    for (int z = 0; z < g3; ++z)
        for (int y = 0; y < g3; ++y)
            for (int x = 0; x < g3; ++x) {
                for (int dz = -1; dz <= 1; ++dz)
                    for (int dy = -1; dy <= 1; ++dy)
                        for (int dx = -1; dx <= 1; ++dx) {
                            int xx = x + dx, yy = y + dy, zz = z + dz;
                            if (xx < 0 || yy < 0 || zz < 0 || xx >= g3 || yy >= g3 || zz >= g3) continue;
                            B.push(xx + g3 * (yy + g3 * zz), (dx == 0 && dy == 0 && dz == 0) ? 26.0 : -1.0);
                        }
                B.end_row();
            }
}

void gen_mixed(Rng &g, int n, Builder &B, bool unaligned, double share)
{
    PowerLaw pl(n);
    const int run = 128;
    for (int r0 = 0; r0 < n; r0 += run) {
        int r1 = std::min(r0 + run, n);
        bool strip = g.u01() < share && n >= 64;
        int off = g.below(65) - 32;
        const int shift = unaligned ? 1 + g.below(7) : 0;
        for (int r = r0; r < r1; ++r) {
            if (strip) {
                int c0 = 8 * (r / 8 + off) + shift;
                c0 = std::min(std::max(c0, shift), n - 32 - (8 - shift) % 8);
                for (int j = 0; j < 32; ++j) B.push(c0 + j, g.sym());
                B.end_row();
            } else {
                pl.row(g, r, B);
            }
        }
    }
}

template <typename T>
T *dup(const std::vector<T> &v)
{
    T *p = (T *)malloc(std::max<size_t>(v.size(), 1) * sizeof(T));
    if (p && !v.empty()) std::memcpy(p, v.data(), v.size() * sizeof(T));
    return p;
}

}  // namespace

extern "C" int mx_gen_config(int config_id, uint64_t seed, double scale, int *rows, int *cols, int *nnz,
                             mx_dtype *dtype, int **rowPtr, int **colInd, void **val, void **x)
{
    return mx_gen_config_ex(config_id, seed, scale, 0, rows, cols, nnz, dtype, rowPtr, colInd, val, x);
}

extern "C" int mx_gen_config_ex(int config_id, uint64_t seed, double scale, int gen_flags, int *rows, int *cols, int *nnz,
                                mx_dtype *dtype, int **rowPtr, int **colInd, void **val, void **x)
{
    return mx_gen_config_family(config_id, seed, scale, gen_flags, -1.0, rows, cols, nnz, dtype, rowPtr, colInd, val, x);
}

extern "C" int mx_gen_config_family(int config_id, uint64_t seed, double scale, int gen_flags, double dense_share, int *rows, int *cols,
                                    int *nnz, mx_dtype *dtype, int **rowPtr, int **colInd, void **val, void **x)
{
    if (config_id < 1 || config_id > 5 || !(scale > 0.0 && scale <= 1.0) || !rows || !cols || !nnz || !dtype ||
        !rowPtr || !colInd || !val || !x || (gen_flags & ~MX_GEN_UNALIGNED) || dense_share > 1.0 ||
        (dense_share >= 0.0 && config_id != 2 && config_id != 5)) {
        mx::set_error("mx_gen_config: bad argument (config 1..5, scale in (0,1])");
        return MX_ERR_ARG;
    }
    const bool unaligned = (gen_flags & MX_GEN_UNALIGNED) != 0;
    if (seed == 0) seed = 0x9E3779B97F4A7C15ull ^ (uint64_t)config_id;
    Rng g(seed);
    Builder B;
    B.dtype = (config_id >= 4) ? MX_F16 : MX_F64;
    int n = 0;
    bool x_unit = false;  // x in [0,1] instead of [-1,1]
    try {
        switch (config_id) {
        case 1:
            n = std::max(16, (int)std::llround(4096.0 * scale));
            gen_random(g, n, 16, B);
            break;
        case 2:
            n = std::max(64, (int)std::llround(65536.0 * scale) / 8 * 8);
            gen_block_clustered(g, n, B, unaligned, dense_share >= 0.0 ? dense_share : 0.4);
            break;
        case 3: {
            int g3 = std::max(3, (int)std::llround(100.0 * std::cbrt(scale)));
            n = g3 * g3 * g3;
            gen_stencil27(g3, B);
            x_unit = true;
            break;
        }
        case 4: {
            n = std::max(64, (int)std::llround(1048576.0 * scale));
            PowerLaw pl(n);
            for (int r = 0; r < n; ++r) pl.row(g, r, B);
            break;
        }
        case 5:
            n = std::max(256, (int)std::llround(4194304.0 * scale) / 128 * 128);
            gen_mixed(g, n, B, unaligned, dense_share >= 0.0 ? dense_share : 0.2);
            break;
        }
    } catch (const std::bad_alloc &) {
        mx::set_error("mx_gen_config: out of memory");
        return MX_ERR_ALLOC;
    }
    *rows = n;
    *cols = n;
    *nnz = (int)B.colInd.size();
    *dtype = B.dtype;
    *rowPtr = dup(B.rowPtr);
    *colInd = dup(B.colInd);
    void *xv;
    if (B.dtype == MX_F64) {
        *val = dup(B.v64);
        double *xd = (double *)malloc((size_t)n * sizeof(double));
        if (xd)
            for (int i = 0; i < n; ++i) xd[i] = x_unit ? g.u01() : g.sym();
        xv = xd;
    } else {
        *val = dup(B.v16);
        uint16_t *xh = (uint16_t *)malloc((size_t)n * sizeof(uint16_t));
        if (xh)
            for (int i = 0; i < n; ++i) xh[i] = mx::f64_to_f16_bits(x_unit ? g.u01() : g.sym());
        xv = xh;
    }
    *x = xv;
    if (!*rowPtr || !*colInd || !*val || !xv) {
        free(*rowPtr);
        free(*colInd);
        free(*val);
        free(xv);
        mx::set_error("mx_gen_config: out of memory");
        return MX_ERR_ALLOC;
    }
    return MX_OK;
}
