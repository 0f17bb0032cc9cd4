// Matrix-Market coordinate ingest with the behaviour of the reference's mmio_allinone
// (utilities/mmio.cpp:1547-1713): entries stay in file order inside each row (no column
// sort, duplicates kept); `symmetric` and `hermitian` files get the mirrored entry right
// after the stored one; `skew-symmetric` is NOT expanded (the reference only tests
// mm_is_symmetric / mm_is_hermitian, :1581); complex values keep their real part; pattern
// files get value 1.  The text parsing itself is this file's own (fgets + strtol/strtod).
#include <cctype>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "mx_internal.h"

namespace {

std::string lower(std::string s)
{
    for (auto &c : s) c = (char)std::tolower((unsigned char)c);
    return s;
}

}  // namespace

extern "C" int mx_mmio_read(const char *path, mx_dtype dtype, int *rows, int *cols, int *nnz, int *isSymmetric,
                            int **rowPtr, int **colInd, void **val)
{
    if (!path || !rows || !cols || !nnz || !rowPtr || !colInd || !val) {
        mx::set_error("mx_mmio_read: null argument");
        return MX_ERR_ARG;
    }
    FILE *f = std::fopen(path, "r");
    if (!f) {
        mx::set_error(std::string("mx_mmio_read: cannot open ") + path);
        return MX_ERR_IO;
    }
    std::vector<char> line(1 << 16);
    auto fail = [&](const char *why) {
        std::fclose(f);
        mx::set_error(std::string("mx_mmio_read: ") + why + " in " + path);
        return MX_ERR_IO;
    };
    if (!std::fgets(line.data(), (int)line.size(), f)) return fail("empty file");
    char banner[64] = {0}, object[64] = {0}, format[64] = {0}, field[64] = {0}, symm[64] = {0};
    if (std::sscanf(line.data(), "%63s %63s %63s %63s %63s", banner, object, format, field, symm) != 5)
        return fail("could not process Matrix Market banner");
    if (std::strcmp(banner, "%%MatrixMarket") != 0 || lower(object) != "matrix" || lower(format) != "coordinate")
        return fail("not a Matrix Market coordinate matrix");
    const std::string fld = lower(field), sym = lower(symm);
    const bool isPattern = fld == "pattern", isComplex = fld == "complex";
    if (!(isPattern || isComplex || fld == "real" || fld == "integer" || fld == "double"))
        return fail("unsupported value field");
    const bool expand = sym == "symmetric" || sym == "hermitian";

    long m = 0, n = 0, entries = 0;
    for (;;) {  // size line: first line that is neither a comment nor blank
        if (!std::fgets(line.data(), (int)line.size(), f)) return fail("missing size line");
        const char *p = line.data();
        while (*p && std::isspace((unsigned char)*p)) ++p;
        if (*p == '%' || *p == 0) continue;
        if (std::sscanf(p, "%ld %ld %ld", &m, &n, &entries) != 3) return fail("bad size line");
        break;
    }
    if (m < 0 || n < 0 || entries < 0 || m > 2147483646L || n > 2147483646L || entries > 1073741823L)
        return fail("dimensions out of range");

    std::vector<int> ri((size_t)entries), cj((size_t)entries);
    std::vector<double> vv((size_t)entries);
    std::vector<int> counter((size_t)m + 1, 0);
    for (long k = 0; k < entries; ++k) {
        if (!std::fgets(line.data(), (int)line.size(), f)) return fail("fewer entries than announced");
        char *p = line.data(), *end = nullptr;
        long i = std::strtol(p, &end, 10);
        if (end == p) {  // blank line: retry
            --k;
            continue;
        }
        p = end;
        long j = std::strtol(p, &end, 10);
        if (end == p) return fail("bad entry line");
        p = end;
        double v = 1.0;
        if (!isPattern) {
            v = std::strtod(p, &end);
            if (end == p) return fail("missing value");
        }
        if (i < 1 || i > m || j < 1 || j > n) return fail("index out of range");
        ri[k] = (int)(i - 1);
        cj[k] = (int)(j - 1);
        vv[k] = v;
        counter[i - 1]++;
    }
    std::fclose(f);
    if (expand) {
        if (m != n) {
            mx::set_error("mx_mmio_read: symmetric file is not square");
            return MX_ERR_IO;
        }
        for (long k = 0; k < entries; ++k)
            if (ri[k] != cj[k]) counter[cj[k]]++;
    }
    // exclusive scan (utilities/mmio.cpp:949-964)
    long long total = 0;
    std::vector<int> start((size_t)m + 1, 0);
    for (long r = 0; r < m; ++r) {
        start[r] = (int)total;
        total += counter[r];
    }
    if (total > 2147483646LL) {
        mx::set_error("mx_mmio_read: too many entries for 32-bit indices");
        return MX_ERR_IO;
    }
    start[m] = (int)total;
    const size_t es = (size_t)mx::elem_size(dtype);
    int *rp = (int *)malloc(((size_t)m + 1) * sizeof(int));
    int *ci = (int *)malloc((size_t)(total ? total : 1) * sizeof(int));
    unsigned char *va = (unsigned char *)malloc((size_t)(total ? total : 1) * es);
    if (!rp || !ci || !va) {
        free(rp);
        free(ci);
        free(va);
        mx::set_error("mx_mmio_read: out of memory");
        return MX_ERR_ALLOC;
    }
    std::memcpy(rp, start.data(), ((size_t)m + 1) * sizeof(int));
    std::vector<int> fill((size_t)m, 0);
    auto put = [&](int r, int c, double v) {
        size_t q = (size_t)rp[r] + (size_t)fill[r]++;
        ci[q] = c;
        if (dtype == MX_F64)
            ((double *)va)[q] = v;
        else
            ((uint16_t *)va)[q] = mx::f64_to_f16_bits(v);
    };
    for (long k = 0; k < entries; ++k) {
        put(ri[k], cj[k], vv[k]);
        if (expand && ri[k] != cj[k]) put(cj[k], ri[k], vv[k]);
    }
    *rows = (int)m;
    *cols = (int)n;
    *nnz = (int)total;
    if (isSymmetric) *isSymmetric = expand ? 1 : 0;
    *rowPtr = rp;
    *colInd = ci;
    *val = va;
    return MX_OK;
}
