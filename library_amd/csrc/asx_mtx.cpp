// MatrixMarket coordinate reader (host): the loader the reference's test drivers use to get a
// matrix before they sort it and build CSR (hip/test/io.hip:100-179 header, :180-330 bodies).
// Kept from the reference: indices become zero-based; entries come out in file order; for
// symmetric / Hermitian / skew-symmetric files every off-diagonal entry is followed by its
// mirror image carrying the SAME value (the reference does not negate for skew-symmetric);
// `pattern` entries get the value 1; of a `complex` entry the real part is taken (what the
// reference's fp32 reader does; its fp64 reader exits on pattern and complex files, this one
// reads them).  Differences: the field and symmetry keywords are matched without regard to case
// (the reference treats "hermitian" in lower case as general), indices outside the matrix and
// truncated files are errors instead of undefined behaviour, and a dense `array` file is
// NOT_SUPPORTED instead of exit(0).
#include <cctype>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>

#include "../../include/alphasparse_amd.h"

namespace {

bool ieq(const std::string &a, const char *b)
{
    if (a.size() != std::strlen(b)) return false;
    for (size_t i = 0; i < a.size(); ++i)
        if (std::tolower((unsigned char)a[i]) != std::tolower((unsigned char)b[i])) return false;
    return true;
}

// next whitespace-separated token of the line starting at p (stops at end of line)
std::string token(const char *&p, const char *end)
{
    while (p < end && (*p == ' ' || *p == '\t' || *p == '\r')) ++p;
    const char *s = p;
    while (p < end && !std::isspace((unsigned char)*p)) ++p;
    return std::string(s, p);
}

const char *next_line(const char *p, const char *end)
{
    while (p < end && *p != '\n') ++p;
    return p < end ? p + 1 : end;
}

template <typename T>
int read_body(const char *p, const char *end, int32_t m, int32_t n, int64_t lines, bool mirror, bool has_value,
              int32_t *nnz_out, int32_t **row_out, int32_t **col_out, void **val_out)
{
    const int64_t cap = mirror ? 2 * lines : lines;
    if (cap > INT32_MAX) return ASX_STATUS_INVALID_SIZE;
    int32_t *row = (int32_t *)std::malloc(sizeof(int32_t) * (size_t)(cap ? cap : 1));
    int32_t *col = (int32_t *)std::malloc(sizeof(int32_t) * (size_t)(cap ? cap : 1));
    T *val = (T *)std::malloc(sizeof(T) * (size_t)(cap ? cap : 1));
    int st = ASX_STATUS_SUCCESS;
    int64_t k = 0;
    if (!row || !col || !val) st = ASX_STATUS_ALLOC_FAILED;
    for (int64_t i = 0; !st && i < lines; ++i) {
        while (p < end && (*p == '\n' || *p == '\r' || *p == ' ' || *p == '\t')) ++p;  // blank lines
        if (p >= end) {
            st = ASX_STATUS_INVALID_SIZE;  // fewer entries than the size line promises
            break;
        }
        char *q;
        const long r = std::strtol(p, &q, 10);
        if (q == p) {
            st = ASX_STATUS_INVALID_VALUE;
            break;
        }
        p = q;
        const long c = std::strtol(p, &q, 10);
        if (q == p) {
            st = ASX_STATUS_INVALID_VALUE;
            break;
        }
        p = q;
        double v = 1.0;
        if (has_value) {
            while (p < end && (*p == ' ' || *p == '\t')) ++p;
            if (p < end && *p != '\n' && *p != '\r') {
                v = std::strtod(p, &q);
                if (q == p) {
                    st = ASX_STATUS_INVALID_VALUE;
                    break;
                }
                p = q;
            }
        }
        p = next_line(p, end);  // anything else on the line (an imaginary part) is ignored
        if (r < 1 || r > m || c < 1 || c > n) {
            st = ASX_STATUS_INVALID_VALUE;
            break;
        }
        row[k] = (int32_t)r - 1;
        col[k] = (int32_t)c - 1;
        val[k] = (T)v;
        ++k;
        if (mirror && r != c) {
            if (c > m || r > n) {
                st = ASX_STATUS_INVALID_VALUE;
                break;
            }
            row[k] = (int32_t)c - 1;
            col[k] = (int32_t)r - 1;
            val[k] = (T)v;
            ++k;
        }
    }
    if (st) {
        std::free(row);
        std::free(col);
        std::free(val);
        return st;
    }
    *nnz_out = (int32_t)k;
    *row_out = row;
    *col_out = col;
    *val_out = val;
    return ASX_STATUS_SUCCESS;
}

}  // namespace

extern "C" int asx_mtx_read(const char *path, int value_type, int32_t *m, int32_t *n, int32_t *nnz,
                            int32_t **h_row, int32_t **h_col, void **h_val)
{
    if (!path || !m || !n || !nnz || !h_row || !h_col || !h_val) return ASX_STATUS_INVALID_POINTER;
    if (value_type != ASX_R_32F && value_type != ASX_R_64F) return ASX_STATUS_NOT_SUPPORTED;
    FILE *f = std::fopen(path, "rb");
    if (!f) return ASX_STATUS_INVALID_VALUE;
    std::string text;
    {
        char chunk[1 << 16];
        size_t got;
        while ((got = std::fread(chunk, 1, sizeof chunk, f)) > 0) text.append(chunk, got);
    }
    std::fclose(f);
    const char *p = text.data(), *end = p + text.size();

    // %%MatrixMarket matrix coordinate <field> <symmetry>; a file without the banner is read as
    // real general, as the reference does
    bool has_value = true, mirror = false;
    if (p < end && *p == '%') {
        const char *lp = p;
        const char *le = next_line(p, end);
        (void)token(lp, le);  // %%MatrixMarket
        (void)token(lp, le);  // matrix
        const std::string fmt = token(lp, le), field = token(lp, le), sym = token(lp, le);
        if (ieq(fmt, "array")) return ASX_STATUS_NOT_SUPPORTED;
        if (ieq(field, "pattern")) has_value = false;
        mirror = ieq(sym, "symmetric") || ieq(sym, "hermitian") || ieq(sym, "skew-symmetric");
    }
    while (p < end && *p == '%') p = next_line(p, end);
    while (p < end && (*p == '\n' || *p == '\r')) ++p;
    if (p >= end) return ASX_STATUS_INVALID_SIZE;
    long mm = 0, nn = 0, lines = 0;
    {
        char *q;
        mm = std::strtol(p, &q, 10);
        if (q == p) return ASX_STATUS_INVALID_VALUE;
        p = q;
        nn = std::strtol(p, &q, 10);
        if (q == p) return ASX_STATUS_INVALID_VALUE;
        p = q;
        lines = std::strtol(p, &q, 10);
        if (q == p) return ASX_STATUS_INVALID_VALUE;
        p = next_line(q, end);
    }
    if (mm < 0 || nn < 0 || lines < 0 || mm > INT32_MAX || nn > INT32_MAX) return ASX_STATUS_INVALID_SIZE;
    *m = (int32_t)mm;
    *n = (int32_t)nn;
    if (value_type == ASX_R_64F)
        return read_body<double>(p, end, *m, *n, lines, mirror, has_value, nnz, h_row, h_col, h_val);
    return read_body<float>(p, end, *m, *n, lines, mirror, has_value, nnz, h_row, h_col, h_val);
}

extern "C" void asx_host_free(void *p) { std::free(p); }
