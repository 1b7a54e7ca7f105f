/*
 * Deterministic synthetic CSR workloads (host side, C + OpenMP).
 *
 * Every array element is a pure function of (seed, stream, index) through a splitmix64-style
 * mixer, so the same arrays come out on any machine, with any thread count, without
 * shipping files.  Only +,-,*,/ and sqrt are used on floating point (no libm pow/exp/log),
 * and the file is compiled with -ffp-contract=off, so row lengths are reproducible
 * bit for bit.
 *
 * Shapes follow the five benchmark configurations:
 *   banded      rows i hold columns |i-j| <= half_bw
 *   fixed       exactly k distinct uniform columns per row, sorted
 *   zipf        row length = clip(round(z*scale), 1, max_len), z ~ Zipf(alpha), a fraction of
 *               rows emptied; uniform distinct sorted columns
 *   stencil5    2D 5-point Laplacian (4 on the diagonal, -1 neighbours, Dirichlet)
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

static inline uint64_t mix64(uint64_t z)
{
    z += 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}
static inline uint64_t draw(uint64_t seed, uint64_t stream, uint64_t idx)
{
    return mix64(mix64(seed * 0xD1342543DE82EF95ull + stream) ^ mix64(idx));
}
static inline double unit53(uint64_t h) { return (double)(h >> 11) * (1.0 / 9007199254740992.0); }
static inline float unit24(uint64_t h) { return (float)(h >> 40) * (1.0f / 16777216.0f); }
/* uniform integer in [0,n) by multiply-shift on the high 32 bits (n < 2^31) */
static inline int32_t below(uint64_t h, int32_t n) { return (int32_t)(((h >> 32) * (uint64_t)n) >> 32); }

/* ------------------------------------------------------------------ dense fills */
void wl_fill_uniform_f64(double *out, int64_t n, double lo, double hi, uint64_t seed, uint64_t stream)
{
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; ++i)
        out[i] = lo + (hi - lo) * unit53(draw(seed, stream, (uint64_t)i));
}
void wl_fill_uniform_f32(float *out, int64_t n, float lo, float hi, uint64_t seed, uint64_t stream)
{
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; ++i)
        out[i] = lo + (hi - lo) * unit24(draw(seed, stream, (uint64_t)i));
}

static int64_t prefix_in_place(int32_t *row_ptr, int64_t m)
{
    /* row_ptr[1..m] holds lengths on entry */
    int64_t acc = 0;
    row_ptr[0] = 0;
    for (int64_t i = 1; i <= m; ++i) {
        acc += row_ptr[i];
        if (acc > 2147483647)
            return -1;
        row_ptr[i] = (int32_t)acc;
    }
    return acc;
}

/* ------------------------------------------------------------------ banded */
int64_t wl_banded_row_ptr(int32_t m, int32_t half_bw, int32_t *row_ptr)
{
    for (int32_t i = 0; i < m; ++i) {
        int32_t lo = i - half_bw < 0 ? 0 : i - half_bw;
        int32_t hi = i + half_bw > m - 1 ? m - 1 : i + half_bw;
        row_ptr[i + 1] = hi - lo + 1;
    }
    return prefix_in_place(row_ptr, m);
}
void wl_banded_cols(int32_t m, int32_t half_bw, const int32_t *row_ptr, int32_t *col)
{
#pragma omp parallel for schedule(static)
    for (int32_t i = 0; i < m; ++i) {
        int32_t lo = i - half_bw < 0 ? 0 : i - half_bw;
        int32_t len = row_ptr[i + 1] - row_ptr[i];
        for (int32_t j = 0; j < len; ++j)
            col[row_ptr[i] + j] = lo + j;
    }
}

/* ------------------------------------------------------------------ distinct sorted columns */
static int cmp_i32(const void *a, const void *b)
{
    int32_t x = *(const int32_t *)a, y = *(const int32_t *)b;
    return (x > y) - (x < y);
}
/* `len` distinct columns of [0,n), ascending, for row `row` */
static void distinct_sorted_cols(int32_t *out, int32_t len, int32_t n, uint64_t seed, uint64_t stream,
                                 uint64_t row)
{
    uint64_t ctr = row << 32;
    if (len <= 0)
        return;
    if (len >= n) { /* every column */
        for (int32_t j = 0; j < n && j < len; ++j)
            out[j] = j;
        return;
    }
    if (len <= 48) { /* insertion with duplicate rejection */
        int32_t have = 0;
        while (have < len) {
            int32_t c = below(draw(seed, stream, ctr++), n);
            int32_t p = have;
            while (p > 0 && out[p - 1] > c)
                --p;
            if (p > 0 && out[p - 1] == c)
                continue;
            memmove(out + p + 1, out + p, sizeof(int32_t) * (size_t)(have - p));
            out[p] = c;
            ++have;
        }
        return;
    }
    /* draw, sort, drop duplicates, top up until `len` distinct values are held */
    int32_t have = 0;
    while (have < len) {
        for (int32_t j = have; j < len; ++j)
            out[j] = below(draw(seed, stream, ctr++), n);
        qsort(out, (size_t)len, sizeof(int32_t), cmp_i32);
        int32_t w = 0;
        for (int32_t j = 0; j < len; ++j)
            if (w == 0 || out[j] != out[w - 1])
                out[w++] = out[j];
        have = w;
    }
}

/* ------------------------------------------------------------------ fixed k per row */
int64_t wl_fixed_row_ptr(int32_t m, int32_t k, int32_t *row_ptr)
{
    for (int32_t i = 0; i < m; ++i)
        row_ptr[i + 1] = k;
    return prefix_in_place(row_ptr, m);
}
void wl_random_cols(int32_t m, int32_t n, const int32_t *row_ptr, int32_t *col, uint64_t seed,
                    uint64_t stream)
{
#pragma omp parallel for schedule(dynamic, 1024)
    for (int32_t i = 0; i < m; ++i)
        distinct_sorted_cols(col + row_ptr[i], row_ptr[i + 1] - row_ptr[i], n, seed, stream, (uint64_t)i);
}

/* ------------------------------------------------------------------ Zipf row lengths */
/* v^(1/10) for v >= 1 by Newton from above (start: three square roots = v^(1/8) >= v^(1/10)) */
static double root10(double v)
{
    double t = sqrt(sqrt(sqrt(v)));
    for (int it = 0; it < 200; ++it) {
        double t2 = t * t, t4 = t2 * t2, t8 = t4 * t4, t9 = t8 * t;
        double nt = t - (t9 * t - v) / (10.0 * t9);
        if (!(nt < t))
            break;
        t = nt;
    }
    return t;
}
static double ipow(double b, int e)
{
    double r = 1.0;
    for (int i = 0; i < e; ++i)
        r *= b;
    return r;
}
/*
 * alpha = alpha10/10 (> 1).  z is drawn by inverse CDF from a table over 1..K where
 * K = ceil((max_len + 0.5)/scale); the mass beyond K (integral of x^-alpha from K+0.5)
 * collapses onto K.  len = min(max_len, max(1, floor(z*scale + 0.5))); then a row is
 * emptied when its `empty` draw falls below empty_frac.  Returns nnz, or -1 if it would
 * not fit int32 / table allocation failed.
 */
int64_t wl_zipf_row_ptr(int32_t m, int32_t alpha10, double scale, int32_t max_len, double empty_frac,
                        int32_t *row_ptr, uint64_t seed, uint64_t stream_len, uint64_t stream_empty)
{
    int64_t K = (int64_t)ceil(((double)max_len + 0.5) / scale);
    if (K < 1)
        K = 1;
    double *cdf = (double *)malloc(sizeof(double) * (size_t)(K + 1));
    if (!cdf)
        return -1;
    cdf[0] = 0.0;
    double acc = 0.0;
    for (int64_t k = 1; k <= K; ++k) {
        double w = 1.0 / ipow(root10((double)k), alpha10);
        acc += w;
        cdf[k] = acc;
    }
    double tail = 1.0 / ipow(root10((double)K + 0.5), alpha10 - 10) / ((double)(alpha10 - 10) / 10.0);
    double total = acc + tail;
#pragma omp parallel for schedule(static)
    for (int32_t i = 0; i < m; ++i) {
        double u = unit53(draw(seed, stream_len, (uint64_t)i)) * total;
        int64_t lo = 1, hi = K; /* first k with cdf[k] > u, else K */
        while (lo < hi) {
            int64_t mid = (lo + hi) / 2;
            if (cdf[mid] > u)
                hi = mid;
            else
                lo = mid + 1;
        }
        double scaled = floor((double)lo * scale + 0.5);
        int32_t len = scaled < 1.0 ? 1 : (scaled > (double)max_len ? max_len : (int32_t)scaled);
        if (unit53(draw(seed, stream_empty, (uint64_t)i)) < empty_frac)
            len = 0;
        row_ptr[i + 1] = len;
    }
    free(cdf);
    return prefix_in_place(row_ptr, m);
}

/* ------------------------------------------------------------------ 5-point stencil */
int64_t wl_stencil5_row_ptr(int32_t nx, int32_t ny, int32_t *row_ptr)
{
    int64_t m = (int64_t)nx * ny;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < m; ++r) {
        int32_t ix = (int32_t)(r % nx), iy = (int32_t)(r / nx);
        row_ptr[r + 1] = 1 + (iy > 0) + (ix > 0) + (ix < nx - 1) + (iy < ny - 1);
    }
    return prefix_in_place(row_ptr, m);
}
void wl_stencil5_fill_f64(int32_t nx, int32_t ny, const int32_t *row_ptr, int32_t *col, double *val)
{
    int64_t m = (int64_t)nx * ny;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < m; ++r) {
        int32_t ix = (int32_t)(r % nx), iy = (int32_t)(r / nx);
        int64_t p = row_ptr[r];
        if (iy > 0) { col[p] = (int32_t)(r - nx); val[p++] = -1.0; }
        if (ix > 0) { col[p] = (int32_t)(r - 1); val[p++] = -1.0; }
        col[p] = (int32_t)r; val[p++] = 4.0;
        if (ix < nx - 1) { col[p] = (int32_t)(r + 1); val[p++] = -1.0; }
        if (iy < ny - 1) { col[p] = (int32_t)(r + nx); val[p++] = -1.0; }
    }
}

/* ------------------------------------------------------------------ 7-point stencil on nx x ny x nz */
int64_t wl_stencil7_row_ptr(int32_t nx, int32_t ny, int32_t nz, int32_t *row_ptr)
{
    int64_t plane = (int64_t)nx * ny, m = plane * nz;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < m; ++r) {
        int32_t ix = (int32_t)(r % nx), iy = (int32_t)(r / nx % ny), iz = (int32_t)(r / plane);
        row_ptr[r + 1] = 1 + (iz > 0) + (iy > 0) + (ix > 0) + (ix < nx - 1) + (iy < ny - 1) + (iz < nz - 1);
    }
    return prefix_in_place(row_ptr, m);
}
void wl_stencil7_fill_f64(int32_t nx, int32_t ny, int32_t nz, const int32_t *row_ptr, int32_t *col, double *val)
{
    int64_t plane = (int64_t)nx * ny, m = plane * nz;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < m; ++r) {
        int32_t ix = (int32_t)(r % nx), iy = (int32_t)(r / nx % ny), iz = (int32_t)(r / plane);
        int64_t p = row_ptr[r];
        if (iz > 0) { col[p] = (int32_t)(r - plane); val[p++] = -1.0; }
        if (iy > 0) { col[p] = (int32_t)(r - nx); val[p++] = -1.0; }
        if (ix > 0) { col[p] = (int32_t)(r - 1); val[p++] = -1.0; }
        col[p] = (int32_t)r; val[p++] = 6.0;
        if (ix < nx - 1) { col[p] = (int32_t)(r + 1); val[p++] = -1.0; }
        if (iy < ny - 1) { col[p] = (int32_t)(r + nx); val[p++] = -1.0; }
        if (iz < nz - 1) { col[p] = (int32_t)(r + plane); val[p++] = -1.0; }
    }
}
