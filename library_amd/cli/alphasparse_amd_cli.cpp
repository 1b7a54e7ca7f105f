// Command-line driver for CSR SpMV / SpMM on a MatrixMarket file, with the option surface of the
// reference's test drivers (hip/test/args.hip:9-62: --data-file --check --iter --warmup --cols
// --alg_num --transA --layout --data-type --metrics-file) and their flow
// (hip/test/level2/spmv_csr_r_f64_test.hip:274-314: read COO, sort, x = rand seed 2, y = rand
// seed 1, alpha = 2.1 / beta = 3.2 for SpMV, hip/test/level3/spmm_csr_row_r_f32_test.hip:45-46:
// alpha = 2 / beta = 3 for SpMM; coo2csr on the device; bufferSize; warm-up calls; timed calls
// with y restored before each; average time).  The sort runs on the device and --check compares
// with a plain host loop in double precision instead of hipSPARSE.
//
//   alphasparse_amd_cli --data-file=A.mtx [--op=spmv|spmm] [--data-type=S|D] [--alg_num=<id>]
//                       [--iter=100] [--warmup=10] [--cols=64] [--transA=N|T] [--layout=R|C]
//                       [--analysis] [--check] [--metrics-file=out.csv]
#include <getopt.h>
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "alphasparse.h"
#include "alphasparse_amd.h"

#define HIP_OK(e)                                                                                       \
    do {                                                                                                \
        hipError_t _e = (e);                                                                            \
        if (_e != hipSuccess) {                                                                         \
            std::fprintf(stderr, "HIP error: %s at %s:%d\n", hipGetErrorString(_e), __FILE__, __LINE__); \
            std::exit(2);                                                                               \
        }                                                                                               \
    } while (0)
#define ASX_OK(e)                                                                     \
    do {                                                                              \
        int _s = (int)(e);                                                            \
        if (_s != 0) {                                                                \
            std::fprintf(stderr, "status %d from %s at line %d\n", _s, #e, __LINE__); \
            std::exit(3);                                                             \
        }                                                                             \
    } while (0)

namespace {

struct Options {
    std::string file, metrics_file, op = "spmv";
    char data_type = 'S';  // the reference's default
    int alg = -1;          // -1: the list the reference's driver loops over, plus DEFAULT
    int iter = 100, warmup = 10, cols = 64;
    bool check = false, trans = false, col_major = false, analysis = false;
};

void usage()
{
    std::printf(
        "--data-file=<file.mtx>\tMatrixMarket coordinate file\n"
        "--op=<spmv|spmm>\toperation, default spmv\n"
        "--data-type=<S|D>\tvalue type, default S\n"
        "--alg_num=<int>\talgorithm id (alphasparseSpMVAlg_t / alphasparseSpMMAlg_t), default: a list\n"
        "--iter=<int>\ttimed calls, default 100\n"
        "--warmup=<int>\twarm-up calls, default 10\n"
        "--cols=<int>\tcolumns of the dense matrices (spmm), default 64\n"
        "--transA=<N|T>\toperation on A, default N\n"
        "--layout=<R|C>\tlayout of the dense matrices (spmm), default R\n"
        "--analysis\tcall alphasparseSpMV_analysis / alphasparseSpMM_preprocess first\n"
        "--check\tcompare with a host computation\n"
        "--metrics-file=<file>\tappend one CSV line per algorithm\n");
}

Options parse(int argc, char **argv)
{
    static option longopts[] = {{"help", no_argument, nullptr, 1},
                                {"check", no_argument, nullptr, 2},
                                {"transA", required_argument, nullptr, 4},
                                {"data-file", required_argument, nullptr, 12},
                                {"layout", required_argument, nullptr, 15},
                                {"cols", required_argument, nullptr, 18},
                                {"iter", required_argument, nullptr, 20},
                                {"data-type", required_argument, nullptr, 22},
                                {"warmup", required_argument, nullptr, 37},
                                {"metrics-file", required_argument, nullptr, 34},
                                {"alg_num", required_argument, nullptr, 36},
                                {"op", required_argument, nullptr, 50},
                                {"analysis", no_argument, nullptr, 51},
                                {nullptr, 0, nullptr, 0}};
    Options o;
    int opt, idx;
    while ((opt = getopt_long_only(argc, argv, "", longopts, &idx)) != -1) {
        switch (opt) {
        case 1: usage(); std::exit(0);
        case 2: o.check = true; break;
        case 4: o.trans = optarg[0] == 'T' || optarg[0] == 't' || optarg[0] == 'H' || optarg[0] == 'h'; break;
        case 12: o.file = optarg; break;
        case 15: o.col_major = optarg[0] == 'C' || optarg[0] == 'c'; break;
        case 18: o.cols = std::atoi(optarg); break;
        case 20: o.iter = std::atoi(optarg); break;
        case 22: o.data_type = (char)std::toupper((unsigned char)optarg[0]); break;
        case 37: o.warmup = std::atoi(optarg); break;
        case 34: o.metrics_file = optarg; break;
        case 36: o.alg = std::atoi(optarg); break;
        case 50: o.op = optarg; break;
        case 51: o.analysis = true; break;
        default: usage(); std::exit(1);
        }
    }
    if (o.file.empty() || (o.op != "spmv" && o.op != "spmm") || (o.data_type != 'S' && o.data_type != 'D') ||
        o.iter < 1 || o.warmup < 0 || o.cols < 1) {
        usage();
        std::exit(1);
    }
    return o;
}

// include/alphasparse/util/random.h:17-19 under srand(seed), as alpha_fill_random does
// (hip/util/malloc.hip:94-104)
template <typename T>
void fill_random(std::vector<T> &v, unsigned seed)
{
    std::srand(seed);
    for (T &e : v) e = (T)std::rand() / (T)RAND_MAX;
}

template <typename T>
T *to_device(const T *h, size_t count)
{
    T *d = nullptr;
    HIP_OK(hipMalloc((void **)&d, (count ? count : 1) * sizeof(T)));
    if (count) HIP_OK(hipMemcpy(d, h, count * sizeof(T), hipMemcpyHostToDevice));
    return d;
}

// hip/test/check.hip:161-212: max |error| / max |result| against a bound (1e-12 there for fp64)
template <typename T>
bool report_check(const std::vector<double> &want, const std::vector<T> &got)
{
    double max_err = 0, max_res = 0;
    for (size_t i = 0; i < want.size(); ++i) {
        max_err = std::fmax(max_err, std::fabs(want[i] - (double)got[i]));
        max_res = std::fmax(max_res, std::fabs((double)got[i]));
    }
    const double rel = max_res > 0 ? max_err / max_res : max_err;
    const double bound = sizeof(T) == 8 ? 1e-12 : 1e-5;
    std::printf("%s: require %.0e, max relative error: %.3e\n", rel <= bound ? "correct" : "error", bound, rel);
    return rel <= bound;
}

template <typename T>
int run(const Options &o)
{
    const int vt = sizeof(T) == 8 ? ASX_R_64F : ASX_R_32F;
    const alphasparseDataType dt = sizeof(T) == 8 ? ALPHA_R_64F : ALPHA_R_32F;
    int32_t m = 0, n = 0, nnz = 0, *h_row = nullptr, *h_col = nullptr;
    void *h_val_v = nullptr;
    int st = asx_mtx_read(o.file.c_str(), vt, &m, &n, &nnz, &h_row, &h_col, &h_val_v);
    if (st) {
        std::fprintf(stderr, "cannot read %s (status %d)\n", o.file.c_str(), st);
        return 4;
    }
    const T *h_val = (const T *)h_val_v;
    const bool mm = o.op == "spmm";
    const int N = mm ? o.cols : 1;
    const int64_t in_len = o.trans ? m : n, out_len = o.trans ? n : m;
    const T alpha = mm ? (T)2.0f : (T)2.1f, beta = mm ? (T)3.0f : (T)3.2f;

    // COO on the device, sorted by (row, column), then row offsets
    int32_t *d_row = to_device(h_row, (size_t)nnz), *d_col = to_device(h_col, (size_t)nnz);
    T *d_val = to_device(h_val, (size_t)nnz);
    ASX_OK(asx_coo_sort(vt, d_row, d_col, d_val, nnz, nullptr));
    int32_t *d_rp = nullptr;
    HIP_OK(hipMalloc((void **)&d_rp, sizeof(int32_t) * ((size_t)m + 1)));
    ASX_OK(alphasparseXcoo2csr(d_row, nnz, m, d_rp));
    HIP_OK(hipDeviceSynchronize());

    std::vector<T> x((size_t)in_len * N), y0((size_t)out_len * N);
    fill_random(x, 2);
    fill_random(y0, 1);
    T *d_x = to_device(x.data(), x.size()), *d_y = to_device(y0.data(), y0.size());

    std::printf("\nMatrix: %s\nDimensions: %d x %d, NNZ: %d\n", o.file.c_str(), m, n, nnz);
    std::printf("Operation: %s%s, type %c%s\n", o.op.c_str(), o.trans ? " (transA=T)" : "", o.data_type,
                mm ? (o.col_major ? ", layout C" : ", layout R") : "");
    std::printf("Parameters: alpha=%.2f, beta=%.2f\nWarm-up: %d, Trials: %d\n", (double)alpha, (double)beta, o.warmup,
                o.iter);

    // host result for --check (double accumulation over the sorted device CSR copied back)
    std::vector<double> want;
    if (o.check) {
        std::vector<int32_t> rp((size_t)m + 1), col((size_t)nnz);
        std::vector<T> val((size_t)nnz);
        HIP_OK(hipMemcpy(rp.data(), d_rp, rp.size() * sizeof(int32_t), hipMemcpyDeviceToHost));
        if (nnz) HIP_OK(hipMemcpy(col.data(), d_col, col.size() * sizeof(int32_t), hipMemcpyDeviceToHost));
        if (nnz) HIP_OK(hipMemcpy(val.data(), d_val, val.size() * sizeof(T), hipMemcpyDeviceToHost));
        // element (r, c) of the dense operands in the chosen layout
        auto at = [&](int64_t r, int64_t c, int64_t rows) { return o.col_major && mm ? c * rows + r : r * N + c; };
        want.assign(y0.size(), 0.0);
        for (int64_t r = 0; r < out_len; ++r)
            for (int c = 0; c < N; ++c) want[(size_t)at(r, c, out_len)] = (double)beta * (double)y0[(size_t)at(r, c, out_len)];
        for (int32_t r = 0; r < m; ++r)
            for (int32_t k = rp[r]; k < rp[r + 1]; ++k) {
                const int64_t orow = o.trans ? col[k] : r, irow = o.trans ? r : col[k];
                for (int c = 0; c < N; ++c)
                    want[(size_t)at(orow, c, out_len)] +=
                        (double)alpha * (double)val[k] * (double)x[(size_t)at(irow, c, in_len)];
            }
    }

    alphasparseHandle_t handle = nullptr;
    ASX_OK(alphasparseGetHandle(&handle));
    alphasparseSpMatDescr_t A;
    ASX_OK(alphasparseCreateCsr(&A, m, n, nnz, d_rp, d_col, d_val, ALPHA_SPARSE_INDEXTYPE_I32,
                                ALPHA_SPARSE_INDEXTYPE_I32, ALPHA_SPARSE_INDEX_BASE_ZERO, dt));
    const alphasparseOperation_t opA = o.trans ? ALPHA_SPARSE_OPERATION_TRANSPOSE : ALPHA_SPARSE_OPERATION_NON_TRANSPOSE;
    const alphasparseOperation_t opN = ALPHA_SPARSE_OPERATION_NON_TRANSPOSE;
    alphasparseDnVecDescr_t X = nullptr, Y = nullptr;
    alphasparseDnMatDescr_t B = nullptr, C = nullptr;
    if (mm) {
        const alphasparseOrder_t ord = o.col_major ? ALPHASPARSE_ORDER_COL : ALPHASPARSE_ORDER_ROW;
        ASX_OK(alphasparseCreateDnMat(&B, in_len, N, o.col_major ? in_len : N, d_x, dt, ord));
        ASX_OK(alphasparseCreateDnMat(&C, out_len, N, o.col_major ? out_len : N, d_y, dt, ord));
    } else {
        ASX_OK(alphasparseCreateDnVec(&X, in_len, d_x, dt));
        ASX_OK(alphasparseCreateDnVec(&Y, out_len, d_y, dt));
    }

    std::vector<int> algs;
    if (o.alg >= 0)
        algs = {o.alg};
    else if (mm)  // DEFAULT + hip/test/level3/spmm_csr_row_r_f32_test.hip's list (CSR_ALG1..5)
        algs = {0, 5, 6, 7, 8, 9};
    else  // DEFAULT + hip/test/level2/spmv_csr_r_f64_test.hip:56-63
        algs = {0, 6, 7, 9, 11, 12, 13, 16};

    // algorithmic bytes and flops of one call
    const double sv = sizeof(T);
    const double bytes_call = (double)nnz * (sv + 4) + ((double)m + 1) * 4 + (double)in_len * N * sv +
                              (double)out_len * N * sv * 2;
    const double flops_call = 2.0 * (double)nnz * N;
    FILE *mf = o.metrics_file.empty() ? nullptr : std::fopen(o.metrics_file.c_str(), "a");
    if (!o.metrics_file.empty() && !mf) std::fprintf(stderr, "cannot open %s\n", o.metrics_file.c_str());

    bool all_ok = true;
    hipEvent_t e0, e1;
    HIP_OK(hipEventCreate(&e0));
    HIP_OK(hipEventCreate(&e1));
    std::vector<T> got(y0.size());
    for (int alg : algs) {
        size_t bytes = 0;
        alphasparseStatus_t s =
            mm ? alphasparseSpMM_bufferSize(handle, opA, opN, &alpha, A, B, &beta, C, dt, (alphasparseSpMMAlg_t)alg, &bytes)
               : alphasparseSpMV_bufferSize(handle, opA, &alpha, A, X, &beta, Y, dt, (alphasparseSpMVAlg_t)alg, &bytes);
        if (s) {
            std::printf("alphasparse alg %d: not available (status %d)\n", alg, (int)s);
            continue;
        }
        void *buffer = nullptr;
        HIP_OK(hipMalloc(&buffer, bytes ? bytes : 1));
        if (o.analysis) {
            if (mm)
                ASX_OK(alphasparseSpMM_preprocess(handle, opA, opN, &alpha, A, B, &beta, C, dt, (alphasparseSpMMAlg_t)alg,
                                                  nullptr));
            else
                ASX_OK(alphasparseSpMV_analysis(handle, opA, A, (alphasparseSpMVAlg_t)alg));
        }
        double total_ms = 0;
        for (int i = 0; i < o.warmup + o.iter; ++i) {
            HIP_OK(hipMemcpyAsync(d_y, y0.data(), y0.size() * sizeof(T), hipMemcpyHostToDevice, handle->stream));
            HIP_OK(hipEventRecord(e0, handle->stream));
            s = mm ? alphasparseSpMM(handle, opA, opN, &alpha, A, B, &beta, C, dt, (alphasparseSpMMAlg_t)alg, buffer)
                   : alphasparseSpMV(handle, opA, &alpha, A, X, &beta, Y, dt, (alphasparseSpMVAlg_t)alg, buffer);
            HIP_OK(hipEventRecord(e1, handle->stream));
            HIP_OK(hipEventSynchronize(e1));
            if (s) {
                std::fprintf(stderr, "alg %d failed with status %d\n", alg, (int)s);
                return 5;
            }
            float ms = 0;
            HIP_OK(hipEventElapsedTime(&ms, e0, e1));
            if (i >= o.warmup) total_ms += ms;
        }
        const double ms = total_ms / o.iter;
        std::printf("alphasparse alg %d: %lf ms  (%.1f GB/s, %.1f GFLOP/s)\n", alg, ms, bytes_call / ms / 1e6,
                    flops_call / ms / 1e6);
        if (mf)
            std::fprintf(mf, "%s,%s,%c,%d,%d,%d,%d,%d,%.6f,%.3f,%.3f\n", o.file.c_str(), o.op.c_str(), o.data_type, m, n,
                         nnz, N, alg, ms, bytes_call / ms / 1e6, flops_call / ms / 1e6);
        if (o.check) {
            HIP_OK(hipMemcpy(got.data(), d_y, got.size() * sizeof(T), hipMemcpyDeviceToHost));
            all_ok &= report_check<T>(want, got);
        }
        if (o.analysis) {
            if (mm)
                ;  // kept analyses go with the handle
            else
                ASX_OK(alphasparseSpMV_clear(handle, (alphasparseSpMVAlg_t)alg));
        }
        HIP_OK(hipFree(buffer));
    }
    if (mf) std::fclose(mf);
    if (X) alphasparseDestroyDnVec(X);
    if (Y) alphasparseDestroyDnVec(Y);
    if (B) alphasparseDestroyDnMat(B);
    if (C) alphasparseDestroyDnMat(C);
    alphasparseDestroySpMat(A);
    alphasparse_destory_handle(handle);
    for (void *p : {(void *)d_row, (void *)d_col, (void *)d_val, (void *)d_rp, (void *)d_x, (void *)d_y}) (void)hipFree(p);
    asx_host_free(h_row);
    asx_host_free(h_col);
    asx_host_free(h_val_v);
    return all_ok ? 0 : 6;
}

}  // namespace

int main(int argc, char **argv)
{
    const Options o = parse(argc, argv);
    return o.data_type == 'D' ? run<double>(o) : run<float>(o);
}
