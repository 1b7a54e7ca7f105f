// A caller written the way the reference's own GPU tests drive the generic API
// (hip/test/level2/spmv_csr_r_f64_test.hip:143-217, hip/test/level3/spmm_csr_row_r_f32_test.hip):
// get a handle, put the CSR arrays on the device, wrap them in descriptors, ask for the buffer
// size, allocate it, call alphasparseSpMV / alphasparseSpMM, copy the result back.  It compiles
// against include/alphasparse.h of this repository and links libalphasparse_amd.so only.
//
//   generic_api_caller <case_dir>     run the case described by <case_dir>/meta.txt, write out.bin
//   generic_api_caller --selftest     error-path and life-cycle checks of the API on the device
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "alphasparse.h"

#define HIP_OK(e)                                                                          \
    do {                                                                                   \
        hipError_t _e = (e);                                                               \
        if (_e != hipSuccess) {                                                            \
            std::fprintf(stderr, "HIP error %s at %s:%d\n", hipGetErrorString(_e), __FILE__, __LINE__); \
            std::exit(2);                                                                  \
        }                                                                                  \
    } while (0)
#define EXPECT(cond)                                                                       \
    do {                                                                                   \
        if (!(cond)) {                                                                     \
            std::fprintf(stderr, "selftest failed: %s (%s:%d)\n", #cond, __FILE__, __LINE__); \
            std::exit(3);                                                                  \
        }                                                                                  \
    } while (0)

template <typename T>
static std::vector<T> read_bin(const std::string &path, size_t n)
{
    std::vector<T> v(n);
    FILE *f = std::fopen(path.c_str(), "rb");
    if (!f || std::fread(v.data(), sizeof(T), n, f) != n) {
        std::fprintf(stderr, "cannot read %zu items from %s\n", n, path.c_str());
        std::exit(2);
    }
    std::fclose(f);
    return v;
}
template <typename T>
static T *to_device(const std::vector<T> &h)
{
    T *d = nullptr;
    HIP_OK(hipMalloc((void **)&d, (h.size() ? h.size() : 1) * sizeof(T)));
    if (!h.empty()) HIP_OK(hipMemcpy(d, h.data(), h.size() * sizeof(T), hipMemcpyHostToDevice));
    return d;
}

// Operand variants of a case: opA / opB = TRANSPOSE, one-based indices, column-major B / C.
struct Variant {
    int trans_a = 0, base = 0, col_major_b = 0, col_major_c = 0, trans_b = 0;
};

template <typename T>
static int run_case(const std::string &dir, const char *op, long m, long n, long nnz, long ncols, int alg,
                    double alpha_d, double beta_d, int analysis, alphasparseDataType dt, const Variant &v)
{
    auto rp = read_bin<int>(dir + "/row_ptr.bin", m + 1);
    auto col = read_bin<int>(dir + "/col.bin", nnz);
    auto val = read_bin<T>(dir + "/val.bin", nnz);
    const bool mm = std::strcmp(op, "spmm") == 0;
    const long in_len = v.trans_a ? m : n, out_len = v.trans_a ? n : m;  // of op(A)
    auto xin = read_bin<T>(dir + "/x.bin", mm ? in_len * ncols : in_len);
    auto yin = read_bin<T>(dir + "/y.bin", mm ? out_len * ncols : out_len);
    const auto opA = v.trans_a ? ALPHA_SPARSE_OPERATION_TRANSPOSE : ALPHA_SPARSE_OPERATION_NON_TRANSPOSE;
    const auto opB = v.trans_b ? ALPHA_SPARSE_OPERATION_TRANSPOSE : ALPHA_SPARSE_OPERATION_NON_TRANSPOSE;
    int *d_rp = to_device(rp), *d_col = to_device(col);
    T *d_val = to_device(val), *d_x = to_device(xin), *d_y = to_device(yin);
    const T alpha = (T)alpha_d, beta = (T)beta_d;

    alphasparseHandle_t handle = nullptr;
    if (alphasparseGetHandle(&handle) != ALPHA_SPARSE_STATUS_SUCCESS) return 4;
    alphasparseSpMatDescr_t A;
    if (alphasparseCreateCsr(&A, (int)m, (int)n, (int)nnz, d_rp, d_col, d_val, ALPHA_SPARSE_INDEXTYPE_I32,
                             ALPHA_SPARSE_INDEXTYPE_I32,
                             v.base ? ALPHA_SPARSE_INDEX_BASE_ONE : ALPHA_SPARSE_INDEX_BASE_ZERO, dt))
        return 5;
    size_t bytes = 0;
    void *buffer = nullptr;
    alphasparseStatus_t s;
    if (!mm) {
        alphasparseDnVecDescr_t X, Y;
        if (alphasparseCreateDnVec(&X, in_len, d_x, dt) || alphasparseCreateDnVec(&Y, out_len, d_y, dt)) return 6;
        s = alphasparseSpMV_bufferSize(handle, opA, &alpha, A, X, &beta, Y, dt,
                                       (alphasparseSpMVAlg_t)alg, &bytes);
        if (s) return 10 + (int)s;
        HIP_OK(hipMalloc(&buffer, bytes ? bytes : 1));
        if (analysis && analysis != 5) {
            s = alphasparseSpMV_analysis(handle, opA, A, (alphasparseSpMVAlg_t)alg);
            if (s) return 30 + (int)s;
        }
        for (int rep = 0; rep < 2; ++rep) {  // twice: the second call must not depend on the first
            HIP_OK(hipMemcpy(d_y, yin.data(), yin.size() * sizeof(T), hipMemcpyHostToDevice));
            s = alphasparseSpMV(handle, opA, &alpha, A, X, &beta, Y, dt, (alphasparseSpMVAlg_t)alg, buffer);
            if (s) return 50 + (int)s;
        }
        if (!analysis || analysis == 5) {
            // analysis on first use: unless ALPHASPARSE_AMD_AUTO_ANALYSIS=0, the calls above left kept
            // analysis on the descriptor although alphasparseSpMV_analysis was never called ("1": the
            // full one, which may regroup A; unset: only what reads the caller's values in every call)
            const char *e = std::getenv("ALPHASPARSE_AMD_AUTO_ANALYSIS");
            const bool off = e && e[0] == '0';
            if (!v.trans_a && off == A->analysed) return 12;
        }
        std::printf("kernel %s\n", alphasparseAmdKeptKernel(A, opA, 0, alg, 1));
        if (analysis == 2) {
            // the caller changes A's values in place (same pattern) and says so by calling the
            // analysis again; the next product must use the new values
            auto val2 = read_bin<T>(dir + "/val2.bin", nnz);
            HIP_OK(hipStreamSynchronize(handle->stream));
            HIP_OK(hipMemcpy(d_val, val2.data(), val2.size() * sizeof(T), hipMemcpyHostToDevice));
            s = alphasparseSpMV_analysis(handle, opA, A, (alphasparseSpMVAlg_t)alg);
            if (s) return 70 + (int)s;
            HIP_OK(hipMemcpy(d_y, yin.data(), yin.size() * sizeof(T), hipMemcpyHostToDevice));
            s = alphasparseSpMV(handle, opA, &alpha, A, X, &beta, Y, dt, (alphasparseSpMVAlg_t)alg, buffer);
            if (s) return 50 + (int)s;
        }
        if (analysis == 5) {
            // a caller written for the reference: it never calls the analysis, changes A's values in
            // place (same pattern) and multiplies again; the product must use the new values, twice
            auto val2 = read_bin<T>(dir + "/val2.bin", nnz);
            HIP_OK(hipStreamSynchronize(handle->stream));
            HIP_OK(hipMemcpy(d_val, val2.data(), val2.size() * sizeof(T), hipMemcpyHostToDevice));
            for (int rep = 0; rep < 2; ++rep) {
                HIP_OK(hipMemcpy(d_y, yin.data(), yin.size() * sizeof(T), hipMemcpyHostToDevice));
                s = alphasparseSpMV(handle, opA, &alpha, A, X, &beta, Y, dt, (alphasparseSpMVAlg_t)alg, buffer);
                if (s) return 50 + (int)s;
            }
        }
        if (analysis == 3) {
            // a second descriptor that shares A's row offsets and columns but has its own values
            // (the usual "same pattern, new values" set-up): each descriptor must multiply with its
            // own values.  Its product goes to out2.bin; A's product is computed again afterwards.
            auto val2 = read_bin<T>(dir + "/val2.bin", nnz);
            T *d_val2 = to_device(val2);
            alphasparseSpMatDescr_t A2;
            if (alphasparseCreateCsr(&A2, (int)m, (int)n, (int)nnz, d_rp, d_col, d_val2, ALPHA_SPARSE_INDEXTYPE_I32,
                                     ALPHA_SPARSE_INDEXTYPE_I32,
                                     v.base ? ALPHA_SPARSE_INDEX_BASE_ONE : ALPHA_SPARSE_INDEX_BASE_ZERO, dt))
                return 5;
            s = alphasparseSpMV_analysis(handle, opA, A2, (alphasparseSpMVAlg_t)alg);
            if (s) return 70 + (int)s;
            HIP_OK(hipMemcpy(d_y, yin.data(), yin.size() * sizeof(T), hipMemcpyHostToDevice));
            s = alphasparseSpMV(handle, opA, &alpha, A2, X, &beta, Y, dt, (alphasparseSpMVAlg_t)alg, buffer);
            if (s) return 50 + (int)s;
            HIP_OK(hipStreamSynchronize(handle->stream));
            std::vector<T> out2(yin.size());
            HIP_OK(hipMemcpy(out2.data(), d_y, out2.size() * sizeof(T), hipMemcpyDeviceToHost));
            FILE *f2 = std::fopen((dir + "/out2.bin").c_str(), "wb");
            if (!f2 || std::fwrite(out2.data(), sizeof(T), out2.size(), f2) != out2.size()) return 9;
            std::fclose(f2);
            alphasparseDestroySpMat(A2);
            (void)hipFree(d_val2);
            HIP_OK(hipMemcpy(d_y, yin.data(), yin.size() * sizeof(T), hipMemcpyHostToDevice));
            s = alphasparseSpMV(handle, opA, &alpha, A, X, &beta, Y, dt, (alphasparseSpMVAlg_t)alg, buffer);
            if (s) return 50 + (int)s;
        }
        if (analysis == 4) {
            // two handles, each on a stream of its own, multiply the one analysed descriptor at the
            // same time, each call with its own buffer, sized after the analysis (it then holds the
            // call's partial sums or carries when the analysis regrouped A): x -> y as before,
            // x2 -> y2 (out2.bin)
            auto x2 = read_bin<T>(dir + "/x2.bin", in_len);
            T *d_x2 = to_device(x2), *d_y2 = to_device(yin);
            alphasparseHandle_t h2 = nullptr;
            if (alphasparseGetHandle(&h2) != ALPHA_SPARSE_STATUS_SUCCESS) return 4;
            handle->stream = handle->streams[0];
            h2->stream = h2->streams[0];
            alphasparseDnVecDescr_t X2, Y2;
            if (alphasparseCreateDnVec(&X2, in_len, d_x2, dt) || alphasparseCreateDnVec(&Y2, out_len, d_y2, dt)) return 6;
            size_t nb = 0;
            s = alphasparseSpMV_bufferSize(handle, opA, &alpha, A, X, &beta, Y, dt, (alphasparseSpMVAlg_t)alg, &nb);
            if (s) return 10 + (int)s;
            if (nb < bytes) return 8;
            void *b1 = nullptr, *b2 = nullptr;
            HIP_OK(hipMalloc(&b1, nb ? nb : 1));
            HIP_OK(hipMalloc(&b2, nb ? nb : 1));
            for (int rep = 0; rep < 6; ++rep) {
                HIP_OK(hipMemcpy(d_y, yin.data(), yin.size() * sizeof(T), hipMemcpyHostToDevice));
                HIP_OK(hipMemcpy(d_y2, yin.data(), yin.size() * sizeof(T), hipMemcpyHostToDevice));
                s = alphasparseSpMV(handle, opA, &alpha, A, X, &beta, Y, dt, (alphasparseSpMVAlg_t)alg, b1);
                if (s) return 50 + (int)s;
                s = alphasparseSpMV(h2, opA, &alpha, A, X2, &beta, Y2, dt, (alphasparseSpMVAlg_t)alg, b2);
                if (s) return 50 + (int)s;
                HIP_OK(hipStreamSynchronize(handle->stream));
                HIP_OK(hipStreamSynchronize(h2->stream));
            }
            std::vector<T> out2(yin.size());
            HIP_OK(hipMemcpy(out2.data(), d_y2, out2.size() * sizeof(T), hipMemcpyDeviceToHost));
            FILE *f2 = std::fopen((dir + "/out2.bin").c_str(), "wb");
            if (!f2 || std::fwrite(out2.data(), sizeof(T), out2.size(), f2) != out2.size()) return 9;
            std::fclose(f2);
            std::printf("buffer bytes before analysis %zu after %zu\n", bytes, nb);
            alphasparseDestroyDnVec(X2);
            alphasparseDestroyDnVec(Y2);
            alphasparse_destory_handle(h2);
            for (void *q : {(void *)b1, (void *)b2, (void *)d_x2, (void *)d_y2}) (void)hipFree(q);
        }
        if (analysis && alphasparseSpMV_clear(handle, (alphasparseSpMVAlg_t)alg)) return 7;
        alphasparseDestroyDnVec(X);
        alphasparseDestroyDnVec(Y);
    } else {
        alphasparseDnMatDescr_t B, C;
        // the arrays are packed: the leading dimension is the length of a row (row-major) or of a
        // column (column-major) of the matrix the descriptor describes
        const long b_rows = v.trans_b ? ncols : in_len, b_cols = v.trans_b ? in_len : ncols;
        if (alphasparseCreateDnMat(&B, b_rows, b_cols, v.col_major_b ? b_rows : b_cols, d_x, dt,
                                   v.col_major_b ? ALPHASPARSE_ORDER_COL : ALPHASPARSE_ORDER_ROW) ||
            alphasparseCreateDnMat(&C, out_len, ncols, v.col_major_c ? out_len : ncols, d_y, dt,
                                   v.col_major_c ? ALPHASPARSE_ORDER_COL : ALPHASPARSE_ORDER_ROW))
            return 6;
        s = alphasparseSpMM_bufferSize(handle, opA, opB, &alpha, A, B, &beta, C, dt, (alphasparseSpMMAlg_t)alg, &bytes);
        if (s) return 10 + (int)s;
        HIP_OK(hipMalloc(&buffer, bytes ? bytes : 1));
        if (analysis) {
            size_t b2 = 0;
            s = alphasparseSpMM_preprocess(handle, opA, opB, &alpha, A, B, &beta, C, dt, (alphasparseSpMMAlg_t)alg, &b2);
            if (s) return 30 + (int)s;
            if (b2 > bytes) return 8;
        }
        for (int rep = 0; rep < 2; ++rep) {
            HIP_OK(hipMemcpy(d_y, yin.data(), yin.size() * sizeof(T), hipMemcpyHostToDevice));
            s = alphasparseSpMM(handle, opA, opB, &alpha, A, B, &beta, C, dt, (alphasparseSpMMAlg_t)alg, buffer);
            if (s) return 50 + (int)s;
        }
        if (!analysis && alg != 10) {
            const char *e = std::getenv("ALPHASPARSE_AMD_AUTO_ANALYSIS");
            const bool off = e && e[0] == '0';
            if (!v.trans_a && off == A->analysed) return 12;
        }
        std::printf("kernel %s\n", alphasparseAmdKeptKernel(A, opA, 1, alg, (int)ncols));
        if (analysis == 2) {  // new values in place, preprocess again, multiply again
            auto val2 = read_bin<T>(dir + "/val2.bin", nnz);
            HIP_OK(hipStreamSynchronize(handle->stream));
            HIP_OK(hipMemcpy(d_val, val2.data(), val2.size() * sizeof(T), hipMemcpyHostToDevice));
            size_t b2 = 0;
            s = alphasparseSpMM_preprocess(handle, opA, opB, &alpha, A, B, &beta, C, dt, (alphasparseSpMMAlg_t)alg, &b2);
            if (s) return 70 + (int)s;
            if (b2 > bytes) return 8;
            HIP_OK(hipMemcpy(d_y, yin.data(), yin.size() * sizeof(T), hipMemcpyHostToDevice));
            s = alphasparseSpMM(handle, opA, opB, &alpha, A, B, &beta, C, dt, (alphasparseSpMMAlg_t)alg, buffer);
            if (s) return 50 + (int)s;
        }
        alphasparseDestroyDnMat(B);
        alphasparseDestroyDnMat(C);
    }
    HIP_OK(hipStreamSynchronize(handle->stream));
    std::vector<T> out(yin.size());
    HIP_OK(hipMemcpy(out.data(), d_y, out.size() * sizeof(T), hipMemcpyDeviceToHost));
    FILE *f = std::fopen((dir + "/out.bin").c_str(), "wb");
    if (!f || std::fwrite(out.data(), sizeof(T), out.size(), f) != out.size()) return 9;
    std::fclose(f);
    alphasparseDestroySpMat(A);
    alphasparse_destory_handle(handle);
    for (void *p : {(void *)buffer, (void *)d_rp, (void *)d_col, (void *)d_val, (void *)d_x, (void *)d_y}) (void)hipFree(p);
    return 0;
}

static int selftest()
{
    alphasparseHandle_t h = nullptr;
    EXPECT(alphasparseGetHandle(&h) == ALPHA_SPARSE_STATUS_SUCCESS);
    EXPECT(h && h->wavefront_size == 64 && h->buffer && h->buffer_size >= (1u << 20));
    std::vector<int> rp = {0, 2, 3}, col = {0, 1, 1};
    std::vector<double> val = {1, 2, 3}, x = {1, 10}, y = {100, 100};
    int *d_rp = to_device(rp), *d_col = to_device(col);
    double *d_val = to_device(val), *d_x = to_device(x), *d_y = to_device(y);
    alphasparseSpMatDescr_t A;
    EXPECT(alphasparseCreateCsr(&A, 2, 2, 3, d_rp, d_col, d_val, ALPHA_SPARSE_INDEXTYPE_I32, ALPHA_SPARSE_INDEXTYPE_I32,
                                ALPHA_SPARSE_INDEX_BASE_ZERO, ALPHA_R_64F) == 0);
    EXPECT(A->format == ALPHA_SPARSE_FORMAT_CSR && A->rows == 2 && A->nnz == 3 && A->row_data == d_rp && A->descr);
    alphasparseDnVecDescr_t X, Y, Xf;
    EXPECT(alphasparseCreateDnVec(&X, 2, d_x, ALPHA_R_64F) == 0 && alphasparseCreateDnVec(&Y, 2, d_y, ALPHA_R_64F) == 0);
    EXPECT(alphasparseCreateDnVec(&Xf, 2, d_x, ALPHA_R_32F) == 0);
    const double alpha = 2.0, beta = 0.5;
    const auto N = ALPHA_SPARSE_OPERATION_NON_TRANSPOSE;
    size_t bytes = 123;
    // DEFAULT runs a kernel and the handle's own scratch serves a call without a caller's buffer
    EXPECT(alphasparseSpMV(h, N, &alpha, A, X, &beta, Y, ALPHA_R_64F, ALPHA_SPARSE_SPMV_ALG_DEFAULT, nullptr) == 0);
    HIP_OK(hipDeviceSynchronize());
    HIP_OK(hipMemcpy(y.data(), d_y, sizeof(double) * 2, hipMemcpyDeviceToHost));
    EXPECT(y[0] == 2.0 * 21.0 + 50.0 && y[1] == 2.0 * 30.0 + 50.0);
    // opA = TRANSPOSE computes with A^T = [[1,0],[2,3]] and leaves the caller's arrays as they were
    HIP_OK(hipMemcpy(d_y, x.data(), sizeof(double) * 2, hipMemcpyHostToDevice));
    for (int rep = 0; rep < 2; ++rep) {
        HIP_OK(hipMemcpy(d_y, x.data(), sizeof(double) * 2, hipMemcpyHostToDevice));
        EXPECT(alphasparseSpMV(h, ALPHA_SPARSE_OPERATION_TRANSPOSE, &alpha, A, X, &beta, Y, ALPHA_R_64F,
                               ALPHA_SPARSE_SPMV_ALG_DEFAULT, nullptr) == 0);
        HIP_OK(hipDeviceSynchronize());
        HIP_OK(hipMemcpy(y.data(), d_y, sizeof(double) * 2, hipMemcpyDeviceToHost));
        EXPECT(y[0] == 2.0 * 1.0 + 0.5 && y[1] == 2.0 * 32.0 + 5.0);
    }
    {
        std::vector<int> rp2(3), col2(3);
        std::vector<double> val2(3);
        HIP_OK(hipMemcpy(rp2.data(), d_rp, sizeof(int) * 3, hipMemcpyDeviceToHost));
        HIP_OK(hipMemcpy(col2.data(), d_col, sizeof(int) * 3, hipMemcpyDeviceToHost));
        HIP_OK(hipMemcpy(val2.data(), d_val, sizeof(double) * 3, hipMemcpyDeviceToHost));
        EXPECT(rp2 == rp && col2 == col && val2 == val);
    }
    // what is not supported says so
    EXPECT(alphasparseSpMV(h, N, &alpha, A, Xf, &beta, Y, ALPHA_R_64F, ALPHA_SPARSE_SPMV_ALG_DEFAULT, nullptr) ==
           ALPHA_SPARSE_STATUS_NOT_SUPPORTED);
    EXPECT(alphasparseSpMV(h, N, &alpha, A, X, &beta, Y, ALPHA_R_64F, ALPHA_SPARSE_SPMV_ALG_COO, nullptr) ==
           ALPHA_SPARSE_STATUS_NOT_SUPPORTED);
    EXPECT(alphasparseSpMV(nullptr, N, &alpha, A, X, &beta, Y, ALPHA_R_64F, ALPHA_SPARSE_SPMV_ALG_DEFAULT, nullptr) ==
           ALPHA_SPARSE_STATUS_INVALID_HANDLE);
    EXPECT(alphasparseSpMV(h, N, nullptr, A, X, &beta, Y, ALPHA_R_64F, ALPHA_SPARSE_SPMV_ALG_DEFAULT, nullptr) ==
           ALPHA_SPARSE_STATUS_INVALID_POINTER);
    EXPECT(alphasparseSpMV_bufferSize(h, N, &alpha, A, X, &beta, Y, ALPHA_R_64F, ALPHA_SPARSE_SPMV_ALG_VECTOR, &bytes) == 0 &&
           bytes == 0);
    EXPECT(alphasparseSpMV_bufferSize(h, N, &alpha, A, X, &beta, Y, ALPHA_R_64F, ALPHA_SPARSE_SPMV_ALG_MERGE, &bytes) == 0 &&
           bytes > 0);
    // one-based indices
    {
        std::vector<int> rp1 = {1, 3, 4}, col1 = {1, 2, 2};
        int *d_rp1 = to_device(rp1), *d_col1 = to_device(col1);
        alphasparseSpMatDescr_t A1;
        EXPECT(alphasparseCreateCsr(&A1, 2, 2, 3, d_rp1, d_col1, d_val, ALPHA_SPARSE_INDEXTYPE_I32,
                                    ALPHA_SPARSE_INDEXTYPE_I32, ALPHA_SPARSE_INDEX_BASE_ONE, ALPHA_R_64F) == 0);
        HIP_OK(hipMemcpy(d_y, x.data(), sizeof(double) * 2, hipMemcpyHostToDevice));
        EXPECT(alphasparseSpMV(h, N, &alpha, A1, X, &beta, Y, ALPHA_R_64F, ALPHA_SPARSE_SPMV_ALG_DEFAULT, nullptr) == 0);
        HIP_OK(hipDeviceSynchronize());
        HIP_OK(hipMemcpy(y.data(), d_y, sizeof(double) * 2, hipMemcpyDeviceToHost));
        EXPECT(y[0] == 42.5 && y[1] == 65.0);
        // kept copy: analysis, two calls, clear
        EXPECT(alphasparseSpMV_analysis(h, ALPHA_SPARSE_OPERATION_TRANSPOSE, A1, ALPHA_SPARSE_SPMV_ALG_MERGE) == 0);
        size_t nb = 0;
        EXPECT(alphasparseSpMV_bufferSize(h, ALPHA_SPARSE_OPERATION_TRANSPOSE, &alpha, A1, X, &beta, Y, ALPHA_R_64F,
                                          ALPHA_SPARSE_SPMV_ALG_MERGE, &nb) == 0);
        void *tb = nullptr;
        HIP_OK(hipMalloc(&tb, nb ? nb : 1));
        for (int rep = 0; rep < 2; ++rep) {
            HIP_OK(hipMemcpy(d_y, x.data(), sizeof(double) * 2, hipMemcpyHostToDevice));
            EXPECT(alphasparseSpMV(h, ALPHA_SPARSE_OPERATION_TRANSPOSE, &alpha, A1, X, &beta, Y, ALPHA_R_64F,
                                   ALPHA_SPARSE_SPMV_ALG_MERGE, tb) == 0);
            HIP_OK(hipDeviceSynchronize());
            HIP_OK(hipMemcpy(y.data(), d_y, sizeof(double) * 2, hipMemcpyDeviceToHost));
            EXPECT(y[0] == 2.5 && y[1] == 69.0);
        }
        EXPECT(alphasparseSpMV_clear(h, ALPHA_SPARSE_SPMV_ALG_MERGE) == 0);
        alphasparseDestroySpMat(A1);
        (void)hipFree(tb);
        (void)hipFree(d_rp1);
        (void)hipFree(d_col1);
    }
    EXPECT(alphasparseSpMV(h, (alphasparseOperation_t)7, &alpha, A, X, &beta, Y, ALPHA_R_64F,
                           ALPHA_SPARSE_SPMV_ALG_DEFAULT, nullptr) == ALPHA_SPARSE_STATUS_INVALID_VALUE);
    // analysis is kept on the matrix (matA->info), found again, and cleared through the handle
    EXPECT(alphasparseSpMV_analysis(h, N, A, ALPHA_SPARSE_SPMV_ALG_DEFAULT) == 0 && A->analysed);
    EXPECT(A->info && A->info->csrmv_info && A->info->csrmv_info->m == 2 && A->info->csrmv_info->nnz == 3 &&
           A->info->csrmv_info->csr_row_ptr == d_rp);
    EXPECT(alphasparseSpMV_analysis(h, N, A, ALPHA_SPARSE_SPMV_ALG_DEFAULT) == 0);
    HIP_OK(hipMemcpy(d_y, x.data(), sizeof(double) * 2, hipMemcpyHostToDevice));
    EXPECT(alphasparseSpMV(h, N, &alpha, A, X, &beta, Y, ALPHA_R_64F, ALPHA_SPARSE_SPMV_ALG_DEFAULT, nullptr) == 0);
    HIP_OK(hipDeviceSynchronize());
    HIP_OK(hipMemcpy(y.data(), d_y, sizeof(double) * 2, hipMemcpyDeviceToHost));
    EXPECT(y[0] == 42.5 && y[1] == 65.0);
    EXPECT(alphasparseSpMV_clear(h, ALPHA_SPARSE_SPMV_ALG_DEFAULT) == 0);
    // an object of the caller's own behind matA->info (the reference's 176-byte struct) is left
    // alone: no analysis is kept there, and products still work
    {
        _alphasparse_mat_info *foreign = new _alphasparse_mat_info();
        alphasparseSpMatDescr_t F;
        EXPECT(alphasparseCreateCsr(&F, 2, 2, 3, d_rp, d_col, d_val, ALPHA_SPARSE_INDEXTYPE_I32, ALPHA_SPARSE_INDEXTYPE_I32,
                                    ALPHA_SPARSE_INDEX_BASE_ZERO, ALPHA_R_64F) == 0);
        F->info = foreign;
        EXPECT(alphasparseSpMV_analysis(h, N, F, ALPHA_SPARSE_SPMV_ALG_DEFAULT) == ALPHA_SPARSE_STATUS_NOT_SUPPORTED);
        EXPECT(alphasparseSpMV_bufferSize(h, N, &alpha, F, X, &beta, Y, ALPHA_R_64F, ALPHA_SPARSE_SPMV_ALG_DEFAULT, &bytes) == 0);
        EXPECT(F->info == foreign && !F->analysed);
        HIP_OK(hipMemcpy(d_y, x.data(), sizeof(double) * 2, hipMemcpyHostToDevice));
        EXPECT(alphasparseSpMV(h, N, &alpha, F, X, &beta, Y, ALPHA_R_64F, ALPHA_SPARSE_SPMV_ALG_DEFAULT, nullptr) == 0);
        HIP_OK(hipDeviceSynchronize());
        HIP_OK(hipMemcpy(y.data(), d_y, sizeof(double) * 2, hipMemcpyDeviceToHost));
        EXPECT(y[0] == 42.5 && y[1] == 65.0);
        F->info = nullptr;
        alphasparseDestroySpMat(F);
        delete foreign;
    }
    // two-phase form: size query, then compute
    {
        size_t need = 0;
        EXPECT(alphasparse_spmv(h, N, &alpha, A, X, &beta, Y, ALPHA_SPARSE_DATATYPE_DOUBLE,
                                ALPHA_SPARSE_DCU_SPMV_ALG_CSR_ADAPTIVE, &need, nullptr) == 0);
        void *tb = nullptr;
        HIP_OK(hipMalloc(&tb, need ? need : 1));
        HIP_OK(hipMemcpy(d_y, x.data(), sizeof(double) * 2, hipMemcpyHostToDevice));
        EXPECT(alphasparse_spmv(h, N, &alpha, A, X, &beta, Y, ALPHA_SPARSE_DATATYPE_DOUBLE,
                                ALPHA_SPARSE_DCU_SPMV_ALG_CSR_ADAPTIVE, &need, tb) == 0);
        HIP_OK(hipDeviceSynchronize());
        HIP_OK(hipMemcpy(y.data(), d_y, sizeof(double) * 2, hipMemcpyDeviceToHost));
        EXPECT(y[0] == 42.5 && y[1] == 65.0);
        EXPECT(alphasparse_spmv(h, N, &alpha, A, X, &beta, Y, ALPHA_SPARSE_DATATYPE_FLOAT_COMPLEX,
                                ALPHA_SPARSE_DCU_SPMV_ALG_DEFAULT, &need, nullptr) == ALPHA_SPARSE_STATUS_NOT_SUPPORTED);
        (void)hipFree(tb);
    }
    // HIP graph: with kept analysis and a caller's buffer a call is kernels only (no allocation, no
    // copy, no synchronisation), so it can be captured once and replayed; every replay must give
    // the eager result bit for bit
    {
        const int gm = 6000, per = 7;
        std::vector<int> grp(gm + 1), gcol((size_t)gm * per);
        std::vector<double> gval(gcol.size()), gx(gm), gy0(gm), eager(gm), replay(gm);
        for (int i = 0; i <= gm; ++i) grp[i] = i * per;
        for (int i = 0; i < gm; ++i)
            for (int j = 0; j < per; ++j) {
                gcol[(size_t)i * per + j] = (int)(((long)i * 31 + (long)j * 977) % gm);
                gval[(size_t)i * per + j] = 0.25 + 0.001 * ((i + 3 * j) % 17);
            }
        for (int i = 0; i < gm; ++i) gx[i] = 1.0 + 0.01 * (i % 13), gy0[i] = 0.5 - 0.002 * (i % 7);
        int *g_rp = to_device(grp), *g_col = to_device(gcol);
        double *g_val = to_device(gval), *g_x = to_device(gx), *g_y = to_device(gy0);
        alphasparseSpMatDescr_t GA;
        alphasparseDnVecDescr_t GX, GY;
        EXPECT(alphasparseCreateCsr(&GA, gm, gm, gm * per, g_rp, g_col, g_val, ALPHA_SPARSE_INDEXTYPE_I32,
                                    ALPHA_SPARSE_INDEXTYPE_I32, ALPHA_SPARSE_INDEX_BASE_ZERO, ALPHA_R_64F) == 0);
        EXPECT(alphasparseCreateDnVec(&GX, gm, g_x, ALPHA_R_64F) == 0 && alphasparseCreateDnVec(&GY, gm, g_y, ALPHA_R_64F) == 0);
        h->stream = h->streams[0];  // capture needs a stream of its own, not the null stream
        for (alphasparseSpMVAlg_t galg : {ALPHA_SPARSE_SPMV_ALG_MERGE, ALPHA_SPARSE_SPMV_ALG_FLAT8}) {
            size_t nb = 0;
            EXPECT(alphasparseSpMV_bufferSize(h, N, &alpha, GA, GX, &beta, GY, ALPHA_R_64F, galg, &nb) == 0);
            void *gb = nullptr;
            HIP_OK(hipMalloc(&gb, nb ? nb : 1));
            EXPECT(alphasparseSpMV_analysis(h, N, GA, galg) == 0);
            EXPECT(alphasparseSpMV(h, N, &alpha, GA, GX, &beta, GY, ALPHA_R_64F, galg, gb) == 0);
            HIP_OK(hipStreamSynchronize(h->stream));
            HIP_OK(hipMemcpy(eager.data(), g_y, sizeof(double) * gm, hipMemcpyDeviceToHost));
            hipGraph_t graph;
            hipGraphExec_t exec;
            HIP_OK(hipStreamBeginCapture(h->stream, hipStreamCaptureModeGlobal));
            EXPECT(alphasparseSpMV(h, N, &alpha, GA, GX, &beta, GY, ALPHA_R_64F, galg, gb) == 0);
            HIP_OK(hipStreamEndCapture(h->stream, &graph));
            HIP_OK(hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0));
            for (int rep = 0; rep < 3; ++rep) {
                HIP_OK(hipMemcpy(g_y, gy0.data(), sizeof(double) * gm, hipMemcpyHostToDevice));
                HIP_OK(hipGraphLaunch(exec, h->stream));
                HIP_OK(hipStreamSynchronize(h->stream));
                HIP_OK(hipMemcpy(replay.data(), g_y, sizeof(double) * gm, hipMemcpyDeviceToHost));
                EXPECT(replay == eager);
            }
            HIP_OK(hipGraphExecDestroy(exec));
            HIP_OK(hipGraphDestroy(graph));
            EXPECT(alphasparseSpMV_clear(h, galg) == 0);
            (void)hipFree(gb);
            HIP_OK(hipMemcpy(g_y, gy0.data(), sizeof(double) * gm, hipMemcpyHostToDevice));
        }
        h->stream = nullptr;
        alphasparseDestroySpMat(GA);
        alphasparseDestroyDnVec(GX);
        alphasparseDestroyDnVec(GY);
        for (void *p : {(void *)g_rp, (void *)g_col, (void *)g_val, (void *)g_x, (void *)g_y}) (void)hipFree(p);
    }
    // COO -> CSR through the reference's name
    {
        std::vector<int> ri = {0, 0, 1};
        int *d_ri = to_device(ri), *d_out = nullptr;
        HIP_OK(hipMalloc((void **)&d_out, 3 * sizeof(int)));
        EXPECT(alphasparseXcoo2csr(d_ri, 3, 2, d_out) == 0);
        HIP_OK(hipDeviceSynchronize());
        int out[3];
        HIP_OK(hipMemcpy(out, d_out, sizeof out, hipMemcpyDeviceToHost));
        EXPECT(out[0] == 0 && out[1] == 2 && out[2] == 3);
        (void)hipFree(d_ri);
        (void)hipFree(d_out);
    }
    // SpMM: row-major and column-major operands; a leading dimension shorter than a column is refused
    alphasparseDnMatDescr_t B, C, Bc, Bbad;
    EXPECT(alphasparseCreateDnMat(&B, 2, 1, 1, d_x, ALPHA_R_64F, ALPHASPARSE_ORDER_ROW) == 0);
    EXPECT(alphasparseCreateDnMat(&C, 2, 1, 1, d_y, ALPHA_R_64F, ALPHASPARSE_ORDER_ROW) == 0);
    EXPECT(alphasparseCreateDnMat(&Bc, 2, 1, 2, d_x, ALPHA_R_64F, ALPHASPARSE_ORDER_COL) == 0);
    EXPECT(alphasparseCreateDnMat(&Bbad, 2, 1, 1, d_x, ALPHA_R_64F, ALPHASPARSE_ORDER_COL) == 0);
    EXPECT(alphasparseSpMM(h, N, N, &alpha, A, Bbad, &beta, C, ALPHA_R_64F, ALPHASPARSE_SPMM_ALG_DEFAULT, nullptr) ==
           ALPHA_SPARSE_STATUS_INVALID_SIZE);
    {
        size_t nb = 0;
        EXPECT(alphasparseSpMM_bufferSize(h, N, N, &alpha, A, Bc, &beta, C, ALPHA_R_64F, ALPHASPARSE_SPMM_ALG_DEFAULT,
                                          &nb) == 0 && nb > 0);
        void *tb = nullptr;
        HIP_OK(hipMalloc(&tb, nb));
        HIP_OK(hipMemcpy(d_y, x.data(), sizeof(double) * 2, hipMemcpyHostToDevice));
        EXPECT(alphasparseSpMM(h, N, N, &alpha, A, Bc, &beta, C, ALPHA_R_64F, ALPHASPARSE_SPMM_ALG_DEFAULT, tb) == 0);
        HIP_OK(hipDeviceSynchronize());
        HIP_OK(hipMemcpy(y.data(), d_y, sizeof(double) * 2, hipMemcpyDeviceToHost));
        EXPECT(y[0] == 42.5 && y[1] == 65.0);
        (void)hipFree(tb);
    }
    EXPECT(alphasparseSpMM(h, N, N, &alpha, A, B, &beta, C, ALPHA_R_64F, ALPHASPARSE_SPMM_COO_ALG1, nullptr) ==
           ALPHA_SPARSE_STATUS_NOT_SUPPORTED);
    HIP_OK(hipMemcpy(d_y, x.data(), sizeof(double) * 2, hipMemcpyHostToDevice));
    EXPECT(alphasparseSpMM(h, N, N, &alpha, A, B, &beta, C, ALPHA_R_64F, ALPHASPARSE_SPMM_ALG_DEFAULT, nullptr) == 0);
    HIP_OK(hipDeviceSynchronize());
    HIP_OK(hipMemcpy(y.data(), d_y, sizeof(double) * 2, hipMemcpyDeviceToHost));
    EXPECT(y[0] == 42.5 && y[1] == 65.0);
    EXPECT(alphasparse_destory_handle(h) == 0);
    std::printf("selftest ok\n");
    return 0;
}

int main(int argc, char **argv)
{
    if (argc != 2) {
        std::fprintf(stderr, "usage: %s <case_dir> | --selftest\n", argv[0]);
        return 1;
    }
    if (std::strcmp(argv[1], "--selftest") == 0) return selftest();
    const std::string dir = argv[1];
    FILE *f = std::fopen((dir + "/meta.txt").c_str(), "r");
    if (!f) return 1;
    char op[16], dtype[16];
    long m, n, nnz, ncols;
    int alg, analysis;
    double alpha, beta;
    if (std::fscanf(f, "%15s %15s %ld %ld %ld %ld %d %lf %lf %d", op, dtype, &m, &n, &nnz, &ncols, &alg, &alpha, &beta,
                    &analysis) != 10)
        return 1;
    Variant v;  // optional: trans_a base col_major_b col_major_c trans_b
    if (std::fscanf(f, "%d %d %d %d %d", &v.trans_a, &v.base, &v.col_major_b, &v.col_major_c, &v.trans_b) < 0) v = Variant();
    std::fclose(f);
    int rc = std::strcmp(dtype, "f64") == 0
                 ? run_case<double>(dir, op, m, n, nnz, ncols, alg, alpha, beta, analysis, ALPHA_R_64F, v)
                 : run_case<float>(dir, op, m, n, nnz, ncols, alg, alpha, beta, analysis, ALPHA_R_32F, v);
    std::printf("rc %d\n", rc);
    return rc;
}
