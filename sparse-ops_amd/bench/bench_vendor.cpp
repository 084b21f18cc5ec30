// Stand-alone benchmark in the style of the reference's benchmark-mkl/ harness
// (benchmark-mkl/matmul/main_matmul.cpp:49-139, benchmark-mkl/matvec/main_matvec.cpp:49-132):
// same flags (--M --N --C --sparsity --runs --seed --irregular), same data recipe
// (N(0,1) values under an i.i.d. Bernoulli mask, optionally a dense last row; X ~ U(-1,1);
// no bias; benchmark-mkl/common/data_gen.cpp:23-96), 1 warm-up then the median of --runs,
// reported in microseconds.  The matrices come from data_gen.hpp, which Python reaches too
// (sparseops_backend.benchmark_dense): one seed, one matrix on both sides.  --ellpack-file <path> replaces
// the generated matrix by one written by python/datagen.py's save_ellpack (any of the
// benchmark configurations), so the very same matrix runs here and in bench.py.  The comparators are the ROCm counterparts of the reference's:
// rocSPARSE CSR SpMM / SpMV for MKL sparse, rocBLAS SGEMM / SGEMV for the dense BLAS, and
// this library's so_matmul (row-per-wave and LDS-staged) / so_matvec for "Ellpack".
//
//   bench_vendor matmul --M 4096 --N 4096 --C 256 --sparsity 0.9 --runs 100
//   bench_vendor matvec --M 16384 --N 16384 --sparsity 0.95 --runs 100
//   bench_vendor matmul --ellpack-file config3.ellpack --C 256 --runs 100
#include <hip/hip_runtime.h>
#include <rocblas/rocblas.h>
#include <rocsparse/rocsparse.h>

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <string>
#include <vector>

#include "data_gen.hpp"
#include "sparseops_hip.h"

#define HIPCK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { std::fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_)); std::exit(2); } } while (0)
#define SPCK(x) do { rocsparse_status s_ = (x); if (s_ != rocsparse_status_success) { std::fprintf(stderr, "%s: rocsparse status %d\n", #x, (int)s_); std::exit(2); } } while (0)
#define BLCK(x) do { rocblas_status s_ = (x); if (s_ != rocblas_status_success) { std::fprintf(stderr, "%s: rocblas status %d\n", #x, (int)s_); std::exit(2); } } while (0)
#define SOCK(x) do { so_status s_ = (x); if (s_ != SO_OK) { std::fprintf(stderr, "%s: %s\n", #x, so_last_error()); std::exit(2); } } while (0)

namespace {

struct Host {
    int64_t M = 0, N = 0;
    std::vector<float> W;                    // dense row-major
    std::vector<int> row_ptr, col_ind;       // CSR
    std::vector<float> values;
    uint32_t r = 0;                          // ELLPACK
    std::vector<float> Wd;
    std::vector<uint32_t> idx, nnz;
};

// CSR and ELLPACK views of the dense matrix in h.W.
void derive_formats(Host &h);

Host generate(int64_t M, int64_t N, double sparsity, uint64_t seed, bool irregular)
{
    Host h;
    h.M = M; h.N = N;
    h.W = sparseops_bench::dense_matrix(M, N, sparsity, seed, irregular);
    derive_formats(h);
    return h;
}

// A matrix written by python/datagen.py save_ellpack: "SOELLPK1", uint32 m, n, r, 0, then nnz[m],
// idx[m*r] (uint32) and Wd[m*r] (float), little endian.
Host load_ellpack_file(const char *path)
{
    std::FILE *f = std::fopen(path, "rb");
    if (!f) { std::fprintf(stderr, "cannot open %s\n", path); std::exit(2); }
    char magic[8];
    uint32_t hdr[4];
    if (std::fread(magic, 1, 8, f) != 8 || std::memcmp(magic, "SOELLPK1", 8) != 0 || std::fread(hdr, 4, 4, f) != 4) {
        std::fprintf(stderr, "%s: not an ELLPACK file\n", path);
        std::exit(2);
    }
    Host h;
    h.M = hdr[0]; h.N = hdr[1];
    const uint32_t r = hdr[2];
    const size_t slots = size_t(h.M) * r;
    std::vector<uint32_t> nnz(h.M), idx(slots);
    std::vector<float> Wd(slots);
    if (std::fread(nnz.data(), 4, nnz.size(), f) != nnz.size() || std::fread(idx.data(), 4, slots, f) != slots ||
        std::fread(Wd.data(), 4, slots, f) != slots) {
        std::fprintf(stderr, "%s: truncated\n", path);
        std::exit(2);
    }
    std::fclose(f);
    h.W.assign(size_t(h.M) * h.N, 0.0f);
    for (int64_t i = 0; i < h.M; ++i) {
        if (nnz[i] > r) { std::fprintf(stderr, "%s: nnz[%lld] exceeds r\n", path, (long long)i); std::exit(2); }
        for (uint32_t k = 0; k < nnz[i]; ++k) {
            const uint32_t j = idx[size_t(i) * r + k];
            if (j >= h.N) { std::fprintf(stderr, "%s: column out of range\n", path); std::exit(2); }
            h.W[size_t(i) * h.N + j] = Wd[size_t(i) * r + k];
        }
    }
    derive_formats(h);
    return h;
}

void derive_formats(Host &h)
{
    const int64_t M = h.M, N = h.N;
    h.row_ptr.assign(M + 1, 0);
    h.nnz.assign(M, 0);
    for (int64_t i = 0; i < M; ++i) {
        for (int64_t j = 0; j < N; ++j) {
            const float v = h.W[size_t(i) * N + j];
            if (v != 0.0f) { h.col_ind.push_back(int(j)); h.values.push_back(v); ++h.nnz[i]; }
        }
        h.row_ptr[i + 1] = int(h.values.size());
        h.r = std::max(h.r, h.nnz[i]);
    }
    h.Wd.assign(size_t(M) * h.r, 0.0f);
    h.idx.assign(size_t(M) * h.r, 0u);
    for (int64_t i = 0; i < M; ++i)
        for (uint32_t k = 0; k < h.nnz[i]; ++k) {
            h.Wd[size_t(i) * h.r + k] = h.values[h.row_ptr[i] + k];
            h.idx[size_t(i) * h.r + k] = uint32_t(h.col_ind[h.row_ptr[i] + k]);
        }
}

template <typename T>
T *to_device(const std::vector<T> &v)
{
    T *d = nullptr;
    HIPCK(hipMalloc(&d, std::max<size_t>(v.size(), 1) * sizeof(T)));
    if (!v.empty()) HIPCK(hipMemcpy(d, v.data(), v.size() * sizeof(T), hipMemcpyHostToDevice));
    return d;
}

// 1 warm-up, then the median over `runs` of one synchronised call each, in microseconds
// (the reference times each call with a host clock, benchmark-mkl/matmul/bench_matmul.cpp:97-116;
// here each call is bracketed by HIP events on `stream`).
template <typename F>
double median_us(hipStream_t stream, int runs, F &&call)
{
    hipEvent_t e0, e1;
    HIPCK(hipEventCreate(&e0));
    HIPCK(hipEventCreate(&e1));
    call();
    HIPCK(hipStreamSynchronize(stream));
    std::vector<double> t;
    for (int i = 0; i < runs; ++i) {
        HIPCK(hipEventRecord(e0, stream));
        call();
        HIPCK(hipEventRecord(e1, stream));
        HIPCK(hipEventSynchronize(e1));
        float ms = 0;
        HIPCK(hipEventElapsedTime(&ms, e0, e1));
        t.push_back(ms * 1e3);
    }
    std::nth_element(t.begin(), t.begin() + t.size() / 2, t.end());
    HIPCK(hipEventDestroy(e0));
    HIPCK(hipEventDestroy(e1));
    return t[t.size() / 2];
}

double max_rel_diff(const std::vector<float> &a, const std::vector<float> &b)
{
    double num = 0, den = 1e-30;
    for (size_t i = 0; i < a.size(); ++i) {
        num = std::max(num, std::fabs(double(a[i]) - double(b[i])));
        den = std::max(den, std::fabs(double(b[i])));
    }
    return num / den;
}

std::vector<float> fetch(const float *d, size_t n)
{
    std::vector<float> h(n);
    HIPCK(hipDeviceSynchronize());
    HIPCK(hipMemcpy(h.data(), d, n * sizeof(float), hipMemcpyDeviceToHost));
    return h;
}

} // namespace

int main(int argc, char **argv)
{
    if (argc < 2 || (std::strcmp(argv[1], "matmul") && std::strcmp(argv[1], "matvec"))) {
        std::fprintf(stderr, "usage: %s matmul|matvec --M <rows> --N <cols> [--C <cols of X>] --sparsity <p> --runs <r> "
                             "--seed <s> --irregular <0|1> [--device <id>] [--ellpack-file <path>]\n", argv[0]);
        return 1;
    }
    const bool matmul = !std::strcmp(argv[1], "matmul");
    int64_t M = 1000, N = 1000;
    int C = 128, runs = 100;
    double sparsity = 0.9;
    uint64_t seed = 42;
    bool irregular = false;
    int device = 0;
    const char *ellpack_file = nullptr;
    for (int i = 2; i < argc; ++i) {
        const std::string a = argv[i];
        if (i + 1 >= argc) { std::fprintf(stderr, "incomplete arg: %s\n", a.c_str()); return 1; }
        if (a == "--M") M = std::stoll(argv[++i]);
        else if (a == "--N") N = std::stoll(argv[++i]);
        else if (a == "--C") C = std::stoi(argv[++i]);
        else if (a == "--sparsity") sparsity = std::stod(argv[++i]);
        else if (a == "--runs") runs = std::stoi(argv[++i]);
        else if (a == "--seed") seed = std::stoull(argv[++i]);
        else if (a == "--irregular") irregular = std::stoi(argv[++i]) != 0;
        else if (a == "--device") device = std::stoi(argv[++i]);
        else if (a == "--ellpack-file") ellpack_file = argv[++i];
        else { std::fprintf(stderr, "unknown arg: %s\n", a.c_str()); return 1; }
    }
    if (!matmul) C = 1;
    Host h = ellpack_file ? load_ellpack_file(ellpack_file) : generate(M, N, sparsity, seed, irregular);
    if (ellpack_file) {
        M = h.M; N = h.N;
        sparsity = 1.0 - double(h.values.size()) / std::max<double>(1.0, double(M) * double(N));
        std::printf("Matrix file:     %s\n", ellpack_file);
    }
    std::printf("=== Sparse %s benchmark (MI355X) ===\nMatrix dims:     %lld x %lld\nDense cols C:    %d\nSparsity:        %g\n"
                "Repetitions:     %d\nRNG seed:        %llu\nIrregular last row: %d\n\n",
                matmul ? "MatMul" : "MatVec", (long long)M, (long long)N, C, sparsity, runs, (unsigned long long)seed, int(irregular));

    const std::vector<float> X = sparseops_bench::dense_operand(size_t(N) * C, seed);
    const size_t nnz_total = h.values.size();
    std::printf("nnz %zu, ELLPACK r %u (padding %.2fx)\n\n", nnz_total, h.r, nnz_total ? double(M) * h.r / nnz_total : 0.0);

    so_ctx *ctx = nullptr;
    HIPCK(hipSetDevice(device));
    SOCK(so_init(device, &ctx));
    hipStream_t stream = nullptr;                     // vendor libraries run on the null stream
    float *dX = to_device(X), *dW = to_device(h.W), *dval = to_device(h.values);
    int *drow = to_device(h.row_ptr), *dcol = to_device(h.col_ind);
    float *dY = nullptr;
    HIPCK(hipMalloc(&dY, std::max<size_t>(size_t(M) * C, 1) * sizeof(float)));
    const float alpha = 1.0f, beta = 0.0f;
    const double flops = 2.0 * double(nnz_total) * C;

    // --- this library ---------------------------------------------------------
    so_ellpack *E_row = nullptr, *E_tiled = nullptr, *E_rbm = nullptr;
    SOCK(so_ellpack_upload(ctx, h.Wd.data(), h.idx.data(), h.nnz.data(), uint32_t(M), uint32_t(N), h.r,
                           matmul ? SO_LAYOUT_ROW : (SO_LAYOUT_ROW | SO_LAYOUT_BINS), &E_row));
    if (matmul)
        SOCK(so_ellpack_upload(ctx, h.Wd.data(), h.idx.data(), h.nnz.data(), uint32_t(M), uint32_t(N), h.r,
                               SO_LAYOUT_ROW | SO_LAYOUT_TILED, &E_tiled));
    if (matmul)
        SOCK(so_ellpack_upload(ctx, h.Wd.data(), h.idx.data(), h.nnz.data(), uint32_t(M), uint32_t(N), h.r,
                               SO_LAYOUT_ROW | SO_LAYOUT_RBM, &E_rbm));
    auto so_time = [&](auto &&call) {
        call();
        SOCK(so_sync(ctx));
        std::vector<double> t;
        for (int i = 0; i < runs; ++i) {
            float ms = 0;
            SOCK(so_timer_begin(ctx));
            call();
            SOCK(so_timer_end(ctx, &ms));
            t.push_back(ms * 1e3);
        }
        std::nth_element(t.begin(), t.begin() + t.size() / 2, t.end());
        return t[t.size() / 2];
    };
    std::vector<float> y_ref;
    auto report = [&](const char *name, double us, double err) {
        std::printf("%-34s: %10.2f us  %10.1f nnz-GFLOP/s   max rel diff vs so_%s %.1e\n", name, us, flops / us / 1e3,
                    matmul ? "matmul" : "matvec", err);
    };
    if (matmul) {
        const double t_row = so_time([&] { SOCK(so_matmul(ctx, E_row, dX, uint32_t(C), nullptr, dY, SO_ACT_NONE)); });
        y_ref = fetch(dY, size_t(M) * C);
        report("Ellpack so_matmul (row kernel)", t_row, 0.0);
        const double t_tiled = so_time([&] { SOCK(so_matmul(ctx, E_tiled, dX, uint32_t(C), nullptr, dY, SO_ACT_NONE)); });
        report("Ellpack so_matmul (LDS tiled)", t_tiled, max_rel_diff(fetch(dY, size_t(M) * C), y_ref));
        // the handle with the row-block-merged copy: so_matmul takes that kernel where the grid covers the chip
        const double t_rbm = so_time([&] { SOCK(so_matmul(ctx, E_rbm, dX, uint32_t(C), nullptr, dY, SO_ACT_NONE)); });
        report("Ellpack so_matmul (row-block merged)", t_rbm, max_rel_diff(fetch(dY, size_t(M) * C), y_ref));
    } else {
        const double t_row = so_time([&] { SOCK(so_matvec(ctx, E_row, dX, nullptr, dY, SO_LAYOUT_ROW)); });
        y_ref = fetch(dY, size_t(M));
        report("Ellpack so_matvec (wave per row)", t_row, 0.0);
        const double t_bin = so_time([&] { SOCK(so_matvec(ctx, E_row, dX, nullptr, dY, SO_LAYOUT_BINS)); });
        report("Ellpack so_matvec (length bins)", t_bin, max_rel_diff(fetch(dY, size_t(M)), y_ref));
        if (N <= 65536) {           // the same two kernels on a handle that also holds its columns in 16 bits
            so_ellpack *E_c16 = nullptr;
            SOCK(so_ellpack_upload(ctx, h.Wd.data(), h.idx.data(), h.nnz.data(), uint32_t(M), uint32_t(N), h.r,
                                   SO_LAYOUT_ROW | SO_LAYOUT_BINS | SO_LAYOUT_IDX16, &E_c16));
            const double t_row16 = so_time([&] { SOCK(so_matvec(ctx, E_c16, dX, nullptr, dY, SO_LAYOUT_ROW)); });
            report("Ellpack so_matvec (wave per row, 16-bit columns)", t_row16, max_rel_diff(fetch(dY, size_t(M)), y_ref));
            const double t_bin16 = so_time([&] { SOCK(so_matvec(ctx, E_c16, dX, nullptr, dY, SO_LAYOUT_BINS)); });
            report("Ellpack so_matvec (length bins, 16-bit columns)", t_bin16, max_rel_diff(fetch(dY, size_t(M)), y_ref));
            SOCK(so_ellpack_free(ctx, E_c16));
        }
    }

    // --- rocSPARSE CSR ----------------------------------------------------------
    rocsparse_handle sp = nullptr;
    SPCK(rocsparse_create_handle(&sp));
    rocsparse_spmat_descr A = nullptr;
    SPCK(rocsparse_create_csr_descr(&A, M, N, int64_t(nnz_total), drow, dcol, dval, rocsparse_indextype_i32,
                                    rocsparse_indextype_i32, rocsparse_index_base_zero, rocsparse_datatype_f32_r));
    if (matmul) {
        rocsparse_dnmat_descr B = nullptr, Cd = nullptr;
        SPCK(rocsparse_create_dnmat_descr(&B, N, C, C, dX, rocsparse_datatype_f32_r, rocsparse_order_row));
        SPCK(rocsparse_create_dnmat_descr(&Cd, M, C, C, dY, rocsparse_datatype_f32_r, rocsparse_order_row));
        const struct { rocsparse_spmm_alg alg; const char *name; } algs[] = {
            {rocsparse_spmm_alg_default, "rocSPARSE CSR SpMM (default)"},
            {rocsparse_spmm_alg_csr_row_split, "rocSPARSE CSR SpMM (row split)"},
            {rocsparse_spmm_alg_csr_merge_path, "rocSPARSE CSR SpMM (merge path)"}};
        for (const auto &a : algs) {
            size_t bytes = 0;
            if (rocsparse_spmm(sp, rocsparse_operation_none, rocsparse_operation_none, &alpha, A, B, &beta, Cd,
                               rocsparse_datatype_f32_r, a.alg, rocsparse_spmm_stage_buffer_size, &bytes, nullptr) != rocsparse_status_success) {
                std::printf("%-34s: not supported\n", a.name);
                continue;
            }
            void *buf = nullptr;
            HIPCK(hipMalloc(&buf, std::max<size_t>(bytes, 4)));
            SPCK(rocsparse_spmm(sp, rocsparse_operation_none, rocsparse_operation_none, &alpha, A, B, &beta, Cd,
                                rocsparse_datatype_f32_r, a.alg, rocsparse_spmm_stage_preprocess, &bytes, buf));
            const double t = median_us(stream, runs, [&] {
                SPCK(rocsparse_spmm(sp, rocsparse_operation_none, rocsparse_operation_none, &alpha, A, B, &beta, Cd,
                                    rocsparse_datatype_f32_r, a.alg, rocsparse_spmm_stage_compute, &bytes, buf));
            });
            report(a.name, t, max_rel_diff(fetch(dY, size_t(M) * C), y_ref));
            HIPCK(hipFree(buf));
        }
    } else {
        rocsparse_dnvec_descr xv = nullptr, yv = nullptr;
        SPCK(rocsparse_create_dnvec_descr(&xv, N, dX, rocsparse_datatype_f32_r));
        SPCK(rocsparse_create_dnvec_descr(&yv, M, dY, rocsparse_datatype_f32_r));
        const struct { rocsparse_spmv_alg alg; const char *name; } algs[] = {
            {rocsparse_spmv_alg_csr_rowsplit, "rocSPARSE CSR SpMV (row split)"},
            {rocsparse_spmv_alg_csr_adaptive, "rocSPARSE CSR SpMV (adaptive)"},
            {rocsparse_spmv_alg_csr_lrb, "rocSPARSE CSR SpMV (LRB)"}};
        for (const auto &a : algs) {
            size_t bytes = 0;
#pragma GCC diagnostic push
#pragma GCC diagnostic ignored "-Wdeprecated-declarations"
            if (rocsparse_spmv(sp, rocsparse_operation_none, &alpha, A, xv, &beta, yv, rocsparse_datatype_f32_r, a.alg,
                               rocsparse_spmv_stage_buffer_size, &bytes, nullptr) != rocsparse_status_success) {
                std::printf("%-34s: not supported\n", a.name);
                continue;
            }
            void *buf = nullptr;
            HIPCK(hipMalloc(&buf, std::max<size_t>(bytes, 4)));
            SPCK(rocsparse_spmv(sp, rocsparse_operation_none, &alpha, A, xv, &beta, yv, rocsparse_datatype_f32_r, a.alg,
                                rocsparse_spmv_stage_preprocess, &bytes, buf));
            const double t = median_us(stream, runs, [&] {
                SPCK(rocsparse_spmv(sp, rocsparse_operation_none, &alpha, A, xv, &beta, yv, rocsparse_datatype_f32_r, a.alg,
                                    rocsparse_spmv_stage_compute, &bytes, buf));
            });
#pragma GCC diagnostic pop
            report(a.name, t, max_rel_diff(fetch(dY, size_t(M)), y_ref));
            HIPCK(hipFree(buf));
        }
    }

    // --- rocBLAS dense ------------------------------------------------------------
    rocblas_handle bl = nullptr;
    BLCK(rocblas_create_handle(&bl));
    if (matmul) {
        // Row-major Y(MxC) = W(MxN) X(NxC)  ==  column-major Y^T(CxM) = X^T(CxN) W^T(NxM)
        const double t = median_us(stream, runs, [&] {
            BLCK(rocblas_sgemm(bl, rocblas_operation_none, rocblas_operation_none, C, int(M), int(N), &alpha, dX, C, dW, int(N),
                               &beta, dY, C));
        });
        std::printf("%-34s: %10.2f us  %10.1f dense-GFLOP/s (%.1f nnz-GFLOP/s)  max rel diff %.1e\n", "rocBLAS dense SGEMM", t,
                    2.0 * M * N * C / t / 1e3, flops / t / 1e3, max_rel_diff(fetch(dY, size_t(M) * C), y_ref));
    } else {
        // Row-major W(MxN) is column-major W^T(NxM): y = (W^T)^T x
        const double t = median_us(stream, runs, [&] {
            BLCK(rocblas_sgemv(bl, rocblas_operation_transpose, int(N), int(M), &alpha, dW, int(N), dX, 1, &beta, dY, 1));
        });
        std::printf("%-34s: %10.2f us  %10.1f GB/s dense stream             max rel diff %.1e\n", "rocBLAS dense SGEMV", t,
                    4.0 * M * N / t / 1e3, max_rel_diff(fetch(dY, size_t(M)), y_ref));
    }
    return 0;
}
