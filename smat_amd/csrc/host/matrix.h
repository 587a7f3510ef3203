// Host-side containers of the benchmark harness: dense fp16 operand and the
// sparse matrix with its one-off CSR -> BCSR build.  Counterparts of `Matrix`
// and `SparseMatrix` (src/cuda_hgemm/src/common/matrix.h:18-139, 143-721);
// device memory goes through the C ABI, there is no HIP header here.
#pragma once
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <ctime>
#include <random>
#include <string>
#include <vector>

#include "../half.h"
#include "hgemm_compat.h"

class Matrix {
public:
    // fill: 1.0 everywhere, as the reference does (matrix.h:38), or seeded uniform[min,max]
    Matrix(size_t row, size_t col, const std::string &name, bool random = false, unsigned seed = 1,
           float min = -1.0f, float max = 1.0f)
        : row_(row), col_(col), name_(name), host_(row * col)
    {
        if (!row || !col) { HLOG("%s: empty matrix", name.c_str()); exit(EXIT_FAILURE); }
        if (random) {
            std::mt19937 engine(seed);
            std::uniform_real_distribution<float> uniform(min, max);
            for (auto &h : host_) h = smat::half_from_double(uniform(engine));
        } else {
            std::fill(host_.begin(), host_.end(), (half)0x3c00);
        }
        SMAT_CHECK(smat_malloc((void **)&dev_, bytes()));
        moveToDevice();
        HLOG("%s: %zu * %zu, cpu: %p, gpu: %p", name_.c_str(), row_, col_, (void *)host_.data(), (void *)dev_);
    }
    ~Matrix() { smat_free(dev_); }
    Matrix(const Matrix &) = delete;
    Matrix &operator=(const Matrix &) = delete;

    size_t getRow() const { return row_; }
    size_t getCol() const { return col_; }
    size_t getElemNum() const { return host_.size(); }
    size_t bytes() const { return host_.size() * sizeof(half); }
    half *getHostPtr() { return host_.data(); }
    half *getDevPtr() const { return dev_; }

    void tearUp(Matrix *base) { SMAT_CHECK(smat_memcpy_d2d(dev_, base->getDevPtr(), bytes())); }
    void moveToHost() { SMAT_CHECK(smat_memcpy_d2h(host_.data(), dev_, bytes())); }
    void moveToDevice() { SMAT_CHECK(smat_memcpy_h2d(dev_, host_.data(), bytes())); }
    void memSetHost() { std::fill(host_.begin(), host_.end(), (half)0); }
    void memSetDevice() { SMAT_CHECK(smat_memset(dev_, 0, bytes())); }

private:
    size_t row_, col_;
    std::string name_;
    std::vector<half> host_;
    half *dev_ = nullptr;
};

class SparseMatrix {
public:
    // gpu_blocking: CSR -> BCSR on the device (smat_csr_to_bcsr_device) instead of on the host;
    // the arrays are the same, the host copies are fetched back for the plan and the verify step.
    SparseMatrix(const std::string &name, const std::string &file, bool reorder, float tau, bool gpu_blocking = false)
        : name_(name)
    {
        double t0 = wallMs();
        if (isContainer(file)) {  // binary CSR container written by smat_convert: no text parse
            int kind = 0;
            SMAT_CHECK(smat_bin_read(file.c_str(), &kind, &row_, &col_, &nnz_, &csrRowPtr_, &csrColIdx_, &csrVal_,
                                     nullptr, nullptr));
            if (kind != SMAT_BIN_CSR || row_ % 16 || col_ % 16) {
                HLOG("%s: expected a CSR container with dimensions padded to multiples of 16", file.c_str());
                exit(EXIT_FAILURE);
            }
        } else {
            int sym = 0;
            SMAT_CHECK(smat_mtx_read(file.c_str(), &row_, &col_, &nnz_, &sym, &csrRowPtr_, &csrColIdx_, &csrVal_, nullptr));
        }
        HLOG("Read %s in %.1f ms", file.c_str(), wallMs() - t0);
        if (!row_ || !col_ || !nnz_) { HLOG("empty matrix"); exit(EXIT_FAILURE); }
        HLOG("%zu x %zu, nnz = %zu, A[0] = %f", row_, col_, nnz_, smat::half_to_float(csrVal_[0]));
        t0 = wallMs();
        if (reorder) {  // row pass + column pass, values kept (the reference pipeline drops them: src/reorder.py:38-40)
            permRows_.resize(row_);
            permCols_.resize(col_);
            int64_t sr[4], sc[4];
            SMAT_CHECK(smat_reorder_csr(row_, col_, csrRowPtr_, csrColIdx_, 16, 16, tau, 1, permRows_.data(),
                                        permCols_.data(), sr, sc));
            int32_t *rp, *ci;
            uint16_t *v;
            SMAT_CHECK(smat_permute_csr(row_, col_, csrRowPtr_, csrColIdx_, csrVal_, permRows_.data(), permCols_.data(),
                                        &rp, &ci, &v));
            smat_host_free(csrRowPtr_); smat_host_free(csrColIdx_); smat_host_free(csrVal_);
            csrRowPtr_ = rp; csrColIdx_ = ci; csrVal_ = v;
            HLOG("Reordered: row pass %lld nonzero blocks (%lld comparisons), column pass %lld (%lld comparisons)",
                 (long long)sr[2], (long long)sr[0], (long long)sc[2], (long long)sc[0]);
            HLOG("Reorder time: %.1f ms (host, not part of the SpMM time)", wallMs() - t0);
        }
        int64_t counts[3];
        t0 = wallMs();
        if (gpu_blocking) {
            int32_t *rp_d, *ci_d;
            uint16_t *v_d;
            SMAT_CHECK(smat_malloc((void **)&rp_d, (row_ + 1) * sizeof(int)));
            SMAT_CHECK(smat_malloc((void **)&ci_d, nnz_ * sizeof(int)));
            SMAT_CHECK(smat_malloc((void **)&v_d, nnz_ * sizeof(half)));
            SMAT_CHECK(smat_memcpy_h2d(rp_d, csrRowPtr_, (row_ + 1) * sizeof(int)));
            SMAT_CHECK(smat_memcpy_h2d(ci_d, csrColIdx_, nnz_ * sizeof(int)));
            SMAT_CHECK(smat_memcpy_h2d(v_d, csrVal_, nnz_ * sizeof(half)));
            const double t1 = wallMs();
            SMAT_CHECK(smat_csr_to_bcsr_device(row_, col_, rp_d, ci_d, v_d, nnz_, counts, &bcsrRowPtr_dev_,
                                               &bcsrColIdx_dev_, (uint16_t **)&bcsrVal_dev_));
            HLOG("Blocking on the GPU: %.1f ms (+ %.1f ms to copy the CSR to the device)", wallMs() - t1, t1 - t0);
            smat_free(rp_d); smat_free(ci_d); smat_free(v_d);
            nonzeroBlocks_ = (size_t)counts[0];
            bcsrRowPtr_ = (int32_t *)malloc((row_ / 16 + 1) * sizeof(int));
            bcsrColIdx_ = (int32_t *)malloc(std::max<size_t>(nonzeroBlocks_, 1) * sizeof(int));
            bcsrVal_ = (uint16_t *)malloc(std::max<size_t>(nonzeroBlocks_, 1) * 256 * sizeof(half));
            if (!bcsrRowPtr_ || !bcsrColIdx_ || !bcsrVal_) { HLOG("out of host memory"); exit(EXIT_FAILURE); }
            SMAT_CHECK(smat_memcpy_d2h(bcsrRowPtr_, bcsrRowPtr_dev_, (row_ / 16 + 1) * sizeof(int)));
            SMAT_CHECK(smat_memcpy_d2h(bcsrColIdx_, bcsrColIdx_dev_, nonzeroBlocks_ * sizeof(int)));
            SMAT_CHECK(smat_memcpy_d2h(bcsrVal_, bcsrVal_dev_, nonzeroBlocks_ * 256 * sizeof(half)));
        } else {
            SMAT_CHECK(smat_csr_to_bcsr(row_, col_, csrRowPtr_, csrColIdx_, csrVal_, counts, &bcsrRowPtr_, &bcsrColIdx_,
                                        &bcsrVal_, nullptr, nullptr));
            nonzeroBlocks_ = (size_t)counts[0];
            HLOG("Blocking on the host: %.1f ms", wallMs() - t0);
            SMAT_CHECK(smat_malloc((void **)&bcsrVal_dev_, nonzeroBlocks_ * 256 * sizeof(half)));
            SMAT_CHECK(smat_malloc((void **)&bcsrColIdx_dev_, nonzeroBlocks_ * sizeof(int)));
            SMAT_CHECK(smat_malloc((void **)&bcsrRowPtr_dev_, (row_ / 16 + 1) * sizeof(int)));
            SMAT_CHECK(smat_memcpy_h2d(bcsrVal_dev_, bcsrVal_, nonzeroBlocks_ * 256 * sizeof(half)));
            SMAT_CHECK(smat_memcpy_h2d(bcsrColIdx_dev_, bcsrColIdx_, nonzeroBlocks_ * sizeof(int)));
            SMAT_CHECK(smat_memcpy_h2d(bcsrRowPtr_dev_, bcsrRowPtr_, (row_ / 16 + 1) * sizeof(int)));
        }
        HLOG("Finished creating BCSR from CSR");
        HLOG("%zu total blocks, %zu nonzero blocks, %zu dense blocks, %zu sparse blocks", (row_ / 16) * (col_ / 16),
             nonzeroBlocks_, (size_t)counts[1], (size_t)counts[2]);
    }
    static double wallMs()
    {
        struct timespec ts;
        clock_gettime(CLOCK_MONOTONIC, &ts);
        return ts.tv_sec * 1e3 + ts.tv_nsec * 1e-6;
    }
    static bool isContainer(const std::string &file)
    {
        FILE *f = fopen(file.c_str(), "rb");
        if (!f) return false;
        char m[8] = {0};
        const bool ok = fread(m, 1, 8, f) == 8 && memcmp(m, "SMATBIN1", 8) == 0;
        fclose(f);
        return ok;
    }
    ~SparseMatrix()
    {
        smat_host_free(csrRowPtr_); smat_host_free(csrColIdx_); smat_host_free(csrVal_);
        smat_host_free(bcsrRowPtr_); smat_host_free(bcsrColIdx_); smat_host_free(bcsrVal_);
        smat_free(bcsrVal_dev_); smat_free(bcsrColIdx_dev_); smat_free(bcsrRowPtr_dev_);
    }
    SparseMatrix(const SparseMatrix &) = delete;
    SparseMatrix &operator=(const SparseMatrix &) = delete;

    size_t getRow() const { return row_; }
    size_t getCol() const { return col_; }
    size_t getNnz() const { return nnz_; }
    size_t getNonzeroblocks() const { return nonzeroBlocks_; }
    half *getBcsrValues() const { return bcsrVal_dev_; }
    int *getBcsrRowPtr() const { return bcsrRowPtr_dev_; }
    int *getBcsrColIdx() const { return bcsrColIdx_dev_; }
    // the two dense maps of the reference are never built: the kernels do not read them
    int *getBlockInfo_dev() const { return nullptr; }
    int *getRelativeBlockIndexMapping_dev() const { return nullptr; }
    const int32_t *hostBcsrRowPtr() const { return bcsrRowPtr_; }
    const int32_t *hostBcsrColIdx() const { return bcsrColIdx_; }

    // CPU reference product for the verify step: fp16 inputs widened to fp32, fp32
    // accumulation, straight from the CSR (so it does not depend on the blocking).
    // B column-major (k, n) at B[n*K + k]; C row-major fp32.
    void multiplyOnHost(const half *B, size_t N, std::vector<float> &C) const
    {
        std::vector<float> Bt(col_ * N); // widen once, row-major for a unit-stride inner loop
        for (size_t n = 0; n < N; n++)
            for (size_t k = 0; k < col_; k++) Bt[k * N + n] = smat::half_to_float(B[n * col_ + k]);
        C.assign(row_ * N, 0.0f);
        for (size_t i = 0; i < row_; i++)
            for (int32_t p = csrRowPtr_[i]; p < csrRowPtr_[i + 1]; p++) {
                const float a = smat::half_to_float(csrVal_[p]);
                const float *b = &Bt[(size_t)csrColIdx_[p] * N];
                float *c = &C[i * N];
                for (size_t n = 0; n < N; n++) c[n] += a * b[n];
            }
    }

private:
    std::string name_;
    size_t row_ = 0, col_ = 0, nnz_ = 0, nonzeroBlocks_ = 0;
    int32_t *csrRowPtr_ = nullptr, *csrColIdx_ = nullptr;
    uint16_t *csrVal_ = nullptr;
    int32_t *bcsrRowPtr_ = nullptr, *bcsrColIdx_ = nullptr;
    uint16_t *bcsrVal_ = nullptr;
    half *bcsrVal_dev_ = nullptr;
    int *bcsrRowPtr_dev_ = nullptr, *bcsrColIdx_dev_ = nullptr;
    std::vector<int64_t> permRows_, permCols_;
};
