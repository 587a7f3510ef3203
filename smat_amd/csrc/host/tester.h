// Benchmark harness: owns A (sparse), B, C; warm-up, timed loop, throughput, CSV
// row, optional verification.  Counterpart of `Tester`
// (src/cuda_hgemm/src/common/tester.h:9-410), sparse path only:
// evaluateSparse2 (tester.h:166-209) and profileSparse2 (tester.h:337-377).
//
// Differences, all deliberate:
//  * throughput counts 2*nnzb*16*16*N flop; the reference leaves N out
//    (tester.h:362-363) - its figure is printed next to ours for comparison;
//  * time is taken both with the host clock around the asynchronous launches
//    (as the reference does, tester.h:339-361) and with device events;
//  * -enable_check really checks: C against a CPU fp32-accumulated product
//    (the reference's check is compiled out, tester.h:188), reporting the
//    reference's max/mean absolute difference (matrix.h:103-121) and the
//    max error relative to the row L2 norm.
#pragma once
#include <sys/time.h>
#include <unistd.h>

#include <algorithm>
#include <cmath>
#include <string>
#include <vector>

#include "matrix.h"

class Tester {
public:
    Tester(size_t warmup_iterations, size_t profiling_iterations, size_t sleep_duration, bool enable_check,
           int n_mult, const std::string &filename, bool reorder, float tau, bool random_b, bool use_plan, int kernel,
           bool gpu_blocking = false, bool poison_check = false)
        : warmup_(warmup_iterations), iters_(profiling_iterations), sleep_ms_(sleep_duration), check_(enable_check),
          poison_(poison_check), file_(filename), kernel_(kernel)
    {
        if (!warmup_ || !iters_) { HLOG("warmup_iterations and profiling_iterations must be positive"); exit(EXIT_FAILURE); }
        A_ = new SparseMatrix("Sparse Matrix A", filename, reorder, tau, gpu_blocking);
        const size_t N = (size_t)n_mult * 8; // MMA_N of the reference, tester.h:40
        B_ = new Matrix(A_->getCol(), N, "Matrix B for sparse", random_b, 0xB);
        C_ = new Matrix(A_->getRow(), N, "Matrix C for sparse");
        C_->memSetHost(); C_->moveToDevice();
        base_ = new Matrix(A_->getRow(), N, "Matrix Base");
        base_->memSetHost(); base_->moveToDevice();
        if (use_plan) {
            smat_spmm_opts o = {SMAT_B_COL_MAJOR, SMAT_C_F16, kernel_, 0, nullptr};
            SMAT_CHECK(smat_plan_create(&plan_, A_->hostBcsrRowPtr(), A_->hostBcsrColIdx(), A_->getRow(), A_->getCol(),
                                        A_->getNonzeroblocks(), N, &o));
            // the plan also looks at the block values once (which columns of the blocks are nonzero)
            SMAT_CHECK(smat_plan_attach_values(plan_, (const uint16_t *)A_->getBcsrValues(), A_->getBcsrRowPtr(),
                                               A_->getBcsrColIdx(), A_->hostBcsrRowPtr()));
            int64_t info[12];
            SMAT_CHECK(smat_plan_info(plan_, info));
            HLOG("Plan: kernel %lld, %lld work items, %lld split block rows, workspace %lld bytes, %lld sweep ops, "
                 "%lld nonzero block columns",
                 (long long)info[0], (long long)info[1], (long long)info[2], (long long)info[4], (long long)info[6],
                 (long long)info[9]);
        }
    }
    ~Tester()
    {
        smat_plan_destroy(plan_);
        delete A_; delete B_; delete C_; delete base_;
    }

    // hgemm: anything callable with the HGEMM_FUNC_SPARSE2 argument list (main.cu:7)
    template <typename Func> void evaluateSparse2(Func &&hgemm, const std::string &name)
    {
        HLOG("----------------- Sparse Evaluating %s -----------------", name.c_str());
        usleep(sleep_ms_ * 1000);
        C_->tearUp(base_);
        const double t0 = now_ms();
        for (size_t i = 0; i < warmup_; ++i) call(hgemm);
        SMAT_CHECK(smat_device_synchronize());
        HLOG("Warm up time: %.3f ms", (now_ms() - t0) / (double)warmup_);
        if (check_) verify();
        profileSparse2(std::forward<Func>(hgemm), name);
    }

    // the library's own entry point with the plan / kernel choice of the command line
    void evaluatePlanned(const std::string &name)
    {
        auto f = [this](half *v, int *rp, int *ci, half *B, half *C, size_t M, size_t N, size_t K, size_t nnzb, int *,
                        int *) {
            smat_spmm_opts o = {SMAT_B_COL_MAJOR, SMAT_C_F16, kernel_, 0, nullptr};
            SMAT_CHECK(smat_spmm_bcsr_f16_ex(v, rp, ci, B, C, M, N, K, nnzb, &o, plan_));
        };
        evaluateSparse2(f, name);
    }

    // N sweep of the reference harness (createLinePlot, common/tester.h:211-267): for
    // N = 8*mult, mult in [from, to), time the kernel and append "N, ms" to results_smat.csv.
    // The plan (built for the largest N of the sweep) is reused; B and C are re-made per N.
    void createLinePlot(const std::string &name, int from, int to, int step)
    {
        HLOG("----------------- Sparse Lineplot %s -----------------", name.c_str());
        double base_ms = 0, base_tflops = 0;
        for (int mult = from; mult < to; mult += step) {
            const size_t N = (size_t)mult * 8;
            delete B_; delete C_;
            B_ = new Matrix(A_->getCol(), N, "Matrix B for sparse", true, 0xB);
            C_ = new Matrix(A_->getRow(), N, "Matrix C for sparse");
            C_->memSetHost(); C_->moveToDevice();
            auto f = [this](half *v, int *rp, int *ci, half *B, half *C, size_t M, size_t n, size_t K, size_t nnzb,
                            int *, int *) {
                smat_spmm_opts o = {SMAT_B_COL_MAJOR, SMAT_C_F16, kernel_, 0, nullptr};
                SMAT_CHECK(smat_spmm_bcsr_f16_ex(v, rp, ci, B, C, M, n, K, nnzb, &o, plan_));
            };
            for (size_t i = 0; i < warmup_; ++i) call(f);
            void *e0, *e1;
            SMAT_CHECK(smat_event_create(&e0));
            SMAT_CHECK(smat_event_create(&e1));
            SMAT_CHECK(smat_event_record(e0, nullptr));
            for (size_t i = 0; i < iters_; ++i) call(f);
            SMAT_CHECK(smat_event_record(e1, nullptr));
            SMAT_CHECK(smat_device_synchronize());
            float ev = 0;
            SMAT_CHECK(smat_event_elapsed_ms(e0, e1, &ev));
            smat_event_destroy(e0); smat_event_destroy(e1);
            const double ms = ev / (double)iters_;
            const double tflops = (double)A_->getNonzeroblocks() * 256.0 * 2.0 * (double)N * 1e-12 / (ms * 1e-3);
            if (base_ms == 0) { base_ms = ms; base_tflops = tflops; }
            FILE *fout = fopen("results_smat.csv", "a");
            if (fout) { fprintf(fout, "%zu, %lf\n", N, ms); fclose(fout); }
            HLOG("%s exit, N = %zu, profiling time: %.4f ms (%.2f%%), throughput: %.3f TFLOPS (%.2f%%)", name.c_str(), N,
                 ms, ms / base_ms * 100, tflops, tflops / base_tflops * 100);
        }
    }

    double lastMs() const { return event_ms_; }

private:
    static double now_ms()
    {
        struct timeval t;
        gettimeofday(&t, nullptr);
        return t.tv_sec * 1000.0 + t.tv_usec / 1000.0;
    }
    template <typename Func> void call(Func &&hgemm)
    {
        hgemm(A_->getBcsrValues(), A_->getBcsrRowPtr(), A_->getBcsrColIdx(), B_->getDevPtr(), C_->getDevPtr(),
              A_->getRow(), C_->getCol(), A_->getCol(), A_->getNonzeroblocks(), A_->getBlockInfo_dev(),
              A_->getRelativeBlockIndexMapping_dev());
    }
    template <typename Func> void profileSparse2(Func &&hgemm, const std::string &name)
    {
        void *e0, *e1;
        SMAT_CHECK(smat_event_create(&e0));
        SMAT_CHECK(smat_event_create(&e1));
        SMAT_CHECK(smat_device_synchronize());
        const double t0 = now_ms();
        SMAT_CHECK(smat_event_record(e0, nullptr));
        for (size_t i = 0; i < iters_; ++i) call(hgemm);
        SMAT_CHECK(smat_event_record(e1, nullptr));
        SMAT_CHECK(smat_device_synchronize());
        const double wall = (now_ms() - t0) / (double)iters_;
        float ev = 0;
        SMAT_CHECK(smat_event_elapsed_ms(e0, e1, &ev));
        event_ms_ = ev / (double)iters_;
        smat_event_destroy(e0); smat_event_destroy(e1);
        const double blocks = (double)A_->getNonzeroblocks(), N = (double)C_->getCol();
        const double tflops = blocks * 256.0 * 2.0 * N * 1e-12 / (event_ms_ * 1e-3);
        const double ref_style = blocks * 256.0 * 2.0 * 1e-12 / (wall * 1e-3); // the reference's figure (no N)
        FILE *fout = fopen("results_smat.csv", "a");
        if (fout) { fprintf(fout, "%s,%lf\n", file_.c_str(), wall); fclose(fout); }
        HLOG("%s exit, profiling time: %.4f ms wall, %.4f ms device events, throughput: %.3f TFLOPS "
             "(2*nnzb*256*N), %.6f TFLOPS by the reference's N-less formula",
             name.c_str(), wall, event_ms_, tflops, ref_style);
    }
    void verify()
    {
        std::vector<float> ref;
        const double t0 = now_ms();
        A_->multiplyOnHost(B_->getHostPtr(), C_->getCol(), ref);
        HLOG("CPU fp32 reference product: %.1f ms on 1 core", now_ms() - t0);
        C_->moveToHost();
        const size_t M = C_->getRow(), N = C_->getCol();
        if (poison_) { // self-test of this check: one NaN in the copy of C that is looked at must fail the run
            C_->getHostPtr()[(M / 2) * N + N / 2] = 0x7e00;
            HLOG("-poison_check: one element of the result replaced by NaN before the comparison");
        }
        double worst = 0, max_diff = 0, avg = 0;
        size_t non_finite = 0;
        for (size_t i = 0; i < M; i++) {
            double nrm = 0, row_max = 0;
            for (size_t j = 0; j < N; j++) {
                const double r = ref[i * N + j];
                double d = std::fabs((double)smat::half_to_float(C_->getHostPtr()[i * N + j]) - r);
                if (!std::isfinite(d)) { // std::max would drop a NaN: a result that is not a number is a gross error
                    d = 1e30;
                    non_finite++;
                }
                nrm += r * r; row_max = std::max(row_max, d); avg += d;
            }
            max_diff = std::max(max_diff, row_max);
            worst = std::max(worst, nrm > 0 ? row_max / std::sqrt(nrm) : row_max);
        }
        HLOG("Max diff: %f, avg diff: %f", max_diff, avg / (double)(M * N));
        if (non_finite) HLOG("%zu elements of the result are not finite where the reference product is", non_finite);
        HLOG("Max error relative to the row L2 norm: %.3e (%s, bound 1e-3)", worst, worst <= 1e-3 ? "PASS" : "FAIL");
        if (!(worst <= 1e-3)) exit(EXIT_FAILURE);
    }

    size_t warmup_, iters_, sleep_ms_;
    bool check_, poison_;
    std::string file_;
    int kernel_;
    SparseMatrix *A_ = nullptr;
    Matrix *B_ = nullptr, *C_ = nullptr, *base_ = nullptr;
    smat_plan *plan_ = nullptr;
    double event_ms_ = 0;
};
