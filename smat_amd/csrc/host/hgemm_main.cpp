// `hgemm`: the benchmark binary of the matrix-load -> block -> SpMM -> verify flow.
// Accepts the flags of the reference binary (src/cuda_hgemm/src/main.cu:22-34):
//   -filename -n_mult -warmup_iterations -profiling_iterations -sleep_duration
//   -enable_check -gpu_rank -cpu_procs  (-M -N -K -enable_wmma -enable_mma are
//   accepted and ignored: they only sized the dense-GEMM leftovers there)
// and adds: -reorder (row + column clustering before blocking), -tau,
//   -random_b (seeded uniform[-1,1] B instead of all ones), -use_plan, -kernel,
//   -gpu_blocking (CSR -> BCSR on the device), -poison_check (with -enable_check: plants one NaN in the result
//   before it is compared, so the run must end with FAIL and a non-zero status).  -filename also takes a binary container
//   written by smat_convert.  -lineplot [-lineplot_from=14 -lineplot_to=126 -lineplot_step=1] sweeps
//   N = 8*mult like createLinePlot (common/tester.h:211-267) and appends "N, ms" lines to results_smat.csv.  Load, reorder and blocking times are logged apart from the SpMM time.
#include <thread>

#include "flags.h"
#include "tester.h"

int main(int argc, char **argv)
{
    Flags f(argc, argv);
    const int gpu = (int)f.num("gpu_rank", 0);
    SMAT_CHECK(smat_set_device(gpu));
    char name[256];
    SMAT_CHECK(smat_device_name(gpu, name, sizeof name));
    int64_t cus = 0, lds = 0, mem = 0, clk = 0;
    SMAT_CHECK(smat_device_attr(gpu, &cus, &lds, &mem, &clk));
    HLOG("%s start with %ld CPU processes on the %d-th GPU: %s", smat_version(),
         f.num("cpu_procs", (long)std::thread::hardware_concurrency()), gpu, name);
    HLOG("%lld compute units, %lld KBytes LDS per CU, %.0f MBytes global memory, clock %.0f MHz", (long long)cus,
         (long long)(lds / 1024), (double)mem / 1048576.0, (double)clk * 1e-3);

    const std::string file = f.str("filename", "");
    if (file.empty()) { HLOG("usage: hgemm -filename=<matrix.mtx> [-n_mult=<N/8>] [-enable_check] ..."); return 2; }
    const int n_mult = (int)f.num("n_mult", 1);
    HLOG("Input .mtx: %s, N_MULT: %d (N = %d)", file.c_str(), n_mult, n_mult * 8);
    HLOG("Profiling: warmup iterations: %ld, profiling iterations: %ld, sleep duration: %ld ms, enable check: %d",
         f.num("warmup_iterations", 1), f.num("profiling_iterations", 10), f.num("sleep_duration", 100),
         (int)f.flag("enable_check", false));

    const bool lineplot = f.flag("lineplot", false);
    const int lp_from = (int)f.num("lineplot_from", 14), lp_to = (int)f.num("lineplot_to", 126),
              lp_step = (int)f.num("lineplot_step", 1);
    if (lineplot && (lp_from < 1 || lp_to <= lp_from || lp_step < 1)) { HLOG("bad -lineplot_from/_to/_step"); return 2; }
    // with -lineplot the plan is made for the widest N of the sweep
    Tester tester((size_t)f.num("warmup_iterations", 1), (size_t)f.num("profiling_iterations", 10),
                  (size_t)f.num("sleep_duration", 100), f.flag("enable_check", false),
                  lineplot ? lp_from + (lp_to - 1 - lp_from) / lp_step * lp_step : n_mult, file,
                  f.flag("reorder", false), (float)f.real("tau", 0.5), f.flag("random_b", false),
                  f.flag("use_plan", true), (int)f.num("kernel", SMAT_KERNEL_AUTO), f.flag("gpu_blocking", false),
                  f.flag("poison_check", false));
    if (lineplot) {
        if (!f.flag("use_plan", true)) { HLOG("-lineplot needs the plan (-use_plan)"); return 2; }
        tester.createLinePlot("Smat-Plan-Kernel", lp_from, lp_to, lp_step);
    } else if (f.flag("use_plan", true))
        tester.evaluatePlanned("Smat-Plan-Kernel");
    else
        tester.evaluateSparse2(mmaCBTKernel, "Mma-CBT-Kernel"); // the drop-in symbol, as in main.cu:99
    HLOG("Done");
    return 0;
}
