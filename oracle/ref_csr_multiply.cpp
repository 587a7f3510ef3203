// Test/benchmark infrastructure, not part of the product: a small driver around the
// reference's own serial CPU SpMM, CSR::multiply (preprocess/src/general/csr.cpp:47-63),
// compiled together with the reference sources into oracle/_ref/ref_csr_multiply.
//
//   ref_csr_multiply A.el B.f32 B_cols reps [C_out.f32]
//
// A.el    edge list "row col value", rows ascending (CSR::read_from_edgelist, csr.cpp:166-290);
//         the matrix is rows x cols with rows = last row + 1, cols = largest column + 1
// B.f32   float32, column-major with leading dimension `rows` (csr.cpp:59 indexes B with the
//         row count of A, so cols <= rows is required), rows * B_cols values
// prints  rows cols nnz seconds_per_multiply (best of reps); C (column-major, rows x B_cols)
//         of the last repetition goes to C_out.f32 when given.
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <vector>

#include "matrices.h"

int main(int argc, char **argv)
{
    if (argc < 5) {
        fprintf(stderr, "usage: %s A.el B.f32 B_cols reps [C_out.f32]\n", argv[0]);
        return 2;
    }
    std::ifstream fin(argv[1]);
    if (!fin) { fprintf(stderr, "cannot open %s\n", argv[1]); return 1; }
    CSR A(fin, " ", false, el);
    const long b_cols = atol(argv[3]);
    const int reps = atoi(argv[4]);
    if (A.cols > A.rows) { fprintf(stderr, "cols (%ld) > rows (%ld): CSR::multiply needs cols <= rows\n", A.cols, A.rows); return 1; }
    std::vector<DataT> B((size_t)A.rows * b_cols);
    FILE *fb = fopen(argv[2], "rb");
    if (!fb || fread(B.data(), sizeof(DataT), B.size(), fb) != B.size()) { fprintf(stderr, "cannot read %zu floats from %s\n", B.size(), argv[2]); return 1; }
    fclose(fb);
    std::vector<DataT_C> C((size_t)A.rows * b_cols);
    double best = 1e300;
    for (int r = 0; r < reps; r++) {
        memset(C.data(), 0, C.size() * sizeof(DataT_C)); // multiply accumulates into C
        auto t0 = std::chrono::steady_clock::now();
        A.multiply(B.data(), b_cols, C.data());
        double s = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
        if (s < best) best = s;
    }
    printf("%ld %ld %ld %.9f\n", A.rows, A.cols, A.nztot(), best);
    if (argc > 5) {
        FILE *fc = fopen(argv[5], "wb");
        if (!fc || fwrite(C.data(), sizeof(DataT_C), C.size(), fc) != C.size()) { fprintf(stderr, "cannot write %s\n", argv[5]); return 1; }
        fclose(fc);
    }
    return 0;
}
