/*
 * smat_oracle.c -- TEST INFRASTRUCTURE ONLY.
 *
 * A plain-C, single-threaded CPU restatement of the reference's block-sparse
 * SpMM path, used solely as the checker in tests/, in the smoke test and as the
 * timed "cpu_baseline" leg of bench.py.  Nothing in the shipped library
 * (smat_amd/) links, loads or calls this file.
 *
 * Each function cites the reference source (paths relative to the reference
 * root) whose behaviour it restates.  Pin status of every function:
 *
 *   orc_f64_to_f16 / orc_f16_to_f32  pinned: exhaustive round trip over all 65536
 *                                    half patterns, ties-to-even cases by hand,
 *                                    cross-checked with numpy.float16.
 *   orc_mtx_read                     pinned: hand-written .mtx fixtures with
 *                                    hand-written expected CSR (tests/golden/mtx).
 *   orc_csr_to_bcsr                  pinned: closed forms (band, 27-pt stencil,
 *                                    block mask), brute-force dense bitmap in
 *                                    numpy, invariants rel==ptr.
 *   orc_spmm_csr_f32 /               pinned: dense matmul in float64 (numpy) on
 *   orc_spmm_bcsr_f32                small inputs, identity-block and B=ones
 *                                    special cases, CSR-vs-blocked equality
 *                                    (the reference's TEST_matrices check).
 *   reorder                          not restated here: the reference's own
 *                                    C++ sources build with g++ (oracle/Makefile
 *                                    -> oracle/_ref/) and produce the committed
 *                                    golden fixtures.
 */
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <ctype.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define ORC_BS 16 /* MMA_M == MMA_K == 16: src/cuda_hgemm/src/common/matrix.h:13-15 */

/* ------------------------------------------------------------------ fp16 -- */

/* double -> IEEE binary16, round-to-nearest-even, directly from the double
 * (the reference assigns `csrVal_tmp[i] = fval` with fval a double:
 * src/cuda_hgemm/src/common/mmio_highlevel.h:708). */
uint16_t orc_f64_to_f16(double d)
{
    uint64_t x;
    memcpy(&x, &d, 8);
    uint16_t sign = (uint16_t)((x >> 48) & 0x8000u);
    int64_t e = (int64_t)((x >> 52) & 0x7ff);
    uint64_t m = x & 0xfffffffffffffULL;
    if (e == 0x7ff) return (uint16_t)(sign | 0x7c00u | (m ? 0x200u : 0u));
    if (e == 0) return sign; /* zero or double subnormal: far below half range */
    int64_t eh = e - 1023 + 15;
    if (eh >= 31) return (uint16_t)(sign | 0x7c00u);
    uint64_t M = m | (1ULL << 52);
    int shift = 42;
    if (eh <= 0) shift = (int)(42 + 1 - eh);
    if (shift >= 54) return sign;
    uint64_t q = M >> shift;
    uint64_t rem = M & ((1ULL << shift) - 1);
    uint64_t half = 1ULL << (shift - 1);
    if (rem > half || (rem == half && (q & 1))) q++;
    if (eh <= 0) return (uint16_t)(sign | (uint16_t)q);
    return (uint16_t)(sign | (uint16_t)((((uint64_t)(eh - 1)) << 10) + q));
}

float orc_f16_to_f32(uint16_t h)
{
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint32_t e = (h >> 10) & 0x1f;
    uint32_t m = h & 0x3ff;
    uint32_t out;
    if (e == 0) {
        if (m == 0) {
            out = sign;
        } else { /* subnormal: normalise */
            int s = 0;
            while (!(m & 0x400)) { m <<= 1; s++; }
            m &= 0x3ff;
            out = sign | ((uint32_t)(127 - 15 - s + 1) << 23) | (m << 13);
        }
    } else if (e == 31) {
        out = sign | 0x7f800000u | (m << 13);
    } else {
        out = sign | ((e - 15 + 127) << 23) | (m << 13);
    }
    float f;
    memcpy(&f, &out, 4);
    return f;
}

void orc_f16_to_f32_array(const uint16_t *h, float *f, int64_t n)
{
    for (int64_t i = 0; i < n; i++) f[i] = orc_f16_to_f32(h[i]);
}

void orc_f64_to_f16_array(const double *d, uint16_t *h, int64_t n)
{
    for (int64_t i = 0; i < n; i++) h[i] = orc_f64_to_f16(d[i]);
}

/* --------------------------------------------------------- Matrix Market -- */

/* Restates mmio_allinone (src/cuda_hgemm/src/common/mmio_highlevel.h:619-786)
 * with mm_read_banner (common/mmio.h:399-565), mm_read_mtx_crd_size
 * (common/mmio.h:569-625), padSparseMatrix (mmio_highlevel.h:609-616) and
 * exclusive_scan (mmio_highlevel.h:11-26).
 *
 * Returns 0, or the reference's negative codes: -1 cannot open, -2 bad banner,
 * -4 bad size line.  Outputs are malloc'ed; free with orc_free. */
int orc_mtx_read(const char *path, int64_t *m_out, int64_t *n_out, int64_t *nnz_out,
                 int *is_symmetric, int32_t **row_ptr, int32_t **col_idx, uint16_t **val)
{
    FILE *f = fopen(path, "r");
    if (!f) return -1;

    char line[1025], banner[64], mtx[64], crd[64], dtype[64], scheme[64];
    if (!fgets(line, sizeof line, f) ||
        sscanf(line, "%63s %63s %63s %63s %63s", banner, mtx, crd, dtype, scheme) != 5) {
        fclose(f);
        return -2;
    }
    for (char *p = mtx; *p; p++) *p = (char)tolower(*p);
    for (char *p = crd; *p; p++) *p = (char)tolower(*p);
    for (char *p = dtype; *p; p++) *p = (char)tolower(*p);
    for (char *p = scheme; *p; p++) *p = (char)tolower(*p);
    int ok = strncmp(banner, "%%MatrixMarket", 14) == 0 && strcmp(mtx, "matrix") == 0 &&
             (strcmp(crd, "coordinate") == 0 || strcmp(crd, "array") == 0);
    int is_real = strcmp(dtype, "real") == 0, is_cplx = strcmp(dtype, "complex") == 0;
    int is_pat = strcmp(dtype, "pattern") == 0, is_int = strcmp(dtype, "integer") == 0;
    int sym = strcmp(scheme, "symmetric") == 0 || strcmp(scheme, "hermitian") == 0;
    int known_scheme = sym || strcmp(scheme, "general") == 0 || strcmp(scheme, "skew-symmetric") == 0;
    if (!ok || !(is_real || is_cplx || is_pat || is_int) || !known_scheme) {
        fclose(f);
        return -2;
    }

    int m = 0, n = 0, nz = 0;
    do {
        if (!fgets(line, sizeof line, f)) { fclose(f); return -4; }
    } while (line[0] == '%');
    if (sscanf(line, "%d %d %d", &m, &n, &nz) != 3) {
        int got;
        do {
            got = fscanf(f, "%d %d %d", &m, &n, &nz);
            if (got == EOF) { fclose(f); return -4; }
        } while (got != 3);
    }
    /* pad both dimensions up to a multiple of 16 (mmio_highlevel.h:609-616, 649) */
    if (m % ORC_BS) m += ORC_BS - m % ORC_BS;
    if (n % ORC_BS) n += ORC_BS - n % ORC_BS;

    int32_t *counter = (int32_t *)calloc((size_t)m + 1, sizeof(int32_t));
    int32_t *ri = (int32_t *)malloc(sizeof(int32_t) * (size_t)(nz > 0 ? nz : 1));
    int32_t *ci = (int32_t *)malloc(sizeof(int32_t) * (size_t)(nz > 0 ? nz : 1));
    uint16_t *vv = (uint16_t *)malloc(sizeof(uint16_t) * (size_t)(nz > 0 ? nz : 1));

    for (int i = 0; i < nz; i++) {
        int a = 0, b = 0, iv = 0;
        double fv = 0.0, fim = 0.0;
        if (is_real) {
            if (fscanf(f, "%d %d %lg\n", &a, &b, &fv) < 0) { nz = i; break; }
        } else if (is_cplx) {
            if (fscanf(f, "%d %d %lg %lg\n", &a, &b, &fv, &fim) < 0) { nz = i; break; }
        } else if (is_int) {
            if (fscanf(f, "%d %d %d\n", &a, &b, &iv) < 0) { nz = i; break; }
            fv = iv;
        } else {
            if (fscanf(f, "%d %d\n", &a, &b) < 0) { nz = i; break; }
            fv = 1.0;
        }
        a--; b--; /* 1-based -> 0-based (mmio_highlevel.h:702-703) */
        counter[a]++;
        ri[i] = a;
        ci[i] = b;
        vv[i] = orc_f64_to_f16(fv);
    }
    fclose(f);

    if (sym)
        for (int i = 0; i < nz; i++)
            if (ri[i] != ci[i]) counter[ci[i]]++;

    /* exclusive scan over m+1 entries */
    {
        int32_t run = 0;
        for (int i = 0; i <= m; i++) { int32_t c = counter[i]; counter[i] = run; run += c; }
    }
    int32_t *rp = (int32_t *)malloc(sizeof(int32_t) * ((size_t)m + 1));
    memcpy(rp, counter, sizeof(int32_t) * ((size_t)m + 1));
    int32_t total = rp[m];
    int32_t *cj = (int32_t *)malloc(sizeof(int32_t) * (size_t)(total > 0 ? total : 1));
    uint16_t *cv = (uint16_t *)malloc(sizeof(uint16_t) * (size_t)(total > 0 ? total : 1));
    memset(counter, 0, sizeof(int32_t) * ((size_t)m + 1));

    /* scatter in file order; mirrored entry right after its original
     * (mmio_highlevel.h:736-767) */
    for (int i = 0; i < nz; i++) {
        int32_t o = rp[ri[i]] + counter[ri[i]]++;
        cj[o] = ci[i];
        cv[o] = vv[i];
        if (sym && ri[i] != ci[i]) {
            o = rp[ci[i]] + counter[ci[i]]++;
            cj[o] = ri[i];
            cv[o] = vv[i];
        }
    }
    free(counter); free(ri); free(ci); free(vv);
    *m_out = m; *n_out = n; *nnz_out = total; *is_symmetric = sym;
    *row_ptr = rp; *col_idx = cj; *val = cv;
    return 0;
}

void orc_free(void *p) { free(p); }

/* --------------------------------------------------------- CSR -> BCSR ---- */

/* Restates SparseMatrix::csrToBcsr (src/cuda_hgemm/src/common/matrix.h:376-502)
 * including the two dense Mb x Kb maps, so it is only usable where those fit.
 * block_info / rel_map may be NULL if the caller does not want them back.
 * counts[0..2] = nonzeroBlocks, denseBlocks, sparseBlocks (matrix.h:176). */
int orc_csr_to_bcsr(int64_t m, int64_t n, const int32_t *row_ptr, const int32_t *col_idx,
                    const uint16_t *val, int64_t *counts, int32_t **b_row_ptr,
                    int32_t **b_col_idx, uint16_t **b_val, int32_t **block_info_out,
                    int32_t **rel_map_out)
{
    int64_t kb = (n + ORC_BS - 1) / ORC_BS, mb = (m + ORC_BS - 1) / ORC_BS;
    int64_t nblocks = kb * mb;
    int32_t *info = (int32_t *)calloc((size_t)(nblocks > 0 ? nblocks : 1), sizeof(int32_t));
    if (!info) return -1;
    int64_t nzb = 0, dense = 0, sparse = 0;
    /* pass 1: flag blocks, 2:4 heuristic (matrix.h:388-423) */
    for (int64_t row = 0; row < m; row++) {
        for (int64_t j = row_ptr[row]; j < row_ptr[row + 1]; j++) {
            int64_t col = col_idx[j];
            int64_t bi = (row / ORC_BS) * kb + col / ORC_BS;
            if (info[bi] == 0) {
                info[bi] = 1; nzb++; sparse++;
            } else if (info[bi] == 1) {
                int64_t r = col % 4;
                if ((r == 2 || r == 3) && j >= (int64_t)row_ptr[row] + 2 &&
                    col_idx[j - 1] == col - 1 && col_idx[j - 2] == col - 2) {
                    info[bi] = 2; dense++; sparse--;
                }
            }
        }
    }
    /* pass 2: running index of nonzero blocks (matrix.h:425-431) */
    int32_t *rel = (int32_t *)malloc(sizeof(int32_t) * (size_t)(nblocks > 0 ? nblocks : 1));
    {
        int32_t r = 0;
        for (int64_t i = 0; i < nblocks; i++) rel[i] = info[i] ? r++ : -1;
    }
    /* pass 3: row_ptr / col_idx (matrix.h:441-463); col_idx holds the absolute
     * column of the block's first column, not the block index (matrix.h:455) */
    int32_t *brp = (int32_t *)calloc((size_t)(m / ORC_BS + 1), sizeof(int32_t));
    int32_t *bci = (int32_t *)malloc(sizeof(int32_t) * (size_t)(nzb > 0 ? nzb : 1));
    uint16_t *bv = (uint16_t *)calloc((size_t)(nzb > 0 ? nzb : 1) * ORC_BS * ORC_BS, sizeof(uint16_t));
    int64_t nb = 0;
    for (int64_t row = 0; row < m; row += ORC_BS) {
        brp[row / ORC_BS] = (int32_t)nb;
        for (int64_t col = 0; col < n; col += ORC_BS)
            if (info[(row / ORC_BS) * kb + col / ORC_BS]) bci[nb++] = (int32_t)col;
    }
    brp[m / ORC_BS] = (int32_t)nb;
    /* pass 4: values, row-major inside a block, later duplicate wins
     * (matrix.h:470-487) */
    for (int64_t row = 0; row < m; row++) {
        for (int64_t j = row_ptr[row]; j < row_ptr[row + 1]; j++) {
            int64_t col = col_idx[j];
            int64_t bi = (row / ORC_BS) * kb + col / ORC_BS;
            bv[(int64_t)rel[bi] * ORC_BS * ORC_BS + (row % ORC_BS) * ORC_BS + col % ORC_BS] = val[j];
        }
    }
    counts[0] = nzb; counts[1] = dense; counts[2] = sparse;
    *b_row_ptr = brp; *b_col_idx = bci; *b_val = bv;
    if (block_info_out) *block_info_out = info; else free(info);
    if (rel_map_out) *rel_map_out = rel; else free(rel);
    return 0;
}

/* ------------------------------------------------------------- CPU SpMM --- */

/* C (row-major, fp32, M x N) = A_csr * B, fp16 inputs widened to fp32, fp32
 * accumulation, serial.  Loop nest row -> nonzero -> B column follows
 * CSR::multiply (preprocess/src/general/csr.cpp:47-63).  Operand layouts follow
 * the SpMM kernel boundary instead of that routine's column-major C:
 * B column-major with leading dimension K (src/cuda_hgemm/src/mma/mmaCBT.cu:52),
 * C row-major (mmaCBT.cu:78).  b_row_major != 0 selects B[k*N + n]. */
void orc_spmm_csr_f32(int64_t m, int64_t n_cols, int64_t k, const int32_t *row_ptr,
                      const int32_t *col_idx, const uint16_t *val, const uint16_t *B,
                      int b_row_major, float *C)
{
    for (int64_t i = 0; i < m; i++) {
        float *c = C + i * n_cols;
        for (int64_t j = 0; j < n_cols; j++) c[j] = 0.0f;
        for (int64_t p = row_ptr[i]; p < row_ptr[i + 1]; p++) {
            int64_t col = col_idx[p];
            float a = orc_f16_to_f32(val[p]);
            for (int64_t j = 0; j < n_cols; j++) {
                uint16_t b = b_row_major ? B[col * n_cols + j] : B[j * k + col];
                c[j] += a * orc_f16_to_f32(b);
            }
        }
    }
}

/* Blocked multiply: block row -> nonzero block -> i/j/k dense loop, the loop
 * nest of VBR::multiply (preprocess/src/general/vbr.cpp:323-372) applied to the
 * 16x16 BCSR arrays of matrix.h:441-487 (row-major blocks, absolute col_idx).
 * B is first widened to fp32 row-major so the inner loop is a plain saxpy.
 * threads <= 1 runs serially (the reference has no OpenMP pragma); threads > 1
 * splits block rows over OpenMP threads for the all-cores baseline. */
void orc_spmm_bcsr_f32(int64_t m, int64_t n_cols, int64_t k, const int32_t *b_row_ptr,
                       const int32_t *b_col_idx, const uint16_t *b_val, const uint16_t *B,
                       int b_row_major, float *C, int threads)
{
    float *Bf = (float *)malloc(sizeof(float) * (size_t)k * (size_t)n_cols);
    if (b_row_major) {
        for (int64_t i = 0; i < k * n_cols; i++) Bf[i] = orc_f16_to_f32(B[i]);
    } else {
        for (int64_t j = 0; j < n_cols; j++)
            for (int64_t r = 0; r < k; r++) Bf[r * n_cols + j] = orc_f16_to_f32(B[j * k + r]);
    }
    int64_t mb = m / ORC_BS;
    (void)threads;
#ifdef _OPENMP
#pragma omp parallel for schedule(dynamic, 4) num_threads(threads > 1 ? threads : 1)
#endif
    for (int64_t br = 0; br < mb; br++) {
        float *c = C + br * ORC_BS * n_cols;
        for (int64_t i = 0; i < ORC_BS * n_cols; i++) c[i] = 0.0f;
        for (int64_t p = b_row_ptr[br]; p < b_row_ptr[br + 1]; p++) {
            const uint16_t *blk = b_val + p * ORC_BS * ORC_BS;
            const float *bp = Bf + (int64_t)b_col_idx[p] * n_cols;
            for (int i = 0; i < ORC_BS; i++) {
                float *ci = c + i * n_cols;
                for (int kk = 0; kk < ORC_BS; kk++) {
                    float a = orc_f16_to_f32(blk[i * ORC_BS + kk]);
                    const float *bk = bp + kk * n_cols;
                    for (int64_t j = 0; j < n_cols; j++) ci[j] += a * bk[j];
                }
            }
        }
    }
    free(Bf);
}

int orc_max_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* Verification metric named by the port's acceptance bar: for every row i,
 * max_j |C[i][j] - ref[i][j]| / ||ref[i][:]||_2, maximised over rows; rows whose
 * reference norm is 0 contribute their absolute error.  (The reference's own
 * Matrix::checkValue, common/matrix.h:103-121, reports max/mean absolute
 * difference; both are returned: out[0]=max relative-to-row-L2, out[1]=max abs,
 * out[2]=mean abs.) */
void orc_compare_f16_vs_f32(const uint16_t *C, const float *ref, int64_t m, int64_t n_cols,
                            double *out)
{
    double worst = 0.0, max_abs = 0.0, sum_abs = 0.0;
    for (int64_t i = 0; i < m; i++) {
        double nrm = 0.0, row_max = 0.0;
        for (int64_t j = 0; j < n_cols; j++) {
            double r = ref[i * n_cols + j];
            double d = (double)orc_f16_to_f32(C[i * n_cols + j]) - r;
            if (d < 0) d = -d;
            if (!(d == d)) d = 1e30; /* NaN counts as a gross error */
            nrm += r * r;
            if (d > row_max) row_max = d;
            sum_abs += d;
        }
        if (row_max > max_abs) max_abs = row_max;
        double rel = nrm > 0.0 ? row_max / __builtin_sqrt(nrm) : row_max;
        if (rel > worst) worst = rel;
    }
    out[0] = worst;
    out[1] = max_abs;
    out[2] = (m * n_cols) ? sum_abs / (double)(m * n_cols) : 0.0;
}
