// Binary container for CSR / BCSR matrices and their row / column permutations.
//
// The reference stores matrices as text only (Matrix Market `.mtx`, read with one fscanf per
// entry by mmio_allinone, src/cuda_hgemm/src/common/mmio_highlevel.h:619-786, and edge lists
// `.el` for the reorder program, preprocess/src/general/csr.cpp:153-290); parsing dominates its
// start-up.  This container holds exactly the arrays those loaders produce, so a matrix is
// parsed (and reordered, and blocked) once and mapped in afterwards.
//
// Layout (little endian), every section starts on a 64-byte boundary:
//   0   char[8]  "SMATBIN1"
//   8   u32      kind: 1 = CSR (fp16 values), 2 = BCSR 16x16 (fp16 blocks)
//   12  u32      flags: bit 0 = perm_rows present, bit 1 = perm_cols present
//   16  u64      M      24 u64 K      32 u64 n (nnz for CSR, nonzero blocks for BCSR)
//   40  u64      FNV-1a 64 of all section payloads in file order
//   48  u8[16]   zero
//   64  int32    row_ptr[M + 1]  (CSR)  or  b_row_ptr[M/16 + 1]  (BCSR)
//       int32    col_idx[n]
//       u16      val[n]          (CSR)  or  b_val[n * 256]       (BCSR)
//       int64    perm_rows[M]    (flag bit 0)      perm[new] = old
//       int64    perm_cols[K]    (flag bit 1)
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "../../include/smat.h"
#include "errors.h"
#include "half.h"

using namespace smat;

namespace {

constexpr char MAGIC[8] = {'S', 'M', 'A', 'T', 'B', 'I', 'N', '1'};

struct Header {
    char magic[8];
    uint32_t kind, flags;
    uint64_t M, K, n, checksum;
    uint8_t zero[16];
};
static_assert(sizeof(Header) == 64, "header is one 64-byte line");

uint64_t fnv1a(uint64_t h, const void *data, size_t bytes)
{
    const unsigned char *p = static_cast<const unsigned char *>(data);
    for (size_t i = 0; i < bytes; i++) { h ^= p[i]; h *= 0x100000001b3ull; }
    return h;
}

struct Section { const void *data; size_t bytes; };

int write_file(const char *path, uint32_t kind, size_t M, size_t K, size_t n, const Section *sec, int n_sec,
               uint32_t flags)
{
    if (!path) return set_error(SMAT_ERR_INVALID, "path must not be NULL");
    Header h{};
    memcpy(h.magic, MAGIC, 8);
    h.kind = kind; h.flags = flags; h.M = M; h.K = K; h.n = n;
    h.checksum = 0xcbf29ce484222325ull;
    for (int i = 0; i < n_sec; i++) h.checksum = fnv1a(h.checksum, sec[i].data, sec[i].bytes);
    FILE *f = fopen(path, "wb");
    if (!f) return set_error(SMAT_ERR_IO, "cannot open %s for writing", path);
    bool ok = fwrite(&h, sizeof h, 1, f) == 1;
    static const char pad[64] = {0};
    for (int i = 0; ok && i < n_sec; i++) {
        if (sec[i].bytes) ok = fwrite(sec[i].data, 1, sec[i].bytes, f) == sec[i].bytes;
        const size_t rest = (64 - sec[i].bytes % 64) % 64;
        if (ok && rest) ok = fwrite(pad, 1, rest, f) == rest;
    }
    ok = (fclose(f) == 0) && ok;
    if (!ok) return set_error(SMAT_ERR_IO, "short write to %s", path);
    return SMAT_OK;
}

} // namespace

static int smat_bin_write_csr_impl(const char *path, size_t M, size_t K, const int32_t *row_ptr,
                                   const int32_t *col_idx, const uint16_t *val, const int64_t *perm_rows,
                                   const int64_t *perm_cols)
{
    if (!row_ptr) return set_error(SMAT_ERR_INVALID, "row_ptr must not be NULL");
    const size_t nnz = (size_t)row_ptr[M];
    if (nnz && (!col_idx || !val)) return set_error(SMAT_ERR_INVALID, "col_idx/val must not be NULL");
    Section sec[5] = {{row_ptr, (M + 1) * 4}, {col_idx, nnz * 4}, {val, nnz * 2}, {nullptr, 0}, {nullptr, 0}};
    int n_sec = 3;
    uint32_t flags = 0;
    if (perm_rows) { sec[n_sec++] = {perm_rows, M * 8}; flags |= 1; }
    if (perm_cols) { sec[n_sec++] = {perm_cols, K * 8}; flags |= 2; }
    return write_file(path, 1, M, K, nnz, sec, n_sec, flags);
}

extern "C" int smat_bin_write_csr(const char *path, size_t M, size_t K, const int32_t *row_ptr,
                                   const int32_t *col_idx, const uint16_t *val, const int64_t *perm_rows,
                                   const int64_t *perm_cols)
{
    return smat::guarded("smat_bin_write_csr", [&] { return smat_bin_write_csr_impl(path, M, K, row_ptr, col_idx, val, perm_rows, perm_cols); });
}

static int smat_bin_write_bcsr_impl(const char *path, size_t M, size_t K, size_t nnzb, const int32_t *b_row_ptr,
                                    const int32_t *b_col_idx, const uint16_t *b_val, const int64_t *perm_rows,
                                    const int64_t *perm_cols)
{
    if (!b_row_ptr) return set_error(SMAT_ERR_INVALID, "b_row_ptr must not be NULL");
    if (M % 16 || K % 16) return set_error(SMAT_ERR_INVALID, "M and K must be multiples of 16");
    if ((size_t)b_row_ptr[M / 16] != nnzb) return set_error(SMAT_ERR_INVALID, "b_row_ptr[M/16] != nnzb");
    if (nnzb && (!b_col_idx || !b_val)) return set_error(SMAT_ERR_INVALID, "b_col_idx/b_val must not be NULL");
    Section sec[5] = {{b_row_ptr, (M / 16 + 1) * 4}, {b_col_idx, nnzb * 4}, {b_val, nnzb * 512}, {nullptr, 0}, {nullptr, 0}};
    int n_sec = 3;
    uint32_t flags = 0;
    if (perm_rows) { sec[n_sec++] = {perm_rows, M * 8}; flags |= 1; }
    if (perm_cols) { sec[n_sec++] = {perm_cols, K * 8}; flags |= 2; }
    return write_file(path, 2, M, K, nnzb, sec, n_sec, flags);
}

extern "C" int smat_bin_write_bcsr(const char *path, size_t M, size_t K, size_t nnzb, const int32_t *b_row_ptr,
                                    const int32_t *b_col_idx, const uint16_t *b_val, const int64_t *perm_rows,
                                    const int64_t *perm_cols)
{
    return smat::guarded("smat_bin_write_bcsr", [&] { return smat_bin_write_bcsr_impl(path, M, K, nnzb, b_row_ptr, b_col_idx, b_val, perm_rows, perm_cols); });
}

static int smat_bin_read_impl(const char *path, int *kind, size_t *M, size_t *K, size_t *n, int32_t **row_ptr,
                              int32_t **col_idx, uint16_t **val, int64_t **perm_rows, int64_t **perm_cols)
{
    if (!path || !kind || !M || !K || !n || !row_ptr || !col_idx || !val)
        return set_error(SMAT_ERR_INVALID, "NULL argument");
    *row_ptr = nullptr; *col_idx = nullptr; *val = nullptr;
    if (perm_rows) *perm_rows = nullptr;
    if (perm_cols) *perm_cols = nullptr;
    FILE *f = fopen(path, "rb");
    if (!f) return set_error(SMAT_ERR_IO, "cannot open %s", path);
    Header h;
    if (fread(&h, sizeof h, 1, f) != 1 || memcmp(h.magic, MAGIC, 8) != 0) {
        fclose(f);
        return set_error(SMAT_ERR_IO, "%s is not a SMATBIN1 file", path);
    }
    if ((h.kind != 1 && h.kind != 2) || (h.flags & ~3u) || h.M > 0x7fffffffull * 16 || h.K > 0x7fffffffull * 16 ||
        h.n > 0x7fffffffull ||
        (h.kind == 2 && (h.M % 16 || h.K % 16))) {
        fclose(f);
        return set_error(SMAT_ERR_IO, "%s: inconsistent header", path);
    }
    const size_t rows = h.kind == 1 ? h.M : h.M / 16;
    const size_t bytes[5] = {(rows + 1) * 4, h.n * 4, h.n * (h.kind == 1 ? 2u : 512u),
                             (h.flags & 1) ? h.M * 8 : 0, (h.flags & 2) ? h.K * 8 : 0};
    void *buf[5] = {nullptr, nullptr, nullptr, nullptr, nullptr};
    uint64_t sum = 0xcbf29ce484222325ull;
    bool ok = true;
    int rc = SMAT_OK;
    for (int i = 0; ok && i < 5; i++) {
        if (i >= 3 && !bytes[i]) continue;
        buf[i] = malloc(bytes[i] ? bytes[i] : 1);
        if (!buf[i]) { rc = set_error(SMAT_ERR_NOMEM, "out of host memory reading %s", path); ok = false; break; }
        if (bytes[i] && fread(buf[i], 1, bytes[i], f) != bytes[i]) ok = false;
        const size_t rest = (64 - bytes[i] % 64) % 64;
        if (ok && rest && fseek(f, (long)rest, SEEK_CUR) != 0) ok = false;
        if (ok) sum = fnv1a(sum, buf[i], bytes[i]);
    }
    fclose(f);
    if (ok && sum != h.checksum) { ok = false; rc = set_error(SMAT_ERR_IO, "%s: checksum mismatch", path); }
    if (ok) {
        const int32_t *rp = static_cast<const int32_t *>(buf[0]);
        if (rp[0] != 0 || (uint64_t)rp[rows] != h.n) { ok = false; rc = set_error(SMAT_ERR_IO, "%s: row pointer does not match the entry count", path); }
        for (size_t r = 0; ok && r < rows; r++)
            if (rp[r + 1] < rp[r]) { ok = false; rc = set_error(SMAT_ERR_IO, "%s: row pointer decreases at row %zu", path, r); }
        const int32_t *ci = static_cast<const int32_t *>(buf[1]);
        const int32_t step = h.kind == 2 ? 16 : 1;
        for (size_t e = 0; ok && e < h.n; e++)
            if (ci[e] < 0 || (uint64_t)ci[e] >= h.K || ci[e] % step) {
                ok = false;
                rc = set_error(SMAT_ERR_IO, "%s: column index %d of entry %zu is not a %scolumn of K = %llu", path, ci[e], e,
                               h.kind == 2 ? "block " : "", (unsigned long long)h.K);
            }
    }
    if (!ok) {
        for (void *b : buf) free(b);
        return rc != SMAT_OK ? rc : set_error(SMAT_ERR_IO, "%s: truncated file", path);
    }
    *kind = (int)h.kind; *M = h.M; *K = h.K; *n = h.n;
    *row_ptr = static_cast<int32_t *>(buf[0]);
    *col_idx = static_cast<int32_t *>(buf[1]);
    *val = static_cast<uint16_t *>(buf[2]);
    if (perm_rows) *perm_rows = static_cast<int64_t *>(buf[3]); else free(buf[3]);
    if (perm_cols) *perm_cols = static_cast<int64_t *>(buf[4]); else free(buf[4]);
    return SMAT_OK;
}

extern "C" int smat_bin_read(const char *path, int *kind, size_t *M, size_t *K, size_t *n, int32_t **row_ptr,
                              int32_t **col_idx, uint16_t **val, int64_t **perm_rows, int64_t **perm_cols)
{
    return smat::guarded("smat_bin_read", [&] { return smat_bin_read_impl(path, kind, M, K, n, row_ptr, col_idx, val, perm_rows, perm_cols); });
}

// CSR -> Matrix Market "coordinate real general", entries in storage order, 1-based; a value is
// printed with enough digits to read back to the same fp16 (any fp16 is exact in 11 significant
// decimal digits or fewer when printed from its double).
static int smat_mtx_write_impl(const char *path, size_t M, size_t K, const int32_t *row_ptr,
                               const int32_t *col_idx, const uint16_t *val)
{
    if (!path || !row_ptr) return set_error(SMAT_ERR_INVALID, "NULL argument");
    FILE *f = fopen(path, "w");
    if (!f) return set_error(SMAT_ERR_IO, "cannot open %s for writing", path);
    const long nnz = row_ptr[M];
    fprintf(f, "%%%%MatrixMarket matrix coordinate real general\n%zu %zu %ld\n", M, K, nnz);
    for (size_t r = 0; r < M; r++)
        for (long j = row_ptr[r]; j < row_ptr[r + 1]; j++)
            fprintf(f, "%zu %d %.11g\n", r + 1, col_idx[j] + 1, (double)half_to_float(val[j]));
    if (fclose(f) != 0) return set_error(SMAT_ERR_IO, "short write to %s", path);
    return SMAT_OK;
}

extern "C" int smat_mtx_write(const char *path, size_t M, size_t K, const int32_t *row_ptr,
                               const int32_t *col_idx, const uint16_t *val)
{
    return smat::guarded("smat_mtx_write", [&] { return smat_mtx_write_impl(path, M, K, row_ptr, col_idx, val); });
}
