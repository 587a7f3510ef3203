// Matrix Market (coordinate) -> CSR with the loader semantics of the reference:
// mmio_allinone (src/cuda_hgemm/src/common/mmio_highlevel.h:619-786) on top of
// mm_read_banner / mm_read_mtx_crd_size (src/cuda_hgemm/src/common/mmio.h:399-565,
// 569-625), padSparseMatrix (mmio_highlevel.h:609-616) and exclusive_scan
// (mmio_highlevel.h:11-26).
//
// Kept: dimensions rounded up to multiples of 16 before anything else; field
// types real / complex (real part) / integer / pattern (= 1.0); 1-based -> 0-based;
// symmetric and hermitian (not skew-symmetric) entries mirrored right after the
// original; counting sort by row that keeps file order inside a row and keeps
// duplicates; double -> fp16 in one rounding.
// Changed: the body is tokenised from one buffered read instead of one fscanf
// per entry, indices are range-checked, and failures are reported.
#include <cctype>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "../../include/smat.h"
#include "errors.h"
#include "half.h"

using namespace smat;

namespace {

struct Cursor {
    const char *p, *end;
    void skip_ws() { while (p < end && isspace((unsigned char)*p)) ++p; }
    bool read_long(long &v)
    {
        skip_ws();
        if (p >= end) return false;
        char *q;
        v = strtol(p, &q, 10);
        if (q == p) return false;
        p = q;
        return true;
    }
    bool read_double(double &v)
    {
        skip_ws();
        if (p >= end) return false;
        char *q;
        v = strtod(p, &q);
        if (q == p) return false;
        p = q;
        return true;
    }
};

std::string lower(std::string s)
{
    for (auto &c : s) c = (char)tolower((unsigned char)c);
    return s;
}

} // namespace

extern "C" void smat_host_free(void *p) { free(p); }

static int smat_mtx_read_impl(const char *path, size_t *M, size_t *K, size_t *nnz_out,
                              int *is_symmetric, int32_t **row_ptr, int32_t **col_idx,
                              uint16_t **val, int *ref_code)
{
    if (ref_code) *ref_code = 0;
    if (!path || !M || !K || !nnz_out || !row_ptr || !col_idx || !val)
        return set_error(SMAT_ERR_INVALID, "NULL argument");
    FILE *f = fopen(path, "rb");
    if (!f) {
        if (ref_code) *ref_code = -1;
        return set_error(SMAT_ERR_IO, "cannot open %s", path);
    }
    std::string data;
    {
        char buf[1 << 16];
        size_t got;
        while ((got = fread(buf, 1, sizeof buf, f)) > 0) data.append(buf, got);
    }
    fclose(f);
    data.push_back('\0'); // strtol / strtod stop here

    // banner: "%%MatrixMarket matrix coordinate <field> <symmetry>"
    size_t pos = data.find('\n');
    std::string first = data.substr(0, pos == std::string::npos ? data.size() - 1 : pos);
    char banner[64], obj[64], fmt[64], field[64], symm[64];
    if (sscanf(first.c_str(), "%63s %63s %63s %63s %63s", banner, obj, fmt, field, symm) != 5 ||
        strncmp(banner, "%%MatrixMarket", 14) != 0 || lower(obj) != "matrix") {
        if (ref_code) *ref_code = -2;
        return set_error(SMAT_ERR_IO, "%s: not a Matrix Market banner", path);
    }
    const std::string sfmt = lower(fmt), sfield = lower(field), ssymm = lower(symm);
    const bool is_real = sfield == "real", is_complex = sfield == "complex";
    const bool is_integer = sfield == "integer", is_pattern = sfield == "pattern";
    const bool sym = ssymm == "symmetric" || ssymm == "hermitian";
    if (sfmt != "coordinate" || !(is_real || is_complex || is_integer || is_pattern) ||
        !(sym || ssymm == "general" || ssymm == "skew-symmetric")) {
        if (ref_code) *ref_code = -2;
        return set_error(SMAT_ERR_IO, "%s: unsupported Matrix Market type '%s %s %s'", path, fmt, field, symm);
    }

    // comment lines, then "rows cols entries"
    Cursor c{data.data() + (pos == std::string::npos ? data.size() - 1 : pos + 1),
             data.data() + data.size() - 1};
    while (c.p < c.end && *c.p == '%') {
        const char *nl = (const char *)memchr(c.p, '\n', (size_t)(c.end - c.p));
        c.p = nl ? nl + 1 : c.end;
    }
    long m0, n0, nz;
    if (!c.read_long(m0) || !c.read_long(n0) || !c.read_long(nz) || m0 < 0 || n0 < 0 || nz < 0) {
        if (ref_code) *ref_code = -4;
        return set_error(SMAT_ERR_IO, "%s: bad size line", path);
    }
    const long m = (m0 + 15) / 16 * 16, n = (n0 + 15) / 16 * 16;
    // an entry takes at least "1 1\n": a count the rest of the file cannot hold is a garbled size line,
    // and the CSR indices are int32
    if ((size_t)nz > (size_t)(c.end - c.p) / 4 + 1 || m0 > 0x7ffffff0L || n0 > 0x7ffffff0L || nz > 0x3fffffffL) {
        if (ref_code) *ref_code = -4;
        return set_error(SMAT_ERR_IO, "%s: size line '%ld %ld %ld' does not fit the file or the int32 index range", path, m0, n0, nz);
    }

    std::vector<int32_t> ri((size_t)nz), ci((size_t)nz);
    std::vector<uint16_t> vv((size_t)nz);
    std::vector<int64_t> count((size_t)m + 1, 0);
    for (long i = 0; i < nz; i++) {
        long a, b, iv;
        double fv = 1.0, fim;
        bool ok = c.read_long(a) && c.read_long(b);
        if (ok && is_real) ok = c.read_double(fv);
        else if (ok && is_complex) ok = c.read_double(fv) && c.read_double(fim);
        else if (ok && is_integer) { ok = c.read_long(iv); fv = (double)iv; }
        if (!ok) return set_error(SMAT_ERR_IO, "%s: entry %ld of %ld is missing or malformed", path, i + 1, nz);
        if (a < 1 || a > m || b < 1 || b > n)
            return set_error(SMAT_ERR_IO, "%s: entry %ld (%ld,%ld) lies outside the padded %ld x %ld matrix", path, i + 1, a, b, m, n);
        if (sym && b > m)
            return set_error(SMAT_ERR_IO, "%s: symmetric entry %ld cannot be mirrored", path, i + 1);
        ri[i] = (int32_t)(a - 1);
        ci[i] = (int32_t)(b - 1);
        vv[i] = half_from_double(fv);
        count[a - 1]++;
        if (sym && a != b) count[b - 1]++;
    }
    int64_t total = 0;
    for (long r = 0; r <= m; r++) { int64_t t = count[r]; count[r] = total; total += t; }
    if (total > 0x7fffffff) return set_error(SMAT_ERR_INVALID, "%s: more than 2^31-1 entries", path);

    int32_t *rp = (int32_t *)malloc(sizeof(int32_t) * ((size_t)m + 1));
    int32_t *cj = (int32_t *)malloc(sizeof(int32_t) * (size_t)(total ? total : 1));
    uint16_t *cv = (uint16_t *)malloc(sizeof(uint16_t) * (size_t)(total ? total : 1));
    if (!rp || !cj || !cv) {
        free(rp); free(cj); free(cv);
        return set_error(SMAT_ERR_NOMEM, "out of host memory");
    }
    for (long r = 0; r <= m; r++) rp[r] = (int32_t)count[r];
    std::vector<int64_t> fill(count.begin(), count.end() - 1);
    for (long i = 0; i < nz; i++) {
        int64_t o = fill[ri[i]]++;
        cj[o] = ci[i];
        cv[o] = vv[i];
        if (sym && ri[i] != ci[i]) {
            o = fill[ci[i]]++;
            cj[o] = ri[i];
            cv[o] = vv[i];
        }
    }
    *M = (size_t)m; *K = (size_t)n; *nnz_out = (size_t)total;
    if (is_symmetric) *is_symmetric = sym ? 1 : 0;
    *row_ptr = rp; *col_idx = cj; *val = cv;
    return SMAT_OK;
}

extern "C" int smat_mtx_read(const char *path, size_t *M, size_t *K, size_t *nnz_out,
                              int *is_symmetric, int32_t **row_ptr, int32_t **col_idx,
                              uint16_t **val, int *ref_code)
{
    return smat::guarded("smat_mtx_read", [&] { return smat_mtx_read_impl(path, M, K, nnz_out, is_symmetric, row_ptr, col_idx, val, ref_code); });
}
