// `smat_convert`: Matrix Market <-> SMATBIN1 container, with the optional reorder and blocking
// steps of the SpMM flow done once, ahead of time.
//
//   smat_convert -in a.mtx -out a.smat                    CSR container (loader semantics of
//                                                         mmio_allinone, mmio_highlevel.h:619-786)
//   smat_convert -in a.mtx -out a.smat -reorder [-tau 0.5] [-b 16] [-B 16]
//                                                         row pass + column pass of the reference's
//                                                         Matrix_Blocking -a 5 -F 1 (src/reorder.py:107-182),
//                                                         permutations stored with the permuted CSR
//   smat_convert -in a.mtx -out a.smat -bcsr [-reorder]   16x16 BCSR container (matrix.h:376-502)
//   smat_convert -in a.smat -out a.mtx                    back to text (CSR containers only)
#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

#include "../../../include/smat.h"
#include "flags.h"

#define CHECK(call)                                                                   \
    do {                                                                              \
        if ((call) != SMAT_OK) {                                                      \
            fprintf(stderr, "smat_convert: %s\n", smat_last_error());                 \
            return 1;                                                                 \
        }                                                                             \
    } while (0)

static bool is_container(const std::string &path)
{
    FILE *f = fopen(path.c_str(), "rb");
    if (!f) return false;
    char m[8] = {0};
    const bool ok = fread(m, 1, 8, f) == 8 && memcmp(m, "SMATBIN1", 8) == 0;
    fclose(f);
    return ok;
}

int main(int argc, char **argv)
{
    Flags f(argc, argv);
    const std::string in = f.str("in", ""), out = f.str("out", "");
    if (in.empty() || out.empty()) {
        fprintf(stderr, "usage: smat_convert -in <a.mtx|a.smat> -out <a.smat|a.mtx> [-reorder] [-tau t] [-b cb] [-B rb] [-bcsr]\n");
        return 2;
    }
    size_t M = 0, K = 0, n = 0;
    int32_t *rp = nullptr, *ci = nullptr;
    uint16_t *v = nullptr;
    int64_t *pr = nullptr, *pc = nullptr;
    if (is_container(in)) {
        int kind = 0;
        CHECK(smat_bin_read(in.c_str(), &kind, &M, &K, &n, &rp, &ci, &v, &pr, &pc));
        if (kind != SMAT_BIN_CSR) { fprintf(stderr, "smat_convert: %s holds BCSR; only CSR containers convert back to text\n", in.c_str()); return 1; }
        CHECK(smat_mtx_write(out.c_str(), M, K, rp, ci, v));
        printf("%s: %zu x %zu, %zu entries -> %s\n", in.c_str(), M, K, n, out.c_str());
        return 0;
    }
    int sym = 0;
    CHECK(smat_mtx_read(in.c_str(), &M, &K, &n, &sym, &rp, &ci, &v, nullptr));
    std::vector<int64_t> perm_rows, perm_cols;
    if (f.flag("reorder", false)) {
        perm_rows.resize(M);
        perm_cols.resize(K);
        int64_t sr[4], sc[4];
        CHECK(smat_reorder_csr(M, K, rp, ci, f.num("b", 16), f.num("B", 16), (float)f.real("tau", 0.5), 1,
                               perm_rows.data(), perm_cols.data(), sr, sc));
        int32_t *rp2, *ci2;
        uint16_t *v2;
        CHECK(smat_permute_csr(M, K, rp, ci, v, perm_rows.data(), perm_cols.data(), &rp2, &ci2, &v2));
        smat_host_free(rp); smat_host_free(ci); smat_host_free(v);
        rp = rp2; ci = ci2; v = v2;
        printf("reorder: %ld nonzero blocks after the row pass, %ld after the column pass\n", (long)sr[2], (long)sc[2]);
    }
    const int64_t *prp = perm_rows.empty() ? nullptr : perm_rows.data();
    const int64_t *pcp = perm_cols.empty() ? nullptr : perm_cols.data();
    if (f.flag("bcsr", false)) {
        int64_t counts[3];
        int32_t *brp, *bci;
        uint16_t *bv;
        CHECK(smat_csr_to_bcsr(M, K, rp, ci, v, counts, &brp, &bci, &bv, nullptr, nullptr));
        CHECK(smat_bin_write_bcsr(out.c_str(), M, K, (size_t)counts[0], brp, bci, bv, prp, pcp));
        printf("%s: %zu x %zu, %zu entries, %ld blocks -> %s (BCSR)\n", in.c_str(), M, K, n, (long)counts[0], out.c_str());
    } else {
        CHECK(smat_bin_write_csr(out.c_str(), M, K, rp, ci, v, prp, pcp));
        printf("%s: %zu x %zu, %zu entries -> %s (CSR)\n", in.c_str(), M, K, n, out.c_str());
    }
    return 0;
}
