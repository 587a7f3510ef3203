// `Matrix_Blocking`: command-line front end of the row reordering, accepting the
// invocation src/reorder.py:131-132 uses on the reference program
// (preprocess/test/general/Matrix_Blocking.cpp:10-50):
//     Matrix_Blocking -f <file.el> -a 5 -b <col_block> -B <row_block> -F 1 -t <tau> [-o <stats>] [-v 0|1]
// Reads an edge list "row col [value]" with ascending rows
// (preprocess/src/general/csr.cpp:166-290), writes
//   <stats>       two CSV lines (header, values) with the integer fields of
//                 save_blocking_data (preprocess/src/general/utilities.cpp:175-240)
//   <stats>.g     "GROUPING,g0,g1,...," - the block-row id of every row
//   <stem>_reordered.el   "newrow col" per nonzero (Matrix_Blocking.cpp:40-47)
// Only -a 5 with -F 1 (the one path the SpMM flow uses) is implemented.
#include <cstdio>
#include <cstdlib>
#include <fstream>
#include <sstream>
#include <string>
#include <vector>

#include "../../../include/smat.h"
#include "flags.h"

int main(int argc, char **argv)
{
    Flags f(argc, argv);
    const std::string file = f.str("f", "");
    const std::string out = f.str("o", "results/TEST_results.txt");
    const long algo = f.num("a", 3), cb = f.num("b", 3), rb = f.num("B", 3), fixed = f.num("F", 0);
    const float tau = (float)f.real("t", 0.1);
    if (file.empty()) { fprintf(stderr, "No graph input specified.\n"); return 2; }
    if (algo != 5 || fixed != 1) {
        fprintf(stderr, "only '-a 5 -F 1' (iterative blocking with fixed-size groups) is implemented\n");
        return 2;
    }
    std::ifstream in(file);
    if (!in) { fprintf(stderr, "cannot open %s\n", file.c_str()); return 1; }
    std::vector<int64_t> row_ptr{0}, cols;
    std::string line;
    long current = -1, max_col = -1;
    while (std::getline(in, line)) {
        if (line.empty() || line[0] == '#' || line[0] == '%') continue;
        std::istringstream ls(line);
        long r, c;
        if (!(ls >> r >> c)) continue;
        if (r < current) { fprintf(stderr, "CSR.read_from_edgelist indices must be in ascending order\n"); return 1; }
        while (current < r) { row_ptr.push_back((int64_t)cols.size()); current++; }
        cols.push_back(c);
        row_ptr.back() = (int64_t)cols.size();
        if (c > max_col) max_col = c;
    }
    const int64_t rows = (int64_t)row_ptr.size() - 1;
    std::vector<int64_t> grouping(rows), perm(rows);
    int64_t stats[4];
    if (smat_reorder_rows(rows, max_col + 1, row_ptr.data(), cols.data(), cb, rb, tau, grouping.data(), perm.data(),
                          stats) != SMAT_OK) {
        fprintf(stderr, "reorder failed: %s\n", smat_last_error());
        return 1;
    }
    {
        std::ofstream s(out);
        s << "matrix,rows,cols,nonzeros,blocking_algo,tau,row_block_size,col_block_size,VBR_nzblocks_count,"
             "VBR_longest_row,merge_counter,comparison_counter,\n";
        s << file << "," << rows << "," << max_col + 1 << "," << cols.size() << "," << algo << "," << tau << "," << rb
          << "," << cb << "," << stats[2] << "," << stats[3] << "," << stats[1] << "," << stats[0] << ",\n";
        std::ofstream g(out + ".g");
        g << "GROUPING,";
        for (int64_t v : grouping) g << v << ",";
        g << "\n";
    }
    const size_t dot = file.find_last_of('.');
    std::ofstream el(file.substr(0, dot) + "_reordered.el");
    for (int64_t nr = 0; nr < rows; nr++)
        for (int64_t k = row_ptr[perm[nr]]; k < row_ptr[perm[nr] + 1]; k++) el << nr << " " << cols[k] << "\n";
    if (f.num("v", 1) > 0) printf("Nonzero Blocks:%lld\n", (long long)stats[2]);
    return 0;
}
