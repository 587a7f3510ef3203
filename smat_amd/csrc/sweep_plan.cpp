// Builds the op streams of the sweep kernel.  Layout of an op: spmm_kernels.h (SweepOp).
#include "sweep_plan.h"

#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <queue>
#include <utility>

#include <stdexcept>

#include "../../include/smat.h"
#include "errors.h"
#include "sweep_format.h"

namespace smat {

namespace {
constexpr int G = SWEEP_G, RW = SWEEP_RW, WAVES = SWEEP_WAVES, S = SWEEP_S, MIN_OPS = SWEEP_MIN_OPS;
constexpr int AHEAD = SWEEP_AHEAD, COPIES = SWEEP_COPIES;
constexpr int VM_MARK = MIN_OPS; // a chunk boundary waits until at most this many vector memory operations are under way
} // namespace

void build_sweep_plan(const int32_t *row_ptr, const int32_t *col_idx, size_t mb, size_t kb, SweepPlanHost &out,
                      const int32_t *rows, size_t n_rows)
{
    if (!rows) n_rows = mb;
    const size_t n_rg = (n_rows + G - 1) / G;
    // Row groups: G block rows of the list each, in list order - unless that leaves one group with far more blocks
    // than the average.  A workgroup multiplies one row group under several panels, so the launch takes as long as
    // the heaviest group; then the rows are dealt out instead: in descending block count, each to the group with the
    // fewest blocks so far that still has room (the group sizes stay what they were).  Which rows share a group
    // matters for nothing else: the rows of C are found through row_map, and a matrix dense enough for this kernel
    // touches every K chunk from any 64 of its rows.
    std::vector<int32_t> order;
    {
        std::vector<int64_t> blocks_of(n_rg, 0);
        int64_t total = 0, heaviest = 0;
        for (size_t i = 0; i < n_rows; i++) {
            const size_t br = rows ? (size_t)rows[i] : i;
            blocks_of[i / G] += row_ptr[br + 1] - row_ptr[br];
        }
        for (size_t rg = 0; rg < n_rg; rg++) total += blocks_of[rg], heaviest = std::max(heaviest, blocks_of[rg]);
        if (n_rg > 1 && (double)heaviest * (double)n_rows > 1.08 * (double)total * (double)G) {
            std::vector<int32_t> by_count(n_rows);
            for (size_t i = 0; i < n_rows; i++) by_count[i] = rows ? rows[i] : (int32_t)i;
            std::stable_sort(by_count.begin(), by_count.end(), [&](int32_t x, int32_t y) {
                return row_ptr[x + 1] - row_ptr[x] > row_ptr[y + 1] - row_ptr[y];
            });
            std::vector<std::vector<int32_t>> members(n_rg);
            typedef std::pair<int64_t, size_t> Load; // blocks so far, row group
            std::priority_queue<Load, std::vector<Load>, std::greater<Load>> lightest;
            for (size_t rg = 0; rg < n_rg; rg++) lightest.push(Load(0, rg));
            for (int32_t br : by_count) {
                const Load l = lightest.top();
                lightest.pop();
                const size_t rg = l.second;
                members[rg].push_back(br);
                if (members[rg].size() < std::min(n_rows, (rg + 1) * G) - rg * G)
                    lightest.push(Load(l.first + (row_ptr[br + 1] - row_ptr[br]), rg));
            }
            order.reserve(n_rows);
            for (size_t rg = 0; rg < n_rg; rg++) {
                std::sort(members[rg].begin(), members[rg].end());
                order.insert(order.end(), members[rg].begin(), members[rg].end());
            }
        }
    }
    auto row_at = [&](size_t i) { return !order.empty() ? (size_t)order[i] : rows ? (size_t)rows[i] : i; }; // i-th block row of the plan
    const size_t n_kchunks = (kb + S - 1) / S;
    const int32_t nnzb = row_ptr[mb];
    out = SweepPlanHost();
    out.rg_chunk_ptr.assign(n_rg + 1, 0);
    out.op_ptr.reserve(n_rg * WAVES + 1);
    out.row_map.assign(n_rg * G, -1);
    std::vector<int32_t> local(n_kchunks, -1); // K chunk -> position in the row group's chunk list
    struct RowOp { int32_t first, last, hi; SweepOpHost op; }; // the periods it may run in, its later chunk
    std::vector<RowOp> row_ops[G];
    struct Ranked { int rank; int row; int32_t hi; SweepOpHost op; };
    std::vector<std::vector<Ranked>> by_chunk;
    for (size_t rg = 0; rg < n_rg; rg++) {
        const size_t r_begin = rg * G, r_end = std::min(n_rows, (rg + 1) * G);
        // the chunks this row group touches, ascending
        const size_t first_chunk = out.chunk_ids.size();
        for (size_t i = r_begin; i < r_end; i++)
            for (int32_t q = row_ptr[row_at(i)]; q < row_ptr[row_at(i) + 1]; q++) local[(size_t)(col_idx[q] / 16) / S] = 0;
        for (size_t c = 0; c < n_kchunks; c++)
            if (local[c] == 0) {
                local[c] = (int32_t)(out.chunk_ids.size() - first_chunk);
                out.chunk_ids.push_back((int32_t)c);
            }
        const size_t n_chunks = out.chunk_ids.size() - first_chunk;
        out.rg_chunk_ptr[rg + 1] = (int32_t)out.chunk_ids.size();

        // ---- ops of every block row: neighbouring blocks in pairs; w3 gets the local row later ----
        for (int lr = 0; lr < G; lr++) {
            row_ops[lr].clear();
            if (r_begin + (size_t)lr >= r_end) continue;
            const size_t br = row_at(r_begin + (size_t)lr);
            int32_t q = row_ptr[br];
            const int32_t q_end = row_ptr[br + 1];
            while (q < q_end) {
                const int32_t bc0 = col_idx[q] / 16;
                const int32_t cl0 = local[(size_t)bc0 / S];
                const uint32_t off0 = sweep_lds_offset(cl0, bc0 % S);
                SweepOpHost op{0, off0, 0, 0};
                int32_t cl_hi = cl0;
                bool pair = false;
                if (q + 1 < q_end) {
                    const int32_t bc1 = col_idx[q + 1] / 16;
                    const int32_t cl1 = local[(size_t)bc1 / S];
                    if (cl1 - cl0 <= 2) { // three consecutive listed chunks are resident while the middle one is swept
                        op.w0 = (uint32_t)q * 512u;
                        op.w2 = sweep_lds_offset(cl1, bc1 % S) - off0;
                        cl_hi = cl1;
                        pair = true;
                    }
                }
                if (!pair) {
                    // The other half of the MFMA reads zeros instead of rows of B, but the load brings two
                    // neighbouring blocks: take the neighbour from the SAME block row where the row has one, so that
                    // an Inf or NaN in another row's values (times zero: NaN) cannot reach this row of C.
                    if (q + 1 < q_end) { // blocks (q, q + 1), the second multiplies zeros
                        op.w0 = (uint32_t)q * 512u;
                        op.w2 = SWEEP_ZERO_OFF - off0;
                    } else if (q > row_ptr[br]) { // last block of its row: blocks (q - 1, q), the first multiplies zeros
                        op.w0 = (uint32_t)(q - 1) * 512u;
                        op.w1 = SWEEP_ZERO_OFF;
                        op.w2 = off0 - SWEEP_ZERO_OFF;
                    } else if (q + 1 < nnzb) { // the only block of its row: the neighbour is another row's
                        op.w0 = (uint32_t)q * 512u;
                        op.w2 = SWEEP_ZERO_OFF - off0;
                    } else { // and the last block of the matrix: the read stays inside vals
                        op.w0 = (uint32_t)(q - 1) * 512u;
                        op.w1 = SWEEP_ZERO_OFF;
                        op.w2 = off0 - SWEEP_ZERO_OFF;
                    }
                }
                // While chunk p is swept, chunks p - 1, p and p + 1 are in LDS: the op may run in any period p with
                // p - 1 <= cl0 and cl_hi <= p + 1.
                const int32_t first = std::max(cl_hi - 1, 0), last = std::min<int32_t>(cl0 + 1, (int32_t)n_chunks - 1);
                (pair ? out.n_pairs : out.n_singles)++;
                row_ops[lr].push_back(RowOp{first, last, cl_hi, op});
                q += pair ? 2 : 1;
            }
        }

        // ---- block rows -> wavefronts, and which period every op runs in.  All wavefronts meet at a barrier once per
        // period, so a period costs the op count of its busiest wavefront, and an op may run in any period of its
        // window [first, last] (at most three periods).  For a given row assignment the cheapest common caps c_p
        // (every wavefront runs at most c_p ops in period p) are found by going through the periods once: a wavefront
        // that runs its pending ops earliest deadline first, as many as the caps allow, is left at period p with the
        // ops that HAVE to run now, and c_p is the largest such count over the wavefronts (capacity is added as late
        // as possible, where it serves the most windows; with unit jobs and interval windows no other caps have a
        // smaller sum).  Pending ops of a wavefront are three counters (deadline p, p + 1, p + 2), so the sum of the
        // caps of an assignment costs O(periods x wavefronts).  The assignment: rows in descending op count to the
        // wavefront with the fewest ops so far, then swaps of two rows between wavefronts while the sum of the caps
        // falls (deterministic, bounded work per row group). ----
        int wave_of[G];
        for (int lr = 0; lr < G; lr++) wave_of[lr] = lr / RW;
        std::vector<int32_t> caps(n_chunks, MIN_OPS);
        if (n_chunks > 0) {
            const size_t n = n_chunks;
            {
                int order[G], n_rows_of[WAVES] = {0};
                long total_of[WAVES] = {0};
                for (int lr = 0; lr < G; lr++) order[lr] = lr;
                std::stable_sort(order, order + G, [&](int x, int y) { return row_ops[x].size() > row_ops[y].size(); });
                for (int k = 0; k < G; k++) {
                    int best = -1;
                    for (int w = 0; w < WAVES; w++)
                        if (n_rows_of[w] < RW && (best < 0 || total_of[w] < total_of[best])) best = w;
                    wave_of[order[k]] = best;
                    n_rows_of[best]++;
                    total_of[best] += (long)row_ops[order[k]].size();
                }
            }
            std::vector<int32_t> win((size_t)WAVES * n * 3, 0); // ops of wavefront w with window [first, first + len]: win[(w * n + first) * 3 + len]
            auto add_row = [&](int lr, int w, int32_t sign) {
                for (const RowOp &ro : row_ops[lr]) win[((size_t)w * n + (size_t)ro.first) * 3 + (size_t)(ro.last - ro.first)] += sign;
            };
            for (int lr = 0; lr < G; lr++) add_row(lr, wave_of[lr], 1);
            auto sum_of_caps = [&](std::vector<int32_t> *caps_out) {
                long sum = 0;
                int32_t pend[WAVES][3] = {{0}};
                for (size_t p = 0; p < n; p++) {
                    int32_t cap = MIN_OPS;
                    for (int w = 0; w < WAVES; w++) {
                        const int32_t *c = &win[((size_t)w * n + p) * 3];
                        pend[w][0] += c[0]; pend[w][1] += c[1]; pend[w][2] += c[2];
                        cap = std::max(cap, pend[w][0]);
                    }
                    for (int w = 0; w < WAVES; w++) {
                        // the ops due now run; what is left of the cap goes to the next deadlines, but the last pending op
                        // stays for the next period when it may (see the schedule below)
                        int32_t room = cap - pend[w][0];
                        if (p + 1 < n && room >= pend[w][1] + pend[w][2] && pend[w][1] + pend[w][2] > 0) room = pend[w][1] + pend[w][2] - 1;
                        const int32_t r1 = std::min(room, pend[w][1]);
                        room -= r1;
                        const int32_t r2 = std::min(room, pend[w][2]);
                        pend[w][0] = pend[w][1] - r1;
                        pend[w][1] = pend[w][2] - r2;
                        pend[w][2] = 0;
                    }
                    sum += cap;
                    if (caps_out) (*caps_out)[p] = cap;
                }
                return sum;
            };
            long best = sum_of_caps(nullptr);
            // work bound: about 2e8 counter updates per plan, shared evenly by the row groups
            long budget = (long)(2e8 / (double)(n * WAVES * 3) / (double)n_rg);
            for (int pass = 0; pass < 4 && budget > 0; pass++) {
                bool improved = false;
                for (int i = 0; i < G && budget > 0; i++)
                    for (int j = i + 1; j < G && budget > 0; j++) {
                        const int wi = wave_of[i], wj = wave_of[j];
                        if (wi == wj || (row_ops[i].empty() && row_ops[j].empty())) continue;
                        add_row(i, wi, -1); add_row(i, wj, 1); add_row(j, wj, -1); add_row(j, wi, 1);
                        const long now = sum_of_caps(nullptr);
                        budget--;
                        if (now < best) {
                            best = now;
                            std::swap(wave_of[i], wave_of[j]);
                            improved = true;
                        } else {
                            add_row(i, wj, -1); add_row(i, wi, 1); add_row(j, wi, -1); add_row(j, wj, 1);
                        }
                    }
                if (!improved) break;
            }
            sum_of_caps(&caps);
        }

        struct Pending { int32_t last, first, seq, row, hi; SweepOpHost op; };
        std::vector<std::vector<std::vector<Ranked>>> schedule((size_t)WAVES, std::vector<std::vector<Ranked>>(n_chunks));
        if (n_chunks > 0) {
            for (int w = 0; w < WAVES; w++) {
                std::vector<Pending> todo;
                int r = 0;
                for (int lr = 0; lr < G; lr++) {
                    if (wave_of[lr] != w) continue;
                    if (r_begin + (size_t)lr < r_end) out.row_map[(rg * WAVES + (size_t)w) * RW + (size_t)r] = (int32_t)row_at(r_begin + (size_t)lr);
                    for (const RowOp &ro : row_ops[lr]) todo.push_back(Pending{ro.last, ro.first, (int32_t)todo.size(), r, ro.hi, ro.op});
                    r++;
                }
                std::stable_sort(todo.begin(), todo.end(), [](const Pending &a, const Pending &b) { return a.first < b.first; });
                std::vector<Pending> ready;
                size_t next = 0;
                for (size_t c = 0; c < n_chunks; c++) {
                    while (next < todo.size() && todo[next].first <= (int32_t)c) ready.push_back(todo[next++]);
                    std::stable_sort(ready.begin(), ready.end(), [](const Pending &a, const Pending &b) {
                        if (a.last != b.last) return a.last < b.last;
                        return a.seq < b.seq;
                    });
                    // Up to the cap, earliest deadline first.  The op that opens the next period has to be one that is
                    // ready now (its LDS reads are issued before the boundary's barrier, so its chunks must be resident
                    // already): a wavefront that could run everything it has keeps its last op for that.
                    size_t musts = 0;
                    while (musts < ready.size() && ready[musts].last <= (int32_t)c) musts++;
                    size_t k = std::min(ready.size(), (size_t)caps[c]);
                    if (k == ready.size() && k > musts && c + 1 < n_chunks) k--;
                    k = std::max(k, musts);
                    std::vector<Ranked> &list = schedule[(size_t)w][c];
                    for (size_t x = 0; x < k; x++) {
                        const Pending &pe = ready[x];
                        // rank = how many ops of this block row the period already holds: ops of one block
                        // row (same accumulators) end up spread over the period
                        int rank = 0;
                        for (const Ranked &y : list) rank += y.row == pe.row;
                        list.push_back(Ranked{rank, pe.row, pe.hi, pe.op});
                    }
                    ready.erase(ready.begin(), ready.begin() + (long)k);
                    if (!ready.empty() && ready.front().last <= (int32_t)c) throw std::logic_error("sweep plan: an op missed its last period");
                }
                if (!ready.empty() || next != todo.size()) throw std::logic_error("sweep plan: ops left over by the period schedule");
            }
        }

        // ---- streams: ops of chunk 0, ops of chunk 1, ..., end; the first op of a chunk carries the chunk boundary ----
        for (int w = 0; w < WAVES; w++) {
            out.op_ptr.push_back((int32_t)out.ops.size());
            if (n_chunks == 0) continue; // the kernel does not enter the interpreter for an empty row group
            by_chunk = schedule[(size_t)w];
            struct Item { int kind, row; bool opens; SweepOpHost op; }; // kind: 0 op, 2 end; opens: first op of a chunk but the first
            std::vector<Item> items;
            const SweepOpHost idle{0, SWEEP_ZERO_OFF, 0, 0}; // the end: no blocks of its own
            // A filler op multiplies two blocks by zeros and adds the result to one of the wavefront's block rows:
            // two blocks of that very row (then an Inf or NaN in them is in that row of C anyway), blocks 0 and 1
            // of the matrix only when no row of the wavefront has two.
            Item filler{0, 0, false, idle};
            for (int r = 0; r < RW; r++) {
                const int32_t br = out.row_map[(rg * WAVES + (size_t)w) * RW + (size_t)r];
                if (br >= 0 && row_ptr[br + 1] - row_ptr[br] >= 2) {
                    filler.row = r;
                    filler.op.w0 = (uint32_t)row_ptr[br] * 512u;
                    break;
                }
            }
            for (size_t c = 0; c < n_chunks; c++) {
                std::vector<Ranked> &list = by_chunk[c];
                std::stable_sort(list.begin(), list.end(), [](const Ranked &a, const Ranked &b) {
                    if (a.rank != b.rank) return a.rank < b.rank;
                    return a.row < b.row;
                });
                const size_t first_of_chunk = items.size();
                size_t n_here = list.size();
                if (c > 0) {
                    // The LDS reads of the op that opens a chunk are issued by the op before it, before the barrier of
                    // the boundary, when the copies of chunk c + 1 may still be under way: it has to be an op whose
                    // chunks are c or c - 1.
                    size_t ok = 0;
                    while (ok < list.size() && list[ok].hi > (int32_t)c) ok++;
                    if (ok == list.size()) {
                        items.push_back(filler);
                        out.n_fillers++;
                        n_here++;
                    } else if (ok > 0) {
                        std::rotate(list.begin(), list.begin() + (long)ok, list.begin() + (long)ok + 1);
                    }
                }
                for (const Ranked &x : list) items.push_back(Item{0, x.row, false, x.op});
                for (size_t k = n_here; k < (size_t)MIN_OPS; k++) { // filler ops keep the chunk boundaries AHEAD positions apart
                    items.push_back(filler);
                    out.n_fillers++;
                }
                if (c > 0) items[first_of_chunk].opens = true;
            }
            items.push_back(Item{2, 0, false, idle});
            // Which s_waitcnt vmcnt an op needs: vector memory operations complete in order, every position issues
            // one A load (for the op AHEAD positions later), the op that opens a chunk issues the copies of the
            // boundary before that load.
            std::vector<long> a_issue(items.size() + (size_t)AHEAD + 1, 0), copy_seq(n_chunks + 3, 0);
            long seq = 0;
            for (int k = 0; k < AHEAD; k++) a_issue[(size_t)k] = ++seq; // entry code, after the copies of chunks 0..2
            size_t cur = 0;
            for (size_t i = 0; i < items.size(); i++) {
                Item &it = items[i];
                if (it.kind == 2) {
                    it.op.w3 = SWEEP_END_OFF;
                    break;
                }
                if (it.opens) {
                    cur++;
                    // the copies of chunk cur + 1 were issued by the boundary before this one (or by the entry code): the
                    // boundary waits until at most VM_MARK younger operations are under way
                    if (cur + 1 < n_chunks && seq - copy_seq[cur + 1] < VM_MARK) throw std::logic_error("sweep plan: a chunk boundary would not wait for its copies");
                    if (cur + 2 < n_chunks) {
                        seq += COPIES;
                        copy_seq[cur + 2] = seq;
                    }
                }
                a_issue[i + (size_t)AHEAD] = ++seq;
                const long younger = seq - a_issue[i];
                if (younger != AHEAD && younger != AHEAD + COPIES) throw std::logic_error("sweep plan: chunk boundaries closer than the A read-ahead");
                const int v = younger == AHEAD ? 0 : 1;
                it.op.w3 = it.opens ? sweep_boundary_op_code((int)i, it.row, v) : sweep_op_code((int)i, it.row, v);
            }
            if (cur + 1 != n_chunks) throw std::logic_error("sweep plan: a stream does not pass every chunk boundary");
            for (const Item &it : items) out.ops.push_back(it.op);
        }
        for (size_t c = first_chunk; c < out.chunk_ids.size(); c++) local[(size_t)out.chunk_ids[c]] = -1;
    }
    out.op_ptr.push_back((int32_t)out.ops.size());
    // what the kernel reads ahead of the last op: fetched, never executed
    out.ops.resize(out.ops.size() + SWEEP_OP_PAD, SweepOpHost{0, SWEEP_ZERO_OFF, 0, SWEEP_END_OFF});
    out.chunk_ids.resize(out.chunk_ids.size() + SWEEP_CHUNK_PAD, 0);
}

} // namespace smat

// Test hook (not part of smat.h): builds the work list on the host (rows != NULL: of these block rows only) and hands it out.  Arrays are
// allocated with malloc; release each with smat_host_free.  row_map: n_rg * 64 block rows (-1 = none).  counts[0..5] = row groups, listed
// chunks, stream entries (ops, fillers, ends; without padding), pairs, singles, fillers.
static int smat_internal_sweep_plan_impl(const int32_t *row_ptr, const int32_t *col_idx, size_t M, size_t K,
                                         const int32_t *rows, size_t n_rows, int32_t **rg_chunk_ptr, int32_t **chunk_ids, int32_t **op_ptr,
                                         uint32_t **ops, int32_t **row_map, int64_t *counts)
{
    if (!row_ptr || !col_idx || !rg_chunk_ptr || !chunk_ids || !op_ptr || !ops || !row_map || !counts) return SMAT_ERR_INVALID;
    if (M == 0 || M % 16 || K % 16 || row_ptr[M / 16] < 2) return SMAT_ERR_INVALID;
    smat::SweepPlanHost p;
    try {
        smat::build_sweep_plan(row_ptr, col_idx, M / 16, K / 16, p, rows, n_rows);
    } catch (...) {
        return SMAT_ERR_NOMEM;
    }
    auto dup = [](const void *src, size_t bytes) -> void * {
        void *d = malloc(bytes ? bytes : 1);
        if (d && bytes) memcpy(d, src, bytes);
        return d;
    };
    *rg_chunk_ptr = (int32_t *)dup(p.rg_chunk_ptr.data(), p.rg_chunk_ptr.size() * 4);
    *chunk_ids = (int32_t *)dup(p.chunk_ids.data(), p.chunk_ids.size() * 4);
    *op_ptr = (int32_t *)dup(p.op_ptr.data(), p.op_ptr.size() * 4);
    *ops = (uint32_t *)dup(p.ops.data(), p.ops.size() * 16);
    *row_map = (int32_t *)dup(p.row_map.data(), p.row_map.size() * 4);
    if (!*rg_chunk_ptr || !*chunk_ids || !*op_ptr || !*ops || !*row_map) return SMAT_ERR_NOMEM;
    counts[0] = (int64_t)p.rg_chunk_ptr.size() - 1;
    counts[1] = (int64_t)p.chunk_ids.size() - smat::SWEEP_CHUNK_PAD;
    counts[2] = (int64_t)p.ops.size() - smat::SWEEP_OP_PAD;
    counts[3] = (int64_t)p.n_pairs;
    counts[4] = (int64_t)p.n_singles;
    counts[5] = (int64_t)p.n_fillers;
    return SMAT_OK;
}

// Test hook: the pipeline depths this build was compiled with {A read-ahead, LDS read-ahead, minimum ops per chunk, copies per chunk boundary}.
extern "C" void smat_internal_sweep_params(int32_t *out)
{
    out[0] = smat::SWEEP_AHEAD; out[1] = smat::SWEEP_LDS_AHEAD; out[2] = smat::SWEEP_MIN_OPS; out[3] = smat::SWEEP_COPIES;
}

extern "C" int smat_internal_sweep_plan(const int32_t *row_ptr, const int32_t *col_idx, size_t M, size_t K,
                                         const int32_t *rows, size_t n_rows, int32_t **rg_chunk_ptr, int32_t **chunk_ids, int32_t **op_ptr,
                                         uint32_t **ops, int32_t **row_map, int64_t *counts)
{
    return smat::guarded("smat_internal_sweep_plan", [&] { return smat_internal_sweep_plan_impl(row_ptr, col_idx, M, K, rows, n_rows, rg_chunk_ptr, chunk_ids, op_ptr, ops, row_map, counts); });
}
