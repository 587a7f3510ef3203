// CPU row/column reordering that clusters rows with similar block-column
// patterns so that fewer 16x16 blocks are nonzero.  This is the reference
// algorithm (it must produce the same grouping and permutation bit for bit),
// restated over block-column patterns instead of raw column lists:
//
//   BlockingEngine::GetGrouping      preprocess/src/general/blocking.cpp:616-657
//   IterativeBlockingKeeper (-a 5)   preprocess/src/general/blocking.cpp:431-547
//   JaccardDistanceGroup             preprocess/src/general/blocking.cpp:904-975
//   merge_rows                       preprocess/src/general/utilities.cpp:145-173
//   get_permutation / get_fixed_size_grouping   utilities.cpp:8-20, 45-54
//   CollectBlockingInfo              preprocess/src/general/blocking.cpp:562-614
//   CSR::reorder / permute_rows      preprocess/src/general/csr.cpp:65-74, 97-105
//   row pass + column pass via the transpose   src/reorder.py:107-139, 143-182
//
// Behaviours of the reference that are kept on purpose because they decide the
// output:
//   * The per-row distance cache starts as {-1, 0, 0, ...}: only element 0 of
//     `float distances[rows] = {-1}` is -1 (blocking.cpp:434).
//   * merge_rows is not a set union: after merging row B into pattern A the new
//     pattern is B plus those elements of A that are smaller than the largest
//     element of B that does not exceed max(A); larger elements of A are dropped
//     (the tail of A is never copied, utilities.cpp:153-171).
//   * The candidate set is trimmed with `it = end(); advance(it, room);
//     erase(it, end())` (blocking.cpp:505-510).  Stepping forward from end() of a
//     libstdc++ red-black tree walks the cycle end -> [left child of the largest
//     node, if it has one] -> largest -> end, so 0, 1 or 2 of the largest
//     candidates are removed depending on `room` and on the shape of the tree.
//     CandidateTree below is a red-black tree with libstdc++'s insertion and
//     erasure rebalancing, which makes that shape, and therefore the result,
//     reproducible with any standard library.
//   * Rows taken from the candidate set are not merged into the pattern
//     (blocking.cpp:515-523), and the `use_groups` flag is ignored: the current
//     group size always weights the distance (blocking.cpp:477-478).
//   * Ties inside a group are ordered by the (unstable) std::sort of
//     get_permutation; the same call on the same keys is made here.
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <atomic>
#include <chrono>
#include <functional>
#include <numeric>
#include <thread>
#include <utility>
#include <vector>

#include "../../include/smat.h"
#include "errors.h"

namespace smat {
namespace {

// Ordered set of (distance, row) with the node layout decisions of libstdc++'s
// _Rb_tree (insert_and_rebalance / rebalance_for_erase).  Index 0 is "null".
class CandidateTree {
public:
    struct Node { // 24 bytes: the set grows to tens of thousands of rows on power-law matrices
        float dist;
        int32_t row;
        int32_t parent, left, right;
        bool red, alive;
    };

    void clear()
    {
        nodes_.resize(1);
        free_.clear();
        generation_++; // forgets every hint
        hints_used_ = 0;
        root_ = 0;
        rightmost_ = 0;
        leftmost_ = 0;
        size_ = 0;
    }
    size_t size() const { return size_; }

    // Rows come in ascending order, and the distances take few different values (they are ratios of small
    // block counts): the node that was inserted last with the same distance, if it is still in the tree, is the
    // in-order predecessor of the new key, and a key goes below its predecessor (if that has no right child) or
    // below its successor (the leftmost node of that right subtree).  With unique keys a search tree has one
    // place for a key, so this is the place the descent from the root ends at, found without the descent.
    void insert(float dist, int64_t row)
    {
        int32_t y = 0;
        bool less_than = true;
        Hint *hint = hint_for(dist);
        const int32_t h = hint && hint->generation == generation_ ? hint->node : 0;
        if (h && nodes_[h].alive && nodes_[h].dist == dist && nodes_[h].row < row) {
            if (!nodes_[h].right) {
                y = h;
                less_than = false;
            } else {
                y = nodes_[h].right;
                while (nodes_[y].left) y = nodes_[y].left;
            }
        } else {
            int32_t x = root_;
            while (x) {
                y = x;
                less_than = key_less(dist, row, nodes_[x]);
                x = less_than ? nodes_[x].left : nodes_[x].right;
            }
        }
        int32_t z;
        if (!free_.empty()) { // which slot a node lives in does not show in the shape of the tree
            z = free_.back();
            free_.pop_back();
            nodes_[z] = Node{dist, (int32_t)row, y, 0, 0, true, true};
        } else {
            nodes_.push_back(Node{dist, (int32_t)row, y, 0, 0, true, true});
            z = (int32_t)nodes_.size() - 1;
        }
        if (hint) {
            if (hint->generation != generation_) hints_used_++;
            *hint = Hint{dist, z, generation_};
        }
        if (!y) {
            root_ = leftmost_ = rightmost_ = z;
        } else if (less_than) {
            nodes_[y].left = z;
            if (y == leftmost_) leftmost_ = z;
        } else {
            nodes_[y].right = z;
            if (y == rightmost_) rightmost_ = z;
        }
        ++size_;
        insert_fixup(z);
    }

    // True if insert(dist, row) followed by trim_from_end(steps) with an odd `steps` would leave the tree as it is:
    // a key above the largest one becomes the right child of the largest node; under a black parent nothing is
    // rebalanced; the new node, a red leaf without a left child, is then the only one the trim removes (cycle of
    // two, odd step count), and removing a red leaf rebalances nothing either.
    bool insert_then_trim_is_noop(float dist, int64_t row) const
    {
        return rightmost_ && !nodes_[rightmost_].red && !key_less(dist, row, nodes_[rightmost_]);
    }

    // Emulates `it = end(); advance(it, steps); erase(it, end());`.
    void trim_from_end(size_t steps)
    {
        if (!size_) return;
        const int32_t pred = nodes_[rightmost_].left; // a red leaf, or null
        const size_t cycle = pred ? 3 : 2;
        const size_t pos = steps % cycle;
        if (pos == 0) return; // back at end(): nothing erased
        if (pred && pos == 1) {
            erase(pred);
            erase(rightmost_);
        } else {
            erase(rightmost_);
        }
    }

    template <class F> void for_each_ascending(F f) const
    {
        for (int32_t x = leftmost_; x; x = successor(x))
            if (!f(nodes_[x])) break;
    }

private:
    static bool key_less(float d, int64_t r, const Node &n)
    {
        return d < n.dist || (!(n.dist < d) && r < n.row); // std::pair ordering
    }
    int32_t successor(int32_t x) const
    {
        if (nodes_[x].right) {
            x = nodes_[x].right;
            while (nodes_[x].left) x = nodes_[x].left;
            return x;
        }
        int32_t y = nodes_[x].parent;
        while (y && x == nodes_[y].right) { x = y; y = nodes_[y].parent; }
        return y;
    }
    void rotate_left(int32_t x)
    {
        const int32_t y = nodes_[x].right;
        nodes_[x].right = nodes_[y].left;
        if (nodes_[y].left) nodes_[nodes_[y].left].parent = x;
        nodes_[y].parent = nodes_[x].parent;
        if (x == root_) root_ = y;
        else if (x == nodes_[nodes_[x].parent].left) nodes_[nodes_[x].parent].left = y;
        else nodes_[nodes_[x].parent].right = y;
        nodes_[y].left = x;
        nodes_[x].parent = y;
    }
    void rotate_right(int32_t x)
    {
        const int32_t y = nodes_[x].left;
        nodes_[x].left = nodes_[y].right;
        if (nodes_[y].right) nodes_[nodes_[y].right].parent = x;
        nodes_[y].parent = nodes_[x].parent;
        if (x == root_) root_ = y;
        else if (x == nodes_[nodes_[x].parent].right) nodes_[nodes_[x].parent].right = y;
        else nodes_[nodes_[x].parent].left = y;
        nodes_[y].right = x;
        nodes_[x].parent = y;
    }
    bool is_red(int32_t x) const { return x && nodes_[x].red; }

    void insert_fixup(int32_t x)
    {
        while (x != root_ && nodes_[nodes_[x].parent].red) {
            int32_t p = nodes_[x].parent, g = nodes_[p].parent;
            if (p == nodes_[g].left) {
                const int32_t u = nodes_[g].right;
                if (is_red(u)) {
                    nodes_[p].red = false; nodes_[u].red = false; nodes_[g].red = true;
                    x = g;
                } else {
                    if (x == nodes_[p].right) { x = p; rotate_left(x); }
                    p = nodes_[x].parent; g = nodes_[p].parent;
                    nodes_[p].red = false; nodes_[g].red = true;
                    rotate_right(g);
                }
            } else {
                const int32_t u = nodes_[g].left;
                if (is_red(u)) {
                    nodes_[p].red = false; nodes_[u].red = false; nodes_[g].red = true;
                    x = g;
                } else {
                    if (x == nodes_[p].left) { x = p; rotate_right(x); }
                    p = nodes_[x].parent; g = nodes_[p].parent;
                    nodes_[p].red = false; nodes_[g].red = true;
                    rotate_left(g);
                }
            }
        }
        nodes_[root_].red = false;
    }

    void erase(int32_t z)
    {
        int32_t y = z, x = 0, x_parent = 0;
        if (!nodes_[y].left) x = nodes_[y].right;
        else if (!nodes_[y].right) x = nodes_[y].left;
        else {
            y = nodes_[y].right;
            while (nodes_[y].left) y = nodes_[y].left;
            x = nodes_[y].right;
        }
        if (y != z) { // put the successor y where z was
            nodes_[nodes_[z].left].parent = y;
            nodes_[y].left = nodes_[z].left;
            if (y != nodes_[z].right) {
                x_parent = nodes_[y].parent;
                if (x) nodes_[x].parent = nodes_[y].parent;
                nodes_[nodes_[y].parent].left = x;
                nodes_[y].right = nodes_[z].right;
                nodes_[nodes_[z].right].parent = y;
            } else {
                x_parent = y;
            }
            if (root_ == z) root_ = y;
            else if (nodes_[nodes_[z].parent].left == z) nodes_[nodes_[z].parent].left = y;
            else nodes_[nodes_[z].parent].right = y;
            nodes_[y].parent = nodes_[z].parent;
            std::swap(nodes_[y].red, nodes_[z].red);
            y = z;
        } else {
            x_parent = nodes_[y].parent;
            if (x) nodes_[x].parent = nodes_[y].parent;
            if (root_ == z) root_ = x;
            else if (nodes_[nodes_[z].parent].left == z) nodes_[nodes_[z].parent].left = x;
            else nodes_[nodes_[z].parent].right = x;
            if (leftmost_ == z) {
                if (!nodes_[z].right) leftmost_ = nodes_[z].parent;
                else { int32_t m = x; while (nodes_[m].left) m = nodes_[m].left; leftmost_ = m; }
            }
            if (rightmost_ == z) {
                if (!nodes_[z].left) rightmost_ = nodes_[z].parent;
                else { int32_t m = x; while (nodes_[m].right) m = nodes_[m].right; rightmost_ = m; }
            }
        }
        if (!nodes_[y].red) {
            while (x != root_ && !is_red(x)) {
                if (x == nodes_[x_parent].left) {
                    int32_t w = nodes_[x_parent].right;
                    if (nodes_[w].red) {
                        nodes_[w].red = false; nodes_[x_parent].red = true;
                        rotate_left(x_parent);
                        w = nodes_[x_parent].right;
                    }
                    if (!is_red(nodes_[w].left) && !is_red(nodes_[w].right)) {
                        nodes_[w].red = true;
                        x = x_parent; x_parent = nodes_[x_parent].parent;
                    } else {
                        if (!is_red(nodes_[w].right)) {
                            nodes_[nodes_[w].left].red = false; nodes_[w].red = true;
                            rotate_right(w);
                            w = nodes_[x_parent].right;
                        }
                        nodes_[w].red = nodes_[x_parent].red; nodes_[x_parent].red = false;
                        if (nodes_[w].right) nodes_[nodes_[w].right].red = false;
                        rotate_left(x_parent);
                        break;
                    }
                } else {
                    int32_t w = nodes_[x_parent].left;
                    if (nodes_[w].red) {
                        nodes_[w].red = false; nodes_[x_parent].red = true;
                        rotate_right(x_parent);
                        w = nodes_[x_parent].left;
                    }
                    if (!is_red(nodes_[w].right) && !is_red(nodes_[w].left)) {
                        nodes_[w].red = true;
                        x = x_parent; x_parent = nodes_[x_parent].parent;
                    } else {
                        if (!is_red(nodes_[w].left)) {
                            nodes_[nodes_[w].right].red = false; nodes_[w].red = true;
                            rotate_left(w);
                            w = nodes_[x_parent].left;
                        }
                        nodes_[w].red = nodes_[x_parent].red; nodes_[x_parent].red = false;
                        if (nodes_[w].left) nodes_[nodes_[w].left].red = false;
                        rotate_right(x_parent);
                        break;
                    }
                }
            }
            if (x) nodes_[x].red = false;
        }
        --size_;
        nodes_[z].alive = false;
        free_.push_back(z); // unlinked above (y == z by now): the slot is reused by the next insert
    }

    // distance -> node inserted last with it: open addressing, entries of an older generation are free
    struct Hint {
        float dist;
        int32_t node;
        uint32_t generation;
    };
    static constexpr size_t HINTS = 4096;
    Hint *hint_for(float dist)
    {
        uint32_t bits;
        memcpy(&bits, &dist, 4);
        size_t at = (bits * 2654435761u) >> 20; // 12 bits
        for (size_t probe = 0; probe < 16; probe++, at = (at + 1) & (HINTS - 1)) {
            Hint &e = hints_[at];
            if (e.generation != generation_) return hints_used_ < HINTS / 2 ? &e : nullptr;
            if (e.dist == dist) return &e;
        }
        return nullptr; // crowded: this distance goes without a hint
    }

    std::vector<Node> nodes_{1};
    std::vector<int32_t> free_;
    std::vector<Hint> hints_ = std::vector<Hint>(HINTS, Hint{0.0f, 0, 0});
    uint32_t generation_ = 1;
    size_t hints_used_ = 0;
    int32_t root_ = 0, leftmost_ = 0, rightmost_ = 0;
    size_t size_ = 0;
};

struct Pattern { // per-row sorted unique block columns (col / col_block)
    std::vector<int64_t> ptr;
    std::vector<int32_t> blk;
};

Pattern build_block_patterns(int64_t rows, const int64_t *row_ptr, const int64_t *col_idx,
                             int64_t col_block)
{
    Pattern p;
    p.ptr.resize(rows + 1);
    p.blk.reserve((size_t)row_ptr[rows]);
    for (int64_t r = 0; r < rows; r++) {
        p.ptr[r] = (int64_t)p.blk.size();
        int64_t last = -1;
        for (int64_t k = row_ptr[r]; k < row_ptr[r + 1]; k++) {
            const int64_t b = col_idx[k] / col_block;
            if (b != last) { p.blk.push_back((int32_t)b); last = b; }
        }
    }
    p.ptr[rows] = (int64_t)p.blk.size();
    return p;
}

// get_permutation (utilities.cpp:8-20): unstable sort of row ids by group id,
// comparator arguments narrowed to int exactly as in the reference.
std::vector<int64_t> permutation_by_group(const std::vector<int64_t> &grouping)
{
    auto comp = [&](int i, int j) { return grouping[i] < grouping[j]; };
    std::vector<int64_t> v(grouping.size());
    std::iota(v.begin(), v.end(), 0);
    std::sort(v.begin(), v.end(), comp);
    return v;
}

// Helper threads for the row scan of keeper_grouping.  A job is a function of the thread index that every
// thread (the caller as index 0) runs once; run() returns when all have.  Helpers spin between jobs (jobs
// follow each other within microseconds) and yield when none comes for a while.
class ScanPool {
public:
    explicit ScanPool(int n_threads) : n_(std::max(n_threads, 1))
    {
        for (int t = 1; t < n_; t++) helpers_.emplace_back([this, t] { loop(t); });
    }
    ~ScanPool()
    {
        stop_.store(true, std::memory_order_release);
        generation_.fetch_add(1, std::memory_order_release);
        for (std::thread &h : helpers_) h.join();
    }
    int size() const { return n_; }
    // All threads, the caller included, run the job; returns when every one has.
    void run(const std::function<void(int)> &job)
    {
        if (n_ == 1) { job(0); return; }
        start(job);
        job(0);
        wait();
    }
    // The helpers run the job while the caller does something else; wait() before the next start() or run().
    void start(const std::function<void(int)> &job)
    {
        if (n_ == 1) return;
        job_ = &job;
        pending_.store(n_ - 1, std::memory_order_relaxed);
        generation_.fetch_add(1, std::memory_order_release);
    }
    void wait()
    {
        while (pending_.load(std::memory_order_acquire)) spin_pause();
    }

private:
    static void spin_pause()
    {
#if defined(__x86_64__) || defined(__i386__)
        __builtin_ia32_pause();
#endif
    }
    void loop(int t)
    {
        uint64_t seen = 0;
        for (;;) {
            int idle = 0;
            while (generation_.load(std::memory_order_acquire) == seen) {
                // short gaps between jobs are spun through; in the long serial phases of a run the helpers
                // give the core away and finally sleep, 50 us at a time
                if (++idle < 4096) spin_pause();
                else if (idle < 65536) std::this_thread::yield();
                else std::this_thread::sleep_for(std::chrono::microseconds(50));
            }
            seen = generation_.load(std::memory_order_acquire);
            if (stop_.load(std::memory_order_acquire)) return;
            (*job_)(t);
            pending_.fetch_sub(1, std::memory_order_release);
        }
    }
    const int n_;
    std::vector<std::thread> helpers_;
    const std::function<void(int)> *job_ = nullptr;
    std::atomic<uint64_t> generation_{0};
    std::atomic<int> pending_{0};
    std::atomic<bool> stop_{false};
};

// Threads for the scan: SMAT_REORDER_THREADS, else the hardware's count, at most 16.
int scan_threads()
{
    if (const char *e = getenv("SMAT_REORDER_THREADS")) {
        const int n = atoi(e);
        if (n >= 1) return std::min(n, 256);
    }
    const unsigned hw = std::thread::hardware_concurrency();
    return (int)std::min(std::max(hw, 1u), 16u);
}

// What looking at a row needs, by value: the helper threads take a copy per job, so that they read nothing that
// the scanning thread writes while it applies results (its locals share cache lines with these fields otherwise).
struct RowView {
    static constexpr float PRUNED = -1.0f, TAKEN = -2.0f; // marks next to the distances (which are >= 0)
    const int64_t *row_ptr, *pat_ptr, *stamp, *grouping;
    const int32_t *pat_blk;
    const float *dist_cache;
    int64_t seed, pattern_blocks, group_size;
    float seed_cached, tau;
    bool pattern_empty;

    // what the reference does with row j before it touches any state: skipped by the cached distances,
    // already in a group, or compared with the pattern
    float look(int64_t j) const
    {
        if (seed_cached != -1 && dist_cache[j] != -1 && std::fabs(seed_cached - dist_cache[j]) > tau) return PRUNED;
        if (grouping[j] != -1) return TAKEN;
        const int64_t nb = pat_ptr[j + 1] - pat_ptr[j];
        const bool b_empty = row_ptr[j + 1] == row_ptr[j];
        if (pattern_empty && b_empty) return 0.0f;
        if (pattern_empty || b_empty) return 1.0f;
        int64_t common = 0;
        for (int64_t k = pat_ptr[j]; k < pat_ptr[j + 1]; k++) common += stamp[pat_blk[k]] == seed;
        const int64_t na = pattern_blocks;
        // count_zeros weighting: blocks only in the group count once, blocks
        // only in the row count group_size times (blocking.cpp:912-917)
        const int64_t count = (na - common) + (nb - common) * group_size;
        return (float)((2.0 * (double)count) / (double)(na * group_size + nb + count));
    }
};

// IterativeBlockingKeeper with use_pattern = 1 and the Jaccard group distance.
//
// The scan over the later rows j of one seed row i is sequential in the reference: the distance of row j is
// taken against the pattern as the merges before j left it.  Here the scan runs in batches.  What happens to
// row j depends on the scan so far only through the pattern and the group size, which change at a merge and
// nowhere else (at most row_block - 1 times per seed): the rows of a batch are therefore evaluated in
// parallel against the current pattern, and their results are applied in row order up to and including the
// first merge; what was evaluated behind it is thrown away and the next batch starts there.  Every write
// (distance cache, grouping, candidate set, counters) happens in that ordered pass, so the output is the one
// of the sequential scan whatever the number of threads.
std::vector<int64_t> keeper_grouping(int64_t rows, const int64_t *row_ptr, const int64_t *col_idx,
                                     const Pattern &pat, int64_t nblk_cols, int64_t col_block,
                                     int64_t max_rows, float tau, int64_t &comparisons,
                                     int64_t &merges)
{
    std::vector<int64_t> grouping((size_t)rows, -1);
    std::vector<float> dist_cache((size_t)rows, 0.0f);
    if (rows > 0) dist_cache[0] = -1.0f;

    std::vector<int64_t> stamp((size_t)nblk_cols + 1, -1); // stamp[b] == seed  <=>  b in pattern
    std::vector<int32_t> pattern, scratch;
    std::vector<int64_t> merged_rows;
    CandidateTree candidates;

    constexpr float TAKEN = RowView::TAKEN;
    // Row by row for SERIAL_ROWS rows behind a change of the pattern, then batches that grow with the distance
    // from it.  The two environment variables exist for the tests, which run small matrices through the batches.
    auto tunable = [](const char *name, int64_t fallback) {
        const char *e = getenv(name);
        const long long v = e ? atoll(e) : 0;
        return v >= 1 ? (int64_t)v : fallback;
    };
    const int64_t SERIAL_ROWS = tunable("SMAT_REORDER_SERIAL_ROWS", 512), FIRST_BATCH = tunable("SMAT_REORDER_FIRST_BATCH", 4096);
    const int64_t MAX_BATCH = std::max<int64_t>(131072, FIRST_BATCH), GRAIN = std::max<int64_t>(1, std::min<int64_t>(512, FIRST_BATCH / 8));
    const int want_threads = rows >= 4 * FIRST_BATCH ? scan_threads() : 1;
    ScanPool pool(want_threads);
    // Three result buffers: one being applied, one being filled for the rows behind it, one whose distances
    // are being copied into the cache.
    std::vector<float> results[3];
    if (pool.size() > 1)
        for (std::vector<float> &r : results) r.resize((size_t)std::min<int64_t>(rows, MAX_BATCH));
    struct Span { int buf; int64_t first, count; };
    std::atomic<int64_t> next_store{0}, next_look{0};

    for (int64_t i = 0; i < rows; i++) {
        if (grouping[i] != -1) continue;
        candidates.clear();
        merged_rows.clear();
        const int64_t group_number = i + rows;
        int64_t group_size = 1;
        grouping[i] = group_number;
        merged_rows.push_back(i);

        pattern.assign(pat.blk.begin() + pat.ptr[i], pat.blk.begin() + pat.ptr[i + 1]);
        for (int32_t b : pattern) stamp[b] = i;
        bool pattern_empty = row_ptr[i + 1] == row_ptr[i];
        int64_t pattern_max = pattern_empty ? -1 : col_idx[row_ptr[i + 1] - 1];
        const float seed_cached = dist_cache[i];
        auto view = [&] {
            return RowView{row_ptr, pat.ptr.data(), stamp.data(), grouping.data(), pat.blk.data(), dist_cache.data(),
                           i, (int64_t)pattern.size(), group_size, seed_cached, tau, pattern_empty};
        };

        auto look = [&](int64_t j) { return view().look(j); };
        // a compared row that is not merged competes for the places left in the group
        auto keep_candidate = [&](int64_t j, float dist) {
            const size_t room = (size_t)(max_rows - (int64_t)merged_rows.size());
            // most rows are farther than every candidate kept so far: see insert_then_trim_is_noop
            if (candidates.size() >= room && (room & 1) && candidates.insert_then_trim_is_noop(dist, j)) return;
            candidates.insert(dist, j);
            if (candidates.size() > room) candidates.trim_from_end(room);
        };
        auto merge = [&](int64_t j) {
            merges++;
            grouping[j] = group_number;
            merged_rows.push_back(j);
            // merge_rows(pattern, row j): row j's columns, plus the pattern's
            // columns below the largest column of row j that is <= max(pattern).
            // An empty row j therefore empties the pattern.
            const bool b_empty = row_ptr[j + 1] == row_ptr[j];
            int64_t cut = -1; // pattern blocks with id < cut survive
            if (!b_empty && !pattern_empty) {
                const int64_t *bb = col_idx + row_ptr[j], *be = col_idx + row_ptr[j + 1];
                const int64_t *ub = std::upper_bound(bb, be, pattern_max);
                if (ub != bb) cut = *(ub - 1) / col_block;
            }
            scratch.clear();
            for (int32_t b : pattern) {
                if (b < cut) scratch.push_back(b);
                else stamp[b] = -1;
            }
            pattern.clear();
            size_t a = 0;
            int64_t k = pat.ptr[j];
            while (a < scratch.size() || k < pat.ptr[j + 1]) {
                if (k >= pat.ptr[j + 1] || (a < scratch.size() && scratch[a] < pat.blk[k])) {
                    pattern.push_back(scratch[a++]);
                } else {
                    if (a < scratch.size() && scratch[a] == pat.blk[k]) a++;
                    pattern.push_back(pat.blk[k++]);
                }
            }
            for (int32_t b : pattern) stamp[b] = i;
            pattern_empty = b_empty;
            pattern_max = b_empty ? -1 : col_idx[row_ptr[j + 1] - 1];
            group_size++;
        };
        // one row, start to end; true if it was merged
        auto scan_row = [&](int64_t j) -> bool {
            const float r = look(j);
            if (r == TAKEN) return false;
            dist_cache[j] = r; // PRUNED is the cache's own mark for "unknown"
            if (r < 0) return false;
            comparisons++;
            if (r > tau) {
                keep_candidate(j, r);
                return false;
            }
            merge(j);
            return true;
        };

        int64_t j = i + 1;
        int64_t since_change = 0; // rows scanned since the pattern last changed
        if (pool.size() == 1) {
            for (; j < rows && group_size != max_rows; j++) scan_row(j);
        }
        // ---- with helpers: `looked` = rows whose results are in a buffer, `stored` = rows applied whose distances
        // still have to go into the cache (the helpers do that on their next job) ----
        Span looked{0, 0, 0}, stored{0, 0, 0}, ahead{0, 0, 0};
        auto free_buffer = [&] { // the one that neither `looked` nor `stored` uses
            for (int b = 0; b < 3; b++)
                if (!(looked.count && looked.buf == b) && !(stored.count && stored.buf == b)) return b;
            return 0; // not reached
        };
        // helpers' job: results of `st` into the distance cache, then rows of `lk` looked at
        Span job_store{0, 0, 0}, job_look{0, 0, 0};
        RowView job_view = view();
        const std::function<void(int)> job = [&](int) {
            const RowView v = job_view;
            const Span st = job_store, lk = job_look;
            float *cache = dist_cache.data();
            for (;;) {
                const int64_t g0 = next_store.fetch_add(GRAIN, std::memory_order_relaxed);
                if (g0 >= st.count) break;
                const int64_t g1 = std::min(st.count, g0 + GRAIN);
                const float *res = results[st.buf].data();
                for (int64_t x = g0; x < g1; x++)
                    if (res[x] != TAKEN) cache[st.first + x] = res[x];
            }
            for (;;) {
                const int64_t g0 = next_look.fetch_add(GRAIN, std::memory_order_relaxed);
                if (g0 >= lk.count) break;
                const int64_t g1 = std::min(lk.count, g0 + GRAIN);
                float *res = results[lk.buf].data();
                for (int64_t x = g0; x < g1; x++) res[x] = v.look(lk.first + x);
            }
        };
        auto batch_rows = [&](int64_t first, int64_t since) {
            return std::min(std::min<int64_t>(rows - first, MAX_BATCH), std::max(FIRST_BATCH, since));
        };
        auto set_job = [&](Span st, Span lk) {
            job_view = view();
            job_store = st;
            job_look = lk;
            next_store.store(0, std::memory_order_relaxed);
            next_look.store(0, std::memory_order_relaxed);
        };
        while (pool.size() > 1 && j < rows && group_size != max_rows) {
            if (since_change < SERIAL_ROWS || rows - j < FIRST_BATCH) {
                // right behind a merge the next one is often near: row by row (rows >= j are in no buffer)
                const int64_t stop = std::min(rows, j + std::max<int64_t>(SERIAL_ROWS - since_change, rows - j < FIRST_BATCH ? rows - j : 0));
                for (; j < stop && group_size != max_rows; j++) since_change = scan_row(j) ? 0 : since_change + 1;
                continue;
            }
            if (!looked.count) { // nothing looked at yet from j on: everybody looks
                looked = Span{free_buffer(), j, batch_rows(j, since_change)};
                set_job(stored, looked);
                pool.run(job);
                stored.count = 0;
            }
            // the helpers look at the rows behind this batch while its results are applied here
            const int64_t behind = looked.first + looked.count;
            ahead = Span{free_buffer(), behind, behind < rows ? batch_rows(behind, since_change + looked.count) : 0};
            set_job(stored, ahead);
            pool.start(job);
            // whatever ends this iteration (an insertion that runs out of memory throws), the helpers have left the
            // job before the buffers and the job itself go away
            struct WaitOnExit { ScanPool &p; ~WaitOnExit() { p.wait(); } } wait_on_exit{pool};
            const float *res = results[looked.buf].data();
            int64_t x = 0;
            bool merged = false;
            // no merge inside the loop: the room for candidates stays what it is
            const size_t room = (size_t)(max_rows - (int64_t)merged_rows.size());
            const bool odd_room = room & 1;
            int64_t compared = 0;
            for (; x < looked.count; x++) {
                const float r = res[x];
                if (r < 0) continue;
                compared++;
                if (r > tau) {
                    const int64_t row = looked.first + x;
                    // most rows are farther than every candidate kept so far: see insert_then_trim_is_noop
                    if (odd_room && candidates.size() >= room && candidates.insert_then_trim_is_noop(r, row)) continue;
                    candidates.insert(r, row);
                    if (candidates.size() > room) candidates.trim_from_end(room);
                    continue;
                }
                merged = true; // applied below, when the helpers no longer read the pattern
                x++;
                break;
            }
            comparisons += compared;
            pool.wait();
            stored = Span{looked.buf, looked.first, x};
            j = looked.first + x;
            if (merged) {
                merge(j - 1);
                since_change = 0;
                looked.count = 0; // what was looked at behind the merge saw the old pattern
            } else {
                since_change += x;
                looked = ahead;
            }
        }
        if (stored.count) { // distances of the last rows applied
            const float *res = results[stored.buf].data();
            for (int64_t x = 0; x < stored.count; x++)
                if (res[x] != TAKEN) dist_cache[stored.first + x] = res[x];
        }

        if (group_size < max_rows) {
            candidates.for_each_ascending([&](const CandidateTree::Node &n) {
                if (group_size == max_rows) return false;
                grouping[n.row] = group_number;
                merged_rows.push_back(n.row);
                group_size++;
                return true;
            });
        }
        if (group_size == max_rows)
            for (int64_t r : merged_rows) grouping[r] -= rows; // complete groups sort first
        for (int32_t b : pattern) stamp[b] = -1;
    }
    return grouping;
}


// CollectBlockingInfo (blocking.cpp:562-614) restricted to the two integer
// statistics that do not depend on timers: number of nonzero blocks and the
// longest block row, for the fixed-size grouping.
void blocking_stats(int64_t rows, const Pattern &pat, const std::vector<int64_t> &grouping,
                    const std::vector<int64_t> &perm, int64_t nblk_cols, int64_t &nzblocks,
                    int64_t &longest)
{
    nzblocks = 0;
    longest = 0;
    std::vector<int64_t> seen((size_t)nblk_cols + 1, -1);
    int64_t r = 0, gid = 0;
    while (r < rows) {
        const int64_t g = grouping[perm[r]];
        int64_t cnt = 0;
        for (; r < rows && grouping[perm[r]] == g; r++) {
            const int64_t row = perm[r];
            for (int64_t k = pat.ptr[row]; k < pat.ptr[row + 1]; k++)
                if (seen[pat.blk[k]] != gid) { seen[pat.blk[k]] = gid; cnt++; }
        }
        nzblocks += cnt;
        longest = std::max(longest, cnt);
        gid++;
    }
}

int reorder_rows_impl(int64_t rows, int64_t cols, const int64_t *row_ptr, const int64_t *col_idx,
                      int64_t col_block, int64_t row_block, float tau, int64_t *grouping_out,
                      int64_t *perm_out, int64_t *stats)
{
    if (rows < 0 || cols < 0 || !row_ptr || (rows && row_ptr[rows] && !col_idx))
        return set_error(SMAT_ERR_INVALID, "bad CSR arguments");
    if (col_block <= 0 || row_block <= 0)
        return set_error(SMAT_ERR_INVALID, "col_block and row_block must be positive");
    if (rows > 0x7fffffff)
        return set_error(SMAT_ERR_INVALID, "more than 2^31-1 rows: the reference narrows row ids to int");
    int64_t max_col = -1;
    for (int64_t r = 0; r < rows; r++) {
        if (row_ptr[r + 1] < row_ptr[r]) return set_error(SMAT_ERR_INVALID, "row_ptr must be non-decreasing");
        for (int64_t k = row_ptr[r]; k < row_ptr[r + 1]; k++) {
            if (col_idx[k] < 0) return set_error(SMAT_ERR_INVALID, "negative column index");
            if (k > row_ptr[r] && col_idx[k] < col_idx[k - 1])
                return set_error(SMAT_ERR_INVALID, "columns of row %lld are not ascending", (long long)r);
            max_col = std::max(max_col, col_idx[k]);
        }
    }
    cols = std::max(cols, max_col + 1);
    const int64_t nblk_cols = (cols + col_block - 1) / col_block;
    if (nblk_cols > 0x7fffffff) return set_error(SMAT_ERR_INVALID, "too many block columns");

    const Pattern pat = build_block_patterns(rows, row_ptr, col_idx, col_block);
    int64_t comparisons = 0, merges = 0;
    std::vector<int64_t> groups = keeper_grouping(rows, row_ptr, col_idx, pat, nblk_cols, col_block,
                                                  row_block, tau, comparisons, merges);
    // force_fixed_size (-F 1): rank rows by group id, cut into chunks of row_block
    std::vector<int64_t> rank = permutation_by_group(groups);
    std::vector<int64_t> fixed((size_t)rows, -1);
    for (int64_t i = 0; i < rows; i++) fixed[rank[i]] = i / row_block;
    // CSR::reorder(grouping) sorts once more, by the fixed-size group id
    std::vector<int64_t> perm = permutation_by_group(fixed);

    if (grouping_out) std::copy(fixed.begin(), fixed.end(), grouping_out);
    if (perm_out) std::copy(perm.begin(), perm.end(), perm_out);
    if (stats) {
        stats[0] = comparisons;
        stats[1] = merges;
        blocking_stats(rows, pat, fixed, perm, nblk_cols, stats[2], stats[3]);
    }
    return SMAT_OK;
}

} // namespace
} // namespace smat

using namespace smat;

static int smat_reorder_rows_impl(int64_t rows, int64_t cols, const int64_t *row_ptr,
                                  const int64_t *col_idx, int64_t col_block, int64_t row_block,
                                  float tau, int64_t *grouping, int64_t *perm, int64_t *stats)
{
    return reorder_rows_impl(rows, cols, row_ptr, col_idx, col_block, row_block, tau, grouping, perm,
                             stats);
}

extern "C" int smat_reorder_rows(int64_t rows, int64_t cols, const int64_t *row_ptr,
                                  const int64_t *col_idx, int64_t col_block, int64_t row_block,
                                  float tau, int64_t *grouping, int64_t *perm, int64_t *stats)
{
    return smat::guarded("smat_reorder_rows", [&] { return smat_reorder_rows_impl(rows, cols, row_ptr, col_idx, col_block, row_block, tau, grouping, perm, stats); });
}

static int smat_reorder_csr_impl(size_t M, size_t K, const int32_t *row_ptr, const int32_t *col_idx,
                                 int64_t col_block, int64_t row_block, float tau, int do_cols,
                                 int64_t *perm_rows, int64_t *perm_cols, int64_t *stats_rows,
                                 int64_t *stats_cols)
{
    if (!row_ptr || !perm_rows || (do_cols && !perm_cols))
        return set_error(SMAT_ERR_INVALID, "row_ptr / perm outputs must not be NULL");
    const int64_t nnz = row_ptr[M];
    if (nnz && !col_idx) return set_error(SMAT_ERR_INVALID, "col_idx must not be NULL");
    // Pattern with ascending columns per row (src/reorder.py:76 sorts by (row, col));
    // rows after the last nonempty one do not exist in an edge list (csr.cpp:262).
    int64_t rows_eff = 0;
    for (size_t r = 0; r < M; r++)
        if (row_ptr[r + 1] > row_ptr[r]) rows_eff = (int64_t)r + 1;
    std::vector<int64_t> rp((size_t)rows_eff + 1), ci((size_t)(rows_eff ? row_ptr[rows_eff] : 0));
    int64_t cols_eff = 0;
    for (int64_t r = 0; r < rows_eff; r++) {
        rp[r] = row_ptr[r];
        for (int64_t k = row_ptr[r]; k < row_ptr[r + 1]; k++) {
            if (col_idx[k] < 0 || (size_t)col_idx[k] >= K)
                return set_error(SMAT_ERR_INVALID, "column index out of range in row %lld", (long long)r);
            ci[k] = col_idx[k];
            cols_eff = std::max<int64_t>(cols_eff, (int64_t)col_idx[k] + 1);
        }
        std::sort(ci.begin() + row_ptr[r], ci.begin() + row_ptr[r + 1]);
    }
    rp[rows_eff] = rows_eff ? row_ptr[rows_eff] : 0;

    std::vector<int64_t> pr((size_t)rows_eff);
    int rc = reorder_rows_impl(rows_eff, cols_eff, rp.data(), ci.data(), col_block, row_block, tau,
                               nullptr, pr.data(), stats_rows);
    if (rc) return rc;
    for (int64_t r = 0; r < rows_eff; r++) perm_rows[r] = pr[r];
    for (size_t r = (size_t)rows_eff; r < M; r++) perm_rows[r] = (int64_t)r;
    if (!do_cols) {
        if (perm_cols) for (size_t c = 0; c < K; c++) perm_cols[c] = (int64_t)c;
        return SMAT_OK;
    }

    // Transpose of the row-permuted pattern: row c of T lists the new row ids
    // that hold column c, ascending (src/reorder.py:82-104).
    std::vector<int64_t> tp((size_t)cols_eff + 1, 0), ti((size_t)rp[rows_eff]);
    for (int64_t k = 0; k < rp[rows_eff]; k++) tp[ci[k] + 1]++;
    for (int64_t c = 0; c < cols_eff; c++) tp[c + 1] += tp[c];
    {
        std::vector<int64_t> fill(tp.begin(), tp.end() - 1);
        for (int64_t rn = 0; rn < rows_eff; rn++) {
            const int64_t ro = pr[rn];
            for (int64_t k = rp[ro]; k < rp[ro + 1]; k++) ti[fill[ci[k]]++] = rn;
        }
    }
    std::vector<int64_t> pc((size_t)cols_eff);
    rc = reorder_rows_impl(cols_eff, rows_eff, tp.data(), ti.data(), col_block, row_block, tau, nullptr,
                           pc.data(), stats_cols);
    if (rc) return rc;
    for (int64_t c = 0; c < cols_eff; c++) perm_cols[c] = pc[c];
    for (size_t c = (size_t)cols_eff; c < K; c++) perm_cols[c] = (int64_t)c;
    return SMAT_OK;
}

extern "C" int smat_reorder_csr(size_t M, size_t K, const int32_t *row_ptr, const int32_t *col_idx,
                                 int64_t col_block, int64_t row_block, float tau, int do_cols,
                                 int64_t *perm_rows, int64_t *perm_cols, int64_t *stats_rows,
                                 int64_t *stats_cols)
{
    return smat::guarded("smat_reorder_csr", [&] { return smat_reorder_csr_impl(M, K, row_ptr, col_idx, col_block, row_block, tau, do_cols, perm_rows, perm_cols, stats_rows, stats_cols); });
}

static int smat_permute_csr_impl(size_t M, size_t K, const int32_t *row_ptr, const int32_t *col_idx,
                                 const uint16_t *val, const int64_t *perm_rows,
                                 const int64_t *perm_cols, int32_t **out_row_ptr,
                                 int32_t **out_col_idx, uint16_t **out_val)
{
    if (!row_ptr || !out_row_ptr || !out_col_idx || !out_val)
        return set_error(SMAT_ERR_INVALID, "NULL argument");
    const int64_t nnz = row_ptr[M];
    std::vector<int32_t> inv_col;
    if (perm_cols) {
        inv_col.assign(K, -1);
        for (size_t c = 0; c < K; c++) {
            if (perm_cols[c] < 0 || (size_t)perm_cols[c] >= K || inv_col[perm_cols[c]] != -1)
                return set_error(SMAT_ERR_INVALID, "perm_cols is not a permutation of 0..K-1");
            inv_col[perm_cols[c]] = (int32_t)c;
        }
    }
    if (perm_rows) {
        std::vector<char> seen(M, 0);
        for (size_t r = 0; r < M; r++) {
            if (perm_rows[r] < 0 || (size_t)perm_rows[r] >= M || seen[perm_rows[r]])
                return set_error(SMAT_ERR_INVALID, "perm_rows is not a permutation of 0..M-1");
            seen[perm_rows[r]] = 1;
        }
    }
    int32_t *rp = (int32_t *)malloc(sizeof(int32_t) * (M + 1));
    int32_t *ci = (int32_t *)malloc(sizeof(int32_t) * (size_t)std::max<int64_t>(nnz, 1));
    uint16_t *vv = (uint16_t *)malloc(sizeof(uint16_t) * (size_t)std::max<int64_t>(nnz, 1));
    if (!rp || !ci || !vv) {
        free(rp); free(ci); free(vv);
        return set_error(SMAT_ERR_NOMEM, "out of host memory");
    }
    std::vector<std::pair<int32_t, uint16_t>> row;
    int64_t o = 0;
    for (size_t rn = 0; rn < M; rn++) {
        const size_t ro = perm_rows ? (size_t)perm_rows[rn] : rn;
        rp[rn] = (int32_t)o;
        row.clear();
        for (int64_t k = row_ptr[ro]; k < row_ptr[ro + 1]; k++) {
            if (col_idx[k] < 0 || (size_t)col_idx[k] >= K) {
                free(rp); free(ci); free(vv);
                return set_error(SMAT_ERR_INVALID, "column index out of range");
            }
            row.emplace_back(perm_cols ? inv_col[col_idx[k]] : col_idx[k], val ? val[k] : (uint16_t)0x3c00);
        }
        std::stable_sort(row.begin(), row.end(),
                         [](const std::pair<int32_t, uint16_t> &a, const std::pair<int32_t, uint16_t> &b) {
                             return a.first < b.first;
                         });
        for (auto &e : row) { ci[o] = e.first; vv[o] = e.second; o++; }
    }
    rp[M] = (int32_t)o;
    *out_row_ptr = rp; *out_col_idx = ci; *out_val = vv;
    return SMAT_OK;
}

extern "C" int smat_permute_csr(size_t M, size_t K, const int32_t *row_ptr, const int32_t *col_idx,
                                 const uint16_t *val, const int64_t *perm_rows,
                                 const int64_t *perm_cols, int32_t **out_row_ptr,
                                 int32_t **out_col_idx, uint16_t **out_val)
{
    return smat::guarded("smat_permute_csr", [&] { return smat_permute_csr_impl(M, K, row_ptr, col_idx, val, perm_rows, perm_cols, out_row_ptr, out_col_idx, out_val); });
}
