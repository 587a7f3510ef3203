"""Seeded synthetic inputs for the five benchmark/parity configurations.

All randomness comes from a counter-based generator (splitmix64 of seed and
element index), so any machine regenerates bit-identical matrices without
shipping data.  Values are rounded to fp16 at generation.

The band pattern follows the reference generator generate_band_mtx_matrix
(src/generate_matrices.py:5-35): row i holds columns max(0, i-b) .. min(N, i+b+1)-1.
"""
import numpy as np

_GOLDEN = np.uint64(0x9E3779B97F4A7C15)
_M1 = np.uint64(0xBF58476D1CE4E5B9)
_M2 = np.uint64(0x94D049BB133111EB)


def rand_u64(seed, idx):
    """splitmix64 output for counter `idx` (array of uint64) under `seed`."""
    with np.errstate(over="ignore"):
        z = np.uint64(seed) + (np.asarray(idx, dtype=np.uint64) + np.uint64(1)) * _GOLDEN
        z = (z ^ (z >> np.uint64(30))) * _M1
        z = (z ^ (z >> np.uint64(27))) * _M2
        return z ^ (z >> np.uint64(31))


def rand_uniform(seed, idx):
    """float64 in [0, 1)."""
    return (rand_u64(seed, idx) >> np.uint64(11)).astype(np.float64) * (1.0 / 9007199254740992.0)


def rand_normal(seed, idx):
    """Standard normal via Box-Muller on counters 2*idx and 2*idx+1."""
    idx = np.asarray(idx, dtype=np.uint64)
    u1 = 1.0 - rand_uniform(seed, idx * np.uint64(2))  # (0, 1]
    u2 = rand_uniform(seed, idx * np.uint64(2) + np.uint64(1))
    return np.sqrt(-2.0 * np.log(u1)) * np.cos(2.0 * np.pi * u2)


def f16_bits(x):
    return np.asarray(x, dtype=np.float64).astype(np.float16).view(np.uint16)


def dense_b(K, N, seed, dist="normal", chunk=1 << 24):
    """Column-major K x N fp16 operand as a flat uint16 array: element (k,n) at [n*K+k]."""
    total = K * N
    out = np.empty(total, dtype=np.uint16)
    for s in range(0, total, chunk):
        idx = np.arange(s, min(total, s + chunk), dtype=np.uint64)
        v = rand_normal(seed, idx) if dist == "normal" else 2.0 * rand_uniform(seed, idx) - 1.0
        out[s:s + idx.size] = f16_bits(v)
    return out


def _csr_from_sorted_coo(M, rows, cols, vals):
    row_ptr = np.zeros(M + 1, dtype=np.int64)
    np.add.at(row_ptr, rows + 1, 1)
    row_ptr = np.cumsum(row_ptr)
    return row_ptr.astype(np.int32), cols.astype(np.int32), vals


def band(M=4096, bandwidth=64, seed=0x5A170001):
    """Config 1: |i-j| <= bandwidth, values U[-1,1]. Returns CSR dict."""
    i = np.arange(M, dtype=np.int64)
    lo = np.maximum(0, i - bandwidth)
    hi = np.minimum(M, i + bandwidth + 1)
    cnt = hi - lo
    row_ptr = np.concatenate([[0], np.cumsum(cnt)])
    rows = np.repeat(i, cnt)
    cols = np.arange(row_ptr[-1], dtype=np.int64) - np.repeat(row_ptr[:-1], cnt) + np.repeat(lo, cnt)
    vals = f16_bits(2.0 * rand_uniform(seed, rows * np.int64(M) + cols) - 1.0)
    return {"M": M, "K": M, "row_ptr": row_ptr.astype(np.int32), "col_idx": cols.astype(np.int32), "val": vals}


def erdos_renyi(M=16384, density=0.001, seed=0x5A170002):
    """Config 2: round(density*M*M) i.i.d. uniform (row, col) draws, duplicates merged, values N(0,1)."""
    draws = int(round(density * M * M))
    idx = np.arange(draws, dtype=np.uint64)
    r = (rand_u64(seed, idx * np.uint64(2)) % np.uint64(M)).astype(np.int64)
    c = (rand_u64(seed, idx * np.uint64(2) + np.uint64(1)) % np.uint64(M)).astype(np.int64)
    key = np.unique(r * M + c)
    rows, cols = key // M, key % M
    vals = f16_bits(rand_normal(seed ^ 0xA5A5, key))
    rp, ci, v = _csr_from_sorted_coo(M, rows, cols, vals)
    return {"M": M, "K": M, "row_ptr": rp, "col_idx": ci, "val": v}


def rmat(scale=20, avg_degree=16, probs=(0.57, 0.19, 0.19, 0.05), seed=0x5A170003, chunk=1 << 22):
    """Config 3: R-MAT, 2^scale rows, avg_degree*2^scale edge draws, duplicates merged, values U[-1,1]."""
    M = 1 << scale
    edges = avg_degree * M
    a, b, c, _ = probs
    keys = []
    for s in range(0, edges, chunk):
        e = np.arange(s, min(edges, s + chunk), dtype=np.uint64)
        r = np.zeros(e.size, dtype=np.int64)
        col = np.zeros(e.size, dtype=np.int64)
        for lvl in range(scale):
            u = rand_uniform(seed, e * np.uint64(scale) + np.uint64(lvl))
            down = (u >= a + b).astype(np.int64)                      # quadrants c, d: lower half
            right = (((u >= a) & (u < a + b)) | (u >= a + b + c)).astype(np.int64)  # quadrants b, d
            r = (r << 1) | down
            col = (col << 1) | right
        keys.append(r * M + col)
    key = np.unique(np.concatenate(keys))
    rows, cols = key // M, key % M
    vals = f16_bits(2.0 * rand_uniform(seed ^ 0xA5A5, key) - 1.0)
    rp, ci, v = _csr_from_sorted_coo(M, rows, cols, vals)
    return {"M": M, "K": M, "row_ptr": rp, "col_idx": ci, "val": v}


def block_pruned(M=8192, keep=0.10, sigma=0.02, seed=0x5A170004):
    """Config 4: 16x16 block mask with exactly round(keep * (M/16)^2) blocks kept (the
    blocks with the smallest hash), kept blocks fully dense with N(0, sigma) values.
    Returns the BCSR arrays directly (row_ptr, col_idx absolute, val) plus CSR on demand."""
    mb = M // 16
    cells = mb * mb
    kept = int(round(keep * cells))
    h = rand_u64(seed, np.arange(cells, dtype=np.uint64))
    sel = np.sort(np.argpartition(h, kept - 1)[:kept]) if kept < cells else np.arange(cells)
    br, bc = sel // mb, sel % mb
    row_ptr = np.zeros(mb + 1, dtype=np.int64)
    np.add.at(row_ptr, br + 1, 1)
    row_ptr = np.cumsum(row_ptr).astype(np.int32)
    col_idx = (bc * 16).astype(np.int32)
    # value of element (row, col) is drawn from counter row*M + col, independent of blocking
    e = np.arange(256, dtype=np.int64)
    rows = (br[:, None] * 16 + e[None, :] // 16)
    cols = (bc[:, None] * 16 + e[None, :] % 16)
    val = f16_bits(sigma * rand_normal(seed ^ 0xA5A5, (rows * M + cols).ravel()))
    return {"M": M, "K": M, "b_row_ptr": row_ptr, "b_col_idx": col_idx, "b_val": val, "nnzb": kept}


def block_pruned_skewed(M=8192, keep_first=0.18, keep_last=0.02, sigma=0.02, seed=0x5A170008):
    """A block-pruned weight whose rows were pruned unevenly: block row i keeps each of its blocks with a probability
    that falls linearly from keep_first (row 0) to keep_last (last row); kept blocks dense with N(0, sigma) values
    drawn as in block_pruned.  BCSR arrays like block_pruned."""
    mb = M // 16
    cells = mb * mb
    keep = keep_first + (keep_last - keep_first) * np.arange(mb, dtype=np.float64) / max(mb - 1, 1)
    u = (rand_u64(seed, np.arange(cells, dtype=np.uint64)) >> np.uint64(11)).astype(np.float64) * 2.0 ** -53
    sel = np.nonzero(u < np.repeat(keep, mb))[0]
    br, bc = sel // mb, sel % mb
    row_ptr = np.zeros(mb + 1, dtype=np.int64)
    np.add.at(row_ptr, br + 1, 1)
    e = np.arange(256, dtype=np.int64)
    rows = (br[:, None] * 16 + e[None, :] // 16)
    cols = (bc[:, None] * 16 + e[None, :] % 16)
    val = f16_bits(sigma * rand_normal(seed ^ 0xA5A5, (rows * M + cols).ravel()))
    return {"M": M, "K": M, "b_row_ptr": np.cumsum(row_ptr).astype(np.int32), "b_col_idx": (bc * 16).astype(np.int32),
            "b_val": val, "nnzb": int(sel.size)}


def half_pruned_half_er(M=8192, keep=0.10, density=0.001, seed=0x5A170006):
    """A matrix of two kinds of rows: the upper half of its block rows from block_pruned (dense 16x16 blocks), the
    lower half the blocking of an Erdos-Renyi matrix (about one nonzero per block).  BCSR arrays like block_pruned."""
    from . import host
    mb = M // 16
    top = block_pruned(M, keep, 0.02, seed)
    er = erdos_renyi(M, density, seed ^ 0x77)
    low = host.csr_to_bcsr(er["M"], er["K"], er["row_ptr"], er["col_idx"], er["val"])
    h = mb // 2
    t_end = int(top["b_row_ptr"][h])
    l_begin = int(low.row_ptr[h])
    row_ptr = np.concatenate([top["b_row_ptr"][:h + 1], low.row_ptr[h + 1:] - l_begin + t_end]).astype(np.int32)
    col_idx = np.concatenate([top["b_col_idx"][:t_end], low.col_idx[l_begin:]]).astype(np.int32)
    val = np.concatenate([top["b_val"][:t_end * 256], low.val[l_begin * 256:]])
    return {"M": M, "K": M, "b_row_ptr": row_ptr, "b_col_idx": col_idx, "b_val": val, "nnzb": int(col_idx.size),
            "dense_blocks": t_end}


def pruned_plus_er(M=8192, keep=0.10, density=0.001, seed=0x5A170007):
    """Every block row holds both kinds of blocks: the dense 16x16 blocks of block_pruned, and between them the
    blocks of an Erdos-Renyi matrix (about one nonzero each; where one falls on a dense block the dense block stays).
    BCSR arrays like block_pruned, plus "dense_blocks"."""
    from . import host
    mb = M // 16
    top = block_pruned(M, keep, 0.02, seed)
    er = erdos_renyi(M, density, seed ^ 0x77)
    low = host.csr_to_bcsr(er["M"], er["K"], er["row_ptr"], er["col_idx"], er["val"])
    key_d = np.repeat(np.arange(mb, dtype=np.int64), np.diff(top["b_row_ptr"])) * mb + top["b_col_idx"].astype(np.int64) // 16
    key_s = np.repeat(np.arange(mb, dtype=np.int64), np.diff(low.row_ptr)) * mb + low.col_idx.astype(np.int64) // 16
    only_s = ~np.isin(key_s, key_d)
    keys = np.concatenate([key_d, key_s[only_s]])
    vals = np.concatenate([np.asarray(top["b_val"]).reshape(-1, 256), np.asarray(low.val).reshape(-1, 256)[only_s]])
    order = np.argsort(keys, kind="stable")
    keys, vals = keys[order], vals[order]
    row_ptr = np.zeros(mb + 1, np.int64)
    np.add.at(row_ptr, keys // mb + 1, 1)
    return {"M": M, "K": M, "b_row_ptr": np.cumsum(row_ptr).astype(np.int32), "b_col_idx": ((keys % mb) * 16).astype(np.int32),
            "b_val": np.ascontiguousarray(vals).ravel(), "nnzb": int(keys.size), "dense_blocks": int(key_d.size)}


def bcsr_to_csr(M, b_row_ptr, b_col_idx, b_val, drop_zeros=False):
    """Expands BCSR blocks to a CSR (all 256 entries per block unless drop_zeros)."""
    mb = M // 16
    nnzb = b_col_idx.shape[0]
    br = np.repeat(np.arange(mb, dtype=np.int64), np.diff(b_row_ptr))
    e = np.arange(256, dtype=np.int64)
    rows = (br[:, None] * 16 + e[None, :] // 16).ravel()
    cols = (b_col_idx.astype(np.int64)[:, None] + e[None, :] % 16).ravel()
    vals = np.asarray(b_val).reshape(nnzb * 256)
    if drop_zeros:
        keep = (vals & 0x7FFF) != 0
        rows, cols, vals = rows[keep], cols[keep], vals[keep]
    order = np.lexsort((cols, rows))
    rows, cols, vals = rows[order], cols[order], vals[order]
    return _csr_from_sorted_coo(M, rows, cols, vals)


def stencil27(n=64, seed=0):
    """Config 5: 27-point stencil on an n^3 grid, index x + n*y + n*n*z, diagonal 26, others -1."""
    del seed
    M = n ** 3
    idx = np.arange(M, dtype=np.int64)
    x, y, z = idx % n, (idx // n) % n, idx // (n * n)
    rows_l, cols_l, vals_l = [], [], []
    for dz in (-1, 0, 1):
        for dy in (-1, 0, 1):
            for dx in (-1, 0, 1):
                ok = (x + dx >= 0) & (x + dx < n) & (y + dy >= 0) & (y + dy < n) & (z + dz >= 0) & (z + dz < n)
                rows_l.append(idx[ok])
                cols_l.append(idx[ok] + dx + n * dy + n * n * dz)
                v = 26.0 if (dx == 0 and dy == 0 and dz == 0) else -1.0
                vals_l.append(np.full(int(ok.sum()), v))
    rows, cols, vals = np.concatenate(rows_l), np.concatenate(cols_l), np.concatenate(vals_l)
    order = np.lexsort((cols, rows))
    rp, ci, v = _csr_from_sorted_coo(M, rows[order], cols[order], f16_bits(vals[order]))
    return {"M": M, "K": M, "row_ptr": rp, "col_idx": ci, "val": v}


def random_bcsr(mb, kb, density, seed, row_lengths=None):
    """Small random BCSR for tests: Bernoulli(density) block mask (or given row lengths with
    random distinct block columns), values U[-1,1] in every block entry."""
    rng_idx = np.arange(mb * kb, dtype=np.uint64)
    if row_lengths is None:
        mask = (rand_uniform(seed, rng_idx) < density).reshape(mb, kb)
    else:
        mask = np.zeros((mb, kb), dtype=bool)
        score = rand_uniform(seed, rng_idx).reshape(mb, kb)
        for r, ln in enumerate(row_lengths):
            if ln > 0:
                mask[r, np.argsort(score[r], kind="stable")[:ln]] = True
    br, bc = np.nonzero(mask)
    row_ptr = np.concatenate([[0], np.cumsum(mask.sum(axis=1))]).astype(np.int32)
    col_idx = (bc * 16).astype(np.int32)
    n = br.shape[0] * 256
    val = f16_bits(2.0 * rand_uniform(seed ^ 0x77, np.arange(n, dtype=np.uint64)) - 1.0)
    return {"M": mb * 16, "K": kb * 16, "b_row_ptr": row_ptr, "b_col_idx": col_idx, "b_val": val,
            "nnzb": int(br.shape[0])}
