"""How the compact kernel's launch deals its workgroups to the eight XCDs, checked on the CPU.

The hardware gives an XCD the workgroup ids that are equal modulo 8, whatever their work costs.  The launcher lays the
(panel, item) space out in runs of consecutive workgroups (4 items each) that the XCDs take in turn, and picks the
run length from the cost of the items: one run per XCD (neighbouring block rows on one L2) where that is balanced,
shorter runs where the cost changes along the list.  The choice is a host function; here it is compared with the
loads that the same deal gives in numpy."""
import ctypes as C

import numpy as np
import pytest

from smat_amd._lib import lib

CANDIDATES = (1024, 256, 64, 16, 4)
LIMIT = 1.04

_fn = lib.smat_internal_choose_xcd_run
_fn.restype = C.c_uint
_fn.argtypes = [C.c_void_p, C.c_uint64, C.c_int]


def choose(costs, n_panels):
    prefix = np.concatenate([[0], np.cumsum(np.asarray(costs, np.uint64))]).astype(np.uint64)
    return int(_fn(prefix.ctypes.data, len(costs), n_panels))


def busiest_over_mean(costs, n_panels, run):
    """Load of the busiest XCD over the mean load when run q (workgroups q*run ..) goes to XCD q % 8."""
    w = np.tile(np.asarray(costs, np.float64), n_panels)
    wgs = (len(w) + 3) // 4
    w = np.concatenate([w, np.zeros(4 * wgs - len(w))]).reshape(wgs, 4).sum(axis=1)
    n_runs = (wgs + run - 1) // run
    w = np.concatenate([w, np.zeros(n_runs * run - wgs)]).reshape(n_runs, run).sum(axis=1)
    load = np.array([w[x::8].sum() for x in range(8)])
    return load.max() / load.mean()


def eighth(n_items, n_panels):
    return max(((n_items * n_panels + 3) // 4 + 7) // 8, 1)


@pytest.mark.parametrize("n_items,n_panels", [(16384, 1), (1024, 4), (70596, 2), (4096, 64), (33, 1), (1, 1), (7, 3)])
def test_items_of_one_cost_stay_in_one_run_per_xcd(n_items, n_panels):
    assert choose(np.full(n_items, 9), n_panels) == eighth(n_items, n_panels)


def test_no_items_and_no_cost():
    assert choose([], 1) == 1
    assert choose(np.zeros(100, np.uint64), 2) == eighth(100, 2)


@pytest.mark.parametrize("n_panels", [1, 2, 3, 5])
def test_cost_that_falls_along_the_list_gets_short_runs(n_panels):
    """A list like that of an R-MAT matrix: chunks of split rows first (47 steps each), then block rows whose cost
    falls with the row number.  One run per XCD would leave the first XCD with far more than the mean."""
    rng = np.random.default_rng(5)
    n = 60000
    tail = 2 + np.ceil(40.0 / (1 + np.arange(n) / 800.0) * rng.random(n)).astype(np.uint64)
    costs = np.concatenate([np.full(6000, 47, np.uint64), tail])
    assert busiest_over_mean(costs, n_panels, eighth(len(costs), n_panels)) > 1.3
    run = choose(costs, n_panels)
    assert run in CANDIDATES
    assert busiest_over_mean(costs, n_panels, run) <= LIMIT + 1e-9
    longer = [r for r in CANDIDATES if run < r < eighth(len(costs), n_panels)]
    assert all(busiest_over_mean(costs, n_panels, r) > LIMIT for r in longer)   # the longest run that is balanced
    # with eight panels one run per XCD is a whole panel each: the same list for everyone
    assert choose(costs, 8) == eighth(len(costs), 8)


def test_nothing_balanced_takes_the_best_candidate():
    """One item that outweighs the rest: no deal is within the limit, the choice is the candidate with the lowest
    busiest-to-mean ratio."""
    costs = np.full(4000, 3, np.uint64)
    costs[17] = 100000
    run = choose(costs, 1)
    cands = [eighth(len(costs), 1)] + [r for r in CANDIDATES if r < eighth(len(costs), 1)]
    ratios = {r: busiest_over_mean(costs, 1, r) for r in cands}
    assert min(ratios.values()) > LIMIT
    assert ratios[run] <= min(ratios.values()) + 1e-9


def test_random_lists_agree_with_the_numpy_deal():
    rng = np.random.default_rng(11)
    for trial in range(40):
        n = int(rng.integers(1, 5000))
        n_panels = int(rng.integers(1, 6))
        shape = rng.random()
        costs = (2 + rng.integers(0, 60, n) * (rng.random(n) < shape) * (np.arange(n) < n * rng.random())).astype(np.uint64)
        run = choose(costs, n_panels)
        e = eighth(n, n_panels)
        cands = [e] + [r for r in CANDIDATES if r < e]
        assert run in cands
        ratios = [busiest_over_mean(costs, n_panels, r) for r in cands]
        first_ok = next((r for r, q in zip(cands, ratios) if q <= LIMIT), None)
        if first_ok is not None:
            # a ratio within rounding of the limit may fall either way in the two computations
            assert run == first_ok or abs(ratios[cands.index(first_ok)] - LIMIT) < 1e-6 or abs(ratios[cands.index(run)] - LIMIT) < 1e-6
        else:
            assert ratios[cands.index(run)] <= min(ratios) + 1e-9

