"""The step planner (include/qw_par.h) without a GPU: the averaging rule, the estimate and the cut of the reference
(src/engine.c:8762-8797, 9037) restated with groups of up to 16 rows — the cut against a brute force over every
composition, the tie and never-measured rules on hand cases — and the choice between groups and the packing path."""
import functools
import itertools

import numpy as np
import pytest

import qwental_amd as q


def feed(par, b, values, packed=False):
    """Observe a dummy first sample (dropped: it would contain the kernel build) and then the values."""
    for v in [1e6] + list(values):
        (par.observe_packed if packed else par.observe)(b, v)


def test_running_average():
    p = q.Par()
    assert p.group_cost(4) == 0 and p.cost(4) == 0 and p.split(4) == [4]
    p.observe(4, 50.0)
    assert p.group_cost(4) == 0          # the first sample of a size is dropped
    p.observe(4, 2.0)
    assert p.group_cost(4) == 2.0        # the second starts the average
    p.observe(4, 3.0)
    assert p.group_cost(4) == pytest.approx(0.9 * 2.0 + 0.1 * 3.0, rel=0, abs=1e-15)
    p.observe(4, 1.0)
    assert p.group_cost(4) == pytest.approx(0.9 * (0.9 * 2.0 + 0.1 * 3.0) + 0.1, rel=0, abs=1e-15)
    for bad in (0, -1, 17):
        p.observe(bad, 1.0)
        assert p.group_cost(bad) == 0
    p.observe(5, -1.0)
    p.observe(5, 0.0)
    p.observe(5, 7.0)                    # non-positive samples do not count, so this is still the first
    assert p.group_cost(5) == 0
    p.free()


def test_estimate_fills_unmeasured_sizes_on_a_line():
    p = q.Par()
    feed(p, 4, [2.0])
    # one size measured: every size costs the same, so B rows cost one group per 16
    assert p.cost(1) == p.cost(16) == 2.0 and p.cost(17) == p.cost(32) == 4.0 and p.cost(64) == 8.0
    assert p.cost(200) == p.cost(64)     # more rows than a step holds count as a full step
    assert p.cost(0) == 0 and p.cost(-3) == 0
    feed(p, 16, [3.2])                   # line through (4, 2.0) and (16, 3.2): 1.6 + 0.1 b
    c = lambda b: 2.0 if b == 4 else 3.2 if b == 16 else 1.6 + 0.1 * b
    assert p.cost(10) == pytest.approx(c(10)) and p.cost(1) == pytest.approx(1.7)
    assert p.cost(20) == pytest.approx(min(c(a) + c(20 - a) for a in range(4, 17)))
    assert p.cost(40) == pytest.approx(min(c(a) + c(b) + c(40 - a - b) for a in range(8, 17) for b in range(8, 17) if 1 <= 40 - a - b <= 16))
    p.free()


def test_estimate_is_never_zero_or_negative():
    """Two measured sizes close together whose times fall with the size (a launch's time varies by a few per cent): the
    line is taken as flat and no estimate goes below half of the cheapest measured size."""
    p = q.Par()
    feed(p, 14, [0.30])
    feed(p, 16, [0.216])
    assert p.cost(1) == pytest.approx(0.216) and p.cost(8) == pytest.approx(0.216)  # flat at the cheapest measured size
    assert p.cost(46) == pytest.approx(3 * 0.216)
    p.free()
    p = q.Par()
    feed(p, 15, [1.0])
    feed(p, 16, [2.0])  # a steep rising line through two neighbours would cross zero at 14
    assert p.cost(1) == pytest.approx(0.5) and p.cost(3) == pytest.approx(0.5)
    p.free()


def brute(cost, B):
    """Cheapest sum over every multiset of group sizes 1..16 that adds up to B."""
    @functools.lru_cache(None)
    def best(n):
        return 0.0 if n == 0 else min(best(n - b) + cost[b] for b in range(1, min(16, n) + 1))
    return best(B)


@pytest.mark.parametrize("seed", range(6))
def test_cut_is_optimal(seed):
    rng = np.random.default_rng(seed)
    p = q.Par()
    # anything from concave (large groups pay) to convex (small groups pay) tables, all sizes measured
    base = rng.uniform(0.5, 3.0)
    cost = [0.0] + [float(base + rng.uniform(0.0, 0.4) * b ** rng.uniform(0.5, 1.8) + rng.uniform(0, 0.2)) for b in range(1, 17)]
    for b in range(1, 17):
        feed(p, b, [cost[b]])
    for B in list(range(1, 41)) + [47, 63, 64]:
        g = p.split(B)
        assert sum(g) == B and all(1 <= x <= 16 for x in g)
        assert sum(cost[x] for x in g) == pytest.approx(brute(tuple(cost), B), rel=1e-12)
        assert p.cost(B) == pytest.approx(brute(tuple(cost), B), rel=1e-12)
    assert p.split(0) == [] and p.split(65) == [] and p.split(-1) == []
    p.free()


def test_ties_take_the_larger_group_and_unmeasured_sizes_get_tried():
    p = q.Par()
    for b in range(1, 17):
        feed(p, b, [1.0])
    assert p.split(40) == [16, 16, 8] and p.split(16) == [16] and p.split(17) == [16, 1] and p.split(64) == [16] * 4
    p.free()
    p = q.Par()
    feed(p, 16, [5.0])                   # only full groups were ever measured: every other size counts as free
    assert p.split(16) == [15, 1]        # ... so two untried sizes beat the one measured group
    assert p.split(20) == [15, 5]        # two untried sizes beat one measured group plus an untried one
    assert p.split(12) == [12]
    assert p.cost(20) == pytest.approx(10.0)  # the estimate does not take untried sizes as free: two groups at the flat 5.0
    p.free()


def test_groups_or_packing_path():
    """Per-layer times of the kind measured on the device (microseconds): groups 36 + 2.6 b, packing 55 + 0.63 rows."""
    p = q.Par()
    assert p.choose(20) == (False, [16, 4])  # nothing measured: groups, untried sizes first, the larger group on ties
    for b in range(1, 17):
        feed(p, b, [36 + 2.6 * b])
    assert p.packed_cost(40) == 0 and p.choose(40)[0] is False  # the packing path was never measured: groups
    for rows in (16, 64, 128):
        feed(p, rows, [55 + 0.63 * rows], packed=True)
    assert p.packed_cost(16) == pytest.approx(55 + 0.63 * 16) and p.packed_cost(9) == p.packed_cost(16)
    assert p.packed_cost(40) == pytest.approx(55 + 0.63 * 48)      # bucket of 33..48 rows, on the line through the measured ones
    assert p.packed_cost(1000) == p.packed_cost(256)
    packed, groups = p.choose(8)
    assert not packed and groups == [8]                              # 56.8 in one group against 65.1
    packed, groups = p.choose(16)
    assert packed and groups == [16]                                 # 77.6 against 65.1: already at a full group
    packed, groups = p.choose(35)
    assert packed and sum(groups) == 35                              # three groups (>= 140) against 85
    assert p.choose(200)[0] and p.choose(200)[1] == []               # beyond a step's rows the caller cuts full groups itself
    assert p.choose(0) == (False, [])
    # a table on which the packing path never pays
    s = q.Par()
    for b in (1, 16):
        feed(s, b, [10.0])
    feed(s, 16, [500.0], packed=True)
    assert all(not s.choose(r)[0] for r in (1, 16, 40, 64, 200))
    s.free()
    p.free()


def test_time_slices_or_a_joint_step():
    """qw_par_want_slice, the rule of the reference's tools/serve.c:1715-1729: the trivial counts, the figures it falls
    back on, and the five per cent either way before the mode changes."""
    p = q.Par()
    # one conversation: slices, whatever the figures; more than QW_PAR_SLICE_MAX = 3: a joint step, whatever the figures
    assert p.want_slice(1, False) and p.want_slice(0, False, batched_rate=1e9)
    assert not p.want_slice(4, True, sliced_rate=1e9, batched_rate=1.0)
    # no figure on one side: together
    assert not p.want_slice(2, True, sliced_rate=100.0)
    assert not p.want_slice(2, True, batched_rate=100.0)
    assert not p.want_slice(2, True)
    # both measured: slices stay while they reach 95 % of the joint rate, and are taken up only above 105 %
    for n in (2, 3):
        assert p.want_slice(n, True, sliced_rate=96.0, batched_rate=100.0)
        assert not p.want_slice(n, True, sliced_rate=94.0, batched_rate=100.0)
        assert not p.want_slice(n, False, sliced_rate=104.0, batched_rate=100.0)
        assert p.want_slice(n, False, sliced_rate=106.0, batched_rate=100.0)
        assert not p.want_slice(n, True, sliced_rate=95.0, batched_rate=100.0)   # the comparison is strict
    # slices never measured: the mean of the conversations' own rates, the default standing in for a missing one
    assert p.want_slice(2, False, solo_rates=[150.0, 70.0], solo_default=40.0, batched_rate=100.0)       # mean 110
    assert not p.want_slice(2, False, solo_rates=[150.0, 0.0], solo_default=40.0, batched_rate=100.0)    # mean 95
    assert p.want_slice(2, True, solo_rates=[150.0, 0.0], solo_default=42.0, batched_rate=100.0)         # mean 96, already slicing
    assert p.want_slice(3, False, solo_default=120.0, batched_rate=100.0)                                # nothing per conversation
    assert not p.want_slice(3, False, solo_default=0.0, batched_rate=100.0)
    # the joint step never measured: n rows per estimated step from the table of group times
    feed(p, 2, [10.0])   # a group of two rows takes 10 ms: 200 tokens/s together
    assert p.cost(2) == 10.0
    assert p.want_slice(2, False, sliced_rate=211.0) and not p.want_slice(2, False, sliced_rate=209.0)
    assert p.want_slice(2, True, sliced_rate=191.0) and not p.want_slice(2, True, sliced_rate=189.0)
    assert p.want_slice(3, False, sliced_rate=3e3 / p.cost(3) * 1.06) and not p.want_slice(3, False, sliced_rate=3e3 / p.cost(3) * 1.04)
    p.free()
