"""Exact check of the sampler's mechanics, by exhaustion.

A sampling step is a deterministic function of its uniforms and a uniform takes only 2^24 values, so the law of a
step's result under ONE of its draws can be counted exactly: run the oracle's step for every value of that draw and
compare the counts with what the prefix sums of the biases fix in exact arithmetic.  Nothing of the oracle's code is
restated here: the expectations are closed forms over f64 sums of the biases in the order the definition gives the
elements (all of lane 0's 16 biases, then lane 1's, ...; a lane's biases are quartet j = 0..3 of its group, element
0..3; quartets are aligned to the absolute CSR index).  A wrong element order, a transposed lane / quartet index, a
dropped head or tail element, an off-by-one in the group boundary or an inverted acceptance test all move the counts
by thousands; rounding in the f32 scan tree moves a boundary by a few units.

Reference semantics: the winner of a step is element i with probability w_i / sum w (include/sampler.cuh:26-44, :76).
"""
import numpy as np
import pytest

import fw_oracle_binding as orc

U24 = 1 << 24


def _definition_order(deg, off):
    """Local indices of a list's elements in the order the sampler's inverse transform runs through them, per group."""
    a0 = off & ~3
    nq = (off + deg - a0 + 3) // 4
    groups = []
    for g in range((nq + 255) // 256):
        order = []
        for lane in range(64):
            for j in range(4):
                k = g * 256 + j * 64 + lane
                for e in range(4):
                    i = a0 + 4 * k + e - off
                    if k < nq and 0 <= i < deg:
                        order.append(i)
        groups.append(np.array(order, dtype=np.int64))
    return groups


def _interval_counts(weights):
    """#{v in [0, 2^24) : P_{i-1} <= v * T / 2^24 < P_i} for the exact prefix sums P of `weights` (f64, exact here)."""
    P = np.concatenate([[0.0], np.cumsum(weights.astype(np.float64))])
    edges = np.ceil(P / P[-1] * U24).astype(np.int64)
    edges[-1] = U24
    return np.diff(edges)


def _biases(rng, deg, zero_fraction):
    # multiples of 2^-10 below 128: every partial sum of up to 4096 of them is exact in f64 (and in no way special in f32)
    b = (rng.randint(1, 1 << 17, size=deg) / 1024.0).astype(np.float32)
    b[rng.random_sample(deg) < zero_fraction] = 0.0
    return b


# one boundary moves by (f32 error of a prefix of <= 22 additions) / T * 2^24 plus the rounding of u * T
TOL = 12


def _check_pick_function(bias, off, order, nw, stream, index, seed, walker, step, n_points=3000):
    """The counts fix how many values of the draw give each element, not which: the pick as a function of the draw
    must run through the elements in the definition's order.  For sampled values v the step must return the element
    whose exact interval holds v * T / 2^24 (or a neighbour, within TOL of an interval's end)."""
    w = bias[order].astype(np.float64)
    P = np.concatenate([[0.0], np.cumsum(w)])
    edges = P / P[-1] * U24
    rng = np.random.RandomState(len(bias) + index)
    vs = np.concatenate([rng.randint(0, U24, size=n_points), [0, 1, U24 - 1, U24 // 2]])
    for v in vs.tolist():
        got = orc.sample_forced(bias, off, nw, stream, index, v / U24, seed=seed, walker=walker, step=step)
        lo = np.searchsorted(edges, v - TOL, side="right") - 1
        hi = np.searchsorted(edges, v + TOL, side="right") - 1
        allowed = {int(order[k]) for k in range(max(lo, 0), min(hi, len(order) - 1) + 1) if w[k] > 0}
        assert got in allowed, (v, got, sorted(allowed))


@pytest.mark.parametrize("deg,off,zero_fraction", [(1017, 3, 0.1), (333, 1, 0.0), (1024, 0, 0.3)])
def test_single_group_pick_is_the_inverse_transform(deg, off, zero_fraction):
    """Lists of one group: the pick is a function of the first draw alone."""
    rng = np.random.RandomState(deg + off)
    bias = _biases(rng, deg, zero_fraction)
    counts = orc.enumerate_draw(bias, off, nw=1, stream=0, index=0, seed=5)
    assert counts[0] == 0 and counts.sum() == U24
    got = counts[1:]
    assert (got[bias == 0] == 0).all()                       # a zero bias is never picked
    (order,) = _definition_order(deg, off)
    assert sorted(order.tolist()) == list(range(deg))        # the order covers the list exactly once
    want = np.zeros(deg, dtype=np.int64)
    want[order] = _interval_counts(bias[order])
    assert np.abs(got - want).max() <= TOL, np.abs(got - want).max()
    _check_pick_function(bias, off, order, 1, 0, 0, seed=5, walker=0, step=0)


def test_second_group_is_accepted_with_probability_of_its_share():
    """Two groups: group 1 replaces group 0's pick iff S_1 * u > S_0 for the jump uniform u (draw 1 of the wave's
    stream), i.e. for 2^24 * (1 - S_0 / S_1) of its values, up to rounding; inside either group the conditional law
    is untouched by the jump draw (its target is another draw)."""
    rng = np.random.RandomState(9)
    deg, off = 1500, 2
    bias = _biases(rng, deg, 0.1)
    g0, g1 = _definition_order(deg, off)
    assert len(g0) == 1024 - off and len(g1) == deg - len(g0)
    S0 = bias[g0].astype(np.float64).sum()
    S1 = S0 + bias[g1].astype(np.float64).sum()
    counts = orc.enumerate_draw(bias, off, nw=1, stream=0, index=1, seed=6, walker=3, step=2)
    assert counts[0] == 0 and counts.sum() == U24
    got = counts[1:]
    accepted = int(got[g1].sum())
    assert abs(accepted - U24 * (1.0 - S0 / S1)) <= 4
    # the targets inside the groups are fixed draws here: exactly one element of each group is ever returned
    assert (got[g0] > 0).sum() == 1 and (got[g1] > 0).sum() == 1


def test_second_group_target_follows_its_own_prefix_sums():
    """Two groups, enumerating the target draw of group 1 (draw 2 of the stream; it exists only when the jump draw
    accepted group 1, so a (walker, step) whose jump draw does is looked for first)."""
    rng = np.random.RandomState(10)
    deg, off = 2040, 1
    bias = _biases(rng, deg, 0.05)
    bias[:1023] *= np.float32(1.0 / 64.0)                    # group 1 carries nearly all the weight: accepted almost surely
    g0, g1 = _definition_order(deg, off)
    S0 = bias[g0].astype(np.float64).sum()
    S1 = S0 + bias[g1].astype(np.float64).sum()
    walker = next(w for w in range(64) if orc.uniform(7, w, 0, 0, 1) * S1 > S0 * 1.001)
    counts = orc.enumerate_draw(bias, off, nw=1, stream=0, index=2, seed=7, walker=walker, step=0)
    got = counts[1:]
    assert counts[0] == 0 and got[g0].sum() == 0             # group 1 always wins for this jump draw
    want = np.zeros(deg, dtype=np.int64)
    want[g1] = _interval_counts(bias[g1])
    assert np.abs(got - want).max() <= TOL
    _check_pick_function(bias, off, g1, 1, 0, 2, seed=7, walker=walker, step=0, n_points=1500)


def test_workgroup_combine_picks_a_wave_by_its_total():
    """Workgroup granularity with 4 waves over 8 groups: wave w owns groups w, w + 4.  The combine draw picks wave w
    for a share W_w / sum W of its values; every wave's own pick is fixed by other draws."""
    rng = np.random.RandomState(11)
    deg, off, nw = 8000, 0, 4
    bias = _biases(rng, deg, 0.1)
    groups = _definition_order(deg, off)
    assert len(groups) == 8
    W = np.array([sum(bias[groups[g]].astype(np.float64).sum() for g in range(w, 8, nw)) for w in range(nw)])
    counts = orc.enumerate_draw(bias, off, nw=nw, stream=orc.STREAM_WAVE, index=0, seed=8, walker=1, step=4)
    got = counts[1:]
    assert counts[0] == 0 and counts.sum() == U24
    want = _interval_counts(W)
    for w in range(nw):
        own = np.concatenate([groups[g] for g in range(w, 8, nw)])
        assert abs(int(got[own].sum()) - int(want[w])) <= TOL
        assert (got[own] > 0).sum() == 1                     # one fixed pick per wave
