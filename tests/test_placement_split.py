"""The rule that tells the device's memory groups apart (morphserve_amd/csrc/vmm_arena.hip::split_by_rate,
used by mkv_arena_pair_grow; no counterpart in the reference, whose pool is two torch.zeros calls,
MorphServe/worker/model.py:187-190).  Runs on the CPU: the rule is host code, reached through the diagnostic
library, and the rates are a recording from one MI355X (tests/golden/group_probe_rates.json)."""
import ctypes as C
import json
import os

import numpy as np
import pytest

from morphserve_amd import _capi

HERE = os.path.dirname(os.path.abspath(__file__))


def split(rates, self_rate):
    rates = np.ascontiguousarray(rates, dtype=np.float64)
    same = np.zeros(len(rates), dtype=np.uint8)
    _capi.check(_capi.diag_lib().mkv_diag_split_by_rate(
        rates.ctypes.data_as(C.POINTER(C.c_double)), len(rates), float(self_rate),
        same.ctypes.data_as(C.POINTER(C.c_uint8))))
    return same.astype(bool)


@pytest.fixture(scope="module")
def recorded():
    with open(os.path.join(HERE, "golden", "group_probe_rates.json")) as f:
        return json.load(f)["sets"]


def _truth(s):
    """A chunk's group = the anchor it fills slowest beside (every chunk lies in exactly one group)."""
    return np.argmin(np.asarray(s["vs_anchor"], dtype=np.float64), axis=0)


def test_recorded_sets_split_without_error(recorded):
    """256-286 chunks per set, fresh memory and memory recycled in shuffled order: the gap between the two kinds of
    rate is as narrow as 6 % there, which is what a rule that looks for one wide step between neighbours misses."""
    for s in recorded:
        truth = _truth(s)
        for a in range(3):
            rates = np.asarray(s["vs_anchor"][a], dtype=np.float64)
            same = split(rates, s["self"][s["anchors"][a]])
            assert np.array_equal(same, truth == a), (s["name"], a)
            srt = np.sort(rates)
            assert (srt[1:] / srt[:-1]).max() < 1.12          # no step a fixed 12 % test would find


def test_second_stage_separates_the_other_two_groups(recorded):
    for s in recorded:
        truth = _truth(s)
        others = np.flatnonzero(truth != 0)                   # what the first anchor called "another group"
        rates = np.asarray(s["vs_anchor"][1], dtype=np.float64)[others]
        same = split(rates, s["self"][s["anchors"][1]])
        assert np.array_equal(same, truth[others] == 1), s["name"]


def test_one_kind_only_is_recognised(recorded):
    """Only chunks of the anchor's group, or only chunks of other groups: no cut, the anchor's own rate decides."""
    for s in recorded:
        truth = _truth(s)
        rates = np.asarray(s["vs_anchor"][0], dtype=np.float64)
        self_rate = s["self"][s["anchors"][0]]
        assert split(rates[truth == 0], self_rate).all(), s["name"]
        assert not split(rates[truth != 0], self_rate).any(), s["name"]


def test_small_samples(recorded):
    """A later growth measures a handful of chunks: random subsets of 2 ... 16 of the recorded rates."""
    rng = np.random.default_rng(3)
    wrong = trials = 0
    for s in recorded:
        truth = _truth(s)
        rates = np.asarray(s["vs_anchor"][0], dtype=np.float64)
        self_rate = s["self"][s["anchors"][0]]
        for n in (2, 3, 4, 8, 16):
            for _ in range(200):
                idx = rng.choice(len(rates), size=n, replace=False)
                wrong += not np.array_equal(split(rates[idx], self_rate), truth[idx] == 0)
                trials += 1
    assert wrong <= 0.02 * trials, (wrong, trials)


def test_edge_cases():
    assert split([], 5000.0).size == 0
    assert split([5100.0], 5000.0).all()                      # one chunk, as fast as the anchor's own halves
    assert not split([6800.0], 5000.0).any()                  # one chunk, a third faster
    assert list(split([5000.0, 6800.0, 5200.0, 6700.0], 5100.0)) == [True, False, True, False]
