"""The session pool's two selection rules on the host (crates/runtime/src/session_pool.rs:116-129), with the
reference's own unit scenarios (session_pool.rs:131-171) and the tie rules of the iterators it is written with."""
import ctypes as C

import numpy as np

from turbospark_amd import ffi


def best(scores):
    a = np.ascontiguousarray(scores, np.int64)
    out = C.c_int64(-7)
    idx = ffi.lib().tsv_session_best_match(C.c_void_p(a.ctypes.data) if a.size else None, a.size, C.byref(out))
    return (int(idx), int(out.value)) if idx >= 0 else None


def lru(ticks):
    a = np.ascontiguousarray(ticks, np.uint64)
    idx = ffi.lib().tsv_session_lru(C.c_void_p(a.ctypes.data) if a.size else None, a.size)
    return int(idx) if idx >= 0 else None


def test_the_reference_scenarios():
    assert best([3, 5, 2]) == (1, 5)             # the_highest_score_wins
    assert best([]) is None                      # an_empty_iterator_never_scores
    assert best([0, 0, 0]) is None               # an_all_zero_pool_offers_no_match
    assert best([0, 7, 0]) == (1, 7)             # a_lone_nonzero_score_wins_at_its_own_value
    assert lru([5, 1, 3]) == 1                   # the_oldest_tick_is_evicted
    assert lru([]) is None                       # an_empty_pool_has_no_lru


def test_ties_resolve_as_the_iterators_do():
    # Iterator::max_by_key returns the last maximum, Iterator::min_by_key the first minimum
    assert best([4, 9, 9, 1]) == (2, 9)
    assert lru([2, 0, 0, 5]) == 1
    assert best([1]) == (0, 1) and lru([0]) == 0
    assert lru([2 ** 63 + 5, 2 ** 63 + 4]) == 1  # ticks are unsigned
