"""The record of what the cache rows were built from (crates/runtime/src/kv_prefix.rs:49-137), held
to the reference's own unit scenarios (kv_prefix.rs:143-218).  Pure host state inside the C-ABI
library: no GPU is touched."""
from turbospark_amd.ffi import KvPrefix


def test_a_strict_prefix_reports_its_whole_length():
    assert KvPrefix([1, 2, 3]).common_prefix([1, 2, 3, 4]) == 3


def test_divergence_truncates_rather_than_refusing():
    assert KvPrefix([1, 2, 3, 9, 9]).common_prefix([1, 2, 3, 7, 7, 8]) == 3
    assert KvPrefix([1, 2, 3]).common_prefix([9, 2, 3, 4]) == 0


def test_at_least_one_token_is_always_left_to_feed():
    assert KvPrefix([1, 2, 3]).common_prefix([1, 2, 3]) == 2
    assert KvPrefix([1, 2, 3]).common_prefix([1, 2]) == 1
    assert KvPrefix([1]).common_prefix([1]) == 0


def test_taint_refuses_everything_and_only_clear_lifts_it():
    p = KvPrefix([1, 2, 3])
    p.taint()
    p.record([4], 3)
    assert p.common_prefix([1, 2, 3, 4, 5]) == 0 and p.untainted_len() is None
    p.clear()
    p.record([1, 2, 3], 0)
    assert p.common_prefix([1, 2, 3, 4]) == 3 and p.untainted_len() == 3


def test_a_gap_in_the_positions_taints_rather_than_claiming_coverage():
    p = KvPrefix([1, 2, 3])
    p.record([9], 5)
    assert p.common_prefix([1, 2, 3, 9, 0, 0, 7]) == 0 and p.untainted_len() is None


def test_re_recording_over_the_same_span_replaces_it():
    p = KvPrefix([1, 2, 3])
    p.record([7, 8], 1)
    assert p.common_prefix([1, 7, 8, 4]) == 3 and p.untainted_len() == 3


def test_a_rewind_shortens_what_is_reusable():
    p = KvPrefix([1, 2, 3, 4])
    p.rewind_to(2)
    assert p.common_prefix([1, 2, 3, 4]) == 2
    p.rewind_to(99)
    assert p.common_prefix([1, 2, 3, 4]) == 2


def test_an_empty_record_reuses_nothing():
    assert KvPrefix().common_prefix([1, 2, 3]) == 0
    assert KvPrefix([1, 2, 3]).common_prefix([]) == 0


def test_token_by_token_recording_matches_a_block_and_a_brute_force_prefix():
    import numpy as np
    rng = np.random.default_rng(11)
    for _ in range(200):
        a = rng.integers(0, 3, rng.integers(0, 12)).tolist()
        b = rng.integers(0, 3, rng.integers(0, 12)).tolist()
        p, q = KvPrefix(), KvPrefix()
        p.record(a, 0)
        for i, t in enumerate(a):
            q.record([t], i)
        lcp = 0
        while lcp < min(len(a), len(b)) and a[lcp] == b[lcp]:
            lcp += 1
        want = 0 if not a or not b else min(lcp, len(b) - 1)
        assert p.common_prefix(b) == q.common_prefix(b) == want
