"""How many walk launches a sampled tree round is given: the bound the library computes from the parent array
against a brute-force walk of every accept / reject outcome (the walk rule: children of the current node are tested in
slot order; an accepted child becomes the current node, a rejected one is skipped; the walk ends when the current
node has no untested child left)."""
import ctypes as C

import numpy as np

from turbospark_amd import ffi


def bound(parent):
    a = np.ascontiguousarray(parent, np.int32)
    return int(ffi.lib().tsv_tree_walk_bound(C.c_void_p(a.ctypes.data), a.size))


def brute(parent):
    m = len(parent)
    kids = [[c for c in range(1, m) if parent[c] == n] for n in range(m)]

    def worst(node, start):   # most tests from `node` on, its children from position `start` still untested
        if start >= len(kids[node]):
            return 0
        c = kids[node][start]
        return 1 + max(worst(c, 0),            # accepted: go on below c
                       worst(node, start + 1))  # rejected: the next sibling
    return worst(0, 0)


def test_known_shapes():
    assert bound([-1]) == 0
    assert bound([-1, 0, 1, 2, 3]) == 4                                      # a chain: one test per level
    assert bound([-1, 0, 0, 0, 0]) == 4                                      # a star: every child may be rejected
    assert bound([-1, 0, 0, 0, 0, 1, 5, 6, 2, 8, 9, 3, 11, 12, 4, 14]) == 6  # a root with four chains
    assert bound([-1] + list(range(15))) == 15                               # the longest chain a pass takes
    assert bound([-1] + [0] * 15) == 15


def test_every_tree_of_up_to_seven_slots_and_random_larger_ones():
    def trees(m):
        if m == 1:
            yield [-1]
            return
        for t in trees(m - 1):
            for p in range(m - 1):
                yield t + [p]
    n = 0
    for m in range(1, 8):
        for t in trees(m):
            assert bound(t) == brute(t), t
            n += 1
    assert n == 1 + 1 + 2 + 6 + 24 + 120 + 720
    rng = np.random.default_rng(3)
    for _ in range(3000):
        m = int(rng.integers(8, 17))
        # mixtures of bushy and deep trees: the parent is drawn from the last few slots or from all of them
        t = [-1] + [int(rng.integers(max(0, s - int(rng.integers(1, 4))), s)) if rng.integers(0, 2) else int(rng.integers(0, s))
                    for s in range(1, m)]
        assert bound(t) == brute(t) <= m - 1, t


def test_malformed_trees_are_refused():
    assert bound([0, 0, 1]) == -1
    assert bound([-1, 0, 2]) == -1
    assert bound([-1, -1]) == -1
    assert bound([-1] + list(range(16))) == -1   # seventeen slots
