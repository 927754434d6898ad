"""The allocation-free greedy acceptance entry point (tsv_accept_greedy_noalloc: logits, result and
stream are the caller's, the partial results live in a static device array) against tsv_accept on the
same logits: every integer equal, on two calls in a row, the second smaller than the first."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _planted(rng, m, vocab, parent, hits):
    """Random fp16 logits and a feed whose first `hits` proposals along slot order are the rows' arg-max."""
    logits = rng.standard_normal((m, vocab)).astype(np.float16)
    logits[:, vocab // 2] = logits[:, vocab - 1]          # ties somewhere in every row
    amax = logits.astype(np.float32).argmax(axis=1)
    feed = rng.integers(0, vocab, m).astype(np.int32)
    at = 0
    for _ in range(hits):
        kids = [s for s in range(1, m) if (parent[s] if parent is not None else s - 1) == at]
        if not kids:
            break
        pick = kids[-1] if len(kids) > 1 else kids[0]     # not the first child: the walk has to look
        feed[pick] = amax[at]
        at = pick
    return logits, feed


def _noalloc(logits, feed, parent, base, stops, generated, budget, stream=None):
    from turbospark_amd import ffi, hip
    m, vocab = logits.shape
    dev = hip.DeviceBuffer(logits.nbytes).upload(np.ascontiguousarray(logits.view(np.uint16)))
    out_dev = hip.DeviceBuffer(C.sizeof(ffi.RoundResultC))
    feed = np.ascontiguousarray(feed, np.int32)
    par = np.ascontiguousarray(parent, np.int32) if parent is not None else None
    st = np.ascontiguousarray(stops, np.int32)
    ffi.check(ffi.lib().tsv_accept_greedy_noalloc(stream, dev.ptr, vocab, feed.ctypes.data,
                                                  par.ctypes.data if par is not None else None, m, base,
                                                  st.ctypes.data if st.size else None, st.size, generated, budget, out_dev.ptr))
    hip.check(hip.rt().hipStreamSynchronize(C.c_void_p(stream)), "sync")
    out = ffi.RoundResultC()
    hip.check(hip.rt().hipMemcpy(C.byref(out), out_dev.ptr, C.sizeof(out), 2), "copy back")
    return out


CASES = [  # (rows, tree, planted hits, stop at hit, budget slack): the second and fourth are smaller than their predecessors
    (16, True, 3, None, 0), (5, False, 2, None, 0), (9, False, 8, 2, 0), (3, True, 1, None, 1), (1, False, 0, None, 0),
]
TREE16 = [-1, 0, 0, 0, 0, 1, 5, 6, 2, 8, 9, 3, 11, 12, 4, 14]


@pytest.mark.parametrize("vocab", [4096, 1000])
def test_the_allocation_free_greedy_round_equals_tsv_accept(vocab):
    import turbospark_amd as ts
    from turbospark_amd import synth
    cfg = dict(synth.CONFIGS["tiny_q8_0"], max_context=64, vocab=vocab)
    gpu = ts.HipVerifier(cfg, synth.make_weights(cfg, seed=5))
    rng = np.random.default_rng(vocab)
    base = 7
    for case, (m, tree, hits, stop_at, slack) in enumerate(CASES):
        parent = TREE16[:m] if tree else None
        logits, feed = _planted(rng, m, vocab, parent, hits)
        amax = logits.astype(np.float32).argmax(axis=1)
        stops = [int(amax[stop_at])] if stop_at is not None else []
        generated, budget = 10, (10 + slack if slack else 0)
        gpu.write_logits(logits, base)
        want = gpu.accept(feed, base, ts.shaping(0.0), parent=parent, stop_tokens=stops, generated=generated,
                          max_new_tokens=budget)
        got = _noalloc(logits, feed, parent, base, stops, generated, budget, stream=gpu.stream if case % 2 else None)
        assert (got.accepted, got.committed, got.next, got.stopped, got.path_len, got.kv_position) == \
            (want.accepted, want.committed, want.next, want.stopped, len(want.path), want.kv_position), (case, want)
        assert list(got.path[: got.path_len]) == want.path
        if hits and stop_at is None and not slack:
            assert got.accepted >= 1
    # a non-finite logit is reported in band (no host round trip to refuse through)
    logits, feed = _planted(rng, 4, vocab, None, 1)
    logits[2, 17] = np.float16(np.inf)
    bad = _noalloc(logits, feed, None, base, [], 0, 0)
    assert bad.stopped == -1 and bad.next == -1 and bad.path_len == 0
    # the next call starts from a clear flag
    logits[2, 17] = np.float16(0.5)
    gpu.write_logits(logits, base)
    want = gpu.accept(feed, base, ts.shaping(0.0))
    good = _noalloc(logits, feed, None, base, [], 0, 0)
    assert (good.accepted, good.next, good.stopped) == (want.accepted, want.next, 0)


def test_the_entry_point_captured_into_a_graph_replays_like_the_eager_round():
    """The call recorded once into a HIP graph on a stream of the caller's own (a handle was opened first, so the
    scratch address is known and the call makes no runtime query), then replayed three times with the program's own
    eager work and synchronizations between the replays and new logits in the same device buffer each time: every
    replay equals tsv_accept on those logits."""
    import turbospark_amd as ts
    from turbospark_amd import ffi, hip, synth
    vocab, m, base = 4096, 6, 11
    cfg = dict(synth.CONFIGS["tiny_q8_0"], max_context=64, vocab=vocab)
    gpu = ts.HipVerifier(cfg, synth.make_weights(cfg, seed=5))
    rng = np.random.default_rng(77)
    dev = hip.DeviceBuffer(m * vocab * 2)
    out_dev = hip.DeviceBuffer(C.sizeof(ffi.RoundResultC))
    # the graph bakes the host arguments in (feed, tree, limits): the proposals stay, the logits change
    feed = rng.integers(0, vocab, m).astype(np.int32)
    stream = hip.Stream()

    def record(s):
        ffi.check(ffi.lib().tsv_accept_greedy_noalloc(s.h, dev.ptr, vocab, feed.ctypes.data, None, m, base, None, 0, 0, 0,
                                                      out_dev.ptr))
    graph = hip.CapturedGraph(stream, record)
    outcomes = set()
    for replay in range(3):
        logits = rng.standard_normal((m, vocab)).astype(np.float16)
        for row in range(replay + 1):                      # the first rows' arg-max is the next proposal: 1, 2, 3 hits
            logits[row, feed[row + 1]] = np.float16(9.0)
        gpu.write_logits(logits, base)                     # eager work on another stream, and its synchronization
        want = gpu.accept(feed, base, ts.shaping(0.0))
        dev.upload(np.ascontiguousarray(logits.view(np.uint16)))
        graph.launch()
        stream.sync()
        got = ffi.RoundResultC()
        hip.check(hip.rt().hipMemcpy(C.byref(got), out_dev.ptr, C.sizeof(got), 2), "copy back")
        assert (got.accepted, got.committed, got.next, got.stopped, got.kv_position) == \
            (want.accepted, want.committed, want.next, want.stopped, want.kv_position), (replay, want)
        outcomes.add(got.accepted)
    assert len(outcomes) == 3                              # the replays really judged different logits


def test_sizes_beyond_the_static_scratch_are_refused_by_name():
    from turbospark_amd import ffi, hip
    buf = hip.DeviceBuffer(1 << 16)
    feed = np.zeros(32, np.int32)
    rc = ffi.lib().tsv_accept_greedy_noalloc(None, buf.ptr, 64, feed.ctypes.data, None, 17, 0, None, 0, 0, 0, buf.ptr)
    assert rc != 0 and "16 rows" in ffi.last_error()
    rc = ffi.lib().tsv_accept_greedy_noalloc(None, None, 64, feed.ctypes.data, None, 4, 0, None, 0, 0, 0, buf.ptr)
    assert rc != 0 and "null" in ffi.last_error()
