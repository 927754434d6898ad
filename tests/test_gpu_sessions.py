"""The session pool behind the handle (crates/runtime/src/session_pool.rs; RealForwardRunner::select_session,
swap_live_session and reset, real_forward_traits.rs:12-31,173-289,655-724): several conversations' KV state kept
side by side, swapped by pointer, chosen by the longest common prefix.  A swap must never change what is computed:
a conversation taken back out of the pool continues, by bits, as on a handle that never saw another one."""
import os

import numpy as np
import pytest

import turbospark_amd as ts
from turbospark_amd import synth

pytestmark = pytest.mark.gpu


def _open(name="tiny_q8_0", slots=2, kv_bits=None, max_context=160, ring=False, **over):
    cfg = dict(synth.CONFIGS[name], max_context=max_context, **over)
    w = synth.make_weights(cfg, seed=77)
    if ring:   # the windowed layers keep rings (and the handle a finite rewind budget): they are swapped like the rest
        for lw in w["layers"]:
            lw["ring"] = 1 if lw.get("window", 0) else 0
    g = ts.HipVerifier(cfg, w, kv_bits=kv_bits, session_slots=slots)
    g.set_prefix_reuse(True)
    return cfg, w, g


def _ids(cfg, n, seed):
    return np.random.default_rng(seed).integers(0, cfg["vocab"], n).astype(np.int32)


def _fresh_continuation(cfg, w, prompt, feed, kv_bits=None):
    ref = ts.HipVerifier(cfg, w, kv_bits=kv_bits)
    ref.prefill(prompt, 0, want_logits=False)
    return ref.verify(feed, len(prompt))


@pytest.mark.parametrize("name,kv_bits,layers,ring", [("tiny_q8_0", None, 2, False), ("small_q4_k", (3, 4), 3, False),
                                                      ("gptoss_small", None, 2, False), ("gptoss_small", None, 2, True)])
def test_two_conversations_alternate_without_losing_each_other(name, kv_bits, layers, ring):
    cfg, w, g = _open(name, 2, kv_bits, ring=ring, n_layers=layers)
    assert g.session_pool_size == 2
    a, b = _ids(cfg, 40, 1), _ids(cfg, 33, 2)
    feed_a, feed_b = _ids(cfg, 5, 3), _ids(cfg, 4, 4)
    # turn 1 of A, then B arrives: nothing matches, the caller resets -- A is parked, not overwritten
    g.reset()
    g.prefill(a, 0, want_logits=False)
    assert g.try_reuse_prefix(np.concatenate([b, feed_b])) == 0 and g.position == 40
    g.reset()
    assert g.position == 0 and not g.session_slot_evicted
    g.prefill(b, 0, want_logits=False)
    # A comes back: the pool hands its state over and it goes on as if B had never been here
    assert g.try_reuse_prefix(np.concatenate([a, feed_a])) == 40
    assert g.position == 40 and g.prefix_len() == 40 and ts.ffi.lib().tsv_session_swapped(g._h) == 1
    assert np.array_equal(g.verify(feed_a, 40), _fresh_continuation(cfg, w, a, feed_a, kv_bits))
    g.record_committed(feed_a, 40)
    # and B likewise, from where it stood
    assert g.try_reuse_prefix(np.concatenate([b, feed_b])) == 33 and g.position == 33
    assert np.array_equal(g.verify(feed_b, 33), _fresh_continuation(cfg, w, b, feed_b, kv_bits))
    # A again, now five rows longer
    longer = np.concatenate([a, feed_a, _ids(cfg, 3, 5)])
    assert g.try_reuse_prefix(longer) == 45 and g.position == 45 and ts.ffi.lib().tsv_session_swapped(g._h) == 1
    assert g.try_reuse_prefix(longer) == 45 and ts.ffi.lib().tsv_session_swapped(g._h) == 0   # already live


def test_a_full_pool_evicts_the_least_recently_used_conversation():
    cfg, w, g = _open(slots=2)
    a, b, c = _ids(cfg, 30, 1), _ids(cfg, 30, 2), _ids(cfg, 30, 3)
    g.reset()
    g.prefill(a, 0, want_logits=False)
    g.reset()                                   # A parked in the slot nobody had used
    assert not g.session_slot_evicted
    g.prefill(b, 0, want_logits=False)
    g.reset()                                   # B parked, A -- the only other slot -- promoted and overwritten
    assert g.session_slot_evicted and g.position == 0
    g.prefill(c, 0, want_logits=False)
    assert g.try_reuse_prefix(np.concatenate([a, a[:3]])) == 0 and g.position == 30   # A is gone, C stays live
    assert g.try_reuse_prefix(np.concatenate([b, b[:3]])) == 30                      # B is still there
    # three slots keep all three
    cfg, w, g = _open(slots=3)
    for ids in (a, b, c):
        g.reset()
        assert not g.session_slot_evicted
        g.prefill(ids, 0, want_logits=False)
    for ids in (a, b, c, a):
        assert g.try_reuse_prefix(np.concatenate([ids, ids[:2]])) == 30
    # a reset with nothing live parks nothing
    g.reset()
    g.reset()
    assert not g.session_slot_evicted


def test_ties_stay_live_and_shallow_matches_on_an_unvetted_live_session_are_refused():
    """session_pool.rs:116-121 (an all-zero pool offers nothing), real_forward_traits.rs:664-668 (a tie favours the
    live session) and :283 (with a pool, a rewind deeper than what it keeps would overwrite the live conversation in
    place instead of parking it)."""
    cfg, w, g = _open(slots=2)
    x = _ids(cfg, 40, 1)
    g.reset()
    g.prefill(x, 0, want_logits=False)
    shallow = np.concatenate([x[:5], _ids(cfg, 30, 9)])
    assert g.try_reuse_prefix(shallow) == 0 and g.position == 40          # back 35 > keep 5: refused, nothing moved
    deep = np.concatenate([x[:25], _ids(cfg, 10, 8)])
    assert g.try_reuse_prefix(deep) == 25 and g.position == 25            # back 15 <= keep 25: an ordinary rewind
    # without a pool the shallow rewind is harmless and taken
    cfg, w, solo = _open(slots=1)
    assert solo.session_pool_size == 1
    solo.reset()
    solo.prefill(x, 0, want_logits=False)
    assert solo.try_reuse_prefix(shallow) == 5 and solo.position == 5
    # a parked conversation that matches exactly as far as the live one does not displace it
    cfg, w, g = _open(slots=2)
    g.reset()
    g.prefill(x[:20], 0, want_logits=False)
    g.reset()
    g.prefill(np.concatenate([x[:20], _ids(cfg, 6, 4)]), 0, want_logits=False)
    assert g.try_reuse_prefix(np.concatenate([x[:20], _ids(cfg, 5, 6)])) == 20
    assert g.position == 20 and g.prefix_len() == 20
    # ... the parked twenty-row one is still parked: a prompt only it explains brings it in
    # (the live one was cut back to the same twenty rows, so this is again a tie and nothing swaps)
    assert g.try_reuse_prefix(x[:21]) == 20


def test_tree_rounds_after_a_swap_use_the_swapped_buffers():
    cfg, w, g = _open("small_q4_k", 2, None, n_layers=2)
    a, b = _ids(cfg, 37, 1), _ids(cfg, 20, 2)
    feed = _ids(cfg, 16, 3)
    parent = [-1, 0, 0, 0, 0, 1, 5, 6, 2, 8, 9, 3, 11, 12, 4, 14]
    path = [0, 2, 8, 9]
    g.reset()
    g.prefill(a, 0, want_logits=False)
    g.reset()
    g.prefill(b, 0, want_logits=False)
    assert g.try_reuse_prefix(np.concatenate([a, feed[:1]])) == 37
    point = g.checkpoint()
    g.verify_tree(feed, parent, 37)
    g.compact_tree(37, path)
    g.rollback_retaining(point, 4)
    got = g.produce(int(feed[10]), 41)
    ref = ts.HipVerifier(cfg, w)
    ref.prefill(a, 0, want_logits=False)
    p2 = ref.checkpoint()
    ref.verify_tree(feed, parent, 37)
    ref.compact_tree(37, path)
    ref.rollback_retaining(p2, 4)
    assert np.array_equal(got, ref.produce(int(feed[10]), 41))
    for layer in range(2):
        (ka, va), (kb, vb) = g.read_kv(layer, 0, 42), ref.read_kv(layer, 0, 42)
        assert np.array_equal(ka.view(np.uint16), kb.view(np.uint16)) and np.array_equal(va.view(np.uint16), vb.view(np.uint16))


def test_what_a_pool_refuses():
    cfg, w, _ = _open(slots=1)
    with pytest.raises(ts.ffi.TsvError, match="session slots"):
        ts.HipVerifier(cfg, w, session_slots=65)
    os.environ["TSV_GRAPH"] = "1"
    try:
        with pytest.raises(ts.ffi.TsvError, match="session pool"):
            ts.HipVerifier(cfg, w, session_slots=2)
    finally:
        del os.environ["TSV_GRAPH"]


def test_the_loop_with_a_pool_keeps_both_conversations_and_generates_what_a_fresh_handle_generates():
    """speculative.rs:240-251 with real_forward_traits.rs:199-239: the loop's drafter holds context of its own, so a
    conversation swapped in from the pool is not continued from -- the loop starts over (which parks what was live) --
    while a plain second turn of the live conversation still is.  Either way the tokens are those of a handle that
    never saw anything else."""
    from tests.loop_common import GpuTarget, LmDrafter

    class ContinuingDrafter(LmDrafter):
        def context_position(self):
            return self.pos - 1

    cfg, w, g = _open(slots=2, max_context=256)
    V = cfg["vocab"]
    lm = ts.HipVerifier(cfg, w)
    shaping = ts.shaping(0.0)
    a, b = _ids(cfg, 14, 1), _ids(cfg, 11, 2)
    da = ContinuingDrafter(GpuTarget(lm), a[0], V, 0.5, 9)
    one = g.run_speculative(a, da, shaping, 16, 4)
    held = one["kv_position"]
    # the same conversation goes on: a pure continuation
    a2 = np.concatenate([a, np.asarray(one["tokens"][: held - len(a)], np.int32), _ids(cfg, 5, 3)])
    two = g.run_speculative(a2, da, shaping, 16, 4)
    assert two["reused"] == held
    # another conversation: nothing matches, the loop resets, A is parked
    lm_b = ts.HipVerifier(cfg, w)
    db = ContinuingDrafter(GpuTarget(lm_b), b[0], V, 0.5, 9)
    other = g.run_speculative(b, db, shaping, 16, 4)
    assert other["reused"] == 0 and not g.session_slot_evicted
    # A's third turn: the pool has its rows, the drafter does not -- the loop starts over
    a3 = np.concatenate([a2, np.asarray(two["tokens"][: two["kv_position"] - len(a2)], np.int32), _ids(cfg, 4, 5)])
    da3 = ContinuingDrafter(GpuTarget(lm), a3[0], V, 0.5, 9)
    three = g.run_speculative(a3, da3, shaping, 16, 4)
    assert three["reused"] == 0
    fresh = ts.HipVerifier(cfg, w)
    fresh.set_prefix_reuse(True)
    base = fresh.run_speculative(a3, ContinuingDrafter(GpuTarget(ts.HipVerifier(cfg, w)), a3[0], V, 0.5, 9), shaping, 16, 4)
    for key in ("tokens", "stop_reason", "rounds", "offered", "accepted", "kv_position"):
        assert three[key] == base[key], key
    # that start-over re-parked the conversation the pool had just handed out and promoted the other slot: the
    # cascade the reference describes for installs with a drafter (real_forward_traits.rs:268-281)
    assert g.session_slot_evicted
    # the new conversation's own rows explain its transcript: no swap
    assert g.try_reuse_prefix(np.concatenate([a2, a2[:1]])) == len(a2)
    assert ts.ffi.lib().tsv_session_swapped(g._h) == 0
