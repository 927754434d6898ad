"""The generation loop and the adaptive draft depth (CPU): the controller against the reference's
own unit scenarios (crates/runtime/src/speculative_adaptive_tests.rs), on both the oracle's and
the library's implementation; the oracle's loop against the invariants speculative decoding
guarantees (greedy output == plain greedy decoding whatever the drafter proposes; exact budget;
stop tokens; a perfect drafter is always accepted)."""
import numpy as np
import pytest

from oracle import binding as ob
from tests.loop_common import LmDrafter, OracleTarget, TreeTwinDrafter


def _oracle_adaptive(floor, cap):
    return ob.Adaptive(floor, cap)


def _library_adaptive(floor, cap):
    from turbospark_amd import ffi
    return ffi.AdaptiveDepth(floor, cap)


def _tile_cap(make):
    if make is _oracle_adaptive:
        return ob.Adaptive.tile_cap
    from turbospark_amd import ffi
    return ffi.AdaptiveDepth.tile_cap


def _full(c, n):
    for _ in range(n):
        d = c.depth()
        c.observe(d, d)


@pytest.mark.parametrize("make", [_oracle_adaptive, _library_adaptive])
def test_adaptive_depth_reference_scenarios(make):
    # speculative_adaptive_tests.rs, scenario by scenario; thresholds 8 / 6 / 4, drop 2
    assert make(2, 8).depth() == 2
    assert make(4, 2).depth() == 2 and make(0, 0).depth() == 1
    c = make(3, 3)
    _full(c, 50)
    assert c.depth() == 3
    tc = _tile_cap(make)
    assert tc(8, 8) == 7 and tc(4, 8) == 4 and tc(8, None) == 8 and tc(8, 1) == 1
    c = make(2, tc(8, 8))
    _full(c, 200)
    assert c.depth() == 7
    # climbs after exactly the threshold streak
    c = make(2, 8)
    _full(c, 7)
    assert c.depth() == 2
    _full(c, 1)
    assert c.depth() == 3
    # a miss resets the streak
    c = make(2, 8)
    _full(c, 7)
    c.observe(2, 1)
    _full(c, 7)
    assert c.depth() == 2
    _full(c, 1)
    assert c.depth() == 3
    c = make(2, 5)
    _full(c, 500)
    assert c.depth() == 5
    # pressure drops one step and resets
    c = make(2, 8)
    _full(c, 500)
    assert c.depth() == 8
    c.observe(8, 7)
    assert c.depth() == 8
    c.observe(8, 7)
    assert c.depth() == 7
    c.observe(7, 6)
    assert c.depth() == 7
    # a total miss above the floor drops at once
    c = make(2, 8)
    _full(c, 500)
    c.observe(8, 0)
    assert c.depth() == 7
    # a full accept clears accumulated pressure
    c = make(2, 8)
    _full(c, 500)
    c.observe(8, 7)
    c.observe(8, 8)
    c.observe(8, 7)
    assert c.depth() == 8
    # no pressure builds at the floor
    c = make(2, 8)
    for _ in range(1000):
        c.observe(2, 0)
    assert c.depth() == 2
    _full(c, 8)
    assert c.depth() == 3
    c.observe(3, 2)
    assert c.depth() == 3
    # an empty round is not a signal
    c = make(2, 8)
    _full(c, 7)
    c.observe(0, 0)
    assert c.depth() == 2
    _full(c, 1)
    assert c.depth() == 3
    # accepted beyond offered is clamped
    c = make(2, 8)
    c.observe(2, 99)
    assert c.climb == 1
    # prose-like and every-eighth-miss streams stay at the floor
    c = make(2, 12)
    for r in range(600):
        c.observe(2, 1 if r % 4 == 3 else 2)
    assert c.depth() == 2
    c = make(2, 8)
    for r in range(800):
        c.observe(2, 1 if r % 8 == 7 else 2)
    assert c.depth() == 2
    # a perfect stream reaches the cap, a collapse returns to the floor
    c = make(2, 10)
    _full(c, 500)
    assert c.depth() == 10
    for _ in range(500):
        c.observe(c.depth(), 0)
    assert c.depth() == 2
    # the climb from each band takes 8, 8, 6, 4, 4 ... clean rounds
    c = make(2, 8)
    need = []
    while c.depth() < 8:
        d, n = c.depth(), 0
        while c.depth() == d:
            c.observe(d, d)
            n += 1
        need.append(n)
    assert need == [8, 8, 6, 4, 4, 4]


def test_the_two_controllers_walk_identically_on_a_random_stream():
    rng = np.random.default_rng(4)
    a, b = _oracle_adaptive(2, 9), _library_adaptive(2, 9)
    for _ in range(5000):
        d = a.depth()
        assert d == b.depth()
        acc = d if rng.random() < 0.8 else int(rng.integers(0, d + 1))
        off = d if rng.random() < 0.95 else 0
        a.observe(off, acc)
        b.observe(off, acc)
    assert a.climb == b.climb and a.pressure == b.pressure


# ---- the oracle's loop -------------------------------------------------------------------------
def _models(seed_target=1234, seed_draft=77, max_context=96):
    from turbospark_amd import synth
    cfg = dict(synth.CONFIGS["tiny_q8_0"])
    cfg.update(vocab=512, max_context=max_context, n_layers=1)
    wt = synth.make_weights(cfg, seed=seed_target)
    wd = wt if seed_draft is None else synth.make_weights(cfg, seed=seed_draft)
    return cfg, ob.Model(cfg, wt, threads=4), ob.Model(cfg, wd, threads=4)


def _plain_greedy(model, prompt, n_new, stop=()):
    model.reset()
    for i, t in enumerate(prompt[:-1]):
        model.verify([t], i)
    out, tok, pos = [], int(prompt[-1]), len(prompt) - 1
    for _ in range(n_new):
        row = model.verify([tok], pos)[0]
        tok = int(np.argmax(row.view(np.float16).astype(np.float32)))
        pos += 1
        if tok in stop:
            return out, 1
        out.append(tok)
    return out, 2


@pytest.mark.parametrize("seed_draft,block,floor", [(77, 4, 0), (None, 4, 0), (77, 1, 0), (None, 7, 2), (77, 15, 2)])
def test_greedy_speculation_equals_plain_greedy_decoding(seed_draft, block, floor):
    cfg, target, lm = _models(seed_draft=seed_draft)
    prompt = np.random.default_rng(1).integers(0, cfg["vocab"], 9).astype(np.int32)
    want, why = _plain_greedy(target, prompt, 40)
    drafter = LmDrafter(OracleTarget(lm), prompt[0], cfg["vocab"])
    got = ob.run_speculative(OracleTarget(target), drafter, prompt, ob.shaping(0.0), 40, block, cfg["vocab"],
                             cfg["max_context"], adaptive_floor=floor)
    assert got["tokens"] == want and got["stop_reason"] == 2 == why
    assert target.position == len(prompt) + 39      # every reported token but the last has a KV row
    if seed_draft is None:
        # the target drafting for itself is never wrong; only budget-shortened rounds offer less
        assert got["accepted"] == got["offered"] and got["rollbacks"] <= 1  # (the budget round keeps one row less)
        if floor:
            assert got["final_depth"] > floor
    else:
        assert got["accepted"] < got["offered"] and got["rollbacks"] > 0
    # a stop token ends the run before it is reported
    stop = want[17]
    first = want.index(stop)
    drafter = LmDrafter(OracleTarget(lm), prompt[0], cfg["vocab"])
    got = ob.run_speculative(OracleTarget(target), drafter, prompt, ob.shaping(0.0), 40, block, cfg["vocab"],
                             cfg["max_context"], stop_tokens=[stop], adaptive_floor=floor)
    assert got["tokens"] == want[:first] and got["stop_reason"] == 1


@pytest.mark.parametrize("nodes", [7, 15])
def test_greedy_tree_rounds_equal_plain_greedy_decoding(nodes):
    """speculative.rs:467-575: a drafter that offers trees of `block` nodes; the walk accepts the child
    that carries the target's pick, the accepted path is compacted, and what is reported is plain
    greedy decoding whatever the tree held.  The tree hides the true continuation behind junk siblings
    and cuts it at a seeded depth, so rounds accept anything from nothing to five nodes."""
    cfg, target, lm = _models(seed_draft=None)
    prompt = np.random.default_rng(2).integers(0, cfg["vocab"], 9).astype(np.int32)
    want, why = _plain_greedy(target, prompt, 40)
    drafter = TreeTwinDrafter(OracleTarget(lm), prompt[0], cfg["vocab"], nodes, seed=4)
    got = ob.run_speculative(OracleTarget(target), drafter, prompt, ob.shaping(0.0), 40, nodes, cfg["vocab"], cfg["max_context"])
    assert got["tokens"] == want and got["stop_reason"] == 2 == why
    assert target.position == len(prompt) + 39
    assert 0 < got["accepted"] < got["offered"] and got["rollbacks"] > 0 and got["rounds"] < 40
    stop = want[21]
    drafter = TreeTwinDrafter(OracleTarget(lm), prompt[0], cfg["vocab"], nodes, seed=4)
    got = ob.run_speculative(OracleTarget(target), drafter, prompt, ob.shaping(0.0), 40, nodes, cfg["vocab"], cfg["max_context"],
                             stop_tokens=[stop])
    assert got["tokens"] == want[:want.index(stop)] and got["stop_reason"] == 1
    # an adaptive run keeps the chain (speculative.rs:390-392): the drafter is then stepped, never asked for a tree
    drafter = TreeTwinDrafter(OracleTarget(lm), prompt[0], cfg["vocab"], nodes, seed=4)
    drafter.draft_tree = None
    got = ob.run_speculative(OracleTarget(target), drafter, prompt, ob.shaping(0.0), 40, nodes, cfg["vocab"], cfg["max_context"],
                             adaptive_floor=2)
    assert got["tokens"] == want


def test_the_loop_fills_the_context_window_exactly_and_refuses_past_it():
    cfg, target, lm = _models(seed_draft=None, max_context=40)
    prompt = np.arange(1, 11).astype(np.int32)
    drafter = LmDrafter(OracleTarget(lm), prompt[0], cfg["vocab"])
    got = ob.run_speculative(OracleTarget(target), drafter, prompt, ob.shaping(0.0), 30, 8, cfg["vocab"], 40)
    assert len(got["tokens"]) == 30 and got["stop_reason"] == 2
    want, _ = _plain_greedy(target, prompt, 30)
    assert got["tokens"] == want
    for bad in (dict(max_new=31), dict(max_new=0), dict(prompt=[])):
        with pytest.raises(ValueError):
            ob.run_speculative(OracleTarget(target), drafter, bad.get("prompt", prompt), ob.shaping(0.0),
                               bad.get("max_new", 30), 8, cfg["vocab"], 40)


def test_a_sampled_run_with_the_target_as_its_own_drafter_accepts_everything():
    """q == p at every position, so r * q(x) <= p(x) always holds: any misalignment of the
    drafter's positions, the history or the draw counter shows up as a rejection."""
    cfg, target, lm = _models(seed_draft=None)
    prompt = np.random.default_rng(2).integers(0, cfg["vocab"], 6).astype(np.int32)
    drafter = LmDrafter(OracleTarget(lm), prompt[0], cfg["vocab"])
    got = ob.run_speculative(OracleTarget(target), drafter, prompt, ob.shaping(0.9, seed=5, top_p=0.95), 33, 4,
                             cfg["vocab"], cfg["max_context"])
    assert got["accepted"] == got["offered"] and got["rollbacks"] <= 1 and len(got["tokens"]) == 33
    # draw counter: one per proposal, one per row-only step, one per acceptance test, one per bonus
    # draw -- the round the budget ends has no bonus (speculative.rs:396-402, 618-624, 861-879)
    assert got["draw_step"] == 2 * got["offered"] + 2 * got["rounds"] - 1
    # a poor drafter still reproduces: same seed, same stream
    cfg, target, lm = _models(seed_draft=77)
    runs = []
    for _ in range(2):
        drafter = LmDrafter(OracleTarget(lm), prompt[0], cfg["vocab"])
        runs.append(ob.run_speculative(OracleTarget(target), drafter, prompt, ob.shaping(0.9, seed=5), 25, 4,
                                       cfg["vocab"], cfg["max_context"]))
    assert runs[0] == runs[1] and runs[0]["accepted"] < runs[0]["offered"]
