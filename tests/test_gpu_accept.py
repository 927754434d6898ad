"""GPU parity of device-side acceptance (+ KV truncation) against the oracle's restatement of
the host half of a round (crates/runtime/src/speculative.rs:694-754, 861-879, 494-550).

The oracle judges the SAME fp16 logits the GPU pass produced (copied back), so every integer
output -- accepted count, committed count, corrected/bonus token, draw counter, rolled-back KV
length -- must match exactly."""
import numpy as np
import pytest

from oracle import binding as ob
from tests import gpu_common as gc

pytestmark = pytest.mark.gpu


def _setup(name="tiny_q8_0", ctx=40, max_context=256):
    import turbospark_amd as ts
    cfg, w, gpu, cpu = gc.build_pair(name, max_context=max_context)
    prompt = np.random.default_rng(5).integers(0, cfg["vocab"], ctx).astype(np.int32)
    gpu.prefill(prompt, 0, want_logits=False)
    return cfg, gpu, prompt


def _same(res, want, base):
    assert (res.accepted, res.committed, res.next, res.stopped, res.draw_step) == \
        (want["accepted"], want["committed"], want["next"], want["stopped"], want["draw_step"]), (res, want)
    assert res.kv_position == base + want["committed"] + 1


TRUNCATIONS = [dict(), dict(top_k=40), dict(top_p=0.9), dict(min_p=0.02), dict(top_k=50, top_p=0.95, min_p=0.01),
               dict(top_k=1), dict(top_p=0.3), dict(top_k=256, top_p=0.999)]


@pytest.mark.parametrize("temperature,kw", [(0.8, TRUNCATIONS[0]), (1.0, TRUNCATIONS[0]), (0.3, TRUNCATIONS[0])] +
                         [(0.8, t) for t in TRUNCATIONS[1:]] + [(1.3, TRUNCATIONS[4])])
def test_sampled_chain_rounds_match_the_oracle_bit_for_bit(temperature, kw):
    import turbospark_amd as ts
    cfg, gpu, prompt = _setup()
    V, k = cfg["vocab"], 4
    rng = np.random.default_rng(11)
    base = len(prompt) - 1
    history = list(prompt)
    point = gpu.checkpoint()
    gpu.rollback_retaining(point, 0)
    gpu.rollback(ts.ffi.Point(base))       # cursor to the position of the last prompt token
    margins, accepted_hist = [], []
    draw_step = 0
    nxt = int(prompt[-1])
    history = history[:-1]
    for rnd in range(24):
        seed = 1000 + rnd
        gcfg = ts.shaping(temperature, seed=seed, **kw)
        ocfg = ob.shaping(temperature, seed=seed, **kw)
        draft = rng.standard_normal((k, V)).astype(np.float16)
        if rnd % 3 == 0:
            draft[0, :] = 0  # a flat drafter row
        if rnd % 4 == 1:
            draft[1] = np.round(draft[1] * 2) / 2  # many equal logits: the cut falls inside a rank bin
        if rnd % 2 == 1:
            # a drafter that resembles the target: its row i is the target's own row after the first i
            # proposals, plus noise, so that truncated candidate sets overlap and proposals get accepted
            here = gpu.checkpoint()
            tok = nxt
            for i in range(k):
                row = gc.f16(gpu.produce(tok, gpu.position))
                draft[i] = (row + rng.standard_normal(V) * 0.3).astype(np.float16)
                one, _ = gpu.draft_chain(draft[i:i + 1], gcfg, draw_step + i)
                tok = int(one[0])
            gpu.rollback(here)
        # draft half on the device vs the oracle
        props, ds1 = gpu.draft_chain(draft, gcfg, draw_step)
        oprops, ods1 = ob.draft_chain(draft, ocfg, history + [nxt], len(history), draw_step)
        assert list(props) == list(oprops) and ds1 == ods1
        feed = [nxt] + [int(t) for t in props]
        base = gpu.position
        res, logits = gpu.verify_accept(feed, base, gcfg, draft_logits=draft, draw_step=ds1, want_logits=True)
        want = ob.chain_round(logits, draft, props, ocfg, history=history + [nxt], generated=0, draw_step=ds1)
        _same(res, want, base)
        assert res.path == list(range(want["accepted"] + 1))
        margins.append(res.min_margin)
        accepted_hist.append(res.accepted)
        history = history + feed[: 1 + want["committed"]]
        nxt = want["next"]
        draw_step = want["draw_step"]
        assert gpu.position == len(history)
    print("accepted per round:", accepted_hist, " min margin:", min(margins))
    assert min(margins) > 1e-9          # no decision was anywhere near flipping
    if kw.get("top_k") != 1:
        assert len(set(accepted_hist)) > 1  # the rounds really exercised different outcomes


PENALTIES = [dict(repetition_penalty=1.3), dict(presence_penalty=0.6, frequency_penalty=0.25),
             dict(repetition_penalty=1.2, presence_penalty=0.4, frequency_penalty=0.1, top_k=50, top_p=0.95, min_p=0.01),
             dict(repetition_penalty=0.7, top_p=0.9), dict(repetition_penalty=1.15, top_k=40),
             dict(repetition_penalty=1.1, min_p=0.02), dict(presence_penalty=2.0, top_p=0.6),
             dict(frequency_penalty=0.5, top_k=8)]


@pytest.mark.parametrize("dense", [False, True])
@pytest.mark.parametrize("kw", PENALTIES)
def test_penalised_chain_rounds_match_the_oracle_bit_for_bit(kw, dense):
    """Repetition / presence / frequency penalties (crates/selection/src/penalty.rs:15-82) in the draft
    draws and in the acceptance of a sampled chain round: each target row is shaped with the history
    a sequential decode would have had there (the proposals accepted before it included).  `dense`
    hands over a long synthetic history that touches a third of the vocabulary, so penalised scores
    sit between fp16 values in most rank bins, the truncation cuts' and the draws' bins included."""
    import turbospark_amd as ts
    cfg, gpu, prompt = _setup()
    V, k = cfg["vocab"], 4
    rng = np.random.default_rng(23)
    gpu.rollback(ts.ffi.Point(len(prompt) - 1))
    nxt = int(prompt[-1])
    if dense:
        history = [int(t) for t in rng.integers(-3, V + 3, 2500)]  # ids outside the vocabulary are skipped
        n_prompt = 700
    else:
        history = [int(t) for t in prompt[:-1]]
        n_prompt = len(history)
    draw_step = 0
    margins, accepted_hist = [], []
    for rnd in range(16):
        seed = 500 + rnd
        gcfg = ts.shaping(0.8 if rnd % 2 else 1.0, seed=seed, **kw)
        ocfg = ob.shaping(0.8 if rnd % 2 else 1.0, seed=seed, **kw)
        hist_now = history + [nxt]
        generated = len(hist_now) - n_prompt
        draft = rng.standard_normal((k, V)).astype(np.float16)
        if rnd % 4 == 1:
            draft[1] = np.round(draft[1] * 2) / 2
        if rnd % 2 == 1:  # a drafter that resembles the target, so that proposals get accepted
            here = gpu.checkpoint()
            tok = nxt
            for i in range(k):
                row = gc.f16(gpu.produce(tok, gpu.position))
                draft[i] = (row + rng.standard_normal(V) * 0.3).astype(np.float16)
                one, _ = gpu.draft_chain(draft[i:i + 1], gcfg, draw_step + i, history=hist_now, generated=generated)
                tok = int(one[0])
            gpu.rollback(here)
        if rnd % 5 == 2:  # the proposals repeat themselves: later rows count the earlier ones
            draft[1:] = draft[0]
        props, ds1 = gpu.draft_chain(draft, gcfg, draw_step, history=hist_now, generated=generated)
        oprops, ods1 = ob.draft_chain(draft, ocfg, hist_now, generated, draw_step)
        assert list(props) == list(oprops) and ds1 == ods1
        feed = [nxt] + [int(t) for t in props]
        base = gpu.position
        res, logits = gpu.verify_accept(feed, base, gcfg, draft_logits=draft, draw_step=ds1, want_logits=True,
                                        history=hist_now, generated=generated)
        want = ob.chain_round(logits, draft, props, ocfg, history=hist_now, generated=generated, draw_step=ds1)
        _same(res, want, base)
        margins.append(res.min_margin)
        accepted_hist.append(res.accepted)
        history = hist_now + feed[1: 1 + want["committed"]]
        nxt = want["next"]
        draw_step = want["draw_step"]
    print("accepted per round:", accepted_hist, " min margin:", min(margins))
    assert min(margins) > 1e-9
    assert len(set(accepted_hist)) > 1


def test_penalties_change_the_outcome_and_greedy_ignores_them():
    """The penalised rounds are not the plain ones in disguise: with the proposal in the history a
    strong penalty flips decisions the plain round makes; at temperature 0 the arg-max ignores
    penalties (choose.rs:84-88)."""
    import turbospark_amd as ts
    cfg, gpu, prompt = _setup()
    V = cfg["vocab"]
    rng = np.random.default_rng(3)
    base = gpu.position
    point = gpu.checkpoint()
    differs = 0
    for seed in range(12):
        draft = rng.standard_normal((3, V)).astype(np.float16)
        plain = ts.shaping(0.9, seed=seed)
        props, ds = gpu.draft_chain(draft, plain, 0)
        feed = [5] + [int(t) for t in props]
        hist = list(prompt) + feed  # every proposal is already in the history
        a = gpu.verify_accept(feed, base, plain, draft_logits=draft, draw_step=ds)
        gpu.rollback(point)
        pen = ts.shaping(0.9, seed=seed, repetition_penalty=3.0, presence_penalty=4.0)
        b, logits = gpu.verify_accept(feed, base, pen, draft_logits=draft, draw_step=ds, history=hist, generated=3,
                                      want_logits=True)
        gpu.rollback(point)
        want = ob.chain_round(logits, draft, props, ob.shaping(0.9, seed=seed, repetition_penalty=3.0, presence_penalty=4.0),
                              history=hist, generated=3, draw_step=ds)
        _same(b, want, base)
        differs += (a.accepted, a.next) != (b.accepted, b.next)
    assert differs > 0
    g = gpu.verify_accept([5, 6, 7], base, ts.shaping(0.0, repetition_penalty=2.0, presence_penalty=1.0),
                          history=list(prompt), generated=2)
    gpu.rollback(point)
    h = gpu.verify_accept([5, 6, 7], base, ts.shaping(0.0))
    assert (g.accepted, g.next) == (h.accepted, h.next)


@pytest.mark.parametrize("kw", [dict(), dict(top_p=0.8), dict(repetition_penalty=1.4, frequency_penalty=0.3)])
def test_a_round_without_proposals_is_one_draw_from_the_target(kw):
    """m = 1 (nothing offered: the budget or the context left room for no proposal): the round is the
    bonus draw from row 0 (speculative.rs:861-879), sampled or arg-max; penalties with an empty
    history are no-ops (penalty.rs:16-18,66-69)."""
    import turbospark_amd as ts
    cfg, gpu, prompt = _setup()
    V = cfg["vocab"]
    base = gpu.position
    point = gpu.checkpoint()
    none = np.zeros((0, V), np.float16)
    for seed, hist in enumerate([[], [int(t) for t in prompt] + [9], [9] * 30]):
        gcfg, ocfg = ts.shaping(0.8, seed=seed, **kw), ob.shaping(0.8, seed=seed, **kw)
        res, logits = gpu.verify_accept([9], base, gcfg, draft_logits=np.zeros((1, V), np.float16), draw_step=5,
                                        want_logits=True, history=hist, generated=min(len(hist), 12))
        want = ob.chain_round(logits, none, [], ocfg, history=hist, generated=min(len(hist), 12), draw_step=5)
        _same(res, want, base)
        assert res.accepted == 0 and res.draw_step == 6
        gpu.rollback(point)
    res, logits = gpu.verify_accept([9], base, ts.shaping(0.0), want_logits=True)
    assert res.next == int(np.argmax(gc.f16(logits)[0])) and res.accepted == 0
    gpu.rollback(point)


def test_identical_drafter_is_always_accepted_and_the_bonus_is_a_p_draw():
    import turbospark_amd as ts
    cfg, gpu, prompt = _setup()
    base = gpu.position
    point = gpu.checkpoint()
    feed0 = [7]
    row0 = gpu.verify(feed0, base)            # the target's own distribution after token 7
    gpu.rollback(point)
    for seed in range(8):
        gcfg, ocfg = ts.shaping(0.8, seed=seed), ob.shaping(0.8, seed=seed)
        props, ds = gpu.draft_chain(row0, gcfg, 0)   # q == p for the only proposal
        res, logits = gpu.verify_accept(feed0 + [int(props[0])], base, gcfg, draft_logits=row0, draw_step=ds,
                                        want_logits=True)
        want = ob.chain_round(logits, row0, props, ocfg, history=list(prompt) + feed0, draw_step=ds)
        assert want["accepted"] == 1
        _same(res, want, base)
        gpu.rollback(point)


def test_greedy_chain_rounds_stop_tokens_and_budget():
    import turbospark_amd as ts
    cfg, gpu, prompt = _setup()
    V = cfg["vocab"]
    base = gpu.position
    point = gpu.checkpoint()
    gcfg, ocfg = ts.shaping(0.0), ob.shaping(0.0)
    # learn the target's greedy continuation so proposals can be made to hit or miss
    truth = []
    tok = 3
    for i in range(5):
        row = gpu.produce(tok, base + i)
        truth.append(int(np.argmax(gc.f16(row))))
        tok = truth[-1]
    gpu.rollback(point)
    cases = [truth[:4], truth[:2] + [(truth[2] + 1) % V, truth[3]], [(truth[0] + 1) % V] + truth[1:4]]
    for props in cases:
        res, logits = gpu.verify_accept([3] + props, base, gcfg, want_logits=True)
        want = ob.chain_round(logits, None, props, ocfg, history=list(prompt) + [3])
        _same(res, want, base)
        gpu.rollback(point)
    # a stop token inside the block, and an exact budget
    res, logits = gpu.verify_accept([3] + truth[:4], base, gcfg, stop_tokens=[truth[1]], want_logits=True)
    want = ob.chain_round(logits, None, truth[:4], ocfg, history=list(prompt) + [3], stop_tokens=[truth[1]])
    assert want["stopped"] == 1 and want["committed"] == 1
    _same(res, want, base)
    gpu.rollback(point)
    res, logits = gpu.verify_accept([3] + truth[:4], base, gcfg, generated=5, max_new_tokens=7, want_logits=True)
    want = ob.chain_round(logits, None, truth[:4], ocfg, history=list(prompt) + [3], generated=5, max_new_tokens=7)
    assert want["stopped"] == 2
    _same(res, want, base)


def test_greedy_tree_round_walks_compacts_and_truncates():
    import turbospark_amd as ts
    cfg, gpu, prompt = _setup("small_q4_k", ctx=37, max_context=128)
    V = cfg["vocab"]
    base = gpu.position
    point = gpu.checkpoint()
    gcfg, ocfg = ts.shaping(0.0), ob.shaping(0.0)
    truth, tok = [], 9
    for i in range(4):
        row = gpu.produce(tok, base + i)
        truth.append(int(np.argmax(gc.f16(row))))
        tok = truth[-1]
    gpu.rollback(point)
    parent = [-1, 0, 0, 0, 0, 1, 5, 6, 2, 8, 9, 3, 11, 12, 4, 14]
    feed = list(np.random.default_rng(2).integers(0, V, 16))
    feed[0] = 9
    feed[2], feed[8], feed[9] = truth[0], truth[1], truth[2]   # the truth lives on branch 0-2-8-9
    res, logits = gpu.verify_accept(feed, base, gcfg, parent=parent, want_logits=True)
    want = ob.tree_round_greedy(logits, feed, parent, ocfg, history=list(prompt))
    assert want["path"] == [0, 2, 8, 9]
    assert res.path == want["path"] and res.next == want["next"] and res.accepted == 3
    assert gpu.position == base + 4
    # after compaction + truncation the engine continues exactly like a chain that fed the path
    nxt = gpu.produce(res.next, base + 4)
    gpu.rollback(point)
    gpu.verify([9] + truth[:3], base)
    ref = gpu.produce(res.next, base + 4)
    assert gc.logit_error(nxt[None], ref[None]) <= 2e-3


@pytest.mark.parametrize("name,temperature,kw", [("tiny_q8_0", 1.0, {}), ("small_q4_k", 0.8, {}),
                                                 ("tiny_q8_0", 1.0, dict(top_k=64, top_p=0.9)),
                                                 ("tiny_q8_0", 1.0, dict(repetition_penalty=1.3, presence_penalty=0.5,
                                                                         frequency_penalty=0.2)),
                                                 ("small_q4_k", 0.8, dict(repetition_penalty=1.15, top_p=0.9, min_p=0.01))])
def test_sampled_tree_rounds_match_the_oracle_bit_for_bit(name, temperature, kw):
    """Multi-branch rejection over a 16-node tree.  The rule is the oracle's own (the reference
    keeps tree rounds greedy, speculative.rs:390-392), so this pins the device against the
    oracle only: parity with the reference is unpinned for this mode."""
    import turbospark_amd as ts
    cfg, gpu, prompt = _setup(name, ctx=37, max_context=128)
    V = cfg["vocab"]
    base = gpu.position
    point = gpu.checkpoint()
    parent = [-1, 0, 0, 0, 0, 1, 5, 6, 2, 8, 9, 3, 11, 12, 4, 14]
    rng = np.random.default_rng(17)
    depths, margins = [], []
    row0 = gc.f16(gpu.verify([9], base))[0]
    gpu.rollback(point)
    likely = np.argsort(-row0)[:8]
    for rnd in range(12):
        feed = [int(t) for t in rng.integers(0, V, 16)]
        feed[0] = 9
        feed[1:5] = [int(t) for t in rng.choice(likely, 4, replace=False)]  # children inside a truncated set
        logits = gpu.verify_tree(feed, parent, base)
        # drafter rows: the target's own rows plus noise, so that p(x) / q(x) scatters around one
        noise = rng.standard_normal((16, V)) * (0.25 if rnd % 2 else 1.5)
        draft = (gc.f16(logits).astype(np.float64) + noise).astype(np.float16)
        if rnd == 3:
            draft = gc.f16(logits).copy()      # q == p: the first child of every node is accepted
        seed = 500 + rnd
        gcfg, ocfg = ts.shaping(temperature, seed=seed, **kw), ob.shaping(temperature, seed=seed, **kw)
        # (with penalties every node is shaped with the history of its own root path; the history
        # handed over holds the likely children, so the penalties bite where decisions are made)
        hist = list(prompt) + [int(t) for t in likely[:5]] + [9]
        res = gpu.accept(feed, base, gcfg, parent=parent, draft_logits=draft, draw_step=7 * rnd, history=hist,
                         generated=6)
        want = ob.tree_round_sampled(logits, draft, feed, parent, ocfg, history=hist, generated=6, draw_step=7 * rnd)
        assert res.path == want["path"], (rnd, res, want)
        assert (res.accepted, res.committed, res.next, res.draw_step, res.stopped) == \
            (want["accepted"], want["committed"], want["next"], want["draw_step"], 0), (rnd, res, want)
        assert res.kv_position == base + want["committed"] + 1 == gpu.position
        if rnd == 3:
            assert res.path == [0, 1, 5, 6, 7]
        depths.append(res.accepted)
        margins.append(res.min_margin)
        gpu.rollback(point)
    print("accepted depth per round:", depths, " min margin:", min(margins))
    assert min(margins) > 1e-9
    if not (kw.get("top_k") or kw.get("top_p")):  # (random deeper nodes fall outside both truncated sets, where 0 <= 0 accepts)
        assert len(set(depths)) > 2
    # the compacted cache continues like a chain that fed the accepted path
    feed = [int(t) for t in rng.integers(0, V, 16)]
    logits = gpu.verify_tree(feed, parent, base)
    gcfg = ts.shaping(temperature, seed=4)
    res = gpu.accept(feed, base, gcfg, parent=parent, draft_logits=gc.f16(logits).copy())
    assert res.accepted == 4
    nxt = gpu.produce(res.next, base + 5)
    gpu.rollback(point)
    gpu.verify([feed[i] for i in res.path], base)
    ref = gpu.produce(res.next, base + 5)
    assert gc.logit_error(nxt[None], ref[None]) <= 2e-3
    with pytest.raises(ts.TsvError, match="stop tokens"):
        gpu.rollback(point)
        gpu.verify_tree(feed, parent, base)
        gpu.accept(feed, base, gcfg, parent=parent, draft_logits=gc.f16(logits).copy(), stop_tokens=[3])


def test_refusals_by_name():
    import turbospark_amd as ts
    from turbospark_amd import TsvError
    cfg, gpu, prompt = _setup()
    base = gpu.position
    with pytest.raises(TsvError, match="seed"):
        gpu.verify_accept([1, 2], base, ts.shaping(0.8), draft_logits=np.zeros((1, cfg["vocab"]), np.float16))
    with pytest.raises(TsvError, match="drafter"):
        gpu.verify_accept([1, 2], base, ts.shaping(0.8, seed=3))
    assert gpu.position == base + 2 or gpu.position == base  # the refusal happened before or after the pass, never mid-way
    bad = np.zeros((1, cfg["vocab"]), np.float16)
    bad[0, 5] = np.inf
    gpu.rollback(ts.ffi.Point(base))
    with pytest.raises(TsvError, match="non-finite"):
        gpu.verify_accept([1, 2], base, ts.shaping(0.8, seed=3), draft_logits=bad)
    # the tree a round names has to be well formed, and the one the pass attended by
    gpu.rollback(ts.ffi.Point(base))
    feed = [1, 2, 3, 4]
    gpu.verify(feed, base)                                   # a chain pass ...
    with pytest.raises(TsvError, match="not the one the last verify pass attended by"):
        gpu.accept(feed, base, ts.shaping(0.0), parent=[-1, 0, 0, 1])        # ... judged as a tree
    with pytest.raises(TsvError, match=r"parent\[s\] in \[0, s\)"):
        gpu.accept(feed, base, ts.shaping(0.0), parent=[-1, 0, 2, 1])        # a link that does not lead towards slot 0
    with pytest.raises(TsvError, match=r"parent\[0\] must be -1"):
        gpu.accept(feed, base, ts.shaping(0.0), parent=[0, 0, 1, 2])
    assert gpu.accept(feed, base, ts.shaping(0.0), parent=[-1, 0, 1, 2]).committed >= 0   # the chain, spelled out
    gpu.rollback(ts.ffi.Point(base))
    gpu.verify_tree(feed, [-1, 0, 0, 1], base)               # a tree pass ...
    with pytest.raises(TsvError, match="not the one the last verify pass attended by"):
        gpu.accept(feed, base, ts.shaping(0.0))                               # ... judged as a chain
    with pytest.raises(TsvError, match="not the one the last verify pass attended by"):
        gpu.accept(feed, base, ts.shaping(0.0), parent=[-1, 0, 0, 2])
    assert gpu.accept(feed, base, ts.shaping(0.0), parent=[-1, 0, 0, 1]).committed >= 0


def test_a_vocabulary_that_is_not_a_multiple_of_anything_convenient():
    """4099 rows in the head (a padded last tile) and logit rows that start at odd byte offsets (no
    16-byte loads in the acceptance walks): forward parity and sampled rounds equal to the oracle."""
    import turbospark_amd as ts
    cfg, w, gpu, cpu = gc.build_pair("tiny_q8_0", max_context=96, vocab=4099)
    V = cfg["vocab"]
    prompt = np.random.default_rng(5).integers(0, V, 33).astype(np.int32)
    gpu.prefill(prompt, 0, want_logits=False)
    for i in range(0, 33, 16):
        cpu.verify(prompt[i:i + 16], i)
    rng = np.random.default_rng(6)
    feed = rng.integers(0, V, 5).astype(np.int32)
    point = gpu.checkpoint()
    assert gc.logit_error(gpu.verify(feed, 33), cpu.verify(feed, 33)) <= 2e-3
    gpu.rollback(point)
    for seed, kw in enumerate([{}, dict(top_k=40), dict(top_p=0.9), dict(min_p=0.05)]):
        gcfg, ocfg = ts.shaping(0.8, seed=seed, **kw), ob.shaping(0.8, seed=seed, **kw)
        draft = rng.standard_normal((4, V)).astype(np.float16)
        draft[2] = np.round(draft[2] * 2) / 2
        props, ds = gpu.draft_chain(draft, gcfg, 0)
        oprops, ods = ob.draft_chain(draft, ocfg, list(prompt) + [7], len(prompt), 0)
        assert list(props) == list(oprops) and ds == ods
        res, logits = gpu.verify_accept([7] + [int(t) for t in props], 33, gcfg, draft_logits=draft, draw_step=ds,
                                        want_logits=True)
        want = ob.chain_round(logits, draft, props, ocfg, history=list(prompt) + [7], draw_step=ds)
        _same(res, want, 33)
        gpu.rollback(point)
