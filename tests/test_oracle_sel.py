"""Pins the oracle's selection pipeline and round logic.

Ports the host-checkable cases of crates/selection/tests/{distribution,rejection_sampling,
reference_drift,rank_top_k,min_p}.rs, crates/selection/src/distribution.rs:128-285,
crates/runtime/src/dflash_tree.rs:168-194 and the distributional law of
crates/runtime/tests/speculative.rs:870-1000.
"""
import math

import numpy as np
import pytest

from oracle import binding as ob

GOLDEN = 0x9E3779B97F4A7C15


def test_mix_is_the_published_splitmix64_output_function():
    # splitmix64 seeded with 0 emits these (Vigna's reference vectors); output i is
    # mix(i * GOLDEN) in the reference's formulation, which adds the increment first.
    want = [0xE220A8397B1DCDAF, 0x6E789E6AA1B965F4, 0x06C45D188009454F]
    for i, w in enumerate(want):
        assert ob.lib().tso_mix((i * GOLDEN) & (2**64 - 1)) == w
    # derive_step_value(seed, position) = mix(seed ^ position * GOLDEN)
    assert ob.lib().tso_derive_step_value(0, 1) == want[1]
    assert ob.lib().tso_derive_step_value(0, 2) == want[2]
    assert ob.lib().tso_derive_step_value(7, 3) == ob.lib().tso_mix(7 ^ ((3 * GOLDEN) & (2**64 - 1)))
    assert ob.lib().tso_derive_step_value(7, 3) != ob.lib().tso_derive_step_value(7, 4)


def test_unit_interval_uses_the_top_53_bits():
    L = ob.lib()
    assert L.tso_to_unit_interval(0) == 0.0
    assert L.tso_to_unit_interval(2**64 - 1) == 1.0 - 2.0**-53
    assert L.tso_to_unit_interval(1 << 11) == 2.0**-53
    assert L.tso_to_unit_interval((1 << 11) - 1) == 0.0
    for p in range(50):
        assert 0.0 <= L.tso_to_unit_interval(L.tso_derive_step_value(1, p)) < 1.0


# ---- an independent numpy restatement of the shaping pipeline (composition law) ----------
def np_shape(logits_f16, T, top_k, top_p, min_p):
    w = logits_f16.astype(np.float32)
    e = np.exp(w.astype(np.float64) - np.float64(w.max()))
    s = 0.0
    for v in e:          # sequential, index order
        s += v
    order = sorted(range(len(e)), key=lambda i: (-e[i], i))
    ranked = order if top_k == 0 else order[:top_k]
    if top_p is None:
        surv = list(ranked)
    else:
        surv, cum = [], 0.0
        for i in ranked:
            surv.append(i)
            cum += e[i] / s
            if cum >= top_p:
                break
    if top_k:
        surv = surv[:top_k]
    if min_p is not None:
        thr = min_p * e[ranked[0]]
        kept = [i for i in surv if e[i] >= thr]
        surv = kept or [ranked[0]]
    p = np.array([e[i] / s for i in surv])
    top = p.max()
    wgt = (p / top) ** (1.0 / T)
    tot = 0.0
    for v in wgt:
        tot += v
    return surv, wgt / tot


def xorshift_scores(n, seed):
    s = seed or 1
    out = []
    for _ in range(n):
        s ^= (s << 13) & 0xFFFFFFFF
        s ^= s >> 17
        s ^= (s << 5) & 0xFFFFFFFF
        out.append(((s & 0xFFFF) / 65535.0) * 12.0 - 6.0)
    return np.array(out, np.float16)


@pytest.mark.parametrize("case", range(6))
def test_pipeline_matches_the_composed_helper_restatement(case):
    n = [5, 64, 257, 1000, 4096, 300][case]
    scores = xorshift_scores(n, 1234 + case)
    if case == 5:
        scores[10:40] = scores[10]  # a long tie run: ascending index must break it
    for top_k in (0, 1, 8, 64, 256):
        for top_p in (None, 0.5, 0.9, 1.0):
            for min_p in (None, 0.05, 0.5):
                for T in (0.3, 1.0):
                    cfg = ob.shaping(T, top_k, top_p, 1.0, seed=3, min_p=min_p)
                    sup, pr = ob.shaped_distribution(scores, cfg)
                    wsup, wpr = np_shape(scores, T, top_k, top_p, min_p)
                    assert list(sup) == wsup, (top_k, top_p, min_p, T)
                    assert np.allclose(pr, wpr, rtol=1e-13, atol=0)
                    assert abs(pr.sum() - 1.0) < 1e-12


def structured_scores():
    base = {7: 6.0, 19: 4.5, 20: 4.2, 33: 3.0}
    return np.array([base.get(i, -1.0 - i * 0.01) for i in range(64)], np.float16)


def test_shaped_distribution_draws_what_select_draws():
    scores = structured_scores()
    history = [3, 7, 11]
    for (T, k, p, seed) in [(0.2, 64, 0.95, 7), (0.7, 0, None, 9), (1.3, 8, 0.9, 11),
                            (0.5, 64, 0.95, 20260911)]:
        cfg = ob.shaping(T, k, p, 1.0, seed=seed)
        for position in (0, 1, 2, 5, 17, 100):
            sel = ob.select(scores, cfg, history, position)
            sup, pr = ob.shaped_distribution(scores, cfg, history, position)
            assert sel == ob.dist_draw(sup, pr, seed, position)
            assert abs(pr.sum() - 1) < 1e-12 and sel in sup


def test_deterministic_arm_is_first_max_argmax_and_tiny_temperature_is_greedy():
    scores = np.array([1.0, 5.0, 5.0, -2.0], np.float16)
    cfg = ob.shaping(0.0, 3, 0.5, 1.3, seed=1)  # penalties/truncation ignored at T=0
    assert ob.select(scores, cfg, [1, 1, 1], 2) == 1
    sup, pr = ob.shaped_distribution(scores, cfg)
    assert list(sup) == [1] and list(pr) == [1.0]
    cfg = ob.shaping(1e-6, 0, None, 1.0, seed=5)
    s2 = structured_scores()
    for pos in range(20):
        assert ob.select(s2, cfg, None, pos) == 7


def test_refusals():
    cfg = ob.shaping(0.7, 0, None, 1.0, seed=1)
    bad = np.array([0.0, np.inf, 1.0], np.float16)
    with pytest.raises(ValueError):
        ob.select(bad, cfg)
    with pytest.raises(ValueError):
        ob.select(np.array([0.0, np.nan], np.float16), cfg)
    with pytest.raises(ValueError):
        ob.select(np.array([0.0, 1.0], np.float16), ob.shaping(0.7))  # sampled, no seed


def test_penalties():
    scores = np.array([2.0, -2.0, 1.0, 3.0], np.float16)
    cfg = ob.shaping(1.0, 0, None, 2.0, seed=1)
    sup, pr = ob.shaped_distribution(scores, cfg, [0, 1, 1], 0)
    # token 0: 2/2 = 1, token 1: -2*2 = -4 (each distinct id once), others untouched
    w = np.array([1.0, -4.0, 1.0, 3.0])
    want = np.exp(w) / np.exp(w).sum()
    got = np.zeros(4)
    got[sup] = pr
    assert np.allclose(got, want, rtol=1e-12)
    # presence/frequency only over the GENERATED suffix (position = generated count)
    cfg = ob.shaping(1.0, 0, None, 1.0, seed=1, presence_penalty=0.5, frequency_penalty=0.25)
    sup, pr = ob.shaped_distribution(scores, cfg, [3, 3, 2, 2, 2], 3)  # suffix = [2,2,2]
    w = np.array([2.0, -2.0, 1.0 - np.float32(0.5 + 0.25 * 3), 3.0])
    want = np.exp(w) / np.exp(w).sum()
    got = np.zeros(4)
    got[sup] = pr
    assert np.allclose(got, want, rtol=1e-6)


def _shaped_scores(scores, cfg, history, position):
    """The penalised scores behind a shaped distribution at temperature 1 with no truncation: p is the
    softmax of them, so log p differences give them back."""
    sup, pr = ob.shaped_distribution(np.array(scores, np.float16), cfg, history, position)
    got = np.zeros(len(scores))
    got[sup] = pr
    return got


@pytest.mark.parametrize("scores,history,position,kw,want", [
    # crates/selection/src/penalty.rs:105-119: a repeated entry is attenuated once; positive scores
    # divide, negative ones multiply
    ([4.0, 1.0], [0, 0, 0], 0, dict(repetition_penalty=2.0), [2.0, 1.0]),
    ([4.0, -4.0], [0, 1], 0, dict(repetition_penalty=2.0), [2.0, -8.0]),
    # :143-160: presence once whatever the count, frequency per occurrence, both add
    ([10.0, 7.0], [0, 0, 0], 3, dict(presence_penalty=1.5), [8.5, 7.0]),
    ([10.0, 7.0], [0, 0, 0], 3, dict(frequency_penalty=1.5), [5.5, 7.0]),
    ([10.0, 7.0], [0, 0], 2, dict(presence_penalty=1.0, frequency_penalty=0.5), [8.0, 7.0]),
    ([10.0, 10.0], [0, 0], 2, dict(presence_penalty=1.0, frequency_penalty=1.0), [7.0, 10.0]),
    # tests/presence_frequency.rs:80-116: a candidate that only appears in the prompt half is untouched
    ([2.0, 2.0, 2.0, 2.0], [0, 0, 0], 0, dict(presence_penalty=2.0, frequency_penalty=2.0), [2.0, 2.0, 2.0, 2.0]),
    # choose.rs:147-148: a position beyond the history counts all of it as generated
    ([2.0, 2.0], [0], 7, dict(presence_penalty=1.5), [0.5, 2.0]),
    # ids outside the candidate domain are skipped (penalty.rs:27-33)
    ([3.0, 1.0], [-1, 5, 1], 3, dict(repetition_penalty=2.0, frequency_penalty=0.25), [3.0, 0.25]),
])
def test_penalties_reproduce_the_reference_unit_vectors(scores, history, position, kw, want):
    cfg = ob.shaping(1.0, seed=1, **kw)
    got = _shaped_scores(scores, cfg, history, position)
    w = np.array(want, np.float64)
    ref = np.exp(w - w.max()) / np.exp(w - w.max()).sum()
    assert np.allclose(got, ref, rtol=1e-12, atol=0)


def test_residual_unit_cases():
    # Leviathan worked example
    r = ob.residual(([0, 1], [0.5, 0.5]), ([0], [1.0]))
    assert list(r[0]) == [1] and list(r[1]) == [1.0]
    r = ob.residual(([0, 1], [0.6, 0.4]), ([0, 1, 2], [0.2, 0.1, 0.7]))
    assert list(r[0]) == [0, 1]
    assert abs(r[1][0] - 0.4 / 0.7) < 1e-12 and abs(r[1][1] - 0.3 / 0.7) < 1e-12
    assert ob.residual(([0, 1], [0.5, 0.5]), ([0, 1], [0.5, 0.5])) is None
    r = ob.residual(([5], [1.0]), ([9], [1.0]))
    assert list(r[0]) == [5] and list(r[1]) == [1.0]
    # p-order preserved, first occurrence of a duplicate q token wins, bit-exact division
    p = ([9, 2, 40, 7, 1000], [0.3, 0.25, 0.2, 0.15, 0.1])
    q = ([7, 40, 40, 2, 11], [0.05, 0.1, 0.6, 0.3, 0.05])
    mass = [max(w - ob.dist_probability(q[0], q[1], t), 0.0) for t, w in zip(*p)]
    total = 0.0
    for m in mass:
        if m > 0:
            total += m
    r = ob.residual(p, q)
    assert list(r[0]) == [9, 40, 7, 1000]
    assert [float(x) for x in r[1]] == [m / total for m in mass if m > 0]
    assert ob.dist_probability([3, 7], [0.25, 0.75], 4) == 0.0


def test_greedy_chain_round_accepts_the_argmax_prefix_and_returns_the_bonus():
    V = 32
    target = np.full((5, V), -5.0, np.float16)
    picks = [4, 9, 9, 30, 2]
    for i, t in enumerate(picks):
        target[i, t] = 3.0
    cfg = ob.shaping(0.0)
    r = ob.chain_round(target, None, [4, 9, 1, 30], cfg, history=[1, 2, 3])
    assert (r["accepted"], r["committed"], r["next"], r["stopped"]) == (2, 2, 9, 0)
    r = ob.chain_round(target, None, [4, 9, 9, 30], cfg, history=[1, 2, 3])
    assert (r["accepted"], r["next"]) == (4, 2)
    r = ob.chain_round(target, None, [0, 9, 9, 30], cfg, history=[1])
    assert (r["accepted"], r["next"]) == (0, 4)
    # a stop token inside the block is counted, not committed, and ends the round
    r = ob.chain_round(target, None, [4, 9, 9, 30], cfg, history=[1], stop_tokens=[9])
    assert (r["accepted"], r["committed"], r["stopped"], r["next"]) == (2, 1, 1, -1)
    # exact budget: generated=5, max_new=7 -> the second accepted token hits the budget
    r = ob.chain_round(target, None, [4, 9, 9, 30], cfg, history=[1], generated=5, max_new_tokens=7)
    assert (r["accepted"], r["committed"], r["stopped"]) == (2, 1, 2)


def test_draw_step_accounting_of_a_sampled_round():
    V, k = 16, 3
    rng = np.random.default_rng(0)
    draft = rng.standard_normal((k, V)).astype(np.float16)
    target = rng.standard_normal((k + 1, V)).astype(np.float16)
    cfg = ob.shaping(0.8, seed=11)
    props, ds = ob.draft_chain(draft, cfg, draw_step=100)
    assert ds == 100 + k + 1          # k draws + the row-only step
    r = ob.chain_round(target, draft, props, cfg, draw_step=ds)
    # one uniform per judged proposal, +1 for the correction or the bonus
    judged = r["accepted"] + (1 if r["accepted"] < k else 0)
    assert r["draw_step"] == ds + judged + 1
    # identical target and draft rows: every proposal accepted (p == q), bonus drawn
    r = ob.chain_round(np.vstack([draft, draft[:1]]), draft, props, cfg, draw_step=ds)
    assert r["accepted"] == k and r["draw_step"] == ds + k + 1


def test_rejection_round_matches_the_target_distribution_in_law():
    """Leviathan/Chen: whatever the drafter, the first token a round emits is distributed as the
    target's shaped p.  Mutations this rejects: accept-all, correction drawn from p instead of the
    residual, acceptance on q/p instead of p/q."""
    V, T, N = 6, 0.7, 6000
    target = np.array([[2.0, 1.0, 0.0, -1.0, 0.5, -3.0], [0.0] * 6], np.float16)
    for draft_row in ([2.0, 1.0, 0.0, -1.0, 0.5, -3.0], [-3.0, 0.5, -1.0, 0.0, 1.0, 2.0],
                      [0.0, 0.0, 4.0, 0.0, 0.0, 0.0]):
        draft = np.array([draft_row], np.float16)
        counts = np.zeros(V)
        acc = 0
        for seed in range(N):
            cfg = ob.shaping(T, seed=seed)
            props, ds = ob.draft_chain(draft, cfg)
            r = ob.chain_round(target, draft, props, cfg, draw_step=ds)
            counts[props[0] if r["accepted"] else r["next"]] += 1
            acc += r["accepted"]
        sup, pr = ob.shaped_distribution(target[0], ob.shaping(T, seed=0))
        p = np.zeros(V)
        p[sup] = pr
        tv = 0.5 * np.abs(counts / N - p).sum()
        assert tv < 0.03, (draft_row, tv)
        qs, qp = ob.shaped_distribution(draft[0], ob.shaping(T, seed=0))
        q = np.zeros(V)
        q[qs] = qp
        assert abs(acc / N - np.minimum(p, q).sum()) < 0.03   # acceptance rate = 1 - TV(p, q)


def test_tree_greedy_walk_unit_case():
    # dflash_tree.rs:168-194: nodes (parent None, None, Some(1)), tokens [10, 11, 20];
    # picks: anchor -> 11, node 1 -> 20, else 99.  Slot parents [-1, 0, 0, 2].
    V = 128
    feed = [5, 10, 11, 20]
    parent = [-1, 0, 0, 2]
    logits = np.full((4, V), -4.0, np.float16)
    logits[0, 11] = 2.0
    logits[2, 20] = 2.0
    logits[1, 99] = 2.0
    logits[3, 99] = 2.0
    r = ob.tree_round_greedy(logits, feed, parent, ob.shaping(0.0), history=[1, 2])
    assert r["path"] == [0, 2, 3] and r["accepted"] == 2 and r["next"] == 99
    # first child in slot order wins on duplicate tokens; a miss at the anchor gives bonus only
    logits[0, 11] = -4.0
    logits[0, 7] = 2.0
    r = ob.tree_round_greedy(logits, feed, parent, ob.shaping(0.0))
    assert r["path"] == [0] and r["accepted"] == 0 and r["next"] == 7
    with pytest.raises(ValueError):
        ob.tree_round_greedy(logits, feed, parent, ob.shaping(0.7, seed=1))


def test_sampled_tree_round_reduces_to_the_chain_round_on_a_chain():
    """This project's own definition (absent upstream): on a tree that is a chain it must
    be the reference's chain round, uniform for uniform."""
    V, k = 24, 4
    rng = np.random.default_rng(4)
    for seed in range(40):
        draft = rng.standard_normal((k, V)).astype(np.float16)
        target = (draft + rng.standard_normal((k, V)).astype(np.float16) * 0.5)
        target = np.vstack([target, rng.standard_normal((1, V))]).astype(np.float16)
        cfg = ob.shaping(1.0, seed=seed)
        props, ds = ob.draft_chain(draft, cfg)
        a = ob.chain_round(target, draft, props, cfg, history=[3], draw_step=ds)
        feed = [3] + list(props)
        draft_rows = np.vstack([draft, draft[:1]])
        b = ob.tree_round_sampled(target, draft_rows, feed, [-1, 0, 1, 2, 3], cfg, history=[3],
                                  draw_step=ds)
        assert (a["accepted"], a["next"], a["draw_step"]) == (b["accepted"], b["next"], b["draw_step"])
        assert b["path"] == list(range(a["accepted"] + 1))


def test_sampled_tree_round_matches_the_target_in_law_with_two_siblings():
    V, T, N = 5, 1.0, 6000
    target = np.array([[1.5, 0.5, 0.0, -1.0, 0.2]] * 3, np.float16)
    draft = np.array([[-1.0, 0.0, 2.0, 0.5, 0.1]] * 3, np.float16)
    counts = np.zeros(V)
    for seed in range(N):
        cfg = ob.shaping(T, seed=seed)
        # two siblings drawn i.i.d. from q (draw positions 0 and 1)
        sup, pr = ob.shaped_distribution(draft[0], cfg)
        a = ob.dist_draw(sup, pr, seed, 0)
        b = ob.dist_draw(sup, pr, seed, 1)
        r = ob.tree_round_sampled(target, draft, [0, a, b], [-1, 0, 0], cfg, draw_step=2)
        first = [0, a, b][r["path"][1]] if r["accepted"] else r["next"]
        counts[first] += 1
    sup, pr = ob.shaped_distribution(target[0], ob.shaping(T, seed=0))
    p = np.zeros(V)
    p[sup] = pr
    assert 0.5 * np.abs(counts / N - p).sum() < 0.03


def _softmax(row):
    e = np.exp(np.asarray(row, np.float64) - np.max(row))
    return e / e.sum()


def test_sampled_tree_round_matches_the_target_in_law_with_three_siblings():
    """Three children drawn i.i.d. from q under the root.  The first emitted token must follow p whatever q is, and
    the chance that one of the three is accepted has a closed form: stage s accepts with sum min(p_s, q), where
    p_0 = p and p_{s+1} = normalise(max(p_s - q, 0)) -- so a residual that is not carried from sibling to sibling, or
    is carried wrongly, moves both figures."""
    V, N = 5, 6000
    target = np.array([[1.2, 0.3, -0.5, 0.8, -1.5]] * 4, np.float16)
    draft = np.array([[-0.8, 1.0, 0.6, -0.2, 0.4]] * 4, np.float16)
    counts, accepted = np.zeros(V), 0
    for seed in range(N):
        cfg = ob.shaping(1.0, seed=seed)
        sup, pr = ob.shaped_distribution(draft[0], cfg)
        kids = [ob.dist_draw(sup, pr, seed, i) for i in range(3)]
        r = ob.tree_round_sampled(target, draft, [0] + kids, [-1, 0, 0, 0], cfg, draw_step=3)
        assert r["draw_step"] == 3 + (r["path"][1] if r["accepted"] else 3) + 1   # one uniform per child tried, one final draw
        counts[([0] + kids)[r["path"][1]] if r["accepted"] else r["next"]] += 1
        accepted += r["accepted"] > 0
    p, q = _softmax(target[0].astype(np.float64)), _softmax(draft[0].astype(np.float64))
    assert 0.5 * np.abs(counts / N - p).sum() < 0.03
    miss, ps = 1.0, p.copy()
    for _ in range(3):
        miss *= 1.0 - np.minimum(ps, q).sum()
        ps = np.maximum(ps - q, 0.0)
        ps /= ps.sum()
    assert abs(accepted / N - (1.0 - miss)) < 0.03


def test_sampled_tree_round_matches_the_target_in_law_below_an_accepted_child():
    """Depth two: two siblings under the root, two children under each of them, every node's children drawn i.i.d.
    from the drafter's row of that node.  Target and drafter rows of a depth-one node depend on the node's token (as a
    model's would), so the law to meet is the chain rule: the first token follows p0, and below an accepted child
    holding x the second token follows p(. | x) -- freshly, not what the root's rejections left over, and also
    where the first sibling's subtree was rejected and the second sibling accepted."""
    V, N = 4, 40000
    rng = np.random.default_rng(11)
    p0, q0 = rng.standard_normal(V), rng.standard_normal(V)
    pc, qc = rng.standard_normal((V, V)) * 1.3, rng.standard_normal((V, V))
    parent = [-1, 0, 0, 1, 1, 2, 2]
    first = np.zeros(V)
    second = np.zeros((V, V))
    second_via_sibling = np.zeros((V, V))
    for seed in range(N):
        cfg = ob.shaping(1.0, seed=seed)
        sup, pr = ob.shaped_distribution(q0.astype(np.float16), cfg)
        a, b = ob.dist_draw(sup, pr, seed, 0), ob.dist_draw(sup, pr, seed, 1)
        feed, step = [0, a, b], 2
        for x in (a, b):
            sup, pr = ob.shaped_distribution(qc[x].astype(np.float16), cfg)
            feed += [ob.dist_draw(sup, pr, seed, step), ob.dist_draw(sup, pr, seed, step + 1)]
            step += 2
        target = np.stack([p0, pc[a], pc[b]] + [p0] * 4).astype(np.float16)
        draft = np.stack([q0, qc[a], qc[b]] + [q0] * 4).astype(np.float16)
        r = ob.tree_round_sampled(target, draft, feed, parent, cfg, draw_step=step)
        if not r["accepted"]:
            first[r["next"]] += 1
            continue
        x = feed[r["path"][1]]
        first[x] += 1
        y = feed[r["path"][2]] if r["accepted"] >= 2 else r["next"]
        second[x, y] += 1
        if r["path"][1] == 2:
            second_via_sibling[x, y] += 1
    f16 = lambda v: np.asarray(v, np.float16).astype(np.float64)
    assert 0.5 * np.abs(first / N - _softmax(f16(p0))).sum() < 0.03
    for table, bound in ((second, 0.03), (second_via_sibling, 0.06)):
        n = table.sum()
        assert n > 1500
        tv = sum(0.5 * np.abs(table[x] / table[x].sum() - _softmax(f16(pc[x]))).sum() * table[x].sum() / n
                 for x in range(V) if table[x].sum() > 0)
        assert tv < bound, tv
