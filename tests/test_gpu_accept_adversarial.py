"""Acceptance on scores no model would hand over: flat rows, two-valued rows, heavy ties, spreads that
underflow every exponential but one, the fp16 extremes, subnormals and signed zeros, tiny and odd
vocabularies.  The target rows are written to the device directly (`tsv_write_logits`), so the whole
round -- statistics, truncation cuts, the acceptance walk, residual and bonus draws, penalties, tree
walks -- is compared with the oracle's restatement of crates/runtime/src/speculative.rs:694-754,
861-879 and crates/selection/src/choose.rs:111-338, integers equal.

A case whose smallest decision margin the device itself reports below 1e-9 is not compared (a
comparison that close may legitimately fall the other way against host libm / summation order); such
cases must stay rare."""
import numpy as np
import pytest

from oracle import binding as ob
from tests import gpu_common as gc

pytestmark = pytest.mark.gpu

F16_MAX = 65504.0


def _row(r, V, kind):
    if kind == "flat":
        return np.full(V, float(r.choice([0.0, -3.5, 11.0])), np.float32)
    if kind == "two":
        a, b = r.choice([-2.0, 0.0, 0.5, 3.0, 8.0], 2, replace=False)
        return np.where(r.random(V) < r.uniform(0.01, 0.6), a, b).astype(np.float32)
    if kind == "ties":
        q = float(r.choice([1, 2, 4, 8]))
        return (np.round(r.standard_normal(V) * 2 * q) / q).astype(np.float32)
    if kind == "wide":
        return np.clip(r.standard_normal(V) * 3000.0, -F16_MAX, F16_MAX).astype(np.float32)
    if kind == "extremes":
        x = np.full(V, -F16_MAX, np.float32)
        x[r.integers(0, V, max(1, V // 50))] = F16_MAX
        x[r.integers(0, V, max(1, V // 50))] = float(r.choice([0.0, 60000.0, F16_MAX - 32.0]))
        return x
    if kind == "tiny":
        x = (r.integers(-6, 7, V) * 5.96e-8).astype(np.float32)          # fp16 subnormals around zero
        x[r.random(V) < 0.3] = -0.0
        return x
    if kind == "peaked":
        x = r.standard_normal(V).astype(np.float32)
        x[r.integers(0, V)] += float(r.choice([12.0, 30.0, 200.0]))
        return x
    return (r.standard_normal(V) * 2).astype(np.float32)


KINDS = ["flat", "two", "ties", "wide", "extremes", "tiny", "peaked", "normal"]


def _shaping(r, seed, penalties):
    import turbospark_amd as ts
    kw = {}
    if r.integers(0, 2):
        kw["top_k"] = int(r.integers(1, 257))
    if r.integers(0, 2):
        kw["top_p"] = float(r.uniform(0.05, 1.0))
    if r.integers(0, 2):
        kw["min_p"] = float(r.uniform(1e-4, 0.5))
    if penalties and r.integers(0, 2):
        kw["repetition_penalty"] = float(r.uniform(0.5, 2.0))
    if penalties and r.integers(0, 2):
        kw["presence_penalty"] = float(r.uniform(-2.0, 2.0))
        kw["frequency_penalty"] = float(r.uniform(-2.0, 2.0))
    t = float(r.choice([0.05, 0.3, 0.8, 1.0, 1.7, 4.0]))
    return ts.shaping(t, seed=seed, **kw), ob.shaping(t, seed=seed, **kw), kw


@pytest.mark.parametrize("vocab", [4096, 1000, 37, 2, 128256, 201088])
def test_adversarial_chain_rounds(vocab):
    """(128256 and 201088: the vocabularies of the benchmark configurations, fewer and narrower rounds.)"""
    cfg, w, gpu, cpu = gc.build_pair("tiny_q8_0", max_context=64, vocab=vocab)
    V = vocab
    r = np.random.default_rng(77 + vocab)
    base = 20
    compared = skipped = 0
    outcomes = set()
    big = V > 100000
    for case in range(14 if big else 60):
        k = int(r.integers(0, 6 if big else 16))
        kind_t, kind_d = r.choice(KINDS), r.choice(KINDS)
        target = np.stack([_row(r, V, kind_t) for _ in range(k + 1)]).astype(np.float16)
        # the drafter: adversarial rows of its own, or the target's rows nudged (so that proposals get accepted)
        if r.integers(0, 2) and k:
            draft = (target[:k].astype(np.float32) + (r.standard_normal((k, V)) * 0.05).astype(np.float32)).astype(np.float16)
        else:
            draft = np.stack([_row(r, V, kind_d) for _ in range(max(k, 1))]).astype(np.float16)[:max(k, 1)]
        # (a penalised score below every fp16 value is refused by name: no penalties on the rows that sit there)
        gcfg, ocfg, kw = _shaping(r, 100 + case, penalties=not {kind_t, kind_d} & {"wide", "extremes"})
        hist = [int(t) for t in r.integers(-2, V + 2, int(r.integers(0, 300)))]
        generated = int(r.integers(0, len(hist) + 2))
        ds = int(r.integers(0, 1000))
        stops = [int(t) for t in r.integers(0, V, int(r.integers(0, 3)))]
        budget = generated + int(r.integers(1, 20))
        try:
            if k:
                props, ds1 = gpu.draft_chain(draft[:k], gcfg, ds, history=hist, generated=generated)
                oprops, ods1 = ob.draft_chain(draft[:k], ocfg, hist, generated, ds)
            else:
                props, ds1, oprops, ods1 = np.zeros(0, np.int32), ds, np.zeros(0, np.int32), ds
        except Exception as e:  # a refusal by name (more penalised candidates in one rank bin than the list holds)
            assert "not built" in str(e), e
            skipped += 1
            continue
        feed = [int(r.integers(0, V))] + [int(t) for t in oprops]
        gpu.write_logits(target, base)
        try:
            res = gpu.accept(feed, base, gcfg, draft_logits=draft, draw_step=ods1, stop_tokens=stops, generated=generated,
                             max_new_tokens=budget, history=hist)
        except Exception as e:
            assert "not built" in str(e), e
            skipped += 1
            continue
        want = ob.chain_round(target.view(np.uint16), draft.view(np.uint16)[:k] if k else np.zeros((0, V), np.uint16), oprops, ocfg,
                              history=hist, generated=generated, max_new_tokens=budget, stop_tokens=stops, draw_step=ods1)
        if res.min_margin < 1e-9:
            skipped += 1
            continue
        assert list(props) == list(oprops) and ds1 == ods1, (case, kind_d, kw)
        got = (res.accepted, res.committed, res.next, res.stopped, res.draw_step)
        assert got == (want["accepted"], want["committed"], want["next"], want["stopped"], want["draw_step"]), \
            (case, kind_t, kind_d, k, kw, res, want)
        assert res.kv_position == base + want["committed"] + 1
        compared += 1
        outcomes.add((res.accepted == k, res.stopped))
    print(f"vocab {vocab}: {compared} rounds compared, {skipped} too close to call or refused by name; outcomes {sorted(outcomes)}")
    assert compared >= (10 if big else 45) and len(outcomes) >= 2


@pytest.mark.parametrize("vocab", [4096, 333])
def test_adversarial_tree_rounds(vocab):
    cfg, w, gpu, cpu = gc.build_pair("tiny_q8_0", max_context=64, vocab=vocab)
    V = vocab
    r = np.random.default_rng(5 + vocab)
    base = 20
    compared = skipped = 0
    for case in range(40):
        m = int(r.integers(2, 17))
        parent = [-1] + [int(r.integers(0, s)) for s in range(1, m)]
        kind_t, kind_d = r.choice(KINDS), r.choice(KINDS)
        target = np.stack([_row(r, V, kind_t) for _ in range(m)]).astype(np.float16)
        if r.integers(0, 2):
            draft = (target.astype(np.float32) + (r.standard_normal((m, V)) * 0.05).astype(np.float32)).astype(np.float16)
        else:
            draft = np.stack([_row(r, V, kind_d) for _ in range(m)]).astype(np.float16)
        feed = [int(t) for t in r.integers(0, V, m)]
        # children drawn from where the mass is, so that walks go deep
        for s in range(1, m):
            if r.integers(0, 2):
                feed[s] = int(np.argmax(target[parent[s]].astype(np.float32) + r.standard_normal(V) * 0.5))
        sampled = bool(r.integers(0, 4))
        gcfg, ocfg, kw = _shaping(r, 300 + case, penalties=not {kind_t, kind_d} & {"wide", "extremes"})
        if not sampled:
            import turbospark_amd as ts
            gcfg, ocfg = ts.shaping(0.0), ob.shaping(0.0)
        hist = [int(t) for t in r.integers(0, V, int(r.integers(0, 200)))]
        generated = int(r.integers(0, len(hist) + 2))
        gpu.write_logits(target, base)
        try:
            res = gpu.accept(feed, base, gcfg, parent=parent, draft_logits=draft if sampled else None, draw_step=9,
                             history=hist, generated=generated)
        except Exception as e:
            assert "not built" in str(e), e
            skipped += 1
            continue
        if sampled:
            want = ob.tree_round_sampled(target.view(np.uint16), draft.view(np.uint16), feed, parent, ocfg, history=hist,
                                         generated=generated, draw_step=9)
        else:
            want = ob.tree_round_greedy(target.view(np.uint16), feed, parent, ocfg, history=hist)
        if res.min_margin < 1e-9:
            skipped += 1
            continue
        assert res.path == want["path"] and res.next == want["next"], (case, kind_t, kind_d, kw, res, want)
        if sampled:
            assert res.draw_step == want["draw_step"]
        compared += 1
    print(f"vocab {vocab}: {compared} tree rounds compared, {skipped} too close to call or refused by name")
    assert compared >= 30
