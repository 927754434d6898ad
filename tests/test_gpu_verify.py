"""GPU parity of the verify pass (target forward over the drafted rows) against the oracle."""
import numpy as np
import pytest

from tests import gpu_common as gc

pytestmark = pytest.mark.gpu


def _prompt(n, vocab, seed):
    return np.random.default_rng(seed).integers(0, vocab, n).astype(np.int32)


@pytest.mark.parametrize("name,ctx,k", [("tiny_q8_0", 256, 4), ("small_q4_k", 70, 4), ("small_q4_k", 33, 15),
                                        ("xcd_q4_k", 70, 4), ("xcd_q4_k", 33, 7), ("xcd_q4_k", 40, 0),
                                        ("xcd_q8_0", 70, 4), ("xcd_q4_k", 33, 15),
                                        ("small_q4_k_m", 70, 4), ("small_q4_k_m", 21, 15),
                                        ("small_q5_k_m", 70, 4), ("small_q5_k_m", 21, 15)])
def test_verify_logits_match_the_oracle(name, ctx, k):
    cfg, w, gpu, cpu = gc.build_pair(name, max_context=ctx + 32)
    prompt = _prompt(ctx, cfg["vocab"], 7)
    gpu.prefill(prompt, 0, want_logits=False)
    for i in range(0, ctx, 64):
        cpu.verify(prompt[i:i + 64], i)
    # the caches agree (fp16 store on both sides)
    for layer in range(cfg["n_layers"]):
        kg, vg = gpu.read_kv(layer, 0, ctx)
        kc, vc = cpu.kv(layer)
        assert np.abs(kg.astype(np.float32) - kc[:ctx]).max() <= 2e-2 * np.abs(kc[:ctx]).max()
        assert np.abs(vg.astype(np.float32) - vc[:ctx]).max() <= 2e-2 * np.abs(vc[:ctx]).max()
    feed = _prompt(k + 1, cfg["vocab"], 8)
    got = gpu.verify(feed, ctx)
    want = cpu.verify(feed, ctx)
    err = gc.logit_error(got, want)
    print(f"{name} ctx={ctx} m={k+1}: max-abs logit error / range = {err:.2e}")
    assert err <= gc.TOL[cfg["dtype"]], err
    assert gpu.position == ctx + k + 1


@pytest.mark.parametrize("name", ["small_q4_k", "xcd_q4_k", "xcd_q8_0", "small_q4_k_m", "small_q5_k_m"])
def test_a_batched_pass_equals_the_same_tokens_fed_one_at_a_time(name):
    """crates/runtime/tests/real_forward_qwen35_mtp.rs:962-1032: the row-invariance gate."""
    cfg, w, gpu, cpu = gc.build_pair(name, max_context=96)
    prompt = _prompt(40, cfg["vocab"], 3)
    gpu.prefill(prompt, 0, want_logits=False)
    feed = _prompt(6, cfg["vocab"], 4)
    point = gpu.checkpoint()
    batch = gpu.verify(feed, 40)
    gpu.rollback(point)
    seq = np.stack([gpu.produce(t, 40 + i) for i, t in enumerate(feed)])
    assert np.array_equal(batch, seq)


@pytest.mark.parametrize("name", ["tiny_q8_0", "xcd_q4_k"])
def test_rollback_equals_a_fresh_run(name):
    """crates/bench/tests/rollback_probe.rs:1-140: after feeding and rolling back a rejected block,
    the kept continuation's logits equal, by bits, a run that never saw the rejected block."""
    cfg, w, gpu, cpu = gc.build_pair(name, max_context=128)
    prompt = _prompt(50, cfg["vocab"], 11)
    rejected = _prompt(5, cfg["vocab"], 12)
    kept = _prompt(5, cfg["vocab"], 13)
    kept[0] = rejected[0]
    gpu.prefill(prompt, 0, want_logits=False)
    point = gpu.checkpoint()
    gpu.verify(rejected, 50)
    gpu.rollback_retaining(point, 1)          # keep only the confirmed token's row
    assert gpu.position == 51
    a = gpu.verify(kept[1:], 51)
    gpu.reset()
    gpu.prefill(prompt, 0, want_logits=False)
    gpu.verify(kept[:1], 50)
    b = gpu.verify(kept[1:], 51)
    assert np.array_equal(a, b)


def test_tree_rows_see_the_prefix_and_their_root_path_only():
    """crates/gpu/tests/attention_tree_parity.rs:1-11 and the oracle's tree pass."""
    cfg, w, gpu, cpu = gc.build_pair("small_q4_k", max_context=96)
    prompt = _prompt(37, cfg["vocab"], 21)
    gpu.prefill(prompt, 0, want_logits=False)
    cpu.verify(prompt, 0)
    parent = [-1, 0, 0, 0, 0, 1, 5, 6, 2, 8, 9, 3, 11, 12, 4, 14]
    feed = _prompt(16, cfg["vocab"], 22)
    point = gpu.checkpoint()
    got = gpu.verify_tree(feed, parent, 37)
    want = cpu.verify(feed, 37, parent=parent)
    assert gc.logit_error(got, want) <= gc.TOL[cfg["dtype"]]
    # identity path: a chain handed over as a tree is the chain pass, bit for bit
    gpu.rollback(point)
    chain = gpu.verify(feed[:6], 37)
    gpu.rollback(point)
    as_tree = gpu.verify_tree(feed[:6], [-1, 0, 1, 2, 3, 4], 37)
    assert np.array_equal(chain, as_tree)
    # a branch node equals the chain over its own root path (slots 0,2,8,9 -> rows 0..3)
    gpu.rollback(point)
    gpu.verify_tree(feed, parent, 37)
    tree = got
    gpu.rollback(point)
    path_chain = gpu.verify(feed[[0, 2, 8, 9]], 37)
    assert gc.logit_error(tree[[0, 2, 8, 9]], path_chain) <= 2e-3
    # compaction: after gathering that path the next token's logits equal the chain's continuation
    nxt = gpu.produce(int(feed[10]), 41)
    gpu.rollback(point)
    gpu.verify_tree(feed, parent, 37)
    gpu.compact_tree(37, [0, 2, 8, 9])
    gpu.rollback_retaining(point, 4)
    nxt2 = gpu.produce(int(feed[10]), 41)
    assert gc.logit_error(nxt2[None], nxt[None]) <= 2e-3


def test_refusals_by_name():
    from turbospark_amd import TsvError
    cfg, w, gpu, cpu = gc.build_pair("tiny_q8_0", max_context=24)
    with pytest.raises(TsvError, match="cursor"):
        gpu.verify([1, 2], 3)
    with pytest.raises(TsvError, match="vocabulary"):
        gpu.verify([cfg["vocab"]], 0)
    with pytest.raises(TsvError, match="more rows"):
        gpu.verify(list(range(17)), 0)
    gpu.verify(list(range(16)), 0)
    with pytest.raises(TsvError, match="capacity"):
        gpu.verify(list(range(9)), 16)
    with pytest.raises(TsvError, match="parent"):
        gpu.verify_tree([1, 2], [-1, 1], 16)
    assert gpu.position == 16
    # a rollback retires the pass: its logits must not be judged at a position behind the cursor's past
    import turbospark_amd as ts
    gpu.rollback(ts.ffi.Point(8))
    with pytest.raises(TsvError, match="last verify pass"):
        gpu.accept(list(range(16)), 0, ts.shaping(0.0))
    assert gpu.position == 8
    point = gpu.checkpoint()
    gpu.verify([1, 2, 3], 8, want_logits=False)
    gpu.rollback_retaining(point, 1)
    with pytest.raises(TsvError, match="last verify pass"):
        gpu.accept([1, 2, 3], 8, ts.shaping(0.0))
    assert gpu.position == 9


def test_graph_replay_of_the_pass_equals_plain_launches():
    """The opt-in captured launch sequence (one graph per row count; positions, tokens and the tree
    shape are read from device memory at replay): every replay, with eager work and
    synchronisations between them, must give the bits the plain launches give."""
    import os
    import turbospark_amd as ts
    from turbospark_amd import synth
    cfg = dict(synth.CONFIGS["small_q4_k"], max_context=160)
    w = synth.make_weights(cfg, seed=5)
    plain = ts.HipVerifier(cfg, w)
    os.environ["TSV_GRAPH"] = "1"
    try:
        graph = ts.HipVerifier(cfg, w)
    finally:
        os.environ["TSV_GRAPH"] = "0"
    prompt = _prompt(37, cfg["vocab"], 3)
    for eng in (plain, graph):
        eng.prefill(prompt, 0, want_logits=False)
    rng = np.random.default_rng(9)
    base = 37
    for rnd, m in enumerate([5, 5, 3, 5, 16, 5, 3]):
        feed = rng.integers(0, cfg["vocab"], m).astype(np.int32)
        a = plain.verify(feed, base)
        b = graph.verify(feed, base)
        assert np.array_equal(a, b), (rnd, m)
        keep = 1 + rnd % 3                      # eager work between replays: a partial rollback
        for eng in (plain, graph):
            eng.rollback(ts.ffi.Point(base + keep))
        base += keep
    parent = [-1, 0, 0, 1, 1]
    feed = rng.integers(0, cfg["vocab"], 5).astype(np.int32)
    assert np.array_equal(plain.verify_tree(feed, parent, base), graph.verify_tree(feed, parent, base))
