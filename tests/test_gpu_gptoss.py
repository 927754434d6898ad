"""GPU parity of the gpt-oss arrangement (crates/runtime/src/families/gptoss/mod.rs:11-23) against
the oracle: bf16 attention / router / head with projection biases, YaRN rotation, attention sinks,
a sliding window on even layers, MXFP4 experts with biases and the clamped SwiGLU, hidden and
expert widths that are not whole 256-element chunks."""
import numpy as np
import pytest

from oracle import binding as ob
from tests import gpu_common as gc
from tests.test_gpu_moe import _clean_inputs, _prompt

pytestmark = pytest.mark.gpu

TOL = 1e-2   # max-abs logit error relative to the logit range (the MXFP4 bar)


@pytest.mark.parametrize("ctx,k", [(40, 8), (23, 4), (49, 15), (16, 0)])
def test_gptoss_verify_logits_match_the_oracle(ctx, k):
    cfg, w, gpu, cpu = gc.build_pair("gptoss_small", max_context=ctx + 32)
    prompt, feed, want, margin = _clean_inputs(cfg, cpu, ctx, k)
    gpu.prefill(prompt, 0, want_logits=False)
    got = gpu.verify(feed, ctx)
    err = gc.logit_error(got, want)
    print(f"gptoss_small ctx={ctx} m={k+1}: max-abs logit error / range = {err:.2e}, route margin {margin:.3e}")
    assert err <= TOL, err
    for layer in range(cfg["n_layers"]):
        kg, vg = gpu.read_kv(layer, 0, ctx)
        kc, vc = cpu.kv(layer)
        assert np.abs(kg.astype(np.float32) - kc[:ctx]).max() <= 2e-2 * np.abs(kc[:ctx]).max()
        assert np.abs(vg.astype(np.float32) - vc[:ctx]).max() <= 2e-2 * np.abs(vc[:ctx]).max()


def test_projection_biases_and_yarn_with_128_wide_heads():
    """The same arrangement with 128-wide heads: the fused q/k/v projection then holds the rows of
    q and k in rotation-pair order (a load-time row map), and its biases, the YaRN table and the K / V
    cache stores must follow that order (families/gptoss/attn.rs:88-118)."""
    over = dict(head_dim=128, n_q_heads=4, n_kv_heads=1, hidden=576)
    cfg, w, gpu, cpu = gc.build_pair("gptoss_small", max_context=96, **over)
    ctx = 40
    prompt, feed, want, margin = _clean_inputs(cfg, cpu, ctx, 8)
    gpu.prefill(prompt, 0, want_logits=False)
    got = gpu.verify(feed, ctx)
    err = gc.logit_error(got, want)
    print(f"gptoss_small with 128-wide heads: max-abs logit error / range = {err:.2e}")
    assert err <= TOL, err
    for layer in range(cfg["n_layers"]):
        kg, vg = gpu.read_kv(layer, 0, ctx + 9)
        kc, vc = cpu.kv(layer)
        assert np.abs(kg.astype(np.float32) - kc[:ctx + 9]).max() <= 2e-2 * np.abs(kc[:ctx + 9]).max()
        assert np.abs(vg.astype(np.float32) - vc[:ctx + 9]).max() <= 2e-2 * np.abs(vc[:ctx + 9]).max()


def test_gptoss_tree_rows_and_batch_invariance():
    cfg, w, gpu, cpu = gc.build_pair("gptoss_small", max_context=96)
    ctx = 37
    prompt, feed, _, _ = _clean_inputs(cfg, cpu, ctx, 15)
    parent = [-1, 0, 0, 0, 0, 1, 5, 6, 2, 8, 9, 3, 11, 12, 4, 14]
    gpu.prefill(prompt, 0, want_logits=False)
    point = gpu.checkpoint()
    got = gpu.verify_tree(feed, parent, ctx)
    cpu.rewind_to(ctx)
    want = cpu.verify(feed, ctx, parent=parent)
    assert cpu.route_margin > 5e-4
    assert gc.logit_error(got, want) <= TOL
    # a chain pass equals the same tokens fed one at a time, bit for bit
    gpu.rollback(point)
    batch = gpu.verify(feed[:9], ctx)
    gpu.rollback(point)
    seq = np.stack([gpu.produce(t, ctx + i) for i, t in enumerate(feed[:9])])
    assert np.array_equal(batch, seq)


def test_gptoss_sampled_round_on_the_device():
    """Configuration-5 style round: chain k = 8, T = 1.0 rejection on the gpt-oss target's logits."""
    import turbospark_amd as ts
    cfg, w, gpu, cpu = gc.build_pair("gptoss_small", max_context=96)
    prompt = _prompt(30, cfg["vocab"], 5)
    gpu.prefill(prompt, 0, want_logits=False)
    base = gpu.position
    rng = np.random.default_rng(8)
    for seed in range(6):
        gcfg, ocfg = ts.shaping(1.0, seed=seed), ob.shaping(1.0, seed=seed)
        draft = rng.standard_normal((8, cfg["vocab"])).astype(np.float16)
        props, ds = gpu.draft_chain(draft, gcfg, 0)
        feed = [3] + [int(t) for t in props]
        res, logits = gpu.verify_accept(feed, base, gcfg, draft_logits=draft, draw_step=ds, want_logits=True)
        want = ob.chain_round(logits, draft, props, ocfg, history=list(prompt) + [3], draw_step=ds)
        assert (res.accepted, res.committed, res.next, res.draw_step) == \
            (want["accepted"], want["committed"], want["next"], want["draw_step"])
        assert res.min_margin > 1e-9
        gpu.rollback(ts.ffi.Point(base))


def test_a_rewind_deeper_than_the_window_is_safe_in_the_linear_layout(monkeypatch):
    """`KvCacheManager::max_safe_rewind` (crates/gpu/src/kv_cache_rewind.rs:26-35) bounds a rollback by
    the ring's slack; without `ring` the windowed layers store position p at slot p, so it is unbounded: after
    rolling back 40 rows (the window is 24) the continuation equals, by bits, a run that never went
    further.  (Both runs in 16-row passes: a 64-row pass sums in another order, so its rows differ from a
    16-row pass's in the last bits and the comparison by bits would measure that instead.)"""
    import turbospark_amd as ts
    monkeypatch.setenv("TSV_WIDE_PREFILL", "0")
    cfg, w, gpu, cpu = gc.build_pair("gptoss_small", max_context=128)
    assert gpu.max_safe_rewind() == 2 ** 63 - 1
    prompt = _prompt(80, cfg["vocab"], 5)
    tail = _prompt(6, cfg["vocab"], 6)
    gpu.prefill(prompt, 0, want_logits=False)
    gpu.rollback(ts.ffi.Point(40))
    assert gpu.position == 40
    a = gpu.verify(tail, 40)
    gpu.reset()
    gpu.prefill(prompt[:40], 0, want_logits=False)
    b = gpu.verify(tail, 40)
    assert np.array_equal(a, b)


def _ring_pair(name, max_context, n_layers=None, seed=1234, **over):
    """The same weights twice: windowed layers as rings (kv_cache.rs:122-131) and in the linear layout."""
    import turbospark_amd as ts
    from turbospark_amd import synth
    cfg = dict(synth.CONFIGS[name], max_context=max_context, **over)
    if n_layers:
        cfg["n_layers"] = n_layers
    w = synth.make_weights(cfg, seed=seed, n_layers=n_layers)
    # (both handles are held to 16-row prompt passes, so that "equal by bits" compares the two layouts: inside a
    #  64-row pass a ring layer attends block by block while a linear one attends the four blocks at once, and a
    #  64-row matmul sums in another order than a 16-row one)
    import os
    ringed = dict(w, layers=[dict(lw, ring=1 if lw.get("window") else 0) for lw in w["layers"]])
    os.environ["TSV_WIDE_PREFILL"] = "0"
    try:
        return cfg, ts.HipVerifier(cfg, w), ts.HipVerifier(cfg, ringed)
    finally:
        del os.environ["TSV_WIDE_PREFILL"]


def test_windowed_layers_as_rings_equal_the_linear_layout_by_bits():
    """N rows fed through both layouts, far past the ring's capacity (window 24 -> a ring of 64 slots):
    prompt passes, verify passes, rollbacks inside the budget, a tree pass with compaction across the
    ring's seam -- every logit equal by bits; the budget is capacity - window
    (kv_cache_rewind.rs:26-35) and a rollback beyond it is refused by name (:46-55)."""
    import turbospark_amd as ts
    from turbospark_amd import TsvError
    cfg, lin, ring = _ring_pair("gptoss_small", 400)
    V = cfg["vocab"]
    assert lin.max_safe_rewind() == 2 ** 63 - 1 and ring.max_safe_rewind() == 64 - 24
    prompt = _prompt(150, V, 5)
    a = lin.prefill(prompt, 0)
    b = ring.prefill(prompt, 0)
    assert np.array_equal(a, b)
    rng = np.random.default_rng(2)
    base = 150
    for rnd in range(30):                       # verify, keep a few rows, continue: crosses the seam several times
        m = int(rng.integers(1, 17))
        feed = rng.integers(0, V, m).astype(np.int32)
        pa, pb = lin.checkpoint(), ring.checkpoint()
        assert np.array_equal(lin.verify(feed, base), ring.verify(feed, base)), rnd
        keep = int(rng.integers(1, m + 1))
        lin.rollback_retaining(pa, keep)
        ring.rollback_retaining(pb, keep)
        base += keep
        assert lin.position == ring.position == base
    # a tree pass whose rows straddle the seam, compacted
    parent = [-1, 0, 0, 1, 1, 2, 3, 5]
    feed = rng.integers(0, V, 8).astype(np.int32)
    for eng in (lin, ring):
        eng.verify_tree(feed, parent, base, want_logits=False)
        eng.compact_tree(base, [0, 2, 5, 7])
        eng.rollback_retaining(ts.ffi.Point(base), 4)
    nxt = rng.integers(0, V, 3).astype(np.int32)
    assert np.array_equal(lin.verify(nxt, base + 4), ring.verify(nxt, base + 4))
    base += 8                                   # one past the last row ever written (the tree's eighth row)
    # the budget: 40 rows behind the last row written is the limit
    ring.rollback(ts.ffi.Point(base - 40))
    lin.rollback(ts.ffi.Point(base - 40))
    assert np.array_equal(lin.verify(nxt, base - 40), ring.verify(nxt, base - 40))
    with pytest.raises(TsvError, match="exceeds the ring slack"):
        ring.rollback(ts.ffi.Point(base - 41))
    assert ring.position == base - 37
    with pytest.raises(TsvError, match="no longer holds"):
        ring.read_kv(0, 0, 4)                   # layer 0 slides: its first rows are long overwritten
    k_full, _ = ring.read_kv(1, 0, 4)           # layer 1 is full attention: everything is there
    assert np.array_equal(k_full, lin.read_kv(1, 0, 4)[0])
    k_ring, v_ring = ring.read_kv(0, base - 60, 20)
    k_lin, v_lin = lin.read_kv(0, base - 60, 20)
    assert np.array_equal(k_ring, k_lin) and np.array_equal(v_ring, v_lin)
    # a reset starts the ring over
    ring.reset()
    lin.reset()
    assert np.array_equal(lin.prefill(prompt[:70], 0), ring.prefill(prompt[:70], 0))


def test_after_rejected_rounds_the_rewind_budget_counts_from_the_last_row_written():
    """Rounds that write sixteen rows and keep one (everything else rejected) leave the cursor fifteen rows
    behind the last row written; the rows of a ring are overwritten up to that row, so the budget
    (capacity - window = 40, kv_cache_rewind.rs:26-35) is counted from it: a rollback may go 40 rows below the
    last row written -- 25 committed rows here -- and one row more is refused by name.  The rings give the
    linear layout's logits after that deepest rollback."""
    import turbospark_amd as ts
    from turbospark_amd import TsvError
    cfg, lin, ring = _ring_pair("gptoss_small", 400)
    V = cfg["vocab"]
    prompt = _prompt(120, V, 9)
    assert np.array_equal(lin.prefill(prompt, 0), ring.prefill(prompt, 0))
    rng = np.random.default_rng(4)
    base = 120
    for rnd in range(30):
        feed = rng.integers(0, V, 16).astype(np.int32)
        pa, pb = lin.checkpoint(), ring.checkpoint()
        assert np.array_equal(lin.verify(feed, base), ring.verify(feed, base)), rnd
        lin.rollback_retaining(pa, 1)
        ring.rollback_retaining(pb, 1)
        base += 1
    written = base + 15                          # one past the last row written: the last round's sixteenth row
    assert ring.position == base
    with pytest.raises(TsvError, match="exceeds the ring slack"):
        ring.rollback(ts.ffi.Point(written - 41))
    assert ring.position == base                 # a refused rollback moves nothing
    ring.rollback(ts.ffi.Point(written - 40))    # 25 committed rows back
    lin.rollback(ts.ffi.Point(written - 40))
    nxt = rng.integers(0, V, 5).astype(np.int32)
    assert np.array_equal(lin.verify(nxt, written - 40), ring.verify(nxt, written - 40))


def test_gptoss_120b_geometry_ring_equals_linear_at_long_context():
    """The gpt-oss-120B geometry (window 128 -> a ring of 160 slots beside a 3000-token context): seeded
    rows written into both layouts, a nine-row pass, a rollback and a second pass, equal by bits."""
    import turbospark_amd as ts
    ctx = 3000
    cfg, lin, ring = _ring_pair("gptoss_120b", ctx + 64, n_layers=2, vocab=4096)
    rng = np.random.default_rng(3)
    shape = (ctx, cfg["n_kv_heads"], cfg["head_dim"])
    for layer in range(2):
        k = (rng.standard_normal(shape) * 0.5).astype(np.float16)
        v = (rng.standard_normal(shape) * 0.5).astype(np.float16)
        lin.write_kv(layer, 0, k, v)
        ring.write_kv(layer, 0, k, v)
    assert ring.position == lin.position == ctx and ring.max_safe_rewind() == 160 - 128
    feed = rng.integers(0, cfg["vocab"], 9).astype(np.int32)
    pa, pb = lin.checkpoint(), ring.checkpoint()
    assert np.array_equal(lin.verify(feed, ctx), ring.verify(feed, ctx))
    lin.rollback_retaining(pa, 3)
    ring.rollback_retaining(pb, 3)
    feed2 = rng.integers(0, cfg["vocab"], 9).astype(np.int32)
    assert np.array_equal(lin.verify(feed2, ctx + 3), ring.verify(feed2, ctx + 3))
