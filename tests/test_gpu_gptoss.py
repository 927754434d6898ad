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


def test_a_rewind_deeper_than_the_window_is_safe_in_the_linear_layout():
    """`KvCacheManager::max_safe_rewind` (crates/gpu/src/kv_cache_rewind.rs:26-35) bounds a rollback by
    the ring's slack; the windowed layers here store position p at slot p, so it is unbounded: after
    rolling back 40 rows (the window is 24) the continuation equals, by bits, a run that never went
    further."""
    import turbospark_amd as ts
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
