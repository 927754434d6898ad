"""Prompt passes of 64 rows (crates/runtime/src/producer.rs:122-150, ChunkedPrefillRunner; families/llama/prefill.rs):
the cache they fill and the logits that follow, against the oracle and against the 16-row passes of the same
library.  The two GPU paths multiply the same integers by the same fp16 activations and differ in the order of
the fp32 additions only, so they agree to a few fp16 ulps per layer, not by bits."""
import os

import numpy as np
import pytest

from tests import gpu_common as gc

pytestmark = pytest.mark.gpu


def _engine(cfg, weights, wide):
    import turbospark_amd as ts
    os.environ["TSV_WIDE_PREFILL"] = "1" if wide else "0"
    try:
        return ts.HipVerifier(cfg, weights)
    finally:
        del os.environ["TSV_WIDE_PREFILL"]


@pytest.mark.parametrize("name,n_prompt", [("small_q4_k", 150), ("small_q4_k", 64), ("xcd_q4_k", 200), ("small_q4_k", 129),
                                           ("tiny_q8_0", 150), ("xcd_q8_0", 200), ("tiny_q8_0", 64),
                                           ("small_q4_k_m", 150), ("small_q5_k_m", 150)])   # the K-quant mixes: Q6_K value / down matrices
def test_a_prompt_fed_in_blocks_of_64_fills_the_cache_the_oracle_fills(name, n_prompt):
    from turbospark_amd import synth
    from oracle import binding as ob
    cfg = dict(synth.CONFIGS[name], max_context=n_prompt + 48)
    w = synth.make_weights(cfg, seed=11)
    wide, narrow = _engine(cfg, w, True), _engine(cfg, w, False)
    cpu = ob.Model(cfg, w, round_kv_f16=True, threads=16)
    rng = np.random.default_rng(2)
    prompt = rng.integers(0, cfg["vocab"], n_prompt).astype(np.int32)
    feed = rng.integers(0, cfg["vocab"], 5).astype(np.int32)
    wide.prefill(prompt, 0, want_logits=False)
    narrow.prefill(prompt, 0, want_logits=False)
    for i in range(0, n_prompt, 16):
        cpu.verify(prompt[i:i + 16], i)
    assert wide.position == narrow.position == n_prompt
    for layer in range(cfg["n_layers"]):
        kw, vw = wide.read_kv(layer, 0, n_prompt)
        kn, vn = narrow.read_kv(layer, 0, n_prompt)
        kc, vc = cpu.kv(layer)
        for got, other, want in ((kw, kn, kc), (vw, vn, vc)):
            got, other, want = got.astype(np.float32), other.astype(np.float32), want[:n_prompt]
            scale = np.abs(want).max()
            assert np.abs(got - want).max() <= 2e-2 * scale
            # the two GPU paths: a few fp16 ulps of the largest value
            assert np.abs(got - other).max() <= 4e-3 * scale, (layer, np.abs(got - other).max() / scale)
    want = cpu.verify(feed, n_prompt)
    got_w, got_n = wide.verify(feed, n_prompt), narrow.verify(feed, n_prompt)
    err_w, err_n, err_wn = gc.logit_error(got_w, want), gc.logit_error(got_n, want), gc.logit_error(got_w, got_n)
    print(f"{name}, prompt of {n_prompt}: logits after 64-row passes vs oracle {err_w:.2e}, after 16-row passes {err_n:.2e}, "
          f"the two GPU paths {err_wn:.2e}")
    assert err_w <= gc.TOL.get(cfg["dtype"], 1e-2) and err_wn <= 2e-3


@pytest.mark.parametrize("name,over", [("small_q4_k", {}), ("xcd_q8_0", {}), ("xcd_q8_0", dict(qk_norm=True)),
                                       ("xcd_q8_0", dict(dtype="bf16")), ("small_q4_k", dict(dtype="bf16", qk_norm=True))])
def test_wide_passes_where_the_rotation_is_a_kernel_of_its_own(name, over, monkeypatch):
    """Models whose q/k/v projection does not rotate its own rows (heavy tiles, per-head q / k norms -- here forced by
    TSV_ROPE_FUSED=0 as well): the 64-row projection leaves partial sums and the 16-row pass's rotation kernel runs
    once per block of sixteen."""
    from turbospark_amd import synth
    from oracle import binding as ob
    from turbospark_amd import ffi
    if over.get("dtype") == "bf16":
        over = dict(over, dtype=ffi.BF16)
    if not (over.get("dtype") == ffi.BF16 and not over.get("qk_norm")):   # (one bf16 case keeps the rotating epilogue)
        monkeypatch.setenv("TSV_ROPE_FUSED", "0")
    n_prompt = 150
    cfg = dict(synth.CONFIGS[name], max_context=n_prompt + 48, **over)
    w = synth.make_weights(cfg, seed=21)
    wide, narrow = _engine(cfg, w, True), _engine(cfg, w, False)
    cpu = ob.Model(cfg, w, round_kv_f16=True, threads=16)
    rng = np.random.default_rng(5)
    prompt = rng.integers(0, cfg["vocab"], n_prompt).astype(np.int32)
    feed = rng.integers(0, cfg["vocab"], 5).astype(np.int32)
    wide.prefill(prompt, 0, want_logits=False)
    narrow.prefill(prompt, 0, want_logits=False)
    for i in range(0, n_prompt, 16):
        cpu.verify(prompt[i:i + 16], i)
    for layer in range(cfg["n_layers"]):
        (kw, vw), (kn, vn), (kc, vc) = wide.read_kv(layer, 0, n_prompt), narrow.read_kv(layer, 0, n_prompt), cpu.kv(layer)
        for got, other, want in ((kw, kn, kc), (vw, vn, vc)):
            got, other, want = got.astype(np.float32), other.astype(np.float32), want[:n_prompt]
            scale = np.abs(want).max()
            assert np.abs(got - want).max() <= 2e-2 * scale
            assert np.abs(got - other).max() <= 4e-3 * scale
    want = cpu.verify(feed, n_prompt)
    got_w, got_n = wide.verify(feed, n_prompt), narrow.verify(feed, n_prompt)
    err_w, err_wn = gc.logit_error(got_w, want), gc.logit_error(got_w, got_n)
    print(f"{name} {over}: logits after 64-row passes vs oracle {err_w:.2e}, the two GPU paths {err_wn:.2e}")
    assert err_w <= gc.TOL.get(cfg["dtype"], 1e-2) and err_wn <= 2e-3


@pytest.mark.parametrize("name,n_prompt,seed,over", [
    ("moe_small", 150, 31, {}), ("gptoss_small", 150, 31, {}), ("moe_small", 64, 32, {}), ("gptoss_small", 200, 33, {}),
    # many experts, few slots: an expert has two members on average (the four-members-at-a-time walk); the cases above
    # give an expert sixteen or eight (the sixteen-at-a-time walk of an expert many rows chose, and the mix of both)
    ("moe_small", 150, 35, dict(n_experts=64, top_k=2)), ("gptoss_small", 150, 36, dict(n_experts=128, top_k=4))])
def test_routed_layers_in_passes_of_64_rows(name, n_prompt, seed, over):
    """Routed experts over the 64 rows of a prompt pass: every expert is multiplied once against all the rows of the
    pass that chose it (crates/runtime/src/families/llama/moe.rs, the grouping of moe.hip taken to 64 rows).  Held to
    the oracle and to the 16-row passes of the same library.  (The rows' inputs to the router differ by rounding
    between the two GPU paths, so a near tie can fall either way; these seeds have none inside that band, and the
    selections of the following verify pass are compared to say so.)"""
    from turbospark_amd import synth
    from oracle import binding as ob
    cfg = dict(synth.CONFIGS[name], max_context=n_prompt + 48, **over)
    w = synth.make_weights(cfg, seed=seed)
    wide, narrow = _engine(cfg, w, True), _engine(cfg, w, False)
    cpu = ob.Model(cfg, w, round_kv_f16=True, threads=16)
    rng = np.random.default_rng(seed)
    prompt = rng.integers(0, cfg["vocab"], n_prompt).astype(np.int32)
    feed = rng.integers(0, cfg["vocab"], 5).astype(np.int32)
    wide.prefill(prompt, 0, want_logits=False)
    narrow.prefill(prompt, 0, want_logits=False)
    for i in range(0, n_prompt, 16):
        cpu.verify(prompt[i:i + 16], i)
    assert wide.position == narrow.position == n_prompt
    for layer in range(cfg["n_layers"]):
        (kw, vw), (kn, vn), (kc, vc) = wide.read_kv(layer, 0, n_prompt), narrow.read_kv(layer, 0, n_prompt), cpu.kv(layer)
        for got, other, want in ((kw, kn, kc), (vw, vn, vc)):
            got, other, want = got.astype(np.float32), other.astype(np.float32), want[:n_prompt]
            scale = np.abs(want).max()
            assert np.abs(got - want).max() <= 2e-2 * scale, (layer, np.abs(got - want).max() / scale)
            assert np.abs(got - other).max() <= 4e-3 * scale, (layer, np.abs(got - other).max() / scale)
    want = cpu.verify(feed, n_prompt)
    got_w, got_n = wide.verify(feed, n_prompt), narrow.verify(feed, n_prompt)
    k = cfg["top_k"]
    assert np.array_equal(wide.route_selected()[:, :5, :k], narrow.route_selected()[:, :5, :k])
    err_w, err_wn = gc.logit_error(got_w, want), gc.logit_error(got_w, got_n)
    print(f"{name}, prompt of {n_prompt}: logits after 64-row passes vs oracle {err_w:.2e}, the two GPU paths {err_wn:.2e}")
    assert err_w <= 1e-2 and err_wn <= 2e-3


@pytest.mark.parametrize("name", ["small_q4_k", "xcd_q4_k", "tiny_q8_0"])
def test_the_rotating_epilogue_in_64_row_passes(name, monkeypatch):
    """TSV_WIDE_ROPE_FUSED=1 keeps the projection that rotates and stores its own rows (one workgroup per tile) in the
    64-row passes as well; by default they split the projection along K and leave the rotation to its kernel."""
    from turbospark_amd import synth
    from oracle import binding as ob
    cfg = dict(synth.CONFIGS[name], max_context=200)
    w = synth.make_weights(cfg, seed=17)
    monkeypatch.setenv("TSV_WIDE_ROPE_FUSED", "1")
    fused = _engine(cfg, w, True)
    monkeypatch.delenv("TSV_WIDE_ROPE_FUSED")
    split = _engine(cfg, w, True)
    cpu = ob.Model(cfg, w, round_kv_f16=True, threads=16)
    rng = np.random.default_rng(9)
    prompt = rng.integers(0, cfg["vocab"], 150).astype(np.int32)
    feed = rng.integers(0, cfg["vocab"], 5).astype(np.int32)
    fused.prefill(prompt, 0, want_logits=False)
    split.prefill(prompt, 0, want_logits=False)
    for i in range(0, 150, 16):
        cpu.verify(prompt[i:i + 16], i)
    for layer in range(cfg["n_layers"]):
        (kf, vf), (ks, vs), (kc, vc) = fused.read_kv(layer, 0, 150), split.read_kv(layer, 0, 150), cpu.kv(layer)
        for got, other, want in ((kf, ks, kc), (vf, vs, vc)):
            got, other, want = got.astype(np.float32), other.astype(np.float32), want[:150]
            scale = np.abs(want).max()
            assert np.abs(got - want).max() <= 2e-2 * scale and np.abs(got - other).max() <= 4e-3 * scale
    want = cpu.verify(feed, 150)
    a, b = fused.verify(feed, 150), split.verify(feed, 150)
    print(f"{name}: epilogue {gc.logit_error(a, want):.2e}, split {gc.logit_error(b, want):.2e}, between {gc.logit_error(a, b):.2e}")
    assert gc.logit_error(a, want) <= gc.TOL.get(cfg["dtype"], 1e-2) and gc.logit_error(a, b) <= 2e-3


@pytest.mark.parametrize("kv_bits", [None, (4, 4)])
def test_ring_layers_take_the_blocks_of_a_64_row_pass_one_after_the_other(kv_bits):
    """Windowed layers as rings (kv_cache.rs:122-131: window 24 -> a ring of 64 slots, fewer than a 64-row pass would
    write ahead of its first block's window): inside a 64-row pass such a layer stores and attends block by block, the
    cache states of four 16-row passes.  A 300-token prompt wraps the ring several times; then verify passes and
    rollbacks inside the budget, against the oracle and against the 16-row passes of the same library."""
    import turbospark_amd as ts
    from turbospark_amd import synth
    from oracle import binding as ob
    cfg = dict(synth.CONFIGS["gptoss_small"], max_context=400)
    w = synth.make_weights(cfg, seed=41)
    ringed = dict(w, layers=[dict(lw, ring=1 if lw.get("window") else 0) for lw in w["layers"]])
    kw = dict(kv_bits=kv_bits) if kv_bits else {}

    def engine(wide):
        os.environ["TSV_WIDE_PREFILL"] = "1" if wide else "0"
        try:
            return ts.HipVerifier(cfg, ringed, **kw)
        finally:
            del os.environ["TSV_WIDE_PREFILL"]

    wide, narrow = engine(True), engine(False)
    assert wide.max_safe_rewind() == narrow.max_safe_rewind() == 64 - 24
    cpu = ob.Model(cfg, w, round_kv_f16=True, threads=16, **kw)
    rng = np.random.default_rng(41)
    n = 300
    prompt = rng.integers(0, cfg["vocab"], n).astype(np.int32)
    wide.prefill(prompt, 0, want_logits=False)
    narrow.prefill(prompt, 0, want_logits=False)
    for i in range(0, n, 16):
        cpu.verify(prompt[i:i + 16], i)
    base = n
    bound = 5e-2 if kv_bits else 1e-2
    errs = []
    for rnd in range(6):
        m = int(rng.integers(3, 17))
        feed = rng.integers(0, cfg["vocab"], m).astype(np.int32)
        pw, pn = wide.checkpoint(), narrow.checkpoint()
        got_w, got_n, want = wide.verify(feed, base), narrow.verify(feed, base), cpu.verify(feed, base)
        errs.append((gc.logit_error(got_w, want), gc.logit_error(got_w, got_n)))
        keep = int(rng.integers(1, m + 1))
        wide.rollback_retaining(pw, keep)
        narrow.rollback_retaining(pn, keep)
        cpu.rewind_to(base + keep)
        base += keep
    print(f"rings, kv_bits {kv_bits}: (vs oracle, vs 16-row passes) per round", [f"{a:.1e}/{b:.1e}" for a, b in errs])
    assert max(a for a, _ in errs) <= bound and max(b for _, b in errs) <= (bound if kv_bits else 2e-3)


def test_logits_of_the_last_prompt_token_after_wide_passes():
    """tsv_prefill hands out the last row's logits: the rows before it go in blocks of 64, the tail in
    16-row passes whose last one carries the output head."""
    from turbospark_amd import synth
    from oracle import binding as ob
    cfg = dict(synth.CONFIGS["small_q4_k"], max_context=256)
    w = synth.make_weights(cfg, seed=12)
    wide = _engine(cfg, w, True)
    cpu = ob.Model(cfg, w, round_kv_f16=True, threads=16)
    prompt = np.random.default_rng(3).integers(0, cfg["vocab"], 128).astype(np.int32)  # exactly two blocks: the second is not wide
    got = wide.prefill(prompt, 0, want_logits=True)
    want = None
    for i in range(0, 128, 16):
        want = cpu.verify(prompt[i:i + 16], i)
    err = gc.logit_error(got.reshape(1, -1), want[-1:])
    print(f"last prompt row after wide passes: {err:.2e}")
    assert err <= 1e-2
    assert wide.position == 128


def test_wide_passes_are_deterministic_and_leave_the_prefix_record_intact():
    from turbospark_amd import synth
    cfg = dict(synth.CONFIGS["small_q4_k"], max_context=256)
    w = synth.make_weights(cfg, seed=13)
    a, b = _engine(cfg, w, True), _engine(cfg, w, True)
    prompt = np.random.default_rng(4).integers(0, cfg["vocab"], 200).astype(np.int32)
    a.prefill(prompt, 0, want_logits=False)
    b.prefill(prompt[:70], 0, want_logits=False)     # another split of the same prompt: 64 + 6, then 64 + 64 + 2
    b.prefill(prompt[70:], 70, want_logits=False)
    feed = prompt[:4]
    la, lb = a.verify(feed, 200), b.verify(feed, 200)
    assert gc.logit_error(la, lb) <= 2e-3
    a.reset()
    a.prefill(prompt, 0, want_logits=False)
    assert np.array_equal(a.verify(feed, 200), la)
