"""Parity at the benchmark configurations' real shapes: two layers + output head of the Llama-3-8B
geometry (hidden 4096, 32q / 8kv x 128, ffn 14336, vocab 128256, Q4_K) at a 4096-token context,
chain k = 4 and the 16-node tree; KV rows are seeded values written into both caches (prefilling
4096 tokens through the CPU oracle is not feasible), the new rows come from the pass itself."""
import numpy as np
import pytest

from oracle import binding as ob
from tests import gpu_common as gc

pytestmark = pytest.mark.gpu


def _filled(name, ctx, n_layers, seed=3, **over):
    import turbospark_amd as ts
    from turbospark_amd import synth
    cfg = dict(synth.CONFIGS[name])
    cfg.update(n_layers=n_layers, max_context=ctx + 32, **over)
    w = synth.make_weights(cfg, seed=seed, n_layers=n_layers)
    gpu = ts.HipVerifier(cfg, w)
    cpu = ob.Model(cfg, w, round_kv_f16=True, threads=16)
    rng = np.random.default_rng(seed)
    for layer in range(n_layers):
        shape = (ctx, cfg["n_kv_heads"], cfg["head_dim"])
        k = (rng.standard_normal(shape) * 0.5).astype(np.float16)
        v = (rng.standard_normal(shape) * 0.5).astype(np.float16)
        gpu.write_kv(layer, 0, k, v)
        kc, vc = cpu.kv(layer)
        kc[:ctx] = k.astype(np.float32)
        vc[:ctx] = v.astype(np.float32)
    cpu.rewind_to(ctx)
    assert gpu.position == ctx
    return cfg, gpu, cpu


def test_llama3_8b_shape_chain_and_tree_at_4096_context():
    import turbospark_amd as ts
    ctx = 4096
    cfg, gpu, cpu = _filled("llama3_8b_q4_k", ctx, 2)
    V = cfg["vocab"]
    rng = np.random.default_rng(1)
    feed = rng.integers(0, V, 5).astype(np.int32)
    point = gpu.checkpoint()
    got = gpu.verify(feed, ctx)
    want = cpu.verify(feed, ctx)
    err = gc.logit_error(got, want)
    print(f"8B shape, 2 layers, ctx 4096, m=5: max-abs logit error / range = {err:.2e}")
    assert err <= 1e-2
    # the new K rows of the pass agree too (rotation at positions 4096..4100)
    kg, vg = gpu.read_kv(1, ctx, 5)
    kc, vc = cpu.kv(1)
    assert np.abs(kg.astype(np.float32) - kc[ctx:ctx + 5]).max() <= 2e-2 * np.abs(kc[ctx:ctx + 5]).max()
    # acceptance at the full vocabulary on these logits, sampled T = 0.8: integers equal
    draft = rng.standard_normal((4, V)).astype(np.float16)
    gcfg, ocfg = ts.shaping(0.8, seed=9), ob.shaping(0.8, seed=9)
    res = gpu.accept(feed, ctx, gcfg, draft_logits=draft, draw_step=3)
    ref = ob.chain_round(got, draft, feed[1:], ocfg, history=[0] * ctx + [int(feed[0])], draw_step=3)
    assert (res.accepted, res.committed, res.next, res.draw_step) == (ref["accepted"], ref["committed"], ref["next"], ref["draw_step"])
    # the same with penalties over a 4097-token history that touches a few thousand vocabulary entries,
    # a drafter close to the target (so proposals are accepted and later rows count them) and truncation
    hist = [int(t) for t in rng.integers(0, V, ctx)] + [int(feed[0])]
    near = (gc.f16(got)[:4] + rng.standard_normal((4, V)).astype(np.float32) * 0.3).astype(np.float16)
    for seed, kw in enumerate([dict(repetition_penalty=1.3), dict(presence_penalty=0.7, frequency_penalty=0.3, top_p=0.9),
                               dict(repetition_penalty=1.1, frequency_penalty=0.2, top_k=50, min_p=0.01)]):
        gcfg, ocfg = ts.shaping(0.8, seed=seed, **kw), ob.shaping(0.8, seed=seed, **kw)
        props, ds = gpu.draft_chain(near, gcfg, 7, history=hist, generated=600)
        oprops, ods = ob.draft_chain(near, ocfg, hist, 600, 7)
        assert list(props) == list(oprops) and ds == ods
        res = gpu.accept(feed, ctx, gcfg, draft_logits=near, draw_step=3, history=hist, generated=600)
        ref = ob.chain_round(got, near, feed[1:], ocfg, history=hist, generated=600, draw_step=3)
        assert (res.accepted, res.committed, res.next, res.draw_step) == (ref["accepted"], ref["committed"], ref["next"], ref["draw_step"])
    # the 16-node tree of configuration 3 on the same cache
    gpu.rollback(point)
    cpu.rewind_to(ctx)
    parent = [-1, 0, 0, 0, 0, 1, 5, 6, 2, 8, 9, 3, 11, 12, 4, 14]
    feed = rng.integers(0, V, 16).astype(np.int32)
    got = gpu.verify_tree(feed, parent, ctx)
    want = cpu.verify(feed, ctx, parent=parent)
    err = gc.logit_error(got, want)
    print(f"8B shape, 2 layers, ctx 4096, 16-node tree: max-abs logit error / range = {err:.2e}")
    assert err <= 1e-2
    draft = (gc.f16(got) + rng.standard_normal((16, V)).astype(np.float32)).astype(np.float16)
    gcfg, ocfg = ts.shaping(1.0, seed=2), ob.shaping(1.0, seed=2)
    res = gpu.accept(feed, ctx, gcfg, parent=parent, draft_logits=draft)
    ref = ob.tree_round_sampled(got, draft, feed, parent, ocfg, history=[0] * ctx)
    assert res.path == ref["path"] and res.next == ref["next"] and res.draw_step == ref["draw_step"]


def test_gptoss_120b_shape_one_windowed_and_one_full_layer_at_long_context():
    """Hidden 2880 (not whole 256-chunks), 64q / 8kv x 64, 128 experts top-4 with biases, window 128
    on layer 0, full attention on layer 1, sinks, YaRN; vocabulary cut to 4096 to keep the CPU side short."""
    ctx = 3000
    cfg, gpu, cpu = _filled("gptoss_120b", ctx, 2, vocab=4096)
    for attempt in range(8):
        feed = np.random.default_rng(20 + attempt).integers(0, cfg["vocab"], 9).astype(np.int32)
        cpu.rewind_to(ctx)
        want = cpu.verify(feed, ctx)
        if cpu.route_margin > 2e-3:
            break
    else:
        raise AssertionError("no feed without a near-tie routing decision")
    got = gpu.verify(feed, ctx)
    err = gc.logit_error(got, want)
    print(f"gpt-oss-120B shape, 2 layers, ctx {ctx}, m=9: max-abs logit error / range = {err:.2e}, "
          f"route margin {cpu.route_margin:.2e}")
    assert err <= 1e-2


def test_gptoss_120b_shape_full_vocabulary_head_against_the_oracle():
    """The same geometry with its own output head: 201 088 rows of bf16 (the largest head of the five configurations,
    and the only bf16 one), two layers, a 512-token context, nine rows."""
    ctx = 512
    cfg, gpu, cpu = _filled("gptoss_120b", ctx, 2)
    assert cfg["vocab"] == 201088
    for attempt in range(8):
        feed = np.random.default_rng(60 + attempt).integers(0, cfg["vocab"], 9).astype(np.int32)
        cpu.rewind_to(ctx)
        want = cpu.verify(feed, ctx)
        if cpu.route_margin > 2e-3:
            break
    else:
        raise AssertionError("no feed without a near-tie routing decision")
    got = gpu.verify(feed, ctx)
    err = gc.logit_error(got, want)
    print(f"gpt-oss-120B shape, 2 layers, ctx {ctx}, m=9, vocab {cfg['vocab']}: max-abs logit error / range = {err:.2e}, "
          f"route margin {cpu.route_margin:.2e}")
    assert err <= 1e-2


def test_llama3_8b_all_32_layers_size_independent_properties():
    """The headline configuration at its real depth (32 layers, 4096-token context, vocabulary 128256),
    where the oracle cannot follow: properties that hold at any size.  A pass is deterministic by bits;
    a batched pass equals the same tokens fed one at a time by bits (families/qwen/batched.rs:92-110:
    verify == sequential decode); a chain-shaped tree equals the chain; a rollback to the checkpoint
    followed by the same pass reproduces it; the fused round equals verify followed by accept."""
    import turbospark_amd as ts
    from turbospark_amd import synth
    ctx = 4096
    cfg = dict(synth.CONFIGS["llama3_8b_q4_k"], max_context=ctx + 32)
    gpu = ts.HipVerifier(cfg, synth.make_weights(cfg, seed=3))
    rng = np.random.default_rng(3)
    shape = (ctx, cfg["n_kv_heads"], cfg["head_dim"])
    for layer in range(cfg["n_layers"]):
        gpu.write_kv(layer, 0, (rng.standard_normal(shape) * 0.5).astype(np.float16),
                     (rng.standard_normal(shape) * 0.5).astype(np.float16))
    assert gpu.position == ctx
    V = cfg["vocab"]
    feed = rng.integers(0, V, 5).astype(np.int32)
    point = gpu.checkpoint()
    a = gpu.verify(feed, ctx)
    gpu.rollback(point)
    b = gpu.verify(feed, ctx)
    assert np.array_equal(a, b)                       # deterministic, and the rollback left nothing behind
    gpu.rollback(point)
    seq = np.stack([gpu.produce(int(t), ctx + i) for i, t in enumerate(feed)])
    assert np.array_equal(a, seq)                     # batched == sequential
    gpu.rollback(point)
    t = gpu.verify_tree(feed, [-1, 0, 1, 2, 3], ctx)
    assert np.array_equal(a, t)                       # a chain-shaped tree is the chain
    gpu.rollback(point)
    draft = rng.standard_normal((4, V)).astype(np.float16)
    cfg_s = ts.shaping(0.8, seed=11, top_p=0.95, repetition_penalty=1.1)
    hist = [int(x) for x in rng.integers(0, V, 200)] + [int(feed[0])]
    fused = gpu.verify_accept(feed, ctx, cfg_s, draft_logits=draft, draw_step=9, history=hist, generated=50)
    gpu.rollback(point)
    gpu.verify(feed, ctx, want_logits=False)
    split = gpu.accept(feed, ctx, cfg_s, draft_logits=draft, draw_step=9, history=hist, generated=50)
    assert fused == split and fused.kv_position == ctx + fused.committed + 1
    ref = ob.chain_round(a, draft, feed[1:], ob.shaping(0.8, seed=11, top_p=0.95, repetition_penalty=1.1), history=hist,
                         generated=50, draw_step=9)
    assert (fused.accepted, fused.committed, fused.next, fused.draw_step) == \
        (ref["accepted"], ref["committed"], ref["next"], ref["draw_step"])


def test_llama3_8b_all_32_layers_tree_of_16_at_16384_context():
    """Configuration 3 at its real size (32 layers, 16384-token context, the 16-node tree, T = 1.0): a
    chain-shaped tree of 16 rows equals the chain by bits; the pass is deterministic; multi-branch
    rejection on the device equals the oracle's walk over the GPU's own logits; after compaction the
    cache continues like one that was only ever fed the accepted path (families/qwen/dflash_tree.rs:106-207)."""
    import turbospark_amd as ts
    from turbospark_amd import synth
    ctx = 16384
    cfg = dict(synth.CONFIGS["llama3_8b_q4_k"], max_context=ctx + 32)
    gpu = ts.HipVerifier(cfg, synth.make_weights(cfg, seed=3))
    rng = np.random.default_rng(4)
    shape = (ctx, cfg["n_kv_heads"], cfg["head_dim"])
    for layer in range(cfg["n_layers"]):
        k = (rng.standard_normal(shape, dtype=np.float32) * 0.5).astype(np.float16)
        gpu.write_kv(layer, 0, k, k[::-1].copy())
    V = cfg["vocab"]
    feed = rng.integers(0, V, 16).astype(np.int32)
    point = gpu.checkpoint()
    chain = gpu.verify(feed, ctx)
    gpu.rollback(point)
    as_tree = gpu.verify_tree(feed, list(range(-1, 15)), ctx)
    assert np.array_equal(chain, as_tree)
    gpu.rollback(point)
    parent = [-1, 0, 0, 0, 0, 1, 5, 6, 2, 8, 9, 3, 11, 12, 4, 14]
    a = gpu.verify_tree(feed, parent, ctx)
    gpu.rollback(point)
    b = gpu.verify_tree(feed, parent, ctx)
    assert np.array_equal(a, b)
    # rows on the first root path see what the chain's rows saw: slots 0, 1, 5, 6, 7 are chain rows 0..4
    # of a chain that fed those tokens
    path = [0, 1, 5, 6, 7]
    gpu.rollback(point)
    alone = gpu.verify(feed[path], ctx)
    assert gc.logit_error(a[path], alone) <= 2e-3
    gpu.rollback(point)
    gpu.verify_tree(feed, parent, ctx, want_logits=False)
    draft = (gc.f16(a) + rng.standard_normal((16, V)).astype(np.float32) * 0.4).astype(np.float16)
    res = gpu.accept(feed, ctx, ts.shaping(1.0, seed=6), parent=parent, draft_logits=draft, draw_step=2)
    ref = ob.tree_round_sampled(a, draft, feed, parent, ob.shaping(1.0, seed=6), history=[0] * 8, draw_step=2)
    assert res.path == ref["path"] and res.next == ref["next"] and res.draw_step == ref["draw_step"]
    assert gpu.position == ctx + len(res.path)
    # the compacted cache against a cache that only ever saw the accepted path
    nxt = gpu.produce(res.next, gpu.position)
    gpu.rollback(point)
    gpu.verify(feed[res.path], ctx, want_logits=False)
    assert gc.logit_error(nxt[None], gpu.produce(res.next, gpu.position)[None]) <= 2e-3


def test_llama3_8b_all_32_layers_generation_loop_properties():
    """The generation loop at the headline configuration's real depth and vocabulary: greedy
    speculation reports exactly what plain greedy decoding reports whatever the drafter proposes
    (speculative.rs:736-754), and a drafter that is the target itself has every proposal accepted,
    greedy and sampled (r * q(x) <= p(x) with q == p)."""
    import turbospark_amd as ts
    from turbospark_amd import synth
    from tests.loop_common import GpuTarget, LmDrafter
    cfg = dict(synth.CONFIGS["llama3_8b_q4_k"], max_context=128)
    w = synth.make_weights(cfg, seed=3)
    gpu, twin = ts.HipVerifier(cfg, w), ts.HipVerifier(cfg, w)
    V = cfg["vocab"]
    prompt = np.random.default_rng(8).integers(0, V, 9).astype(np.int32)
    new = 24
    noisy = gpu.run_speculative(prompt, LmDrafter(GpuTarget(twin), prompt[0], V, noise=2.0, seed=3), ts.shaping(0.0), new, 4)
    exact = gpu.run_speculative(prompt, LmDrafter(GpuTarget(twin), prompt[0], V), ts.shaping(0.0), new, 4)
    gpu.reset()
    gpu.prefill(prompt[:-1], 0, want_logits=False)
    tok, plain = int(prompt[-1]), []
    for i in range(new):
        tok = int(np.argmax(gc.f16(gpu.produce(tok, len(prompt) - 1 + i))))
        plain.append(tok)
    assert noisy["tokens"] == plain == exact["tokens"]
    assert exact["accepted"] == exact["offered"] and noisy["accepted"] < noisy["offered"]
    sampled = gpu.run_speculative(prompt, LmDrafter(GpuTarget(twin), prompt[0], V), ts.shaping(0.8, seed=2, top_p=0.95), new, 4)
    assert sampled["accepted"] == sampled["offered"] and len(sampled["tokens"]) == new
    assert sampled["min_margin"] >= 0.0


def test_llama3_8b_all_32_layers_prompt_in_blocks_of_64_against_16_row_passes():
    """The headline configuration at its real depth: a 1000-token prompt fed in 64-row passes (producer.rs:122-150)
    leaves the cache and the following logits of the same prompt fed in 16-row passes, which the smaller cases hold
    to the oracle.  The two paths multiply the same integers by the same fp16 activations in another order of fp32
    additions, so they agree to a few fp16 ulps per layer; the tail of 40 tokens goes in 16-row passes in both."""
    import os
    import turbospark_amd as ts
    from turbospark_amd import synth
    cfg = dict(synth.CONFIGS["llama3_8b_q4_k"], max_context=1088)
    w = synth.make_weights(cfg, seed=3)
    rng = np.random.default_rng(8)
    prompt = rng.integers(0, cfg["vocab"], 1000).astype(np.int32)
    feed = rng.integers(0, cfg["vocab"], 5).astype(np.int32)
    out = {}
    for wide in (True, False):
        os.environ["TSV_WIDE_PREFILL"] = "1" if wide else "0"
        try:
            gpu = ts.HipVerifier(cfg, w)
        finally:
            del os.environ["TSV_WIDE_PREFILL"]
        gpu.prefill(prompt, 0, want_logits=False)
        assert gpu.position == 1000
        kv = [gpu.read_kv(layer, 0, 1000) for layer in (0, 15, 31)]
        out[wide] = (kv, gpu.verify(feed, 1000))
        del gpu
    for (kw, vw), (kn, vn) in zip(out[True][0], out[False][0]):
        for a, b in ((kw, kn), (vw, vn)):
            a, b = a.astype(np.float32), b.astype(np.float32)
            assert np.abs(a - b).max() <= 1e-2 * np.abs(b).max()
    err = gc.logit_error(out[True][1], out[False][1])
    print(f"8B shape, 32 layers, 1000-token prompt: logits after 64-row passes vs after 16-row passes {err:.2e}")
    assert err <= 5e-3


def test_qwen3_30b_a3b_shape_two_layers_at_long_context():
    """Configuration 4 at its own geometry: hidden 2048, 32q / 4kv x 128 with the per-head q / k norm,
    128 MXFP4 experts of width 768 routed top-8, Q8_0 attention / router / head, the full 151 936-row
    vocabulary, nine rows (72 (row, q head) pairs per KV head: three attention row groups), two layers
    at a 3000-token context.  Logits, the new cache rows and the greedy round against the oracle."""
    import turbospark_amd as ts
    ctx = 3000
    cfg, gpu, cpu = _filled("qwen3_30b_a3b", ctx, 2)
    V = cfg["vocab"]
    for attempt in range(40):
        rng = np.random.default_rng(40 + attempt)
        # proposals: the oracle's own greedy continuation for three tokens, then junk
        toks = [int(rng.integers(0, V))]
        margins = []
        for i in range(3):
            cpu.rewind_to(ctx + i)
            row = cpu.verify(toks[-1:], ctx + i)
            margins.append(cpu.route_margin)
            toks.append(int(np.argmax(gc.f16(row[0]))))
        feed = np.array(toks + [int(t) for t in rng.integers(0, V, 5)], np.int32)
        cpu.rewind_to(ctx)
        want = cpu.verify(feed, ctx)
        margins.append(cpu.route_margin)
        # the GPU's router logits carry about 1e-4 of the logit range in fp16 rounding (the largest margin
        # at which a decision was seen to differ from the oracle's at this router shape: 1.4e-4)
        if min(margins) > 1e-3:
            break
    else:
        raise AssertionError("no feed without a near-tie routing decision")
    got = gpu.verify(feed, ctx)
    err = gc.logit_error(got, want)
    print(f"Qwen3-30B-A3B shape, 2 layers, ctx {ctx}, m=9, vocab {V}: max-abs logit error / range = {err:.2e}, "
          f"route margin {min(margins):.2e}")
    assert err <= 1e-2
    for layer in range(2):
        kg, vg = gpu.read_kv(layer, ctx, 9)
        kc, vc = cpu.kv(layer)
        assert np.abs(kg.astype(np.float32) - kc[ctx:ctx + 9]).max() <= 2e-2 * np.abs(kc[ctx:ctx + 9]).max()
        assert np.abs(vg.astype(np.float32) - vc[ctx:ctx + 9]).max() <= 2e-2 * np.abs(vc[ctx:ctx + 9]).max()
    # the same rows fed one at a time (families/qwen/batched.rs:92-110: verify == sequential decode): the
    # attention chunks differ with the row count at eight q heads per KV head, so to tolerance
    point = ts.ffi.Point(ctx)
    gpu.rollback(point)
    seq = np.stack([gpu.produce(int(t), ctx + i) for i, t in enumerate(feed)])
    err = gc.logit_error(seq, got)
    print(f"  batched vs one row at a time: max-abs / range = {err:.2e}")
    assert err <= 2e-3
    gpu.rollback(point)
    assert np.array_equal(gpu.verify(feed, ctx), got)
    # the greedy round on the device: integers equal to the oracle's walk over the same fp16 logits ...
    res = gpu.accept(feed, ctx, ts.shaping(0.0))
    ref = ob.chain_round(got, None, feed[1:], ob.shaping(0.0))
    assert (res.accepted, res.committed, res.next, res.stopped) == (ref["accepted"], ref["committed"], ref["next"], 0)
    assert res.kv_position == ctx + ref["committed"] + 1 == gpu.position
    # ... and, the routing decisions being clear of ties, to the walk over the oracle's own logits
    own = ob.chain_round(want, None, feed[1:], ob.shaping(0.0))
    assert res.accepted == own["accepted"] >= 3 and res.next == own["next"]


def _cycled(name, ctx, distinct, seed=3):
    """The configuration at its full depth with `distinct` seeded layers repeated down the stack (the
    size-independent properties below do not care that layers repeat; synthesizing 128 experts for every
    one of 36-48 layers would take minutes of host time).  Every layer still gets its own copy on the device."""
    import turbospark_amd as ts
    from turbospark_amd import synth
    cfg = dict(synth.CONFIGS[name], max_context=ctx + 32)
    w = synth.make_weights(cfg, seed=seed, n_layers=distinct)
    w["layers"] = [w["layers"][i % distinct] for i in range(cfg["n_layers"])]
    gpu = ts.HipVerifier(cfg, w)
    rng = np.random.default_rng(seed)
    shape = (ctx, cfg["n_kv_heads"], cfg["head_dim"])
    k = (rng.standard_normal(shape, dtype=np.float32) * 0.5).astype(np.float16)
    v = (rng.standard_normal(shape, dtype=np.float32) * 0.5).astype(np.float16)
    for layer in range(cfg["n_layers"]):
        s = 37 * layer % ctx
        gpu.write_kv(layer, 0, np.roll(k, s, axis=0), np.roll(v, -s, axis=0))
    assert gpu.position == ctx
    return cfg, gpu


def _cycled_pair(name, ctx, distinct, seed=3):
    """_cycled with the oracle beside it: the same weights and the same seeded K / V rows on both sides."""
    import turbospark_amd as ts
    from turbospark_amd import synth
    cfg = dict(synth.CONFIGS[name], max_context=ctx + 32)
    w = synth.make_weights(cfg, seed=seed, n_layers=distinct)
    w["layers"] = [w["layers"][i % distinct] for i in range(cfg["n_layers"])]
    gpu = ts.HipVerifier(cfg, w)
    cpu = ob.Model(cfg, w, round_kv_f16=True, threads=16)
    rng = np.random.default_rng(seed)
    shape = (ctx, cfg["n_kv_heads"], cfg["head_dim"])
    k = (rng.standard_normal(shape, dtype=np.float32) * 0.5).astype(np.float16)
    v = (rng.standard_normal(shape, dtype=np.float32) * 0.5).astype(np.float16)
    for layer in range(cfg["n_layers"]):
        s = 37 * layer % ctx
        kl, vl = np.roll(k, s, axis=0), np.roll(v, -s, axis=0)
        gpu.write_kv(layer, 0, kl, vl)
        kc, vc = cpu.kv(layer)
        kc[:ctx] = kl.astype(np.float32)
        vc[:ctx] = vl.astype(np.float32)
    cpu.rewind_to(ctx)
    assert gpu.position == ctx
    return cfg, gpu, cpu


def _logits_at_full_depth(name, ctx, m, distinct, parent=None):
    """GPU logits against the oracle at a configuration's real depth, context and vocabulary.  Routed models take
    the oracle's expert choice (read back from it, forced onto the device): through 36-48 random-init layers some
    router decision always sits within rounding of a tie, and what is compared here is the arithmetic."""
    cfg, gpu, cpu = _cycled_pair(name, ctx, distinct)
    feed = np.random.default_rng(5).integers(0, cfg["vocab"], m).astype(np.int32)
    want = cpu.verify(feed, ctx, parent=parent)
    if cfg.get("n_experts"):
        sel, _ = cpu.route_record()
        forced = np.full((cfg["n_layers"], 16, 8), -1, np.int32)
        forced[:, :m, :] = sel[:, :m, :]
        gpu.force_route(forced)
    got = gpu.verify_tree(feed, parent, ctx) if parent is not None else gpu.verify(feed, ctx)
    err = gc.logit_error(got, want)
    print(f"{name}: {cfg['n_layers']} layers, ctx {ctx}, m={m}, vocab {cfg['vocab']}: max-abs logit error / range = {err:.2e}")
    return err


def test_llama3_8b_all_32_layers_logits_against_the_oracle():
    """The headline configuration whole: 32 layers, 4096-token context, five rows, the 128 256-row head."""
    assert _logits_at_full_depth("llama3_8b_q4_k", 4096, 5, 32) <= 1e-2


def test_llama3_8b_all_32_layers_tree_of_16_logits_against_the_oracle():
    """Configuration 3 whole: 32 layers, 16 384-token context, the 16-node tree."""
    parent = [-1, 0, 0, 0, 0, 1, 5, 6, 2, 8, 9, 3, 11, 12, 4, 14]
    assert _logits_at_full_depth("llama3_8b_q4_k", 16384, 16, 32, parent=parent) <= 1e-2


def test_qwen3_30b_a3b_all_48_layers_logits_against_the_oracle():
    """Configuration 4 whole: 48 layers, 8192-token context, nine rows, the 151 936-row head, MXFP4 experts."""
    assert _logits_at_full_depth("qwen3_30b_a3b", 8192, 9, 6) <= 1e-2


def test_gptoss_120b_all_36_layers_logits_against_the_oracle():
    """Configuration 5 whole: 36 layers alternating a 128-token window with full attention, 32 768-token context,
    nine rows, the 201 088-row bf16 head, MXFP4 experts top-4."""
    assert _logits_at_full_depth("gptoss_120b", 32768, 9, 4) <= 1e-2


def _size_independent_properties(cfg, gpu, ctx, m, shaping_kw, temperature):
    """Deterministic by bits; a rollback leaves nothing behind; a chain-shaped tree is the chain by bits;
    the fused round equals verify followed by accept and the oracle's walk over the same logits."""
    import turbospark_amd as ts
    V = cfg["vocab"]
    rng = np.random.default_rng(5)
    feed = rng.integers(0, V, m).astype(np.int32)
    point = gpu.checkpoint()
    a = gpu.verify(feed, ctx)
    gpu.rollback(point)
    b = gpu.verify(feed, ctx)
    assert np.array_equal(a, b)
    gpu.rollback(point)
    t = gpu.verify_tree(feed, list(range(-1, m - 1)), ctx)
    assert np.array_equal(a, t)
    gpu.rollback(point)
    # Rows fed one at a time (families/qwen/batched.rs:92-110: verify == sequential decode).  With eight q heads
    # per KV head a nine-row pass splits the context into other attention chunks than a one-row pass does, so the
    # two agree to rounding per layer, not by bits -- and through 36-48 random-init routed layers one router
    # decision that sits within that rounding of a tie would send a row to another expert, after which its logits
    # have little in common.  So the one-row passes are made to take the experts the batched pass took (its
    # selections read back, forced row by row; the weights stay each pass's own softmax over them): what is left
    # is the arithmetic.  Measured 3e-3 of the logit range at 48 layers -- the distance either pass keeps from the
    # oracle at that depth (3.4e-3); random-init stacks of that depth amplify every rounding difference.
    sel = gpu.route_selected()
    rows = []
    for i, tok in enumerate(feed):
        forced = np.full_like(sel, -1)
        forced[:, 0, :] = sel[:, i, :]
        gpu.force_route(forced)
        rows.append(gpu.produce(int(tok), ctx + i))
    gpu.force_route(None)
    seq = np.stack(rows)
    err = gc.logit_error(seq, a)
    print(f"{cfg['n_layers']} layers, ctx {ctx}, m={m}: batched vs one row at a time under the batched pass's routing, "
          f"max-abs / range = {err:.2e}")
    assert err <= 6e-3
    gpu.rollback(point)
    draft = rng.standard_normal((m - 1, V)).astype(np.float16) if temperature else None
    gs = ts.shaping(temperature, seed=11 if temperature else None, **shaping_kw)
    os_ = ob.shaping(temperature, seed=11 if temperature else None, **shaping_kw)
    fused = gpu.verify_accept(feed, ctx, gs, draft_logits=draft, draw_step=9)
    gpu.rollback(point)
    gpu.verify(feed, ctx, want_logits=False)
    split = gpu.accept(feed, ctx, gs, draft_logits=draft, draw_step=9)
    assert fused == split and fused.kv_position == ctx + fused.committed + 1
    ref = ob.chain_round(a, draft, feed[1:], os_, history=[int(feed[0])], draw_step=9)
    assert (fused.accepted, fused.committed, fused.next) == (ref["accepted"], ref["committed"], ref["next"])
    if temperature:
        assert fused.draw_step == ref["draw_step"]


def test_qwen3_30b_a3b_all_48_layers_size_independent_properties():
    """Configuration 4 at its real depth, context and vocabulary (48 layers, 8192 tokens, 151 936 rows,
    chain k = 8, greedy), where the oracle cannot follow."""
    ctx = 8192
    cfg, gpu = _cycled("qwen3_30b_a3b", ctx, 6)
    _size_independent_properties(cfg, gpu, ctx, 9, {}, 0.0)


def test_gptoss_120b_all_36_layers_size_independent_properties():
    """Configuration 5 at its real depth, context and vocabulary (36 layers alternating a 128-token
    window with full attention, 32 768 tokens, 201 088 rows, 128 experts top-4 resident, chain k = 8,
    rejection sampling at T = 1.0)."""
    ctx = 32768
    cfg, gpu = _cycled("gptoss_120b", ctx, 4)
    _size_independent_properties(cfg, gpu, ctx, 9, {}, 1.0)
