"""TurboQuant KV rows on the GPU against the oracle (oracle/tq.cpp, pinned on the reference's recorded vectors by
tests/test_oracle_tq.py).

Three layers of checks, because the codec is discontinuous: a coordinate that sits on a midpoint takes either
neighbour, so two forwards whose K / V rows differ in the last fp16 bit store a few different indices, and the
logits of a random-weight model move by percents (the oracle itself moves by 2-3 % of its largest logit at four bits
when its staging rows are left in f32 instead of fp16).
  1. the stored rows -- norm and packed words -- of given fp16 staging rows: equal to the oracle's by bits
     (the bar of crates/gpu/tests/kv_quantize_parity.rs, whose two shapes and input formula are the first cases);
  2. attention over those stored rows against the oracle's rotated-space attention
     (crates/compute/src/kv_quant_attention.rs:58-136), to fp16 accuracy (crates/gpu/tests/attention_tq_parity.rs);
  3. the model: a pass of m rows equals m single-row passes by bits -- the per-token semantics of
     crates/runtime/src/kv_write.rs:66-118 -- rollback and replay by bits, and the logits against the oracle model with
     the bound that the codec's own sensitivity allows."""
import os

import numpy as np
import pytest

from tests import gpu_common as gc

pytestmark = pytest.mark.gpu


def _sides(hd, kb, vb):
    from oracle import binding as ob
    ks, vs = ob.tq_sign_vector(hd, ob.TQ_KEY_SEED), ob.tq_sign_vector(hd, ob.TQ_VALUE_SEED)
    kc, vc = ob.tq_codebook(hd, kb), ob.tq_codebook(hd, vb)
    return ks, kc, ob.tq_midpoints(kc), vs, vc, ob.tq_midpoints(vc)


def _indices(stored, bits, hd):
    """The codebook indices of stored rows [..., 1 + words] (LSB-first fields, kv_quant.rs:315-334) as [..., hd]."""
    words = np.ascontiguousarray(stored[..., 1:])
    stream = np.unpackbits(words.view(np.uint8), axis=-1, bitorder="little")[..., :hd * bits]
    fields = stream.reshape(stream.shape[:-1] + (hd, bits)).astype(np.uint32)
    return (fields << np.arange(bits, dtype=np.uint32)).sum(-1)


def _check_rows(rows16, stored, signs, mid, bits):
    """stored [n, heads, 1 + words] against the oracle's quantize_row of the same fp16 rows."""
    from oracle import binding as ob
    n, heads, hd = rows16.shape
    for p in range(n):
        for h in range(heads):
            norm, words = ob.tq_quantize_row(rows16[p, h].astype(np.float32), signs, mid, bits)
            assert np.array_equal(stored[p, h, 1:], words), (p, h)
            assert stored[p, h, 0] == np.float32(norm).view(np.uint32), (p, h, stored[p, h, :1].view(np.float32), norm)


@pytest.mark.parametrize("hd,bits,rows,heads", [(64, 2, 3, 2), (128, 3, 2, 3), (128, 4, 5, 1), (64, 4, 16, 8), (64, 3, 9, 2),
                                               (128, 2, 16, 4)])
def test_stored_rows_of_a_pass_equal_the_oracles_by_bits(hd, bits, rows, heads):
    """crates/gpu/tests/kv_quantize_parity.rs:41-110: hashed, non-degenerate rows read through fp16."""
    from turbospark_amd import ffi
    total = rows * heads * hd
    x = (np.sin(np.arange(total, dtype=np.float32) * np.float32(0.913) + np.float32(0.37)) * 3).astype(np.float16)
    x = x.reshape(rows, heads, hd)
    q = np.zeros((rows, heads, hd), np.float16)
    _, kr, vr = ffi.attention_quantized(q, x, x[::-1].copy(), 0, bits, bits)
    ks, _, km, vs, _, vm = _sides(hd, bits, bits)
    _check_rows(x, kr, ks, km, bits)
    _check_rows(x[::-1], vr, vs, vm, bits)


@pytest.mark.parametrize("nq,nkv,hd,m,base,kb,vb,sinks", [
    (4, 1, 128, 7, 0, 4, 4, False), (8, 2, 64, 16, 37, 3, 4, False), (32, 8, 128, 5, 300, 4, 4, False),
    (8, 2, 64, 1, 129, 2, 2, True), (16, 8, 64, 8, 1000, 3, 3, True), (32, 8, 128, 16, 2049, 3, 4, False)])
def test_attention_over_stored_rows_matches_the_rotated_space_oracle(nq, nkv, hd, m, base, kb, vb, sinks):
    from oracle import binding as ob
    from turbospark_amd import ffi
    rng = np.random.default_rng(nq * 1000 + base)
    seq = base + m
    q = rng.standard_normal((m, nq, hd)).astype(np.float16)
    k = (rng.standard_normal((seq, nkv, hd)) * rng.uniform(0.2, 3.0, (seq, nkv, 1))).astype(np.float16)
    v = (rng.standard_normal((seq, nkv, hd)) * rng.uniform(0.2, 3.0, (seq, nkv, 1))).astype(np.float16)
    sk = rng.standard_normal(nq).astype(np.float32) if sinks else None
    got, kr, vr = ffi.attention_quantized(q, k, v, base, kb, vb, sinks=sk)
    ks, kc, km, vs, vc, vm = _sides(hd, kb, vb)
    # the rows stored ahead of the pass and by the pass: a sample of them by bits (all of them when few)
    pick = np.unique(np.concatenate([np.arange(min(seq, 24)), np.arange(max(0, base - 8), seq),
                                     rng.integers(0, seq, 24)]))
    _check_rows(k[pick], kr[pick], ks, km, kb)
    _check_rows(v[pick], vr[pick], vs, vm, vb)
    worst = 0.0
    for i in range(m):
        want = ob.tq_attention(q[i].astype(np.float32), kr[:, :, 1:], kr[:, :, 0].view(np.float32), vr[:, :, 1:],
                               vr[:, :, 0].view(np.float32), hd, nq, nkv, base + i + 1, kb, ks, kc, vs, vc, sinks=sk,
                               v_bits=vb).reshape(nq, hd)
        worst = max(worst, float(np.abs(got[i] - want).max() / np.abs(want).max()))
    print(f"nq {nq} nkv {nkv} hd {hd} m {m} base {base} K{kb}/V{vb}: worst relative error {worst:.2e}")
    assert worst <= 4e-3


def _open(name, kv_bits, max_context=96, seed=21, **over):
    import turbospark_amd as ts
    from turbospark_amd import synth
    cfg = dict(synth.CONFIGS[name], max_context=max_context, **over)
    w = synth.make_weights(cfg, seed=seed)
    return cfg, w, ts.HipVerifier(cfg, w, kv_bits=kv_bits)


@pytest.mark.parametrize("name,kv_bits,layers", [("small_q4_k", (4, 4), 3), ("xcd_q4_k", (3, 4), 2), ("tiny_q8_0", (2, 2), 4),
                                                 ("gptoss_small", (4, 4), 4), ("moe_small", (3, 3), 3)])
def test_a_pass_of_m_rows_is_m_single_row_passes_by_bits(name, kv_bits, layers):
    """What the reference's per-token path does (kv_write.rs:66-118: stage, commit, attend over stored rows, the
    token's own included) is what every row of a wider pass must see."""
    cfg, w, a = _open(name, kv_bits, n_layers=layers)
    import turbospark_amd as ts
    b = ts.HipVerifier(cfg, w, kv_bits=kv_bits)
    rng = np.random.default_rng(5)
    prompt = rng.integers(0, cfg["vocab"], 37).astype(np.int32)
    feed = rng.integers(0, cfg["vocab"], 8).astype(np.int32)
    a.prefill(prompt, 0, want_logits=False)
    b.prefill(prompt, 0, want_logits=False)
    wide = a.verify(feed, 37)
    narrow = np.concatenate([b.verify(feed[i:i + 1], 37 + i) for i in range(8)])
    assert np.array_equal(wide, narrow)
    quantized = [l for l in range(layers) if int(w["layers"][l].get("window", 0)) == 0 and (layers <= 2 or l + 1 < layers)]
    assert quantized
    for l in quantized:
        ka, va = a.read_kv_quantized(l, 0, 45)
        kb_, vb_ = b.read_kv_quantized(l, 0, 45)
        assert np.array_equal(ka, kb_) and np.array_equal(va, vb_)
    for l in set(range(layers)) - set(quantized):
        with pytest.raises(ts.ffi.TsvError):
            a.read_kv_quantized(l, 0, 1)
        a.read_kv(l, 40, 4)
    with pytest.raises(ts.ffi.TsvError):
        a.read_kv(quantized[0], 0, 1)


def test_rollback_and_replay_by_bits():
    cfg, w, g = _open("small_q4_k", (3, 4), n_layers=3)
    rng = np.random.default_rng(6)
    prompt = rng.integers(0, cfg["vocab"], 20).astype(np.int32)
    g.prefill(prompt, 0, want_logits=False)
    cp = g.checkpoint()
    f1 = rng.integers(0, cfg["vocab"], 8).astype(np.int32)
    f2 = rng.integers(0, cfg["vocab"], 5).astype(np.int32)
    first = g.verify(f1, 20)
    g.rollback(cp)
    other = g.verify(f2, 20)          # other rows over the same slots
    g.rollback(cp)
    again = g.verify(f1, 20)
    assert np.array_equal(first, again) and not np.array_equal(first[:5], other)
    # keep three of the rows and go on: the kept rows are read from the store, the rest recomputed
    g.rollback_retaining(cp, 3)
    assert g.position == 23
    assert np.array_equal(g.verify(f1[3:], 23), first[3:])


@pytest.mark.parametrize("name,kv_bits,layers,bound", [("small_q4_k", (4, 4), 3, 3e-2), ("xcd_q4_k", (4, 4), 3, 4e-2),
                                                       ("gptoss_small", (4, 4), 4, 1e-2), ("small_q4_k", (3, 4), 3, 3e-2),
                                                       ("xcd_q4_k", (2, 2), 3, 1.5e-1), ("tiny_q8_0", (3, 3), 4, 6e-2)])
def test_logits_against_the_oracle_model_within_the_codecs_own_sensitivity(name, kv_bits, layers, bound):
    """The same forward with the same codec on both sides.  The bound is not fp16 accuracy: indices of coordinates
    near a midpoint differ between any two forwards whose K / V rows differ in the last bit.  What is asserted is
    that the GPU is no further from the oracle than the oracle is from itself under such a change (its own
    f32-staging variant), and far closer than the codec's effect (the distance to the fp16-row oracle)."""
    from oracle import binding as ob
    cfg, w, g = _open(name, kv_bits, n_layers=layers)
    rng = np.random.default_rng(7)
    prompt = rng.integers(0, cfg["vocab"], 40).astype(np.int32)
    feed = rng.integers(0, cfg["vocab"], 12).astype(np.int32)

    def oracle(**kw):
        m = ob.Model(cfg, w, threads=16, **kw)
        for i in range(0, 40, 16):
            m.verify(prompt[i:i + 16], i)
        return m.verify(feed, 40)

    want = oracle(round_kv_f16=True, kv_bits=kv_bits)
    twin = oracle(round_kv_f16=False, kv_bits=kv_bits)
    plain = oracle(round_kv_f16=True)
    g.prefill(prompt, 0, want_logits=False)
    got = g.verify(feed, 40)
    err, self_err, effect = gc.logit_error(got, want), gc.logit_error(twin, want), gc.logit_error(plain, want)
    print(f"{name} K{kv_bits[0]}/V{kv_bits[1]}: GPU vs oracle {err:.2e}; oracle vs its f32-staging twin {self_err:.2e}; "
          f"codec vs fp16 rows {effect:.2e}")
    assert err <= bound and err <= max(3 * self_err, 2e-2) and err < 0.6 * effect


@pytest.mark.parametrize("name,kv_bits", [("small_q4_k", (3, 4)), ("xcd_q4_k", (4, 4)), ("tiny_q8_0", (2, 2)), ("small_q4_k", (3, 3))])
def test_tree_compaction_moves_the_stored_rows_by_bits_and_the_round_goes_on(name, kv_bits):
    """crates/runtime/src/speculative.rs:518-536: after a tree pass the accepted path's rows become rows
    base .. base + n - 1.  The stored rows must move unchanged; the continuation is then compared with a handle that
    fed the path as a chain (its rows come from a narrower pass, so a few indices near midpoints differ)."""
    import turbospark_amd as ts
    cfg, w, g = _open(name, kv_bits, n_layers=3)
    rng = np.random.default_rng(9)
    prompt = rng.integers(0, cfg["vocab"], 37).astype(np.int32)
    feed = rng.integers(0, cfg["vocab"], 16).astype(np.int32)
    parent = [-1, 0, 0, 0, 0, 1, 5, 6, 2, 8, 9, 3, 11, 12, 4, 14]
    path = [0, 2, 8, 9]
    g.prefill(prompt, 0, want_logits=False)
    point = g.checkpoint()
    g.verify_tree(feed, parent, 37)
    before = [g.read_kv_quantized(l, 0, 53) for l in (0, 1)]
    plain_before = g.read_kv(2, 37, 16)
    g.compact_tree(37, path)
    after = [g.read_kv_quantized(l, 0, 53) for l in (0, 1)]
    plain_after = g.read_kv(2, 37, 4)
    for (kb, vb), (ka, va) in zip(before, after):
        assert np.array_equal(ka[:37], kb[:37]) and np.array_equal(va[:37], vb[:37])
        assert np.array_equal(ka[37:41], kb[37 + np.array(path)]) and np.array_equal(va[37:41], vb[37 + np.array(path)])
    assert np.array_equal(plain_after[0], plain_before[0][path]) and np.array_equal(plain_after[1], plain_before[1][path])
    g.rollback_retaining(point, 4)
    nxt = g.produce(int(feed[10]), 41)
    ref = ts.HipVerifier(cfg, w, kv_bits=kv_bits)
    ref.prefill(prompt, 0, want_logits=False)
    ref.verify(feed[path], 37)
    want = ref.produce(int(feed[10]), 41)
    err = gc.logit_error(nxt[None], want[None])
    same = np.mean([np.mean(a[0][37:41, :, 1:] == r[0][:, :, 1:]) for a, r in zip(after, [ref.read_kv_quantized(l, 37, 4) for l in (0, 1)])])
    print(f"{name} K{kv_bits[0]}/V{kv_bits[1]}: continuation after compaction vs chain {err:.2e}; K words equal {same:.3f}")
    assert err <= 3e-2 and same >= 0.8


def test_what_a_quantized_handle_refuses():
    import turbospark_amd as ts
    from turbospark_amd import synth
    cfg, w, g = _open("small_q4_k", (4, 4))
    g.verify(np.arange(6, dtype=np.int32), 0)
    with pytest.raises(ts.ffi.TsvError, match="quantized"):
        g.read_kv(0, 0, 1)
    for bad in ((4, 3), (1, 1), (5, 5), (2, 4), (0, 4)):
        with pytest.raises(ts.ffi.TsvError, match="widths"):
            ts.HipVerifier(cfg, w, kv_bits=bad)
    # gpt-oss with a window on every layer: nothing to quantize, refused by name
    # (crates/runtime/src/real_forward_init.rs:186-197)
    oss = dict(synth.CONFIGS["gptoss_small"], max_context=96)
    wo = synth.make_weights(oss, seed=3)
    for lw in wo["layers"]:
        lw["window"] = 24
    with pytest.raises(ts.ffi.TsvError, match="nothing to quantize"):
        ts.HipVerifier(oss, wo, kv_bits=(4, 4))


def test_rings_on_a_quantized_handle_equal_the_linear_layout_by_bits():
    """gpt-oss arrangement with both options at once: the sliding layers as rings (kv_cache.rs:360-378), the full layers'
    rows quantized (kv_quant.rs:102-107).  Prompt passes far past the rings' capacity, verify rounds with rollbacks
    inside the budget, a tree round with compaction across a ring's seam: every logit equal to the same handle with
    the sliding layers laid out linearly, and the rewind budget is the rings'."""
    import turbospark_amd as ts
    from turbospark_amd import synth
    cfg = dict(synth.CONFIGS["gptoss_small"], max_context=400, n_layers=4)
    w = synth.make_weights(cfg, seed=21)
    ringed = dict(w, layers=[dict(lw, ring=1 if lw.get("window") else 0) for lw in w["layers"]])
    # (both handles in 16-row prompt passes: the comparison is of the layouts, not of the passes' summation orders)
    import os
    os.environ["TSV_WIDE_PREFILL"] = "0"
    try:
        lin, ring = ts.HipVerifier(cfg, w, kv_bits=(4, 4)), ts.HipVerifier(cfg, ringed, kv_bits=(4, 4))
    finally:
        del os.environ["TSV_WIDE_PREFILL"]
    assert lin.max_safe_rewind() == 2 ** 63 - 1 and ring.max_safe_rewind() == 64 - 24
    V = cfg["vocab"]
    rng = np.random.default_rng(8)
    prompt = rng.integers(0, V, 150).astype(np.int32)
    assert np.array_equal(lin.prefill(prompt, 0), ring.prefill(prompt, 0))
    base = 150
    for rnd in range(20):
        m = int(rng.integers(1, 17))
        feed = rng.integers(0, V, m).astype(np.int32)
        pa, pb = lin.checkpoint(), ring.checkpoint()
        assert np.array_equal(lin.verify(feed, base), ring.verify(feed, base)), rnd
        keep = int(rng.integers(1, m + 1))
        lin.rollback_retaining(pa, keep)
        ring.rollback_retaining(pb, keep)
        base += keep
    parent = [-1, 0, 0, 1, 1, 2, 3, 5]
    feed = rng.integers(0, V, 8).astype(np.int32)
    for eng in (lin, ring):
        eng.verify_tree(feed, parent, base, want_logits=False)
        eng.compact_tree(base, [0, 2, 5, 7])
        eng.rollback_retaining(ts.ffi.Point(base), 4)
    nxt = rng.integers(0, V, 3).astype(np.int32)
    assert np.array_equal(lin.verify(nxt, base + 4), ring.verify(nxt, base + 4))
    with pytest.raises(ts.ffi.TsvError, match="exceeds the ring slack"):
        ring.rollback(ts.ffi.Point(base - 60))


def test_a_gguf_target_takes_the_width_from_the_environment(tmp_path):
    """The option is a session's, not the file's (crates/model-io/src/kv_quant.rs:48-72): TSV_KV_BITS carries it to
    tsv_open_gguf, and the handle then equals the directly installed one with the same widths, by bits."""
    import turbospark_amd as ts
    from tests.gguf_writer import llama_gguf
    cfg, w, direct = _open("tiny_q8_0", (3, 4), n_layers=3)
    path = os.path.join(tmp_path, "kv.gguf")
    llama_gguf(path, cfg, w, arch="llama", permute=True)
    os.environ["TSV_KV_BITS"] = "3.5"
    try:
        filed = ts.HipVerifier.from_gguf(path, max_context=96)
        os.environ["TSV_KV_BITS"] = "7"
        with pytest.raises(ts.ffi.TsvError, match="TSV_KV_BITS"):
            ts.HipVerifier.from_gguf(path, max_context=96)
    finally:
        del os.environ["TSV_KV_BITS"]
    filed.kv_bits = (3, 4)
    rng = np.random.default_rng(8)
    prompt = rng.integers(0, cfg["vocab"], 21).astype(np.int32)
    assert np.array_equal(direct.prefill(prompt, 0), filed.prefill(prompt, 0))
    feed = rng.integers(0, cfg["vocab"], 5).astype(np.int32)
    assert np.array_equal(direct.verify(feed, 21), filed.verify(feed, 21))
    for layer in (0, 1):
        (ka, va), (kb, vb) = direct.read_kv_quantized(layer, 0, 26), filed.read_kv_quantized(layer, 0, 26)
        assert np.array_equal(ka, kb) and np.array_equal(va, vb)


def test_llama3_8b_shape_two_layers_at_4096_context_with_four_bit_rows():
    """The headline geometry (32 q heads over 8 kv heads of 128, hidden 4096, the 128 256-row head) with both
    layers' rows quantized: the context is written through the quantizer on both sides, then a pass of five rows
    against the oracle, and the same pass as five single-row passes by bits."""
    import turbospark_amd as ts
    from oracle import binding as ob
    from turbospark_amd import synth
    ctx, kv_bits = 4096, (4, 4)
    cfg = dict(synth.CONFIGS["llama3_8b_q4_k"], n_layers=2, max_context=ctx + 32)
    w = synth.make_weights(cfg, seed=3, n_layers=2)
    gpu = ts.HipVerifier(cfg, w, kv_bits=kv_bits)
    cpu = ob.Model(cfg, w, round_kv_f16=True, threads=16, kv_bits=kv_bits)
    rng = np.random.default_rng(3)
    for layer in range(2):
        shape = (ctx, cfg["n_kv_heads"], cfg["head_dim"])
        k = (rng.standard_normal(shape) * 0.5).astype(np.float16)
        v = (rng.standard_normal(shape) * 0.5).astype(np.float16)
        gpu.write_kv(layer, 0, k, v)
        kc, vc = cpu.kv(layer)
        kc[:ctx] = ob.tq_roundtrip_rows(k, kv_bits[0], ob.TQ_KEY_SEED)
        vc[:ctx] = ob.tq_roundtrip_rows(v, kv_bits[1], ob.TQ_VALUE_SEED)
        # the stored rows are the oracle's, by bits, on a sample of the context
        pick = rng.integers(0, ctx, 12)
        kr, vr = gpu.read_kv_quantized(layer, 0, ctx)
        ks, _, km, vs, _, vm = _sides(cfg["head_dim"], *kv_bits)
        _check_rows(k[pick], kr[pick], ks, km, kv_bits[0])
        _check_rows(v[pick], vr[pick], vs, vm, kv_bits[1])
    cpu.rewind_to(ctx)
    assert gpu.position == ctx
    feed = rng.integers(0, cfg["vocab"], 5).astype(np.int32)
    point = gpu.checkpoint()
    got = gpu.verify(feed, ctx)
    want = cpu.verify(feed, ctx)
    err = gc.logit_error(got, want)
    print(f"8B shape, 2 layers, ctx 4096, m=5, K4/V4 rows: max-abs logit error / range = {err:.2e}")
    # fp16 rows reach 4e-4 here.  The rotated-space pass rounds the codebook levels and the rotated q to fp16 and the
    # pass's own ten rows are requantized from staging rows that differ in the last bit; the reference's own GPU
    # test of this attention allows 0.06 absolute on outputs of order one (crates/gpu/tests/attention_tq_parity.rs:603)
    assert err <= 3e-2
    gpu.rollback(point)
    single = np.concatenate([gpu.verify(feed[i:i + 1], ctx + i) for i in range(5)])
    assert np.array_equal(got, single)


def test_graph_replay_over_quantized_rows_equals_plain_launches():
    """The captured launch sequence reads its positions from device memory at replay; the quantizer and the pass
    over the stores must do so too: every replay, with rollbacks between them, gives the bits of the plain launches,
    logits and stored rows."""
    import turbospark_amd as ts
    from turbospark_amd import synth
    cfg = dict(synth.CONFIGS["small_q4_k"], max_context=160, n_layers=3)
    w = synth.make_weights(cfg, seed=5)
    plain = ts.HipVerifier(cfg, w, kv_bits=(4, 4))
    os.environ["TSV_GRAPH"] = "1"
    try:
        graph = ts.HipVerifier(cfg, w, kv_bits=(4, 4))
    finally:
        os.environ["TSV_GRAPH"] = "0"
    rng = np.random.default_rng(9)
    prompt = rng.integers(0, cfg["vocab"], 37).astype(np.int32)
    for eng in (plain, graph):
        eng.prefill(prompt, 0, want_logits=False)
    base = 37
    for rnd, m in enumerate([5, 5, 3, 5, 16, 5, 3]):
        feed = rng.integers(0, cfg["vocab"], m).astype(np.int32)
        assert np.array_equal(plain.verify(feed, base), graph.verify(feed, base)), (rnd, m)
        keep = 1 + rnd % 3
        for eng in (plain, graph):
            eng.rollback(ts.ffi.Point(base + keep))
        base += keep
    for layer in (0, 1):
        (ka, va), (kb, vb) = plain.read_kv_quantized(layer, 0, base), graph.read_kv_quantized(layer, 0, base)
        assert np.array_equal(ka, kb) and np.array_equal(va, vb)


def test_gptoss_120b_shape_with_the_full_layers_rows_quantized():
    """Hidden 2880, 64 q heads over 8 kv heads of 64 (eight q heads per kv head: the widest group), sinks, YaRN, a
    windowed layer (fp16 rows) beside a full one (K3/V4 rows), 128 experts top-4; 3000 positions written through the
    quantizer on both sides; vocabulary cut to 4096 to keep the CPU side short."""
    import turbospark_amd as ts
    from oracle import binding as ob
    from turbospark_amd import synth
    ctx, kv_bits = 3000, (3, 4)
    cfg = dict(synth.CONFIGS["gptoss_120b"], n_layers=2, max_context=ctx + 32, vocab=4096)
    w = synth.make_weights(cfg, seed=3, n_layers=2)
    gpu = ts.HipVerifier(cfg, w, kv_bits=kv_bits)
    cpu = ob.Model(cfg, w, round_kv_f16=True, threads=16, kv_bits=kv_bits)
    assert [cpu.layer_quantized(l) for l in range(2)] == [False, True]
    rng = np.random.default_rng(3)
    for layer in range(2):
        shape = (ctx, cfg["n_kv_heads"], cfg["head_dim"])
        k = (rng.standard_normal(shape) * 0.5).astype(np.float16)
        v = (rng.standard_normal(shape) * 0.5).astype(np.float16)
        gpu.write_kv(layer, 0, k, v)
        kc, vc = cpu.kv(layer)
        if layer == 1:
            kc[:ctx] = ob.tq_roundtrip_rows(k, kv_bits[0], ob.TQ_KEY_SEED)
            vc[:ctx] = ob.tq_roundtrip_rows(v, kv_bits[1], ob.TQ_VALUE_SEED)
        else:
            kc[:ctx] = k.astype(np.float32)
            vc[:ctx] = v.astype(np.float32)
    cpu.rewind_to(ctx)
    for attempt in range(40):
        feed = np.random.default_rng(20 + attempt).integers(0, cfg["vocab"], 9).astype(np.int32)
        cpu.rewind_to(ctx)
        want = cpu.verify(feed, ctx)
        if cpu.route_margin > 1e-3:
            break
    else:
        raise AssertionError("no feed without a near-tie routing decision")
    point = gpu.checkpoint()
    got = gpu.verify(feed, ctx)
    err = gc.logit_error(got, want)
    print(f"gpt-oss-120B shape, 2 layers, ctx {ctx}, m=9, K3/V4 rows on the full layer: max-abs logit error / range = {err:.2e}")
    assert err <= 3e-2
    gpu.rollback(point)
    # with eight q heads per kv head a nine-row pass splits the context into other attention chunks than a one-row
    # pass does (fp16 rows or not), so the two agree to rounding here, not by bits
    single = np.concatenate([gpu.verify(feed[i:i + 1], ctx + i) for i in range(9)])
    gap = gc.logit_error(single, got)
    print(f"  the same nine rows one at a time: {gap:.2e}")
    assert gap <= 2e-2


@pytest.mark.parametrize("name,kv_bits,n_prompt", [("small_q4_k", (4, 4), 150), ("xcd_q4_k", (3, 4), 129), ("small_q4_k", (2, 2), 64),
                                                   ("xcd_q8_0", (4, 4), 150), ("moe_small", (4, 4), 150)])
def test_prompt_passes_of_64_rows_over_quantized_rows(name, kv_bits, n_prompt):
    """crates/runtime/src/producer.rs:122-150 with --kv-bits: all 64 rows of a pass are quantized before any of its four
    blocks attends, so every row sees what sixteen-row passes would show it.  The two paths multiply the same integers
    in another order (tests/test_gpu_prefill_wide.py), so their staging rows differ in the last bit, a few indices near
    midpoints with them, and the comparison is the codec's: stored words mostly equal, logits within its sensitivity."""
    import turbospark_amd as ts
    from oracle import binding as ob
    from turbospark_amd import synth
    cfg = dict(synth.CONFIGS[name], max_context=n_prompt + 48, n_layers=3)
    w = synth.make_weights(cfg, seed=11)

    def engine(wide):
        os.environ["TSV_WIDE_PREFILL"] = "1" if wide else "0"
        try:
            return ts.HipVerifier(cfg, w, kv_bits=kv_bits)
        finally:
            del os.environ["TSV_WIDE_PREFILL"]

    wide, narrow = engine(True), engine(False)
    cpu = ob.Model(cfg, w, round_kv_f16=True, threads=16, kv_bits=kv_bits)
    rng = np.random.default_rng(2)
    prompt = rng.integers(0, cfg["vocab"], n_prompt).astype(np.int32)
    feed = rng.integers(0, cfg["vocab"], 5).astype(np.int32)
    wide.prefill(prompt, 0, want_logits=False)
    narrow.prefill(prompt, 0, want_logits=False)
    for i in range(0, n_prompt, 16):
        cpu.verify(prompt[i:i + 16], i)
    assert wide.position == narrow.position == n_prompt
    same = []
    for layer in (0, 1):
        (kw, vw), (kn, vn) = wide.read_kv_quantized(layer, 0, n_prompt), narrow.read_kv_quantized(layer, 0, n_prompt)
        hd = cfg["head_dim"]
        same.append(np.mean(_indices(kw, kv_bits[0], hd) == _indices(kn, kv_bits[0], hd)))
        same.append(np.mean(_indices(vw, kv_bits[1], hd) == _indices(vn, kv_bits[1], hd)))
        # layer 0 sees the same inputs on both paths up to the matmuls' rounding: norms agree to fp16 accuracy
        if layer == 0:
            assert np.allclose(kw[:, :, 0].view(np.float32), kn[:, :, 0].view(np.float32), rtol=2e-3)
    want = cpu.verify(feed, n_prompt)
    got_w, got_n = wide.verify(feed, n_prompt), narrow.verify(feed, n_prompt)
    err_w, err_n, err_wn = gc.logit_error(got_w, want), gc.logit_error(got_n, want), gc.logit_error(got_w, got_n)
    print(f"{name} K{kv_bits[0]}/V{kv_bits[1]}, prompt of {n_prompt}: stored indices equal between the paths {min(same):.4f}; logits after "
          f"64-row passes vs oracle {err_w:.2e}, after 16-row passes {err_n:.2e}, the two GPU paths {err_wn:.2e}")
    bound = 1.5e-1 if kv_bits == (2, 2) else 5e-2
    assert min(same) >= 0.97 and err_w <= bound and err_wn <= bound


@pytest.mark.parametrize("seed", range(16))
def test_random_shapes_of_attention_over_stored_rows(seed):
    """A seeded sweep over head widths, head groupings, pass widths, prefix lengths (block boundaries, short and long
    contexts), the four width pairs and sinks: stored rows by bits on a sample, the pass against the oracle."""
    from oracle import binding as ob
    from turbospark_amd import ffi
    rng = np.random.default_rng(1000 + seed)
    hd = int(rng.choice([64, 128]))
    nkv = int(rng.choice([1, 2, 4, 8]))
    g = int(rng.choice([1, 2, 4, 8]))
    nq = nkv * g
    m = int(rng.integers(1, 17))
    base = int(rng.choice([0, 1, 15, 16, 17, 31, int(rng.integers(32, 600)), int(rng.integers(600, 7000))]))
    kb, vb = [(2, 2), (3, 3), (3, 4), (4, 4)][int(rng.integers(0, 4))]
    sinks = rng.standard_normal(nq).astype(np.float32) if rng.random() < 0.4 else None
    scale = float(rng.choice([0.0, 0.1, 0.2]))
    seq = base + m
    q = rng.standard_normal((m, nq, hd)).astype(np.float16)
    k = (rng.standard_normal((seq, nkv, hd)) * rng.uniform(0.1, 4.0, (seq, nkv, 1))).astype(np.float16)
    v = (rng.standard_normal((seq, nkv, hd)) * rng.uniform(0.1, 4.0, (seq, nkv, 1))).astype(np.float16)
    print(f"seed {seed}: hd={hd} q/kv={nq}/{nkv} m={m} base={base} K{kb}/V{vb} sinks={'yes' if sinks is not None else 'no'} scale={scale}",
          flush=True)
    got, kr, vr = ffi.attention_quantized(q, k, v, base, kb, vb, scale=scale, sinks=sinks)
    ks, kc, km, vs, vc, vm = _sides(hd, kb, vb)
    pick = np.unique(np.concatenate([np.arange(min(seq, 8)), np.arange(max(0, base - 3), seq), rng.integers(0, seq, 8)]))
    _check_rows(k[pick], kr[pick], ks, km, kb)
    _check_rows(v[pick], vr[pick], vs, vm, vb)
    rows = sorted(set([0, m - 1, int(rng.integers(0, m))]))
    worst = 0.0
    for i in rows:
        want = ob.tq_attention(q[i].astype(np.float32), kr[:, :, 1:], kr[:, :, 0].view(np.float32), vr[:, :, 1:],
                               vr[:, :, 0].view(np.float32), hd, nq, nkv, base + i + 1, kb, ks, kc, vs, vc, scale=scale,
                               sinks=sinks, v_bits=vb).reshape(nq, hd)
        worst = max(worst, float(np.abs(got[i] - want).max() / np.abs(want).max()))
    print(f"  worst relative error {worst:.2e}")
    assert worst <= 5e-3


@pytest.mark.parametrize("seed", range(24))
def test_random_model_shapes_with_quantized_rows(seed):
    """The seeded decoder shapes of tests/test_gpu_random_shapes.py with a random width pair: the pass (chain or tree)
    against the oracle with the same codec within the codec's sensitivity, determinism by bits, and -- for chains of at
    most eight rows, where the fp16-row path holds it too -- the pass as single-row passes by bits."""
    import turbospark_amd as ts
    from oracle import binding as ob
    from tests.test_gpu_random_shapes import _case
    from turbospark_amd import ffi
    cfg, ctx, m, parent, r = _case(seed)
    kv_bits = [(2, 2), (3, 3), (3, 4), (4, 4)][int(r.integers(0, 4))]
    cfg = dict(cfg, max_context=ctx + 40)
    from turbospark_amd import synth
    w = synth.make_weights(cfg, seed=77 + seed)
    gpu = ts.HipVerifier(cfg, w, kv_bits=kv_bits)
    cpu = ob.Model(cfg, w, round_kv_f16=True, threads=16, kv_bits=kv_bits)
    V = cfg["vocab"]
    print(f"seed {seed}: {'q4_k' if cfg['dtype'] == ffi.Q4_K else 'q8_0'} L={cfg['n_layers']} H={cfg['hidden']} "
          f"q/kv={cfg['n_q_heads']}/{cfg['n_kv_heads']}x{cfg['head_dim']} ctx={ctx} m={m} {'tree' if parent else 'chain'}"
          f"{' qk-norm' if cfg['qk_norm'] else ''} K{kv_bits[0]}/V{kv_bits[1]}", flush=True)
    prompt = r.integers(0, V, ctx).astype(np.int32)
    feed = r.integers(0, V, m).astype(np.int32)
    gpu.prefill(prompt, 0, want_logits=False)
    for i in range(0, ctx, 16):
        cpu.verify(prompt[i:i + 16], i)
    point = gpu.checkpoint()
    got = gpu.verify_tree(feed, parent, ctx) if parent else gpu.verify(feed, ctx)
    want = cpu.verify(feed, ctx, parent=parent)
    err = gc.logit_error(got, want)
    print(f"   max-abs logit error / range = {err:.2e}", flush=True)
    assert err <= (2e-1 if kv_bits == (2, 2) else 8e-2)
    gpu.rollback(point)
    again = gpu.verify_tree(feed, parent, ctx) if parent else gpu.verify(feed, ctx)
    assert np.array_equal(got, again)
    if not parent and m <= 8 and m * (cfg["n_q_heads"] // cfg["n_kv_heads"]) <= 32:
        gpu.rollback(point)
        single = np.concatenate([gpu.verify(feed[i:i + 1], ctx + i) for i in range(m)])
        assert np.array_equal(got, single)


def _greedy_decode(eng, steps, vocab):
    """crates/runtime/tests/real_forward_llama_kv_quant.rs:56-80: produce, take the arg-max, feed it back."""
    eng.reset()
    token, out = 5, []
    for position in range(steps):
        logits = gc.f16(eng.produce(token, position))
        assert np.isfinite(logits).all(), position
        out.append(logits)
        token = int(np.argmax(logits))
    return np.stack(out)


def test_the_reference_runtime_scenarios_for_kv_bits():
    """crates/runtime/tests/real_forward_llama_kv_quant.rs: `off` is the plain handle by bits; every width the option
    names decodes finite and deterministic over several tokens; turning it on moves the output past the first token
    (where a single key makes the key side invisible); an unsupported head width is refused by name."""
    import turbospark_amd as ts
    from turbospark_amd import synth
    cfg = dict(synth.CONFIGS["tiny_q8_0"], max_context=64, n_layers=4)
    w = synth.make_weights(cfg, seed=9)
    V = cfg["vocab"]
    plain = _greedy_decode(ts.HipVerifier(cfg, w), 6, V)
    off = _greedy_decode(ts.HipVerifier(cfg, w, kv_bits=ts.producer.parse_kv_bits("off")), 6, V)
    assert np.array_equal(plain, off)
    for text in ("2", "3", "3.5", "4"):
        bits = ts.producer.parse_kv_bits(text)
        first = _greedy_decode(ts.HipVerifier(cfg, w, kv_bits=bits), 5, V)
        second = _greedy_decode(ts.HipVerifier(cfg, w, kv_bits=bits), 5, V)
        assert np.array_equal(first, second), text
    on = _greedy_decode(ts.HipVerifier(cfg, w, kv_bits=(3, 4)), 5, V)
    assert np.abs(on[1:] - plain[1:5]).max() > 1e-3
    bad = dict(cfg, head_dim=32, n_q_heads=16, n_kv_heads=16)
    with pytest.raises(ts.ffi.TsvError, match="head_dim"):
        ts.HipVerifier(bad, synth.make_weights(bad, seed=9), kv_bits=(4, 4))
