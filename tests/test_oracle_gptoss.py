"""Pins of the oracle's gpt-oss pieces (YaRN table, clamped SwiGLU, sinks / window / biases in the
layer graph) against what the reference's own tests fix and against an independent numpy
restatement of the whole forward (crates/runtime/src/families/gptoss/mod.rs:11-23)."""
import numpy as np

from oracle import binding as ob


def test_yarn_scalars_of_gpt_oss_give_llama_cpps_mscale_and_an_untouched_fast_end():
    # crates/runtime/src/families/gptoss/state.rs:405-440 with arch_baselines/gpt_oss.rs:93-96
    f, ms = ob.yarn_frequencies(64, 150000.0, 32.0, 4096, 32.0, 1.0)
    assert abs(ms - 1.3465736) < 1e-6
    assert f.size == 32 and abs(f[0] - 1.0) < 1e-6 and f[0] > f[-1]
    plain = np.float32(150000.0) ** (-(np.arange(32, dtype=np.float32) * 2) / np.float32(64))
    # the slow end is fully interpolated (divided by the factor), the fast end keeps its frequency
    assert abs(f[-1] / plain[-1] - 1 / 32.0) < 1e-6
    ratio = f / plain
    assert np.all(np.diff(ratio) <= 1e-7) and ratio[0] == 1.0
    # the ramp runs between the two correction dimensions ggml computes, in pair units
    corr = lambda rot: 64 * np.log(4096 / (rot * 2 * np.pi)) / (2 * np.log(150000.0))
    lo, hi = max(np.floor(corr(32.0)), 0), min(np.ceil(corr(1.0)), 63)
    inside = [p for p in range(32) if lo < p < hi]
    assert inside and all(1 / 32.0 < ratio[p] < 1.0 for p in inside)
    assert all(ratio[p] == 1.0 for p in range(32) if p <= lo) and all(abs(ratio[p] - 1 / 32.0) < 1e-7 for p in range(32) if p >= hi)
    # swapped betas invert the ramp (the silent mistake the reference's test names)
    g, _ = ob.yarn_frequencies(64, 150000.0, 32.0, 4096, 1.0, 32.0)
    assert not np.allclose(f, g)
    # factor <= 0: the ordinary table, scale 1 (rope.rs:318-322, :498)
    h, one = ob.yarn_frequencies(128, 500000.0, 0.0, 0, 0.0, 0.0)
    assert one == 1.0
    want = np.float32(500000.0) ** (-(np.arange(64, dtype=np.float32) * 2) / np.float32(128))
    assert np.allclose(h, want, rtol=2e-7)


def test_the_library_table_is_the_oracle_table():
    from turbospark_amd import ffi
    for args in [(64, 150000.0, 32.0, 4096, 32.0, 1.0), (64, 150000.0, 32.0, 64, 32.0, 1.0), (128, 1e6, 4.0, 8192, 16.0, 2.0),
                 (128, 500000.0, 0.0, 0, 0.0, 0.0)]:
        a, am = ffi.yarn_frequencies(*args)
        b, bm = ob.yarn_frequencies(*args)
        assert np.array_equal(a, b) and am == bm, args


def test_scaled_rotation_is_the_table_rotation_times_mscale():
    rng = np.random.default_rng(1)
    x = rng.standard_normal((3, 64)).astype(np.float32)
    f, ms = ob.yarn_frequencies(64, 150000.0, 32.0, 4096, 32.0, 1.0)
    a = ob.rope_neox_freqs_scaled(x, 1, 3, 64, 32, 977, f, ms)
    b = ob.rope_neox_freqs(x, 1, 3, 64, 32, 977, f)
    assert np.allclose(a, b * ms, rtol=1e-6, atol=1e-7)
    # norm grows by exactly mscale: a rotation preserves it
    assert np.allclose(np.linalg.norm(a, axis=1), np.linalg.norm(x, axis=1) * ms, rtol=1e-5)


def test_swiglu_oai_closed_forms():
    a, lim = 1.702, 7.0
    sw = lambda g, u: ob.swiglu_oai(g, u, a, lim)
    assert sw(0.0, 3.0) == 0.0
    # (y + 1): an up of zero does not kill the unit
    assert abs(sw(1.0, 0.0) - 1.0 / (1.0 + np.exp(-a))) < 1e-6
    # gate is clamped from above only, up on both sides
    assert abs(sw(50.0, 0.0) - 7.0 / (1.0 + np.exp(-a * 7.0))) < 1e-5
    assert abs(sw(-50.0, 0.0) - (-50.0 / (1.0 + np.exp(a * 50.0)))) < 1e-6
    assert abs(sw(1.0, 100.0) - sw(1.0, 7.0)) < 1e-7 and abs(sw(1.0, -100.0) - sw(1.0, -7.0)) < 1e-7
    assert abs(sw(1.0, -7.0) - (-6.0) / (1.0 + np.exp(-a))) < 1e-5
    # alpha = 1, no clamp in reach: silu(g) * (u + 1)
    assert abs(ob.swiglu_oai(0.7, 0.3, 1.0, 1e9) - 0.7 / (1 + np.exp(-0.7)) * 1.3) < 1e-6


# ---- an independent numpy forward of the gpt-oss arrangement -----------------------------------
def _deq(entry):
    dtype, data, rows, cols = entry
    return ob.dequantize(dtype, data, cols).astype(np.float64)


def _numpy_forward(cfg, w, tokens):
    """float64, straight from the layer description: every row attends causally."""
    H, nq, nkv, hd, F = cfg["hidden"], cfg["n_q_heads"], cfg["n_kv_heads"], cfg["head_dim"], cfg["ffn"]
    G = nq // nkv
    n = len(tokens)
    eps = cfg["rms_eps"]
    freqs = np.asarray(cfg["rope_freqs"], np.float64)
    ms = cfg["rope_mscale"]
    rms = lambda x, g: x / np.sqrt((x * x).mean(-1, keepdims=True) + eps) * g

    def rope(x, heads):  # x [n, heads*hd]
        x = x.reshape(n, heads, hd).copy()
        ang = np.arange(n)[:, None] * freqs[None, :]
        c, s = np.cos(ang)[:, None, :] * ms, np.sin(ang)[:, None, :] * ms
        a, b = x[..., : hd // 2].copy(), x[..., hd // 2:].copy()
        x[..., : hd // 2] = a * c - b * s
        x[..., hd // 2:] = a * s + b * c
        return x

    x = _deq(w["embed"])[tokens]
    for lw in w["layers"]:
        h = rms(x, _deq(lw["attn_norm"])[0])
        q = h @ _deq(lw["wq"]).T + _deq(lw["bq"])[0]
        k = h @ _deq(lw["wk"]).T + _deq(lw["bk"])[0]
        v = (h @ _deq(lw["wv"]).T + _deq(lw["bv"])[0]).reshape(n, nkv, hd)
        q, k = rope(q, nq), rope(k, nkv)
        sinks = _deq(lw["sinks"])[0]
        att = np.zeros((n, nq, hd))
        for i in range(n):
            lo = max(0, i + 1 - lw["window"]) if lw.get("window") else 0
            for qh in range(nq):
                sc = (k[lo:i + 1, qh // G] @ q[i, qh]) * cfg["attn_scale"]
                mx = max(sc.max(), sinks[qh])
                e = np.exp(sc - mx)
                att[i, qh] = (e[:, None] * v[lo:i + 1, qh // G]).sum(0) / (e.sum() + np.exp(sinks[qh] - mx))
        x = x + att.reshape(n, nq * hd) @ _deq(lw["wo"]).T + _deq(lw["bo"])[0]
        m = rms(x, _deq(lw["ffn_norm"])[0])
        E, K = lw["n_experts"], lw["top_k"]
        logits = m @ _deq(lw["router"]).T + _deq(lw["router_bias"])[0]
        wg, wu, wd = _deq(lw["we_gate"]), _deq(lw["we_up"]), _deq(lw["we_down"])
        bg, bu, bd = _deq(lw["be_gate"]), _deq(lw["be_up"]), _deq(lw["be_down"])
        out = np.zeros_like(x)
        for i in range(n):
            sel = np.argsort(-logits[i], kind="stable")[:K]
            p = np.exp(logits[i, sel] - logits[i, sel].max())
            p /= p.sum()
            for e, pw in zip(sel, p):
                g = wg[e * F:(e + 1) * F] @ m[i] + bg[e]
                u = wu[e * F:(e + 1) * F] @ m[i] + bu[e]
                gx, uy = np.minimum(g, cfg["act_limit"]), np.clip(u, -cfg["act_limit"], cfg["act_limit"])
                act = gx / (1 + np.exp(-cfg["act_alpha"] * gx)) * (uy + 1)
                out[i] += pw * (wd[e * H:(e + 1) * H] @ act + bd[e])
        x = x + out
    x = rms(x, _deq(w["final_norm"])[0])
    return x @ _deq(w["lm_head"]).T


def _small(window):
    from turbospark_amd import synth
    cfg = dict(synth.CONFIGS["gptoss_small"])
    cfg.update(vocab=512, max_context=64)
    cfg["gptoss"] = dict(cfg["gptoss"], window=window)
    w = synth.make_weights(cfg, seed=11)
    return cfg, w


def test_gptoss_forward_matches_an_independent_numpy_restatement():
    cfg, w = _small(window=6)
    tokens = np.random.default_rng(2).integers(0, cfg["vocab"], 21).astype(np.int32)
    want = _numpy_forward(cfg, w, tokens)
    cpu = ob.Model(cfg, w, round_kv_f16=False, threads=4)
    a, a32 = cpu.verify(tokens[:16], 0, want_f32=True)
    b, b32 = cpu.verify(tokens[16:], 16, want_f32=True)
    got = np.concatenate([a32, b32])
    rng = want.max() - want.min()
    assert np.abs(got - want).max() <= 2e-4 * rng, np.abs(got - want).max() / rng
    assert cpu.route_margin > 1e-4


def test_each_gptoss_term_moves_the_logits():
    """Dropping any one term (a mutation a restatement could suffer) is visible."""
    cfg, w = _small(window=6)
    tokens = np.random.default_rng(3).integers(0, cfg["vocab"], 12).astype(np.int32)

    def run(c, ww):
        return ob.Model(c, ww, round_kv_f16=False, threads=4).verify(tokens, 0, want_f32=True)[1]

    base = run(cfg, w)
    rng = base.max() - base.min()
    for name in ("bq", "bk", "bv", "bo", "sinks", "router_bias", "be_gate", "be_up", "be_down"):
        ww = dict(w, layers=[{k: v for k, v in lw.items() if k != name} for lw in w["layers"]])
        if name in ("bq", "bk", "bv"):   # they come together: zero one instead of dropping it
            ww = dict(w, layers=[dict(lw, **{name: (lw[name][0], np.zeros_like(lw[name][1]), 1, lw[name][3])})
                                 for lw in w["layers"]])
        assert np.abs(run(cfg, ww) - base).max() > 1e-4 * rng, name
    for key, val in (("rope_mscale", 1.0), ("act_alpha", 0.0), ("attn_scale", 0.2)):
        assert np.abs(run(dict(cfg, **{key: val}), w) - base).max() > 1e-4 * rng, key
    nowin = dict(w, layers=[dict(lw, window=0) for lw in w["layers"]])
    assert np.abs(run(cfg, nowin) - base).max() > 1e-4 * rng
    wide = dict(w, layers=[dict(lw, window=64 if lw["window"] else 0) for lw in w["layers"]])
    assert np.array_equal(run(cfg, wide), run(cfg, nowin))  # a window wider than the context is no window
