"""Pins the oracle's operators: closed forms, the reference's literal profiles and
independent brute-force restatements (crates/compute/src/{rms_norm,rope,attention}.rs tests)."""
import json
import math
import os

import numpy as np

from oracle import binding as ob


def test_rms_norm_closed_forms():
    x = np.array([3.0, 4.0], np.float32)
    y = ob.rms_norm(x, np.ones(2, np.float32), 0.0)
    assert np.allclose(y, x / math.sqrt(12.5), rtol=1e-6)
    # weight multiplies, eps joins the mean (a dropped eps or a sum-instead-of-mean fails)
    y = ob.rms_norm(np.array([1, 1, 1, 1], np.float32), np.array([1, 2, 3, 4], np.float32), 3.0)
    assert np.allclose(y, np.array([1, 2, 3, 4]) / 2.0, rtol=1e-6)
    rng = np.random.default_rng(1)
    x = rng.standard_normal(512).astype(np.float32)
    w = rng.standard_normal(512).astype(np.float32)
    want = x.astype(np.float64) * w / math.sqrt(np.mean(x.astype(np.float64) ** 2) + 1e-5)
    assert np.allclose(ob.rms_norm(x, w, 1e-5), want, rtol=2e-6, atol=1e-6)


def test_rope_neox_is_a_rotation_of_half_split_pairs():
    hd = 8
    x = np.arange(1, hd + 1, dtype=np.float32)
    # position 0: identity
    assert np.array_equal(ob.rope_neox(x, 1, 1, hd, hd // 2, 0, 10000.0), x)
    pos, theta = 5, 10000.0
    y = ob.rope_neox(x, 1, 1, hd, hd // 2, pos, theta)
    for i in range(hd // 2):
        ang = pos * theta ** (-2 * i / hd)
        c, s = math.cos(ang), math.sin(ang)
        assert abs(y[i] - (x[i] * c - x[i + hd // 2] * s)) < 1e-5          # pair is (i, i + hd/2)
        assert abs(y[i + hd // 2] - (x[i] * s + x[i + hd // 2] * c)) < 1e-5  # not (2i, 2i+1)
    # norm of each pair is preserved; partial rotation leaves the tail alone
    y2 = ob.rope_neox(x, 1, 1, hd, 2, pos, theta)
    assert np.array_equal(y2[2:4], x[2:4]) and np.array_equal(y2[6:8], x[6:8])
    # heads and tokens are independent copies of the same rotation
    xx = np.tile(x, 6)
    yy = ob.rope_neox(xx, 2, 3, hd, hd // 2, pos, theta)
    assert np.array_equal(yy.reshape(6, hd), np.tile(y, (6, 1)))


def test_llama3_factors_match_the_published_profile(golden):
    g = json.load(open(os.path.join(golden, "llama3_rope_profile.json")))
    p = g["params"]
    f = ob.llama3_rope_factors(p["rotary_dim"], p["base"], p["factor"], p["low"], p["high"],
                               p["original_context"])
    assert f.size == 64
    assert np.all(f[:29] == 1.0)
    assert np.all(np.abs(f[29:35] - np.array(g["ramp"], np.float32)) < 1e-5)
    assert np.all(f[35:] == 8.0)
    tiny = ob.llama3_rope_factors(8, 10000.0, 4.0, 1.0, 4.0, 8.0)
    assert np.all(np.abs(tiny - np.float32([math.pi, 4, 4, 4])) < 1e-6)
    for bad in [(128, 500000.0, 0.0, 1.0, 4.0, 8192.0), (128, 500000.0, 8.0, 4.0, 4.0, 8192.0),
                (128, 500000.0, 8.0, 1.0, 4.0, 0.0), (127, 500000.0, 8.0, 1.0, 4.0, 8192.0),
                (128, float("nan"), 8.0, 1.0, 4.0, 8192.0)]:
        assert ob.llama3_rope_factors(*bad) is None


def test_frequency_table_divides_and_unit_divisors_reproduce_plain_rope():
    f = ob.llama3_rope_factors(128, 500000.0, 8.0, 1.0, 4.0, 8192.0)
    scaled = ob.rope_frequencies_with_factors(128, 500000.0, f)
    plain = ob.rope_frequencies_with_factors(128, 500000.0, np.ones(64, np.float32))
    assert scaled[0] == plain[0]
    assert abs(scaled[63] * 8.0 - plain[63]) <= plain[63] * 1e-6
    # with unit divisors the table variant is the scalar-theta rotation (to fp32 rounding of
    # exp(log) vs pow)
    x = np.random.default_rng(2).standard_normal(128).astype(np.float32)
    a = ob.rope_neox(x, 1, 1, 128, 64, 77, 500000.0)
    b = ob.rope_neox_freqs(x, 1, 1, 128, 64, 77, plain)
    assert np.allclose(a, b, atol=2e-4)


def brute_attention(q, k, v, hd, nq, nkv, seq, window, scale, sinks):
    group = nq // nkv
    out = np.zeros((nq, hd))
    start = max(0, seq - window) if window else 0
    for h in range(nq):
        kh = h // group
        s = np.array([np.dot(q[h], k[p, kh]) * scale for p in range(start, seq)], np.float64)
        m = s.max() if sinks is None else max(s.max(), sinks[h])
        e = np.exp(s - m)
        den = e.sum() + (0.0 if sinks is None else math.exp(sinks[h] - m))
        out[h] = (e[:, None] * v[start:seq, kh]).sum(0) / den
    return out


def test_attention_against_brute_force_with_gqa_window_and_sinks():
    rng = np.random.default_rng(3)
    hd, nq, nkv, seq = 16, 6, 2, 37
    q = rng.standard_normal((nq, hd)).astype(np.float32)
    k = rng.standard_normal((seq, nkv, hd)).astype(np.float32)
    v = rng.standard_normal((seq, nkv, hd)).astype(np.float32)
    sinks = rng.standard_normal(nq).astype(np.float32)
    for window in (0, 9):
        for sk in (None, sinks):
            for scale in (0.0, 0.125):
                eff = scale if scale > 0 else 1 / math.sqrt(hd)
                got = ob.causal_attention(q, k, v, hd, nq, nkv, seq, window, scale, sk).reshape(nq, hd)
                want = brute_attention(q.astype(np.float64), k.astype(np.float64), v.astype(np.float64),
                                       hd, nq, nkv, seq, window, eff, sk)
                assert np.allclose(got, want, atol=2e-6), (window, sk is not None, scale)
    # a sink only ever removes mass: with a huge sink the output collapses to ~0
    # (the wrong version that adds it to the numerator would not)
    got = ob.causal_attention(q, k, v, hd, nq, nkv, seq, 0, 0.0, np.full(nq, 50.0, np.float32))
    assert np.max(np.abs(got)) < 1e-6


def test_attention_single_key_returns_its_value_and_uniform_scores_average():
    hd = 4
    q = np.ones((1, hd), np.float32)
    k = np.zeros((3, 1, hd), np.float32)
    v = np.arange(12, dtype=np.float32).reshape(3, 1, hd)
    assert np.array_equal(ob.causal_attention(q, k, v, hd, 1, 1, 1), v[0, 0])
    assert np.allclose(ob.causal_attention(q, k, v, hd, 1, 1, 3), v[:, 0].mean(0), rtol=1e-6)


def test_silu():
    for x in (-3.0, -0.5, 0.0, 0.7, 4.0):
        assert abs(ob.lib().tso_silu(x) - x / (1 + math.exp(-x))) < 1e-6
