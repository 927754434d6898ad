"""The oracle's TurboQuant KV codec (oracle/tq.cpp) pinned on the reference's own vectors and laws:
crates/compute/tests/generated/kv_quant_oracle.rs (packed words, norms and codebooks recorded from mlx-vlm, kept as
tests/golden/kv_quant_oracle.json) and the properties crates/compute/tests/kv_quant.rs asserts, with its tolerances."""
import json
import math
import os

import numpy as np
import pytest

from oracle import binding as ob

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "kv_quant_oracle.json")
MASK = (1 << 64) - 1


class Lcg:
    """The generator of crates/compute/tests/kv_quant.rs:42-74."""

    def __init__(self, seed):
        self.s = seed

    def next(self):
        self.s = (self.s * 6364136223846793005 + 1442695040888963407) & MASK
        return self.s

    def u01(self):
        return (self.next() >> 11) / float(1 << 53)

    def f32(self):
        return np.float32(self.u01() * 2.0 - 1.0)

    def normal(self):
        u1, u2 = max(self.u01(), 1e-12), self.u01()
        return np.float32(math.sqrt(-2.0 * math.log(u1)) * math.cos(2.0 * math.pi * u2))

    def unit(self, dim):
        v = np.array([self.normal() for _ in range(dim)], np.float32)
        return v / np.float32(np.sqrt(np.sum(v * v, dtype=np.float32)))


def shapes():
    return json.load(open(GOLDEN))["shapes"]


@pytest.mark.parametrize("i", range(4))
def test_quantize_row_reproduces_the_recorded_words_and_norms(i):
    """kv_quant.rs (tests):447-505: the recorded signs go in, the packed words must match exactly."""
    s = shapes()[i]
    dim, bits = s["dim"], s["bits"]
    width = ob.tq_packed_words(dim, bits)
    assert width == len(s["packed"]) // 4
    cb = ob.tq_codebook(dim, bits)
    assert cb.size == len(s["codebook"]) and np.abs(cb - np.array(s["codebook"], np.float32)).max() < 1e-4
    mp = ob.tq_midpoints(cb)
    signs = np.array(s["signs"], np.float32)
    rows = np.array(s["input_rows"], np.float32).reshape(4, dim)
    packed = np.array(s["packed"], np.uint32).reshape(4, width)
    for r in range(4):
        norm, words = ob.tq_quantize_row(rows[r], signs, mp, bits)
        assert np.array_equal(words, packed[r]), (dim, bits, r)
        assert abs(norm - s["norms"][r]) / max(s["norms"][r], 1e-6) < 2.0 ** -11
        back = ob.tq_dequantize_row(norm, words, signs, cb, bits, dim)
        # what the recorded words decode to, written out here: norm * H(signs * ...) undone by hand
        idx = ob.tq_unpack(words, bits, dim)
        rot = cb[idx] * np.float32(norm)
        assert np.allclose(back, ob.tq_rht(rot, signs, inverse=True), atol=1e-6)


def test_codebook_is_sorted_symmetric_and_bounded():
    for dim in (64, 128, 256, 512):
        for bits in (2, 3, 4):
            cb = ob.tq_codebook(dim, bits)
            assert cb.size == 1 << bits
            assert np.all(np.diff(cb) > 0) and np.all((cb >= -1) & (cb < 1))
            assert np.abs(cb + cb[::-1]).max() < 3e-4
    assert ob.tq_codebook(64, 0).size == 0 and ob.tq_packed_words(64, 0) == 0 and ob.tq_packed_words(0, 4) == 0


def test_one_bit_codebook_is_the_half_normal_mean_of_the_coordinate_law():
    """A closed form the Lloyd-Max loop does not know: for 1 bit the two centroids are +-E|x| under
    (1-x^2)^((d-3)/2), which is Gamma(d/2) / (sqrt(pi) Gamma((d+1)/2))."""
    for dim in (64, 128, 256):
        want = math.exp(math.lgamma(dim / 2) - math.lgamma((dim + 1) / 2)) / math.sqrt(math.pi)
        cb = ob.tq_codebook(dim, 1)
        assert cb.size == 2 and abs(cb[1] - want) < 2e-4 and abs(cb[0] + want) < 2e-4


def test_index_rule_is_nearest_centroid():
    for dim in (64, 256):
        for bits in (2, 4):
            cb = ob.tq_codebook(dim, bits)
            mp = ob.tq_midpoints(cb)
            assert np.allclose(mp, (cb[:-1] + cb[1:]) / 2)
            g = Lcg(12345)
            # a row whose rotation is known: x * e_0 + sqrt(1 - x^2) * e_1 sent through the inverse rotation
            signs = ob.tq_sign_vector(dim, 0)
            for _ in range(200):
                x = float(g.f32())
                rot = np.zeros(dim, np.float32)
                rot[0], rot[1] = x, math.sqrt(max(0.0, 1 - x * x))
                row = ob.tq_rht(rot, signs, inverse=True)
                _, words = ob.tq_quantize_row(row, signs, mp, bits)
                idx = ob.tq_unpack(words, bits, dim)
                got = ob.tq_rht(row / np.float32(np.linalg.norm(row)), signs)
                for j in (0, 1):
                    d = np.abs(cb - got[j])
                    assert d[idx[j]] <= d.min() + 1e-6


def test_packing_straddles_a_word_boundary_and_round_trips():
    idx = np.zeros(11, np.uint32)
    idx[10] = 7
    pk = ob.tq_pack(idx, 3)
    assert pk.size == ob.tq_packed_words(11, 3) == 2
    assert pk[0] == (3 << 30) and pk[1] == 1
    assert np.array_equal(ob.tq_unpack(pk, 3, 11), idx)
    g = Lcg(99)
    for bits in range(1, 17):
        for length in (0, 1, 7, 31, 32, 33, 64, 100, 257):
            v = np.array([g.next() >> 40 & ((1 << bits) - 1) for _ in range(length)], np.uint32)
            pk = ob.tq_pack(v, bits)
            assert pk.size == ob.tq_packed_words(length, bits) == (length * bits + 31) // 32
            assert np.array_equal(ob.tq_unpack(pk, bits, length), v)
    with pytest.raises(ValueError):
        ob.tq_pack(np.array([4], np.uint32), 2)
    with pytest.raises(ValueError):
        ob.tq_pack(np.array([1], np.uint32), 17)
    with pytest.raises(ValueError):
        ob.tq_unpack(np.zeros(2, np.uint32), 17, 1)


def test_wht_is_the_orthonormal_hadamard_matrix():
    for n in (1, 2, 8, 64):
        h = np.array([[1.0]])
        while h.shape[0] < n:
            h = np.block([[h, h], [h, -h]])
        h /= math.sqrt(n)
        x = np.random.default_rng(n).standard_normal(n).astype(np.float32)
        assert np.allclose(ob.tq_wht(x), h @ x, atol=1e-5)


def test_rht_inverse_undoes_forward_and_preserves_norm():
    g = Lcg(2024)
    for dim in (64, 128, 256, 512):
        for seed in (0, 1, 7):
            signs = ob.tq_sign_vector(dim, seed)
            assert np.all(np.abs(signs) == 1)
            x = np.array([g.f32() for _ in range(dim)], np.float32)
            y = ob.tq_rht(x, signs)
            assert abs(np.linalg.norm(y) - np.linalg.norm(x)) < 1e-4 * np.linalg.norm(x)
            assert np.abs(ob.tq_rht(y, signs, inverse=True) - x).max() < 1e-5


def test_key_and_value_signs_differ_and_repeat():
    for dim in (64, 128, 256):
        k, v = ob.tq_sign_vector(dim, ob.TQ_KEY_SEED), ob.tq_sign_vector(dim, ob.TQ_VALUE_SEED)
        assert not np.array_equal(k, v)
        assert np.array_equal(k, ob.tq_sign_vector(dim, ob.TQ_KEY_SEED))
        assert 0.25 * dim < (k > 0).sum() < 0.75 * dim


def test_distortion_on_unit_vectors_matches_the_published_figures():
    """kv_quant.rs (tests):294-331, mlx-vlm's recorded mean squared errors at d=64."""
    g = Lcg(7)
    vecs = [g.unit(64) for _ in range(256)]
    signs = ob.tq_sign_vector(64, 0)
    for bits, target in ((1, 0.36), (2, 0.117), (3, 0.03)):
        cb = ob.tq_codebook(64, bits)
        mp = ob.tq_midpoints(cb)
        mse = 0.0
        for v in vecs:
            norm, words = ob.tq_quantize_row(v, signs, mp, bits)
            back = ob.tq_dequantize_row(norm, words, signs, cb, bits, 64)
            mse += float(np.sum((v - back) ** 2))
        mse /= len(vecs)
        assert abs(mse - target) <= max(0.25 * target, 0.02), (bits, mse)


def _quantized(g, dim, seq, nkv, kbits, vbits):
    ks, vs = ob.tq_sign_vector(dim, ob.TQ_KEY_SEED), ob.tq_sign_vector(dim, ob.TQ_VALUE_SEED)
    kc, vc = ob.tq_codebook(dim, kbits), ob.tq_codebook(dim, vbits)
    km, vm = ob.tq_midpoints(kc), ob.tq_midpoints(vc)
    kw, kn, vw, vn, kd, vd = [], [], [], [], [], []
    for _ in range(seq * nkv):
        x = np.array([g.f32() for _ in range(dim)], np.float32)
        n, w = ob.tq_quantize_row(x, ks, km, kbits)
        kw.append(w), kn.append(n), kd.append(ob.tq_dequantize_row(n, w, ks, kc, kbits, dim))
        x = np.array([g.f32() for _ in range(dim)], np.float32)
        n, w = ob.tq_quantize_row(x, vs, vm, vbits)
        vw.append(w), vn.append(n), vd.append(ob.tq_dequantize_row(n, w, vs, vc, vbits, dim))
    t = dict(k_signs=ks, k_cb=kc, v_signs=vs, v_cb=vc)
    return (np.array(kw), np.array(kn, np.float32), np.array(vw), np.array(vn, np.float32),
            np.array(kd).reshape(seq, nkv, dim), np.array(vd).reshape(seq, nkv, dim), t)


def test_rotated_space_attention_equals_attention_over_the_decoded_rows():
    """kv_quant.rs (tests):381-440, widened to grouped heads, sinks and the K3/V4 split; the decoded rows go
    through the plain attention the other tests pin."""
    for dim, nq, nkv, seq, bits, vbits in ((64, 1, 1, 5, 4, 4), (128, 4, 2, 9, 3, 3), (64, 6, 3, 17, 2, 2), (128, 4, 1, 11, 3, 4)):
        g = Lcg(321 + dim + bits)
        q = np.array([g.f32() for _ in range(nq * dim)], np.float32)
        kw, kn, vw, vn, kd, vd, t = _quantized(g, dim, seq, nkv, bits, vbits)
        for sinks in (None, np.linspace(-1, 1, nq).astype(np.float32)):
            got = ob.tq_attention(q, kw, kn, vw, vn, dim, nq, nkv, seq, bits, sinks=sinks, v_bits=vbits, **t)
            want = ob.causal_attention(q.reshape(nq, dim), kd, vd, dim, nq, nkv, seq, 0, 0.0, sinks)
            assert np.abs(got - want).max() < 1e-3, (dim, nq, nkv, seq, bits)


def test_sinks_enter_the_denominator_only():
    g = Lcg(55)
    q = np.array([g.f32() for _ in range(64)], np.float32)
    kw, kn, vw, vn, _, _, t = _quantized(g, 64, 6, 1, 3, 3)
    a = ob.tq_attention(q, kw, kn, vw, vn, 64, 1, 1, 6, 3, **t)
    b = ob.tq_attention(q, kw, kn, vw, vn, 64, 1, 1, 6, 3, sinks=np.array([10.0], np.float32), **t)
    assert np.linalg.norm(b) < 0.5 * np.linalg.norm(a)
    # and the direction is unchanged: only the scale moves
    assert np.abs(b / np.linalg.norm(b) - a / np.linalg.norm(a)).max() < 1e-4


def test_the_oracle_model_keeps_decoded_rows_on_the_layers_the_policy_names():
    """crates/model-io/src/kv_quant.rs:102-107 (every full-attention layer but the last, all of them in a stack
    of two) and crates/runtime/src/kv_write.rs:66-118 (the fp16 staging row is what gets quantized).  Layer 0
    sees the same inputs with and without the codec, so its cached rows must be the decoded fp16 rows of the
    plain model; the last layer's rows stay fp16."""
    from turbospark_amd import synth
    two = dict(synth.CONFIGS["small_q4_k"], max_context=32)
    m2 = ob.Model(two, synth.make_weights(two, seed=5), kv_bits=(4, 4))
    assert [m2.layer_quantized(l) for l in range(2)] == [True, True]
    cfg = dict(two, n_layers=3)
    w = synth.make_weights(cfg, seed=5)
    n, nkv, hd = cfg["n_layers"], cfg["n_kv_heads"], cfg["head_dim"]
    plain = ob.Model(cfg, w, round_kv_f16=True, threads=8)
    quant = ob.Model(cfg, w, round_kv_f16=True, threads=8, kv_bits=(3, 4))
    assert [quant.layer_quantized(l) for l in range(n)] == [True] * (n - 1) + [False]
    assert not any(plain.layer_quantized(l) for l in range(n))
    feed = np.arange(7, dtype=np.int32) * 11 % cfg["vocab"]
    lp, lq = plain.verify(feed, 0, want_f32=True), quant.verify(feed, 0, want_f32=True)
    kp, vp = plain.kv(0)
    kq, vq = quant.kv(0)
    for side, rows, got, bits, seed in (("k", kp, kq, 3, ob.TQ_KEY_SEED), ("v", vp, vq, 4, ob.TQ_VALUE_SEED)):
        signs, cb = ob.tq_sign_vector(hd, seed), ob.tq_codebook(hd, bits)
        mp = ob.tq_midpoints(cb)
        for pos in range(7):
            for h in range(nkv):
                x = rows[pos, h]
                norm, words = ob.tq_quantize_row(x, signs, mp, bits)
                want = ob.tq_dequantize_row(norm, words, signs, cb, bits, hd)
                assert np.array_equal(got[pos, h], want), (side, pos, h)
    # the last layer keeps fp16 rows: every value is its own fp16 rounding
    kl, _ = quant.kv(n - 1)
    assert np.array_equal(kl[:7], kl[:7].astype(np.float16).astype(np.float32))
    # and the codec does move the logits
    a, b = np.asarray(lp[1], np.float32), np.asarray(lq[1], np.float32)
    assert np.abs(a - b).max() / np.abs(a).max() > 1e-4
