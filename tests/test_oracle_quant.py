"""Pins the oracle's block formats against the reference's own golden data and laws.

Mirrors crates/compute/tests/quant_gguf.rs and quant_gguf_mxfp4.rs.
"""
import json
import os

import numpy as np

from oracle import binding as ob


def lcg_weights(n, seed):
    """The reference's test weight generator (crates/compute/tests/quant_gguf.rs:26-34)."""
    s = (seed * 2654435761 + 1) & 0xFFFFFFFF
    out = np.empty(n, np.float32)
    for i in range(n):
        s = (s * 1664525 + 1013904223) & 0xFFFFFFFF
        out[i] = np.float32(np.float32(s >> 8) / np.float32(1 << 23)) - np.float32(1.0)
    return out


def test_f16_conversion_matches_ieee_for_every_bit_pattern():
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = np.array([ob.lib().tso_f16_to_f32(int(b)) for b in bits], np.float32)
    finite = np.isfinite(want)
    assert np.array_equal(got[finite], want[finite])
    assert np.all(np.isnan(got[np.isnan(want)]))
    # and back: every finite f16 round-trips; halfway cases round to even
    back = np.array([ob.lib().tso_f32_to_f16(float(v)) for v in want[finite]], np.uint16)
    assert np.array_equal(back, bits[finite])
    rng = np.random.default_rng(0)
    x = np.concatenate([rng.standard_normal(20000).astype(np.float32) * 10.0 ** rng.integers(-9, 6, 20000),
                        np.float32([65504, 65519.99, 65520, 1e-8, 5.96e-8, 2.98e-8, 2.9802322e-8, 0.0, -0.0])])
    got = np.array([ob.lib().tso_f32_to_f16(float(v)) for v in x], np.uint16)
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    assert np.array_equal(got, want)


def test_bf16_rne_and_nan_quieting():
    L = ob.lib()
    assert L.tso_f32_to_bf16(1.0) == 0x3F80
    # 1 + 2^-8 is exactly halfway between 0x3F80 and 0x3F81 -> even (0x3F80)
    assert L.tso_f32_to_bf16(float(np.float32(1.0 + 2.0 ** -8))) == 0x3F80
    assert L.tso_f32_to_bf16(float(np.float32(1.0 + 3 * 2.0 ** -8))) == 0x3F82
    nanbits = L.tso_f32_to_bf16(float("nan"))
    assert (nanbits & 0x7F80) == 0x7F80 and (nanbits & 0x007F) != 0
    assert L.tso_bf16_to_f32(0x4049) == np.float32(3.140625)


def test_q4k_hand_packed_superblock_decodes_to_the_documented_formula(golden):
    g = json.load(open(os.path.join(golden, "q4k_handpacked.json")))
    quants = [(e * 7 + 3) % 16 for e in range(256)]
    block = bytes(g["D_BITS"] + g["DMIN_BITS"] + g["PACKED"])
    body = bytearray()
    for grp in range(4):
        for l in range(32):
            at = grp * 64 + l
            body.append(quants[at] | (quants[at + 32] << 4))
    block = np.frombuffer(block + bytes(body), np.uint8)
    assert block.size == 144
    got = ob.dequantize(ob.Q4_K, block, 256)[0]
    for e in range(256):
        j = e // 32
        want = np.float32(g["d"]) * np.float32(g["LS"][j]) * np.float32(quants[e]) - np.float32(g["dmin"]) * np.float32(g["LM"][j])
        assert got[e] == want, (e, j)
    # the scale/min unpack on its own, all eight sub-blocks
    import ctypes as C
    packed = np.array(g["PACKED"], np.uint8)
    for j in range(8):
        sc, mn = C.c_uint8(), C.c_uint8()
        ob.lib().tso_q4_k_scale_min(j, C.c_void_p(packed.ctypes.data), C.byref(sc), C.byref(mn))
        assert (sc.value, mn.value) == (g["LS"][j], g["LM"][j])


def test_q4k_round_trip_stays_inside_one_quantization_step():
    w = lcg_weights(512, 11)
    out = ob.dequantize(ob.Q4_K, ob.quantize(ob.Q4_K, w.reshape(1, -1)), 512)[0]
    for j in range(16):
        sub = w[j * 32:(j + 1) * 32]
        lo = min(0.0, sub.min())
        hi = max(lo, sub.max())
        step = (hi - lo) / 15.0
        bound = step * 0.5 + (hi - lo) * 0.05
        assert np.all(np.abs(out[j * 32:(j + 1) * 32] - sub) <= bound)


def test_q4k_min_term_carries_the_sign_and_zero_block_is_zero():
    w = np.array([-1.0 + (e % 32) / 64.0 for e in range(256)], np.float32)
    out = ob.dequantize(ob.Q4_K, ob.quantize(ob.Q4_K, w.reshape(1, -1)), 256)[0]
    assert np.all(out < 0) and np.all(np.abs(out - w) < 0.05)
    z = ob.quantize(ob.Q4_K, np.zeros((1, 256), np.float32))
    assert np.all(z == 0)
    assert np.all(ob.dequantize(ob.Q4_K, z, 256) == 0)


def test_q4k_quantizer_is_idempotent_on_its_own_output():
    w = lcg_weights(1024, 3) * 0.05
    q1 = ob.quantize(ob.Q4_K, w.reshape(1, -1))
    d1 = ob.dequantize(ob.Q4_K, q1, 1024)
    q2 = ob.quantize(ob.Q4_K, d1)
    d2 = ob.dequantize(ob.Q4_K, q2, 1024)
    # a second pass may re-fit ranges, but must stay within one step of the first decode
    assert np.max(np.abs(d2 - d1)) <= np.max(np.abs(d1 - w)) * 2 + 1e-6


def _q6k_golden_block(golden):
    g = json.load(open(os.path.join(golden, "q6k_handpacked.json")))
    block = bytes([g["ql_byte"]] * 128 + [g["qh_byte"]] * 64 + [s & 0xFF for s in g["scales"]]) + \
        int(g["d_bits"]).to_bytes(2, "little")
    assert len(block) == 210
    return g, np.frombuffer(block, np.uint8)


def test_q6k_hand_packed_superblock_decodes_to_the_documented_formula(golden):
    """crates/compute/tests/quant_gguf.rs:413-445: ql = 0x93, qh = 0xB1 give the levels 19, 3, 57, 41,
    i.e. quants -13, -29, 25, 9; half of the sixteen signed scales are negative; `==` throughout."""
    g, block = _q6k_golden_block(golden)
    out = ob.dequantize(ob.Q6_K, block, 256)[0]
    for h in range(2):
        for k in range(4):
            for l in range(32):
                want = np.float32(g["d"]) * np.float32(g["scales"][h * 8 + l // 16 + 2 * k]) * np.float32(g["quants"][k])
                assert out[h * 128 + k * 32 + l] == want, (h, k, l)
    for at, want in g["spot"].items():
        assert out[int(at)] == want


def test_q6k_round_trip_signed_scales_and_zero_block():
    # quant_gguf.rs:447-500: inside one quantization step; both scale signs occur and no element flips
    w = lcg_weights(512, 41)
    out = ob.dequantize(ob.Q6_K, ob.quantize(ob.Q6_K, w.reshape(1, -1)), 512)[0]
    for j in range(32):
        sub = w[16 * j:16 * j + 16]
        amax = np.abs(sub).max()
        assert np.abs(out[16 * j:16 * j + 16] - sub).max() <= amax / 32.0 * 0.5 + amax * 2e-2
    e = np.arange(256)
    w = (np.where((e // 16) % 2 == 0, 1.0, -1.0) * (1.0 + (e % 16) / 16.0)).astype(np.float32)
    q = ob.quantize(ob.Q6_K, w.reshape(1, -1))[0]
    scales = q[192:208].view(np.int8)
    assert (scales < 0).any() and (scales > 0).any()
    out = ob.dequantize(ob.Q6_K, q, 256)[0]
    assert np.array_equal(np.sign(out), np.sign(w)) and np.abs(out - w).max() < 0.1
    z = ob.quantize(ob.Q6_K, np.zeros((1, 256), np.float32))[0]
    assert np.all(ob.dequantize(ob.Q6_K, z, 256) == 0.0) and ob.row_bytes(ob.Q6_K, 512) == 420


def test_q8_0_round_trip_sign_zero_and_idempotence():
    w = lcg_weights(96, 7)
    q = ob.quantize(ob.Q8_0, w.reshape(1, -1))
    assert q.shape == (1, 3 * 34)
    out = ob.dequantize(ob.Q8_0, q, 96)[0]
    for b in range(3):
        blk = w[b * 32:(b + 1) * 32]
        amax = np.abs(blk).max()
        assert np.all(np.abs(out[b * 32:(b + 1) * 32] - blk) <= amax / 127.0 * 0.5 + amax * 1e-3)
    assert np.all(np.sign(out[np.abs(w) > 0.02]) == np.sign(w[np.abs(w) > 0.02]))
    q2 = ob.quantize(ob.Q8_0, out.reshape(1, -1))
    assert np.array_equal(q, q2)  # quantize(dequantize(q)) == q
    z = ob.quantize(ob.Q8_0, np.zeros((1, 32), np.float32))
    assert np.all(z == 0) and np.all(ob.dequantize(ob.Q8_0, z, 32) == 0)
    # independent numpy restatement of the decode
    qi = q[0].reshape(3, 34)
    d = qi[:, :2].copy().view(np.float16).astype(np.float32)
    want = (qi[:, 2:].view(np.int8).astype(np.float32) * d).reshape(-1)
    assert np.array_equal(out, want)


def test_mxfp4_decode_matches_ggml_bytes_and_floats(golden):
    g = json.load(open(os.path.join(golden, "mxfp4_ggml_oracle.json")))
    b = np.array(g["bytes"], np.uint8)
    got = ob.dequantize(ob.MXFP4, b, 128)[0]
    assert np.array_equal(got, np.array(g["floats"], np.float32))
    for e in range(256):
        assert np.float32(ob.lib().tso_mxfp4_scale(e)) * np.float32(g["codebook"][1]) == np.float32(g["e8m0_times_codebook1"][e])
    # codebook through a unit-scale block (byte 128), every index in both nibble halves
    blk = np.zeros(17, np.uint8)
    blk[0] = 128
    for j in range(16):
        blk[1 + j] = j | ((15 - j) << 4)
    dec = ob.dequantize(ob.MXFP4, blk, 32)[0]
    assert np.array_equal(dec[:16], np.array(g["codebook"], np.float32))
    assert np.array_equal(dec[16:], np.array(g["codebook"], np.float32)[::-1])
    # split halves: low nibble -> element j, high nibble -> j + 16 (mutation: adjacent would differ)
    assert not np.array_equal(dec[0:32:2], np.array(g["codebook"], np.float32))


def test_mxfp4_encoder_is_nearest_codebook_value_brute_force():
    rng = np.random.default_rng(5)
    w = (rng.standard_normal((4, 64)) * np.array([[0.02], [1.0], [37.0], [1e-4]])).astype(np.float32)
    q = ob.quantize(ob.MXFP4, w)
    dec = ob.dequantize(ob.MXFP4, q, 64)
    code = np.array([0, 1, 2, 3, 4, 6, 8, 12], np.float32)
    code = np.concatenate([code, -code[1:]])
    for r in range(4):
        for b in range(2):
            e = q[r, b * 17]
            d = np.float32(ob.lib().tso_mxfp4_scale(int(e)))
            blk = w[r, b * 32:(b + 1) * 32]
            assert 12 * d >= np.abs(blk).max() > 6 * d * 0.99  # tightest exponent that covers amax
            best = np.abs(blk[:, None] / d - code[None, :]).min(axis=1)
            err = np.abs(dec[r, b * 32:(b + 1) * 32] / d - blk / d)
            assert np.allclose(err, best, rtol=0, atol=1e-6)


def test_gemv_is_dequantize_then_sequential_dot():
    w = lcg_weights(4 * 256, 21).reshape(4, 256) * 0.1
    x = lcg_weights(256, 22)
    for dt in (ob.Q4_K, ob.Q8_0, ob.F32):
        qb = ob.quantize(dt, w)
        deq = ob.dequantize(dt, qb, 256)
        want = np.empty(4, np.float32)
        for r in range(4):
            acc = np.float32(0)
            for k in range(256):
                acc = np.float32(acc + np.float32(deq[r, k] * x[k]))
            want[r] = acc
        assert np.array_equal(ob.gemv(dt, qb, 4, 256, x), want)


def test_q5k_decodes_exactly_what_ggml_decodes(golden):
    """crates/compute/tests/quant_gguf.rs:548-600: two superblocks ggml quantized, the floats ggml decoded
    from them, `==`; without the fifth-bit run the values change (the bit carries 16 quant levels)."""
    import json
    g = json.load(open(os.path.join(golden, "q5k_ggml_oracle.json")))
    raw = np.array(g["bytes"], np.uint8)
    want = np.array(g["floats"], np.float32)
    assert raw.size == 2 * 176 and want.size == 512 and ob.row_bytes(ob.Q5_K, 512) == 352
    got = ob.dequantize(ob.Q5_K, raw, 512)[0]
    assert np.array_equal(got, want)
    stripped = raw.copy()
    for b in range(2):
        stripped[b * 176 + 16:b * 176 + 48] = 0
    assert not np.array_equal(ob.dequantize(ob.Q5_K, stripped, 512)[0], want)


def test_q5k_encoder_round_trip():
    """The encoder is this project's (the reference only decodes Q5_K): decode(encode(x)) stays inside
    half a quantization step of each sub-block plus the 6-bit scale / min rounding; a zero block is zeros."""
    w = lcg_weights(1024, 43)
    out = ob.dequantize(ob.Q5_K, ob.quantize(ob.Q5_K, w.reshape(1, -1)), 1024)[0]
    for j in range(32):
        sub = w[32 * j:32 * j + 32]
        span = max(sub.max(), 0.0) - min(sub.min(), 0.0)
        assert np.abs(out[32 * j:32 * j + 32] - sub).max() <= span / 31.0 * 0.5 + span * 3e-2
    q4 = ob.dequantize(ob.Q4_K, ob.quantize(ob.Q4_K, w.reshape(1, -1)), 1024)[0]
    assert np.abs(out - w).mean() < 0.7 * np.abs(q4 - w).mean()   # the fifth bit buys precision
    z = ob.quantize(ob.Q5_K, np.zeros((1, 256), np.float32))[0]
    assert np.all(ob.dequantize(ob.Q5_K, z, 256) == 0.0)
