"""The KV codec's tables as the library computes them on the host (no GPU): equal, by bits, to the oracle's, which
tests/test_oracle_tq.py pins on the reference's recorded vectors; and within the reference's own tolerance of the
recorded codebooks (crates/compute/tests/kv_quant.rs:466-480)."""
import ctypes as C
import json
import os

import numpy as np
import pytest

from oracle import binding as ob
from turbospark_amd import ffi
from turbospark_amd.producer import parse_kv_bits

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "kv_quant_oracle.json")


@pytest.mark.parametrize("dim", [64, 128, 256])
@pytest.mark.parametrize("bits", [1, 2, 3, 4])
def test_library_tables_equal_the_oracles(dim, bits):
    for value_side, seed in ((False, ob.TQ_KEY_SEED), (True, ob.TQ_VALUE_SEED)):
        signs, cb, mid = ffi.kv_quant_tables(dim, bits, value_side)
        assert np.array_equal(signs, ob.tq_sign_vector(dim, seed))
        want = ob.tq_codebook(dim, bits)
        assert np.array_equal(cb, want)
        assert np.array_equal(mid, ob.tq_midpoints(want))


def test_library_codebooks_against_the_recorded_ones():
    for s in json.load(open(GOLDEN))["shapes"]:
        _, cb, _ = ffi.kv_quant_tables(s["dim"], s["bits"])
        assert np.abs(cb - np.array(s["codebook"], np.float32)).max() < 1e-4


def test_tables_refuse_what_the_rotation_cannot_take():
    """crates/model-io/src/kv_quant.rs:116-122: a power of two in 32..=512."""
    for dim, bits in ((96, 4), (16, 4), (1024, 4), (128, 0), (128, 5)):
        with pytest.raises(ffi.TsvError):
            ffi.kv_quant_tables(dim, bits)


def test_kv_bits_spelling():
    """crates/model-io/src/kv_quant.rs:48-72."""
    assert parse_kv_bits("off") is None
    assert parse_kv_bits("2") == (2, 2) and parse_kv_bits("3") == (3, 3) and parse_kv_bits("4") == (4, 4)
    assert parse_kv_bits("3.5") == (3, 4)
    for bad in ("", "5", "1", "3.0", "on"):
        with pytest.raises(ValueError):
            parse_kv_bits(bad)
    assert ffi.packed_words(128, 3) == 12 and ffi.packed_words(128, 4) == 16 and ffi.packed_words(64, 3) == 6
    assert ffi.packed_words(0, 4) == 0 and ffi.packed_words(64, 0) == 0


def _desc(n_layers, nkv, hd, windows=None, rings=None, kv_bits=(0, 0)):
    layers = (ffi.Layer * n_layers)()
    for l in range(n_layers):
        layers[l].window = (windows or [0] * n_layers)[l]
        layers[l].ring = (rings or [0] * n_layers)[l]
    d = ffi.ModelDesc()
    d.n_layers, d.n_kv_heads, d.head_dim = n_layers, nkv, hd
    d.kv_k_bits, d.kv_v_bits = kv_bits
    d.layers = C.cast(layers, C.POINTER(ffi.Layer))
    d._keep = layers
    return d


def _row(d, layer):
    k, v = C.c_int64(), C.c_int64()
    ffi.check(ffi.lib().tsv_kv_row_bytes(C.byref(d), layer, C.byref(k), C.byref(v)))
    return k.value, v.value


def test_what_a_position_costs():
    """crates/model-io/src/kv_quant.rs:141-205 (tq_row_bytes, kv_layer_strides): per kv head an f32 norm and
    ceil(head_dim * bits / 32) words; K and V can differ (12 against 16 words at K3/V4, head_dim 128); the last layer of a
    stack of more than two, and every windowed layer, keep fp16 rows."""
    fp16 = 8 * 128 * 2
    d = _desc(32, 8, 128)
    assert _row(d, 0) == (fp16, fp16) and _row(d, 31) == (fp16, fp16)
    d = _desc(32, 8, 128, kv_bits=(4, 4))
    assert _row(d, 0) == (8 * (4 + 4 * 16), 8 * (4 + 4 * 16)) == (544, 544)
    assert _row(d, 30) == (544, 544) and _row(d, 31) == (fp16, fp16)
    d = _desc(32, 8, 128, kv_bits=(3, 4))
    assert _row(d, 5) == (8 * (4 + 4 * 12), 544)
    d = _desc(32, 8, 128, kv_bits=(2, 2))
    assert _row(d, 5) == (8 * (4 + 4 * 8), 8 * (4 + 4 * 8)) == (288, 288)
    # the value side at three bits is kept sixteen positions to 64 bits per dimension: a third more than the packed row
    d = _desc(32, 8, 128, kv_bits=(3, 3))
    assert _row(d, 5) == (8 * (4 + 4 * 12), 544)
    # a stack of two quantizes both layers; windowed layers never
    d = _desc(2, 2, 64, kv_bits=(4, 4))
    assert _row(d, 0) == _row(d, 1) == (2 * (4 + 32), 2 * (4 + 32))
    d = _desc(4, 2, 64, windows=[24, 0, 24, 0], kv_bits=(4, 4))
    assert _row(d, 0) == _row(d, 2) == (256, 256) and _row(d, 1) == (72, 72) and _row(d, 3) == (256, 256)
    with pytest.raises(ffi.TsvError):
        _row(d, 4)


def test_what_a_context_costs():
    """crates/model-io/src/context_policy.rs:294-333: capacity times stride, layer by layer; a ring stops growing."""
    kvb = ffi.lib().tsv_kv_bytes_for_context
    d = _desc(32, 8, 128)
    assert kvb(C.byref(d), 4096) == 32 * 4096 * 4096 == 536870912        # the 8B shape: 4096 B per position and layer
    assert kvb(C.byref(d), 4090) == 32 * 4096 * 4096                      # rounded up to blocks of sixteen
    d = _desc(32, 8, 128, kv_bits=(4, 4))
    assert kvb(C.byref(d), 4096) == 4096 * (31 * 1088 + 4096)
    d = _desc(4, 2, 64, windows=[24, 0, 24, 0], rings=[1, 0, 1, 0])
    assert kvb(C.byref(d), 1024) == 2 * 1024 * 512 + 2 * (32 + 32) * 512  # two rings of round16(24) + 32 positions
    assert kvb(C.byref(d), 48) == 4 * 48 * 512                            # a ring is never larger than the context
    assert kvb(C.byref(d), 0) == -1
