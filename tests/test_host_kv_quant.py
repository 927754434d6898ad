"""The KV codec's tables as the library computes them on the host (no GPU): equal, by bits, to the oracle's, which
tests/test_oracle_tq.py pins on the reference's recorded vectors; and within the reference's own tolerance of the
recorded codebooks (crates/compute/tests/kv_quant.rs:466-480)."""
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
