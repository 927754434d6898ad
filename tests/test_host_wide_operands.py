"""Arithmetic the 64-row prompt matmuls rest on, checked exhaustively on the host: every unpacked operand must be an
integer fp16 holds exactly, or the products would not be those of the 16-row kernels (crates/compute/src/quant_gguf/
{q4_k,q5_k,q6_k,q8_0}.rs give the code ranges), and the column order the rotation kernel reads for a projection tiled
for the rotating epilogue must be the order the tiler wrote."""
import numpy as np


def _exact(v):
    return np.array_equal(np.asarray(v, np.float64), np.asarray(v, np.float64).astype(np.float16).astype(np.float64))


def test_q4_k_and_q5_k_operands_are_exact_fp16_integers():
    sc = np.arange(64)[:, None]                       # 6-bit sub-block scales
    assert _exact(sc * np.arange(16)[None, :])         # Q4_K codes
    assert _exact(sc * np.arange(32)[None, :])         # Q5_K codes (fifth bit OR-ed in before the fma)
    # the offset forms the fma starts from, and the offsets it takes back out
    assert _exact(1024 + np.arange(32)) and _exact(1024 * np.arange(64)) and _exact(64 * np.arange(64))
    # 64 + q in the 1/16-ulp form: the high nibble sits at bits 4..7 of a half whose ulp is 1/16, the fifth bit at bit 8
    for q in range(32):
        bits = np.uint16(0x5400 | ((q & 15) << 4) | ((q >> 4) << 8))
        assert float(bits.view(np.float16)) == 64 + q


def test_q6_k_scale_split_keeps_both_operands_exact():
    sc = np.arange(-128, 128)
    a, b = sc >> 4, sc & 15                            # arithmetic shift: a in -8..7, b in 0..15
    assert np.array_equal(16 * a + b, sc)
    level = np.arange(64) - 32
    assert _exact(level[:, None] * a[None, :]) and _exact(level[:, None] * b[None, :])
    assert not _exact(level[:, None] * sc[None, :])    # (why the scale cannot go in whole: 31 * 127 is not an fp16)
    # 1024 + level as (low nibble | 0x6400) | (high pair << 4), and one add of -1056 leaves level - 32
    for lv in range(64):
        bits = np.uint16(0x6400 | (lv & 15) | ((lv >> 4) << 4))
        assert float(bits.view(np.float16)) - 1056.0 == lv - 32


def test_q8_0_bytes_to_signed_codes():
    for q in range(-128, 128):
        byte = (q & 0xFF) ^ 0x80                        # the stored byte with its sign bit flipped: q + 128
        bits = np.uint16(0x6400 | byte)                 # byte permuted under 0x64
        assert float(bits.view(np.float16)) - 1152.0 == q


def test_paired_column_order_of_a_128_wide_head():
    """The tiler puts dim d of a head at t * 64 + half * 32 + j (half = d / 64, t = (d % 64) / 32, j = d % 32); the
    rotation kernel reads dims i and i + 64 at (i / 32) * 64 + i % 32 and 32 further on."""
    where = {}
    for d in range(128):
        half, w = d >> 6, d & 63
        where[d] = (w >> 5) * 64 + half * 32 + (w & 31)
    assert sorted(where.values()) == list(range(128))
    for i in range(64):
        c0 = (i >> 5) * 64 + (i & 31)
        assert where[i] == c0 and where[i + 64] == c0 + 32


def test_member_lists_by_ballot_order():
    """k_moe_groups: an expert's members are the pass's (row, slot) pairs that name it, in pair order; a lane's place is
    the members counted before it.  The same by sorting, on random selections without repeats inside a row."""
    rng = np.random.default_rng(0)
    rows, k, ne = 64, 8, 128
    sel = np.stack([rng.permutation(ne)[:k] for _ in range(rows)])
    for e in (0, 5, 77, 127):
        want = [(r, s) for r in range(rows) for s in range(k) if sel[r, s] == e]
        got, cnt = {}, 0
        flat = sel.reshape(-1)
        for p0 in range(0, rows * k, 64):              # sixty-four pairs at a time, as the wave walks them
            hit = flat[p0:p0 + 64] == e
            before = np.cumsum(hit) - hit
            for lane in np.nonzero(hit)[0]:
                got[cnt + int(before[lane])] = divmod(p0 + int(lane), k)
            cnt += int(hit.sum())
        assert [got[i] for i in range(cnt)] == want and cnt <= rows
