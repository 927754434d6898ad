"""GPU parity of the dequant-fused small-M matmul against the oracle's dequantize-then-dot.

Mirrors crates/gpu/tests/dequant_q4_k_gemv_parity.rs (bound scale*1e-2 + n*1e-4, :34-45) and
dequant_kquant_gemm_parity.rs (every width 1..16; a row's result must not depend on how many
rows ride with it)."""
import numpy as np
import pytest

from oracle import binding as ob
from tests.test_oracle_quant import lcg_weights

pytestmark = pytest.mark.gpu


def _case(dtype, rows, cols, seed):
    from turbospark_amd import ffi
    w = lcg_weights(rows * cols, seed).reshape(rows, cols) * 0.05
    entry = ffi.quantize(dtype, w)
    x = lcg_weights(16 * cols, seed + 1).reshape(16, cols)
    x16 = x.astype(np.float16).astype(np.float32)  # the kernel's operand precision
    want = np.stack([ob.gemv(dtype, entry[1], rows, cols, x16[b]) for b in range(16)])
    return entry, x, x16, want


@pytest.mark.parametrize("dtype,rows,cols", [(12, 64, 512), (12, 48, 2048), (8, 64, 512), (8, 32, 1408),
                                             (39, 64, 512), (39, 48, 2048), (39, 200, 768),
                                             (39, 64, 576), (39, 96, 2880),      # MXFP4 rows ending inside a 256-chunk
                                             (30, 64, 512), (30, 40, 576), (30, 130, 2880),   # bf16
                                             (14, 64, 512), (14, 48, 2048), (14, 200, 768),    # Q6_K
                                             (13, 64, 512), (13, 48, 2048), (13, 200, 768)])   # Q5_K
def test_matmul_matches_dequantize_then_dot_for_every_width(dtype, rows, cols):
    from turbospark_amd import ffi
    entry, x, x16, want = _case(dtype, rows, cols, 31)
    scale = np.abs(want).max()
    bound = scale * 1e-2 + cols * 1e-4
    first = None
    for m in range(1, 17):
        got = ffi.matmul(entry, x[:m])
        assert got.shape == (m, rows)
        err = np.abs(got - want[:m]).max()
        assert err <= bound, (m, err, bound)
        # much tighter than the reference's bound: fp32 accumulation of exact products
        assert err <= scale * 2e-4 + 1e-5, (m, err)
        # row invariance: row 0 is bit-identical whatever rides with it -- within one MFMA form: Q4_K passes
        # of nine to sixteen rows run on the 16x16x32 instruction, which sums a sub-block in another order
        if first is None or (dtype == 12 and m == 9):
            first = got[0].copy()
        assert np.array_equal(got[0], first), m


@pytest.mark.parametrize("dtype", [12, 8, 39, 30, 14, 13])
def test_split_k_changes_nothing_but_rounding_and_is_deterministic(dtype):
    from turbospark_amd import ffi
    entry, x, x16, want = _case(dtype, 32, 2048, 77)
    a = ffi.matmul(entry, x[:5], splits=1)
    b = ffi.matmul(entry, x[:5], splits=4)
    c = ffi.matmul(entry, x[:5], splits=4)
    assert np.array_equal(b, c)
    assert np.abs(a - b).max() <= np.abs(want).max() * 1e-5 + 1e-6
    assert np.abs(a - want[:5]).max() <= np.abs(want).max() * 2e-4 + 1e-5


def test_q4k_hand_packed_superblock_through_the_kernel(golden):
    """The reference's literal superblock (quant_gguf.rs:226-267) as a 16-row weight matrix:
    one-hot activations read the decoded weights back out of the kernel."""
    import json, os
    from turbospark_amd import ffi
    g = json.load(open(os.path.join(golden, "q4k_handpacked.json")))
    quants = [(e * 7 + 3) % 16 for e in range(256)]
    body = bytearray(g["D_BITS"] + g["DMIN_BITS"] + g["PACKED"])
    for grp in range(4):
        for l in range(32):
            at = grp * 64 + l
            body.append(quants[at] | (quants[at + 32] << 4))
    blk = np.frombuffer(bytes(body), np.uint8)
    raw = np.tile(blk, (16, 1))
    entry = (ffi.Q4_K, np.ascontiguousarray(raw), 16, 256)
    want = np.array([g["d"] * g["LS"][e // 32] * quants[e] - g["dmin"] * g["LM"][e // 32] for e in range(256)],
                    np.float32)
    for e0 in range(0, 256, 16):
        x = np.zeros((16, 256), np.float32)
        for b in range(16):
            x[b, e0 + b] = 1.0
        got = ffi.matmul(entry, x)
        for b in range(16):
            assert np.all(got[b] == want[e0 + b]), (e0 + b, got[b, 0], want[e0 + b])


def test_mxfp4_ggml_golden_blocks_through_the_kernel(golden):
    """The ggml-produced MXFP4 bytes -> floats fixture of the reference
    (crates/compute/tests/generated/quant_gguf_mxfp4_oracle.rs) as a weight matrix: one-hot
    activations read the decoded weights back out of the kernel, which must equal ggml's floats
    exactly (every value is a codebook entry times a power of two)."""
    import json, os
    from turbospark_amd import ffi
    g = json.load(open(os.path.join(golden, "mxfp4_ggml_oracle.json")))
    blocks = np.array(g["bytes"], np.uint8).reshape(4, 17)
    pad = np.zeros((4, 17), np.uint8)
    pad[:, 0] = 127                                   # scale 2^-1, all codes zero
    row = np.concatenate([blocks, pad]).reshape(1, -1)  # 8 blocks = one 256-element chunk
    raw = np.tile(row, (16, 1))
    entry = (ffi.MXFP4, np.ascontiguousarray(raw), 16, 256)
    want = np.concatenate([np.array(g["floats"], np.float32), np.zeros(128, np.float32)])
    for e0 in range(0, 128, 16):
        x = np.zeros((16, 256), np.float32)
        for b in range(16):
            x[b, e0 + b] = 1.0
        got = ffi.matmul(entry, x)
        for b in range(16):
            assert np.all(got[b] == want[e0 + b]), (e0 + b, got[b, 0], want[e0 + b])


def test_q6k_hand_packed_superblock_through_the_kernel(golden):
    """The reference's literal Q6_K superblock (crates/compute/tests/quant_gguf.rs:413-445) as every row
    of a weight matrix: one-hot activations read the decoded weights back out of the kernel, `==`."""
    import json
    import os
    from turbospark_amd import ffi
    g = json.load(open(os.path.join(golden, "q6k_handpacked.json")))
    block = bytes([g["ql_byte"]] * 128 + [g["qh_byte"]] * 64 + [s & 0xFF for s in g["scales"]]) + \
        int(g["d_bits"]).to_bytes(2, "little")
    rows = 16
    data = np.frombuffer(block * rows, np.uint8).reshape(rows, 210).copy()
    entry = (ffi.Q6_K, data, rows, 256)
    for k0 in range(0, 256, 16):
        x = np.zeros((16, 256), np.float32)
        x[np.arange(16), k0 + np.arange(16)] = 1.0
        got = ffi.matmul(entry, x)
        for b in range(16):
            e = k0 + b
            h, k, l = e // 128, (e % 128) // 32, e % 32
            want = np.float32(g["d"]) * np.float32(g["scales"][h * 8 + l // 16 + 2 * k]) * np.float32(g["quants"][k])
            assert np.all(got[b] == want), (e, got[b][0], want)


@pytest.mark.parametrize("seed", range(40))
def test_random_matmul_shapes(seed):
    """Seeded sweep over format, row count (padded last tiles), K (one chunk to dozens, MXFP4 / bf16 rows
    that end inside a chunk), batch width and split-K count."""
    from turbospark_amd import ffi
    r = np.random.default_rng(6000 + seed)
    dtype = int(r.choice([12, 8, 39, 30, 14, 13]))
    unit = {12: 256, 13: 256, 14: 256, 8: 128, 39: 32, 30: 64}[dtype]
    cols = unit * int(r.integers(1, {12: 24, 13: 24, 14: 24, 8: 48, 39: 120, 30: 60}[dtype]))
    rows = int(r.integers(1, 400))
    m = int(r.integers(1, 17))
    kchunks = -(-cols // {12: 256, 13: 256, 14: 256, 8: 128, 39: 256, 30: 64}[dtype])
    splits = int(r.integers(0, min(8, kchunks) + 1))
    w = (r.standard_normal((rows, cols)) * 0.05).astype(np.float32)
    entry = ffi.quantize(dtype, w)
    x = r.standard_normal((m, cols)).astype(np.float32)
    x16 = x.astype(np.float16).astype(np.float32)
    want = np.stack([ob.gemv(dtype, entry[1], rows, cols, x16[b]) for b in range(m)])
    print(f"seed {seed}: dtype {dtype} {rows} x {cols}, m={m}, splits={splits}", flush=True)
    try:
        got = ffi.matmul(entry, x, splits=splits)
    except Exception as e:  # a split count that leaves an empty K slice is refused by name
        assert "empty K slice" in str(e), e
        got = ffi.matmul(entry, x)
    scale = np.abs(want).max()
    assert np.abs(got - want).max() <= scale * 2e-4 + 1e-5


def test_q5k_ggml_golden_superblocks_through_the_kernel(golden):
    """The two Q5_K superblocks ggml quantized (crates/compute/tests/generated/quant_gguf_q5_k_oracle.rs), as
    a one-row matrix, multiplied by unit vectors through the kernel: every weight reads back as the
    float ggml decoded (fp16 unit activations select one weight each; products are exact in fp32)."""
    import json
    import os
    from turbospark_amd import ffi
    g = json.load(open(os.path.join(golden, "q5k_ggml_oracle.json")))
    raw = np.array(g["bytes"], np.uint8).reshape(1, -1)
    want = np.array(g["floats"], np.float32)
    entry = (13, raw, 1, 512)
    for k0 in range(0, 512, 16):
        x = np.zeros((16, 512), np.float32)
        x[np.arange(16), k0 + np.arange(16)] = 1.0
        got = ffi.matmul(entry, x)[:, 0]
        assert np.allclose(got, want[k0:k0 + 16], rtol=0, atol=2e-6), (k0, got, want[k0:k0 + 16])
