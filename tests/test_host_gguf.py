"""The GGUF header parser behind the C ABI (crates/repack/src/gguf_header/parser.rs:124-239) on
files a test writer lays out as the public format says: what it reads back, and what it refuses
by name.  No GPU is touched."""
import os

import numpy as np
import pytest

from tests.gguf_writer import permute_rotary_rows, write_gguf
from turbospark_amd import ffi


def _tensors():
    rng = np.random.default_rng(0)
    w = (rng.standard_normal((8, 256)) * 0.02).astype(np.float32)
    q4 = ffi.quantize(ffi.Q4_K, w)
    q8 = ffi.quantize(ffi.Q8_0, w)
    norm = np.arange(256, dtype=np.float32)
    experts = ffi.quantize(ffi.MXFP4, (rng.standard_normal((3 * 4, 64))).astype(np.float32))
    return [("a.weight", [256, 8], ffi.Q4_K, q4[1].tobytes()), ("b.weight", [256, 8], ffi.Q8_0, q8[1].tobytes()),
            ("n.weight", [256], ffi.F32, norm.tobytes()), ("e_exps.weight", [64, 4, 3], ffi.MXFP4, experts[1].tobytes())], q4, q8, norm, experts


META = [("general.architecture", "str", "llama"), ("llama.block_count", "u32", 2), ("llama.rope.freq_base", "f32", 500000.0),
        ("x.i64", "i64", -5), ("x.f64", "f64", 2.5), ("x.bool", "bool", 1), ("x.u8", "u8", 200),
        ("tokenizer.ggml.tokens", "arr", ("str", ["a", "bc", ""])), ("nested", "arr", ("arr", [("u16", [1, 2]), ("u16", [])]))]


def test_a_written_file_reads_back(tmp_path):
    tensors, q4, q8, norm, experts = _tensors()
    for alignment in (None, 64, 4096):
        path = os.path.join(tmp_path, f"m{alignment}.gguf")
        start = write_gguf(path, META, tensors, alignment=alignment)
        g = ffi.Gguf(path)
        assert g.tensor_count == 4 and g.data_start == start and start % (alignment or 32) == 0
        assert g.string("general.architecture") == "llama"
        assert g.number("llama.block_count") == 2 and g.number("llama.rope.freq_base") == 500000.0
        assert g.number("x.i64") == -5 and g.number("x.f64") == 2.5 and g.number("x.bool") == 1 and g.number("x.u8") == 200
        dt, raw, rows, cols = g.tensor("a.weight")
        assert (dt, rows, cols) == (ffi.Q4_K, 8, 256) and np.array_equal(raw, q4[1])
        dt, raw, rows, cols = g.tensor("b.weight")
        assert (dt, rows, cols) == (ffi.Q8_0, 8, 256) and np.array_equal(raw, q8[1])
        dt, raw, rows, cols = g.tensor("n.weight")
        assert (dt, rows, cols) == (ffi.F32, 1, 256) and np.array_equal(raw.view(np.float32)[0], norm)
        # stacked experts: every dimension past the first folds into expert-major rows
        dt, raw, rows, cols = g.tensor("e_exps.weight")
        assert (dt, rows, cols) == (ffi.MXFP4, 12, 64) and np.array_equal(raw, experts[1])
        with pytest.raises(ffi.TsvError, match="no tensor"):
            g.tensor("missing.weight")
        with pytest.raises(ffi.TsvError, match="no numeric metadata"):
            g.number("general.architecture")
        g.close()


def _refused(tmp_path, match, **kw):
    tensors = kw.pop("tensors", None) or _tensors()[0]
    meta = kw.pop("meta", META)
    cut = kw.pop("cut", None)
    path = os.path.join(tmp_path, "bad.gguf")
    write_gguf(path, meta, tensors, **kw)
    if cut is not None:
        data = open(path, "rb").read()
        open(path, "wb").write(data[:cut] if cut > 0 else data[:len(data) + cut])
    with pytest.raises(ffi.TsvError, match=match):
        ffi.Gguf(path).close()


def test_the_parsers_refusals(tmp_path):
    _refused(tmp_path, "bad magic", magic=b"GGML")
    _refused(tmp_path, "version 2", version=2)
    _refused(tmp_path, "too short", cut=250)                       # the header itself is cut
    _refused(tmp_path, "shorter than a GGUF header", cut=10)
    _refused(tmp_path, "duplicate metadata key", meta=META + [("x.u8", "u8", 1)])
    t = _tensors()[0]
    _refused(tmp_path, "duplicate tensor", tensors=t + [t[0]])
    _refused(tmp_path, "a zero dimension", tensors=[("z", [256, 0], ffi.F32, b"")])
    _refused(tmp_path, "5 dimensions", tensors=[("z", [2, 2, 2, 2, 2], ffi.F32, b"\0" * 128)])
    _refused(tmp_path, "not a multiple of the file's alignment", misalign="b.weight")
    _refused(tmp_path, "not a power of two", alignment=48)
    with pytest.raises(ffi.TsvError, match="cannot read"):
        ffi.Gguf(os.path.join(tmp_path, "absent.gguf"))


def test_a_bad_value_type_and_deep_nesting_are_refused(tmp_path):
    import struct
    from tests import gguf_writer as gw
    # a value type id the format does not define
    gw.TYPE_IDS["bogus"], gw.PACK["bogus"] = 13, "<B"
    try:
        _refused(tmp_path, "is not a GGUF type", meta=[("k", "bogus", 1)])
    finally:
        del gw.TYPE_IDS["bogus"], gw.PACK["bogus"]
    # arrays nested deeper than the parser walks: 70 array headers of one element each
    body = b"".join(struct.pack("<IQ", 9, 1) for _ in range(70)) + struct.pack("<IQ", 0, 0)
    head = b"GGUF" + struct.pack("<IQQ", 3, 0, 1) + struct.pack("<Q", 1) + b"k" + struct.pack("<I", 9) + body
    path = os.path.join(tmp_path, "deep.gguf")
    open(path, "wb").write(head + b"\0" * 64)
    with pytest.raises(ffi.TsvError, match="nested deeper"):
        ffi.Gguf(path)
    # counts no file of this size could hold
    open(path, "wb").write(b"GGUF" + struct.pack("<IQQ", 3, 1 << 40, 0) + b"\0" * 64)
    with pytest.raises(ffi.TsvError, match="counts larger"):
        ffi.Gguf(path)


def test_tensor_views_are_checked_against_the_file(tmp_path):
    tensors = _tensors()[0]
    path = os.path.join(tmp_path, "cut.gguf")
    write_gguf(path, META, tensors)
    data = open(path, "rb").read()
    open(path, "wb").write(data[:-40])                             # the last tensor's tail is gone
    g = ffi.Gguf(path)
    assert g.tensor("a.weight")[2] == 8
    with pytest.raises(ffi.TsvError, match="runs past the end"):
        g.tensor("e_exps.weight")
    g.close()
    # a block type without a kernel here (Q4_0) and a row length that is not whole blocks
    write_gguf(path, META, [("q40.weight", [256, 2], 2, b"\0" * 288), ("odd.weight", [100, 2], ffi.Q4_K, b"\0" * 288)])
    g = ffi.Gguf(path)
    for name in ("q40.weight", "odd.weight"):
        with pytest.raises(ffi.TsvError, match="no kernel here"):
            g.tensor(name)
    g.close()


def test_dimensions_that_would_wrap_the_byte_count_are_refused(tmp_path):
    """A hostile tensor table: bf16 with a first dimension of 2^61 and four rows makes rows * row_bytes
    wrap to zero in 64 bits, which would pass an end-of-file check done after the multiplication."""
    path = os.path.join(tmp_path, "wrap.gguf")
    write_gguf(path, META, [("wrap.weight", [1 << 61, 4], ffi.BF16, b"\0" * 64),
                            ("tall.weight", [64, 1 << 39], ffi.BF16, b"\0" * 64),
                            ("ok.weight", [64, 2], ffi.BF16, b"\1" * 256)])
    g = ffi.Gguf(path)
    with pytest.raises(ffi.TsvError, match="first dimension outside"):
        g.tensor("wrap.weight")
    with pytest.raises(ffi.TsvError, match="runs past the end"):
        g.tensor("tall.weight")
    dt, raw, rows, cols = g.tensor("ok.weight")
    assert (dt, rows, cols) == (ffi.BF16, 2, 64)
    g.close()


def test_the_writers_permutation_is_the_converters():
    # conventions.rs:133-143: GGUF row j of a head holds the original row (j % 2) * (D/2) + j // 2,
    # so the original row i is found at GGUF row (i % (D/2)) * 2 + i // (D/2)
    D = 8
    rows = np.arange(2 * D).reshape(2 * D, 1)
    perm = permute_rotary_rows(rows, D)[:, 0]
    assert perm[:D].tolist() == [0, 4, 1, 5, 2, 6, 3, 7] and perm[D:].tolist() == [8, 12, 9, 13, 10, 14, 11, 15]
    for i in range(D):
        assert perm[(i % (D // 2)) * 2 + i // (D // 2)] == i


def _nested(depth):
    """`depth` array headers of one element each around a u32 7 (crates/repack/tests/gguf_header.rs:191-216)."""
    import struct
    body = b"".join(struct.pack("<IQ", 9, 1) for _ in range(depth - 1)) + struct.pack("<IQ", 4, 1) + struct.pack("<I", 7)
    return b"GGUF" + struct.pack("<IQQ", 3, 0, 1) + struct.pack("<Q", 6) + b"nested" + struct.pack("<I", 9) + body + b"\0" * 64


def test_the_array_nesting_limit_is_exact(tmp_path):
    # crates/repack/tests/gguf_header.rs:259-285: 64 levels parse, 65 are refused
    path = os.path.join(tmp_path, "n.gguf")
    open(path, "wb").write(_nested(64))
    g = ffi.Gguf(path)
    assert g.tensor_count == 0
    g.close()
    open(path, "wb").write(_nested(65))
    with pytest.raises(ffi.TsvError, match="nested deeper than 64"):
        ffi.Gguf(path)


def test_the_references_own_fixture_scenario(tmp_path):
    # crates/repack/tests/gguf_header.rs:18-110: mixed metadata kinds, a 3-D stacked tensor, the
    # default alignment, and tensor ranges that are the writer's own
    rng = np.random.default_rng(1)
    gate = rng.integers(0, 256, 512 // 32 * 34, dtype=np.uint8).tobytes()
    q = rng.integers(0, 256, 64 * 32 // 32 * 34, dtype=np.uint8).tobytes()
    meta = [("general.architecture", "str", "gemma4"), ("gemma4.block_count", "u32", 2),
            ("gemma4.attention.layer_norm_rms_epsilon", "f32", 1e-6), ("general.file_type", "u8", 7),
            ("truncated", "bool", 1), ("signed", "i32", -3), ("wide", "u64", 1 << 40),
            ("tokenizer.ggml.tokens", "arr", ("str", ["<pad>", "hi"])), ("nested", "arr", ("arr", [("u32", [1, 2])]))]
    path = os.path.join(tmp_path, "f.gguf")
    start = write_gguf(path, meta, [("blk.0.ffn_gate_exps.weight", [64, 2, 4], 8, gate),
                                    ("blk.0.attn_q.weight", [64, 32], 8, q), ("output_norm.weight", [8], 0, b"\0" * 32)])
    g = ffi.Gguf(path)
    assert g.string("general.architecture") == "gemma4" and g.number("gemma4.block_count") == 2
    assert g.number("wide") == float(1 << 40) and g.number("signed") == -3 and g.number("truncated") == 1
    assert g.number("gemma4.attention.layer_norm_rms_epsilon") == float(np.float32(1e-6))
    assert g.data_start == start and start % 32 == 0 and g.tensor_count == 3
    dt, raw, rows, cols = g.tensor("blk.0.ffn_gate_exps.weight")
    assert (dt, rows, cols) == (8, 8, 64) and raw.size == 512 // 32 * 34 and raw.tobytes() == gate
    dt, raw, rows, cols = g.tensor("blk.0.attn_q.weight")
    assert (dt, rows, cols) == (8, 32, 64) and raw.tobytes() == q
    # block sizes of the types this library has kernels for, as the format's table gives them
    # (crates/repack/tests/gguf_header.rs:548-560): (elements, bytes) per block
    for tid, (elems, nbytes) in {0: (1, 4), 1: (1, 2), 8: (32, 34), 12: (256, 144), 13: (256, 176), 14: (256, 210),
                                 30: (1, 2), 39: (32, 17)}.items():
        assert ffi.row_bytes(tid, 256) == 256 // elems * nbytes, tid
    g.close()


def test_the_independent_reader_recovers_what_the_writer_was_given(tmp_path):
    """tests/gguf_reader.py (the oracle side of the GGUF parity tests) against tests/gguf_writer.py: every
    tensor of a llama file (q / k rows permuted by the converter and un-permuted by the reader,
    conventions.rs:133-151), a routed qwen3moe file and a gpt-oss file comes back byte for byte under the
    names of gguf_names/llama.rs:14-60 and gpt_oss.rs:30-72, with the sizes read from the metadata."""
    from tests import gguf_reader
    from tests.gguf_writer import llama_gguf
    from turbospark_amd import synth
    for name, arch, permute in [("tiny_q8_0", "llama", True), ("moe_small", "qwen3moe", False), ("gptoss_small", "gpt-oss", False)]:
        cfg = dict(synth.CONFIGS[name], max_context=96)
        w = synth.make_weights(cfg, seed=4321)
        path = os.path.join(tmp_path, name + ".gguf")
        llama_gguf(path, cfg, w, arch=arch, permute=permute)
        ocfg, ow = gguf_reader.load_model(path, 96)
        for key in ("n_layers", "hidden", "n_q_heads", "n_kv_heads", "head_dim", "ffn", "vocab"):
            assert ocfg[key] == cfg[key], (name, key)
        for a, b in zip(w["layers"], ow["layers"]):
            for k, v in a.items():
                if isinstance(v, tuple):
                    assert v[0] == b[k][0] and v[2:] == b[k][2:], (name, k)
                    assert np.array_equal(np.asarray(v[1]).reshape(-1), np.asarray(b[k][1]).reshape(-1)), (name, k)
                elif k in ("n_experts", "top_k", "window"):
                    assert b.get(k, 0) == v, (name, k)
        for k in ("embed", "final_norm", "lm_head"):
            assert np.array_equal(np.asarray(w[k][1]).reshape(-1), np.asarray(ow[k][1]).reshape(-1)), (name, k)
        if arch == "gpt-oss":
            assert np.allclose(ocfg["rope_freqs"], cfg["rope_freqs"]) and abs(ocfg["rope_mscale"] - cfg["rope_mscale"]) < 1e-7


def test_mutated_headers_are_refused_or_read_within_the_file(tmp_path):
    """Seeded damage to a valid file's header -- flipped bytes, huge little-endian integers dropped onto 8-byte
    fields, truncation -- must end in a refusal by name or in reads that stay inside the file: the process surviving
    the loop is the assertion (a parser that trusts a count or an offset dies here)."""
    tensors = _tensors()[0]
    path = os.path.join(tmp_path, "base.gguf")
    start = write_gguf(path, META, tensors)
    good = open(path, "rb").read()
    names = [t[0] for t in tensors]
    rng = np.random.default_rng(11)
    big = [2 ** 64 - 1, 2 ** 63, 2 ** 63 - 1, 2 ** 61, 2 ** 40, 2 ** 32, 2 ** 31, len(good), len(good) + 1, 0]
    refused = opened = 0
    for case in range(600):
        data = bytearray(good)
        kind = case % 3
        if kind == 0:      # a few flipped bytes in the header
            for _ in range(int(rng.integers(1, 5))):
                data[int(rng.integers(4, start))] = int(rng.integers(0, 256))
        elif kind == 1:    # a huge or boundary integer over an 8-byte field
            at = int(rng.integers(8, start - 8))
            data[at:at + 8] = int(big[int(rng.integers(0, len(big)))]).to_bytes(8, "little")
        else:              # truncation anywhere, header or data
            data = data[:int(rng.integers(0, len(good)))]
        p = os.path.join(tmp_path, "m.gguf")
        open(p, "wb").write(bytes(data))
        try:
            g = ffi.Gguf(p)
        except ffi.TsvError:
            refused += 1
            continue
        opened += 1
        assert 0 <= g.tensor_count <= 4096
        for name in names:
            try:
                dt, raw, rows, cols = g.tensor(name)
                assert raw.nbytes <= len(data)
            except ffi.TsvError:
                pass
        for key in ("llama.block_count", "x.i64", "general.architecture"):
            try:
                g.number(key)
            except ffi.TsvError:
                pass
            try:
                g.string(key)
            except ffi.TsvError:
                pass
        g.close()
    print(f"600 damaged files: {refused} refused at open, {opened} opened and read within bounds")
    assert refused > 100 and opened > 20
