"""The C-ABI library loads and exports every symbol include/*.h declares (no GPU needed),
and the host-side install helpers agree with the oracle bit for bit."""
import os
import re

import numpy as np

from oracle import binding as ob

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    """Every entry point the two headers declare: the drop-in surface and the test / measurement hooks."""
    names = set()
    for header in ("tsverify.h", "tsverify_testing.h"):
        text = open(os.path.join(ROOT, "include", header)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names |= set(re.findall(r"\b(tsv_[a-z_0-9]+)\s*\(", text))
    return sorted(names)


def test_the_hooks_live_in_their_own_header():
    surface = open(os.path.join(ROOT, "include", "tsverify.h")).read()
    for hook in ("tsv_matmul_time", "tsv_copy_time", "tsv_set_repeat", "tsv_write_logits", "tsv_write_kv", "tsv_read_kv",
                 "tsv_set_profile", "tsv_route_selected"):
        assert hook + "(" not in surface, hook


def test_every_declared_entry_point_is_exported():
    from turbospark_amd import ffi
    lib = ffi.lib()
    names = _declared()
    assert len(names) >= 25
    for n in names:
        assert hasattr(lib, n), n
    assert sorted(ffi.EXPORTS) == names


def test_struct_layouts_match_the_header_sizes():
    import ctypes as C
    from turbospark_amd import ffi
    assert C.sizeof(ffi.Tensor) == 32
    assert C.sizeof(ffi.Layer) == 11 * 32 + 8 + 4 * 32 + 9 * 32 + 8
    assert C.sizeof(ffi.Shaping) == 80
    assert C.sizeof(ffi.RoundResultC) == 4 * 4 + 8 + 17 * 4 + 4 + 8 + 8


def test_install_encoders_are_bit_identical_to_the_oracle():
    from turbospark_amd import ffi
    rng = np.random.default_rng(3)
    w = (rng.standard_normal((24, 1024)) * 0.02).astype(np.float32)
    w[3] = 0.0                      # an all-zero row: zero scales, no division
    w[5, :32] = 1e-9                # a nearly flat sub-block
    for dt in (ffi.Q4_K, ffi.Q6_K, ffi.Q8_0, ffi.MXFP4, ffi.F16, ffi.BF16, ffi.F32):
        assert np.array_equal(ffi.quantize(dt, w)[1], ob.quantize(dt, w)), dt
    assert ffi.row_bytes(ffi.Q4_K, 4096) == 2304 and ffi.row_bytes(ffi.Q8_0, 4096) == 4352
    assert ffi.row_bytes(ffi.Q4_K, 100) < 0


def test_synthetic_tensor_is_seeded_normal_and_stream_separated():
    from turbospark_amd import ffi
    a = ffi.synth_tensor(ffi.F32, 7, 1, 0.02, 64, 512)[1].view(np.float32)
    b = ffi.synth_tensor(ffi.F32, 7, 1, 0.02, 64, 512)[1].view(np.float32)
    c = ffi.synth_tensor(ffi.F32, 7, 2, 0.02, 64, 512)[1].view(np.float32)
    assert np.array_equal(a, b) and not np.array_equal(a, c)
    assert abs(a.std() - 0.02) < 5e-4 and abs(a.mean()) < 5e-4
    assert abs(np.corrcoef(a.reshape(-1), c.reshape(-1))[0, 1]) < 0.02
    # row r of a taller tensor is the same row (counter-based: no dependence on generation order)
    tall = ffi.synth_tensor(ffi.F32, 7, 1, 0.02, 128, 512)[1].view(np.float32)
    assert np.array_equal(tall[:64], a)
    q = ffi.synth_tensor(ffi.Q4_K, 7, 1, 0.02, 64, 512)
    assert np.array_equal(q[1], ob.quantize(ob.Q4_K, a.reshape(64, 512)))


def test_shaping_validation_mirrors_the_reference():
    import pytest
    from turbospark_amd import ffi
    for bad in (dict(temperature=-1.0), dict(temperature=float("nan")), dict(top_k=257),
                dict(top_p=0.0), dict(top_p=1.5), dict(repetition_penalty=0.0)):
        with pytest.raises(ValueError):
            ffi.shaping(**bad)
    s = ffi.shaping(0.7, top_k=0, top_p=0.95, seed=9)  # ordinary top-p sampling is accepted
    assert s.has_top_p and s.has_seed and s.seed == 9


def test_product_sources_never_touch_the_oracle():
    pkg = os.path.join(ROOT, "turbospark_amd")
    for base, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cpp")):
                text = open(os.path.join(base, f), errors="replace").read()
                assert "tsoracle" not in text and "from oracle" not in text and "import oracle" not in text, f


def test_null_handles_are_refused_by_name_without_a_gpu():
    """Every entry point that takes a handle answers a null one with an error (or -1 / null for the plain
    getters) before any device call is made; a descriptor with a zero head count is refused by tsv_open."""
    import ctypes as C
    from turbospark_amd import ffi
    L = ffi.lib()
    assert L.tsv_kv_position(None) == -1 and L.tsv_max_context(None) == -1 and L.tsv_vocab(None) == -1
    assert L.tsv_stream(None) is None and L.tsv_device_logits(None) is None
    L.tsv_close(None)
    point = ffi.Point()
    tok = (C.c_int32 * 4)(1, 2, 3, 4)
    out = (C.c_uint16 * 8)()
    calls = [
        lambda: L.tsv_reset(None),
        lambda: L.tsv_set_profile(None, 1),
        lambda: L.tsv_set_repeat(None, 0, 1),
        lambda: L.tsv_get_profile(None, None, None, 0),
        lambda: L.tsv_checkpoint(None, C.byref(point)),
        lambda: L.tsv_rollback(None, C.byref(point)),
        lambda: L.tsv_rollback_retaining(None, C.byref(point), 0),
        lambda: L.tsv_verify(None, tok, 4, 0, out),
        lambda: L.tsv_verify_tree(None, tok, tok, 4, 0, out),
        lambda: L.tsv_produce(None, 1, 0, out),
        lambda: L.tsv_prefill(None, tok, 4, 0, out),
        lambda: L.tsv_compact_tree(None, 0, tok, 1),
        lambda: L.tsv_accept(None, None, None),
        lambda: L.tsv_verify_accept(None, None, None),
        lambda: L.tsv_read_kv(None, 0, 0, 1, out, out),
        lambda: L.tsv_write_kv(None, 0, 0, 1, out, out),
        lambda: L.tsv_write_logits(None, out, 1, 0),
        lambda: L.tsv_set_prefix_reuse(None, 1),
        lambda: L.tsv_record_committed(None, tok, 4, 0),
        lambda: L.tsv_try_reuse_prefix(None, tok, 4),          # -1
        lambda: L.tsv_gguf_open(None, None),
        lambda: L.tsv_gguf_tensor(None, b"x", None),
        lambda: L.tsv_gguf_meta_number(None, b"x", None),
        lambda: L.tsv_gguf_meta_string(None, b"x", None, 0),
        lambda: L.tsv_open_gguf(None, 0, C.byref(C.c_void_p())),
        lambda: L.tsv_mtp_open(None, None, C.byref(C.c_void_p())),
        lambda: L.tsv_mtp_step(None, 1, 0, None, 0),
        lambda: L.tsv_mtp_rewind(None, 0),
        lambda: L.tsv_mtp_prefill_chunk(None, tok, 4, 0, out, -1),
        lambda: L.tsv_mtp_draft_block(None, 1, 1, 2, tok),
        lambda: L.tsv_mtp_drafter(None, None),
    ]
    for i, call in enumerate(calls):
        assert call() != 0, i
        assert ffi.last_error(), i
    assert L.tsv_prefix_len(None) == -1 and L.tsv_gguf_tensor_count(None) == -1 and L.tsv_gguf_data_start(None) == -1
    # the record on its own tolerates null and empty arguments
    L.tsv_prefix_free(None)
    L.tsv_prefix_clear(None)
    L.tsv_prefix_record(None, tok, 4, 0)
    assert L.tsv_prefix_common(None, tok, 4) == 0 and L.tsv_prefix_untainted_len(None) == -1
    rec = ffi.KvPrefix([1, 2, 3])
    L.tsv_prefix_record(rec._p, None, 0, 3)                    # nothing fed at the end: no change
    assert rec.untainted_len() == 3 and L.tsv_prefix_common(rec._p, None, 0) == 0
    desc = ffi.ModelDesc()
    layers = (ffi.Layer * 1)()
    desc.layers = C.cast(layers, type(desc.layers))
    desc.n_layers, desc.hidden, desc.n_q_heads, desc.n_kv_heads, desc.head_dim = 1, 64, 4, 0, 64
    desc.ffn, desc.vocab, desc.max_context = 64, 100, 16
    handle = C.c_void_p()
    assert L.tsv_open(C.byref(desc), C.byref(handle)) != 0 and "positive" in ffi.last_error()


def test_measurement_hooks_answer_only_under_their_switch(monkeypatch):
    """The timing loops refuse by name in a process without TSV_MEASUREMENT_HOOKS=1 -- before any device call,
    so this runs without a GPU."""
    import ctypes as C
    from turbospark_amd import ffi
    L = ffi.lib()
    monkeypatch.delenv("TSV_MEASUREMENT_HOOKS", raising=False)
    t = C.c_float()
    for call in (lambda: L.tsv_copy_time(1 << 20, 1, C.byref(t)),
                 lambda: L.tsv_matmul_time(ffi.Q4_K, 64, 256, 4, 0, 0, 1, 1, C.byref(t))):
        assert call() == -3 and "TSV_MEASUREMENT_HOOKS=1" in ffi.last_error()
