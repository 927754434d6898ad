"""ctypes binding of include/tsverify.h and include/tsverify_testing.h."""
import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, os.environ.get("TSV_LIB_NAME", "libtsverify.so"))

F32, F16, Q8_0, Q4_K, Q5_K, Q6_K, BF16, MXFP4 = 0, 1, 8, 12, 13, 14, 30, 39
MAX_ROWS = 16


class TsvError(RuntimeError):
    def __init__(self, code, text):
        super().__init__(f"tsverify error {code}: {text}")
        self.code = code
        self.text = text


class Tensor(C.Structure):
    _fields_ = [("data", C.c_void_p), ("dtype", C.c_int32), ("rows", C.c_int64), ("cols", C.c_int64)]


LAYER_TENSORS = ("attn_norm", "wq", "wk", "wv", "wo", "q_norm", "k_norm", "ffn_norm", "w_gate", "w_up", "w_down")
LAYER_MOE_TENSORS = ("router", "we_gate", "we_up", "we_down")
LAYER_GPTOSS_TENSORS = ("bq", "bk", "bv", "bo", "sinks", "router_bias", "be_gate", "be_up", "be_down")


class Layer(C.Structure):
    _fields_ = ([(n, Tensor) for n in LAYER_TENSORS] + [("n_experts", C.c_int32), ("top_k", C.c_int32)] +
                [(n, Tensor) for n in LAYER_MOE_TENSORS] + [(n, Tensor) for n in LAYER_GPTOSS_TENSORS] +
                [("window", C.c_int32), ("ring", C.c_int32)])


class ModelDesc(C.Structure):
    _fields_ = [
        ("n_layers", C.c_int32), ("hidden", C.c_int32), ("n_q_heads", C.c_int32),
        ("n_kv_heads", C.c_int32), ("head_dim", C.c_int32), ("ffn", C.c_int32),
        ("vocab", C.c_int32), ("max_context", C.c_int32),
        ("rms_eps", C.c_float), ("rope_theta", C.c_float), ("attn_scale", C.c_float),
        ("rope_factors", C.POINTER(C.c_float)),
        ("embed", Tensor), ("final_norm", Tensor), ("lm_head", Tensor),
        ("layers", C.POINTER(Layer)),
        ("rope_freqs", C.POINTER(C.c_float)), ("rope_mscale", C.c_float),
        ("act_alpha", C.c_float), ("act_limit", C.c_float),
        ("kv_k_bits", C.c_int32), ("kv_v_bits", C.c_int32), ("session_slots", C.c_int32),
    ]


class Shaping(C.Structure):
    _fields_ = [
        ("temperature", C.c_double), ("top_k", C.c_uint32), ("has_top_p", C.c_int32),
        ("top_p", C.c_double), ("repetition_penalty", C.c_double), ("has_seed", C.c_int32),
        ("seed", C.c_uint64), ("presence_penalty", C.c_double), ("frequency_penalty", C.c_double),
        ("has_min_p", C.c_int32), ("min_p", C.c_double),
    ]


def shaping(temperature=0.0, top_k=0, top_p=None, repetition_penalty=1.0, seed=None,
            presence_penalty=0.0, frequency_penalty=0.0, min_p=None):
    """`ShapingConfig::new` (crates/selection/src/shaping.rs:84-123): validated at construction."""
    if not np.isfinite(temperature) or temperature < 0:
        raise ValueError(f"temperature must be finite and non-negative, got {temperature}")
    if top_k > 256:
        raise ValueError(f"top_k must be between 0 and 256, got {top_k}")
    if top_p is not None and not (np.isfinite(top_p) and 0.0 < top_p <= 1.0):
        raise ValueError(f"top_p must be finite and in (0, 1], got {top_p}")
    if not np.isfinite(repetition_penalty) or repetition_penalty <= 0:
        raise ValueError("repetition_penalty must be finite and greater than zero")
    s = Shaping()
    s.temperature = temperature
    s.top_k = top_k
    s.has_top_p = top_p is not None
    s.top_p = top_p or 0.0
    s.repetition_penalty = repetition_penalty
    s.has_seed = seed is not None
    s.seed = seed or 0
    s.presence_penalty = presence_penalty
    s.frequency_penalty = frequency_penalty
    s.has_min_p = min_p is not None
    s.min_p = min_p or 0.0
    return s


class AdaptiveDepth(C.Structure):
    """`AdaptiveDepth` of crates/runtime/src/speculative_adaptive.rs:105-227 (state lives here, the
    transitions in the library)."""
    _fields_ = [("floor", C.c_int32), ("cap", C.c_int32), ("cur", C.c_int32), ("climb", C.c_int32),
                ("pressure", C.c_int32), ("climb_low", C.c_int32), ("climb_mid", C.c_int32),
                ("climb_high", C.c_int32), ("drop", C.c_int32)]

    def __init__(self, floor, cap):
        super().__init__()
        lib().tsv_adaptive_init(C.byref(self), floor, cap)

    def depth(self):
        return lib().tsv_adaptive_depth(C.byref(self))

    def observe(self, offered, accepted):
        lib().tsv_adaptive_observe(C.byref(self), offered, accepted)

    @staticmethod
    def tile_cap(cap, tile_rows=None):
        return lib().tsv_adaptive_tile_cap(cap, tile_rows or 0)


class KvPrefix:
    """`KvPrefix` of crates/runtime/src/kv_prefix.rs:49-137: the token ids behind the cache rows
    (pure host state inside the library; no GPU involved)."""

    def __init__(self, ids=None):
        self._p = lib().tsv_prefix_new()
        if not self._p:
            raise MemoryError("tsv_prefix_new")
        if ids is not None:
            self.record(ids, 0)

    def __del__(self):
        if getattr(self, "_p", None):
            lib().tsv_prefix_free(self._p)
            self._p = None

    def clear(self):
        lib().tsv_prefix_clear(self._p)

    def taint(self):
        lib().tsv_prefix_taint(self._p)

    def record(self, tokens, pos0):
        t = np.ascontiguousarray(tokens, np.int32)
        lib().tsv_prefix_record(self._p, t.ctypes.data, t.size, int(pos0))

    def rewind_to(self, position):
        lib().tsv_prefix_rewind_to(self._p, int(position))

    def untainted_len(self):
        n = lib().tsv_prefix_untainted_len(self._p)
        return None if n < 0 else int(n)

    def common_prefix(self, prompt):
        t = np.ascontiguousarray(prompt, np.int32)
        return int(lib().tsv_prefix_common(self._p, t.ctypes.data, t.size))


class Gguf:
    """A GGUF file's header and tensors through the library's parser (read-only mapping)."""

    def __init__(self, path):
        h = C.c_void_p()
        check(lib().tsv_gguf_open(os.fsencode(path), C.byref(h)))
        self._h = h

    def close(self):
        if getattr(self, "_h", None):
            lib().tsv_gguf_close(self._h)
            self._h = None

    __del__ = close

    @property
    def tensor_count(self):
        return int(lib().tsv_gguf_tensor_count(self._h))

    @property
    def data_start(self):
        return int(lib().tsv_gguf_data_start(self._h))

    def number(self, key):
        v = C.c_double()
        check(lib().tsv_gguf_meta_number(self._h, key.encode(), C.byref(v)))
        return v.value

    def string(self, key):
        buf = C.create_string_buffer(256)
        check(lib().tsv_gguf_meta_string(self._h, key.encode(), buf, 256))
        return buf.value.decode()

    def tensor(self, name):
        """(dtype, bytes as uint8 [rows, row_bytes] -- a copy --, rows, cols)"""
        t = Tensor()
        check(lib().tsv_gguf_tensor(self._h, name.encode(), C.byref(t)))
        rb = row_bytes(t.dtype, t.cols)
        raw = np.ctypeslib.as_array(C.cast(t.data, C.POINTER(C.c_uint8)), shape=(t.rows * rb,)).copy()
        return t.dtype, raw.reshape(t.rows, rb), int(t.rows), int(t.cols)


DRAFT_PRIME = C.CFUNCTYPE(C.c_int32, C.c_void_p, C.c_int32, C.c_int64)
DRAFT_STEP = C.CFUNCTYPE(C.c_int32, C.c_void_p, C.c_int32, C.c_int64, C.POINTER(C.c_uint16))
DRAFT_REWIND = C.CFUNCTYPE(C.c_int32, C.c_void_p, C.c_int64)
DRAFT_POSITION = C.CFUNCTYPE(C.c_int64, C.c_void_p)


DRAFT_TREE = C.CFUNCTYPE(C.c_int32, C.c_void_p, C.c_int32, C.c_int64, C.c_int32, C.POINTER(C.c_int32), C.POINTER(C.c_int32))


DRAFT_BLOCK = C.CFUNCTYPE(C.c_int32, C.c_void_p, C.c_int32, C.c_int64, C.c_int32, C.POINTER(C.c_int32))
DRAFT_PREFILL_CHUNK = C.CFUNCTYPE(C.c_int32, C.c_void_p, C.POINTER(C.c_int32), C.c_int64, C.c_int64, C.POINTER(C.c_uint16),
                                  C.c_int32)


class Drafter(C.Structure):
    _fields_ = [("user", C.c_void_p), ("prime", DRAFT_PRIME), ("step", DRAFT_STEP), ("rewind", DRAFT_REWIND),
                ("device_logits", C.c_int32), ("position", DRAFT_POSITION), ("tree_nodes", C.c_int32),
                ("draft_tree", DRAFT_TREE), ("draft_block", DRAFT_BLOCK), ("prefill_chunk", DRAFT_PREFILL_CHUNK)]


class MtpDesc(C.Structure):
    _fields_ = [("model", ModelDesc), ("fc", Tensor), ("norm_embedding", Tensor), ("norm_hidden", Tensor)]


class Generation(C.Structure):
    _fields_ = [("shaping", Shaping), ("max_new_tokens", C.c_uint64), ("stop_tokens", C.POINTER(C.c_int32)),
                ("n_stop", C.c_int32), ("block", C.c_int32), ("adaptive_floor", C.c_int32)]


class GenerationResult(C.Structure):
    _fields_ = [("tokens", C.POINTER(C.c_int32)), ("capacity", C.c_int64), ("n_tokens", C.c_int64),
                ("stop_reason", C.c_int32), ("final_depth", C.c_int32), ("rounds", C.c_int64),
                ("offered", C.c_int64), ("accepted", C.c_int64), ("rollbacks", C.c_int64),
                ("draw_step", C.c_uint64), ("kv_position", C.c_int64), ("min_margin", C.c_double),
                ("reused", C.c_int64)]


class Point(C.Structure):
    _fields_ = [("position", C.c_int64)]


class Round(C.Structure):
    _fields_ = [
        ("feed", C.POINTER(C.c_int32)), ("parent", C.POINTER(C.c_int32)), ("m", C.c_int32),
        ("base", C.c_int64), ("shaping", Shaping), ("draft_logits", C.c_void_p),
        ("draw_step", C.c_uint64), ("stop_tokens", C.POINTER(C.c_int32)), ("n_stop", C.c_int32),
        ("generated", C.c_uint64), ("max_new_tokens", C.c_uint64), ("logits_out", C.c_void_p),
        ("history", C.POINTER(C.c_int32)), ("n_history", C.c_int64),
    ]


class RoundResultC(C.Structure):
    _fields_ = [
        ("accepted", C.c_int32), ("committed", C.c_int32), ("next", C.c_int32), ("stopped", C.c_int32),
        ("draw_step", C.c_uint64), ("path", C.c_int32 * (MAX_ROWS + 1)), ("path_len", C.c_int32),
        ("kv_position", C.c_int64), ("min_margin", C.c_double),
    ]


EXPORTS = [
    "tsv_open", "tsv_close", "tsv_last_error", "tsv_stream", "tsv_reset", "tsv_kv_position", "tsv_max_safe_rewind", "tsv_device_logits",
    "tsv_produce", "tsv_prefill", "tsv_checkpoint", "tsv_rollback", "tsv_rollback_retaining",
    "tsv_commit_pending", "tsv_discard_pending", "tsv_verify", "tsv_verify_tree", "tsv_compact_tree",
    "tsv_accept", "tsv_verify_accept", "tsv_accept_greedy_noalloc", "tsv_draft_chain", "tsv_row_bytes", "tsv_quantize_rows",
    "tsv_synth_tensor", "tsv_read_kv", "tsv_write_kv", "tsv_write_logits", "tsv_matmul", "tsv_attention", "tsv_set_profile", "tsv_get_profile", "tsv_matmul_time", "tsv_copy_time", "tsv_set_repeat",
    "tsv_yarn_frequencies", "tsv_adaptive_init", "tsv_adaptive_depth", "tsv_adaptive_observe", "tsv_adaptive_tile_cap",
    "tsv_run_speculative", "tsv_max_context", "tsv_vocab",
    "tsv_prefix_new", "tsv_prefix_free", "tsv_prefix_clear", "tsv_prefix_taint", "tsv_prefix_record",
    "tsv_prefix_rewind_to", "tsv_prefix_untainted_len", "tsv_prefix_common",
    "tsv_set_prefix_reuse", "tsv_try_reuse_prefix", "tsv_record_committed", "tsv_prefix_len",
    "tsv_gguf_open", "tsv_gguf_close", "tsv_gguf_tensor_count", "tsv_gguf_data_start", "tsv_gguf_tensor",
    "tsv_gguf_meta_number", "tsv_gguf_meta_string", "tsv_open_gguf", "tsv_route_selected", "tsv_force_route", "tsv_tree_walk_bound",
    "tsv_read_kv_quantized", "tsv_attention_quantized", "tsv_kv_quant_tables",
    "tsv_session_pool_size", "tsv_session_slot_evicted", "tsv_session_best_match", "tsv_session_lru", "tsv_session_swapped",
    "tsv_kv_row_bytes", "tsv_kv_bytes_for_context",
    "tsv_mtp_open", "tsv_mtp_step", "tsv_mtp_rewind", "tsv_mtp_prefill_chunk", "tsv_mtp_draft_block", "tsv_mtp_drafter",
]

_lib = None


def lib():
    """Loads libtsverify.so.  Fails loudly when it has not been built: there is no fallback."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
                "(hipcc, gfx950).  turbospark_amd has no CPU path.")
        L = C.CDLL(LIB_PATH)
        L.tsv_stream.restype = C.c_void_p
        L.tsv_stream.argtypes = [C.c_void_p]
        L.tsv_session_pool_size.argtypes = [C.c_void_p]
        L.tsv_kv_row_bytes.argtypes = [C.c_void_p, C.c_int32, C.POINTER(C.c_int64), C.POINTER(C.c_int64)]
        L.tsv_kv_bytes_for_context.restype = C.c_int64
        L.tsv_kv_bytes_for_context.argtypes = [C.c_void_p, C.c_int64]
        L.tsv_session_swapped.argtypes = [C.c_void_p]
        L.tsv_session_best_match.restype = C.c_int64
        L.tsv_session_best_match.argtypes = [C.c_void_p, C.c_int64, C.POINTER(C.c_int64)]
        L.tsv_session_lru.restype = C.c_int64
        L.tsv_session_lru.argtypes = [C.c_void_p, C.c_int64]
        L.tsv_session_slot_evicted.argtypes = [C.c_void_p]
        L.tsv_kv_position.restype = C.c_int64
        L.tsv_kv_position.argtypes = [C.c_void_p]
        L.tsv_max_safe_rewind.restype = C.c_int64
        L.tsv_max_safe_rewind.argtypes = [C.c_void_p]
        L.tsv_device_logits.restype = C.c_void_p
        L.tsv_device_logits.argtypes = [C.c_void_p]
        L.tsv_max_context.restype = C.c_int64
        L.tsv_max_context.argtypes = [C.c_void_p]
        L.tsv_vocab.restype = C.c_int64
        L.tsv_vocab.argtypes = [C.c_void_p]
        L.tsv_adaptive_observe.restype = None
        L.tsv_adaptive_init.restype = None
        L.tsv_run_speculative.argtypes = [C.c_void_p, C.POINTER(Drafter), C.c_void_p, C.c_int64,
                                          C.POINTER(Generation), C.POINTER(GenerationResult)]
        L.tsv_row_bytes.restype = C.c_int64
        L.tsv_row_bytes.argtypes = [C.c_int32, C.c_int64]
        L.tsv_yarn_frequencies.argtypes = [C.c_int32, C.c_float, C.c_float, C.c_int64, C.c_float, C.c_float,
                                           C.c_void_p, C.POINTER(C.c_float)]
        L.tsv_close.restype = None
        L.tsv_close.argtypes = [C.c_void_p]
        L.tsv_open.argtypes = [C.POINTER(ModelDesc), C.POINTER(C.c_void_p)]
        L.tsv_reset.argtypes = [C.c_void_p]
        L.tsv_produce.argtypes = [C.c_void_p, C.c_int32, C.c_int64, C.c_void_p]
        L.tsv_prefill.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_int64, C.c_void_p]
        L.tsv_checkpoint.argtypes = [C.c_void_p, C.POINTER(Point)]
        L.tsv_rollback.argtypes = [C.c_void_p, C.POINTER(Point)]
        L.tsv_rollback_retaining.argtypes = [C.c_void_p, C.POINTER(Point), C.c_int32]
        L.tsv_commit_pending.argtypes = [C.c_void_p, C.c_int32]
        L.tsv_discard_pending.argtypes = [C.c_void_p]
        L.tsv_verify.argtypes = [C.c_void_p, C.c_void_p, C.c_int32, C.c_int64, C.c_void_p]
        L.tsv_verify_tree.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32, C.c_int64, C.c_void_p]
        L.tsv_compact_tree.argtypes = [C.c_void_p, C.c_int64, C.c_void_p, C.c_int32]
        L.tsv_accept.argtypes = [C.c_void_p, C.POINTER(Round), C.POINTER(RoundResultC)]
        L.tsv_route_selected.argtypes = [C.c_void_p, C.c_void_p, C.c_int32]
        L.tsv_force_route.argtypes = [C.c_void_p, C.c_void_p, C.c_int32]
        L.tsv_accept_greedy_noalloc.argtypes = [C.c_void_p, C.c_void_p, C.c_int32, C.c_void_p, C.c_void_p, C.c_int32,
                                                C.c_int64, C.c_void_p, C.c_int32, C.c_uint64, C.c_uint64, C.c_void_p]
        L.tsv_verify_accept.argtypes = [C.c_void_p, C.POINTER(Round), C.POINTER(RoundResultC)]
        L.tsv_draft_chain.argtypes = [C.c_void_p, C.c_void_p, C.c_int32, C.POINTER(Shaping),
                                      C.POINTER(C.c_uint64), C.c_void_p, C.c_void_p, C.c_int64, C.c_uint64]
        L.tsv_quantize_rows.argtypes = [C.c_int32, C.c_void_p, C.c_int64, C.c_int64, C.c_void_p]
        L.tsv_synth_tensor.argtypes = [C.c_int32, C.c_uint64, C.c_uint64, C.c_float, C.c_int64, C.c_int64,
                                       C.c_void_p]
        L.tsv_read_kv.argtypes = [C.c_void_p, C.c_int32, C.c_int64, C.c_int64, C.c_void_p, C.c_void_p]
        L.tsv_write_kv.argtypes = [C.c_void_p, C.c_int32, C.c_int64, C.c_int64, C.c_void_p, C.c_void_p]
        L.tsv_write_logits.argtypes = [C.c_void_p, C.c_void_p, C.c_int32, C.c_int64]
        L.tsv_matmul.argtypes = [C.POINTER(Tensor), C.c_void_p, C.c_int32, C.c_void_p, C.c_int32]
        L.tsv_attention.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32, C.c_int32, C.c_int32, C.c_int32,
                                    C.c_int64, C.c_void_p, C.c_float, C.c_int32, C.c_void_p, C.c_void_p]
        L.tsv_read_kv_quantized.argtypes = [C.c_void_p, C.c_int32, C.c_int64, C.c_int64, C.c_void_p, C.c_void_p]
        L.tsv_attention_quantized.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32, C.c_int32, C.c_int32, C.c_int32,
                                              C.c_int64, C.c_int32, C.c_int32, C.c_float, C.c_void_p, C.c_void_p,
                                              C.c_void_p, C.c_void_p]
        L.tsv_mtp_open.argtypes = [C.c_void_p, C.POINTER(MtpDesc), C.POINTER(C.c_void_p)]
        L.tsv_mtp_step.argtypes = [C.c_void_p, C.c_int32, C.c_int64, C.c_void_p, C.c_int32]
        L.tsv_mtp_rewind.argtypes = [C.c_void_p, C.c_int64]
        L.tsv_mtp_prefill_chunk.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_int64, C.c_void_p, C.c_int32]
        L.tsv_mtp_draft_block.argtypes = [C.c_void_p, C.c_int32, C.c_int64, C.c_int32, C.c_void_p]
        L.tsv_mtp_drafter.argtypes = [C.c_void_p, C.POINTER(Drafter)]
        L.tsv_set_profile.argtypes = [C.c_void_p, C.c_int32]
        L.tsv_get_profile.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32]
        L.tsv_copy_time.argtypes = [C.c_int64, C.c_int32, C.POINTER(C.c_float)]
        L.tsv_matmul_time.argtypes = [C.c_int32, C.c_int64, C.c_int64, C.c_int32, C.c_int32, C.c_int32, C.c_int32,
                                      C.c_int32, C.POINTER(C.c_float)]
        L.tsv_last_error.argtypes = [C.c_char_p, C.c_int32]
        L.tsv_gguf_open.argtypes = [C.c_char_p, C.POINTER(C.c_void_p)]
        L.tsv_gguf_close.restype = None
        L.tsv_gguf_close.argtypes = [C.c_void_p]
        L.tsv_gguf_tensor_count.restype = C.c_int64
        L.tsv_gguf_tensor_count.argtypes = [C.c_void_p]
        L.tsv_gguf_data_start.restype = C.c_int64
        L.tsv_gguf_data_start.argtypes = [C.c_void_p]
        L.tsv_gguf_tensor.argtypes = [C.c_void_p, C.c_char_p, C.POINTER(Tensor)]
        L.tsv_gguf_meta_number.argtypes = [C.c_void_p, C.c_char_p, C.POINTER(C.c_double)]
        L.tsv_gguf_meta_string.argtypes = [C.c_void_p, C.c_char_p, C.c_char_p, C.c_int32]
        L.tsv_open_gguf.argtypes = [C.c_char_p, C.c_int32, C.POINTER(C.c_void_p)]
        L.tsv_prefix_new.restype = C.c_void_p
        L.tsv_prefix_new.argtypes = []
        for name in ("tsv_prefix_free", "tsv_prefix_clear", "tsv_prefix_taint"):
            getattr(L, name).restype = None
            getattr(L, name).argtypes = [C.c_void_p]
        L.tsv_prefix_record.restype = None
        L.tsv_prefix_record.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_int64]
        L.tsv_prefix_rewind_to.restype = None
        L.tsv_prefix_rewind_to.argtypes = [C.c_void_p, C.c_int64]
        L.tsv_prefix_untainted_len.restype = C.c_int64
        L.tsv_prefix_untainted_len.argtypes = [C.c_void_p]
        L.tsv_prefix_common.restype = C.c_int64
        L.tsv_prefix_common.argtypes = [C.c_void_p, C.c_void_p, C.c_int64]
        L.tsv_set_prefix_reuse.argtypes = [C.c_void_p, C.c_int32]
        L.tsv_try_reuse_prefix.restype = C.c_int64
        L.tsv_try_reuse_prefix.argtypes = [C.c_void_p, C.c_void_p, C.c_int64]
        L.tsv_record_committed.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_int64]
        L.tsv_prefix_len.restype = C.c_int64
        L.tsv_prefix_len.argtypes = [C.c_void_p]
        _lib = L
    return _lib


def last_error():
    buf = C.create_string_buffer(1024)
    lib().tsv_last_error(buf, 1024)
    return buf.value.decode(errors="replace")


def check(rc):
    if rc != 0:
        raise TsvError(rc, last_error())


def tensor(entry):
    """entry: None | (dtype, uint8 ndarray [rows, row_bytes], rows, cols)."""
    t = Tensor()
    if entry is None:
        return t
    dtype, data, rows, cols = entry
    t.data = data.ctypes.data
    t.dtype = dtype
    t.rows = rows
    t.cols = cols
    return t


def row_bytes(dtype, cols):
    return lib().tsv_row_bytes(dtype, cols)


def quantize(dtype, w):
    """fp32 [rows, cols] -> (dtype, uint8 [rows, row_bytes], rows, cols) with the install-time encoders."""
    w = np.ascontiguousarray(w, np.float32)
    rows, cols = w.shape
    rb = row_bytes(dtype, cols)
    if rb < 0:
        raise ValueError("column count is not whole blocks of this dtype")
    out = np.empty((rows, rb), np.uint8)
    check(lib().tsv_quantize_rows(dtype, w.ctypes.data, rows, cols, out.ctypes.data))
    return (dtype, out, rows, cols)


def synth_tensor(dtype, seed, stream, sigma, rows, cols):
    rb = row_bytes(dtype, cols)
    out = np.empty((rows, rb), np.uint8)
    check(lib().tsv_synth_tensor(dtype, seed, stream, sigma, rows, cols, out.ctypes.data))
    return (dtype, out, rows, cols)


def matmul(entry, x, splits=0):
    """y[m][r] = sum_k W[r][k] x[m][k] through the verify pass's own matmul kernel."""
    x = np.ascontiguousarray(x, np.float32)
    m = x.shape[0]
    t = tensor(entry)
    y = np.empty((m, entry[2]), np.float32)
    check(lib().tsv_matmul(C.byref(t), x.ctypes.data, m, y.ctypes.data, splits))
    return y


def attention(q, k, v, base, parent=None, scale=0.0, window=0, sinks=None):
    """q [m, nq, hd], k/v [base+m, nkv, hd] (any float dtype; rounded to fp16) -> fp32 [m, nq, hd]."""
    q16 = np.ascontiguousarray(np.asarray(q, np.float32).astype(np.float16))
    k16 = np.ascontiguousarray(np.asarray(k, np.float32).astype(np.float16))
    v16 = np.ascontiguousarray(np.asarray(v, np.float32).astype(np.float16))
    m, nq, hd = q16.shape
    nkv = k16.shape[1]
    assert k16.shape[0] == base + m
    out = np.empty((m, nq, hd), np.float16)
    pa = np.ascontiguousarray(parent, np.int32) if parent is not None else None
    sk = np.ascontiguousarray(sinks, np.float32) if sinks is not None else None
    check(lib().tsv_attention(C.c_void_p(q16.ctypes.data), C.c_void_p(k16.ctypes.data), C.c_void_p(v16.ctypes.data),
                              m, nq, nkv, hd, C.c_int64(base), C.c_void_p(pa.ctypes.data) if pa is not None else None,
                              C.c_float(scale), int(window), C.c_void_p(sk.ctypes.data) if sk is not None else None,
                              C.c_void_p(out.ctypes.data)))
    return out.astype(np.float32)


def kv_quant_tables(head_dim, bits, value_side=False):
    """(signs, codebook, midpoints) of one side of the KV codec, as the library computes them on the host."""
    signs = np.empty(head_dim, np.float32)
    cb = np.empty(1 << bits, np.float32)
    mid = np.empty((1 << bits) - 1, np.float32)
    check(lib().tsv_kv_quant_tables(int(head_dim), int(bits), int(bool(value_side)), C.c_void_p(signs.ctypes.data),
                                    C.c_void_p(cb.ctypes.data), C.c_void_p(mid.ctypes.data)))
    return signs, cb, mid


def packed_words(head_dim, bits):
    """crates/model-io/src/kv_quant.rs:128-133."""
    return (head_dim * bits + 31) // 32 if head_dim > 0 and bits > 0 else 0


def attention_quantized(q, k, v, base, k_bits, v_bits, scale=0.0, sinks=None):
    """q [m, nq, hd], k/v [base+m, nkv, hd] fp16 staging rows -> (fp32 [m, nq, hd], stored K rows, stored V rows);
    a stored row is [norm bits, words...] u32 per (position, kv head)."""
    q16, k16, v16 = (np.ascontiguousarray(np.asarray(a, np.float32).astype(np.float16)) for a in (q, k, v))
    m, nq, hd = q16.shape
    nkv = k16.shape[1]
    assert k16.shape[0] == base + m
    out = np.empty((m, nq, hd), np.float16)
    kr = np.zeros((base + m, nkv, 1 + packed_words(hd, k_bits)), np.uint32)
    vr = np.zeros((base + m, nkv, 1 + packed_words(hd, v_bits)), np.uint32)
    sk = np.ascontiguousarray(sinks, np.float32) if sinks is not None else None
    check(lib().tsv_attention_quantized(q16.ctypes.data, k16.ctypes.data, v16.ctypes.data, m, nq, nkv, hd, C.c_int64(base),
                                        int(k_bits), int(v_bits), C.c_float(scale),
                                        C.c_void_p(sk.ctypes.data) if sk is not None else None, out.ctypes.data,
                                        kr.ctypes.data, vr.ctypes.data))
    return out.astype(np.float32), kr, vr


def copy_time(nbytes, iters=20):
    """Average microseconds per launch of a plain device copy kernel over nbytes (HIP events)."""
    t = C.c_float()
    check(lib().tsv_copy_time(nbytes, iters, C.byref(t)))
    return t.value


def matmul_time(dtype, rows, cols, m, epi=0, splits=0, iters=50, rotate=4):
    """Average microseconds per launch of the verify matmul kernel (HIP events)."""
    t = C.c_float()
    check(lib().tsv_matmul_time(dtype, rows, cols, m, epi, splits, iters, rotate, C.byref(t)))
    return t.value


def yarn_frequencies(rotary_dim, base, factor, original_context, beta_fast, beta_slow):
    """(frequencies[rotary_dim // 2], mscale) of crates/compute/src/rope.rs:324-372."""
    f = np.empty(rotary_dim // 2, np.float32)
    ms = C.c_float()
    check(lib().tsv_yarn_frequencies(rotary_dim, base, factor, original_context, beta_fast, beta_slow,
                                     f.ctypes.data, C.byref(ms)))
    return f, float(ms.value)
