"""ctypes view of oracle/libtsoracle.so (the CPU restatement of the reference path).

Test infrastructure only: imported by tests/, by __graft_entry__.smoke() and by the
cpu_baseline leg of bench.py as the checker.  The product package never imports it.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_DIR = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_DIR, "libtsoracle.so")

F32, F16, Q8_0, Q4_K, Q5_K, Q6_K, BF16, MXFP4 = 0, 1, 8, 12, 13, 14, 30, 39


def build():
    subprocess.check_call(["make", "-C", _DIR, "-s", "-B"])


class Shaping(C.Structure):
    _fields_ = [
        ("temperature", C.c_double),
        ("top_k", C.c_uint32),
        ("has_top_p", C.c_int32),
        ("top_p", C.c_double),
        ("repetition_penalty", C.c_double),
        ("has_seed", C.c_int32),
        ("seed", C.c_uint64),
        ("presence_penalty", C.c_double),
        ("frequency_penalty", C.c_double),
        ("has_min_p", C.c_int32),
        ("min_p", C.c_double),
    ]


def shaping(temperature=0.0, top_k=0, top_p=None, repetition_penalty=1.0, seed=None,
            presence_penalty=0.0, frequency_penalty=0.0, min_p=None):
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


class RoundResult(C.Structure):
    _fields_ = [
        ("accepted", C.c_int32),
        ("committed", C.c_int32),
        ("next", C.c_int32),
        ("stopped", C.c_int32),
        ("draw_step", C.c_uint64),
        ("path", C.c_int32 * 17),
        ("path_len", C.c_int32),
    ]

    def as_dict(self):
        return dict(accepted=self.accepted, committed=self.committed, next=self.next,
                    stopped=self.stopped, draw_step=self.draw_step,
                    path=list(self.path[: self.path_len]))


class Tensor(C.Structure):
    _fields_ = [("data", C.c_void_p), ("dtype", C.c_int32), ("rows", C.c_int64), ("cols", C.c_int64)]


LAYER_TENSORS = ("attn_norm", "wq", "wk", "wv", "wo", "q_norm", "k_norm", "ffn_norm", "w_gate", "w_up", "w_down")
LAYER_MOE_TENSORS = ("router", "we_gate", "we_up", "we_down")
LAYER_GPTOSS_TENSORS = ("bq", "bk", "bv", "bo", "sinks", "router_bias", "be_gate", "be_up", "be_down")


class Layer(C.Structure):
    _fields_ = ([(n, Tensor) for n in LAYER_TENSORS] + [("n_experts", C.c_int32), ("top_k", C.c_int32)] +
                [(n, Tensor) for n in LAYER_MOE_TENSORS] + [(n, Tensor) for n in LAYER_GPTOSS_TENSORS] +
                [("window", C.c_int32)])


class ModelDesc(C.Structure):
    _fields_ = [
        ("n_layers", C.c_int32), ("hidden", C.c_int32), ("n_q_heads", C.c_int32),
        ("n_kv_heads", C.c_int32), ("head_dim", C.c_int32), ("ffn", C.c_int32),
        ("vocab", C.c_int32), ("max_context", C.c_int32),
        ("rms_eps", C.c_float), ("rope_theta", C.c_float), ("attn_scale", C.c_float),
        ("rope_factors", C.POINTER(C.c_float)),
        ("round_kv_f16", C.c_int32), ("threads", C.c_int32),
        ("embed", Tensor), ("final_norm", Tensor), ("lm_head", Tensor),
        ("layers", C.POINTER(Layer)),
        ("rope_freqs", C.POINTER(C.c_float)), ("rope_mscale", C.c_float),
        ("act_alpha", C.c_float), ("act_limit", C.c_float),
        ("kv_k_bits", C.c_int32), ("kv_v_bits", C.c_int32),
    ]


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        L = C.CDLL(_SO)
        L.tso_f32_to_f16.argtypes = [C.c_float]
        L.tso_f32_to_f16.restype = C.c_uint16
        L.tso_f16_to_f32.argtypes = [C.c_uint16]
        L.tso_f16_to_f32.restype = C.c_float
        L.tso_f32_to_bf16.argtypes = [C.c_float]
        L.tso_f32_to_bf16.restype = C.c_uint16
        L.tso_bf16_to_f32.argtypes = [C.c_uint16]
        L.tso_bf16_to_f32.restype = C.c_float
        L.tso_row_bytes.argtypes = [C.c_int, C.c_int64]
        L.tso_row_bytes.restype = C.c_int64
        L.tso_mxfp4_scale.argtypes = [C.c_uint8]
        L.tso_mxfp4_scale.restype = C.c_float
        L.tso_silu.argtypes = [C.c_float]
        L.tso_silu.restype = C.c_float
        L.tso_swiglu_oai.restype = C.c_float
        L.tso_mix.argtypes = [C.c_uint64]
        L.tso_mix.restype = C.c_uint64
        L.tso_derive_step_value.argtypes = [C.c_uint64, C.c_uint64]
        L.tso_derive_step_value.restype = C.c_uint64
        L.tso_to_unit_interval.argtypes = [C.c_uint64]
        L.tso_to_unit_interval.restype = C.c_double
        L.tso_dist_probability.restype = C.c_double
        L.tso_dist_draw.restype = C.c_uint32
        L.tso_model_create.restype = C.c_void_p
        L.tso_model_position.restype = C.c_int64
        L.tso_model_route_margin.restype = C.c_float
        L.tso_model_route_record.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p]
        L.tso_model_force_route.argtypes = [C.c_void_p, C.c_void_p, C.c_int64]
        L.tso_model_last_hidden.argtypes = [C.c_void_p, C.c_int, C.c_void_p]
        L.tso_mtp_step.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int64, C.c_void_p,
                                   C.c_void_p, C.c_void_p]
        L.tso_model_k.restype = C.POINTER(C.c_float)
        L.tso_model_v.restype = C.POINTER(C.c_float)
        L.tso_last_error.restype = C.c_char_p
        _lib = L
    return _lib


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


def last_error():
    return lib().tso_last_error().decode()


# ---------------------------------------------------------------- conversions
def f32_to_f16_bits(x):
    x = np.asarray(x, np.float32)
    f = np.vectorize(lambda v: lib().tso_f32_to_f16(float(v)), otypes=[np.uint16])
    return f(x)


def row_bytes(dtype, n):
    return lib().tso_row_bytes(dtype, n)


def quantize(dtype, w):
    """w: [rows, cols] fp32 -> uint8 [rows, row_bytes]."""
    w = np.ascontiguousarray(w, np.float32)
    rows, cols = w.shape
    if dtype == F32:
        return w.view(np.uint8).reshape(rows, cols * 4).copy()
    if dtype == F16:
        return w.astype(np.float16).view(np.uint8).reshape(rows, cols * 2).copy()
    if dtype == BF16:
        out = np.empty((rows, cols), np.uint16)
        flat = w.reshape(-1)
        o = out.reshape(-1)
        for i in range(flat.size):
            o[i] = lib().tso_f32_to_bf16(float(flat[i]))
        return out.view(np.uint8).reshape(rows, cols * 2)
    fn = {Q8_0: lib().tso_quantize_q8_0, Q4_K: lib().tso_quantize_q4_k, Q5_K: lib().tso_quantize_q5_k,
          Q6_K: lib().tso_quantize_q6_k,
          MXFP4: lib().tso_quantize_mxfp4}[dtype]
    rb = row_bytes(dtype, cols)
    out = np.empty((rows, rb), np.uint8)
    for r in range(rows):
        fn(_p(w[r]), C.c_int64(cols), C.c_void_p(out[r].ctypes.data))
    return out


def dequantize(dtype, b, cols):
    b = np.ascontiguousarray(b, np.uint8)
    if b.ndim == 1:
        b = b.reshape(1, -1)
    rows = b.shape[0]
    out = np.empty((rows, cols), np.float32)
    for r in range(rows):
        lib().tso_dequantize_row(C.c_int(dtype), C.c_void_p(b[r].ctypes.data), C.c_int64(cols),
                                 C.c_void_p(out[r].ctypes.data))
    return out


def gemv(dtype, wbytes, rows, cols, x):
    wbytes = np.ascontiguousarray(wbytes, np.uint8)
    x = np.ascontiguousarray(x, np.float32)
    y = np.empty(rows, np.float32)
    lib().tso_gemv(C.c_int(dtype), _p(wbytes), C.c_int64(rows), C.c_int64(cols), _p(x), _p(y))
    return y


# ---------------------------------------------------------------------- ops
def rms_norm(x, w, eps):
    x = np.ascontiguousarray(x, np.float32)
    w = np.ascontiguousarray(w, np.float32)
    y = np.empty_like(x)
    lib().tso_rms_norm(_p(x), _p(w), C.c_int64(x.size), C.c_float(eps), _p(y))
    return y


def rope_neox(x, num_tokens, num_heads, head_dim, rotated_pairs, position, theta):
    x = np.array(x, np.float32, copy=True)
    lib().tso_rope_neox(_p(x), num_tokens, num_heads, head_dim, rotated_pairs, C.c_int64(position),
                        C.c_float(theta))
    return x


def rope_neox_freqs(x, num_tokens, num_heads, head_dim, rotated_pairs, position, freqs):
    x = np.array(x, np.float32, copy=True)
    freqs = np.ascontiguousarray(freqs, np.float32)
    lib().tso_rope_neox_freqs(_p(x), num_tokens, num_heads, head_dim, rotated_pairs,
                              C.c_int64(position), _p(freqs))
    return x


def yarn_frequencies(rotary_dim, base, factor, original_context, beta_fast, beta_slow):
    f = np.empty(rotary_dim // 2, np.float32)
    ms = C.c_float()
    lib().tso_yarn_frequencies(rotary_dim, C.c_float(base), C.c_float(factor), C.c_int64(original_context),
                               C.c_float(beta_fast), C.c_float(beta_slow), _p(f), C.byref(ms))
    return f, float(ms.value)


def rope_neox_freqs_scaled(x, num_tokens, num_heads, head_dim, rotated_pairs, position, freqs, mscale):
    x = np.ascontiguousarray(x, np.float32).copy()
    freqs = np.ascontiguousarray(freqs, np.float32)
    lib().tso_rope_neox_freqs_scaled(_p(x), num_tokens, num_heads, head_dim, rotated_pairs,
                                     C.c_int64(position), _p(freqs), C.c_float(mscale))
    return x


def swiglu_oai(gate, up, alpha, limit):
    return float(lib().tso_swiglu_oai(C.c_float(gate), C.c_float(up), C.c_float(alpha), C.c_float(limit)))


def llama3_rope_factors(rotary_dim, base, factor, low, high, original_context):
    out = np.empty(max(rotary_dim // 2, 1), np.float32)
    rc = lib().tso_llama3_rope_factors(rotary_dim, C.c_double(base), C.c_double(factor),
                                       C.c_double(low), C.c_double(high),
                                       C.c_double(original_context), _p(out))
    return None if rc < 0 else out


def rope_frequencies_with_factors(rotary_dim, base, factors):
    factors = np.ascontiguousarray(factors, np.float32)
    out = np.empty(rotary_dim // 2, np.float32)
    lib().tso_rope_frequencies_with_factors(rotary_dim, C.c_float(base), _p(factors), _p(out))
    return out


def causal_attention(q, k, v, head_dim, nq, nkv, seq_len, window=0, scale=0.0, sinks=None):
    q = np.ascontiguousarray(q, np.float32)
    k = np.ascontiguousarray(k, np.float32)
    v = np.ascontiguousarray(v, np.float32)
    out = np.empty(nq * head_dim, np.float32)
    sp = _p(np.ascontiguousarray(sinks, np.float32)) if sinks is not None else None
    lib().tso_causal_attention(_p(q), _p(k), _p(v), head_dim, nq, nkv, C.c_int64(seq_len),
                               C.c_int64(window), C.c_float(scale), sp, _p(out))
    return out


# ----------------------------------------------------------------- TurboQuant KV codec (tq.cpp)
TQ_KEY_SEED, TQ_VALUE_SEED = 0, 1   # kv_quant.rs:33-36


def tq_sign_vector(dim, seed):
    out = np.empty(dim, np.float32)
    lib().tso_tq_sign_vector(dim, C.c_uint64(seed), _p(out))
    return out


def tq_wht(x):
    x = np.ascontiguousarray(x, np.float32)
    y = np.empty_like(x)
    lib().tso_tq_wht(_p(x), x.size, _p(y))
    return y


def tq_rht(x, signs, inverse=False):
    x, signs = np.ascontiguousarray(x, np.float32), np.ascontiguousarray(signs, np.float32)
    y = np.empty_like(x)
    (lib().tso_tq_rht_inverse if inverse else lib().tso_tq_rht_forward)(_p(x), _p(signs), x.size, _p(y))
    return y


def tq_codebook(dim, bits):
    out = np.empty(max(1 << bits, 1), np.float32)
    n = lib().tso_tq_codebook(dim, bits, _p(out))
    return out[:n].copy()


def tq_midpoints(codebook):
    cb = np.ascontiguousarray(codebook, np.float32)
    out = np.empty(max(cb.size - 1, 0), np.float32)
    lib().tso_tq_midpoints(_p(cb), cb.size, _p(out))
    return out


def tq_packed_words(length, bits):
    return lib().tso_tq_packed_words(length, bits)


def tq_pack(indices, bits):
    idx = np.ascontiguousarray(indices, np.uint32)
    out = np.zeros(max(tq_packed_words(idx.size, bits), 1) + 1, np.uint32)
    n = lib().tso_tq_pack(_p(idx), idx.size, bits, _p(out))
    if n < 0:
        raise ValueError("index does not fit, or bits outside 1..16")
    return out[:n].copy()


def tq_unpack(packed, bits, length):
    pk = np.ascontiguousarray(np.concatenate([np.asarray(packed, np.uint32), np.zeros(1, np.uint32)]))
    out = np.zeros(length, np.uint32)
    if lib().tso_tq_unpack(_p(pk), bits, length, _p(out)) < 0:
        raise ValueError("bits outside 1..16")
    return out


def tq_quantize_row(x, signs, midpoints, bits):
    x, signs, mp = (np.ascontiguousarray(a, np.float32) for a in (x, signs, midpoints))
    words = np.zeros(tq_packed_words(x.size, bits) + 1, np.uint32)
    norm = C.c_float(0)
    lib().tso_tq_quantize_row(_p(x), x.size, _p(signs), _p(mp), bits, C.byref(norm), _p(words))
    return norm.value, words[:-1].copy()


def tq_dequantize_row(norm, words, signs, codebook, bits, dim):
    pk = np.ascontiguousarray(np.concatenate([np.asarray(words, np.uint32), np.zeros(1, np.uint32)]))
    signs, cb = np.ascontiguousarray(signs, np.float32), np.ascontiguousarray(codebook, np.float32)
    out = np.empty(dim, np.float32)
    lib().tso_tq_dequantize_row(C.c_float(norm), _p(pk), _p(signs), _p(cb), bits, dim, _p(out))
    return out


def tq_roundtrip_rows(rows, bits, seed):
    """rows [..., dim] -> what a quantized layer holds of them (decode of the stored norm and indices), same shape."""
    x = np.ascontiguousarray(rows, np.float32)
    dim = x.shape[-1]
    signs, cb = tq_sign_vector(dim, seed), tq_codebook(dim, bits)
    mid = tq_midpoints(cb)
    out = np.empty_like(x)
    lib().tso_tq_roundtrip_rows(_p(x), C.c_int64(x.size // dim), dim, _p(signs), _p(cb), _p(mid), bits, _p(out))
    return out


def tq_attention(q, k_words, k_norms, v_words, v_norms, hd, nq, nkv, seq_len, bits, k_signs, k_cb, v_signs, v_cb,
                 scale=0.0, sinks=None, v_bits=None):
    """kv_quant_attention.rs:58-136.  k / v words: [seq_len, nkv, words per row] uint32, norms [seq_len, nkv];
    bits is the key width and, unless v_bits is given, the value width too."""
    q = np.ascontiguousarray(q, np.float32)
    kw = np.ascontiguousarray(np.concatenate([np.asarray(k_words, np.uint32).reshape(-1), np.zeros(1, np.uint32)]))
    vw = np.ascontiguousarray(np.concatenate([np.asarray(v_words, np.uint32).reshape(-1), np.zeros(1, np.uint32)]))
    kn, vn = np.ascontiguousarray(k_norms, np.float32), np.ascontiguousarray(v_norms, np.float32)
    ks, kc, vs, vc = (np.ascontiguousarray(a, np.float32) for a in (k_signs, k_cb, v_signs, v_cb))
    out = np.empty(nq * hd, np.float32)
    sp = _p(np.ascontiguousarray(sinks, np.float32)) if sinks is not None else None
    lib().tso_tq_attention(_p(q), _p(kw), _p(kn), _p(vw), _p(vn), hd, nq, nkv, seq_len, C.c_float(scale), sp,
                           _p(ks), _p(kc), _p(vs), _p(vc), bits, bits if v_bits is None else v_bits, _p(out))
    return out


# ----------------------------------------------------------------- selection
def _hist(history):
    h = np.ascontiguousarray(history if history is not None else [], np.int32)
    return h, _p(h), C.c_int64(h.size)


def _logits_bits(logits):
    a = np.asarray(logits)
    if a.dtype == np.uint16:
        return np.ascontiguousarray(a)
    return np.ascontiguousarray(a.astype(np.float16)).view(np.uint16)


def select(logits, cfg, history=None, position=0):
    lb = _logits_bits(logits)
    h, hp, hn = _hist(history)
    out = C.c_int32()
    rc = lib().tso_select(_p(lb), C.c_int64(lb.size), C.byref(cfg), hp, hn, C.c_uint64(position),
                          C.byref(out))
    if rc < 0:
        raise ValueError(last_error())
    return out.value


def shaped_distribution(logits, cfg, history=None, position=0):
    lb = _logits_bits(logits)
    h, hp, hn = _hist(history)
    sup = np.empty(lb.size, np.uint32)
    pr = np.empty(lb.size, np.float64)
    n = C.c_int64()
    rc = lib().tso_shaped_distribution(_p(lb), C.c_int64(lb.size), C.byref(cfg), hp, hn,
                                       C.c_uint64(position), _p(sup), _p(pr), C.byref(n))
    if rc < 0:
        raise ValueError(last_error())
    return sup[: n.value].copy(), pr[: n.value].copy()


def dist_probability(support, probs, token):
    s = np.ascontiguousarray(support, np.uint32)
    p = np.ascontiguousarray(probs, np.float64)
    return lib().tso_dist_probability(_p(s), _p(p), C.c_int64(s.size), C.c_uint32(token))


def dist_draw(support, probs, seed, position):
    s = np.ascontiguousarray(support, np.uint32)
    p = np.ascontiguousarray(probs, np.float64)
    return lib().tso_dist_draw(_p(s), _p(p), C.c_int64(s.size), C.c_uint64(seed), C.c_uint64(position))


def residual(p, q):
    ps, pp = np.ascontiguousarray(p[0], np.uint32), np.ascontiguousarray(p[1], np.float64)
    qs, qp = np.ascontiguousarray(q[0], np.uint32), np.ascontiguousarray(q[1], np.float64)
    os_ = np.empty(ps.size, np.uint32)
    op = np.empty(ps.size, np.float64)
    n = C.c_int64()
    rc = lib().tso_residual(_p(ps), _p(pp), C.c_int64(ps.size), _p(qs), _p(qp), C.c_int64(qs.size),
                            _p(os_), _p(op), C.byref(n))
    if rc == 0:
        return None
    return os_[: n.value].copy(), op[: n.value].copy()


def draft_chain(draft_logits, cfg, history=None, generated=0, draw_step=0):
    lb = _logits_bits(draft_logits)
    k, vocab = lb.shape
    h, hp, hn = _hist(history)
    ds = C.c_uint64(draw_step)
    props = np.empty(k, np.int32)
    rc = lib().tso_draft_chain(_p(lb), k, C.c_int64(vocab), C.byref(cfg), hp, hn,
                               C.c_uint64(generated), C.byref(ds), _p(props))
    if rc < 0:
        raise ValueError(last_error())
    return props, ds.value


def chain_round(target_logits, draft_logits, proposals, cfg, history=None, generated=0,
                max_new_tokens=1 << 40, stop_tokens=None, draw_step=0):
    tb = _logits_bits(target_logits)
    k = len(proposals)
    vocab = tb.shape[1]
    db = _logits_bits(draft_logits) if draft_logits is not None else None
    h, hp, hn = _hist(history)
    pr = np.ascontiguousarray(proposals, np.int32)
    st = np.ascontiguousarray(stop_tokens if stop_tokens is not None else [], np.int32)
    out = RoundResult()
    rc = lib().tso_chain_round(_p(tb), _p(db) if db is not None else None, _p(pr), k,
                               C.c_int64(vocab), C.byref(cfg), hp, hn, C.c_uint64(generated),
                               C.c_uint64(max_new_tokens), _p(st), int(st.size),
                               C.c_uint64(draw_step), C.byref(out))
    if rc < 0:
        raise ValueError(last_error())
    return out.as_dict()


def tree_round_greedy(target_logits, feed, parent, cfg, history=None, generated=0,
                      max_new_tokens=1 << 40, stop_tokens=None):
    tb = _logits_bits(target_logits)
    m, vocab = tb.shape
    h, hp, hn = _hist(history)
    fd = np.ascontiguousarray(feed, np.int32)
    pa = np.ascontiguousarray(parent, np.int32)
    st = np.ascontiguousarray(stop_tokens if stop_tokens is not None else [], np.int32)
    out = RoundResult()
    rc = lib().tso_tree_round_greedy(_p(tb), _p(fd), _p(pa), m, C.c_int64(vocab), C.byref(cfg), hp,
                                     hn, C.c_uint64(generated), C.c_uint64(max_new_tokens), _p(st),
                                     int(st.size), C.byref(out))
    if rc < 0:
        raise ValueError(last_error())
    return out.as_dict()


def tree_round_sampled(target_logits, draft_logits, feed, parent, cfg, history=None, generated=0,
                       draw_step=0):
    tb = _logits_bits(target_logits)
    db = _logits_bits(draft_logits)
    m, vocab = tb.shape
    h, hp, hn = _hist(history)
    fd = np.ascontiguousarray(feed, np.int32)
    pa = np.ascontiguousarray(parent, np.int32)
    out = RoundResult()
    rc = lib().tso_tree_round_sampled(_p(tb), _p(db), _p(fd), _p(pa), m, C.c_int64(vocab),
                                      C.byref(cfg), hp, hn, C.c_uint64(generated),
                                      C.c_uint64(draw_step), C.byref(out))
    if rc < 0:
        raise ValueError(last_error())
    return out.as_dict()


# --------------------------------------------------------------------- model
def _tensor(entry):
    """entry: None | (dtype, uint8 array [rows, row_bytes], rows, cols)."""
    t = Tensor()
    if entry is None:
        return t
    dtype, data, rows, cols = entry
    t.data = data.ctypes.data
    t.dtype = dtype
    t.rows = rows
    t.cols = cols
    return t


class Model:
    """Oracle target model over host weight bytes.

    `weights` is the dict produced by turbospark_amd.synth / tests: keys embed, final_norm,
    lm_head (optional) and layers (list of dicts with attn_norm, wq, wk, wv, wo,
    [q_norm, k_norm], ffn_norm, w_gate, w_up, w_down); every tensor is
    (dtype, uint8 ndarray, rows, cols).  The arrays must outlive the model.
    """

    def __init__(self, cfg, weights, round_kv_f16=True, threads=1, kv_bits=None):
        """kv_bits: None (fp16 rows) or (key bits, value bits) of the TurboQuant KV codec."""
        self._keep = weights
        n = cfg["n_layers"]
        self._layers = (Layer * n)()
        for i, lw in enumerate(weights["layers"]):
            for name in LAYER_TENSORS + LAYER_MOE_TENSORS + LAYER_GPTOSS_TENSORS:
                setattr(self._layers[i], name, _tensor(lw.get(name)))
            self._layers[i].n_experts = int(lw.get("n_experts", 0))
            self._layers[i].top_k = int(lw.get("top_k", 0))
            self._layers[i].window = int(lw.get("window", 0))
        d = ModelDesc()
        for key in ("n_layers", "hidden", "n_q_heads", "n_kv_heads", "head_dim", "ffn", "vocab",
                    "max_context"):
            setattr(d, key, cfg[key])
        d.rms_eps = cfg.get("rms_eps", 1e-5)
        d.rope_theta = cfg.get("rope_theta", 10000.0)
        d.attn_scale = cfg.get("attn_scale", 0.0)
        self._factors = None
        if cfg.get("rope_factors") is not None:
            self._factors = np.ascontiguousarray(cfg["rope_factors"], np.float32)
            d.rope_factors = self._factors.ctypes.data_as(C.POINTER(C.c_float))
        self._freqs = None
        if cfg.get("rope_freqs") is not None:
            self._freqs = np.ascontiguousarray(cfg["rope_freqs"], np.float32)
            d.rope_freqs = self._freqs.ctypes.data_as(C.POINTER(C.c_float))
        d.rope_mscale = cfg.get("rope_mscale", 0.0)
        d.act_alpha = cfg.get("act_alpha", 0.0)
        d.act_limit = cfg.get("act_limit", 0.0)
        d.round_kv_f16 = int(round_kv_f16)
        d.threads = threads
        d.kv_k_bits, d.kv_v_bits = kv_bits if kv_bits else (0, 0)
        d.embed = _tensor(weights["embed"])
        d.final_norm = _tensor(weights["final_norm"])
        d.lm_head = _tensor(weights.get("lm_head"))
        d.layers = C.cast(self._layers, C.POINTER(Layer))
        self.cfg = cfg
        self._h = C.c_void_p(lib().tso_model_create(C.byref(d)))

    def __del__(self):
        if getattr(self, "_h", None):
            lib().tso_model_destroy(self._h)
            self._h = None

    @property
    def position(self):
        return lib().tso_model_position(self._h)

    def layer_quantized(self, layer):
        return bool(lib().tso_model_layer_quantized(self._h, layer))

    def reset(self):
        lib().tso_model_reset(self._h)

    @property
    def route_margin(self):
        """Smallest relative gap between the last chosen and the first rejected router logit
        over the last verify call (1.0 for a dense model)."""
        return float(lib().tso_model_route_margin(self._h))

    def route_record(self):
        """(selected [layers, 16, 8] expert ids in rank order, -1 past top_k; gap [layers, 16]) of the last verify."""
        n = self.cfg["n_layers"]
        sel = np.full((n, 16, 8), -1, np.int32)
        gap = np.ones((n, 16), np.float32)
        if lib().tso_model_route_record(self._h, _p(sel), _p(gap)) != 0:
            raise ValueError("no routed layer has run")
        return sel, gap

    def force_route(self, sel=None):
        """Test hook: take these experts ([layers, 16, 8]) instead of the top-k; None restores the ranking."""
        if sel is None:
            lib().tso_model_force_route(self._h, None, 0)
        else:
            a = np.ascontiguousarray(sel, np.int32)
            lib().tso_model_force_route(self._h, _p(a), a.size)

    def rewind_to(self, position):
        lib().tso_model_rewind_to(self._h, C.c_int64(position))

    def verify(self, feed, base, parent=None, want_f32=False, n_layers_run=-1):
        feed = np.ascontiguousarray(feed, np.int32)
        m = feed.size
        vocab = self.cfg["vocab"]
        f16 = np.empty((m, vocab), np.uint16)
        f32 = np.empty((m, vocab), np.float32) if want_f32 else None
        pa = np.ascontiguousarray(parent, np.int32) if parent is not None else None
        rc = lib().tso_model_verify(self._h, _p(feed), _p(pa) if pa is not None else None, m,
                                    C.c_int64(base), _p(f16), _p(f32) if want_f32 else None,
                                    n_layers_run)
        if rc < 0:
            raise ValueError(last_error())
        return (f16, f32) if want_f32 else f16

    def prime(self, feed, base):
        """A pass taken for its cache rows alone: no final norm, no output head."""
        feed = np.ascontiguousarray(feed, np.int32)
        rc = lib().tso_model_verify(self._h, _p(feed), None, int(feed.size), C.c_int64(base), None, None, -1)
        if rc < 0:
            raise ValueError(last_error())

    def last_hidden(self, row):
        """Row `row` of the last pass's residual stream after the last layer (what the final norm consumes)."""
        out = np.empty(self.cfg["hidden"], np.float32)
        if lib().tso_model_last_hidden(self._h, int(row), _p(out)) != 0:
            raise ValueError(last_error())
        return out

    def kv(self, layer):
        c = self.cfg
        n = c["max_context"] * c["n_kv_heads"] * c["head_dim"]
        shape = (c["max_context"], c["n_kv_heads"], c["head_dim"])
        k = np.ctypeslib.as_array(lib().tso_model_k(self._h, layer), shape=(n,)).reshape(shape)
        v = np.ctypeslib.as_array(lib().tso_model_v(self._h, layer), shape=(n,)).reshape(shape)
        return k, v

    def compact_tree(self, base, path):
        p = np.ascontiguousarray(path, np.uint32)
        lib().tso_model_compact_tree(self._h, C.c_int64(base), _p(p), int(p.size))


class MtpDesc(C.Structure):
    _fields_ = [("fc", Tensor), ("norm_embedding", Tensor), ("norm_hidden", Tensor), ("trunk_norm", Tensor)]


class MtpHead:
    """The drafter head of docs/MTP.md:53-60 over host weight bytes: a one-layer Model (its final_norm the
    head's own norm, embed / lm_head the trunk's) plus fc and the norms of fc's two halves.  `weights`
    is a Model weights dict with the extra keys fc, norm_embedding, norm_hidden, trunk_norm."""

    def __init__(self, cfg, weights, round_kv_f16=True, threads=1):
        assert cfg["n_layers"] == 1
        self.model = Model(cfg, weights, round_kv_f16=round_kv_f16, threads=threads)
        self.cfg = cfg
        self._d = MtpDesc()
        for name in ("fc", "norm_embedding", "norm_hidden", "trunk_norm"):
            setattr(self._d, name, _tensor(weights[name]))

    @property
    def position(self):
        return self.model.position

    def rewind_to(self, position):
        self.model.rewind_to(position)

    def reset(self):
        self.model.reset()

    def step(self, next_tokens, h_rows, position, want="f16", want_x0=False):
        """Rows at position .. position + n - 1.  want: "f16", "f32" (both), or None (a priming step)."""
        toks = np.ascontiguousarray(next_tokens, np.int32)
        h = np.ascontiguousarray(h_rows, np.float32).reshape(toks.size, self.cfg["hidden"])
        vocab = self.cfg["vocab"]
        f16 = np.empty((toks.size, vocab), np.uint16) if want else None
        f32 = np.empty((toks.size, vocab), np.float32) if want == "f32" else None
        x0 = np.empty((toks.size, self.cfg["hidden"]), np.float32) if want_x0 else None
        rc = lib().tso_mtp_step(self.model._h, C.byref(self._d), _p(toks), _p(h), int(toks.size), C.c_int64(position),
                                _p(f16) if f16 is not None else None, _p(f32) if f32 is not None else None,
                                _p(x0) if x0 is not None else None)
        if rc < 0:
            raise ValueError(last_error())
        out = (f16, f32) if want == "f32" else f16
        return (out, x0) if want_x0 else out

    def last_hidden(self, row=0):
        return self.model.last_hidden(row)


# ------------------------------------------------------- adaptive depth and the generation loop
class Adaptive(C.Structure):
    """crates/runtime/src/speculative_adaptive.rs:105-227."""
    _fields_ = [("floor", C.c_int), ("cap", C.c_int), ("cur", C.c_int), ("climb", C.c_int),
                ("pressure", C.c_int), ("params", C.c_int * 4)]

    def __init__(self, floor, cap):
        super().__init__()
        lib().tso_adaptive_new(C.byref(self), floor, cap)

    def depth(self):
        return self.cur

    def observe(self, offered, accepted):
        lib().tso_adaptive_observe(C.byref(self), offered, accepted)

    @staticmethod
    def tile_cap(cap, tile_rows):
        return lib().tso_adaptive_tile_cap(cap, tile_rows if tile_rows else 0)


_CB_I = C.CFUNCTYPE(C.c_int, C.c_void_p)
_CB_PRODUCE = C.CFUNCTYPE(C.c_int, C.c_void_p, C.c_int32, C.c_int64, C.POINTER(C.c_uint16))
_CB_TOKPOS = C.CFUNCTYPE(C.c_int, C.c_void_p, C.c_int32, C.c_int64)
_CB_VERIFY = C.CFUNCTYPE(C.c_int, C.c_void_p, C.POINTER(C.c_int32), C.c_int, C.c_int64, C.POINTER(C.c_uint16))
_CB_ROLL = C.CFUNCTYPE(C.c_int, C.c_void_p, C.c_int64, C.c_int)
_CB_POS = C.CFUNCTYPE(C.c_int, C.c_void_p, C.c_int64)


_CB_DRAFT_TREE = C.CFUNCTYPE(C.c_int, C.c_void_p, C.c_int32, C.c_int64, C.c_int, C.POINTER(C.c_int32), C.POINTER(C.c_int32))
_CB_VERIFY_TREE = C.CFUNCTYPE(C.c_int, C.c_void_p, C.POINTER(C.c_int32), C.POINTER(C.c_int32), C.c_int, C.c_int64,
                              C.POINTER(C.c_uint16))
_CB_COMPACT = C.CFUNCTYPE(C.c_int, C.c_void_p, C.c_int64, C.POINTER(C.c_uint32), C.c_int)


class Producer(C.Structure):
    _fields_ = [("user", C.c_void_p), ("reset", _CB_I), ("produce", _CB_PRODUCE), ("prefill", _CB_TOKPOS),
                ("verify", _CB_VERIFY), ("rollback_retaining", _CB_ROLL), ("prime", _CB_TOKPOS),
                ("step", _CB_PRODUCE), ("rewind", _CB_POS), ("tree_nodes", C.c_int),
                ("draft_tree", _CB_DRAFT_TREE), ("verify_tree", _CB_VERIFY_TREE), ("compact_tree", _CB_COMPACT)]


class Generation(C.Structure):
    _fields_ = [("shaping", Shaping), ("max_new_tokens", C.c_uint64), ("stop_tokens", C.POINTER(C.c_int32)),
                ("n_stop", C.c_int32), ("block", C.c_int32), ("adaptive_floor", C.c_int32)]


class GenerationResult(C.Structure):
    _fields_ = [("tokens", C.POINTER(C.c_int32)), ("n_tokens", C.c_int64), ("stop_reason", C.c_int32),
                ("final_depth", C.c_int32), ("rounds", C.c_int64), ("offered", C.c_int64),
                ("accepted", C.c_int64), ("rollbacks", C.c_int64), ("draw_step", C.c_uint64)]


def run_speculative(target, drafter, prompt, cfg, max_new_tokens, block, vocab, max_context,
                    stop_tokens=(), adaptive_floor=0):
    """The reference loop over Python producers.  `target` offers reset(), produce(token, pos) ->
    uint16[vocab], prefill(token, pos), verify(feed, base) -> uint16[m, vocab],
    rollback_retaining(point, keep_rows); `drafter` offers prime(next, pos), step(token, pos) ->
    uint16[vocab], rewind(pos).  A drafter with `tree_nodes` > 0 also offers draft_tree(anchor, base,
    nodes) -> (node parents, tokens), and the target then verify_tree(feed, slot_parents, base) and
    compact_tree(base, path)."""
    def put(dst, arr, n):
        C.memmove(dst, np.ascontiguousarray(arr, np.uint16).ctypes.data, n * 2)

    def guard(fn):
        def inner(*a):
            try:
                fn(*a)
                return 0
            except Exception as e:  # an exception cannot cross the C frame
                errs.append(e)
                return 1
        return inner

    errs = []
    cbs = dict(
        reset=_CB_I(guard(lambda u: target.reset())),
        produce=_CB_PRODUCE(guard(lambda u, t, p, out: put(out, target.produce(t, p), vocab))),
        prefill=_CB_TOKPOS(guard(lambda u, t, p: target.prefill(t, p))),
        verify=_CB_VERIFY(guard(lambda u, f, m, b, out: put(out, target.verify([f[i] for i in range(m)], b), m * vocab))),
        rollback_retaining=_CB_ROLL(guard(lambda u, pt, k: target.rollback_retaining(pt, k))),
        prime=_CB_TOKPOS(guard(lambda u, t, p: drafter.prime(t, p))),
        step=_CB_PRODUCE(guard(lambda u, t, p, out: put(out, drafter.step(t, p), vocab))),
        rewind=_CB_POS(guard(lambda u, p: drafter.rewind(p))),
    )
    prod = Producer(None, *[cbs[k] for k in ("reset", "produce", "prefill", "verify", "rollback_retaining",
                                             "prime", "step", "rewind")])
    if getattr(drafter, "tree_nodes", 0):  # a drafter that offers trees (producer.rs:253-294)
        def draft_tree(u, anchor, base, nodes, parent_out, tokens_out):
            parent, tokens = drafter.draft_tree(anchor, base, nodes)
            assert len(parent) == len(tokens) == nodes
            for i in range(nodes):
                parent_out[i], tokens_out[i] = int(parent[i]), int(tokens[i])

        cbs["draft_tree"] = _CB_DRAFT_TREE(guard(draft_tree))
        cbs["verify_tree"] = _CB_VERIFY_TREE(guard(lambda u, f, par, m, b, out: put(
            out, target.verify_tree([f[i] for i in range(m)], [par[i] for i in range(m)], b), m * vocab)))
        cbs["compact_tree"] = _CB_COMPACT(guard(lambda u, b, path, n: target.compact_tree(b, [path[i] for i in range(n)])))
        prod.tree_nodes = int(drafter.tree_nodes)
        prod.draft_tree, prod.verify_tree, prod.compact_tree = cbs["draft_tree"], cbs["verify_tree"], cbs["compact_tree"]
    g = Generation()
    g.shaping = cfg
    g.max_new_tokens = max_new_tokens
    st = np.ascontiguousarray(list(stop_tokens), np.int32)
    g.stop_tokens = st.ctypes.data_as(C.POINTER(C.c_int32))
    g.n_stop = st.size
    g.block = block
    g.adaptive_floor = adaptive_floor
    toks = np.zeros(max_new_tokens + 1, np.int32)
    res = GenerationResult()
    res.tokens = toks.ctypes.data_as(C.POINTER(C.c_int32))
    pr = np.ascontiguousarray(prompt, np.int32)
    rc = lib().tso_run_speculative(C.byref(prod), _p(pr), C.c_int64(pr.size), C.byref(g), C.c_int64(max_context),
                                   C.c_int64(vocab), C.byref(res))
    if errs:
        raise errs[0]
    if rc < 0:
        raise ValueError(f"run_speculative failed ({rc}): {last_error()}")
    return dict(tokens=[int(t) for t in toks[: res.n_tokens]], stop_reason=res.stop_reason, rounds=res.rounds,
                offered=res.offered, accepted=res.accepted, rollbacks=res.rollbacks, draw_step=res.draw_step,
                final_depth=res.final_depth)
