"""Host-side mirror of the reference's producer traits for the verify path.

`HipVerifier` carries the method names and argument meaning of `LogitProducer` and
`SpeculativeProducer` (crates/runtime/src/producer.rs:17-104,164-387) over the C ABI of
libtsverify.so.  Errors surface as `TsvError` carrying the engine's message (the reference
returns `Result<(), String>`).
"""
import ctypes as C
from dataclasses import dataclass, field
from typing import List, Optional

import numpy as np

from . import ffi


@dataclass
class RoundResult:
    accepted: int
    committed: int
    next: int
    stopped: int
    draw_step: int
    path: List[int] = field(default_factory=list)
    kv_position: int = 0
    min_margin: float = 1.0


def _i32(a):
    return np.ascontiguousarray(a, np.int32)


def parse_kv_bits(text):
    """`--kv-bits` as crates/model-io/src/kv_quant.rs:48-72 reads it: "off" -> None, "2" / "3" / "4" -> the same
    width on both sides, "3.5" -> 3 bits for keys and 4 for values."""
    table = {"off": None, "2": (2, 2), "3": (3, 3), "3.5": (3, 4), "4": (4, 4)}
    if text not in table:
        raise ValueError(f"--kv-bits must be one of off|2|3|3.5|4, got {text!r}")
    return table[text]


def model_desc(cfg, weights, kv_bits=None, session_slots=1, shared_tables=False):
    """(tsv_model_desc, what must stay alive while it is used) for a weight dictionary; `shared_tables` leaves the
    embedding table and the output head empty (a drafter head takes the target's)."""
    n = len(weights["layers"])
    layers = (ffi.Layer * n)()
    for i, lw in enumerate(weights["layers"]):
        for name in ffi.LAYER_TENSORS + ffi.LAYER_MOE_TENSORS + ffi.LAYER_GPTOSS_TENSORS:
            setattr(layers[i], name, ffi.tensor(lw.get(name)))
        layers[i].n_experts = int(lw.get("n_experts", 0))
        layers[i].top_k = int(lw.get("top_k", 0))
        layers[i].window = int(lw.get("window", 0))
        layers[i].ring = int(bool(lw.get("ring", 0)))
    d = ffi.ModelDesc()
    d.n_layers = n
    for key in ("hidden", "n_q_heads", "n_kv_heads", "head_dim", "ffn", "vocab", "max_context"):
        setattr(d, key, cfg[key])
    d.rms_eps = cfg.get("rms_eps", 1e-5)
    d.rope_theta = cfg.get("rope_theta", 10000.0)
    d.attn_scale = cfg.get("attn_scale", 0.0)
    factors = freqs = None
    if cfg.get("rope_factors") is not None:
        factors = np.ascontiguousarray(cfg["rope_factors"], np.float32)
        d.rope_factors = factors.ctypes.data_as(C.POINTER(C.c_float))
    if cfg.get("rope_freqs") is not None:
        freqs = np.ascontiguousarray(cfg["rope_freqs"], np.float32)
        d.rope_freqs = freqs.ctypes.data_as(C.POINTER(C.c_float))
    d.rope_mscale = cfg.get("rope_mscale", 0.0)
    d.act_alpha = cfg.get("act_alpha", 0.0)
    d.act_limit = cfg.get("act_limit", 0.0)
    d.kv_k_bits, d.kv_v_bits = kv_bits if kv_bits else (0, 0)
    d.session_slots = int(session_slots)
    if not shared_tables:
        d.embed = ffi.tensor(weights["embed"])
        d.lm_head = ffi.tensor(weights.get("lm_head"))
    d.final_norm = ffi.tensor(weights["final_norm"])
    d.layers = C.cast(layers, C.POINTER(ffi.Layer))
    return d, (weights, layers, factors, freqs)


class MtpHead:
    """The drafter head that predicts one token further from the target's own state (docs/MTP.md:53-60,
    crates/runtime/src/families/qwen/mtp.rs), resident beside a HipVerifier and attached to it: one decoder
    layer with a cache of its own, fc over [norm(embedding of the next token); norm(target's final state)],
    the target's embedding table and output head.  `weights`: a one-layer weight dictionary (final_norm the
    head's own norm) with the extra keys fc, norm_embedding, norm_hidden.  Close it before the target."""

    def __init__(self, target, cfg, weights):
        md = ffi.MtpDesc()
        md.model, self._keep = model_desc(cfg, weights, shared_tables=True)
        md.fc = ffi.tensor(weights["fc"])
        md.norm_embedding = ffi.tensor(weights["norm_embedding"])
        md.norm_hidden = ffi.tensor(weights["norm_hidden"])
        h = C.c_void_p()
        ffi.check(ffi.lib().tsv_mtp_open(target._h, C.byref(md), C.byref(h)))
        self._h = h
        self.target = target
        self.vocab = target.vocab
        self.cfg = dict(cfg)

    def close(self):
        if getattr(self, "_h", None):
            ffi.lib().tsv_close(self._h)
            self._h = None

    def __del__(self):
        self.close()

    @property
    def position(self):
        return int(ffi.lib().tsv_kv_position(self._h))

    def step(self, next_token, position):
        """mtp_draft_step: the head's logits (uint16[vocab] fp16 bits) for the token after `next_token`."""
        out = np.empty(self.vocab, np.uint16)
        ffi.check(ffi.lib().tsv_mtp_step(self._h, int(next_token), int(position), out.ctypes.data, 0))
        return out

    def step_device(self, next_token, position, address):
        ffi.check(ffi.lib().tsv_mtp_step(self._h, int(next_token), int(position), C.c_void_p(address), 1))

    def prime(self, next_token, position):
        """mtp_prime_step: the cache row alone."""
        ffi.check(ffi.lib().tsv_mtp_step(self._h, int(next_token), int(position), None, 0))

    def rewind(self, position):
        ffi.check(ffi.lib().tsv_mtp_rewind(self._h, int(position)))

    def context_position(self):
        return self.position

    def prefill_chunk(self, tokens, start_position, next_token=None, want_logits=True):
        """The target's prefill of the chunk, priming the head over every position whose next token is known."""
        ids = _i32(tokens)
        out = np.empty(self.vocab, np.uint16) if want_logits else None
        ffi.check(ffi.lib().tsv_mtp_prefill_chunk(self._h, ids.ctypes.data, ids.size, int(start_position),
                                                  out.ctypes.data if want_logits else None,
                                                  -1 if next_token is None else int(next_token)))
        return out

    def draft_block(self, anchor, base, block):
        """`block` greedy proposals chained on the device; the head then stands at base + block."""
        out = np.empty(int(block), np.int32)
        ffi.check(ffi.lib().tsv_mtp_draft_block(self._h, int(anchor), int(base), int(block), out.ctypes.data))
        return [int(t) for t in out]

    def read_kv(self, pos0, n):
        return HipVerifier.read_kv(self, 0, pos0, n)


class HipVerifier:
    """One target model resident on the GPU with its KV cache: fp16 rows, or TurboQuant rows on the layers
    crates/model-io/src/kv_quant.rs:102-107 names when kv_bits = (key bits, value bits) is given
    (RealForwardRunner::open_with_kv_quant, crates/runtime/src/real_forward_api.rs:568-590)."""

    def __init__(self, cfg, weights, kv_bits=None, session_slots=1):
        self.cfg = dict(cfg)
        d, self._keep = model_desc(cfg, weights, kv_bits, session_slots)
        self.kv_bits = tuple(kv_bits) if kv_bits else None
        h = C.c_void_p()
        ffi.check(ffi.lib().tsv_open(C.byref(d), C.byref(h)))
        self._h = h
        self.vocab = cfg["vocab"]

    @classmethod
    def from_gguf(cls, path, max_context=0):
        """Opens a llama-family GGUF file (llama, qwen2, qwen3, qwen3moe) as the target; the sizes
        come from the file's metadata.  max_context 0: the file's context_length."""
        import os
        self = cls.__new__(cls)
        h = C.c_void_p()
        ffi.check(ffi.lib().tsv_open_gguf(os.fsencode(path), int(max_context), C.byref(h)))
        self._h = h
        self._keep = None
        self.kv_bits = None
        self.vocab = int(ffi.lib().tsv_vocab(h))
        g = ffi.Gguf(path)
        arch = g.string("general.architecture")
        heads = int(g.number(arch + ".attention.head_count"))
        hidden = int(g.number(arch + ".embedding_length"))

        def opt(key, default):
            try:
                return g.number(arch + "." + key)
            except ffi.TsvError:
                return default
        self.cfg = dict(n_layers=int(g.number(arch + ".block_count")), hidden=hidden, n_q_heads=heads,
                        n_kv_heads=int(opt("attention.head_count_kv", heads)),
                        head_dim=int(opt("attention.key_length", hidden // heads)), vocab=self.vocab,
                        max_context=int(ffi.lib().tsv_max_context(h)))
        g.close()
        return self

    def close(self):
        if getattr(self, "_h", None):
            ffi.lib().tsv_close(self._h)
            self._h = None

    def __del__(self):
        self.close()

    # ---- LogitProducer ----------------------------------------------------------------
    @property
    def session_pool_size(self):
        """Conversations whose KV state the handle keeps, the live one included (RealForwardRunner::session_pool_size)."""
        return int(ffi.lib().tsv_session_pool_size(self._h))

    @property
    def session_slot_evicted(self):
        """Whether the last reset overwrote a parked conversation."""
        return bool(ffi.lib().tsv_session_slot_evicted(self._h))

    def reset(self):
        ffi.check(ffi.lib().tsv_reset(self._h))

    @property
    def position(self):
        return ffi.lib().tsv_kv_position(self._h)

    @property
    def device_logits(self):
        """Device address of the logits the last pass left on the GPU (rows x vocab fp16)."""
        return ffi.lib().tsv_device_logits(self._h)

    def max_safe_rewind(self):
        """`KvCacheManager::max_safe_rewind`: rows a rollback may drop; 2**63 - 1 when no layer keeps a ring."""
        return ffi.lib().tsv_max_safe_rewind(self._h)

    @property
    def stream(self):
        """The hipStream_t (as an integer) every kernel of this handle runs on."""
        return ffi.lib().tsv_stream(self._h)

    def produce(self, token, position):
        out = np.empty(self.vocab, np.uint16)
        ffi.check(ffi.lib().tsv_produce(self._h, int(token), int(position), out.ctypes.data))
        return out

    def prefill(self, ids, pos0=0, want_logits=True):
        ids = _i32(ids)
        out = np.empty(self.vocab, np.uint16) if want_logits else None
        ffi.check(ffi.lib().tsv_prefill(self._h, ids.ctypes.data, ids.size, int(pos0),
                                        out.ctypes.data if want_logits else None))
        return out

    # ---- SpeculativeProducer ----------------------------------------------------------
    # ---- prefix reuse (LogitProducer::try_reuse_prefix, SpeculativeProducer::record_committed) ----
    def set_prefix_reuse(self, on):
        """RealForwardRunner::set_prefix_reuse: reuse answers 0 until the host opts in."""
        ffi.check(ffi.lib().tsv_set_prefix_reuse(self._h, int(bool(on))))

    def try_reuse_prefix(self, prompt_ids):
        """producer.rs:24-47: commits to continuing from the current state for the leading N tokens
        of the prompt (moving the cursor back to them when it ran past) and returns N; 0 = reset."""
        p = _i32(prompt_ids)
        n = ffi.lib().tsv_try_reuse_prefix(self._h, p.ctypes.data, p.size)
        if n < 0:
            raise ffi.TsvError(-1, ffi.last_error())
        return int(n)

    def record_committed(self, tokens, pos0):
        """producer.rs:322-330: the rows of a verify pass that the round committed."""
        t = _i32(tokens)
        ffi.check(ffi.lib().tsv_record_committed(self._h, t.ctypes.data, t.size, int(pos0)))

    def prefix_len(self):
        """Positions the record describes; None when tainted."""
        n = ffi.lib().tsv_prefix_len(self._h)
        return None if n < 0 else int(n)

    def checkpoint(self):
        p = ffi.Point()
        ffi.check(ffi.lib().tsv_checkpoint(self._h, C.byref(p)))
        return p

    def rollback(self, point):
        ffi.check(ffi.lib().tsv_rollback(self._h, C.byref(point)))

    def supports_retaining_rollback(self):
        return True

    def rollback_retaining(self, point, keep_rows):
        ffi.check(ffi.lib().tsv_rollback_retaining(self._h, C.byref(point), int(keep_rows)))

    def commit_pending(self, keep_rows):
        ffi.check(ffi.lib().tsv_commit_pending(self._h, int(keep_rows)))

    def discard_pending(self):
        ffi.check(ffi.lib().tsv_discard_pending(self._h))

    def verify(self, feed, base, want_logits=True):
        feed = _i32(feed)
        out = np.empty((feed.size, self.vocab), np.uint16) if want_logits else None
        ffi.check(ffi.lib().tsv_verify(self._h, feed.ctypes.data, feed.size, int(base),
                                       out.ctypes.data if want_logits else None))
        return out

    def verify_tree(self, feed, parent, base, want_logits=True):
        feed, parent = _i32(feed), _i32(parent)
        out = np.empty((feed.size, self.vocab), np.uint16) if want_logits else None
        ffi.check(ffi.lib().tsv_verify_tree(self._h, feed.ctypes.data, parent.ctypes.data, feed.size,
                                            int(base), out.ctypes.data if want_logits else None))
        return out

    def compact_tree(self, base, path):
        p = np.ascontiguousarray(path, np.uint32)
        ffi.check(ffi.lib().tsv_compact_tree(self._h, int(base), p.ctypes.data, p.size))

    # ---- device-side acceptance -----------------------------------------------------------
    def _round(self, feed, base, cfg, parent, draft_logits, draw_step, stop_tokens, generated,
               max_new_tokens, want_logits, history=None):
        keep = {}
        r = ffi.Round()
        if history is not None and len(history):
            keep["history"] = _i32(history)
            r.history = keep["history"].ctypes.data_as(C.POINTER(C.c_int32))
            r.n_history = keep["history"].size
        keep["feed"] = _i32(feed)
        r.feed = keep["feed"].ctypes.data_as(C.POINTER(C.c_int32))
        r.m = keep["feed"].size
        if parent is not None:
            keep["parent"] = _i32(parent)
            r.parent = keep["parent"].ctypes.data_as(C.POINTER(C.c_int32))
        r.base = int(base)
        r.shaping = cfg
        if draft_logits is not None:
            if isinstance(draft_logits, int):
                r.draft_logits = draft_logits  # a device pointer
            else:
                a = np.asarray(draft_logits)
                if a.dtype != np.uint16:
                    a = a.astype(np.float16).view(np.uint16)
                keep["draft"] = np.ascontiguousarray(a)
                r.draft_logits = keep["draft"].ctypes.data
        r.draw_step = int(draw_step)
        if stop_tokens is not None and len(stop_tokens):
            keep["stop"] = _i32(stop_tokens)
            r.stop_tokens = keep["stop"].ctypes.data_as(C.POINTER(C.c_int32))
            r.n_stop = keep["stop"].size
        r.generated = int(generated)
        r.max_new_tokens = int(max_new_tokens)
        if want_logits:
            keep["logits"] = np.empty((r.m, self.vocab), np.uint16)
            r.logits_out = keep["logits"].ctypes.data
        return r, keep

    @staticmethod
    def _result(c):
        return RoundResult(c.accepted, c.committed, c.next, c.stopped, c.draw_step,
                           list(c.path[: c.path_len]), c.kv_position, c.min_margin)

    def accept(self, feed, base, cfg, parent=None, draft_logits=None, draw_step=0, stop_tokens=None,
               generated=0, max_new_tokens=0, history=None):
        """Acceptance + truncation over the logits the last verify left on the device.  `history`
        (the sink's tokens when the round starts) is what the penalties of `cfg` look at."""
        r, keep = self._round(feed, base, cfg, parent, draft_logits, draw_step, stop_tokens, generated,
                              max_new_tokens, False, history)
        out = ffi.RoundResultC()
        ffi.check(ffi.lib().tsv_accept(self._h, C.byref(r), C.byref(out)))
        return self._result(out)

    def verify_accept(self, feed, base, cfg, parent=None, draft_logits=None, draw_step=0,
                      stop_tokens=None, generated=0, max_new_tokens=0, want_logits=False, history=None):
        """The whole verify step: target forward, acceptance, KV truncation."""
        r, keep = self._round(feed, base, cfg, parent, draft_logits, draw_step, stop_tokens, generated,
                              max_new_tokens, want_logits, history)
        out = ffi.RoundResultC()
        ffi.check(ffi.lib().tsv_verify_accept(self._h, C.byref(r), C.byref(out)))
        res = self._result(out)
        return (res, keep["logits"]) if want_logits else res

    def draft_chain(self, draft_logits, cfg, draw_step=0, history=None, generated=0):
        """Draw the k proposals of a chain round from the drafter's rows; returns (proposals, draw_step).
        `history` / `generated`: the sink's state, read by the penalties of `cfg`."""
        if isinstance(draft_logits, tuple):  # (device pointer, k)
            ptr, k = draft_logits
        else:
            a = np.asarray(draft_logits)
            if a.dtype != np.uint16:
                a = a.astype(np.float16).view(np.uint16)
            a = np.ascontiguousarray(a)
            ptr, k = a.ctypes.data, a.shape[0]
        ds = C.c_uint64(int(draw_step))
        props = np.empty(k, np.int32)
        hist = _i32(history) if history is not None and len(history) else None
        ffi.check(ffi.lib().tsv_draft_chain(self._h, ptr, k, C.byref(cfg), C.byref(ds), props.ctypes.data,
                                            hist.ctypes.data if hist is not None else None,
                                            hist.size if hist is not None else 0, int(generated)))
        return props, ds.value

    # ---- the generation loop --------------------------------------------------------------
    def run_speculative(self, prompt, drafter, cfg, max_new_tokens, block, stop_tokens=(), adaptive_floor=0,
                        device_logits=False, block_drafts=True, chunked_prefill=True):
        """`run_speculative` (crates/runtime/src/speculative.rs:194-900) for a step-wise drafter and
        chain rounds, acceptance and truncation on the device.  `drafter` offers prime(next, pos),
        step(token, pos) -> uint16[vocab] and rewind(pos); with `device_logits` it offers
        step_device(token, pos, device_address) instead and fills vocab fp16 values there on the GPU.
        Returns a dict with the reported tokens, the stop reason (1 stop token, 2 budget) and the
        round statistics."""
        vocab = self.vocab
        failure = []

        def guard(fn):
            def inner(*a):
                try:
                    fn(*a)
                    return 0
                except Exception as e:  # an exception cannot cross the C frame
                    failure.append(e)
                    return 1
            return inner

        def step(user, token, pos, out):
            if device_logits:
                drafter.step_device(token, pos, C.cast(out, C.c_void_p).value)
                return
            row = np.ascontiguousarray(drafter.step(token, pos), np.uint16)
            C.memmove(out, row.ctypes.data, vocab * 2)

        if isinstance(drafter, MtpHead):
            # the library's own callbacks; `block_drafts` / `chunked_prefill` False hand the loop a drafter
            # without that callback (the step-wise walk of the same head)
            d = ffi.Drafter()
            ffi.check(ffi.lib().tsv_mtp_drafter(drafter._h, C.byref(d)))
            if not block_drafts:
                d.draft_block = ffi.DRAFT_BLOCK()
            if not chunked_prefill:
                d.prefill_chunk = ffi.DRAFT_PREFILL_CHUNK()
            drafter = None
        else:
            d = ffi.Drafter(None, ffi.DRAFT_PRIME(guard(lambda u, t, p: drafter.prime(t, p))),
                            ffi.DRAFT_STEP(guard(step)), ffi.DRAFT_REWIND(guard(lambda u, p: drafter.rewind(p))),
                            1 if device_logits else 0)
        if hasattr(drafter, "draft_block"):  # a block drafter: draft_block(anchor, base, block) -> tokens
            def draft_block(user, anchor, base, block, out):
                try:
                    toks = drafter.draft_block(anchor, base, block)
                    for i in range(min(len(toks), block)):  # (a short answer is the loop's to refuse)
                        out[i] = int(toks[i])
                    return 0 if len(toks) == block else 1
                except Exception as e:
                    failure.append(e)
                    return 1
            d.draft_block = ffi.DRAFT_BLOCK(draft_block)
        if hasattr(drafter, "prefill_chunk"):  # prefill_chunk(tokens, start, next_token or None) -> uint16[vocab]
            def prefill_chunk(user, tokens, n, start, out, next_token):
                try:
                    row = drafter.prefill_chunk([int(tokens[i]) for i in range(n)], int(start),
                                                None if next_token < 0 else int(next_token))
                    row = np.ascontiguousarray(row, np.uint16)
                    C.memmove(out, row.ctypes.data, vocab * 2)
                    return 0
                except Exception as e:
                    failure.append(e)
                    return 1
            d.prefill_chunk = ffi.DRAFT_PREFILL_CHUNK(prefill_chunk)
        if hasattr(drafter, "context_position"):  # lets the loop take over a prefix (the continuity guard)
            def where(user):
                try:
                    return int(drafter.context_position())
                except Exception as e:
                    failure.append(e)
                    return -1
            d.position = ffi.DRAFT_POSITION(where)
        if getattr(drafter, "tree_nodes", 0):  # a drafter that offers trees: draft_tree(anchor, base, nodes) -> (parents, tokens)
            def draft_tree(user, anchor, base, nodes, parent_out, tokens_out):
                try:
                    parent, tokens = drafter.draft_tree(anchor, base, nodes)
                    assert len(parent) == len(tokens) == nodes
                    for i in range(nodes):
                        parent_out[i], tokens_out[i] = int(parent[i]), int(tokens[i])
                    return 0
                except Exception as e:
                    failure.append(e)
                    return 1
            d.tree_nodes = int(drafter.tree_nodes)
            d.draft_tree = ffi.DRAFT_TREE(draft_tree)
        g = ffi.Generation()
        g.shaping = cfg
        g.max_new_tokens = int(max_new_tokens)
        st = _i32(list(stop_tokens))
        g.stop_tokens = st.ctypes.data_as(C.POINTER(C.c_int32))
        g.n_stop = st.size
        g.block = int(block)
        g.adaptive_floor = int(adaptive_floor)
        toks = np.zeros(int(max_new_tokens) + 1, np.int32)
        res = ffi.GenerationResult()
        res.tokens = toks.ctypes.data_as(C.POINTER(C.c_int32))
        res.capacity = toks.size
        pr = _i32(prompt)
        rc = ffi.lib().tsv_run_speculative(self._h, C.byref(d), pr.ctypes.data, pr.size, C.byref(g), C.byref(res))
        if failure:
            raise failure[0]
        ffi.check(rc)
        return dict(tokens=[int(t) for t in toks[: res.n_tokens]], stop_reason=res.stop_reason, rounds=res.rounds,
                    offered=res.offered, accepted=res.accepted, rollbacks=res.rollbacks, draw_step=res.draw_step,
                    final_depth=res.final_depth, kv_position=res.kv_position, min_margin=res.min_margin,
                    reused=res.reused)

    PROFILE_CLASSES = ("embed", "norm", "qkv", "rope_kv", "attention", "wo", "gate_up", "down", "head", "accept",
                       "event_pair")

    def set_profile(self, on):
        ffi.check(ffi.lib().tsv_set_profile(self._h, int(bool(on))))

    def set_repeat(self, profile_class, times):
        """Launch the kernels of one class `times` times in a row per pass (measurement hook)."""
        ffi.check(ffi.lib().tsv_set_repeat(self._h, self.PROFILE_CLASSES.index(profile_class), int(times)))

    def get_profile(self):
        """{class: (total ms, launches)} since the last call (HIP events around every launch)."""
        n = len(self.PROFILE_CLASSES)
        ms = np.zeros(n, np.float32)
        cnt = np.zeros(n, np.int32)
        ffi.check(ffi.lib().tsv_get_profile(self._h, ms.ctypes.data, cnt.ctypes.data, n))
        return {k: (float(ms[i]), int(cnt[i])) for i, k in enumerate(self.PROFILE_CLASSES)}

    # ---- test introspection ------------------------------------------------------------------
    def write_kv(self, layer, pos0, k, v):
        """k, v: [n, n_kv_heads, head_dim] (rounded to fp16) stored at cache positions pos0.."""
        k16 = np.ascontiguousarray(np.asarray(k).astype(np.float16))
        v16 = np.ascontiguousarray(np.asarray(v).astype(np.float16))
        ffi.check(ffi.lib().tsv_write_kv(self._h, layer, int(pos0), k16.shape[0], k16.ctypes.data, v16.ctypes.data))

    def write_logits(self, logits, base):
        """logits [m, vocab] (uint16 fp16 bits, or floats rounded to fp16) become what `accept` judges."""
        a = np.asarray(logits)
        if a.dtype != np.uint16:
            a = a.astype(np.float16).view(np.uint16)
        a = np.ascontiguousarray(a)
        ffi.check(ffi.lib().tsv_write_logits(self._h, a.ctypes.data, a.shape[0], int(base)))

    def route_selected(self):
        """[n_layers, 16, 8] expert ids every row of the last pass chose per routed layer, rank order
        (the first top_k entries of a row are valid)."""
        n = len(self._layers) if getattr(self, "_layers", None) is not None else self.cfg["n_layers"]
        out = np.zeros((n, 16, 8), np.int32)
        ffi.check(ffi.lib().tsv_route_selected(self._h, out.ctypes.data, n))
        return out

    def force_route(self, sel):
        """Test hook: the routed layers take the experts of `sel` ([n_layers, 16, 8], a row whose first entry
        is negative routes freely) instead of each row's own top-k; None restores free routing."""
        n = self.cfg["n_layers"]
        if sel is None:
            ffi.check(ffi.lib().tsv_force_route(self._h, None, n))
            return
        a = np.ascontiguousarray(np.asarray(sel, np.int32))
        assert a.shape == (n, 16, 8), a.shape
        ffi.check(ffi.lib().tsv_force_route(self._h, a.ctypes.data, n))

    def read_kv_quantized(self, layer, pos0, n):
        """The stored rows of a quantized layer: (K rows, V rows), each [n, kv heads, 1 + words] u32, norm bits first."""
        c = self.cfg
        kb, vb = self.kv_bits
        k = np.zeros((n, c["n_kv_heads"], 1 + ffi.packed_words(c["head_dim"], kb)), np.uint32)
        v = np.zeros((n, c["n_kv_heads"], 1 + ffi.packed_words(c["head_dim"], vb)), np.uint32)
        ffi.check(ffi.lib().tsv_read_kv_quantized(self._h, layer, int(pos0), int(n), k.ctypes.data, v.ctypes.data))
        return k, v

    def read_kv(self, layer, pos0, n):
        c = self.cfg
        shape = (n, c["n_kv_heads"], c["head_dim"])
        k = np.empty(shape, np.float16)
        v = np.empty(shape, np.float16)
        ffi.check(ffi.lib().tsv_read_kv(self._h, layer, int(pos0), int(n), k.ctypes.data, v.ctypes.data))
        return k, v
