"""A GGUF version-3 reader in plain Python / numpy for the tests: header, metadata, tensor table,
aligned data region as the public format lays them out, the llama-family tensor names of
crates/repack/src/gguf_names/llama.rs:14-60 (`qwen2` biases :47-57) and gpt_oss.rs:30-72, and the
q / k row un-permutation of crates/repack/src/gguf_checkpoint/conventions.rs:133-151.  It shares no
code with the library's parser: it is what the oracle side of a GGUF parity test reads the file with."""
import struct

import numpy as np

_SCALAR = {0: "<B", 1: "<b", 2: "<H", 3: "<h", 4: "<I", 5: "<i", 6: "<f", 7: "<B", 10: "<Q", 11: "<q", 12: "<d"}
# bytes per block / elements per block of the ggml types a verify target uses
_BLOCK = {0: (4, 1), 1: (2, 1), 8: (34, 32), 12: (144, 256), 13: (176, 256), 14: (210, 256), 30: (2, 1), 39: (17, 32)}


class _Cursor:
    def __init__(self, data):
        self.d, self.p = data, 0

    def take(self, fmt):
        v = struct.unpack_from(fmt, self.d, self.p)[0]
        self.p += struct.calcsize(fmt)
        return v

    def string(self):
        n = self.take("<Q")
        s = bytes(self.d[self.p:self.p + n]).decode()
        self.p += n
        return s

    def value(self, kind):
        if kind == 8:
            return self.string()
        if kind == 9:
            ek, n = self.take("<I"), self.take("<Q")
            return [self.value(ek) for _ in range(n)]
        return self.take(_SCALAR[kind])


def read_gguf(path):
    """-> (metadata dict, {name: (ggml type, dims in ggml order, uint8 view of the tensor's bytes)})"""
    data = np.fromfile(path, np.uint8)
    c = _Cursor(memoryview(data))
    assert bytes(data[:4]) == b"GGUF"
    c.p = 4
    version, n_tensors, n_meta = c.take("<I"), c.take("<Q"), c.take("<Q")
    assert version == 3
    meta = {}
    for _ in range(n_meta):
        key = c.string()
        meta[key] = c.value(c.take("<I"))
    table = []
    for _ in range(n_tensors):
        name = c.string()
        nd = c.take("<I")
        dims = [c.take("<Q") for _ in range(nd)]
        table.append((name, dims, c.take("<I"), c.take("<Q")))
    align = int(meta.get("general.alignment", 32))
    start = (c.p + align - 1) // align * align
    tensors = {}
    for name, dims, tid, off in table:
        bb, be = _BLOCK[tid]
        rows = int(np.prod(dims[1:])) if len(dims) > 1 else 1
        nbytes = rows * (dims[0] // be) * bb
        tensors[name] = (tid, dims, data[start + off:start + off + nbytes])
    return meta, tensors


def _rows(entry):
    """(dtype, uint8 [rows, row bytes], rows, cols): every dimension past the first folds into the rows."""
    tid, dims, raw = entry
    bb, be = _BLOCK[tid]
    cols = int(dims[0])
    rows = int(np.prod(dims[1:])) if len(dims) > 1 else 1
    return (tid, np.ascontiguousarray(raw).reshape(rows, (cols // be) * bb), rows, cols)


def _unpermute(t, head_dim):
    """conventions.rs:133-151: install row i of a head is GGUF row (i % (D/2)) * 2 + i // (D/2)."""
    tid, raw, rows, cols = t
    i = np.arange(rows)
    h, r = i // head_dim * head_dim, i % head_dim
    return (tid, np.ascontiguousarray(raw[h + (r % (head_dim // 2)) * 2 + r // (head_dim // 2)]), rows, cols)


def load_model(path, max_context):
    """The configuration and weight dictionary the oracle model takes, read from a llama / qwen2 / qwen3 /
    qwen3moe / gpt-oss GGUF file."""
    from oracle import binding as ob
    meta, ts = read_gguf(path)
    arch = meta["general.architecture"]
    g = lambda key, default=None: meta.get(f"{arch}.{key}", default)
    heads = int(g("attention.head_count"))
    hidden = int(g("embedding_length"))
    n_layers = int(g("block_count"))
    hd = int(g("attention.key_length", hidden // heads))
    E = int(g("expert_count", 0))
    cfg = dict(n_layers=n_layers, hidden=hidden, n_q_heads=heads, n_kv_heads=int(g("attention.head_count_kv", heads)),
               head_dim=hd, ffn=int(g("expert_feed_forward_length" if E else "feed_forward_length")),
               vocab=_rows(ts["token_embd.weight"])[2], max_context=max_context,
               rms_eps=float(g("attention.layer_norm_rms_epsilon", 1e-5)), rope_theta=float(g("rope.freq_base", 10000.0)))
    oss = arch == "gpt-oss"
    if oss:
        assert g("rope.scaling.type") == "yarn"
        cfg["rope_freqs"], cfg["rope_mscale"] = ob.yarn_frequencies(
            hd, cfg["rope_theta"], float(g("rope.scaling.factor")), int(g("rope.scaling.original_context_length")),
            float(g("rope.scaling.yarn_beta_fast", 32.0)), float(g("rope.scaling.yarn_beta_slow", 1.0)))
        cfg.update(attn_scale=hd ** -0.5, act_alpha=1.702, act_limit=7.0)
    if "rope_freqs.weight" in ts:
        cfg["rope_factors"] = ts["rope_freqs.weight"][2].view(np.float32).copy()
    names = dict(attn_norm="attn_norm.weight", wv="attn_v.weight", wo="attn_output.weight",
                 ffn_norm="post_attention_norm.weight" if oss else "ffn_norm.weight",
                 q_norm="attn_q_norm.weight", k_norm="attn_k_norm.weight", w_gate="ffn_gate.weight", w_up="ffn_up.weight",
                 w_down="ffn_down.weight", router="ffn_gate_inp.weight", bq="attn_q.bias", bk="attn_k.bias", bv="attn_v.bias",
                 bo="attn_output.bias", sinks="attn_sinks.weight", router_bias="ffn_gate_inp.bias",
                 we_gate="ffn_gate_exps.weight", we_up="ffn_up_exps.weight", we_down="ffn_down_exps.weight",
                 be_gate="ffn_gate_exps.bias", be_up="ffn_up_exps.bias", be_down="ffn_down_exps.bias")
    layers = []
    for li in range(n_layers):
        p = f"blk.{li}."
        wq, wk = _rows(ts[p + "attn_q.weight"]), _rows(ts[p + "attn_k.weight"])
        if arch == "llama":   # only this architecture's converter permutes (conventions.rs:152-160)
            wq, wk = _unpermute(wq, hd), _unpermute(wk, hd)
        lw = dict(wq=wq, wk=wk)
        for key, name in names.items():
            if p + name in ts:
                lw[key] = _rows(ts[p + name])
        if E:
            lw.update(n_experts=E, top_k=int(g("expert_used_count")))
        if oss and li % 2 == 0:   # even layers slide (families/gptoss/attn.rs:20-23)
            lw["window"] = int(g("attention.sliding_window"))
        layers.append(lw)
    weights = dict(embed=_rows(ts["token_embd.weight"]), final_norm=_rows(ts["output_norm.weight"]), layers=layers)
    if "output.weight" in ts:
        weights["lm_head"] = _rows(ts["output.weight"])
    return cfg, weights
