"""A GGUF version-3 writer for tests: metadata, tensor table and aligned data region as the public
format lays them out (and crates/repack/src/gguf_header/parser.rs:124-239 reads them)."""
import struct

import numpy as np

TYPE_IDS = {"u8": 0, "i8": 1, "u16": 2, "i16": 3, "u32": 4, "i32": 5, "f32": 6, "bool": 7, "str": 8, "arr": 9,
            "u64": 10, "i64": 11, "f64": 12}
PACK = {"u8": "<B", "i8": "<b", "u16": "<H", "i16": "<h", "u32": "<I", "i32": "<i", "f32": "<f", "bool": "<B",
        "u64": "<Q", "i64": "<q", "f64": "<d"}


def _string(s):
    b = s.encode()
    return struct.pack("<Q", len(b)) + b


def _value(kind, v):
    if kind == "str":
        return _string(v)
    if kind == "arr":
        ek, items = v
        return struct.pack("<IQ", TYPE_IDS[ek], len(items)) + b"".join(_value(ek, x) for x in items)
    return struct.pack(PACK[kind], v)


def write_gguf(path, meta, tensors, alignment=None, version=3, magic=b"GGUF", misalign=None):
    """meta: [(key, kind, value)]; tensors: [(name, dims in ggml order, ggml type id, bytes)].
    `alignment` adds general.alignment; `misalign` names a tensor whose offset is pushed off the grid."""
    meta = list(meta)
    if alignment is not None:
        meta.append(("general.alignment", "u32", alignment))
    al = alignment or 32
    head = magic + struct.pack("<IQQ", version, len(tensors), len(meta))
    for key, kind, v in meta:
        head += _string(key) + struct.pack("<I", TYPE_IDS[kind]) + _value(kind, v)
    offsets, pos = [], 0
    for name, dims, tid, raw in tensors:
        pos = (pos + al - 1) // al * al
        offsets.append(pos + (4 if name == misalign else 0))
        pos += len(raw)
    for (name, dims, tid, raw), off in zip(tensors, offsets):
        head += _string(name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims)
        head += struct.pack("<IQ", tid, off)
    start = (len(head) + al - 1) // al * al
    with open(path, "wb") as f:
        f.write(head + b"\0" * (start - len(head)))
        for (name, dims, tid, raw), off in zip(tensors, offsets):
            f.seek(start + off)
            f.write(raw)
    return start


def permute_rotary_rows(raw, head_dim):
    """What llama.cpp's converter does to q / k: each head's rows go from (2, D/2) to (D/2, 2), so
    GGUF row j holds the original row (j % 2) * (D/2) + j // 2 (conventions.rs:133-143)."""
    rows = raw.shape[0]
    j = np.arange(rows)
    i = j % head_dim
    return raw[j - i + (i % 2) * (head_dim // 2) + i // 2]


def llama_gguf(path, cfg, weights, arch="llama", permute=True):
    """The synthetic weights of tests as the GGUF a converter would have written."""
    H, hd = cfg["hidden"], cfg["head_dim"]
    E = int(cfg.get("n_experts", 0))
    meta = [("general.architecture", "str", arch), (f"{arch}.block_count", "u32", len(weights["layers"])),
            (f"{arch}.embedding_length", "u32", H), (f"{arch}.attention.head_count", "u32", cfg["n_q_heads"]),
            (f"{arch}.attention.head_count_kv", "u32", cfg["n_kv_heads"]), (f"{arch}.attention.key_length", "u32", hd),
            (f"{arch}.attention.layer_norm_rms_epsilon", "f32", cfg.get("rms_eps", 1e-5)),
            (f"{arch}.rope.freq_base", "f32", cfg.get("rope_theta", 10000.0)),
            (f"{arch}.context_length", "u32", cfg["max_context"]),
            ("tokenizer.ggml.tokens", "arr", ("str", ["<a>", "<b>", "c"])),   # an array the intake walks past
            ("tokenizer.ggml.scores", "arr", ("f32", [0.0, -1.0, -2.0]))]
    if E:
        meta += [(f"{arch}.expert_count", "u32", E), (f"{arch}.expert_used_count", "u32", cfg["top_k"]),
                 (f"{arch}.expert_feed_forward_length", "u32", cfg["ffn"])]
    else:
        meta.append((f"{arch}.feed_forward_length", "u32", cfg["ffn"]))
    oss = cfg.get("gptoss")
    if oss:
        factor, octx, bf, bs = oss["yarn"]
        meta += [(f"{arch}.attention.sliding_window", "u32", oss["window"]), (f"{arch}.rope.scaling.type", "str", "yarn"),
                 (f"{arch}.rope.scaling.factor", "f32", factor), (f"{arch}.rope.scaling.original_context_length", "u32", octx),
                 (f"{arch}.rope.scaling.yarn_beta_fast", "f32", bf), (f"{arch}.rope.scaling.yarn_beta_slow", "f32", bs)]
    out = []

    def add(name, t, rot=False, expert_rows=0):
        dtype, raw, rows, cols = t
        raw = np.ascontiguousarray(raw)
        if rot:
            raw = permute_rotary_rows(raw, hd)
        dims = [cols] if rows == 1 else [cols, rows]
        if expert_rows:
            dims = [cols, expert_rows, rows // expert_rows]
        out.append((name, dims, dtype, np.ascontiguousarray(raw).tobytes()))

    add("token_embd.weight", weights["embed"])
    add("output_norm.weight", weights["final_norm"])
    if weights.get("lm_head") is not None:
        add("output.weight", weights["lm_head"])
    if cfg.get("rope_factors") is not None:
        f = np.ascontiguousarray(cfg["rope_factors"], np.float32)
        out.append(("rope_freqs.weight", [f.size], 0, f.tobytes()))
    names = dict(attn_norm="attn_norm.weight", wv="attn_v.weight", wo="attn_output.weight", ffn_norm="ffn_norm.weight",
                 q_norm="attn_q_norm.weight", k_norm="attn_k_norm.weight", w_gate="ffn_gate.weight", w_up="ffn_up.weight",
                 w_down="ffn_down.weight", router="ffn_gate_inp.weight", bq="attn_q.bias", bk="attn_k.bias", bv="attn_v.bias",
                 bo="attn_output.bias", sinks="attn_sinks.weight", router_bias="ffn_gate_inp.bias")
    if oss:
        names["ffn_norm"] = "post_attention_norm.weight"
    for li, lw in enumerate(weights["layers"]):
        p = f"blk.{li}."
        add(p + "attn_q.weight", lw["wq"], rot=permute)
        add(p + "attn_k.weight", lw["wk"], rot=permute)
        for key, name in names.items():
            if lw.get(key) is not None:
                add(p + name, lw[key])
        if E:
            add(p + "ffn_gate_exps.weight", lw["we_gate"], expert_rows=cfg["ffn"])
            add(p + "ffn_up_exps.weight", lw["we_up"], expert_rows=cfg["ffn"])
            add(p + "ffn_down_exps.weight", lw["we_down"], expert_rows=H)
            for key, name in (("be_gate", "ffn_gate_exps.bias"), ("be_up", "ffn_up_exps.bias"), ("be_down", "ffn_down_exps.bias")):
                if lw.get(key) is not None:
                    add(p + name, lw[key])
    return write_gguf(path, meta, out)
