"""Loads one of the reference's MLX known-answer language-model fixtures (copied as data
under tests/golden/lm/) into the weight dictionary the oracle model takes."""
import json
import os

import numpy as np
from safetensors.numpy import load_file

from oracle import binding as ob


def _t(a):
    a = np.ascontiguousarray(a, np.float32)
    if a.ndim == 1:
        a = a.reshape(1, -1)
    return (ob.F32, a.view(np.uint8).reshape(a.shape[0], -1), a.shape[0], a.shape[1])


def load(golden_dir, name, max_context=64):
    d = os.path.join(golden_dir, "lm", name)
    conf = json.load(open(os.path.join(d, "config.json")))
    traces = json.load(open(os.path.join(d, "traces.json")))
    st = load_file(os.path.join(d, "model.safetensors"))
    hidden = conf["hidden_size"]
    nq = conf["num_attention_heads"]
    hd = conf.get("head_dim") or hidden // nq
    cfg = dict(n_layers=conf["num_hidden_layers"], hidden=hidden, n_q_heads=nq,
               n_kv_heads=conf["num_key_value_heads"], head_dim=hd, ffn=conf["intermediate_size"],
               vocab=conf["vocab_size"], max_context=max_context, rms_eps=conf["rms_norm_eps"],
               rope_theta=conf["rope_theta"])
    rs = conf.get("rope_scaling")
    if rs and rs["type"] == "llama3":
        cfg["rope_factors"] = ob.llama3_rope_factors(hd, conf["rope_theta"], rs["factor"],
                                                     rs["low_freq_factor"], rs["high_freq_factor"],
                                                     rs["original_max_position_embeddings"])
    elif rs:
        # YaRN (crates/compute/src/rope.rs:324-372): a per-pair frequency table and a magnitude scale
        assert rs["type"] == "yarn" and rs.get("mscale", 1.0) == 1.0 and rs.get("mscale_all_dim", 0.0) == 0.0
        cfg["rope_freqs"], cfg["rope_mscale"] = ob.yarn_frequencies(
            hd, conf["rope_theta"], rs["factor"], rs["original_max_position_embeddings"], rs["beta_fast"], rs["beta_slow"])
    layers = []
    for i in range(cfg["n_layers"]):
        p = f"model.layers.{i}."
        lw = dict(attn_norm=_t(st[p + "input_layernorm.weight"]),
                  wq=_t(st[p + "self_attn.q_proj.weight"]), wk=_t(st[p + "self_attn.k_proj.weight"]),
                  wv=_t(st[p + "self_attn.v_proj.weight"]), wo=_t(st[p + "self_attn.o_proj.weight"]),
                  ffn_norm=_t(st[p + "post_attention_layernorm.weight"]),
                  w_gate=_t(st[p + "mlp.gate_proj.weight"]), w_up=_t(st[p + "mlp.up_proj.weight"]),
                  w_down=_t(st[p + "mlp.down_proj.weight"]))
        if p + "self_attn.q_proj.bias" in st:  # qwen2: biases on the q / k / v projections, added before the rotation
            lw.update(bq=_t(st[p + "self_attn.q_proj.bias"]), bk=_t(st[p + "self_attn.k_proj.bias"]),
                      bv=_t(st[p + "self_attn.v_proj.bias"]))
        if p + "self_attn.q_norm.weight" in st:
            lw["q_norm"] = _t(st[p + "self_attn.q_norm.weight"])
            lw["k_norm"] = _t(st[p + "self_attn.k_norm.weight"])
        layers.append(lw)
    weights = dict(embed=_t(st["model.embed_tokens.weight"]), final_norm=_t(st["model.norm.weight"]),
                   layers=layers)
    assert conf.get("tie_word_embeddings", False)
    return cfg, weights, traces
