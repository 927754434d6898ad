"""tsv_open_gguf: a GGUF file opened as the verify target gives, bit for bit, the logits of the same
weights handed over directly -- so the names (crates/repack/src/gguf_names/llama.rs:14-60), the
sizes read from the metadata and the rotary row un-permutation of a `llama` file
(crates/repack/src/gguf_checkpoint/conventions.rs:133-243) are the install's."""
import os

import numpy as np
import pytest

import turbospark_amd as ts
from tests.gguf_writer import llama_gguf, write_gguf
from turbospark_amd import ffi, synth

pytestmark = pytest.mark.gpu


def _both(tmp_path, name, arch, permute, max_context=96, **over):
    cfg = dict(synth.CONFIGS[name], max_context=max_context, **over)
    w = synth.make_weights(cfg, seed=4321)
    path = os.path.join(tmp_path, f"{name}.gguf")
    llama_gguf(path, cfg, w, arch=arch, permute=permute)
    return cfg, w, path, ts.HipVerifier(cfg, w), ts.HipVerifier.from_gguf(path)


@pytest.mark.parametrize("name,arch,permute", [
    ("tiny_q8_0", "llama", True),          # adjacent-pair q / k rows, un-permuted at intake (64-wide heads)
    ("small_q4_k_m", "llama", True),       # the Q4_K + Q6_K mix of a Q4_K_M file, 128-wide heads
    ("small_q5_k_m", "llama", True),
    ("moe_small", "qwen3moe", False),      # per-head q / k norms, stacked MXFP4 experts, Q8_0 router
    ("gptoss_small", "gpt-oss", False),    # bf16 attention with biases and sinks, window on even layers, YaRN, expert biases
])
def test_a_gguf_target_equals_the_directly_installed_one(tmp_path, name, arch, permute):
    cfg, w, path, direct, filed = _both(tmp_path, name, arch, permute)
    assert filed.cfg["n_layers"] == cfg["n_layers"] and filed.cfg["head_dim"] == cfg["head_dim"]
    assert filed.vocab == cfg["vocab"] and filed.cfg["max_context"] == 96
    rng = np.random.default_rng(8)
    prompt = rng.integers(0, cfg["vocab"], 37).astype(np.int32)
    assert np.array_equal(direct.prefill(prompt, 0), filed.prefill(prompt, 0))
    feed = rng.integers(0, cfg["vocab"], 5).astype(np.int32)
    assert np.array_equal(direct.verify(feed, 37), filed.verify(feed, 37))
    for layer in range(cfg["n_layers"]):
        (ka, va), (kb, vb) = direct.read_kv(layer, 0, 42), filed.read_kv(layer, 0, 42)
        assert np.array_equal(ka.view(np.uint16), kb.view(np.uint16)) and np.array_equal(va.view(np.uint16), vb.view(np.uint16))


def test_the_permutation_matters_and_tied_heads_and_llama3_factors_load(tmp_path):
    # a llama file whose q / k rows were NOT permuted by its converter is read wrongly: the intake
    # really moves rows
    cfg, w, path, direct, filed = _both(tmp_path, "tiny_q8_0", "llama", False)
    prompt = np.random.default_rng(8).integers(0, cfg["vocab"], 20).astype(np.int32)
    assert not np.array_equal(direct.prefill(prompt, 0), filed.prefill(prompt, 0))
    # no output.weight: the head is the embedding table; rope_freqs.weight: llama-3's per-pair divisors
    factors = np.linspace(1.0, 8.0, 32).astype(np.float32)
    cfg = dict(synth.CONFIGS["tiny_q8_0"], max_context=64, rope_factors=factors)
    w = synth.make_weights(cfg, seed=99)
    w["lm_head"] = None
    path = os.path.join(tmp_path, "tied.gguf")
    llama_gguf(path, cfg, w)
    a, b = ts.HipVerifier(cfg, w), ts.HipVerifier.from_gguf(path, max_context=64)
    row = a.prefill(prompt, 0)
    assert np.array_equal(row, b.prefill(prompt, 0))
    plain = ts.HipVerifier(dict(cfg, rope_factors=None), w)
    assert not np.array_equal(row, plain.prefill(prompt, 0))   # the factors are in use


def test_files_the_intake_cannot_express_are_refused_by_name(tmp_path):
    cfg = dict(synth.CONFIGS["tiny_q8_0"], max_context=64)
    w = synth.make_weights(cfg, seed=1)
    path = os.path.join(tmp_path, "x.gguf")
    with pytest.raises(ffi.TsvError, match="architecture 'gemma3'"):
        llama_gguf(path, cfg, w, arch="gemma3")
        ts.HipVerifier.from_gguf(path)
    # a missing projection
    write_gguf(path, [("general.architecture", "str", "llama"), ("llama.block_count", "u32", 1),
                      ("llama.embedding_length", "u32", 512), ("llama.attention.head_count", "u32", 8),
                      ("llama.feed_forward_length", "u32", 1408), ("llama.context_length", "u32", 64)],
               [("token_embd.weight", [512, 4096], w["embed"][0], w["embed"][1].tobytes()),
                ("output_norm.weight", [512], 0, w["final_norm"][1].tobytes())])
    with pytest.raises(ffi.TsvError, match="blk.0.attn_norm.weight' is missing"):
        ts.HipVerifier.from_gguf(path)
    # context extension the intake does not map
    from tests import gguf_writer as gw
    orig = gw.write_gguf

    def with_yarn(p, meta, tensors, **kw):
        return orig(p, list(meta) + [("llama.rope.scaling.type", "str", "yarn")], tensors, **kw)
    gw.write_gguf = with_yarn
    try:
        llama_gguf(path, cfg, w)
    finally:
        gw.write_gguf = orig
    with pytest.raises(ffi.TsvError, match="rope scaling 'yarn'"):
        ts.HipVerifier.from_gguf(path)


@pytest.mark.parametrize("name,arch,permute,tol", [
    ("tiny_q8_0", "llama", True, 2e-3),
    ("small_q4_k_m", "llama", True, 1e-2),
    ("moe_small", "qwen3moe", False, 1e-2),
    ("gptoss_small", "gpt-oss", False, 1e-2),
])
def test_a_gguf_target_agrees_with_the_oracle_reading_the_same_file(tmp_path, name, arch, permute, tol):
    """The engine opened by tsv_open_gguf against the ORACLE fed by an independent reader of the same file
    (tests/gguf_reader.py: header, tensor table, the names of gguf_names/llama.rs:14-60 and
    gpt_oss.rs:30-72, the q / k row un-permutation of conventions.rs:133-151, the YaRN keys): two readings
    of one file that share no code, so a name, a size or a row order taken wrongly by either shows up as
    a logit error.  (The file itself is laid out by this project's writer: no GGUF ships with the reference.)"""
    from oracle import binding as ob
    from tests import gguf_reader
    from tests import gpu_common as gc
    cfg = dict(synth.CONFIGS[name], max_context=96)
    w = synth.make_weights(cfg, seed=4321)
    path = os.path.join(tmp_path, f"{name}.gguf")
    llama_gguf(path, cfg, w, arch=arch, permute=permute)
    filed = ts.HipVerifier.from_gguf(path)
    ocfg, ow = gguf_reader.load_model(path, max_context=96)
    for key in ("n_layers", "hidden", "n_q_heads", "n_kv_heads", "head_dim", "ffn", "vocab"):
        assert ocfg[key] == cfg[key], key
    cpu = ob.Model(ocfg, ow, round_kv_f16=True, threads=8)
    for attempt in range(20):
        rng = np.random.default_rng(8 + attempt)
        prompt = rng.integers(0, cfg["vocab"], 37).astype(np.int32)
        feed = rng.integers(0, cfg["vocab"], 5).astype(np.int32)
        cpu.reset()
        margins = []
        for i in range(0, 37, 16):
            cpu.verify(prompt[i:i + 16], i)
            margins.append(cpu.route_margin)
        want = cpu.verify(feed, 37)
        margins.append(cpu.route_margin)
        if min(margins) > 1e-3:        # (routed models: a prompt without a near-tie routing decision)
            break
    filed.prefill(prompt, 0, want_logits=False)
    got = filed.verify(feed, 37)
    err = gc.logit_error(got, want)
    print(f"{name} from GGUF: GPU engine vs oracle over an independent reader, max-abs / range = {err:.2e}")
    assert err <= tol
    for layer in range(cfg["n_layers"]):
        kg, vg = filed.read_kv(layer, 0, 42)
        kc, vc = cpu.kv(layer)
        assert np.abs(kg.astype(np.float32) - kc[:42]).max() <= 2e-2 * np.abs(kc[:42]).max()
