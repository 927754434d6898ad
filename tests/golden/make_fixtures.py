"""Extract the reference's own golden DATA into small fixtures under tests/golden/.

Reads files below /root/reference as text / data only (nothing is imported or run):
  * the literal arrays of crates/compute/tests/generated/quant_gguf_mxfp4_oracle.rs
    (bytes ggml produced and the floats ggml decoded from them)  -> mxfp4_ggml_oracle.json
  * the literal arrays of crates/compute/tests/generated/quant_gguf_q5_k_oracle.rs (two Q5_K superblocks
    ggml quantized and the floats ggml decoded from them)  -> q5k_ggml_oracle.json
  * the hand-packed Q4_K superblock constants of crates/compute/tests/quant_gguf.rs:226-267
    -> q4k_handpacked.json
  * the llama-3 rope factor profile of crates/compute/src/rope.rs:471-482 -> llama3_rope_profile.json
  * the literal arrays of crates/compute/tests/generated/kv_quant_oracle.rs (TurboQuant KV codec: sign
    vectors, codebooks, input rows, norms and packed words of four (dim, bits) shapes)  -> kv_quant_oracle.json
  * five MLX known-answer fixtures (config.json, model.safetensors, traces.json) of
    crates/audio/testdata/lm/{llama_default,llama_llama3_rope,qwen3_default,llama_yarn_rope,qwen2_default}
    -> lm/<name>/

Run once in the authoring container:  python tests/golden/make_fixtures.py
The outputs are committed; tests never read /root/reference.
"""
import json
import os
import re
import shutil

REF = "/root/reference"
OUT = os.path.dirname(os.path.abspath(__file__))


def rust_array(text, name):
    m = re.search(name + r"\s*:\s*\[[^\]]*\]\s*=\s*\[(.*?)\];", text, re.S)
    assert m, name
    body = re.sub(r"//.*", "", m.group(1))
    vals = [v.strip() for v in body.replace("\n", " ").split(",") if v.strip()]
    return vals


def main():
    src = open(f"{REF}/crates/compute/tests/generated/quant_gguf_mxfp4_oracle.rs").read()
    fixture = {
        "source": "crates/compute/tests/generated/quant_gguf_mxfp4_oracle.rs",
        "codebook": [float(v) for v in rust_array(src, "MXFP4_ORACLE_CODEBOOK")],
        "e8m0_times_codebook1": [float(v) for v in rust_array(src, "MXFP4_ORACLE_E8M0")],
        "bytes": [int(v) for v in rust_array(src, "MXFP4_ORACLE_BYTES")],
        "floats": [float(v) for v in rust_array(src, "MXFP4_ORACLE_FLOATS")],
    }
    assert len(fixture["codebook"]) == 16 and len(fixture["e8m0_times_codebook1"]) == 256
    assert len(fixture["bytes"]) == 68 and len(fixture["floats"]) == 128
    json.dump(fixture, open(f"{OUT}/mxfp4_ggml_oracle.json", "w"))

    src = open(f"{REF}/crates/compute/tests/generated/quant_gguf_q5_k_oracle.rs").read()
    q5 = {
        "source": "crates/compute/tests/generated/quant_gguf_q5_k_oracle.rs",
        "bytes": [int(v) for v in rust_array(src, "Q5_K_ORACLE_BYTES")],
        "floats": [float(v) for v in rust_array(src, "Q5_K_ORACLE_FLOATS")],
    }
    assert len(q5["bytes"]) == 352 and len(q5["floats"]) == 512
    json.dump(q5, open(f"{OUT}/q5k_ggml_oracle.json", "w"))

    src = open(f"{REF}/crates/compute/tests/generated/kv_quant_oracle.rs").read()
    tq = {"source": "crates/compute/tests/generated/kv_quant_oracle.rs", "rows_per_shape": 4, "shapes": []}
    for dim, bits in ((64, 2), (64, 3), (128, 4), (256, 3)):
        tag = f"D{dim}B{bits}"
        f32 = lambda name: [float(v.replace("f32", "")) for v in rust_array(src, f"{tag}_{name}")]
        shape = {"dim": dim, "bits": bits, "signs": f32("SIGNS"), "codebook": f32("CODEBOOK"), "input_rows": f32("INPUT_ROWS"),
                 "norms": f32("NORMS"), "packed": [int(v.replace("u32", ""), 0) for v in rust_array(src, f"{tag}_PACKED")]}
        assert len(shape["signs"]) == dim and len(shape["codebook"]) == 1 << bits and len(shape["input_rows"]) == 4 * dim
        assert len(shape["packed"]) == 4 * ((dim * bits + 31) // 32)
        tq["shapes"].append(shape)
    json.dump(tq, open(f"{OUT}/kv_quant_oracle.json", "w"))

    src = open(f"{REF}/crates/compute/tests/quant_gguf.rs").read()
    q4 = {
        "source": "crates/compute/tests/quant_gguf.rs:226-267",
        "LS": [int(v) for v in rust_array(src, "const LS")],
        "LM": [int(v) for v in rust_array(src, "const LM")],
        "PACKED": [int(v, 16) for v in rust_array(src, "const PACKED")],
        "D_BITS": [int(v, 16) for v in rust_array(src, "const D_BITS")],
        "DMIN_BITS": [int(v, 16) for v in rust_array(src, "const DMIN_BITS")],
        "d": 0.5,
        "dmin": 0.25,
        "quant_rule": "q[e] = (e*7+3) % 16",
    }
    json.dump(q4, open(f"{OUT}/q4k_handpacked.json", "w"))

    src = open(f"{REF}/crates/compute/src/rope.rs").read()
    json.dump(
        {
            "source": "crates/compute/src/rope.rs:462-518",
            "params": {"rotary_dim": 128, "base": 500000.0, "factor": 8.0, "low": 1.0, "high": 4.0,
                       "original_context": 8192.0},
            "ones": 29,
            "ramp": [1.207484, 1.553415, 2.026313, 2.69453, 3.684253, 5.257327],
            "tail": 8.0,
        },
        open(f"{OUT}/llama3_rope_profile.json", "w"),
    )

    for name in ["llama_default", "llama_llama3_rope", "qwen3_default", "llama_yarn_rope", "qwen2_default"]:
        dst = f"{OUT}/lm/{name}"
        os.makedirs(dst, exist_ok=True)
        for f in ["config.json", "model.safetensors", "traces.json"]:
            shutil.copyfile(f"{REF}/crates/audio/testdata/lm/{name}/{f}", f"{dst}/{f}")
            os.chmod(f"{dst}/{f}", 0o644)


if __name__ == "__main__":
    main()
