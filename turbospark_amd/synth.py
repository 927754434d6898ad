"""Seeded random-init target models in GGUF block formats (the reference's synthetic installs,
crates/repack/src/synthetic_*.rs, for the verify path's benchmark configurations)."""
import numpy as np

from . import ffi

# The benchmark configurations of the verify path (dense ones).
CONFIGS = {
    # tiny Llama-style decoder, the reference's CPU-runnable plumbing case
    "tiny_q8_0": dict(n_layers=2, hidden=512, n_q_heads=8, n_kv_heads=8, head_dim=64, ffn=1408,
                      vocab=4096, rms_eps=1e-5, rope_theta=10000.0, dtype=ffi.Q8_0),
    # a small Q4_K stand-in with the 8B model's head geometry (GQA 4, head_dim 128)
    "small_q4_k": dict(n_layers=2, hidden=512, n_q_heads=4, n_kv_heads=1, head_dim=128, ffn=1536,
                       vocab=4096, rms_eps=1e-5, rope_theta=500000.0, dtype=ffi.Q4_K),
    # the tensor mix of a Q4_K_M file: Q4_K with the value and down projections of some layers, the
    # output head (and here the embedding table) in Q6_K
    "small_q4_k_m": dict(n_layers=2, hidden=512, n_q_heads=4, n_kv_heads=1, head_dim=128, ffn=1536,
                         vocab=4096, rms_eps=1e-5, rope_theta=500000.0, dtype=ffi.Q4_K,
                         overrides={(0, "wv"): ffi.Q6_K, (0, "w_down"): ffi.Q6_K, "lm_head": ffi.Q6_K, "embed": ffi.Q6_K}),
    # the mix of a Q5_K_M file: Q5_K, with Q6_K on the value / down projections of a layer and on the head
    "small_q5_k_m": dict(n_layers=2, hidden=512, n_q_heads=4, n_kv_heads=1, head_dim=128, ffn=1536,
                         vocab=4096, rms_eps=1e-5, rope_theta=500000.0, dtype=ffi.Q5_K,
                         overrides={(1, "wv"): ffi.Q6_K, (1, "w_down"): ffi.Q6_K, "lm_head": ffi.Q6_K}),
    # eight KV heads of 64-wide heads (the group sizes 4 and 2), widths that split into eight
    # chunk-aligned slices; norm weights are not all ones here
    "xcd_q4_k": dict(n_layers=2, hidden=1024, n_q_heads=32, n_kv_heads=8, head_dim=64, ffn=2048,
                     vocab=4096, rms_eps=1e-5, rope_theta=500000.0, dtype=ffi.Q4_K, norm_jitter=0.25),
    "xcd_q8_0": dict(n_layers=2, hidden=1024, n_q_heads=16, n_kv_heads=8, head_dim=64, ffn=1024,
                     vocab=4096, rms_eps=1e-5, rope_theta=10000.0, dtype=ffi.Q8_0, norm_jitter=0.25),
    # a small routed-expert decoder in the arrangement of the Qwen3-30B-A3B configuration: Q8_0
    # attention and router, per-head q / k RMSNorm, MXFP4 experts, top-k routing with softmax over the
    # selected logits
    "moe_small": dict(n_layers=2, hidden=512, n_q_heads=8, n_kv_heads=2, head_dim=64, ffn=256,
                      n_experts=16, top_k=4, vocab=4096, rms_eps=1e-6, rope_theta=1000000.0, qk_norm=True,
                      dtype=ffi.Q8_0, expert_dtype=ffi.MXFP4, router_sigma=0.08, norm_jitter=0.25),
    # a small decoder in the arrangement of the gpt-oss configuration: bf16 attention / router / head
    # with projection biases, attention sinks, a sliding window on even layers, YaRN rotation,
    # MXFP4 experts with biases and the clamped SwiGLU; hidden and expert width are NOT multiples
    # of 256 (as 2880 is not), so the MXFP4 tiles end in zero-padded blocks
    "gptoss_small": dict(n_layers=2, hidden=576, n_q_heads=8, n_kv_heads=2, head_dim=64, ffn=288,
                         n_experts=8, top_k=4, vocab=4096, rms_eps=1e-5, rope_theta=150000.0, attn_scale=0.125,
                         dtype=ffi.BF16, expert_dtype=ffi.MXFP4, router_sigma=0.08, norm_jitter=0.25,
                         gptoss=dict(window=24, yarn=(32.0, 64, 32.0, 1.0), act_alpha=1.702, act_limit=7.0)),
    # gpt-oss-120B shape (36 layers, 128 experts top-4, alternating 128-token window / full attention)
    "gptoss_120b": dict(n_layers=36, hidden=2880, n_q_heads=64, n_kv_heads=8, head_dim=64, ffn=2880,
                        n_experts=128, top_k=4, vocab=201088, rms_eps=1e-5, rope_theta=150000.0, attn_scale=0.125,
                        dtype=ffi.BF16, expert_dtype=ffi.MXFP4, router_sigma=0.02,  # "all random-init N(0, 0.02)"
                        gptoss=dict(window=128, yarn=(32.0, 4096, 32.0, 1.0), act_alpha=1.702, act_limit=7.0)),
    # Qwen3-30B-A3B shape: 128 experts, top-8, MXFP4 experts, Q8_0 attention / router / head
    "qwen3_30b_a3b": dict(n_layers=48, hidden=2048, n_q_heads=32, n_kv_heads=4, head_dim=128, ffn=768,
                          n_experts=128, top_k=8, vocab=151936, rms_eps=1e-6, rope_theta=1000000.0, qk_norm=True,
                          # router logits N(0, 1): the normalised input has unit mean square, so sigma = hidden ** -0.5
                          dtype=ffi.Q8_0, expert_dtype=ffi.MXFP4, router_sigma=2048 ** -0.5),
    # Llama-3-8B shape
    "llama3_8b_q4_k": dict(n_layers=32, hidden=4096, n_q_heads=32, n_kv_heads=8, head_dim=128,
                           ffn=14336, vocab=128256, rms_eps=1e-5, rope_theta=500000.0, dtype=ffi.Q4_K),
}


def make_weights(cfg, seed=1234, sigma=0.02, n_layers=None):
    """N(0, sigma) weights quantized to cfg['dtype']; norm weights 1.0.  Returns the weight
    dictionary both the engine and the test oracle take."""
    dt = cfg["dtype"]
    H, F, V = cfg["hidden"], cfg["ffn"], cfg["vocab"]
    qd, kvd = cfg["n_q_heads"] * cfg["head_dim"], cfg["n_kv_heads"] * cfg["head_dim"]
    jitter = float(cfg.get("norm_jitter", 0.0))
    nrng = np.random.default_rng(seed + 99)

    def ones(n):
        v = np.ones((1, n), np.float32)
        if jitter:
            v = (v + jitter * nrng.uniform(-1.0, 1.0, (1, n))).astype(np.float32)
        return (ffi.F32, v.view(np.uint8).reshape(1, -1), 1, n)

    stream = [0]

    over = cfg.get("overrides", {})

    def t(rows, cols, dtype=None, sig=None, name=None):
        stream[0] += 1
        if name in over:
            dtype = over[name]
        return ffi.synth_tensor(dt if dtype is None else dtype, seed, stream[0], sigma if sig is None else sig,
                                rows, cols)

    # weak_layers < 1 scales what each layer adds to the stream (the output and down projections): the logits
    # then follow the last token's embedding more than its context
    weak = float(cfg.get("weak_layers", 1.0)) * sigma
    L = cfg["n_layers"] if n_layers is None else n_layers
    E = int(cfg.get("n_experts", 0))
    oss = cfg.get("gptoss")
    brng = np.random.default_rng(seed + 7)

    def vec(n, scale, dtype=ffi.F32):
        """A small random vector (biases, sinks) stored as f32 or bf16."""
        v = (brng.standard_normal((1, n)) * scale).astype(np.float32)
        return ffi.quantize(dtype, v) if dtype != ffi.F32 else (ffi.F32, v.view(np.uint8).reshape(1, -1), 1, n)

    if oss:
        factor, octx, bf, bs = oss["yarn"]
        cfg["rope_freqs"], cfg["rope_mscale"] = ffi.yarn_frequencies(cfg["head_dim"], cfg["rope_theta"], factor, octx, bf, bs)
        cfg["act_alpha"], cfg["act_limit"] = oss["act_alpha"], oss["act_limit"]
    layers = []
    for li in range(L):
        lw = dict(attn_norm=ones(H), wq=t(qd, H), wk=t(kvd, H), wv=t(kvd, H, name=(li, "wv")), wo=t(H, qd, sig=weak),
                  ffn_norm=ones(H))
        if cfg.get("qk_norm"):  # Qwen3: RMSNorm over each q / k head before the rotation
            lw.update(q_norm=ones(cfg["head_dim"]), k_norm=ones(cfg["head_dim"]))
        if E:
            xd = cfg.get("expert_dtype", dt)
            lw.update(n_experts=E, top_k=int(cfg["top_k"]), router=t(E, H, sig=cfg.get("router_sigma", sigma)),
                      we_gate=t(E * F, H, xd), we_up=t(E * F, H, xd), we_down=t(E * H, F, xd, sig=weak))
        else:
            lw.update(w_gate=t(F, H), w_up=t(F, H), w_down=t(H, F, sig=weak, name=(li, "w_down")))
        if oss:
            # attention biases and sinks are bf16 in the GGUF, expert and router biases f32
            lw.update(bq=vec(qd, 0.05, ffi.BF16), bk=vec(kvd, 0.05, ffi.BF16), bv=vec(kvd, 0.05, ffi.BF16),
                      bo=vec(H, 0.05, ffi.BF16), sinks=vec(cfg["n_q_heads"], 1.0, ffi.BF16),
                      window=oss["window"] if li % 2 == 0 else 0)  # even layers slide (gptoss/attn.rs:20-23)
            if E:
                def mat(r, c, scale):
                    v = (brng.standard_normal((r, c)) * scale).astype(np.float32)
                    return (ffi.F32, v.view(np.uint8).reshape(r, -1), r, c)
                lw.update(router_bias=vec(E, 0.05), be_gate=mat(E, F, 0.05), be_up=mat(E, F, 0.05),
                          be_down=mat(E, H, 0.05))
        layers.append(lw)
    # embed_scale > 1: embedding rows that dwarf what the layers add (the final norm takes the scale out again)
    return dict(embed=t(V, H, sig=sigma * float(cfg.get("embed_scale", 1.0)), name="embed"), final_norm=ones(H),
                lm_head=t(V, H, name="lm_head"), layers=layers)


def make_mtp_weights(cfg, trunk_weights, seed=4321, sigma=0.02, follow=0.0, norm_jitter=0.1):
    """A drafter head for `cfg`'s target (docs/MTP.md:53-60): (head cfg, head weights) -- one decoder layer of
    the target's shapes, its own norm, fc (hidden x 2 hidden) and the norms of fc's two halves, with the target's
    embedding table, output head and final norm by reference.  `follow` > 0 adds that multiple of the identity
    to fc's embedding half: with a target whose layers add little to the stream, both then predict from the
    embedding of the last token, and the head's proposals are often the target's picks."""
    hcfg = dict(cfg, n_layers=1)
    hcfg.pop("overrides", None)
    base = make_weights(hcfg, seed=seed, sigma=sigma, n_layers=1)
    base["layers"][0]["window"] = 0  # the head's one layer attends over everything (docs/MTP.md:76-78)
    H = cfg["hidden"]
    rng = np.random.default_rng(seed + 5)

    def near_one(n):
        v = (1.0 + norm_jitter * rng.uniform(-1.0, 1.0, (1, n))).astype(np.float32)
        return (ffi.F32, v.view(np.uint8).reshape(1, -1), 1, n)

    fc = (rng.standard_normal((H, 2 * H)) * sigma).astype(np.float32)
    if follow:
        fc[:, :H] += follow * np.eye(H, dtype=np.float32)
    fdt = cfg["dtype"] if cfg["dtype"] != ffi.MXFP4 else ffi.BF16
    return hcfg, dict(embed=trunk_weights["embed"], lm_head=trunk_weights.get("lm_head"), final_norm=near_one(H),
                      layers=base["layers"], fc=ffi.quantize(fdt, fc), norm_embedding=near_one(H),
                      norm_hidden=near_one(H), trunk_norm=trunk_weights["final_norm"])
