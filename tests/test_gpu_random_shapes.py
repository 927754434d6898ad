"""Seeded sweep over decoder shapes the verify path accepts: head width, GQA group, hidden / ffn /
vocabulary sizes that are not round, layer count, context length, rows per pass, chain or random
tree.  Each case checks the pass's logits and new K/V rows against the oracle's forward
(families/qwen/batched.rs:92-456 semantics: row i sees the prefix plus its own root path) and then
one sampled round -- random truncation and penalties -- against the oracle's acceptance on the
GPU's own logits (speculative.rs:694-754), integers equal."""
import numpy as np
import pytest

from oracle import binding as ob
from tests import gpu_common as gc
from turbospark_amd import ffi

pytestmark = pytest.mark.gpu


def _case(seed):
    r = np.random.default_rng(1000 + seed)
    q4 = bool(r.integers(0, 2))
    hd = int(r.choice([64, 128]))
    nkv = int(r.choice([1, 2, 4, 8]))
    group = int(r.choice([1, 2, 4, 8]))
    while nkv * group > 32:
        group //= 2
    unit = 256 if q4 else 128            # K of a matmul is whole superblocks (Q4_K) / 128-element chunks (Q8_0)
    hidden = unit * int(r.integers(1, 5 if q4 else 9))
    while (nkv * group * hd) % unit:     # K of the output projection
        group *= 2
    ffn = unit * int(r.integers(1, 7 if q4 else 13))
    cfg = dict(n_layers=int(r.integers(1, 4)), hidden=hidden, n_q_heads=nkv * group, n_kv_heads=nkv, head_dim=hd, ffn=ffn,
               vocab=int(r.integers(700, 5000)), rms_eps=1e-5, rope_theta=float(r.choice([10000.0, 500000.0])),
               dtype=ffi.Q4_K if q4 else ffi.Q8_0, norm_jitter=0.25, qk_norm=bool(r.integers(0, 2)))
    ctx = int(r.integers(1, 90))
    m = int(r.integers(1, 17))
    tree = bool(r.integers(0, 2)) and m > 2
    parent = None
    if tree:
        parent = [-1] + [int(r.integers(0, s)) for s in range(1, m)]
    return cfg, ctx, m, parent, r


@pytest.mark.parametrize("seed", range(48))
def test_random_shape(seed):
    import turbospark_amd as ts
    from turbospark_amd import synth
    cfg, ctx, m, parent, r = _case(seed)
    synth.CONFIGS["_random"] = cfg
    try:
        cfg, w, gpu, cpu = gc.build_pair("_random", max_context=ctx + 40, seed=77 + seed)
    finally:
        del synth.CONFIGS["_random"]
    V = cfg["vocab"]
    print(f"seed {seed}: {'q4_k' if cfg['dtype'] == ffi.Q4_K else 'q8_0'} L={cfg['n_layers']} H={cfg['hidden']} "
          f"q/kv={cfg['n_q_heads']}/{cfg['n_kv_heads']}x{cfg['head_dim']} F={cfg['ffn']} V={V} ctx={ctx} m={m} "
          f"{'tree' if parent else 'chain'}{' qk-norm' if cfg['qk_norm'] else ''}", flush=True)
    prompt = r.integers(0, V, ctx).astype(np.int32)
    feed = r.integers(0, V, m).astype(np.int32)
    gpu.prefill(prompt, 0, want_logits=False)
    for i in range(0, ctx, 16):
        cpu.verify(prompt[i:i + 16], i)
    tol = gc.TOL[cfg["dtype"]]
    if parent:
        got = gpu.verify_tree(feed, parent, ctx)
    else:
        got = gpu.verify(feed, ctx)
    want = cpu.verify(feed, ctx, parent=parent)
    err = gc.logit_error(got, want)
    print(f"   max-abs logit error / range = {err:.2e}", flush=True)
    assert err <= tol, err
    for layer in range(cfg["n_layers"]):
        kg, vg = gpu.read_kv(layer, 0, ctx + m)
        kc, vc = cpu.kv(layer)
        assert np.abs(kg.astype(np.float32) - kc[:ctx + m]).max() <= 2e-2 * np.abs(kc[:ctx + m]).max()
        assert np.abs(vg.astype(np.float32) - vc[:ctx + m]).max() <= 2e-2 * np.abs(vc[:ctx + m]).max()
    # one round of acceptance on these logits
    kw = {}
    if r.integers(0, 2):
        kw["top_k"] = int(r.integers(1, 200))
    if r.integers(0, 2):
        kw["top_p"] = float(r.uniform(0.3, 1.0))
    if r.integers(0, 2):
        kw["min_p"] = float(r.uniform(0.001, 0.2))
    temperature = float(r.choice([0.0, 0.6, 1.0, 1.4]))
    hist = [int(t) for t in prompt] + [int(feed[0])]
    if temperature and r.integers(0, 2):
        kw["repetition_penalty"] = float(r.uniform(0.8, 1.5))
    if temperature and r.integers(0, 2):
        kw["presence_penalty"] = float(r.uniform(-0.5, 1.5))
        kw["frequency_penalty"] = float(r.uniform(-0.2, 0.6))
    generated = int(r.integers(0, len(hist) + 3))
    if parent:
        draft = (gc.f16(got) + r.standard_normal((m, V)).astype(np.float32) * 0.5).astype(np.float16)
        gcfg = ts.shaping(temperature, seed=seed if temperature else None, **kw)
        ocfg = ob.shaping(temperature, seed=seed if temperature else None, **kw)
        res = gpu.accept(feed, ctx, gcfg, parent=parent, draft_logits=draft if temperature else None, draw_step=11,
                         history=hist, generated=generated)
        if temperature:
            ref = ob.tree_round_sampled(got, draft, feed, parent, ocfg, history=hist, generated=generated, draw_step=11)
        else:
            ref = ob.tree_round_greedy(got, feed, parent, ocfg, history=hist[:-1])
        assert res.path == ref["path"] and res.next == ref["next"], (res, ref)
        assert res.draw_step == (ref["draw_step"] if temperature else 11)  # the arg-max walk draws nothing
        assert gpu.position == ctx + len(ref["path"])
    else:
        gcfg = ts.shaping(temperature, seed=seed if temperature else None, **kw)
        ocfg = ob.shaping(temperature, seed=seed if temperature else None, **kw)
        k = m - 1
        draft = (gc.f16(got)[:k] + r.standard_normal((k, V)).astype(np.float32) * 0.5).astype(np.float16)
        res = gpu.accept(feed, ctx, gcfg, draft_logits=draft if temperature else None, draw_step=11, history=hist,
                         generated=generated, max_new_tokens=generated + 40)
        ref = ob.chain_round(got, draft if temperature else None, feed[1:], ocfg, history=hist, generated=generated,
                             max_new_tokens=generated + 40, draw_step=11)
        assert (res.accepted, res.committed, res.next, res.stopped, res.draw_step) == \
            (ref["accepted"], ref["committed"], ref["next"], ref["stopped"], ref["draw_step"]), (res, ref)
        assert gpu.position == ctx + ref["committed"] + 1


def _moe_case(seed):
    r = np.random.default_rng(5000 + seed)
    oss = bool(r.integers(0, 2))
    hd = int(r.choice([64, 128]))
    nkv = int(r.choice([1, 2, 4]))
    group = int(r.choice([1, 2, 4, 8]))
    hidden = 64 * int(r.integers(3, 13))           # MXFP4 / bf16 widths need not be whole 256-element chunks
    if not oss:
        hidden = 128 * int(r.integers(2, 7))       # Q8_0 attention: whole 128-element chunks
        while (nkv * group * hd) % 128:
            group *= 2
    n_experts = int(r.choice([4, 8, 16]))
    cfg = dict(n_layers=int(r.integers(1, 4)), hidden=hidden, n_q_heads=nkv * group, n_kv_heads=nkv, head_dim=hd,
               ffn=32 * int(r.integers(2, 13)), n_experts=n_experts, top_k=int(r.choice([1, 2, 4])),
               vocab=int(r.integers(700, 4000)), rms_eps=1e-6, rope_theta=150000.0,
               dtype=ffi.BF16 if oss else ffi.Q8_0, expert_dtype=ffi.MXFP4, router_sigma=0.08, norm_jitter=0.25)
    cfg["qk_norm"] = not oss and bool(r.integers(0, 2))
    if oss:
        cfg["attn_scale"] = float(r.choice([0.125, 0.1]))
        cfg["gptoss"] = dict(window=int(r.integers(17, 60)), yarn=(32.0, 64, 32.0, 1.0), act_alpha=1.702, act_limit=7.0)
    return cfg, int(r.integers(1, 40)), int(r.integers(0, 16)), r


@pytest.mark.parametrize("seed", range(16))
def test_random_routed_expert_shape(seed):
    """The same sweep over routed-expert decoders (families/llama/moe.rs:1-17, families/gptoss/mod.rs:11-23):
    expert count, top-k, widths that are not whole chunks, and for the gpt-oss arrangement a random
    window, biases, sinks and YaRN.  Inputs whose routing is a near tie in the oracle are skipped by
    re-drawing (the GPU's router logits carry fp16-activation rounding)."""
    from turbospark_amd import synth
    from tests.test_gpu_moe import _clean_inputs
    cfg, ctx, k, r = _moe_case(seed)
    synth.CONFIGS["_random"] = cfg
    try:
        cfg, w, gpu, cpu = gc.build_pair("_random", max_context=ctx + 40, seed=31 + seed)
    finally:
        del synth.CONFIGS["_random"]
    print(f"seed {seed}: {'gpt-oss' if cfg.get('gptoss') else 'qwen-moe'} L={cfg['n_layers']} H={cfg['hidden']} "
          f"q/kv={cfg['n_q_heads']}/{cfg['n_kv_heads']}x{cfg['head_dim']} F={cfg['ffn']} E={cfg['n_experts']} top{cfg['top_k']} "
          f"V={cfg['vocab']} ctx={ctx} m={k + 1}{' qk-norm' if cfg['qk_norm'] else ''}", flush=True)
    prompt, feed, want, margin = _clean_inputs(cfg, cpu, ctx, k, floor=1e-3)
    gpu.prefill(prompt, 0, want_logits=False)
    got = gpu.verify(feed, ctx)
    err = gc.logit_error(got, want)
    print(f"   max-abs logit error / range = {err:.2e}, route margin {margin:.2e}", flush=True)
    assert err <= 1e-2, err
    for layer in range(cfg["n_layers"]):
        kg, vg = gpu.read_kv(layer, 0, ctx + k + 1)
        kc, vc = cpu.kv(layer)
        assert np.abs(kg.astype(np.float32) - kc[:ctx + k + 1]).max() <= 2e-2 * np.abs(kc[:ctx + k + 1]).max()
        assert np.abs(vg.astype(np.float32) - vc[:ctx + k + 1]).max() <= 2e-2 * np.abs(vc[:ctx + k + 1]).max()
