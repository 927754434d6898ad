"""The library's generation loop (device acceptance, device truncation) against the oracle's
restatement of crates/runtime/src/speculative.rs:194-900 driving the SAME GPU target through
`verify` + host acceptance: both see identical logits, so the reported tokens, the stop reason
and every counter must agree exactly."""
import numpy as np
import pytest

from oracle import binding as ob
from tests import gpu_common as gc
from tests.loop_common import GpuTarget, LmDrafter, TreeTwinDrafter

pytestmark = pytest.mark.gpu

KEYS = ("tokens", "stop_reason", "rounds", "offered", "accepted", "rollbacks", "draw_step", "final_depth")


def _pair(name="tiny_q8_0", max_context=200, draft_seed=1234):
    import turbospark_amd as ts
    from turbospark_amd import synth
    cfg, w, gpu, _ = gc.build_pair(name, max_context=max_context)
    dcfg = dict(synth.CONFIGS[name], max_context=max_context)
    dw = w if draft_seed == 1234 else synth.make_weights(dcfg, seed=draft_seed)
    return cfg, gpu, ts.HipVerifier(dcfg, dw)


@pytest.mark.parametrize("temperature,kw,block,floor,noise,draft_seed", [
    (0.0, {}, 4, 0, 0.0, 77),          # greedy, a drafter that is usually wrong
    (0.0, {}, 4, 0, 1.0, 1234),        # greedy, the target plus noise: mixed acceptance
    (0.0, {}, 8, 2, 0.3, 1234),        # adaptive depth
    (0.8, {}, 4, 0, 1.0, 1234),        # rejection sampling
    (1.0, dict(top_p=0.95, top_k=50), 8, 2, 0.5, 1234),
    (0.7, dict(min_p=0.02), 15, 0, 0.0, 1234),   # the widest block, a perfect drafter
    (0.9, dict(repetition_penalty=1.3, presence_penalty=0.5, frequency_penalty=0.2), 4, 0, 0.5, 1234),  # penalties see the growing history
    (0.8, dict(repetition_penalty=1.1, top_p=0.9, top_k=64), 6, 2, 0.3, 1234),
])
def test_the_device_loop_reports_what_the_reference_loop_reports(temperature, kw, block, floor, noise, draft_seed):
    import turbospark_amd as ts
    cfg, gpu, lm = _pair(draft_seed=draft_seed)
    V = cfg["vocab"]
    prompt = np.random.default_rng(3).integers(0, V, 19).astype(np.int32)
    seed = 41 if temperature else None
    gcfg, ocfg = ts.shaping(temperature, seed=seed, **kw), ob.shaping(temperature, seed=seed, **kw)
    new = 70
    want = ob.run_speculative(GpuTarget(gpu), LmDrafter(GpuTarget(lm), prompt[0], V, noise, 9), prompt, ocfg, new, block,
                              V, cfg["max_context"], adaptive_floor=floor)
    got = gpu.run_speculative(prompt, LmDrafter(GpuTarget(lm), prompt[0], V, noise, 9), gcfg, new, block,
                              adaptive_floor=floor)
    print({k: (got[k] if k != "tokens" else len(got[k])) for k in KEYS}, "min margin", got["min_margin"])
    assert {k: got[k] for k in KEYS} == {k: want[k] for k in KEYS}
    assert len(got["tokens"]) == new and got["stop_reason"] == 2
    assert got["kv_position"] == len(prompt) + new - 1 == gpu.position
    assert got["min_margin"] > 1e-9
    if noise:
        assert 0 < got["accepted"] < got["offered"]
    # a stop token taken from the stream ends the run there, unreported
    stop = got["tokens"][23]
    first = got["tokens"].index(stop)
    again = gpu.run_speculative(prompt, LmDrafter(GpuTarget(lm), prompt[0], V, noise, 9), gcfg, new, block,
                                stop_tokens=[stop], adaptive_floor=floor)
    ref = ob.run_speculative(GpuTarget(gpu), LmDrafter(GpuTarget(lm), prompt[0], V, noise, 9), prompt, ocfg, new, block,
                             V, cfg["max_context"], stop_tokens=[stop], adaptive_floor=floor)
    assert {k: again[k] for k in KEYS} == {k: ref[k] for k in KEYS}
    assert again["stop_reason"] == 1 and again["tokens"] == got["tokens"][:first]


def test_greedy_speculation_on_the_device_equals_plain_decoding():
    import turbospark_amd as ts
    cfg, gpu, lm = _pair(draft_seed=77)
    V = cfg["vocab"]
    prompt = np.random.default_rng(5).integers(0, V, 12).astype(np.int32)
    got = gpu.run_speculative(prompt, LmDrafter(GpuTarget(lm), prompt[0], V), ts.shaping(0.0), 50, 5)
    gpu.reset()
    gpu.prefill(prompt[:-1], 0, want_logits=False)
    tok, plain = int(prompt[-1]), []
    for i in range(50):
        tok = int(np.argmax(gc.f16(gpu.produce(tok, len(prompt) - 1 + i))))
        plain.append(tok)
    assert got["tokens"] == plain


def test_the_loop_stays_inside_the_context_window_and_refuses_bad_requests():
    import turbospark_amd as ts
    cfg, gpu, lm = _pair(max_context=64)
    V = cfg["vocab"]
    prompt = np.arange(3, 23).astype(np.int32)
    got = gpu.run_speculative(prompt, LmDrafter(GpuTarget(lm), prompt[0], V), ts.shaping(0.0), 44, 15)
    assert len(got["tokens"]) == 44 and got["kv_position"] == 63
    for kwargs, text in ((dict(max_new_tokens=45), "overflow"), (dict(max_new_tokens=0), "zero"), (dict(block=0), "block"),
                         (dict(block=16), "block")):
        args = dict(max_new_tokens=10, block=4)
        args.update(kwargs)
        with pytest.raises(ts.TsvError, match=text):
            gpu.run_speculative(prompt, LmDrafter(GpuTarget(lm), prompt[0], V), ts.shaping(0.0), args["max_new_tokens"],
                                args["block"])
    with pytest.raises(ts.TsvError, match="empty"):
        gpu.run_speculative([], LmDrafter(GpuTarget(lm), 0, V), ts.shaping(0.0), 4, 2)


@pytest.mark.parametrize("seed", range(10))
def test_random_generation_settings(seed):
    """Seeded sweep over the loop's settings: temperature, truncation, penalties, block, adaptive floor,
    drafter quality, budget, prompt length, and a stop token drawn from the vocabulary's frequent ids
    (so that some runs end on it and some on the budget)."""
    import turbospark_amd as ts
    r = np.random.default_rng(900 + seed)
    cfg, gpu, lm = _pair(draft_seed=1234)
    V = cfg["vocab"]
    temperature = float(r.choice([0.0, 0.5, 0.9, 1.2]))
    kw = {}
    if r.integers(0, 2):
        kw["top_k"] = int(r.integers(2, 120))
    if r.integers(0, 2):
        kw["top_p"] = float(r.uniform(0.5, 1.0))
    if r.integers(0, 2):
        kw["min_p"] = float(r.uniform(0.001, 0.1))
    if r.integers(0, 2):
        kw["repetition_penalty"] = float(r.uniform(0.9, 1.6))
    if r.integers(0, 2):
        kw["presence_penalty"] = float(r.uniform(0.0, 1.5))
        kw["frequency_penalty"] = float(r.uniform(0.0, 0.8))
    block = int(r.integers(1, 16))
    floor = int(r.integers(0, min(block, 3) + 1))
    noise = float(r.choice([0.0, 0.3, 1.0]))
    new = int(r.integers(5, 60))
    prompt = r.integers(0, V, int(r.integers(1, 40))).astype(np.int32)
    sd = 7 + seed if temperature else None
    gcfg, ocfg = ts.shaping(temperature, seed=sd, **kw), ob.shaping(temperature, seed=sd, **kw)
    print(f"seed {seed}: T={temperature} {kw} block={block} floor={floor} noise={noise} budget={new} prompt={len(prompt)}", flush=True)
    free = gpu.run_speculative(prompt, LmDrafter(GpuTarget(lm), prompt[0], V, noise, 9), gcfg, new, block, adaptive_floor=floor)
    stops = [int(free["tokens"][len(free["tokens"]) // 2]), int(r.integers(0, V))]
    for stop_tokens in ([], stops):
        want = ob.run_speculative(GpuTarget(gpu), LmDrafter(GpuTarget(lm), prompt[0], V, noise, 9), prompt, ocfg, new, block,
                                  V, cfg["max_context"], stop_tokens=stop_tokens, adaptive_floor=floor)
        got = gpu.run_speculative(prompt, LmDrafter(GpuTarget(lm), prompt[0], V, noise, 9), gcfg, new, block,
                                  stop_tokens=stop_tokens, adaptive_floor=floor)
        assert {k: got[k] for k in KEYS} == {k: want[k] for k in KEYS}
        assert got["min_margin"] > 1e-10
    assert got["stop_reason"] == 1 and got["tokens"] == free["tokens"][: free["tokens"].index(stops[0])]


class DeviceLmDrafter(LmDrafter):
    """The same drafter leaving its logits on the GPU: a pass of the drafter's own handle, then a
    device-to-device copy into the row the loop hands over."""

    def step_device(self, token, position, address):
        import ctypes as C
        from turbospark_amd import hip
        idx = position + 1
        if self.pos == 0:
            self.t.prefill(self.first, 0)
            self.pos = 1
        assert idx == self.pos, (idx, self.pos)
        eng = self.t.e
        eng.verify([int(token)], idx, want_logits=False)
        self.pos = idx + 1
        hip.check(hip.rt().hipStreamSynchronize(C.c_void_p(eng.stream)), "sync")
        hip.check(hip.rt().hipMemcpy(C.c_void_p(address), C.c_void_p(eng.device_logits), self.vocab * 2, 3), "copy D2D")


@pytest.mark.parametrize("temperature,kw", [(0.0, {}), (0.9, dict(top_p=0.95, repetition_penalty=1.2))])
def test_a_drafter_that_leaves_its_logits_on_the_device(temperature, kw):
    """tsv_drafter.device_logits: the draws and the round read the drafter's rows in device memory;
    the run equals the one whose drafter hands back host logits."""
    import turbospark_amd as ts
    cfg, gpu, lm = _pair(draft_seed=77 if temperature == 0.0 else 1234)
    V = cfg["vocab"]
    prompt = np.random.default_rng(4).integers(0, V, 14).astype(np.int32)
    gcfg = ts.shaping(temperature, seed=5 if temperature else None, **kw)
    host = gpu.run_speculative(prompt, LmDrafter(GpuTarget(lm), prompt[0], V), gcfg, 40, 5)
    dev = gpu.run_speculative(prompt, DeviceLmDrafter(GpuTarget(lm), prompt[0], V), gcfg, 40, 5, device_logits=True)
    assert {k: dev[k] for k in KEYS} == {k: host[k] for k in KEYS}
    assert len(dev["tokens"]) == 40


@pytest.mark.parametrize("nodes,stop_at", [(7, None), (15, None), (7, 30)])
def test_tree_rounds_in_the_loop_report_what_the_reference_loop_reports(nodes, stop_at):
    """speculative.rs:467-575: greedy, fixed-depth rounds of a drafter that offers trees of `block` nodes
    run as draft_tree -> verify_tree -> the walk -> compact_tree -> rollback_retaining.  The library does
    everything after the draft in one device round; the oracle's restatement drives the same GPU target
    through verify_tree / compact_tree with the walk on the host.  Tokens, stop reason and every counter
    agree, the output is plain greedy decoding, and rounds that the budget shortens fall back to chains."""
    import turbospark_amd as ts
    cfg, gpu, lm = _pair()
    V = cfg["vocab"]
    prompt = np.random.default_rng(5).integers(0, V, 11).astype(np.int32)
    new = 60

    def drafter():
        return TreeTwinDrafter(GpuTarget(lm), prompt[0], V, nodes, seed=2)

    plain = gpu.run_speculative(prompt, LmDrafter(GpuTarget(lm), prompt[0], V), ts.shaping(0.0), new, 4)["tokens"]
    stops = [plain[stop_at]] if stop_at is not None else []
    want = ob.run_speculative(GpuTarget(gpu), drafter(), prompt, ob.shaping(0.0), new, nodes, V, cfg["max_context"],
                              stop_tokens=stops)
    got = gpu.run_speculative(prompt, drafter(), ts.shaping(0.0), new, nodes, stop_tokens=stops)
    print({k: (got[k] if k != "tokens" else len(got[k])) for k in KEYS})
    assert {k: got[k] for k in KEYS} == {k: want[k] for k in KEYS}
    if stops:
        cut = plain.index(stops[0])
        assert got["tokens"] == plain[:cut] and got["stop_reason"] == 1
    else:
        assert got["tokens"] == plain and got["stop_reason"] == 2
        assert got["kv_position"] == len(prompt) + new - 1 == gpu.position
    assert 0 < got["accepted"] < got["offered"] and got["rollbacks"] > 0
    # the next token after the run continues from a cache that only ever kept accepted paths
    if not stops:
        nxt = gpu.produce(got["tokens"][-1], gpu.position)
        gpu.reset()
        gpu.prefill(np.concatenate([prompt, np.array(got["tokens"][:-1], np.int32)]), 0, want_logits=False)
        assert gc.logit_error(nxt[None], gpu.produce(got["tokens"][-1], gpu.position)[None]) <= 2e-3
