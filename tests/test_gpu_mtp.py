"""The drafter head inside the library (docs/MTP.md:53-60, crates/runtime/src/families/qwen/mtp.rs) against the
oracle's restatement of the recurrence, and the loop's block-draft and chunked-prefill callbacks
(producer.rs:193-250) against the token-at-a-time, step-by-step walk of the same head."""
import numpy as np
import pytest

import turbospark_amd as ts
from oracle import binding as ob
from tests import gpu_common as gc
from tests.loop_common import GpuTarget
from turbospark_amd import ffi, synth

pytestmark = pytest.mark.gpu

KEYS = ("tokens", "stop_reason", "rounds", "offered", "accepted", "rollbacks", "draw_step", "final_depth")


def _build(name, ctx=160, oracle=True, **over):
    cfg = dict(synth.CONFIGS[name], max_context=ctx)
    cfg.update(over)
    w = synth.make_weights(cfg, seed=1234)
    hcfg, hw = synth.make_mtp_weights(cfg, w, seed=77, follow=over.get("follow", 0.0))
    gpu = ts.HipVerifier(cfg, w)
    head = ts.MtpHead(gpu, hcfg, hw)
    if not oracle:
        return cfg, gpu, head
    return cfg, gpu, head, ob.Model(cfg, w, threads=8), ob.MtpHead(hcfg, hw, threads=8)


def _amax(bits):
    return int(np.argmax(gc.f16(bits)))


@pytest.mark.parametrize("name", ["tiny_q8_0", "small_q4_k", "xcd_q4_k", "moe_small", "gptoss_small"])
def test_the_heads_logits_match_the_oracle_through_priming_steps_chained_steps_and_a_rewind(name):
    cfg, gpu, head, trunk, ohead = _build(name)
    V = cfg["vocab"]
    tol = gc.TOL.get(cfg["dtype"], 1e-2)
    prompt = np.random.default_rng(4).integers(0, V, 21).astype(np.int32)
    n = len(prompt)
    # the prompt: the target's prefill primes the head over every position whose next token is known
    last = head.prefill_chunk(prompt, 0)
    want_last = trunk.verify(prompt, 0)[-1]
    assert gc.logit_error(last, want_last) <= tol
    ohead.step(prompt[1:], np.array([trunk.last_hidden(r) for r in range(n - 1)]), 0, want=None)
    assert head.position == n - 1 == ohead.position
    k_got, v_got = head.read_kv(0, n - 1)
    k_want, v_want = ohead.model.kv(0)
    assert np.abs(k_got.astype(np.float32).reshape(n - 1, -1) - k_want[:n - 1].reshape(n - 1, -1)).max() <= 3e-2
    # a round: the step from the target's state, two chained steps from the head's own
    nxt = _amax(want_last)
    base = n
    got = head.step(nxt, base - 1)
    want = ohead.step([nxt], trunk.last_hidden(n - 1), base - 1)[0]
    errs = [gc.logit_error(got, want)]
    feed = [nxt]
    for d in (1, 2):
        tok = _amax(want)
        feed.append(tok)
        got = head.step(tok, base - 1 + d)
        want = ohead.step([tok], ohead.last_hidden(0), base - 1 + d)[0]
        errs.append(gc.logit_error(got, want))
    # the target verifies the three tokens; say one proposal was committed: both heads go back to base + 1
    gpu.verify(feed, base, want_logits=False)
    trunk.verify(feed, base)
    head.rewind(base + 1)
    ohead.rewind_to(base + 1)
    got = head.step(7, base + 1)
    want = ohead.step([7], trunk.last_hidden(1), base + 1)[0]
    errs.append(gc.logit_error(got, want))
    print(name, "head logit error / range per step:", ["%.2e" % e for e in errs])
    assert max(errs) <= tol


# the longer prompts go through 64-row passes, which prime the head too (Q8_0: the rotation as a kernel of its own
# under TSV_ROPE_FUSED=0 elsewhere, here the epilogue; routed layers: the experts' members over 64 rows)
@pytest.mark.parametrize("name,n", [("xcd_q4_k", 37), ("xcd_q4_k", 171), ("xcd_q8_0", 171), ("moe_small", 171)])
def test_priming_by_the_prefill_equals_priming_token_by_token(name, n):
    cfg, gpu_a, head_a = _build(name, ctx=200, oracle=False)
    _, gpu_b, head_b = _build(name, ctx=200, oracle=False)
    V = cfg["vocab"]
    prompt = np.random.default_rng(6).integers(0, V, n).astype(np.int32)
    la = head_a.prefill_chunk(prompt[:20], 0, next_token=int(prompt[20]))   # two chunks, the first names its next token
    assert head_a.position == 20
    la = head_a.prefill_chunk(prompt[20:], 20)
    for i in range(n):
        lb = gpu_b.produce(int(prompt[i]), i)
        if i + 1 < n:
            head_b.prime(int(prompt[i + 1]), i)
    # (passes of different row counts split their sums differently: equal to rounding, not to the bit)
    assert gc.logit_error(la, lb) <= 5e-4
    assert head_a.position == head_b.position == n - 1
    ka, va = head_a.read_kv(0, n - 1)
    kb, vb = head_b.read_kv(0, n - 1)
    assert np.abs(ka.astype(np.float32) - kb.astype(np.float32)).max() <= 4e-3 * np.abs(kb.astype(np.float32)).max()
    assert np.abs(va.astype(np.float32) - vb.astype(np.float32)).max() <= 4e-3 * np.abs(vb.astype(np.float32)).max()
    assert gc.logit_error(head_a.step(11, n - 1), head_b.step(11, n - 1)) <= 5e-4


@pytest.mark.parametrize("block", [1, 4, 15])
def test_a_block_draft_is_the_chain_of_single_steps(block):
    cfg, gpu, head = _build("small_q4_k", oracle=False)
    V = cfg["vocab"]
    prompt = np.random.default_rng(8).integers(0, V, 18).astype(np.int32)
    n = len(prompt)
    anchor = _amax(head.prefill_chunk(prompt, 0))
    chain, tok = [], anchor
    for d in range(block):
        tok = _amax(head.step(tok, n - 1 + d))
        chain.append(tok)
    head.rewind(n - 1)
    got = head.draft_block(anchor, n, block)
    assert got == chain
    assert head.position == n + block      # the row-only step of the last proposal is in
    # nothing was committed: back to where the round began, and the same block comes out again
    head.rewind(n - 1)
    assert head.draft_block(anchor, n, block) == chain


class _HeadDrafter:
    """The head behind the step-wise drafter methods the reference loop calls."""

    def __init__(self, head):
        self.h = head
        head.rewind(0)

    def prime(self, token, position):
        self.h.prime(token, position)

    def step(self, token, position):
        return self.h.step(token, position)

    def rewind(self, position):
        self.h.rewind(position)


@pytest.mark.parametrize("temperature,kw,block,floor,flags", [
    (0.0, {}, 4, 0, {}),                                     # block drafts, chunked prefill
    (0.0, {}, 8, 2, {}),                                     # adaptive depth
    (0.0, {}, 5, 0, dict(block_drafts=False)),               # the same head step by step
    (0.8, dict(top_p=0.95), 4, 0, {}),                       # sampled rounds: the library's own head chains them on the device
    (0.9, dict(repetition_penalty=1.3, presence_penalty=0.5, top_k=64), 6, 2, {}),   # ... with penalties over the growing history
    (0.8, dict(min_p=0.02), 4, 0, dict(block_drafts=False)), # the same head step by step on device rows
    (0.0, dict(repetition_penalty=1.3), 4, 0, {}),           # the arg-max ignores penalties
])
def test_the_loop_with_the_head_reports_what_the_reference_loop_reports(temperature, kw, block, floor, flags):
    cfg, gpu, head = _build("tiny_q8_0", ctx=200, oracle=False, weak_layers=0.03, follow=16.0)
    V = cfg["vocab"]
    prompt = np.random.default_rng(3).integers(0, V, 19).astype(np.int32)
    seed = 41 if temperature else None
    gcfg, ocfg = ts.shaping(temperature, seed=seed, **kw), ob.shaping(temperature, seed=seed, **kw)
    new = 60
    want = ob.run_speculative(GpuTarget(gpu), _HeadDrafter(head), prompt, ocfg, new, block, V, cfg["max_context"],
                              adaptive_floor=floor)
    got = gpu.run_speculative(prompt, head, gcfg, new, block, adaptive_floor=floor, **flags)
    print({k: (got[k] if k != "tokens" else len(got[k])) for k in KEYS})
    assert {k: got[k] for k in KEYS} == {k: want[k] for k in KEYS}
    assert len(got["tokens"]) == new and got["stop_reason"] == 2
    assert got["kv_position"] == len(prompt) + new - 1 == gpu.position
    assert 0 < got["accepted"] < got["offered"]      # the head proposes what the target picks often, not always
    if temperature == 0.0:
        # greedy speculation is plain decoding
        gpu.reset()
        gpu.prefill(prompt[:-1], 0, want_logits=False)
        tok, plain = int(prompt[-1]), []
        for i in range(new):
            tok = _amax(gpu.produce(tok, len(prompt) - 1 + i))
            plain.append(tok)
        assert got["tokens"] == plain
    # a second run on the same handles starts the head over
    again = gpu.run_speculative(prompt, head, gcfg, new, block, adaptive_floor=floor, **flags)
    assert again["tokens"] == got["tokens"]


def test_refusals_by_name():
    cfg, gpu, head = _build("tiny_q8_0", oracle=False)
    prompt = np.arange(5, 14, dtype=np.int32)
    with pytest.raises(ffi.TsvError, match="holds no row"):
        head.step(3, 0)                                  # nothing has run on the target yet
    head.prefill_chunk(prompt, 0)
    with pytest.raises(ffi.TsvError, match="cache covers"):
        head.step(3, 4)                                  # not where the head's cache ends
    with pytest.raises(ffi.TsvError, match="forward"):
        head.rewind(100)
    with pytest.raises(ffi.TsvError, match="must end where the chunk starts"):
        head.prefill_chunk(prompt, 0)
    with pytest.raises(ffi.TsvError, match="1..15"):
        head.draft_block(3, len(prompt), 16)
    hcfg, hw = synth.make_mtp_weights(cfg, gpu._keep[0], seed=5)
    with pytest.raises(ffi.TsvError, match="already has one"):
        ts.MtpHead(gpu, hcfg, hw)
    with pytest.raises(ffi.TsvError, match="ONE decoder layer"):
        other = ts.HipVerifier(cfg, gpu._keep[0])
        ts.MtpHead(other, dict(hcfg, hidden=cfg["hidden"] * 2), hw)
    # a drafter with neither pair of callbacks
    d = ffi.Drafter()
    ffi.check(ffi.lib().tsv_mtp_drafter(head._h, d))
    d.step = ffi.DRAFT_STEP()
    d.draft_block = ffi.DRAFT_BLOCK()
    import ctypes as C
    g = ffi.Generation()
    g.shaping, g.max_new_tokens, g.block = ts.shaping(0.0), 4, 2
    toks = np.zeros(8, np.int32)
    res = ffi.GenerationResult()
    res.tokens, res.capacity = toks.ctypes.data_as(C.POINTER(C.c_int32)), 8
    rc = ffi.lib().tsv_run_speculative(gpu._h, C.byref(d), prompt.ctypes.data, prompt.size, C.byref(g), C.byref(res))
    assert rc != 0 and "step and prime, or draft_block and prefill_chunk" in ffi.last_error()
