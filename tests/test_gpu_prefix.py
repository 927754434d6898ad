"""Prefix reuse through the C ABI (LogitProducer::try_reuse_prefix, producer.rs:24-47;
real_forward_traits.rs:173-289; SpeculativeProducer::record_committed, producer.rs:322-330; the
loop's reuse contract, speculative.rs:240-251).  Reuse must never change what is generated: a turn
that continues from the previous turn's cache reports the tokens of a turn that started from
nothing."""
import numpy as np
import pytest

from tests import gpu_common as gc
from turbospark_amd import ffi
from tests.loop_common import GpuTarget, LmDrafter

pytestmark = pytest.mark.gpu


class ContinuingDrafter(LmDrafter):
    """An LmDrafter that says where it stands, so the loop may take over a prefix."""

    def context_position(self):
        return self.pos - 1  # prime / step calls taken so far: positions 0 .. pos - 2


def _target(max_context=200):
    return gc.build_pair("tiny_q8_0", max_context=max_context)


def test_reuse_answers_nothing_until_the_host_opts_in_and_keys_on_what_was_fed():
    cfg, w, gpu, _ = _target()
    V = cfg["vocab"]
    ids = np.random.default_rng(1).integers(0, V, 40).astype(np.int32)
    gpu.reset()
    gpu.prefill(ids[:30], 0, want_logits=False)
    assert gpu.prefix_len() == 30
    assert gpu.try_reuse_prefix(ids) == 0                      # not opted in
    gpu.set_prefix_reuse(True)
    assert gpu.try_reuse_prefix(ids) == 30 and gpu.position == 30
    # token by token on top of the block, then a prompt that diverges inside the record
    for i in range(30, 34):
        gpu.produce(int(ids[i]), i)
    assert gpu.prefix_len() == 34
    other = ids.copy()
    other[20] = (other[20] + 1) % V
    assert gpu.try_reuse_prefix(other) == 20
    assert gpu.position == 20 and gpu.prefix_len() == 20       # the cursor went back with the record
    # an exact repeat leaves one token to feed
    assert gpu.try_reuse_prefix(ids[:20]) == 19 and gpu.position == 19
    # verify rows are described only once the caller reports them
    feed = ids[19:24]
    gpu.verify(feed, 19, want_logits=False)
    assert gpu.position == 24 and gpu.prefix_len() == 19
    gpu.record_committed(feed[:3], 19)
    assert gpu.prefix_len() == 22
    gpu.rollback_retaining(ffi.Point(19), 3)
    assert gpu.position == 22 and gpu.try_reuse_prefix(ids) == 22
    # a plain rollback shortens the record with the cache
    gpu.rollback(ffi.Point(10))
    assert gpu.prefix_len() == 10 and gpu.try_reuse_prefix(ids) == 10
    # rows written without token ids describe nothing reusable until the next reset
    k, v = gpu.read_kv(0, 0, 4)
    gpu.write_kv(0, 0, k, v)
    assert gpu.prefix_len() is None and gpu.try_reuse_prefix(ids) == 0
    gpu.reset()
    assert gpu.prefix_len() == 0 and gpu.try_reuse_prefix(ids) == 0


def test_a_reused_prefix_gives_the_logits_of_a_fresh_prefill():
    cfg, w, gpu, _ = _target()
    V = cfg["vocab"]
    rng = np.random.default_rng(2)
    first = rng.integers(0, V, 50).astype(np.int32)
    second = np.concatenate([first[:37], rng.integers(0, V, 20).astype(np.int32)])
    gpu.reset()
    fresh = gc.f16(gpu.prefill(second, 0))
    gpu.reset()
    gpu.set_prefix_reuse(True)
    gpu.prefill(first, 0, want_logits=False)
    keep = gpu.try_reuse_prefix(second)
    assert keep == 37 and gpu.position == 37
    again = gc.f16(gpu.prefill(second[keep:], keep))
    assert gpu.position == len(second) and gpu.prefix_len() == len(second)
    span = float(fresh.max() - fresh.min())
    assert float(np.abs(again - fresh).max()) <= 2e-3 * span   # the Q8_0 bar on logits
    assert int(np.argmax(again)) == int(np.argmax(fresh))


@pytest.mark.parametrize("temperature", [0.0, 0.8])
def test_a_second_turn_continues_from_the_first_turns_cache(temperature):
    import turbospark_amd as ts
    from turbospark_amd import synth
    cfg, w, gpu, _ = _target(max_context=256)
    V = cfg["vocab"]
    dcfg = dict(synth.CONFIGS["tiny_q8_0"], max_context=256)
    lm = ts.HipVerifier(dcfg, w)
    shaping = ts.shaping(temperature, seed=5) if temperature else ts.shaping(0.0)
    rng = np.random.default_rng(3)
    prompt1 = rng.integers(0, V, 14).astype(np.int32)
    gpu.set_prefix_reuse(True)
    drafter = ContinuingDrafter(GpuTarget(lm), prompt1[0], V, 0.5, 9)
    one = gpu.run_speculative(prompt1, drafter, shaping, 24, 4)
    assert one["reused"] == 0 and one["stop_reason"] == 2
    held = one["kv_position"]                     # rows the first turn left behind
    assert gpu.prefix_len() == held and drafter.context_position() == held - 1
    # the chat client sends the transcript back: prompt, the reply, the next message
    reply = one["tokens"][: held - len(prompt1)]
    prompt2 = np.concatenate([prompt1, np.asarray(reply, np.int32), rng.integers(0, V, 9).astype(np.int32)])
    two = gpu.run_speculative(prompt2, drafter, shaping, 24, 4)
    assert two["reused"] == held
    # the same turn from nothing: another handle, another drafter, no reuse
    _, _, gpu_b, _ = _target(max_context=256)
    lm_b = ts.HipVerifier(dcfg, w)
    base = gpu_b.run_speculative(prompt2, ContinuingDrafter(GpuTarget(lm_b), prompt2[0], V, 0.5, 9), shaping, 24, 4)
    assert base["reused"] == 0
    for key in ("tokens", "stop_reason", "rounds", "offered", "accepted", "rollbacks", "draw_step", "kv_position"):
        assert two[key] == base[key], key
    # a transcript that diverges inside the reply is not a pure continuation: with a drafter
    # attached the loop starts over (real_forward_traits.rs:222-239)
    prompt3 = prompt2.copy()
    prompt3[len(prompt1) + 2] = (prompt3[len(prompt1) + 2] + 1) % V
    drafter3 = ContinuingDrafter(GpuTarget(lm), prompt3[0], V, 0.5, 9)
    three = gpu.run_speculative(prompt3, drafter3, shaping, 8, 4)
    assert three["reused"] == 0
    # and a drafter that does not say where it stands never reuses
    four = gpu.run_speculative(prompt3, LmDrafter(GpuTarget(lm), prompt3[0], V, 0.5, 9), shaping, 8, 4)
    assert four["reused"] == 0 and four["tokens"] == three["tokens"]


def test_headless_prefill_passes_leave_the_rows_of_full_passes():
    """produce_prefill (producer.rs:92-103): skipping the output head must not change any other side
    effect of the pass -- the cache rows and the cursor are those of a pass that paid for the head."""
    import turbospark_amd as ts
    cfg, w, gpu, _ = _target()
    V = cfg["vocab"]
    ids = np.random.default_rng(4).integers(0, V, 45).astype(np.int32)
    gpu.reset()
    gpu.prefill(ids, 0, want_logits=False)                     # three passes, none of them runs the head
    assert gpu.position == 45
    rows_a = [gpu.read_kv(layer, 0, 45) for layer in range(cfg["n_layers"])]
    with pytest.raises(ts.ffi.TsvError):                       # no rows on the device to judge
        gpu.accept(ids[:5], 40, ts.shaping(0.0))
    after_a = gpu.produce(7, 45)
    gpu.reset()
    last = gpu.prefill(ids, 0)                                 # the last pass pays for the head
    rows_b = [gpu.read_kv(layer, 0, 45) for layer in range(cfg["n_layers"])]
    for (ka, va), (kb, vb) in zip(rows_a, rows_b):
        assert np.array_equal(ka.view(np.uint16), kb.view(np.uint16))
        assert np.array_equal(va.view(np.uint16), vb.view(np.uint16))
    assert np.array_equal(after_a, gpu.produce(7, 45))
    # and the row handed out is the row token-by-token decoding gives for the last prompt token
    gpu.reset()
    gpu.prefill(ids[:-1], 0, want_logits=False)
    one = gpu.produce(int(ids[-1]), 44)
    assert gc.logit_error(last, one) <= 2e-3
