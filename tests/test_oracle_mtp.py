"""The oracle's drafter-head step (docs/MTP.md:53-60, crates/runtime/src/families/qwen/mtp.rs) pinned without
the oracle's own formulas: fc's input against an independent float64 restatement (with the plausible mistakes
shown to miss it), and the layer it feeds against the already pinned forward pass by the cases in which the
step must reduce to it."""
import numpy as np
import pytest

from oracle import binding as ob
from turbospark_amd import ffi, synth


def _f32(entry):
    dtype, data, rows, cols = entry
    return ob.dequantize(dtype, data, cols).reshape(rows, cols).astype(np.float64)


def _rms(x, w, eps):
    return x * w / np.sqrt(np.mean(x * x) + eps)


def _setup(name="tiny_q8_0", ctx=64, jitter=0.25):
    cfg = dict(synth.CONFIGS[name], max_context=ctx, norm_jitter=jitter)
    w = synth.make_weights(cfg, seed=11)
    hcfg, hw = synth.make_mtp_weights(cfg, w, seed=12)
    return cfg, w, hcfg, hw


def test_fc_input_is_embedding_half_first_and_the_state_goes_through_the_trunk_norm_first():
    cfg, w, hcfg, hw = _setup()
    H, eps = cfg["hidden"], cfg["rms_eps"]
    head = ob.MtpHead(hcfg, hw, round_kv_f16=False)
    rng = np.random.default_rng(0)
    toks = rng.integers(0, cfg["vocab"], 3)
    h = rng.standard_normal((3, H)).astype(np.float32) * 3.0
    _, x0 = head.step(toks, h, 0, want=None, want_x0=True)

    E, FC = _f32(hw["embed"]), _f32(hw["fc"])
    we, wh, wt = _f32(hw["norm_embedding"])[0], _f32(hw["norm_hidden"])[0], _f32(hw["trunk_norm"])[0]

    def restate(order="eh", trunk_norm=True, norm_e=True):
        out = []
        for r in range(3):
            e = E[toks[r]]
            ne = _rms(e, we, eps) if norm_e else e
            t = _rms(h[r].astype(np.float64), wt, eps) if trunk_norm else h[r].astype(np.float64)
            nh = _rms(t, wh, eps)
            out.append(FC @ (np.concatenate([ne, nh]) if order == "eh" else np.concatenate([nh, ne])))
        return np.array(out)

    want = restate()
    scale = np.abs(want).max()
    assert np.abs(x0 - want).max() <= 2e-5 * scale
    # the mistakes a restatement could make are far outside that bound
    for wrong in (restate(order="he"), restate(trunk_norm=False), restate(norm_e=False)):
        assert np.abs(wrong - want).max() > 1e-2 * scale


def test_the_head_layer_is_the_pinned_forward_pass_on_fcs_rows():
    """With fc = [I 0] and unit norm_embedding the rows entering the layer are rms-normalised embeddings; a model
    whose embedding table holds exactly those rows must give the same logits and cache rows by its ordinary pass."""
    cfg, w, hcfg, hw = _setup(jitter=0.0)
    H, V, eps = cfg["hidden"], cfg["vocab"], cfg["rms_eps"]
    eye = np.concatenate([np.eye(H, dtype=np.float32), np.zeros((H, H), np.float32)], axis=1)
    hw = dict(hw, fc=(ffi.F32, eye.view(np.uint8).reshape(H, -1), H, 2 * H),
              norm_embedding=(ffi.F32, np.ones((1, H), np.float32).view(np.uint8).reshape(1, -1), 1, H))
    head = ob.MtpHead(hcfg, hw, round_kv_f16=False)
    E = _f32(hw["embed"])
    En = (E / np.sqrt(np.mean(E * E, axis=1, keepdims=True) + eps)).astype(np.float32)
    plain = ob.Model(hcfg, dict(hw, embed=(ffi.F32, En.view(np.uint8).reshape(V, -1), V, H)), round_kv_f16=False)
    rng = np.random.default_rng(1)
    toks = rng.integers(0, V, 5)
    h = rng.standard_normal((5, H)).astype(np.float32)      # multiplied by fc's zero half
    (_, got) = head.step(toks[:3], h[:3], 0, want="f32")
    (_, more) = head.step(toks[3:], h[3:], 3, want="f32")
    _, want = plain.verify(toks, 0, want_f32=True)
    rng_ = want.max() - want.min()
    assert np.abs(np.concatenate([got, more]) - want).max() <= 1e-5 * rng_
    k1, v1 = head.model.kv(0)
    k2, v2 = plain.kv(0)
    assert np.abs(k1[:5] - k2[:5]).max() <= 1e-5 and np.abs(v1[:5] - v2[:5]).max() <= 1e-5
    assert head.position == 5


def test_rows_of_one_call_are_the_rows_of_single_steps_and_a_priming_step_leaves_the_same_cache_row():
    cfg, w, hcfg, hw = _setup()
    H, V = cfg["hidden"], cfg["vocab"]
    rng = np.random.default_rng(2)
    toks = rng.integers(0, V, 6)
    h = rng.standard_normal((6, H)).astype(np.float32)
    a, b = ob.MtpHead(hcfg, hw), ob.MtpHead(hcfg, hw)
    batch = a.step(toks, h, 0)
    single = [b.step(toks[i:i + 1], h[i:i + 1], i, want=("f16" if i % 2 else None)) for i in range(6)]
    for i in range(1, 6, 2):
        assert np.array_equal(batch[i], single[i][0])
    assert np.array_equal(a.model.kv(0)[0][:6], b.model.kv(0)[0][:6])
    # the head's residual after a step is what a chained step reads
    assert np.array_equal(a.last_hidden(5), b.last_hidden(0))
    # rewinding and stepping again from the same pair reproduces the row
    b.rewind_to(5)
    assert np.array_equal(b.step(toks[5:], h[5:], 5)[0], batch[5])


def test_refusals_by_name():
    cfg, w, hcfg, hw = _setup()
    head = ob.MtpHead(hcfg, hw)
    h = np.zeros((1, cfg["hidden"]), np.float32)
    with pytest.raises(ValueError, match="position"):
        head.step([1], h, 3)
    with pytest.raises(ValueError, match="vocabulary"):
        head.step([cfg["vocab"]], h, 0)


def test_the_trunk_exposes_the_rows_its_final_norm_consumes():
    """last_hidden is the pre-final-norm stream: norm + output head applied to it by hand give the logits."""
    cfg, w, _, _ = _setup()
    m = ob.Model(cfg, w, round_kv_f16=False)
    toks = [5, 9, 200]
    _, logits = m.verify(toks, 0, want_f32=True)
    W = _f32(w["lm_head"])
    wn = _f32(w["final_norm"])[0]
    for r in range(3):
        x = m.last_hidden(r).astype(np.float64)
        want = W @ _rms(x, wn, cfg["rms_eps"])
        assert np.abs(logits[r] - want).max() <= 1e-4 * (want.max() - want.min())
    # a pass taken for its rows alone leaves the same stream and cache rows
    m2 = ob.Model(cfg, w, round_kv_f16=False)
    m2.prime(toks, 0)
    assert np.array_equal(m2.last_hidden(2), m.last_hidden(2)) and m2.position == 3
    assert np.array_equal(m2.kv(1)[0][:3], m.kv(1)[0][:3])
