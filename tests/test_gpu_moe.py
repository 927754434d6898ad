"""GPU parity of the routed-expert (MoE) verify pass against the oracle: Q8_0 attention and
router, MXFP4 experts, top-k routing with softmax over the selected logits (the arrangement of
the Qwen3-30B-A3B configuration, crates/runtime/src/families/llama/moe.rs)."""
import numpy as np
import pytest

from tests import gpu_common as gc

pytestmark = pytest.mark.gpu

MXFP4_TOL = 1e-2   # max-abs logit error relative to the logit range, MXFP4 / Q4_K bar


def _prompt(n, vocab, seed):
    return np.random.default_rng(seed).integers(0, vocab, n).astype(np.int32)


def _clean_inputs(cfg, cpu, ctx, k, floor=1e-3):
    """Seeded prompt + feed for which no routing decision of the reference run is a near tie (the
    GPU's router logits carry fp16-activation rounding, a few 1e-4 of the logit range, so a
    closer call could legitimately go the other way and the comparison would mean nothing).
    Leaves the oracle advanced past both; returns its verify logits."""
    for attempt in range(40):
        prompt = _prompt(ctx, cfg["vocab"], 7 + 100 * attempt)
        feed = _prompt(k + 1, cfg["vocab"], 8 + 100 * attempt)
        cpu.reset()
        margins = []
        for i in range(0, ctx, 16):
            cpu.verify(prompt[i:i + 16], i)
            margins.append(cpu.route_margin)
        want = cpu.verify(feed, ctx)
        margins.append(cpu.route_margin)
        if min(margins) > floor:
            return prompt, feed, want, min(margins)
    raise AssertionError("no seed without a near-tie routing decision in 40 tries")


@pytest.mark.parametrize("ctx,k", [(40, 8), (21, 4), (33, 15), (16, 0)])
def test_moe_verify_logits_match_the_oracle(ctx, k):
    cfg, w, gpu, cpu = gc.build_pair("moe_small", max_context=ctx + 32)
    prompt, feed, want, margin = _clean_inputs(cfg, cpu, ctx, k)
    gpu.prefill(prompt, 0, want_logits=False)
    got = gpu.verify(feed, ctx)
    err = gc.logit_error(got, want)
    print(f"moe_small ctx={ctx} m={k+1}: max-abs logit error / range = {err:.2e}, route margin {margin:.3e}")
    assert err <= MXFP4_TOL, err
    for layer in range(cfg["n_layers"]):
        kg, vg = gpu.read_kv(layer, 0, ctx)
        kc, vc = cpu.kv(layer)
        assert np.abs(kg.astype(np.float32) - kc[:ctx]).max() <= 2e-2 * np.abs(kc[:ctx]).max()


def test_moe_batched_pass_equals_the_same_tokens_fed_one_at_a_time():
    """Row invariance with routed experts: an expert multiplies only the rows that chose it, and a
    row's result must not depend on which other rows share its experts."""
    cfg, w, gpu, cpu = gc.build_pair("moe_small", max_context=96)
    prompt = _prompt(30, cfg["vocab"], 3)
    gpu.prefill(prompt, 0, want_logits=False)
    feed = _prompt(9, cfg["vocab"], 4)
    point = gpu.checkpoint()
    batch = gpu.verify(feed, 30)
    gpu.rollback(point)
    seq = np.stack([gpu.produce(t, 30 + i) for i, t in enumerate(feed)])
    assert np.array_equal(batch, seq)


def test_moe_greedy_round_matches_the_oracle_walk():
    """Configuration-4 style round: chain k=8, greedy acceptance on the MoE target's logits."""
    import turbospark_amd as ts
    from oracle import binding as ob
    cfg, w, gpu, cpu = gc.build_pair("moe_small", max_context=96)
    prompt = _prompt(24, cfg["vocab"], 5)
    gpu.prefill(prompt[:-1], 0, want_logits=False)
    cpu.verify(prompt[:-1], 0)
    base = gpu.position
    # proposals: the oracle's own greedy continuation for the first 3, then junk -> accepted == 3
    point_tokens = [int(prompt[-1])]
    for i in range(3):
        lg = cpu.verify(point_tokens[-1:], base + i)
        point_tokens.append(int(np.argmax(gc.f16(lg[0]))))
    cpu.rewind_to(base)
    feed = point_tokens + [1, 2, 3, 4, 5]
    logits = gc.f16(cpu.verify(feed, base))
    want_acc = 0
    for i in range(8):
        if int(np.argmax(logits[i])) == feed[i + 1]:
            want_acc += 1
        else:
            break
    res = gpu.verify_accept(feed, base, ts.shaping(0.0))
    assert res.accepted == want_acc >= 3
    assert res.next == int(np.argmax(logits[want_acc]))
    assert res.kv_position == base + want_acc + 1


@pytest.mark.parametrize("top_k", [1, 3, 5])
def test_exactly_tied_router_logits_go_to_the_lower_expert(top_k):
    """real_forward_dispatch.rs:1135-1158: experts sort by logit, ties to the lower index.  Every odd
    expert's router row is a copy of its even neighbour's, so each logit comes twice, bit for bit,
    and with an odd top-k the last selection is always one half of a tied pair.  The experts
    themselves differ, so taking the wrong half changes the logits far beyond the tolerance."""
    import turbospark_amd as ts
    from oracle import binding as ob
    from turbospark_amd import synth
    cfg = dict(synth.CONFIGS["moe_small"], max_context=64, top_k=top_k)
    w = synth.make_weights(cfg, seed=77)
    for lw in w["layers"]:
        dt, raw, rows, cols = lw["router"]
        raw = raw.copy()
        raw[1::2] = raw[0::2]
        lw["router"] = (dt, raw, rows, cols)
    gpu = ts.HipVerifier(cfg, w)
    cpu = ob.Model(cfg, w, round_kv_f16=True, threads=8)
    prompt, feed = _prompt(24, cfg["vocab"], 3), _prompt(9, cfg["vocab"], 4)
    for i in range(0, 24, 16):
        cpu.verify(prompt[i:i + 16], i)
    want = cpu.verify(feed, 24)
    gpu.prefill(prompt, 0, want_logits=False)
    err = gc.logit_error(gpu.verify(feed, 24), want)
    print(f"tied router, top-{top_k}: max-abs logit error / range = {err:.2e}")
    assert err <= MXFP4_TOL, err


@pytest.mark.parametrize("name,over", [("qwen3_30b_a3b", dict(vocab=4096)), ("gptoss_120b", dict(vocab=4096))])
def test_routing_agrees_with_the_oracle_except_within_rounding_of_a_tie(name, over):
    """Unfiltered seeds at the two routed configurations' router shapes (128 experts, top-8 of a 2048-wide
    and top-4 of a 2880-wide stream, two layers): how often the GPU's expert set of a row differs from
    the oracle's ranking (real_forward_dispatch.rs:1135-1158), and at what margin.  The GPU's router
    input carries fp16 rounding (a few 1e-4 of the logit range), so a decision can legitimately go the
    other way only when the last chosen and the first rejected logit are closer than that: every
    disagreement must be such a near tie, and with the oracle forced onto the GPU's experts the logits
    must agree again."""
    import turbospark_amd as ts
    from oracle import binding as ob
    from turbospark_amd import synth
    cfg = dict(synth.CONFIGS[name], max_context=64, n_layers=2, **over)
    w = synth.make_weights(cfg, seed=21, n_layers=2)
    gpu = ts.HipVerifier(cfg, w)
    cpu = ob.Model(cfg, w, round_kv_f16=True, threads=16)
    K = cfg["top_k"]
    rows = differ = 0
    worst_gap, checked = 0.0, 0
    bound = 5e-3
    for rnd in range(60):
        feed = _prompt(16, cfg["vocab"], 1000 + rnd)
        gpu.reset()
        cpu.reset()
        cpu.force_route(None)
        got = gpu.verify(feed, 0)
        want = cpu.verify(feed, 0)
        gsel = np.sort(gpu.route_selected()[:, :, :K], axis=-1)
        osel_raw, gap = cpu.route_record()
        osel = np.sort(osel_raw[:, :, :K], axis=-1)
        bad = np.any(gsel != osel, axis=-1).reshape(-1)   # [layer * 16 + row]: the order decisions are made in
        if bad.any():
            # only the earliest disagreement of a pass is a clean sample: everything after it (the row's
            # later layers, later rows through attention) sees inputs the oracle's run no longer shares
            first = int(np.argmax(bad))
            rows += first + 1
            differ += 1
            g = float(gap.reshape(-1)[first])
            assert g < bound, (rnd, first, g)
            worst_gap = max(worst_gap, g)
            if checked < 6:
                # the oracle on the GPU's own routing: the logits agree again
                cpu.reset()
                cpu.force_route(gpu.route_selected())
                forced = cpu.verify(feed, 0)
                assert gc.logit_error(got, forced) <= MXFP4_TOL
                cpu.force_route(None)
                checked += 1
        else:
            rows += bad.size
            assert gc.logit_error(got, want) <= MXFP4_TOL
    print(f"{name} router shape: {differ} of {rows} routing decisions (a row's expert set in a layer) differ from the oracle's, "
          f"largest margin among them {worst_gap:.2e} of the logit range (bound {bound:.0e})")
    assert differ <= rows // 50


@pytest.mark.parametrize("name,over", [("moe_small", {}), ("gptoss_small", {}), ("qwen3_30b_a3b", dict(vocab=4096, n_layers=2)),
                                       ("gptoss_120b", dict(vocab=4096, n_layers=2))])
def test_parity_on_unfiltered_inputs_with_the_oracles_routing_forced_onto_the_device(name, over):
    """No seed is re-drawn here: the oracle routes freely (real_forward_dispatch.rs:1135-1158), its expert
    sets are forced onto the device (tsv_force_route), and the logits must agree on every input -- also on
    those where the device's own ranking would have gone the other way inside the rounding of a tie."""
    import turbospark_amd as ts
    from oracle import binding as ob
    from turbospark_amd import synth
    cfg = dict(synth.CONFIGS[name], max_context=64, **over)
    w = synth.make_weights(cfg, seed=33, n_layers=cfg["n_layers"])
    gpu = ts.HipVerifier(cfg, w)
    cpu = ob.Model(cfg, w, round_kv_f16=True, threads=16)
    worst, flips = 0.0, 0
    rounds = 24 if cfg["hidden"] <= 1024 else 10
    for rnd in range(rounds):
        feed = _prompt(1 + rnd % 16, cfg["vocab"], 5000 + rnd)
        cpu.reset()
        want = cpu.verify(feed, 0)
        sel, _ = cpu.route_record()
        gpu.reset()
        gpu.force_route(None)
        free = gpu.verify(feed, 0)
        own = gpu.route_selected()
        K = cfg["top_k"]
        flips += int(np.any(np.sort(own[:, :len(feed), :K], -1) != np.sort(sel[:, :len(feed), :K], -1)))
        forced = np.full((cfg["n_layers"], 16, 8), -1, np.int32)
        forced[:, :len(feed), :K] = sel[:, :len(feed), :K]
        gpu.reset()
        gpu.force_route(forced)
        got = gpu.verify(feed, 0)
        assert np.array_equal(np.sort(gpu.route_selected()[:, :len(feed), :K], -1), np.sort(forced[:, :len(feed), :K], -1))
        worst = max(worst, gc.logit_error(got, want))
        assert gc.logit_error(got, want) <= MXFP4_TOL, (rnd, gc.logit_error(got, want))
        del free
    gpu.force_route(None)
    print(f"{name}: {rounds} unfiltered passes under the oracle's routing, worst logit error / range {worst:.2e}; "
          f"the device's own ranking differed somewhere in {flips} of them")
