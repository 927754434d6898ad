"""The oracle's whole Llama-style forward against MLX known-answer logits.

The fixtures (crates/audio/testdata/lm/*, tolerance 2e-4 at crates/audio/src/lm/tests.rs:70-71)
are the only in-tree absolute logits for this graph.  They pin op order, NeoX rope, GQA head
mapping, llama-3 rope scaling, the YaRN frequency table and magnitude scale, the q / k / v
projection biases and per-head q/k norm -- and, because the decode tokens are also
fed as ONE batched verify over the prefill's cache, that a verify pass equals sequential decode.
"""
import numpy as np
import pytest

from oracle import binding as ob
from tests import lm_fixture

TOL = 2e-4


@pytest.mark.parametrize("name", ["llama_default", "llama_llama3_rope", "qwen3_default", "llama_yarn_rope", "qwen2_default"])
def test_forward_matches_mlx_traces(golden, name):
    cfg, weights, tr = lm_fixture.load(golden, name)
    tokens, dec = tr["tokens"], tr["decode_tokens"]
    want_prefill = np.array(tr["prefill_logits"], np.float32)
    want_decode = np.array(tr["decode_logits"], np.float32)

    m = ob.Model(cfg, weights, round_kv_f16=False)
    _, got = m.verify(tokens, 0, want_f32=True)
    assert np.max(np.abs(got - want_prefill)) <= TOL
    # sequential decode over the same cache
    seq = []
    for i, t in enumerate(dec):
        _, row = m.verify([t], len(tokens) + i, want_f32=True)
        seq.append(row[0])
    seq = np.array(seq)
    assert np.max(np.abs(seq - want_decode)) <= TOL

    # the same three tokens as ONE verify block over a rewound cache: bit-identical rows
    m.rewind_to(len(tokens))
    _, batch = m.verify(dec, len(tokens), want_f32=True)
    assert np.array_equal(batch, seq)

    # token-at-a-time prefill equals the batched prefill bit for bit (row invariance)
    m2 = ob.Model(cfg, weights, round_kv_f16=False)
    rows = [m2.verify([t], i, want_f32=True)[1][0] for i, t in enumerate(tokens)]
    assert np.array_equal(np.array(rows), got)


def test_a_chain_given_as_a_tree_is_the_chain_and_a_branch_sees_only_its_root_path(golden):
    cfg, weights, tr = lm_fixture.load(golden, "llama_default")
    tokens, dec = tr["tokens"], tr["decode_tokens"]
    m = ob.Model(cfg, weights, round_kv_f16=False)
    m.verify(tokens, 0)
    base = len(tokens)
    _, chain = m.verify(dec, base, want_f32=True)
    m.rewind_to(base)
    _, as_tree = m.verify(dec, base, parent=[-1, 0, 1], want_f32=True)
    assert np.array_equal(chain, as_tree)

    # tree: anchor, two children (tokens a, b), a grandchild under the second child.
    a, b, c = 5, dec[1], dec[2]
    feed = [dec[0], a, b, c]
    m.rewind_to(base)
    _, tree = m.verify(feed, base, parent=[-1, 0, 0, 2], want_f32=True)
    # slots 0,2,3 form the chain dec[0], dec[1], dec[2]: same logits as the chain rows
    assert np.max(np.abs(tree[[0, 2, 3]] - chain)) <= 1e-5
    # slot 1 equals a chain [dec[0], a]
    m.rewind_to(base)
    _, alt = m.verify([dec[0], a], base, want_f32=True)
    assert np.max(np.abs(tree[1] - alt[1])) <= 1e-5
    # compaction of path 0,2,3 then a further token == chain continuation
    m.rewind_to(base)
    m.verify(feed, base, parent=[-1, 0, 0, 2])
    m.compact_tree(base, [0, 2, 3])
    m.rewind_to(base + 3)
    _, nxt = m.verify([9], base + 3, want_f32=True)
    m.rewind_to(base)
    m.verify(dec, base)
    _, want = m.verify([9], base + 3, want_f32=True)
    assert np.array_equal(nxt, want)


def test_refusals(golden):
    cfg, weights, tr = lm_fixture.load(golden, "llama_default", max_context=8)
    m = ob.Model(cfg, weights)
    with pytest.raises(ValueError):
        m.verify([], 0)
    with pytest.raises(ValueError):
        m.verify([1], 3)          # start != cursor
    with pytest.raises(ValueError):
        m.verify([cfg["vocab"]], 0)
    with pytest.raises(ValueError):
        m.verify(list(range(9)), 0)  # past capacity
    with pytest.raises(ValueError):
        m.verify([1, 2], 0, parent=[-1, 1])  # parent[s] < s
