"""GPU parity of the verify-pass attention kernel against the oracle's causal attention.

Mirrors crates/gpu/tests/attention_tree_parity.rs (identity path == chain row; a branch node ==
the chain over its root path) and crates/compute/src/attention.rs' reference arithmetic."""
import numpy as np
import pytest

from oracle import binding as ob

pytestmark = pytest.mark.gpu


def _oracle(q, k, v, base, parent, scale=0.0, window=0, sinks=None):
    m, nq, hd = q.shape
    nkv = k.shape[1]
    out = np.empty((m, nq, hd), np.float32)
    import ctypes as C
    sk = np.ascontiguousarray(sinks, np.float32) if sinks is not None else None
    for i in range(m):
        if parent is None:
            out[i] = ob.causal_attention(q[i], k, v, hd, nq, nkv, base + i + 1, window, scale, sinks).reshape(nq, hd)
        else:
            path = []
            s = i
            while s >= 0:
                path.append(base + s)
                s = parent[s]
            path = np.array(path[::-1], np.int64)
            start = 0
            if window and base + len(path) > window:   # the last `window` members of prefix + root path
                start = base + len(path) - window
                assert start <= base
            o = np.empty(nq * hd, np.float32)
            qq = np.ascontiguousarray(q[i], np.float32)
            kk = np.ascontiguousarray(k, np.float32)
            vv = np.ascontiguousarray(v, np.float32)
            ob.lib().tso_attention_core(qq.ctypes.data_as(C.c_void_p), kk.ctypes.data_as(C.c_void_p),
                                        vv.ctypes.data_as(C.c_void_p), hd, nq, nkv, C.c_int64(start), C.c_int64(base),
                                        path.ctypes.data_as(C.c_void_p), len(path), C.c_float(scale),
                                        sk.ctypes.data_as(C.c_void_p) if sk is not None else None,
                                        o.ctypes.data_as(C.c_void_p))
            out[i] = o.reshape(nq, hd)
    return out


def _rand(m, nq, nkv, hd, base, seed):
    rng = np.random.default_rng(seed)
    r16 = lambda *s: rng.standard_normal(s).astype(np.float16).astype(np.float32)
    return r16(m, nq, hd), r16(base + m, nkv, hd), r16(base + m, nkv, hd)


@pytest.mark.parametrize("nq,nkv,hd", [(8, 8, 64), (4, 1, 128), (32, 8, 128), (16, 2, 64)])
@pytest.mark.parametrize("m,base", [(1, 0), (1, 37), (4, 0), (5, 0), (8, 0), (16, 0), (5, 200), (16, 1000), (9, 15)])
def test_chain_attention_matches_the_oracle(nq, nkv, hd, m, base):
    from turbospark_amd import ffi
    q, k, v = _rand(m, nq, nkv, hd, base, 100 + m + base)
    got = ffi.attention(q, k, v, base)
    want = _oracle(q, k, v, base, None)
    err = np.abs(got - want).reshape(m, -1).max(1)
    assert err.max() <= 5e-3 * max(1.0, np.abs(want).max()), err  # Tolerance::FP16_REDUCTION


def test_tree_attention_sees_prefix_plus_root_path():
    from turbospark_amd import ffi
    parent = [-1, 0, 0, 0, 0, 1, 5, 6, 2, 8, 9, 3, 11, 12, 4, 14]
    for (nq, nkv, hd, base) in [(4, 1, 128, 37), (32, 8, 128, 300), (8, 8, 64, 0)]:
        q, k, v = _rand(16, nq, nkv, hd, base, 5)
        got = ffi.attention(q, k, v, base, parent)
        want = _oracle(q, k, v, base, parent)
        assert np.abs(got - want).max() <= 5e-3 * max(1.0, np.abs(want).max())
        # identity path == chain, bit for bit
        a = ffi.attention(q[:6], k[:base + 6], v[:base + 6], base)
        b = ffi.attention(q[:6], k[:base + 6], v[:base + 6], base, [-1, 0, 1, 2, 3, 4])
        assert np.array_equal(a, b)
        # the identity map over a branching layout must FAIL at branch nodes
        c = ffi.attention(q, k, v, base)
        assert np.abs(c[8] - want[8]).max() > 1e-2


@pytest.mark.parametrize("nq,nkv,hd", [(8, 2, 64), (32, 8, 128)])
@pytest.mark.parametrize("m,base,window", [(1, 0, 17), (5, 10, 17), (9, 200, 128), (16, 300, 24), (16, 1000, 128),
                                           (4, 130, 128), (9, 119, 128), (1, 127, 128), (1, 128, 128)])
def test_sliding_window_and_sinks_match_the_oracle(nq, nkv, hd, m, base, window):
    """crates/compute/src/attention.rs:53-137: kv_start = seq_len - window; the sink joins the
    maximum and the denominator only (it takes probability mass away from the real positions)."""
    from turbospark_amd import ffi
    q, k, v = _rand(m, nq, nkv, hd, base, 400 + m + base)
    sinks = np.random.default_rng(base).standard_normal(nq).astype(np.float32) * 2
    for sk in (None, sinks):
        got = ffi.attention(q, k, v, base, scale=0.125, window=window, sinks=sk)
        want = _oracle(q, k, v, base, None, 0.125, window, sk)
        assert np.abs(got - want).max() <= 5e-3 * max(1.0, np.abs(want).max()), (sk is None)
    plain = ffi.attention(q, k, v, base, scale=0.125)
    sunk = ffi.attention(q, k, v, base, scale=0.125, sinks=sinks + 4)
    assert np.all(np.abs(sunk).sum(-1) < np.abs(plain).sum(-1) + 1e-3)   # mass went to the sink
    if base + 1 > window:
        assert np.abs(ffi.attention(q, k, v, base, scale=0.125, window=window) - plain).max() > 1e-3


def test_tree_attention_with_a_window():
    from turbospark_amd import ffi
    parent = [-1, 0, 0, 0, 0, 1, 5, 6, 2, 8, 9, 3, 11, 12, 4, 14]
    sinks = np.linspace(-1, 1, 8).astype(np.float32)
    for base, window in [(37, 24), (300, 128), (5, 20)]:
        q, k, v = _rand(16, 8, 2, 64, base, 9)
        got = ffi.attention(q, k, v, base, parent, scale=0.125, window=window, sinks=sinks)
        want = _oracle(q, k, v, base, parent, 0.125, window, sinks)
        assert np.abs(got - want).max() <= 5e-3 * max(1.0, np.abs(want).max())


@pytest.mark.parametrize("seed", range(64))
def test_random_attention_shapes_and_long_contexts(seed):
    """Seeded sweep: head width, GQA group 1..8, 1..16 rows, chain or random tree, contexts up to 20000
    positions (several 16-position blocks per wave: the pipelined walk), optional window (wider than
    the pass) and sinks, a scale of its own."""
    from turbospark_amd import ffi
    r = np.random.default_rng(4000 + seed)
    hd = int(r.choice([64, 128]))
    nkv = int(r.choice([1, 2, 4, 8]))
    g = int(r.choice([1, 2, 3, 4, 8]))
    nq = nkv * g
    m = int(r.integers(1, 17))
    base = int(r.choice([0, 1, 15, 16, 17, int(r.integers(18, 600)), int(r.integers(600, 5000)), int(r.integers(5000, 20000))]))
    tree = bool(r.integers(0, 2)) and m > 2
    parent = [-1] + [int(r.integers(0, s)) for s in range(1, m)] if tree else None
    window = int(r.integers(17, 300)) if r.integers(0, 3) == 0 else 0
    sinks = (r.standard_normal(nq) * 2).astype(np.float32) if r.integers(0, 3) == 0 else None
    scale = float(r.choice([0.0, 0.1, 0.2]))
    q, k, v = _rand(m, nq, nkv, hd, base, 9000 + seed)
    print(f"seed {seed}: hd={hd} q/kv={nq}/{nkv} m={m} base={base} {'tree' if tree else 'chain'} window={window} "
          f"sinks={'yes' if sinks is not None else 'no'} scale={scale}", flush=True)
    got = ffi.attention(q, k, v, base, parent=parent, scale=scale, window=window, sinks=sinks)
    want = _oracle(q, k, v, base, parent, scale=scale, window=window, sinks=sinks)
    err = np.abs(got - want).max()
    assert err <= 5e-3 * max(1.0, np.abs(want).max()), err
