"""Shared helpers of the GPU parity tests: model construction on both sides, tolerances."""
import numpy as np

import turbospark_amd as ts
from turbospark_amd import ffi, synth
from oracle import binding as ob


def f16(bits):
    return np.asarray(bits, np.uint16).view(np.float16).astype(np.float32)


def build_pair(name, max_context, seed=1234, threads=8, **over):
    cfg = dict(synth.CONFIGS[name])
    cfg.update(over)
    cfg["max_context"] = max_context
    weights = synth.make_weights(cfg, seed=seed)
    gpu = ts.HipVerifier(cfg, weights)
    cpu = ob.Model(cfg, weights, round_kv_f16=True, threads=threads)
    return cfg, weights, gpu, cpu


def logit_error(got_bits, want_bits):
    """max |got - want| relative to the reference row's logit range (the north-star metric)."""
    g, w = f16(got_bits), f16(want_bits)
    rng = (w.max(axis=-1) - w.min(axis=-1)).max()
    return float(np.abs(g - w).max() / rng)


TOL = {ffi.Q8_0: 2e-3, ffi.Q4_K: 1e-2, ffi.Q5_K: 1e-2}
