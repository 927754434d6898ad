"""Producers for the generation-loop tests: a target and a step-wise drafter over either engine."""
import numpy as np


class OracleTarget:
    """The oracle model behind the producer methods the loop calls."""

    def __init__(self, model):
        self.m = model

    def reset(self):
        self.m.reset()

    def produce(self, token, pos):
        return self.m.verify([token], pos)[0]

    def prefill(self, token, pos):
        self.m.verify([token], pos)

    def verify(self, feed, base):
        return self.m.verify(feed, base)

    def rollback_retaining(self, point, keep_rows):
        self.m.rewind_to(point + keep_rows)


class GpuTarget:
    def __init__(self, eng):
        self.e = eng

    def reset(self):
        self.e.reset()

    def produce(self, token, pos):
        return self.e.produce(token, pos)

    def prefill(self, token, pos):
        self.e.prefill([token], pos, want_logits=False)

    def verify(self, feed, base):
        return self.e.verify(feed, base)

    def rollback_retaining(self, point, keep_rows):
        from turbospark_amd import ffi
        self.e.rollback_retaining(ffi.Point(point), keep_rows)


class LmDrafter:
    """A language model as the step-wise drafter: step(token, position) feeds `token` at index
    position + 1 and returns the logits after it; index 0 (the first prompt token, which the loop
    never hands to the drafter) is fed on the first call.  `noise` adds a seeded perturbation that
    depends on the fed token and index only, so two loops see the same drafter."""

    def __init__(self, target_like, first_token, vocab, noise=0.0, seed=0):
        self.t, self.first, self.vocab, self.noise, self.seed = target_like, int(first_token), vocab, noise, seed
        self.pos = 0
        self.t.reset()

    def _feed(self, token, position):
        idx = position + 1
        if self.pos == 0:
            self.t.prefill(self.first, 0)
            self.pos = 1
        assert idx == self.pos, (idx, self.pos)
        row = self.t.produce(int(token), idx)
        self.pos = idx + 1
        if self.noise:
            rng = np.random.default_rng([self.seed, int(token), idx])
            f = np.asarray(row, np.uint16).view(np.float16).astype(np.float32)
            row = (f + rng.standard_normal(self.vocab).astype(np.float32) * self.noise).astype(np.float16).view(np.uint16)
        return row

    def prime(self, token, position):
        self._feed(token, position)

    def step(self, token, position):
        return self._feed(token, position)

    def rewind(self, position):
        assert position + 1 <= self.pos
        self.t.rollback_retaining(0, position + 1)
        self.pos = position + 1
