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


def _tree_methods(cls, verify_tree, compact_tree):
    cls.verify_tree, cls.compact_tree = verify_tree, compact_tree


_tree_methods(OracleTarget, lambda self, feed, parent, base: self.m.verify(feed, base, parent=parent),
              lambda self, base, path: self.m.compact_tree(base, path))
_tree_methods(GpuTarget, lambda self, feed, parent, base: self.e.verify_tree(feed, parent, base),
              lambda self, base, path: self.e.compact_tree(base, path))


class TreeTwinDrafter:
    """A tree drafter for the loop tests (producer.rs:253-274): a twin of the target (same weights, its
    own cache) computes the target's true greedy continuation from the anchor and hides it in a fixed
    tree shape among seeded junk siblings, cutting it short at a seeded depth -- so rounds accept
    anything from nothing to the whole path, and the accepted node is rarely a parent's first child.
    `twin` offers reset / prefill(token, pos) / produce(token, pos) / rollback_retaining(point, keep)."""

    # node parents (-1: a child of the anchor), parents before children: two children of the anchor,
    # two under each of those that continues, a chain below
    SHAPES = {7: [-1, -1, 1, 1, 3, 3, 5], 15: [-1, -1, -1, 1, 1, 3, 3, 4, 6, 6, 9, 9, 11, 11, 13]}

    def __init__(self, twin, first_token, vocab, nodes, seed=0):
        self.t, self.vocab, self.tree_nodes, self.seed = twin, vocab, nodes, seed
        self.parent = self.SHAPES[nodes]
        self.known = [int(first_token)]   # token at every index the drafter has been told about
        self.at = 0                       # rows of `known` the twin's cache holds
        self.t.reset()

    def _know(self, index, token):
        del self.known[index:]
        assert len(self.known) == index, (len(self.known), index)
        self.known.append(int(token))
        if self.at > index:
            self.t.rollback_retaining(0, index)
            self.at = index

    def _sync(self, upto):
        while self.at < upto:
            self.t.prefill(self.known[self.at], self.at)
            self.at += 1

    def prime(self, token, position):     # `token` sits at index position + 1
        self._know(position + 1, token)

    def step(self, token, position):      # a chain round (one the budget shortened): the row after `token`
        self._know(position + 1, token)
        self._sync(position + 1)
        row = self.t.produce(int(token), position + 1)
        self.at = position + 2
        return row

    def rewind(self, position):           # the accepted prefix ended at index `position`
        keep = position + 1
        del self.known[keep:]
        if self.at > keep:
            self.t.rollback_retaining(0, keep)
            self.at = keep

    def draft_tree(self, anchor, base, nodes):
        self._know(base, anchor)
        self._sync(base)
        rng = np.random.default_rng([self.seed, base])
        cut = int(rng.integers(0, 6))     # how deep the true continuation is offered
        truth, tok = [], int(anchor)
        for d in range(5):
            row = np.asarray(self.t.produce(tok, base + d), np.uint16).view(np.float16).astype(np.float32)
            tok = int(np.argmax(row))
            truth.append(tok)
        self.at = base + 5
        self.known.extend(truth[:4])      # rows base + 1 .. base + 4 of the twin hold these
        tokens = [int(t) for t in rng.integers(0, self.vocab, nodes)]
        # the true path runs through the LAST child of each parent on it
        depth, node = 0, None
        for i in range(nodes):
            par = self.parent[i]
            last_child = max(j for j in range(nodes) if self.parent[j] == par)
            on_path = (par == -1 and node is None) or (node is not None and par == node)
            if on_path and i == last_child and depth < cut and depth < 5:
                tokens[i] = truth[depth]
                node, depth = i, depth + 1
        return list(self.parent), tokens
