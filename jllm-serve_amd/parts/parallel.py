"""Mixers side by side: every branch reads the same input, the result is the sum of the branches' outputs with fixed
weights. Each branch is a mixer part of its own (any registered kind) with its tensors under a prefix of its own; the
pages and the state of the layer run are whatever the branches declare (one branch may own pages; the states of all
branches are handed to them in order)."""
from __future__ import annotations

from ..config.schema import ParallelMixerSpec
from .base import BuildContext, Part, part_factory, register_part
from .block import sublayer_output


class _BranchSlot:
    """A layer run's slot as one branch sees it: the run's pages, and of its state only the branch's own tensors."""

    def __init__(self, slot, state):
        self.group, self.rows, self.page_size, self.writes = slot.group, slot.rows, slot.page_size, slot.writes
        self.state = state


class ParallelMixer(Part):
    def __init__(self, spec: ParallelMixerSpec, prefix: str, build: BuildContext, positions):
        if not spec.branches or len(spec.branches) != len(spec.scales) or len(spec.branches) != len(spec.prefixes):
            raise ValueError(f"{prefix}: every branch has a scale and a prefix")
        self.spec = spec
        self.width = build.hidden
        self.branches = [part_factory("mixer", b.kind)(b, f"{prefix}.{p}" if p else prefix, build, positions)
                         for b, p in zip(spec.branches, spec.prefixes)]
        if sum(1 for b in self.branches if b.cache_spec() is not None) > 1:
            raise ValueError(f"{prefix}: more than one branch owns pages")
        self.capturable = all(getattr(b, "capturable", True) for b in self.branches)
        # which of the run's state tensors belong to which branch
        self._state_at = []
        at = 0
        for b in self.branches:
            st = b.state_spec()
            n = 0 if st is None else (len(st) if isinstance(st, (tuple, list)) else 1)
            self._state_at.append((at, n, isinstance(st, (tuple, list))))
            at += n

    def weight_specs(self):
        return [w for b in self.branches for w in b.weight_specs()]

    def load(self, get):
        for b in self.branches:
            b.load(get)

    def cache_spec(self):
        return next((c for c in (b.cache_spec() for b in self.branches) if c is not None), None)

    def state_spec(self):
        out = []
        for b in self.branches:
            st = b.state_spec()
            if st is not None:
                out += list(st) if isinstance(st, (tuple, list)) else [st]
        return tuple(out) if out else None

    def step_planners(self):
        return [pl for b in self.branches for pl in b.step_planners()]

    def _slot(self, slot, i):
        at, n, many = self._state_at[i]
        if n == 0:
            return _BranchSlot(slot, None)
        states = slot.state if isinstance(slot.state, (tuple, list)) else (slot.state,)
        return _BranchSlot(slot, tuple(states[at:at + n]) if many else states[at])

    def outputs(self, xb, step, slot):
        """Every branch's output as fp32 rows, in order (an arrangement may weigh and add them itself)."""
        return [sublayer_output(b, xb, step, self._slot(slot, i), self.width) for i, b in enumerate(self.branches)]

    def output(self, xb, step, slot):
        outs = self.outputs(xb, step, slot)
        total = outs[0].mul_(self.spec.scales[0])
        for o, s in zip(outs[1:], self.spec.scales[1:]):
            total.add_(o, alpha=s)
        return total

    def forward(self, xb, residual, step, slot):
        residual += self.output(xb, step, slot)


register_part("mixer", "parallel", ParallelMixer, replace=True)
