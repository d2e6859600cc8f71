"""Mixers side by side: every branch reads the same input, the result is the sum of the branches' outputs with fixed
weights. Each branch is a mixer part of its own (any registered kind) with its tensors under a prefix of its own; the
pages and the state of the layer run are whatever the branches declare (one branch may own pages; the states of all
branches are handed to them in order).

Branches that say what their input and output products are (``input_projection``, ``heads_rows_from``,
``output_weight``, ``heads_width``) share them: one product with the branches' input weights stacked, each branch
working from its columns of the result and writing its heads, already multiplied by its weight in the sum, into its
columns of one buffer, and one output product with the branches' output weights side by side, whose result is the
weighted sum. A decode layer then has two product launches for the mixer instead of four."""
from __future__ import annotations

import torch

from ..config.schema import ParallelMixerSpec
from ..kernels import ops
from .base import BuildContext, Part, pad_rows, part_factory, register_part
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
        self.build = build
        self.fused = all(hasattr(b, n) for b in self.branches for n in ("input_projection", "heads_rows_from", "output_weight", "heads_width"))
        self.w_in = self.b_in = self.w_o = None
        self._cols = []
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
        if not self.fused:
            return
        ins = [b.input_projection() for b in self.branches]
        outs = [b.output_weight() for b in self.branches]
        ws = [w for w, _ in ins]
        if any(w.dtype != ws[0].dtype for w in ws) or any(o.dtype != outs[0].dtype for o in outs):
            self.fused = False  # mixed storage types: every branch keeps its own products
            return
        self.w_in = pad_rows(torch.cat(ws, dim=0).contiguous())
        if any(bias is not None for _, bias in ins):
            self.b_in = pad_rows(torch.cat([bias.to(torch.float32) if bias is not None else torch.zeros(w.shape[0], dtype=torch.float32, device=w.device)
                                            for w, bias in ins]).contiguous())
        self.w_o = torch.cat(outs, dim=1).contiguous()
        at = 0
        for w, _ in ins:
            self._cols.append((at, at + w.shape[0]))
            at += w.shape[0]
        for b in self.branches:  # the stacked copies are the ones that run
            for name in ("w_in", "b_in", "w_o"):
                if hasattr(b, name):
                    setattr(b, name, None)

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
        if self.fused:
            raise RuntimeError("the branches of this mixer share their products: ask for output()")
        return [sublayer_output(b, xb, step, self._slot(slot, i), self.width) for i, b in enumerate(self.branches)]

    def output(self, xb, step, slot):
        if self.fused:
            exact = self.build.exact
            y = ops.gemm(xb, self.w_in, bias=self.b_in, out_dtype=self.build.dtype, exact=exact)
            heads = ops.activation_rows(step.n_tokens, self.w_o.shape[1], self.build.dtype, y.device)
            at = 0
            for i, b in enumerate(self.branches):
                lo, hi = self._cols[i]
                b.heads_rows_from(y[:, lo:hi], step, self._slot(slot, i), out=heads[:, at:at + b.heads_width],
                                  out_mul=self.spec.scales[i])
                at += b.heads_width
            return ops.gemm(heads, self.w_o, out_dtype=torch.float32, exact=exact)
        outs = self.outputs(xb, step, slot)
        total = outs[0].mul_(self.spec.scales[0])
        for o, s in zip(outs[1:], self.spec.scales[1:]):
            total.add_(o, alpha=s)
        return total

    def forward(self, xb, residual, step, slot):
        residual += self.output(xb, step, slot)


register_part("mixer", "parallel", ParallelMixer, replace=True)
