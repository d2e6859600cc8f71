"""A gated delta rule with short convolutions: a recurrent mixer whose per-request state has a fixed size.

Per head the state is a matrix S [dim, vdim] in fp32; per token it decays, is corrected along the token's key towards
the token's value (the delta rule) and is read with the token's query. Beside it the state holds the last conv - 1
inputs of the convolutions in front of q, k and v. Both live in the cache manager's state slots (one row per live
request), so nothing grows with the context and nothing is paged.

A step is
  1. one product with the stacked weight [W_q | W_k | W_v | W_g | W_a | W_b],
  2. the convolutions with silu over the first columns, reading and advancing their state (``ops.short_conv``),
  3. the recurrence over each request's rows in order, with unit norms, decay and write strength inside
     (``ops.gated_delta``; its value columns are spread over workgroups, so its read-out comes back raw),
  4. the heads' norm, gain and silu gate (``ops.heads_finish``, the kernel that ends attention heads too),
  5. the output product.
The same launches serve portions of prompts and single rows: the recurrence visits a request's rows one after the
other either way, so its result does not depend on how a prompt was cut.
"""
from __future__ import annotations

import torch

from ..cache.manager import StateSpec
from ..config.schema import GatedDeltaSpec
from ..kernels import ops
from ..weights.loader import WeightSpec
from .base import BuildContext, Part, pad_rows, register_part


class GatedDelta(Part):
    def __init__(self, spec: GatedDeltaSpec, prefix: str, build: BuildContext, positions):
        self.spec = spec
        self.prefix = prefix
        self.build = build
        try:
            ops.check_gated_delta_shape(spec.heads, spec.kv_heads, spec.dim, spec.vdim, spec.conv)
        except ops.KernelError as e:
            raise ValueError(f"{prefix}: {e}") from None
        self.qk_dim = spec.kv_heads * spec.dim
        self.v_dim = spec.heads * spec.vdim
        self.channels = 2 * self.qk_dim + self.v_dim  # what passes the convolutions: q | k | v
        self.gate_at = self.channels
        self.a_at = self.gate_at + self.v_dim
        self.b_at = self.a_at + spec.heads
        self.w_in = self.taps = self.a_log = self.dt_bias = self.gain = self.w_o = None

    def _name(self, which: str, suffix: str = "") -> str:
        return f"{self.prefix}.{getattr(self.spec.names, which)}{suffix}"

    def weight_specs(self):
        s, d, nm = self.spec, self.build.hidden, self.spec.names
        sizes = (("q", self.qk_dim), ("k", self.qk_dim), ("v", self.v_dim))
        out = [WeightSpec(self._name(n), (w, d)) for n, w in sizes]
        out += [WeightSpec(self._name(n, nm.conv_suffix), (w, s.conv)) for n, w in sizes]
        out += [WeightSpec(self._name("beta"), (s.heads, d)), WeightSpec(self._name("decay"), (s.heads, d)),
                WeightSpec(self._name("a_log"), (s.heads,), init="bias"), WeightSpec(self._name("dt_bias"), (s.heads,), init="bias"),
                WeightSpec(self._name("norm"), (s.vdim,), init="gain"), WeightSpec(self._name("gate"), (self.v_dim, d)),
                WeightSpec(self._name("o"), (d, self.v_dim))]
        return out

    def load(self, get):
        nm = self.spec.names
        stack = [get(self._name(n)) for n in ("q", "k", "v", "gate", "decay", "beta")]
        dt = stack[0].dtype if all(t.dtype == stack[0].dtype for t in stack) else torch.float32
        self.w_in = pad_rows(torch.cat([t.to(dt) for t in stack], dim=0).contiguous())
        del stack
        taps = [get(self._name(n, nm.conv_suffix)) for n in "qkv"]
        dt = taps[0].dtype if all(t.dtype == taps[0].dtype for t in taps) else torch.float32
        self.taps = torch.cat([t.to(dt) for t in taps], dim=0).contiguous()
        small = [get(self._name(n)) for n in ("a_log", "dt_bias")]
        if small[0].dtype != small[1].dtype:
            small = [t.float() for t in small]
        self.a_log, self.dt_bias = small
        self.gain = get(self._name("norm"))
        self.w_o = get(self._name("o"))

    def state_spec(self):
        s = self.spec
        return (StateSpec((s.heads, s.dim, s.vdim), torch.float32),
                StateSpec((max(s.conv - 1, 1), self.channels), torch.float32))

    def input_projection(self):
        return self.w_in, None

    def output_weight(self):
        return self.w_o

    @property
    def heads_width(self):
        return self.v_dim

    def heads_rows(self, xb, step, slot):
        """The input of the output product, [rows, heads x vdim] in the run's type."""
        y = ops.gemm(xb, self.w_in, out_dtype=self.build.dtype, exact=self.build.exact)
        return self.heads_rows_from(y, step, slot)

    def heads_rows_from(self, y, step, slot, out=None, out_mul=1.0):
        """The same from the input product's result ``y`` (a view with any row stride); ``out``: where to write."""
        s = self.spec
        matrix, tail = slot.state
        qkv = ops.short_conv(y, self.taps, tail, step.row_req, step.state_slots, step.n_requests)
        o = ops.gated_delta(qkv, y, self.a_at, self.b_at, self.a_log, self.dt_bias, matrix, step.row_req, step.state_slots,
                            step.n_requests, s.heads, s.kv_heads, s.dim, s.vdim)
        return ops.heads_finish(o, s.heads, 1, s.vdim, self.build.dtype, normed=True, eps=s.eps, gain=self.gain,
                                gate=y[:, self.gate_at:self.gate_at + self.v_dim], gate_fn="silu", out=out, out_mul=out_mul)

    def output(self, xb, step, slot):
        return ops.gemm(self.heads_rows(xb, step, slot), self.w_o, out_dtype=torch.float32, exact=self.build.exact)

    def forward(self, xb, residual, step, slot):
        ops.gemm(self.heads_rows(xb, step, slot), self.w_o, out=residual, epilogue=ops.EPI_ADD, exact=self.build.exact)


register_part("mixer", "gated_delta", GatedDelta, replace=True)
