"""The state-space mixer (Mamba-2, state-space duality) as a part.

With h the mixer's input, ``num_heads`` heads of ``value_dim`` entries (inner = heads value_dim), a state of
``state_size`` entries a value channel and ``groups`` groups of heads that share B and C:
  W_in h = [z: inner | x: inner | B: groups state | C: groups state | dt: heads];
  x, B and C together pass a causal convolution per channel (``conv_taps`` taps, a bias) and SiLU;
  step = softplus(dt + dt_bias);  per head (of group g), from a state S [state, value] of zeros:
  S <- exp(-exp(A_log) step) S + step B_g x^T,   y = S^T C_g + D x;
  the heads side by side times silu(z), divided by their root mean square in ``norm_groups`` equal parts of the
  row, times a weight, then W_o.
The state is float32 and belongs to the request (a slot per live request, zeroed when it starts there), and so
do the convolution's last ``conv_taps`` - 1 inputs.  The projections leave as float32 and everything up to the
normed read-out stays float32.  The recurrence is the framework's scan (``ops.delta_scan``) without a removal
term, with decay = exp(-exp(A_log) step) in every key channel, write = step B, read = C: a step's tokens are
walked in order within each request from the slot's state, whatever the cut of the prompt.
"""
from __future__ import annotations

from typing import Dict

import torch

from ..cache.specs import FixedStates
from ..config.registry import MIXERS
from ..kernels import ops
from ..weights.loader import ParamDecl
from .base import BuildContext, Part


def _f32(t: torch.Tensor) -> torch.Tensor:
    return t.to(torch.float32).contiguous()


@MIXERS.register("state_space")
class StateSpace(Part):
    graph_safe = True   # launches only kernels whose arguments stay put between steps

    def __init__(self, hidden_size: int, num_heads: int, value_dim: int, state_size: int, groups: int,
                 conv_taps: int, norm_groups: int, norm_eps: float):
        super().__init__(hidden_size=hidden_size, num_heads=num_heads, value_dim=value_dim, state_size=state_size,
                         groups=groups, conv_taps=conv_taps, norm_groups=norm_groups, norm_eps=norm_eps)
        self.H, self.nh, self.dv, self.N = int(hidden_size), int(num_heads), int(value_dim), int(state_size)
        self.groups, self.taps, self.parts, self.norm_eps = int(groups), int(conv_taps), int(norm_groups), float(norm_eps)
        if self.nh % self.groups:
            raise ValueError(f"state_space: {self.nh} heads are not a multiple of {self.groups} groups")
        self.inner = self.nh * self.dv
        if self.parts < 1 or self.inner % self.parts:
            raise ValueError(f"state_space: {self.inner} channels do not fall into {self.parts} equal parts")
        if not 1 <= self.taps <= ops.SHORT_CONV_MAX_TAPS:
            raise ValueError(f"state_space: {self.taps} taps are outside the kernel's 1..{ops.SHORT_CONV_MAX_TAPS}")
        self.channels = self.inner + 2 * self.groups * self.N           # what passes the convolution: x | B | C
        ops.check_delta_sizes("state_space", self.N, self.dv, self.taps)

    def declare(self) -> Dict[str, ParamDecl]:
        return {"in": ParamDecl((self.inner + self.channels + self.nh, self.H)),
                "conv": ParamDecl((self.channels, self.taps), role="vector"),
                "conv_bias": ParamDecl((self.channels,), role="vector"),
                "dt_bias": ParamDecl((self.nh,), role="vector"), "A_log": ParamDecl((self.nh,), role="vector"),
                "D": ParamDecl((self.nh,), role="vector", init="ones_plus_normal"),
                "norm": ParamDecl((self.inner,), role="vector", init="ones_plus_normal"),
                "o": ParamDecl((self.H, self.inner))}

    def bind(self, tensors, ctx: BuildContext) -> None:
        self.dtype = ctx.dtype
        w = tensors["in"]
        # the checkpoint's rows are z | x | B | C | dt; what passes the convolution goes first here
        self.proj = torch.cat([w[self.inner:self.inner + self.channels], w[:self.inner],
                               w[self.inner + self.channels:]], dim=0).contiguous()
        self.conv, self.conv_bias = _f32(tensors["conv"]), _f32(tensors["conv_bias"])
        self.dt_bias, self.a_log, self.skip = _f32(tensors["dt_bias"]), _f32(tensors["A_log"]), _f32(tensors["D"])
        self.norm, self.o = _f32(tensors["norm"]), tensors["o"]

    def cache_need(self):
        shapes = ((self.nh, self.dv, self.N),)
        if self.taps > 1:
            shapes += ((self.taps - 1, self.channels),)
        return FixedStates(shapes)

    def forward(self, x: torch.Tensor, site) -> torch.Tensor:
        batch = site.batch
        state = site.cache[0]
        tail = site.cache[1] if self.taps > 1 else None
        proj = ops.gemm(x, self.proj, torch.float32)
        coef, xs = ops.state_space_prepare(proj, self.nh, self.groups, self.N, self.dv, self.conv, self.conv_bias, tail,
                                           self.dt_bias, self.a_log, batch.tok_req, batch.q_offsets, batch.slot_ids)
        if self.taps > 1:
            ops.conv_tail_update(proj, tail, self.channels, self.taps, batch.q_offsets, batch.slot_ids,
                                 batch.num_requests)
        o = ops.delta_scan(coef, xs, state, batch.q_offsets, batch.slot_ids, batch.num_requests, self.nh, self.N,
                           self.dv)
        y = ops.state_space_readout(o, xs, proj, self.channels, self.skip, self.nh, self.dv, self.norm, self.parts,
                                    self.norm_eps, self.dtype)
        return ops.gemm(y, self.o, self.dtype, defer=True)
