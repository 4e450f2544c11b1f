"""Lightning attention as a part: linear attention whose state forgets at one fixed rate per head.

With h the mixer's input, H heads, ``key_dim`` query/key and ``value_dim`` value entries a head:
  q = silu(W_q h), k = silu(W_k h), v = silu(W_v h), head by head;
  per head, from a state S [key, value] of zeros:  S <- decay_h S + k v^T,  o = S^T q   (no other scale);
  the heads side by side, divided by their common root mean square (``norm_eps`` inside the root), times
  a weight, times sigmoid(W_g h), then W_o.
The decays are constants of the model (``decays``, one per head), not tensors.  The state is float32 and
belongs to the request (a slot per live request, zeroed when it starts there); the projections leave as
float32 and everything up to the gated read-out stays float32.  The recurrence is the framework's
scan (``ops.delta_scan``) with decay = decay_h in every key channel, no removal, write = k, read = q: a
step's tokens are walked in order within each request from the slot's state, whatever the cut of the
prompt.
"""
from __future__ import annotations

from typing import Dict, Sequence

import torch

from ..cache.specs import FixedStates
from ..config.registry import MIXERS
from ..kernels import ops
from ..weights.loader import ParamDecl
from .base import BuildContext, Part
from .feed_forward import stack_rows


@MIXERS.register("lightning")
class Lightning(Part):
    graph_safe = True   # launches only kernels whose arguments stay put between steps

    def __init__(self, hidden_size: int, num_heads: int, key_dim: int, value_dim: int, decays: Sequence[float],
                 norm_eps: float):
        super().__init__(hidden_size=hidden_size, num_heads=num_heads, key_dim=key_dim, value_dim=value_dim,
                         decays=tuple(decays), norm_eps=norm_eps)
        self.H, self.nh, self.dk, self.dv = int(hidden_size), int(num_heads), int(key_dim), int(value_dim)
        self.decays, self.norm_eps = tuple(float(d) for d in decays), float(norm_eps)
        if len(self.decays) != self.nh:
            raise ValueError(f"lightning: {len(self.decays)} decays for {self.nh} heads")
        ops.check_delta_sizes("lightning", self.dk, self.dv)

    def declare(self) -> Dict[str, ParamDecl]:
        nk, nv = self.nh * self.dk, self.nh * self.dv
        return {"q": ParamDecl((nk, self.H)), "k": ParamDecl((nk, self.H)), "v": ParamDecl((nv, self.H)),
                "gate": ParamDecl((nv, self.H)), "norm": ParamDecl((nv,), role="vector", init="ones_plus_normal"),
                "o": ParamDecl((self.H, nv))}

    def bind(self, tensors, ctx: BuildContext) -> None:
        self.dtype = ctx.dtype
        self.proj = stack_rows([tensors[k] for k in ("q", "k", "v", "gate")])
        self.norm = tensors["norm"].to(torch.float32).contiguous()
        self.o = tensors["o"]
        self.decay = torch.tensor(self.decays, dtype=torch.float32, device=ctx.device)

    def cache_need(self):
        return FixedStates(((self.nh, self.dv, self.dk),))

    def forward(self, x: torch.Tensor, site) -> torch.Tensor:
        batch = site.batch
        (state,) = site.cache
        proj = ops.gemm(x, self.proj, torch.float32)
        coef, v = ops.lightning_prepare(proj, self.nh, self.dk, self.dv, self.decay)
        o = ops.delta_scan(coef, v, state, batch.q_offsets, batch.slot_ids, batch.num_requests,
                           self.nh, self.dk, self.dv)
        # one norm over all heads together, the weight and the gate in the same kernel
        y = ops.lightning_readout(o, proj, 2 * self.nh * self.dk + self.nh * self.dv, self.norm, self.norm_eps,
                                  self.dtype)
        return ops.gemm(y, self.o, self.dtype, defer=True)
