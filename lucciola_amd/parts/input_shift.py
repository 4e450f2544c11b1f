"""What is done to a mixer's normed input before the mixer reads it, as parts of their own family
(``input_shift``).  ``token_shift`` blends every token's row with the row of the token before it:

    y_t = x_t + (x_(t-1) - x_t) * mix          (mix: one learned number per coordinate)

with x as the norm left it, before any blending, and zeros before a sequence's first token.  The last
token's x is state of the request (one float32 row per live request and site, zeroed when the request
starts in its slot), so a prompt may be cut anywhere.  Where the norm in front is an RMS norm with a
single number as its weight, the residual addition, the norm and the shift are one kernel
(``ops.rms_shift``) and the state holds the float32 normed row; behind any other norm the shift is a
kernel of its own over the norm's output (``ops.token_shift``)."""
from __future__ import annotations

from typing import Dict

import torch

from ..cache.specs import FixedState
from ..config.registry import INPUT_SHIFTS
from ..kernels import ops
from ..weights.loader import ParamDecl
from .base import BuildContext, Part, ResidualStream


@INPUT_SHIFTS.register("token_shift")
class TokenShift(Part):
    graph_safe = True

    def __init__(self, size: int, fused: bool = True):
        super().__init__(size=size, fused=fused)
        self.size, self.fused = int(size), bool(fused)
        self.mix = None

    def declare(self) -> Dict[str, ParamDecl]:
        return {"mix": ParamDecl((self.size,), role="vector", init="normal")}

    def bind(self, tensors, ctx: BuildContext) -> None:
        self.mix = tensors["mix"].to(torch.float32).contiguous()
        self.dtype = ctx.dtype

    def cache_need(self):
        return FixedState((self.size,))

    def add_norm_shift(self, norm, stream: ResidualStream, site) -> torch.Tensor:
        """Add the pending branch output into the stream, norm it with ``norm`` and shift: what the mixer
        reads.  ``site.cache`` is this part's state [slots, size]."""
        batch, state = site.batch, site.cache
        if self.fused and getattr(norm, "scalar", False) and norm.gain is not None:
            stream.h, y = ops.rms_shift(stream.h, stream.pending, norm.gain, norm.eps, self.mix, state,
                                        batch.tok_req, batch.q_offsets, batch.slot_ids, self.dtype)
            stream.pending = None
            return y
        x = ops.value(norm.add_norm(stream))
        return ops.token_shift(x, self.mix, state, batch.tok_req, batch.q_offsets, batch.slot_ids)
