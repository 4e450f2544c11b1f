"""The norms.  RMSNorm as a part: ``y = x * rsqrt(mean(x^2) + eps) * w`` over the last dimension
(reference: src/kernels/rmsnorm.cu:56-97; eps is the literal 1e-6 there, src/qwen.cc:588, and
a parameter here)."""
from __future__ import annotations

from typing import Dict, Optional, Tuple

import torch

from ..config.registry import NORMS
from ..kernels import ops
from ..weights.loader import ParamDecl
from .base import BuildContext, Part, ResidualStream


@NORMS.register("rms")
class RMSNorm(Part):
    graph_safe = True   # launches only kernels whose arguments stay put between steps
    offers_scaled_rows = True   # add_norm(stream, scaled=True) may return ops.ScaledRows

    def __init__(self, size: int, eps: float, scalar: bool = False):
        super().__init__(size=size, eps=eps, scalar=scalar)
        self.size, self.eps = int(size), float(eps)
        # scalar: the learned weight is one number for all coordinates (``gain``); the kernels still
        # get a vector, that number in every entry
        self.scalar = bool(scalar)
        self.gain: Optional[float] = None
        self.weight: Optional[torch.Tensor] = None
        self.dtype = None

    def declare(self) -> Dict[str, ParamDecl]:
        return {"weight": ParamDecl(() if self.scalar else (self.size,), role="vector", init="ones_plus_normal")}

    def bind(self, tensors, ctx: BuildContext) -> None:
        self.weight = tensors["weight"]
        if self.scalar:
            self.gain = float(self.weight.to(torch.float32).item())     # a kernel argument; read once, at load
            self.weight = self.weight.to(torch.float32).reshape(1).expand(self.size).contiguous()
        self.dtype = ctx.dtype

    def add_norm(self, stream: ResidualStream, scaled: bool = False):
        """Add the pending branch output into the stream and return the normed stream
        (``scaled``: the caller also takes ops.ScaledRows)."""
        x = ops.rmsnorm(stream.h, stream.pending, self.weight, self.eps, self.dtype, scaled=scaled)
        stream.pending = None
        return x

    def add_norm_rows(self, stream: ResidualStream, rows: torch.Tensor) -> torch.Tensor:
        """The normed stream (pending included) at the given rows only; the stream is not changed."""
        return ops.rmsnorm(stream.h, stream.pending, self.weight, self.eps, self.dtype, rows=rows)

    def apply(self, x: torch.Tensor) -> torch.Tensor:
        """Norm over the last dimension of an activation tensor."""
        return ops.rmsnorm_act(x, self.weight, self.eps)

    def fused_rms(self) -> Optional[Tuple[torch.Tensor, float]]:
        return self.weight, self.eps


@NORMS.register("dynamic_tanh")
class DynamicTanh(Part):
    """``y = tanh(alpha x) w + b``: a norm that takes no mean and no variance of its row.  The
    scalar ``alpha``, the weight and the bias are learned; everything is float32 arithmetic."""

    graph_safe = True

    def __init__(self, size: int):
        super().__init__(size=size)
        self.size = int(size)
        self.weight = self.bias = None
        self.alpha = 1.0
        self.dtype = None

    def declare(self) -> Dict[str, ParamDecl]:
        return {"weight": ParamDecl((self.size,), role="vector", init="ones_plus_normal"),
                "bias": ParamDecl((self.size,), role="vector", init="normal"),
                "alpha": ParamDecl((), role="vector", init="ones_plus_normal")}

    def bind(self, tensors, ctx: BuildContext) -> None:
        self.weight, self.bias = tensors["weight"], tensors["bias"]
        self.alpha = float(tensors["alpha"].item())     # a kernel argument; read once, at load
        self.dtype = ctx.dtype

    def add_norm(self, stream: ResidualStream, scaled: bool = False):
        x = ops.dynamic_tanh(stream.h, ops.value(stream.pending), self.weight, self.bias, self.alpha,
                             self.dtype)
        stream.pending = None
        return x

    def add_norm_rows(self, stream: ResidualStream, rows: torch.Tensor) -> torch.Tensor:
        return ops.dynamic_tanh(stream.h, ops.value(stream.pending), self.weight, self.bias, self.alpha,
                                self.dtype, rows=rows)

    def fused_rms(self):
        return None


@NORMS.register("layer_norm")
class LayerNorm(Part):
    """``y = (x - mean) / sqrt(var + eps) * w + b`` over the last dimension, the variance being
    the mean of the squared deviations; float32 arithmetic.  Where the branch output that waits
    to be added is itself to be normed first (``ops.NormedBranch``: a block with a norm behind
    each branch), one kernel norms the branch, adds it to the stream and norms the stream.  ``bias``
    False: the norm has a weight only.  ``branch_scale``: the branch output that waits is multiplied by
    this number as it is added to the stream (a model whose layers are x + m branch(norm(x)))."""

    graph_safe = True

    def __init__(self, size: int, eps: float, bias: bool = True, branch_scale: float = 1.0):
        super().__init__(size=size, eps=eps, bias=bias, branch_scale=branch_scale)
        self.size, self.eps = int(size), float(eps)
        self.has_bias, self.branch_scale = bool(bias), float(branch_scale)
        self.weight = self.bias = None
        self.dtype = None

    def declare(self) -> Dict[str, ParamDecl]:
        out = {"weight": ParamDecl((self.size,), role="vector", init="ones_plus_normal")}
        if self.has_bias:
            out["bias"] = ParamDecl((self.size,), role="vector", init="normal")
        return out

    def bind(self, tensors, ctx: BuildContext) -> None:
        self.weight = tensors["weight"]
        self.bias = tensors["bias"] if self.has_bias else torch.zeros_like(self.weight)
        self.dtype = ctx.dtype

    def add_norm(self, stream: ResidualStream, scaled: bool = False):
        x = ops.layer_norm(stream.h, stream.pending, self.weight, self.bias, self.eps, self.dtype,
                           branch_scale=self.branch_scale)
        stream.pending = None
        return x

    def add_norm_rows(self, stream: ResidualStream, rows: torch.Tensor) -> torch.Tensor:
        return ops.layer_norm(stream.h, stream.pending, self.weight, self.bias, self.eps, self.dtype, rows=rows,
                              branch_scale=self.branch_scale)

    def behind(self, branch) -> "ops.NormedBranch":
        """``branch`` (a branch's output) as something that is normed by this norm before it is
        added to the stream."""
        return ops.NormedBranch(ops.value(branch), self.weight, self.bias, self.eps)

    def apply(self, x: torch.Tensor) -> torch.Tensor:
        return ops.layer_norm_act(x, self.weight, self.bias, self.eps)

    def fused_rms(self):
        return None
