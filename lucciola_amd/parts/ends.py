"""The parts at a model's two ends: the token embedding, which starts the float32 residual
stream, and the output head, which turns normed rows into float32 logits.

The reference gathers rows of ``model.embed_tokens.weight`` (src/qwen.cc:830-837,
src/kernels/embedding.cu:22-38) and multiplies the normed last rows by ``lm_head.weight``, or by
the embedding table again when the checkpoint has no head (src/qwen.cc:80-84,875-882).  They are
parts like any other, so that an architecture with a scaled embedding, a head with a bias or
capped logits registers its own kind and the model class stays as it is.

Interfaces:
  Embedding   declare() -> {"weight": ...}; forward(ids int32 [T]) -> float32 [T, H]
              (forward(ids, positions int32 [T]) where the part sets takes_positions);
              table() -> the tensor a tied head shares
  Head        declare() (nothing when tied); bind(tensors, ctx, shared=table or None);
              forward(x act [R, H]) -> float32 [R, V]
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..config.registry import EMBEDDINGS, HEADS
from ..kernels import ops
from ..weights.loader import ParamDecl
from .base import BuildContext, Part


@EMBEDDINGS.register("token_embedding")
class TokenEmbedding(Part):
    graph_safe = True

    def __init__(self, vocab_size: int, hidden_size: int, scale: float = 1.0):
        super().__init__(vocab_size=vocab_size, hidden_size=hidden_size, scale=scale)
        self.V, self.H, self.scale = int(vocab_size), int(hidden_size), float(scale)
        self.weight: Optional[torch.Tensor] = None

    def declare(self) -> Dict[str, ParamDecl]:
        return {"weight": ParamDecl((self.V, self.H))}

    def bind(self, tensors, ctx: BuildContext) -> None:
        self.weight = tensors["weight"]

    def table(self) -> torch.Tensor:
        return self.weight

    def forward(self, ids: torch.Tensor) -> torch.Tensor:
        return ops.embedding(ids, self.weight, self.scale)


@EMBEDDINGS.register("normed_token_embedding")
class NormedTokenEmbedding(TokenEmbedding):
    """The table's row divided by its root mean square (``eps`` inside the root) and times one learned
    number (tensor ``norm``, a scalar); float32 arithmetic."""

    def __init__(self, vocab_size: int, hidden_size: int, eps: float, scale: float = 1.0):
        super().__init__(vocab_size, hidden_size, scale)
        self.params["eps"] = eps
        self.eps = float(eps)
        self.gain: Optional[torch.Tensor] = None

    def declare(self) -> Dict[str, ParamDecl]:
        return {"weight": ParamDecl((self.V, self.H)),
                "norm": ParamDecl((), role="vector", init="ones_plus_normal")}

    def bind(self, tensors, ctx: BuildContext) -> None:
        super().bind(tensors, ctx)
        self.gain = tensors["norm"].to(torch.float32).reshape(1).expand(self.H).contiguous()

    def forward(self, ids: torch.Tensor) -> torch.Tensor:
        return ops.rmsnorm(ops.embedding(ids, self.weight, self.scale), None, self.gain, self.eps, torch.float32)


@EMBEDDINGS.register("sinusoid_token_embedding")
class SinusoidTokenEmbedding(TokenEmbedding):
    """The table's row plus a position vector: entry 2i is sin(p f_i), entry 2i + 1 cos(p f_i),
    f_i = base^(-2i/width).  The frequencies are made in float64 and kept as float32; the angle
    and its sine and cosine are float32 arithmetic in the kernel."""

    takes_positions = True

    def __init__(self, vocab_size: int, hidden_size: int, base: float = 10000.0, scale: float = 1.0):
        super().__init__(vocab_size, hidden_size, scale)
        self.params["base"] = base
        self.base = float(base)
        self.frequencies: Optional[torch.Tensor] = None

    def bind(self, tensors, ctx: BuildContext) -> None:
        super().bind(tensors, ctx)
        i = torch.arange((self.H + 1) // 2, dtype=torch.float64)
        f = torch.pow(torch.tensor(self.base, dtype=torch.float64), -2.0 * i / self.H)
        self.frequencies = f.to(torch.float32).to(ctx.device)

    def forward(self, ids: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
        return ops.embedding_sinusoid(ids, self.weight, positions, self.frequencies, self.scale)


@HEADS.register("linear_head")
class LinearHead(Part):
    graph_safe = True

    def __init__(self, vocab_size: int, hidden_size: int, tied: bool = False, scale: float = 1.0):
        super().__init__(vocab_size=vocab_size, hidden_size=hidden_size, tied=tied, scale=scale)
        self.V, self.H, self.tied = int(vocab_size), int(hidden_size), bool(tied)
        self.scale = float(scale)           # the logits are the product times this number
        self.weight: Optional[torch.Tensor] = None

    def declare(self) -> Dict[str, ParamDecl]:
        return {} if self.tied else {"weight": ParamDecl((self.V, self.H))}

    def bind(self, tensors, ctx: BuildContext, shared: Optional[torch.Tensor] = None) -> None:
        self.weight = shared if self.tied else tensors["weight"]
        if self.weight is None:
            raise ValueError("linear_head: a tied head needs the embedding's table")

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        logits = ops.gemm(x, self.weight, torch.float32)
        return logits if self.scale == 1.0 else ops.scale_(logits, self.scale)
