"""Two mixers side by side: both read the same input, and the layer adds ``left_scale`` left + ``right_scale``
right to its stream as one branch.  The two are parts of any registered mixer kinds, each with its own
tensors (``left.*``, ``right.*``) and its own cache needs: the site's needs are the left one's, then the right
one's, and each finds its own as if it were alone."""
from __future__ import annotations

from typing import Dict

import torch

from ..config.registry import MIXERS
from ..config.specs import PartSpec
from ..kernels import ops
from ..weights.loader import ParamDecl
from .base import BuildContext, Part, build_part


def _needs(part) -> tuple:
    need = part.cache_need()
    if need is None:
        return ()
    return tuple(need) if isinstance(need, (tuple, list)) else (need,)


@MIXERS.register("parallel")
class ParallelMixers(Part):
    def __init__(self, left: PartSpec, right: PartSpec, left_scale: float = 1.0, right_scale: float = 1.0):
        super().__init__(left=left, right=right, left_scale=left_scale, right_scale=right_scale)
        self.left, self.right = build_part(MIXERS, left), build_part(MIXERS, right)
        self.left_scale, self.right_scale = float(left_scale), float(right_scale)
        self._left_needs, self._right_needs = len(_needs(self.left)), len(_needs(self.right))
        self.graph_safe = bool(getattr(self.left, "graph_safe", False) and getattr(self.right, "graph_safe", False))
        if self.left.batch_planner() is not None and self.right.batch_planner() is not None:
            raise ValueError("parallel: at most one of the two mixers may bring a batch planner")

    def declare(self) -> Dict[str, ParamDecl]:
        out = {"left." + name: decl for name, decl in self.left.declare().items()}
        out.update({"right." + name: decl for name, decl in self.right.declare().items()})
        return out

    def bind(self, tensors, ctx: BuildContext) -> None:
        self.left.bind({k[5:]: v for k, v in tensors.items() if k.startswith("left.")}, ctx)
        self.right.bind({k[6:]: v for k, v in tensors.items() if k.startswith("right.")}, ctx)

    def cache_need(self):
        needs = _needs(self.left) + _needs(self.right)
        return needs if needs else None

    def batch_planner(self):
        return self.left.batch_planner() or self.right.batch_planner()

    @property
    def portion_multiple(self) -> int:
        import math
        return math.lcm(int(getattr(self.left, "portion_multiple", 1)), int(getattr(self.right, "portion_multiple", 1)))

    def tables_epoch(self) -> int:
        return self.left.tables_epoch() + self.right.tables_epoch()

    def ready(self, position: int) -> bool:
        return self.left.ready(position) and self.right.ready(position)

    def forward(self, x: torch.Tensor, site) -> torch.Tensor:
        if isinstance(x, ops.ScaledRows):
            x = x.value()
        a = self.left.forward(x, site.span(0, self._left_needs))
        b = self.right.forward(x, site.span(self._left_needs, self._right_needs))
        return ops.scaled_sum(a, self.left_scale, b, self.right_scale)
