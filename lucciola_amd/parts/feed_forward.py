"""The gated feed-forward (SwiGLU) as a part: ``down(silu(gate(x)) * up(x))``, no biases
(reference: src/qwen.cc:762-794, src/kernels/swiglu.cu:8,31-35).  gate and up are one matrix
product here: their weights are stacked at load.  The gate's activation is a parameter ("silu",
or "gelu_tanh", which takes a kernel of its own behind the product)."""
from __future__ import annotations

import math
from typing import Dict, Optional

import torch

from ..config.registry import FEED_FORWARDS
from ..kernels import ops
from ..weights.loader import ParamDecl
from .base import BuildContext, Part


def _softplus(z: float) -> float:
    return math.log1p(math.exp(-abs(z))) + max(z, 0.0)


def stack_rows(tensors):
    """Stack weight matrices along their rows; mixed storage widens to float32."""
    dtypes = {t.dtype for t in tensors}
    if len(dtypes) > 1:
        tensors = [t.to(torch.float32) for t in tensors]
    return torch.cat(tensors, dim=0).contiguous()


@FEED_FORWARDS.register("gated_mlp")
class GatedMLP(Part):
    graph_safe = True   # launches only kernels whose arguments stay put between steps
    takes_scaled_rows = True   # x may be ops.ScaledRows; the output may be an ops.PendingProduct

    def __init__(self, hidden_size: int, intermediate_size: int, activation: str = "silu"):
        super().__init__(hidden_size=hidden_size, intermediate_size=intermediate_size,
                         activation=activation)
        if activation not in ops.GATE_ACTIVATIONS:
            raise ValueError(f"gated_mlp: activation '{activation}' has no kernel ({', '.join(ops.GATE_ACTIVATIONS)})")
        self.H, self.I, self.activation = int(hidden_size), int(intermediate_size), activation

    def declare(self) -> Dict[str, ParamDecl]:
        return {"gate_proj": ParamDecl((self.I, self.H)),
                "up_proj": ParamDecl((self.I, self.H)),
                "down_proj": ParamDecl((self.H, self.I))}

    def bind(self, tensors, ctx: BuildContext) -> None:
        gate, up = tensors["gate_proj"], tensors["up_proj"]
        self.down = tensors["down_proj"]
        self.dtype = ctx.dtype
        # where the matrix-core kernel takes the sizes, gate and up rows are interleaved so that
        # silu(gate) * up is formed in the product's epilogue and [T, 2 I] never reaches memory
        self.fused = (self.activation == "silu" and ctx.device.type == "cuda" and self.I % 8 == 0 and gate.dtype == up.dtype
                      and ops.gemm_swiglu_supported(ctx.dtype, gate.new_empty((2 * self.I, 1)), self.H))
        if self.fused:
            self.gate_up = ops.interleave_gate_up(gate, up)
        else:
            self.gate_up = stack_rows([gate, up])

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if self.fused:
            z = ops.gemm_swiglu(x, self.gate_up)
        elif self.activation == "silu":
            z = ops.swiglu(ops.gemm(x, self.gate_up, self.dtype))
        else:
            z = ops.gated_activation(ops.gemm(x, self.gate_up, self.dtype), self.activation)
        return ops.gemm(z, self.down, self.dtype, defer=True)


@FEED_FORWARDS.register("mlp")
class MLP(Part):
    """The plain two-matrix feed-forward ``down(act(up(x)))``, no biases.  ``activation``:
    "gelu_tanh" (0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3)))), "relu_squared", or "xielu": with two
    learned numbers p, q (tensor ``act``), z > 0: softplus(p) z^2 + z/2; z <= 0: (1/2 + softplus(q))
    (e^z - 1 - z) + z/2."""

    graph_safe = True

    def __init__(self, hidden_size: int, intermediate_size: int, activation: str = "gelu_tanh"):
        super().__init__(hidden_size=hidden_size, intermediate_size=intermediate_size,
                         activation=activation)
        if activation not in ops.ACTIVATIONS:
            raise ValueError(f"mlp: activation '{activation}' has no kernel ({', '.join(ops.ACTIVATIONS)})")
        self.H, self.I, self.activation = int(hidden_size), int(intermediate_size), activation

    def declare(self) -> Dict[str, ParamDecl]:
        out = {"up": ParamDecl((self.I, self.H)), "down": ParamDecl((self.H, self.I))}
        if self.activation == "xielu":
            out["act"] = ParamDecl((2,), role="vector", init="normal")
        return out

    def bind(self, tensors, ctx: BuildContext) -> None:
        self.up, self.down = tensors["up"], tensors["down"]
        self.dtype = ctx.dtype
        self.act_params = (0.0, 0.0)
        if self.activation == "xielu":
            # the two numbers as the kernel takes them; read once, at load
            p, q = (float(v) for v in tensors["act"].to(torch.float64).cpu())
            self.act_params = (_softplus(p), 0.5 + _softplus(q))

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        z = ops.gemm_act(x, self.up, self.activation, self.dtype, self.act_params)
        return ops.gemm(z, self.down, self.dtype, defer=True)


@FEED_FORWARDS.register("routed_mlp")
class RoutedMLP(Part):
    """A mixture of small two-matrix feed-forwards.  The router's logits (float32) become
    scores over all experts (``scores``: "softmax"); each token keeps its ``top`` largest, whose
    scores, divided by their sum + ``renormalise_eps`` where ``renormalise``, weigh the experts'
    outputs.  With ``scores`` "sigmoid" the scores are sigmoids of the logits: the choice goes by
    score + a learned correction per expert (tensor ``correction``, where ``correction``), the
    weights by the plain scores times ``weight_scale``, never renormalised; with ``groups`` > 1 the
    experts form that many equal groups of neighbours, a group ranks by the sum of its two largest
    corrected scores, and only experts of the ``keep_groups`` best groups can be chosen.  On the device the (token, expert) pairs are sorted by expert, and the two products
    run once over the sorted rows, each tile of rows with its expert's matrix; nothing of it
    passes the host."""

    graph_safe = True

    def __init__(self, hidden_size: int, intermediate_size: int, experts: int, top: int,
                 activation: str = "relu_squared", scores: str = "softmax", renormalise: bool = True,
                 renormalise_eps: float = 1e-20, correction: bool = False, groups: int = 1, keep_groups: int = 1,
                 weight_scale: float = 1.0):
        super().__init__(hidden_size=hidden_size, intermediate_size=intermediate_size, experts=experts,
                         top=top, activation=activation, scores=scores, renormalise=renormalise,
                         renormalise_eps=renormalise_eps, correction=correction, groups=groups,
                         keep_groups=keep_groups, weight_scale=weight_scale)
        if activation not in ("gelu_tanh", "relu_squared"):
            raise ValueError(f"routed_mlp: activation '{activation}' has no kernel")
        if scores not in ("softmax", "sigmoid"):
            raise ValueError(f"routed_mlp: scores '{scores}' have no kernel (softmax, sigmoid)")
        if not 1 <= int(top) <= int(experts):
            raise ValueError(f"routed_mlp: top {top} of {experts} experts")
        self.scores, self.correction = scores, bool(correction)
        self.groups, self.keep_groups, self.weight_scale = int(groups), int(keep_groups), float(weight_scale)
        if scores == "softmax" and (correction or self.groups > 1 or self.weight_scale != 1.0):
            raise ValueError("routed_mlp: a correction, groups and a weight scale go with sigmoid scores")
        if scores == "sigmoid" and renormalise:
            raise ValueError("routed_mlp: sigmoid scores are not renormalised")
        if self.groups < 1 or int(experts) % self.groups or not 1 <= self.keep_groups <= self.groups \
                or int(top) > self.keep_groups * (int(experts) // self.groups):
            raise ValueError(f"routed_mlp: {self.groups} groups of which {self.keep_groups} are kept do not hold "
                             f"{top} choices among {experts} experts")
        self.H, self.I, self.E, self.top = int(hidden_size), int(intermediate_size), int(experts), int(top)
        self.activation, self.renormalise, self.renormalise_eps = activation, bool(renormalise), float(renormalise_eps)

    def declare(self) -> Dict[str, ParamDecl]:
        out = {"router": ParamDecl((self.E, self.H))}
        if self.correction:
            out["correction"] = ParamDecl((self.E,), role="vector", init="normal")
        for k in range(self.E):
            out[f"experts.{k}.up"] = ParamDecl((self.I, self.H))
            out[f"experts.{k}.down"] = ParamDecl((self.H, self.I))
        return out

    def bind(self, tensors, ctx: BuildContext) -> None:
        self.router = tensors["router"]
        self.correction_vector: Optional[torch.Tensor] = (
            tensors["correction"].to(torch.float32).contiguous() if self.correction else None)
        self.up = stack_rows([tensors[f"experts.{k}.up"] for k in range(self.E)]).view(self.E, self.I, self.H)
        self.down = stack_rows([tensors[f"experts.{k}.down"] for k in range(self.E)]).view(self.E, self.H, self.I)
        self.dtype = ctx.dtype
        self.large_tiles = ctx.device.type == "cuda" and ops.moe_large_tiles(ctx.dtype, self.up, self.down)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        logits = ops.gemm(x, self.router, torch.float32)
        if self.scores == "sigmoid":
            routing = ops.moe_route_sigmoid(logits, self.top, self.correction_vector, self.groups, self.keep_groups,
                                            self.weight_scale, large_tiles=self.large_tiles)
        else:
            routing = ops.moe_route(logits, self.top, self.renormalise, self.renormalise_eps,
                                    large_tiles=self.large_tiles)
        hidden = ops.moe_experts(x, self.up, routing, self.dtype, activation=self.activation, gather=True)
        y = ops.moe_experts(hidden, self.down, routing, torch.float32)
        return ops.moe_combine(y, routing, self.dtype)


@FEED_FORWARDS.register("routed_gated_mlp")
class RoutedGatedMLP(Part):
    """A mixture of small gated feed-forwards ``down(act(gate x) * (up x))``.  The router's logits
    (float32, plus a bias where ``router_bias``) pick the ``top`` largest; their weights are the
    softmax over the chosen logits alone.  ``shared_size`` > 0: a gated feed-forward of that inner
    size runs for every token and is added times sigmoid(w . x), one number per token (its
    weight row rides along in the router's product; ``shared_gate`` False: it is added as it is).
    ``scores`` "sigmoid": the scores are sigmoids of the logits, the ``top`` largest are chosen and weigh as
    they are, not renormalised.  ``weigh`` "input": a chosen expert's weight multiplies what it reads, not what
    it gives, expert(w x); both of its first products being linear, that is act(w gate x) * (w up x), formed
    where the gated activation is.  The experts' products run over the (token, choice) pairs sorted by expert,
    as for ``routed_mlp``; nothing passes the host."""

    graph_safe = True

    def __init__(self, hidden_size: int, intermediate_size: int, experts: int, top: int,
                 activation: str = "silu", router_bias: bool = False, shared_size: int = 0,
                 scores: str = "softmax_chosen", weigh: str = "output", shared_gate: bool = True):
        super().__init__(hidden_size=hidden_size, intermediate_size=intermediate_size, experts=experts, top=top,
                         activation=activation, router_bias=router_bias, shared_size=shared_size, scores=scores,
                         weigh=weigh, shared_gate=shared_gate)
        if activation not in ops.GATE_ACTIVATIONS:
            raise ValueError(f"routed_gated_mlp: activation '{activation}' has no kernel")
        if not 1 <= int(top) <= int(experts):
            raise ValueError(f"routed_gated_mlp: top {top} of {experts} experts")
        if scores not in ("softmax_chosen", "sigmoid"):
            raise ValueError(f"routed_gated_mlp: scores '{scores}' have no kernel (softmax_chosen, sigmoid)")
        if weigh not in ("output", "input"):
            raise ValueError(f"routed_gated_mlp: weigh '{weigh}' is neither 'output' nor 'input'")
        if scores == "sigmoid" and router_bias:
            raise ValueError("routed_gated_mlp: sigmoid scores go without a router bias")
        self.H, self.I, self.E, self.top = int(hidden_size), int(intermediate_size), int(experts), int(top)
        self.activation, self.router_bias, self.S = activation, bool(router_bias), int(shared_size)
        self.scores, self.weigh = scores, weigh
        self.shared_gate = bool(shared_gate) and self.S > 0
        if scores == "sigmoid" and self.shared_gate:
            raise ValueError("routed_gated_mlp: with sigmoid scores the shared expert has no gate of its own")
        self.shared = (GatedMLP(hidden_size=self.H, intermediate_size=self.S, activation=activation)
                       if self.S else None)

    def declare(self) -> Dict[str, ParamDecl]:
        out = {"router": ParamDecl((self.E, self.H))}
        if self.router_bias:
            out["router_bias"] = ParamDecl((self.E,), role="vector")
        for k in range(self.E):
            out[f"experts.{k}.gate"] = ParamDecl((self.I, self.H))
            out[f"experts.{k}.up"] = ParamDecl((self.I, self.H))
            out[f"experts.{k}.down"] = ParamDecl((self.H, self.I))
        if self.shared is not None:
            out.update({"shared.gate": ParamDecl((self.S, self.H)), "shared.up": ParamDecl((self.S, self.H)),
                        "shared.down": ParamDecl((self.H, self.S))})
            if self.shared_gate:
                out["shared_gate"] = ParamDecl((1, self.H))
        return out

    def bind(self, tensors, ctx: BuildContext) -> None:
        self.dtype = ctx.dtype
        # one product gives the router's logits and, in its last column, the shared expert's gate
        self.router = stack_rows([tensors["router"]] + ([tensors["shared_gate"]] if self.shared_gate else []))
        self.bias = tensors["router_bias"].to(torch.float32).contiguous() if self.router_bias else None
        self.gate_up = stack_rows([t for k in range(self.E) for t in (tensors[f"experts.{k}.gate"],
                                                                       tensors[f"experts.{k}.up"])]
                                  ).view(self.E, 2 * self.I, self.H)
        self.down = stack_rows([tensors[f"experts.{k}.down"] for k in range(self.E)]).view(self.E, self.H, self.I)
        self.large_tiles = ctx.device.type == "cuda" and ops.moe_large_tiles(ctx.dtype, self.gate_up, self.down)
        if self.shared is not None:
            self.shared.bind({"gate_proj": tensors["shared.gate"], "up_proj": tensors["shared.up"],
                              "down_proj": tensors["shared.down"]}, ctx)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        logits = ops.gemm(x, self.router, torch.float32)            # [T, E (+ 1)]
        if self.scores == "sigmoid":
            routing = ops.moe_route_sigmoid(logits, self.top, large_tiles=self.large_tiles)
        else:
            routing = ops.moe_route_logits(logits, self.E, self.top, self.bias, large_tiles=self.large_tiles)
        both = ops.moe_experts(x, self.gate_up, routing, self.dtype, gather=True)
        if self.weigh == "input":
            hidden = ops.gated_activation_weighted(both, self.activation, routing)
        else:
            hidden = ops.gated_activation(both, self.activation)
        y = ops.moe_experts(hidden, self.down, routing, torch.float32)
        weighted = self.weigh == "output"
        if self.shared is None:
            if weighted:
                return ops.moe_combine(y, routing, self.dtype)
            return ops.moe_combine_shared(y, routing, None, None, 0, self.dtype, weighted=False)
        extra = ops.value(self.shared.forward(x))
        return ops.moe_combine_shared(y, routing, extra, logits if self.shared_gate else None, self.E, self.dtype,
                                      weighted=weighted)
