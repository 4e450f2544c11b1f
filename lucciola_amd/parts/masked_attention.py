"""Attention whose heads may differ from the plain kind in several ways, each a parameter:

- keys and values of sizes of their own (``head_dim``, ``value_dim``), G key/value heads for H query heads;
- ``maps`` = 2, differential attention: a head has two queries and a kv head two keys ([map 1, map 2] side by
  side); each map is a softmax attention of its own over the same values, and the head's output is
  a_1 - lambda a_2 with lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + ``difference`` from four learned vectors, then
  divided by its root mean square over the value entries and multiplied by 1 - ``difference``;
- ``conv_taps`` > 0: q, k and v pass a short causal convolution per channel right behind their projection
  (no bias, no activation); the last ``conv_taps`` - 1 projected rows of a request are state;
- ``position``: a rotary encoding with interleaved pairs on the first entries of every map of every head;
- ``unit_qk``: every q and k head is divided by its root mean square (no weight);
- ``distance_bias``: r1_h ln(1 + r2_h (i - j)) is taken off the score of query i and key j (two learned numbers a
  head);
- ``sink``: a learned number s_h a head whose exp(s_h) is one more term of the softmax's denominator;
- ``gate``: the heads' outputs times sigmoid(W_g h), entry by entry, before the output projection;
- ``chunk``: position i sees j <= i only inside its own chunk of that many positions, counted from the sequence's
  start; ``window``: only the last so many positions.

The projections leave as float32; one kernel makes q, k and v of them (convolution, rotation, unit norm) and
writes k and v into the cache (keys token-major, values transposed inside a page).  Scores, softmax, bias, sink
and the maps' combination are float32 whatever the cache's type; with a bfloat16 cache of sizes that fit, the two
products run on the matrix cores (``ops.masked_attention``), else in float32 multiply-adds.
"""
from __future__ import annotations

import math
from typing import Dict, Optional

import torch

from ..cache.specs import FixedStates, PagedRows
from ..config.registry import MIXERS, POSITION_ENCODINGS
from ..config.specs import PartSpec
from ..kernels import ops
from ..weights.loader import ParamDecl
from .base import BuildContext, Part, build_part
from .feed_forward import stack_rows


def _f32(t: torch.Tensor) -> torch.Tensor:
    return t.to(torch.float32).contiguous()


@MIXERS.register("masked_attention")
class MaskedAttention(Part):
    graph_safe = True   # launches only kernels whose arguments stay put between steps

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int, value_dim: int,
                 scale: float, eps: float, maps: int = 1, difference: float = 0.0, conv_taps: int = 0,
                 position: Optional[PartSpec] = None, unit_qk: bool = False, distance_bias: bool = False,
                 sink: bool = False, gate: bool = False, chunk: Optional[int] = None, window: Optional[int] = None):
        super().__init__(hidden_size=hidden_size, num_heads=num_heads, num_kv_heads=num_kv_heads, head_dim=head_dim,
                         value_dim=value_dim, scale=scale, eps=eps, maps=maps, difference=difference,
                         conv_taps=conv_taps, position=position, unit_qk=unit_qk, distance_bias=distance_bias,
                         sink=sink, gate=gate, chunk=chunk, window=window)
        if num_heads % num_kv_heads:
            raise ValueError(f"masked_attention: {num_heads} heads are not a multiple of {num_kv_heads} kv heads")
        if maps not in (1, 2):
            raise ValueError(f"masked_attention: {maps} score maps a head (1 or 2)")
        self.H, self.nh, self.nkv = int(hidden_size), int(num_heads), int(num_kv_heads)
        self.d, self.dv, self.maps = int(head_dim), int(value_dim), int(maps)
        if max(self.d, self.dv) > ops.MASKED_ATTENTION_MAX:
            raise ValueError(f"masked_attention: heads of {self.d}/{self.dv} entries are above the kernel's "
                             f"{ops.MASKED_ATTENTION_MAX}")
        self.scale, self.eps, self.difference = float(scale), float(eps), float(difference)
        self.taps = int(conv_taps)
        if not 0 <= self.taps <= ops.SHORT_CONV_MAX_TAPS:
            raise ValueError(f"masked_attention: {self.taps} taps are above the kernel's {ops.SHORT_CONV_MAX_TAPS}")
        self.unit_qk, self.distance_bias, self.has_sink, self.has_gate = (bool(unit_qk), bool(distance_bias),
                                                                          bool(sink), bool(gate))
        self.chunk, self.window = int(chunk) if chunk else 0, int(window) if window else 0
        self.position = build_part(POSITION_ENCODINGS, position) if position else None
        if self.position is not None:
            if getattr(self.position, "pairing", None) != "interleaved":
                raise ValueError("masked_attention: its kernel rotates entry 2i with entry 2i + 1 (pairing 'interleaved')")
            if self.position.rotary_dim > self.d:
                raise ValueError(f"masked_attention: {self.position.rotary_dim} rotated entries in heads of {self.d}")
        self.nq_cols = self.nh * self.maps * self.d
        self.nk_cols = self.nkv * self.maps * self.d
        self.nv_cols = self.nkv * self.dv
        self.channels = self.nq_cols + self.nk_cols + self.nv_cols      # what passes the convolutions

    def declare(self) -> Dict[str, ParamDecl]:
        out = {"q": ParamDecl((self.nq_cols, self.H)), "k": ParamDecl((self.nk_cols, self.H)),
               "v": ParamDecl((self.nv_cols, self.H)), "o": ParamDecl((self.H, self.nh * self.dv))}
        if self.taps:
            out.update({"q_conv": ParamDecl((self.nq_cols, self.taps), role="vector"),
                        "k_conv": ParamDecl((self.nk_cols, self.taps), role="vector"),
                        "v_conv": ParamDecl((self.nv_cols, self.taps), role="vector")})
        if self.maps == 2:
            for name in ("lq1", "lk1", "lq2", "lk2"):
                out[name] = ParamDecl((self.d,), role="vector")
        if self.distance_bias:
            out["r1"] = ParamDecl((self.nh,), role="vector", init="ones_plus_normal")
            out["r2"] = ParamDecl((self.nh,), role="vector", init="ones_plus_normal")
        if self.has_sink:
            out["sink"] = ParamDecl((self.nh,), role="vector")
        if self.has_gate:
            out["g"] = ParamDecl((self.nh * self.dv, self.H))
        return out

    def bind(self, tensors, ctx: BuildContext) -> None:
        self.dtype = ctx.dtype
        mats = [tensors["q"], tensors["k"], tensors["v"]] + ([tensors["g"]] if self.has_gate else [])
        self.proj = stack_rows(mats)
        self.o = tensors["o"]
        self.conv = None
        if self.taps:
            self.conv = torch.cat([_f32(tensors[k]) for k in ("q_conv", "k_conv", "v_conv")], dim=0).contiguous()
        self.subtract = 0.0
        if self.maps == 2:
            # one number for the layer; read once, at load
            lq1, lk1, lq2, lk2 = (tensors[k].to(torch.float64).cpu() for k in ("lq1", "lk1", "lq2", "lk2"))
            self.subtract = math.exp(float((lq1 * lk1).sum())) - math.exp(float((lq2 * lk2).sum())) + self.difference
        self.r1 = _f32(tensors["r1"]) if self.distance_bias else None
        self.r2 = _f32(tensors["r2"]) if self.distance_bias else None
        self.sink = _f32(tensors["sink"]) if self.has_sink else None
        if self.position is not None:
            self.position.bind({}, ctx)

    def cache_need(self):
        rows = PagedRows(self.nk_cols, self.nv_cols, self.window or None)
        if self.taps > 1:
            return rows, FixedStates(((self.taps - 1, self.channels),))
        return rows

    def batch_planner(self):
        # the step's tokens in tiles of up to 16 of one request: the matrix-core kernel's work items
        return ops.LATENT_PLAN, ops.plan_latent_attention

    def tables_epoch(self) -> int:
        return self.position.tables_epoch() if self.position is not None else 0

    def ready(self, position: int) -> bool:
        return self.position.ready(position) if self.position is not None else True

    def forward(self, x: torch.Tensor, site) -> torch.Tensor:
        batch = site.batch
        paged = site.part(0)
        k_cache, v_cache = paged.cache
        pages = paged.pages
        tail = site.part(1).cache[0] if self.taps > 1 else None
        proj = ops.gemm(x, self.proj, torch.float32)
        table, rot = None, 0
        if self.position is not None:
            table, rot = self.position.rotary_table(batch.max_position), self.position.rotary_dim
        q = ops.attention_prepare(
            proj, self.nh * self.maps, self.nkv * self.maps, self.nkv, self.d, self.dv, self.dtype,
            k_cache, v_cache, pages.slots if site.writes_cache else None,
            taps=self.conv, tail=tail, tok_req=batch.tok_req, q_offsets=batch.q_offsets, slot_ids=batch.slot_ids,
            table=table, rot=rot, positions=batch.positions, unit_eps=self.eps if self.unit_qk else None)
        if self.taps > 1:
            ops.conv_tail_update(proj, tail, self.channels, self.taps, batch.q_offsets, batch.slot_ids,
                                 batch.num_requests)
        o = ops.masked_attention(
            q, k_cache, v_cache, batch.tok_req, batch.positions, pages.block_table, pages.page_size, self.nh, self.nkv,
            self.maps, self.d, self.dv, self.scale, chunk=self.chunk, window=self.window, r1=self.r1, r2=self.r2,
            sink=self.sink, subtract=self.subtract, unit_eps=self.eps if self.maps == 2 else None,
            out_scale=1.0 - self.difference if self.maps == 2 else 1.0,
            gate=proj if self.has_gate else None, gate_column=self.channels, plan=batch.plans.get(ops.LATENT_PLAN),
            max_ctx=batch.max_ctx)
        return ops.gemm(o, self.o, self.dtype, defer=True)
