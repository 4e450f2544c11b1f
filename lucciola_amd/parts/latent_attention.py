"""Latent attention as a part: attention whose keys and values are rebuilt from a small latent
that is all the cache keeps of a token.

With h the mixer's input, H heads, per head ``dim`` unrotated and ``rot_dim`` rotated query/key
entries, values of ``vdim`` and a latent of ``kv_rank``:
  q = W_q h, head by head [dim | rot_dim];  W_dkv h = [c' | k_r] with c = rms(c') w_norm the
  latent and k_r (rot_dim entries, rotated by the token's position) a key part that all heads
  share;  per head k_h = W_uk,h c, v_h = W_uv,h c;
  score(i, j) = (q_h,plain(i) . k_h(j) + rot(q_h,rot(i)) . rot(k_r(j))) * scale,
  softmax over the keys j the window lets i see, o_h = sum_j p_j v_h(j);
  the heads side by side, times sigmoid(W_g h) where the part has a gate (an entry per output
  entry, or with ``gate_per_head`` one number per head), then W_o.
With ``q_rank`` the queries pass a latent of their own: q = W_uq (rms(W_dq h) w_qnorm).  With
``sink`` every head has a learned number s_h and its softmax's denominator one more term, exp(s_h):
a key without a value whose score is s_h for every query.
Only [c | rot(k_r)] is cached (``PagedLatent``).  The kernels never build k_h or v_h: because
q_h,plain . W_uk,h c = (W_uk,h^T q_h,plain) . c, the query is taken into the latent's space
(one small product per head), attention runs there with one shared "key" [c | k_r] and the
"value" c for all heads, and W_uv,h is applied to the attended latent afterwards.  A step of
single tokens and a prompt's portion go through the same kernels, so a token's result does not
depend on how the prompt was cut.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..cache.specs import PagedLatent
from ..config.registry import MIXERS, POSITION_ENCODINGS
from ..config.specs import PartSpec
from ..kernels import ops
from ..weights.loader import ParamDecl
from .base import BuildContext, Part, build_part
from .feed_forward import stack_rows


@MIXERS.register("latent_attention")
class LatentAttention(Part):
    graph_safe = True   # launches only kernels whose arguments stay put between steps

    def __init__(self, hidden_size: int, num_heads: int, dim: int, rot_dim: int, vdim: int,
                 kv_rank: int, scale: float, eps: float, position: Optional[PartSpec] = None,
                 window: Optional[int] = None, gate: bool = False, gate_per_head: bool = False,
                 q_rank: Optional[int] = None, sink: bool = False):
        super().__init__(hidden_size=hidden_size, num_heads=num_heads, dim=dim, rot_dim=rot_dim,
                         vdim=vdim, kv_rank=kv_rank, scale=scale, eps=eps, position=position,
                         window=window, gate=gate, gate_per_head=gate_per_head, q_rank=q_rank, sink=sink)
        self.gate_per_head = bool(gate_per_head) and bool(gate)
        self.q_rank = int(q_rank) if q_rank else None
        self.has_sink = bool(sink)
        self.W, self.H = int(hidden_size), int(num_heads)
        self.dim, self.rot, self.vdim, self.rank = int(dim), int(rot_dim), int(vdim), int(kv_rank)
        self.scale, self.eps = float(scale), float(eps)
        self.window = int(window) if window else None
        self.gate = bool(gate)
        self.position = build_part(POSITION_ENCODINGS, position) if position and self.rot else None
        if self.position is not None and self.position.rotary_dim > self.rot:
            raise ValueError(f"latent_attention: {self.position.rotary_dim} rotated entries in a "
                             f"part of {self.rot}")

    def declare(self) -> Dict[str, ParamDecl]:
        q_cols = self.H * (self.dim + self.rot)
        if self.q_rank:
            queries = {"dq": ParamDecl((self.q_rank, self.W)), "uq": ParamDecl((q_cols, self.q_rank)),
                       "dq_norm": ParamDecl((self.q_rank,), role="vector", init="ones_plus_normal")}
        else:
            queries = {"q": ParamDecl((q_cols, self.W))}
        out = {**queries,
               "dkv": ParamDecl((self.rank + self.rot, self.W)),
               "dkv_norm": ParamDecl((self.rank,), role="vector", init="ones_plus_normal"),
               "uk": ParamDecl((self.H * self.dim, self.rank)),
               "uv": ParamDecl((self.H * self.vdim, self.rank)),
               "o": ParamDecl((self.W, self.H * self.vdim))}
        if self.gate:
            out["g"] = ParamDecl((self.H if self.gate_per_head else self.H * self.vdim, self.W))
        if self.has_sink:
            out["sink"] = ParamDecl((self.H,), role="vector", init="normal")
        return out

    def bind(self, tensors, ctx: BuildContext) -> None:
        # one product for everything that reads the mixer's input: [q (or the queries' latent) | dkv | g]
        first = [tensors["dq" if self.q_rank else "q"], tensors["dkv"]] + ([tensors["g"]] if self.gate else [])
        self.qdg = stack_rows(first)
        self.first_cols = self.q_rank or self.H * (self.dim + self.rot)      # columns in front of dkv's
        if self.q_rank:
            self.uq, self.q_norm_weight = tensors["uq"], tensors["dq_norm"].to(torch.float32).contiguous()
        self.sink = tensors["sink"].to(torch.float32).contiguous() if self.has_sink else None
        self.norm_weight = tensors["dkv_norm"]
        # W_uk,h transposed: the matrix that takes a head's plain query into the latent's space
        self.uk_t = tensors["uk"].view(self.H, self.dim, self.rank).transpose(1, 2).contiguous()
        self.uv = tensors["uv"].view(self.H, self.vdim, self.rank).contiguous()
        self.o = tensors["o"]
        self.dtype = ctx.dtype
        if self.position is not None:
            self.position.bind({}, ctx)

    def cache_need(self):
        return PagedLatent(self.rank + self.rot, self.window)

    def batch_planner(self):
        return ops.LATENT_PLAN, ops.plan_latent_attention

    def tables_epoch(self) -> int:
        return self.position.tables_epoch() if self.position is not None else 0

    def ready(self, position: int) -> bool:
        return self.position.ready(position) if self.position is not None else True

    def forward(self, x: torch.Tensor, site) -> torch.Tensor:
        H, dim, rot, rank, vdim = self.H, self.dim, self.rot, self.rank, self.vdim
        batch, pages = site.batch, site.pages
        qdg = ops.gemm(x, self.qdg, self.dtype)
        T = qdg.shape[0]
        if self.q_rank:
            # the queries from their own latent: norm of the first columns, then a product
            q = ops.gemm(ops.rmsnorm_act(qdg, self.q_norm_weight, self.eps, column=0), self.uq, self.dtype)
        else:
            q = qdg
        table = self.position.rotary_table(batch.max_position) if self.position is not None else None
        pairing = self.position.pairing if self.position is not None else "half"
        # the query in the latent's space, head by head [W_uk^T q_plain | rot(q_rot)]
        # (without plain query entries nothing of the query reaches the latent: that part is zero)
        make = torch.empty if dim else torch.zeros
        qa = make((T, H * (rank + rot)), dtype=self.dtype, device=qdg.device)
        ops.latent_prepare(qdg, H, dim, rot, rank, self.norm_weight, self.eps, batch.positions, table,
                           pairing, site.cache, pages.slots if site.writes_cache else None, qa,
                           q=q, kv_column=self.first_cols)
        if dim:
            ops.grouped_gemm(ops.Strided(q, 0, dim + rot), self.uk_t, ops.Strided(qa, 0, rank + rot), T)
        latent = ops.latent_attention(qa, H, rank, rot, batch.tok_req, batch.positions, pages.block_table,
                                      site.cache, pages.page_size, self.scale, self.window or 0,
                                      plan=batch.plans.get(ops.LATENT_PLAN), max_ctx=batch.max_ctx, sink=self.sink)
        heads = torch.empty((T, H * vdim), dtype=self.dtype, device=qdg.device)
        gate = None
        if self.gate:
            gate = ops.Strided(qdg, self.first_cols + rank + rot, 1 if self.gate_per_head else vdim)
        ops.grouped_gemm(ops.Strided(latent, 0, rank), self.uv, ops.Strided(heads, 0, vdim), T, gate=gate,
                         gate_per_group=self.gate_per_head)
        return ops.gemm(heads, self.o, self.dtype, defer=True)
