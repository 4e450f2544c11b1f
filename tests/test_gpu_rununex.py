"""The Rununex design on the GPU: every kernel it brought against the plain torch version of the same operation,
and the engine against the plain whole-sequence implementation (``plain_rununex``) in the four families of
traces, in float32 and in bfloat16."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_rununex
import reference_ops
import rununex_configs as rc
import traces
from helpers import make_runner, prompts_for, random_weights, replay
from lucciola_amd.config.engine_config import EngineConfig
from lucciola_amd.config.registry import architecture_for
from lucciola_amd.engine.llm_engine import LLMEngine
from lucciola_amd.engine.loading import _build
from lucciola_amd.kernels import ops
from lucciola_amd.sampling.sampler import SamplingParams
from lucciola_amd.weights.loader import DictSource

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
# A row's error: root mean square of the difference of the logits, means taken off, over that of the plain
# logits.  In bfloat16 a router's choice between two experts whose scores nearly tie can fall the other way, which
# changes that row by any amount: the bound is on the median row, on the share of rows over 10 % and on the share of
# rows that are unrelated.  What a fault of the cache, the state or the batch does wrong shows in many rows, and in
# float32.
TOL = {"float32": 4e-5, "bfloat16": 1e-1}
LENGTHS = {"A": [5, 1, 47, 90, 130], "B": [2, 61, 33, 100], "C": [150, 9, 230, 70]}
_cache = {}


def weights_for(cfg, seed, std=rc.STD):
    """Random weights; the routers' four times as large, so that few choices are close calls; sinks, biases, decays
    and skips of a size that shows when they are left out or mixed up."""
    weights = random_weights(dict(cfg, initializer_range=std), seed)
    g = torch.Generator().manual_seed(seed)

    def fill(name, values):
        weights[name] = values.to(weights[name].dtype)
    for name in list(weights):
        shape = weights[name].shape
        if name.endswith(".router"):
            fill(name, weights[name].float() * 4)
        elif name.endswith(".sink"):
            fill(name, torch.randn(shape, generator=g) * 1.5)
        elif name.endswith(".r1"):
            fill(name, torch.rand(shape, generator=g) * 1.5)
        elif name.endswith(".r2"):
            fill(name, torch.rand(shape, generator=g) * 2 + 0.05)
        elif name.endswith(".A_log"):
            fill(name, torch.randn(shape, generator=g) * 0.7 - 1.0)
        elif name.endswith(".dt_bias"):
            fill(name, torch.randn(shape, generator=g) * 0.5)
        elif name.endswith(".D"):
            fill(name, torch.randn(shape, generator=g))
        elif name.endswith(".conv") or name.endswith(".conv.b"):
            fill(name, torch.randn(shape, generator=g) * 0.5)
        elif name.split(".")[-1] in ("lq1", "lk1", "lq2", "lk2"):
            fill(name, torch.randn(shape, generator=g) * 0.3)
    return weights


def plain_logits(cfg, weights, prompts):
    w = {k: v.to(torch.float64) for k, v in weights.items()}
    return {n: plain_rununex.forward(cfg, w, ids) for n, ids in prompts.items()}


def case(key):
    if key not in _cache:
        cfg, page, seed = rc.ALL[key]
        weights = weights_for(cfg, seed)
        prompts = prompts_for({"vocab_size": cfg["vocab"]}, LENGTHS[key], seed)
        _cache[key] = (cfg, page, weights, prompts, plain_logits(cfg, weights, prompts))
    return _cache[key]


def row_error(row, ref):
    diff = row - ref
    return float((diff - diff.mean()).pow(2).mean().sqrt() / (ref - ref.mean()).pow(2).mean().sqrt())


def check_rows(got, prompts, refs, dtype, every=True):
    errors = []
    for name, ids in prompts.items():
        for pos in range(len(ids)):
            if (name, pos) not in got:
                assert not every, f"{name} position {pos}: no logits"
                continue
            row, ref = got[(name, pos)], refs[name][pos]
            assert torch.isfinite(row).all(), f"{name} position {pos}: logits are not finite"
            errors.append((row_error(row, ref), name, pos))
    tol = TOL[str(dtype).replace("torch.", "")]
    over = sorted(e for e in errors if e[0] > tol)
    worst = max(errors)
    if tol == TOL["bfloat16"]:
        median = sorted(errors)[len(errors) // 2]
        assert median[0] <= 0.04, f"the median row's error is {median[0]:.3e}"
        assert len(over) <= max(1, len(errors) // 10), f"{len(over)} of {len(errors)} rows over {tol:.1e}"
        unrelated = [e for e in errors if e[0] > 0.6]
        assert len(unrelated) <= max(1, len(errors) // 50), f"{len(unrelated)} of {len(errors)} rows are unrelated"
        return worst[0]
    assert worst[0] <= 3 * tol, f"request {worst[1]} position {worst[2]}: error {worst[0]:.3e} (bound {tol:.1e})"
    assert len(over) <= max(1, len(errors) // 50), (
        f"{len(over)} of {len(errors)} rows over {tol:.1e}; first: request {over[0][1]} position {over[0][2]} "
        f"({over[0][0]:.3e})")
    return worst[0]


def close(got, want, dtype, what, scale=1.0):
    tol = (4e-6 if dtype == torch.float32 else 1.2e-2) * scale
    err = float((got.double() - want.double()).abs().max() / want.double().abs().max().clamp_min(1e-9))
    assert err < tol, f"{what}: relative error {err:.3e}"


def request_lists(lengths, slots):
    q_offsets = torch.tensor([sum(lengths[:i]) for i in range(len(lengths) + 1)], dtype=torch.int32)
    tok_req = torch.tensor([r for r, n in enumerate(lengths) for _ in range(n)], dtype=torch.int32)
    return tok_req, q_offsets, torch.tensor(slots, dtype=torch.int32)


def tiles_of(step):
    """The step's tokens in tiles of up to 16 of one request, as the engine's planner makes them, on the GPU."""
    from lucciola_amd.engine.batch import HostLayout, Plan
    layout = HostLayout(len(step.new), sum(step.new), step.q_offsets.tolist(), list(step.cached), step.page,
                        all(n == 1 for n in step.new))
    arrays, info = ops.plan_latent_attention(layout)
    return Plan({k: torch.from_numpy(v).to(DEV) for k, v in arrays.items()}, info)


class PagedStep:
    """Requests with some tokens cached already and some new ones, pages handed out in a shuffled order."""

    def __init__(self, cached, new, page, seed=0):
        g = torch.Generator().manual_seed(seed)
        self.page, self.cached, self.new = page, cached, new
        need = [-(-(c + n) // page) for c, n in zip(cached, new)]
        order = torch.randperm(sum(need) + 3, generator=g).tolist()
        self.pages = sum(need) + 3
        width = max(need)
        table = torch.full((len(cached), width), -1, dtype=torch.int32)
        at = 0
        for r, n in enumerate(need):
            table[r, :n] = torch.tensor(order[at:at + n], dtype=torch.int32)
            at += n
        self.table = table
        self.tok_req, self.q_offsets, self.slot_ids = request_lists(new, list(range(len(new))))
        self.positions = torch.tensor([c + i for c, n in zip(cached, new) for i in range(n)], dtype=torch.int32)
        self.rows = torch.tensor([int(table[r, p // page]) * page + p % page
                                  for r, p in zip(self.tok_req.tolist(), self.positions.tolist())], dtype=torch.int32)

    def old_rows(self):
        return [int(self.table[r, p // self.page]) * self.page + p % self.page
                for r, c in enumerate(self.cached) for p in range(c)]


# ------------------------------------------------------------------ kernels alone
ATTENTION_CASES = [
    # heads, kv, maps, d, dv, page, chunk, window, taps, rot, unit, bias, sink, gate
    (4, 2, 2, 16, 24, 16, 37, 0, 3, 8, False, False, False, False),
    (3, 3, 2, 10, 7, 4, 0, 0, 2, 10, False, False, False, False),
    (8, 1, 1, 64, 64, 16, 120, 0, 0, 0, True, True, True, True),
    (6, 2, 1, 7, 9, 8, 5, 0, 0, 0, True, True, True, True),
    (2, 2, 1, 32, 16, 16, 0, 33, 4, 0, False, True, False, False),
    (2, 1, 2, 128, 256, 32, 300, 0, 1, 64, False, False, True, False),
    # sizes that the matrix-core kernel takes
    (8, 2, 2, 64, 128, 16, 100, 0, 4, 64, False, False, False, False),
    (4, 4, 2, 48, 96, 16, 0, 0, 2, 48, False, False, False, False),
    (16, 4, 1, 128, 128, 16, 64, 0, 0, 0, True, True, True, True),
    (20, 1, 1, 64, 64, 32, 0, 90, 0, 0, True, True, True, True),
    (2, 2, 1, 24, 16, 48, 33, 0, 0, 8, False, False, True, False),
    # groups of 3, 2 and 8 heads a kv head; sizes between the ones the kernel is built for
    (6, 2, 2, 40, 80, 16, 70, 0, 3, 16, False, False, False, False),
    (4, 2, 1, 72, 48, 16, 0, 0, 0, 0, True, True, True, True),
    (8, 1, 2, 32, 32, 32, 50, 0, 2, 32, False, False, False, False),
    (8, 1, 1, 104, 112, 16, 0, 40, 0, 0, True, True, False, True),
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("case_", ATTENTION_CASES)
def test_prepare_and_masked_attention(case_, dtype):
    """A step of unequal requests (a lone token after many, a portion that crosses chunk borders, a fresh prompt)
    over caches that earlier steps filled; q, the cache rows and the tails against the plain versions."""
    heads, kv, maps, d, dv, page, chunk, window, taps, rot, unit, bias, sink, gate = case_
    g = torch.Generator().manual_seed(heads * 100 + d)
    step = PagedStep([301, 70, 0, 12], [1, 45, 33, 2], page, seed=d)
    T = sum(step.new)
    nq, nk, nv = heads * maps, kv * maps, kv
    C = (nq + nk) * d + nv * dv
    cols = C + (heads * dv if gate else 0)
    proj = torch.randn(T, cols, generator=g)
    k_cache = torch.zeros(step.pages, page, nk * d, dtype=dtype)
    v_cache = torch.zeros(step.pages, nv * dv, page, dtype=dtype)
    old = torch.tensor(step.old_rows())
    k_cache.view(-1, nk * d)[old] = torch.randn(len(old), nk * d, generator=g).to(dtype)
    v_cache[old // page, :, old % page] = torch.randn(len(old), nv * dv, generator=g).to(dtype)
    conv = torch.randn(C, taps, generator=g) * 0.6 if taps else None
    tail = torch.randn(5, max(taps - 1, 0), C, generator=g) if taps > 1 else None
    table = None
    if rot:
        angle = torch.arange(400, dtype=torch.float64)[:, None] * (100.0 ** (-torch.arange(rot // 2, dtype=torch.float64) * 2 / rot))[None, :]
        table = torch.cat([torch.cos(angle), torch.sin(angle)], dim=1).float()
    r1 = torch.rand(heads, generator=g) * 1.5 if bias else None
    r2 = torch.rand(heads, generator=g) * 2 + 0.05 if bias else None
    sinks = torch.randn(heads, generator=g) * 2 if sink else None
    outs = []
    for o, where in ((reference_ops, "cpu"), (ops, DEV)):
        def on(t):
            return None if t is None else t.clone().to(where)
        kc, vc, tl = on(k_cache), on(v_cache), on(tail)
        lists = dict(tok_req=on(step.tok_req), q_offsets=on(step.q_offsets), slot_ids=on(step.slot_ids))
        pj = on(proj)
        prepare = dict(taps=on(conv), tail=tl, table=on(table), rot=rot, positions=on(step.positions),
                       unit_eps=1e-5 if unit else None, **lists)
        q = o.attention_prepare(pj, nq, nk, nv, d, dv, dtype, kc, vc, on(step.rows), **prepare)
        if o is ops and not unit:       # a wave a head and a thread a pair of entries: the same bits
            before = ops.attention_prepare_pairs(False)
            try:
                kc2, vc2 = on(k_cache), on(v_cache)
                q2 = o.attention_prepare(pj, nq, nk, nv, d, dv, dtype, kc2, vc2, on(step.rows), **prepare)
            finally:
                ops.attention_prepare_pairs(before)
            assert torch.equal(q, q2) and torch.equal(kc, kc2) and torch.equal(vc, vc2)
        if taps > 1:
            o.conv_tail_update(pj, tl, C, taps, lists["q_offsets"], lists["slot_ids"], len(step.new))
        out = o.masked_attention(q, kc, vc, lists["tok_req"], on(step.positions), on(step.table), page, heads, kv, maps,
                                 d, dv, 0.21, chunk=chunk, window=window, r1=on(r1), r2=on(r2), sink=on(sinks),
                                 subtract=0.45, unit_eps=1e-5 if maps == 2 else None, out_scale=0.7,
                                 gate=pj if gate else None, gate_column=C)
        fast = plain = None
        if o is ops and ops.masked_attention_on_matrix_cores(dtype, d, dv, page, maps):
            for staged in (True, False):     # tiles of several tokens with their keys staged in LDS, and straight from memory
                before = ops.masked_attention_staged(staged)
                try:
                    got = o.masked_attention(q, kc, vc, lists["tok_req"], on(step.positions), on(step.table), page, heads,
                                             kv, maps, d, dv, 0.21, chunk=chunk, window=window, r1=on(r1), r2=on(r2),
                                             sink=on(sinks), subtract=0.45, unit_eps=1e-5 if maps == 2 else None,
                                             out_scale=0.7, gate=pj if gate else None, gate_column=C, plan=tiles_of(step))
                finally:
                    ops.masked_attention_staged(before)
                fast, plain = (got, plain) if staged else (fast, got)
        outs.append([t.cpu() if t is not None else None for t in (q, kc, vc, tl, out, fast, plain)])
    if dtype == torch.bfloat16 and case_ in ATTENTION_CASES[6:]:
        assert outs[1][5] is not None, "the matrix-core kernel should take these sizes"
    for got, want, what in zip(outs[1], outs[0][:5] + [outs[0][4]] * 2,
                               ("q", "key rows", "value rows", "tails", "attention", "attention on the matrix cores (staged)",
                                "attention on the matrix cores")):
        if want is not None and got is not None:
            close(got, want, torch.float32 if what == "tails" else dtype, what, 3.0 if "attention" in what else 1.0)


@pytest.mark.parametrize("heads,kv,maps,d,dv,chunk", [(8, 2, 2, 64, 128, 0), (20, 1, 1, 128, 64, 700), (4, 4, 1, 32, 32, 0)])
def test_lone_tokens_with_their_keys_over_several_workgroups(heads, kv, maps, d, dv, chunk):
    """A step of lone tokens after histories of unequal length: every token's key blocks shared out over 1, 3 and 8
    workgroups and joined, against the plain version."""
    g = torch.Generator().manual_seed(heads)
    page = 16
    step = PagedStep([300, 70, 5, 1029, 0], [1, 1, 1, 1, 1], page, seed=3)
    T = 5
    nk, nv = kv * maps * d, kv * dv
    k_cache = torch.zeros(step.pages, page, nk, dtype=torch.bfloat16)
    v_cache = torch.zeros(step.pages, nv, page, dtype=torch.bfloat16)
    every = torch.tensor(step.old_rows() + step.rows.tolist())
    k_cache.view(-1, nk)[every] = torch.randn(len(every), nk, generator=g).to(torch.bfloat16)
    v_cache[every // page, :, every % page] = torch.randn(len(every), nv, generator=g).to(torch.bfloat16)
    q = torch.randn(T, heads * maps * d, generator=g).to(torch.bfloat16)
    sinks, r1, r2 = torch.randn(heads, generator=g), torch.rand(heads, generator=g), torch.rand(heads, generator=g) + 0.1
    gate = torch.randn(T, heads * dv + 3, generator=g)
    args = dict(chunk=chunk, r1=r1, r2=r2, sink=sinks, subtract=0.4, unit_eps=1e-5 if maps == 2 else None, out_scale=0.8,
                gate=gate, gate_column=3)
    want = reference_ops.masked_attention(q, k_cache, v_cache, step.tok_req, step.positions, step.table, page, heads, kv,
                                          maps, d, dv, 0.17, **args)
    plan = tiles_of(step)
    assert not plan.info["any_portion"]
    on_gpu = {k: (v.to(DEV) if isinstance(v, torch.Tensor) else v) for k, v in args.items()}
    for splits in (1, 3, 8):
        before = ops.masked_attention_force_splits(splits)
        try:
            got = ops.masked_attention(q.to(DEV), k_cache.to(DEV), v_cache.to(DEV), step.tok_req.to(DEV),
                                       step.positions.to(DEV), step.table.to(DEV), page, heads, kv, maps, d, dv, 0.17,
                                       plan=plan, max_ctx=1030 if splits > 1 else 0, **on_gpu)
        finally:
            ops.masked_attention_force_splits(before)
        close(got.cpu(), want, torch.bfloat16, f"{splits} workgroups a token", 3.0)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("chunk,window,page", [(40, 0, 16), (7, 0, 4), (0, 25, 8), (300, 0, 16)])
def test_one_key_carries_the_weight(dtype, chunk, window, page):
    """Among hundreds of keys one has a score that stands out; its value is one-hot.  A query sees it exactly when it
    lies inside the query's chunk or window: the key at the edge just inside, the one just outside, far keys, and the
    first tokens of a sequence; prompts and lone tokens alike."""
    heads, d, dv = 2, 16, 16
    length = 330
    k_rows = torch.zeros(length, heads * d)
    v_rows = torch.zeros(length, heads * dv)
    v_rows[:, :] = -1.0
    step = PagedStep([0], [length], page, seed=chunk + window)
    k_cache = torch.zeros(step.pages, page, heads * d, dtype=dtype, device=DEV)
    v_cache = torch.zeros(step.pages, heads * dv, page, dtype=dtype, device=DEV)
    places = step.rows.long().to(DEV)
    for marked in (0, 1, 15, 16, 17, 39, 40, 41, 279, 280, 287, 288, 299, 300, 305, 329):
        k = k_rows.clone()
        k[marked, :] = 1.0
        v = v_rows.clone()
        v[marked] = 5.0
        k_cache.view(-1, heads * d)[places] = k.to(dtype).to(DEV)
        v_cache[places // page, :, places % page] = v.to(dtype).to(DEV)
        q = torch.ones(length, heads * d, dtype=dtype, device=DEV)
        for lone, fast in ((False, False), (True, False), (False, True), (True, True)):
            rows = list(range(length)) if not lone else [marked, min(marked + 1, length - 1), length - 1]
            pos = torch.tensor(rows, dtype=torch.int32, device=DEV)
            plan = None
            if fast:        # the same on the matrix cores: the prompt in tiles of 16, or lone tokens of three requests
                if not ops.masked_attention_on_matrix_cores(dtype, d, dv, page, 1):
                    continue
                from lucciola_amd.engine.batch import Plan
                tiles = [[t0, min(16, length - t0), 0, t0] for t0 in range(0, length, 16)] if not lone else \
                    [[i, 1, 0, p] for i, p in enumerate(rows)]
                plan = Plan({"tiles": torch.tensor(tiles, dtype=torch.int32, device=DEV)}, {})
            out = ops.masked_attention(q[:len(rows)].contiguous(), k_cache, v_cache,
                                       torch.zeros(len(rows), dtype=torch.int32, device=DEV), pos, step.table.to(DEV), page,
                                       heads, heads, 1, d, dv, 4.0, chunk=chunk, window=window, plan=plan).float().cpu()
            for at, p in enumerate(rows):
                lo = 0
                if chunk:
                    lo = p - p % chunk
                if window:
                    lo = max(lo, p - window + 1)
                sees = lo <= marked <= p
                want = 5.0 if sees else -1.0
                assert abs(float(out[at, 0]) - want) < 1e-2, (f"key {marked}, query {p} ({'lone' if lone else 'prompt'}, "
                                                              f"{'matrix cores' if fast else 'general'}): "
                                                              f"{float(out[at, 0]):.3f}, expected {want}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("page", [4, 16])
def test_a_sink_that_takes_the_weight_and_one_that_takes_none(dtype, page):
    """Every value is 3, so without a sink every output is 3 whatever the scores are.  A sink far above the scores
    leaves the keys no weight (the output goes to 0), one far below changes nothing, and a sink as large as the one
    visible key's score halves the first token's output; the other head has the opposite sink."""
    heads, d, dv, length = 2, 16, 16, 70
    step = PagedStep([0], [length], page, seed=page)
    k_cache = torch.zeros(step.pages, page, heads * d, dtype=dtype, device=DEV)
    v_cache = torch.full((step.pages, heads * dv, page), 3.0, dtype=dtype, device=DEV)
    q = torch.zeros(length, heads * d, dtype=dtype, device=DEV)          # every score is 0
    common = (k_cache, v_cache, torch.zeros(length, dtype=torch.int32, device=DEV), step.positions.to(DEV),
              step.table.to(DEV), page, heads, heads, 1, d, dv, 1.0)
    plans = [None]
    if ops.masked_attention_on_matrix_cores(dtype, d, dv, page, 1):
        from lucciola_amd.engine.batch import Plan
        tiles = [[t0, min(16, length - t0), 0, t0] for t0 in range(0, length, 16)]
        plans.append(Plan({"tiles": torch.tensor(tiles, dtype=torch.int32, device=DEV)}, {}))
    for plan in plans:
        for sinks, want in (([40.0, -40.0], [0.0, 3.0]), ([-40.0, 40.0], [3.0, 0.0])):
            out = ops.masked_attention(q, *common, chunk=32, sink=torch.tensor(sinks, device=DEV), plan=plan).float().cpu()
            for h in range(heads):
                assert float((out[:, h * dv:(h + 1) * dv] - want[h]).abs().max()) < 1e-3, (sinks, h, plan is not None)
        out = ops.masked_attention(q, *common, chunk=32, sink=torch.zeros(heads, device=DEV), plan=plan).float().cpu()
        for p in range(length):         # p - p % 32 + 1 keys of score 0 beside a sink of 0
            keys = p % 32 + 1
            assert abs(float(out[p, 0]) - 3.0 * keys / (keys + 1)) < 2e-2, (p, float(out[p, 0]))


@pytest.mark.parametrize("heads,groups,N,dv,taps,parts", [(4, 2, 16, 8, 3, 2), (3, 3, 7, 5, 5, 3), (6, 2, 32, 32, 4, 2),
                                                          (1, 1, 11, 9, 1, 1), (8, 1, 64, 16, 2, 4)])
def test_state_space_kernels(heads, groups, N, dv, taps, parts):
    """Two steps in a row over the same slots: the second one's first tokens read the inputs that the first left in
    the tails, and the scan goes on from the first one's state."""
    g = torch.Generator().manual_seed(heads * 10 + N)
    inner = heads * dv
    C = inner + 2 * groups * N
    cols = C + inner + heads
    lengths, slots = [5, 1, 12, 2], [3, 0, 5, 1]
    tok_req, q_offsets, slot_ids = request_lists(lengths, slots)
    T = sum(lengths)
    conv, bias = torch.randn(C, taps, generator=g) * 0.5, torch.randn(C, generator=g) * 0.3
    dt_bias, a_log = torch.randn(heads, generator=g) * 0.5, torch.randn(heads, generator=g) * 0.7 - 1
    skip, weight = torch.randn(heads, generator=g), 1 + 0.2 * torch.randn(inner, generator=g)
    states = {where: (torch.zeros(6, heads, dv, N, device=where), torch.zeros(6, max(taps - 1, 0), C, device=where))
              for where in ("cpu", DEV)}
    for step in range(2):
        proj = torch.randn(T, cols, generator=g)
        outs = []
        for o, where in ((reference_ops, "cpu"), (ops, DEV)):
            state, tail = states[where]
            lists = [t.to(where) for t in (tok_req, q_offsets, slot_ids)]
            pj = proj.to(where)
            coef, x = o.state_space_prepare(pj, heads, groups, N, dv, conv.to(where), bias.to(where),
                                            tail if taps > 1 else None, dt_bias.to(where), a_log.to(where), *lists)
            o.conv_tail_update(pj, tail, C, taps, lists[1], lists[2], len(lengths))
            y = o.delta_scan(coef, x, state, lists[1], lists[2], len(lengths), heads, N, dv)
            out = o.state_space_readout(y, x, pj, C, skip.to(where), heads, dv, weight.to(where), parts, 1e-5, torch.float32)
            outs.append([t.cpu() for t in (coef, x, y, out, state, tail)])
        for got, want, what in zip(outs[1], outs[0], ("scan inputs", "x", "scan", "read-out", "state", "tails")):
            if want.numel():
                close(got, want, torch.float32, f"step {step}: {what}", 4.0)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_small_kernels(dtype):
    """The layer norm without a bias that adds a scaled branch; the sum of two scaled branches; gated experts fed
    their weighted input and their sum with a shared expert."""
    g = torch.Generator().manual_seed(3)
    T, n = 9, 70
    h, delta = torch.randn(T, n, generator=g) * 3, torch.randn(T, n, generator=g).to(dtype)
    w = 1 + 0.1 * torch.randn(n, generator=g)
    rows = torch.tensor([8, 0, 3], dtype=torch.int32)
    for sel in (None, rows):
        h_cpu, h_gpu = h.clone(), h.clone().to(DEV)
        want = reference_ops.layer_norm(h_cpu, delta, w, torch.zeros(n), 1e-5, dtype, rows=sel, branch_scale=0.7)
        got = ops.layer_norm(h_gpu, delta.to(DEV), w.to(DEV), torch.zeros(n, device=DEV), 1e-5, dtype,
                             rows=sel.to(DEV) if sel is not None else None, branch_scale=0.7)
        close(got.cpu(), want, dtype, "layer norm")
        close(h_gpu.cpu(), h_cpu, torch.float32, "stream")
    a, b = torch.randn(T, n, generator=g).to(dtype), torch.randn(T, n, generator=g)
    close(ops.scaled_sum(a.to(DEV), 0.8, b.to(DEV), 1.1).cpu(), reference_ops.scaled_sum(a, 0.8, b, 1.1), torch.float32,
          "scaled sum")
    E, top, I = 5, 2, 12
    logits = torch.randn(T, E, generator=g) * 2
    x = torch.randn(T, n, generator=g).to(dtype)
    gate_up = (torch.randn(E, 2 * I, n, generator=g) * 0.2).to(dtype)
    down = (torch.randn(E, n, I, generator=g) * 0.2).to(dtype)
    shared = torch.randn(T, n, generator=g).to(dtype)
    # by hand: sum over the chosen of down_e (silu(s gate_e x) * (s up_e x)), plus the shared rows
    s = torch.sigmoid(logits.double())
    want = shared.double().clone()
    for t in range(T):
        for e in torch.topk(s[t], top).indices.tolist():
            both = gate_up[e].double() @ (s[t, e] * x[t].double())
            want[t] += down[e].double() @ (torch.nn.functional.silu(both[:I]) * both[I:])
    routing = ops.moe_route_sigmoid(logits.to(DEV), top)
    both = ops.moe_experts(x.to(DEV), gate_up.to(DEV), routing, dtype, gather=True)
    hidden = ops.gated_activation_weighted(both, "silu", routing)
    y = ops.moe_experts(hidden, down.to(DEV), routing, torch.float32)
    got = ops.moe_combine_shared(y, routing, shared.to(DEV), None, 0, torch.float32, weighted=False)
    close(got.cpu(), want, dtype, "experts fed their weighted input", 3.0)
    alone = ops.moe_combine_shared(y, routing, None, None, 0, torch.float32, weighted=False)
    close(alone.cpu(), want - shared.double(), dtype, "without a shared expert", 3.0)


# ------------------------------------------------------------------ the engine
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("key", ["A", "B", "C"])
@pytest.mark.parametrize("family", ["whole", "tail", "chunked", "mixed"])
def test_replay_families(dtype, key, family):
    cfg, page, weights, prompts, refs = case(key)
    steps = {"whole": traces.whole, "tail": traces.tail_decode, "chunked": traces.chunked,
             "mixed": traces.mixed}[family](prompts)
    blocks = traces.max_live_tokens(steps, page) // page
    runner = make_runner(cfg, weights, page, blocks, dtype, DEV)
    check_rows(replay(runner, steps), prompts, refs, dtype)
    assert not runner.cache.requests
    for g in runner.cache.groups:
        assert g.pool.num_free() == blocks


MECHANISMS = {
    "differential attention alone": {"layers": [rc.layer(rc.attention(2, 1, 16, 12, 0.2, 0.3, 0, None), None)]},
    "with convolutions": {"layers": [rc.layer(rc.attention(2, 2, 8, 8, 0.3, 0.2, 4, None), None)]},
    "with rotation of some entries": {"layers": [rc.layer(rc.attention(2, 1, 16, 8, 0.3, 0.2, 0, None, rot_dims=6, base=50.0,
                                                                       scaling=(4.0, 1.0, 3.0, 16)), None)]},
    "in chunks": {"layers": [rc.layer(rc.attention(4, 4, 8, 8, 0.3, 0.5, 2, 13, rot_dims=8), None)]},
    "left mixer alone": {"layers": [rc.layer(rc.parallel((4, 2, 8, 8, 0.4, 10), (2, 4, 4, 1, 2, 1), 1.0, 0.0), None)]},
    "right mixer alone": {"layers": [rc.layer(rc.parallel((1, 1, 4, 4, 0.4, 10), (4, 8, 16, 2, 4, 2), 0.0, 1.0), None)]},
    "both mixers": {"layers": [rc.layer(rc.parallel((2, 1, 16, 16, 0.25, None), (2, 16, 8, 1, 3, 1), 0.8, 1.1), None)]},
    "experts alone": {"layers": [rc.layer(rc.attention(1, 1, 4, 4, 0.3, 0.2, 0, 3), rc.moe(24, 6, 2))]},
    "experts with a shared one": {"layers": [rc.layer(rc.attention(1, 1, 4, 4, 0.3, 0.2, 0, 3), rc.moe(24, 4, 1, shared=40))]},
    "factors at both ends": {"layers": [rc.layer(rc.attention(2, 1, 8, 8, 0.3, 0.2, 2, 9), rc.moe(16, 2, 1))],
                             "embedding": {"scale": 7.5}, "residual_mult": 0.3, "logit_scale": 0.2},
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(MECHANISMS))
def test_each_mechanism(name, dtype):
    cfg = dict({"architecture": "Rununex", "vocab": 90, "width": 48, "norm": {"eps": 1e-5}}, **MECHANISMS[name])
    weights = weights_for(cfg, 5, std=0.08)
    prompts = prompts_for({"vocab_size": 90}, [37, 4, 60], 2)
    refs = plain_logits(cfg, weights, prompts)
    steps = traces.chunked(prompts, sizes=(7, 2, 16, 1, 1, 3, 30))
    runner = make_runner(cfg, weights, 8, traces.max_live_tokens(steps, 8) // 8, dtype, DEV)
    check_rows(replay(runner, steps), prompts, refs, dtype)


def test_float32_logits_do_not_depend_on_the_cut():
    """The same bits whole, in portions and token by token: every sum's order follows from the token alone."""
    cfg, page, seed = rc.ALL["B"]
    weights = weights_for(cfg, seed)
    prompts = prompts_for({"vocab_size": cfg["vocab"]}, [75, 40], seed)
    runs = []
    for steps in (traces.whole(prompts), traces.chunked(prompts), traces.tail_decode(prompts, tail=30), traces.mixed(prompts)):
        runs.append(replay(make_runner(cfg, weights, page, 40, "float32", DEV), steps))
    for other in runs[1:]:
        for key, row in runs[0].items():
            assert torch.equal(row, other[key]), f"{key}: the bits differ between two cuts"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("key", ["A", "B", "C"])
def test_a_batch_of_unequal_requests_against_each_alone(key, dtype):
    cfg, page, weights, prompts, refs = case(key)
    names = list(prompts)[:4]
    alone = {}
    for n in names:
        runner = make_runner(cfg, weights, page, 64, dtype, DEV)
        alone.update(replay(runner, traces.whole({n: prompts[n]})))
    runner = make_runner(cfg, weights, page, 64, dtype, DEV)
    cut = {n: max(1, len(prompts[n]) - 3) for n in names}
    steps = [([(n, prompts[n][:cut[n]], list(range(cut[n]))) for n in names], [])]
    rest = {n: prompts[n][cut[n]:] for n in names}
    for k in range(max(len(r) for r in rest.values())):
        entries = [(n, [rest[n][k]], [0]) for n in names if k < len(rest[n])]
        steps.append((entries, [n for n in names if k == len(rest[n]) - 1]))
    steps[0] = (steps[0][0], [n for n in names if not rest[n]])
    together = replay(runner, [s for s in steps if s[0]])
    assert sorted(together) == sorted(alone)
    errors = []
    for row_key, row in alone.items():
        if dtype == "float32":
            assert torch.equal(row, together[row_key]), f"{row_key}: the bits differ between alone and in a batch"
        else:
            errors.append(row_error(together[row_key], row))
    if errors:      # a router's close call may fall the other way in a few rows
        errors.sort()
        assert errors[len(errors) // 2] < 0.03, f"median difference {errors[len(errors) // 2]:.3e}"
        assert sum(e > 0.1 for e in errors) <= len(errors) // 10


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", range(12))
def test_random_configurations(seed, dtype):
    """Configurations drawn at random, requests in mixed steps with so few pages and slots that they are used
    again, against the plain implementation."""
    cfg, page = rc.random_configuration(seed)
    weights = weights_for(cfg, 100 + seed)
    prompts = prompts_for({"vocab_size": cfg["vocab"]}, [3, 120, 41, 77, 1, 150], seed)
    refs = plain_logits(cfg, weights, prompts)
    steps = traces.mixed(prompts, seed=seed)
    blocks = traces.max_live_tokens(steps, page) // page
    runner = make_runner(cfg, weights, page, blocks, dtype, DEV)
    check_rows(replay(runner, steps), prompts, refs, dtype)
    assert not runner.cache.requests


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_over_chunk_borders_with_used_pages_and_slots(dtype):
    """Two slots and few pages: a request decodes token by token over several chunk borders while others come and go
    in the pages and slots that earlier ones gave back."""
    cfg, page, weights, _, _ = case("A")
    prompts = prompts_for({"vocab_size": cfg["vocab"]}, [100, 30, 26, 41], 9)
    refs = plain_logits(cfg, weights, prompts)
    names = list(prompts)
    steps = [([(names[1], prompts[names[1]], [29])], [names[1]])]
    long_ids = prompts[names[0]]
    steps.append(([(names[0], long_ids[:20], list(range(20)))], []))
    others = [names[2], names[3]]
    fed = {n: 0 for n in others}
    for i in range(20, 100):
        entries, end = [(names[0], [long_ids[i]], [0])], []
        live = next((n for n in others if fed[n] < len(prompts[n])), None)
        if live is not None and i % 2:
            n = min(5, len(prompts[live]) - fed[live])
            entries.append((live, prompts[live][fed[live]:fed[live] + n], list(range(n))))
            fed[live] += n
            if fed[live] == len(prompts[live]):
                end.append(live)
        if i == 99:
            end.append(names[0])
        steps.append((entries, end))
    blocks = traces.max_live_tokens(steps, page) // page
    runner = make_runner(cfg, weights, page, blocks, dtype, DEV, max_seqs=2)
    check_rows(replay(runner, steps), prompts, refs, dtype, every=False)
    assert not runner.cache.requests


@pytest.mark.parametrize("key", ["A", "B", "C"])
def test_greedy_generation_through_the_engine(key):
    cfg, page, seed = rc.ALL[key]
    weights = weights_for(cfg, seed, std=0.2)
    arch = architecture_for(cfg)
    config = arch.read_config(cfg)
    w64 = {k: v.to(torch.float64) for k, v in weights.items()}
    model = _build(arch.model_spec(config), DictSource(weights), "float32", DEV)
    engine = LLMEngine(model, config, EngineConfig(dtype="float32", block_size=page, max_blocks=60, max_seqs=3,
                                                   max_tokens_per_step=24, device=DEV))
    prompts = list(prompts_for({"vocab_size": cfg["vocab"]}, [4, 33, 57, 9], seed + 1).values())
    got = engine.generate(prompts, SamplingParams(max_new_tokens=8))
    for p, tokens in zip(prompts, got):
        ids = list(p)
        for t in tokens:        # every generated token is the plain form's argmax, or a near tie with it
            logits = plain_rununex.forward(cfg, w64, ids)[-1]
            best = int(torch.argmax(logits))
            assert t == best or float(logits[best] - logits[t]) < 1e-4 * float(logits.abs().max()), (ids, t, best)
            ids.append(t)
    engine.runner.cache.check()
    assert not engine.runner.cache.requests


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(tmp_path, dtype):
    """A model folder made from a configuration and a seed, replayed by ``bin/trace_run``: the architecture is found by
    config.json alone, and the pool is as small as the live requests allow."""
    from lucciola_amd.weights.random_init import write_model_folder
    from lucciola_amd.weights.safetensors_io import SafetensorsFile
    cfg, page, seed = rc.ALL["B"]
    folder = write_model_folder(str(tmp_path / "model"), dict(cfg, initializer_range=rc.STD), seed)
    with SafetensorsFile(os.path.join(folder, "model.safetensors")) as f:
        weights = {n: f.get(n).clone() for n in f.names()}
    prompts = prompts_for({"vocab_size": cfg["vocab"]}, [70, 33, 50, 3, 61], seed)
    steps = traces.mixed(prompts, seed=3)
    lines, index, fed = [], {}, {}
    for i, (entries, end) in enumerate(steps):
        lines.append(json.dumps({"step": i, "end": end, "entries": [{"id": n, "tokens": t, "want": w} for n, t, w in entries]}))
        rows = []
        for n, t, w in entries:
            rows += [(n, fed.get(n, 0) + k) for k in w]
            fed[n] = fed.get(n, 0) + len(t)
        index[i] = rows
    out = tmp_path / "out"
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    proc = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", folder, "--dtype", dtype,
                           "--out", str(out), "--max-tokens", str(traces.max_live_tokens(steps, 64))],
                          input="\n".join(lines) + "\n", text=True, capture_output=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert proc.stdout.split() == [x for i in range(len(steps)) for x in ("done", str(i))]
    got = {}
    for i, rows in index.items():
        data = np.fromfile(out / f"{i}.f32", dtype="<f4").reshape(len(rows), cfg["vocab"])
        for r, key in enumerate(rows):
            got[key] = torch.from_numpy(data[r].astype("float64"))
    check_rows(got, prompts, plain_logits(cfg, weights, prompts), dtype)
