"""The Rununex design on the CPU: its configuration and what is refused, its tensors, what its layers need of the
cache, the plain implementation's mechanisms against hand-made cases, and the engine's host logic (step function,
cache, state slots, batches) with the plain torch versions of the kernels put in their place, against the plain
whole-sequence implementation."""
import copy
import math

import pytest
import torch

import plain_rununex
import reference_ops
import rununex_configs
import traces
from helpers import compare, make_runner, prompts_for, random_weights, replay
from lucciola_amd import models  # noqa: F401  (registers the architectures)
from lucciola_amd.cache.specs import FixedStates, PagedRows
from lucciola_amd.config.engine_config import EngineConfig
from lucciola_amd.config.model_config import ConfigError
from lucciola_amd.config.registry import architecture_for
from lucciola_amd.config.rununex_config import RununexConfig
from lucciola_amd.engine.batch import StepEntry
from lucciola_amd.engine.llm_engine import LLMEngine
from lucciola_amd.engine.loading import _build
from lucciola_amd.models.causal_lm import declared_tensors
from lucciola_amd.models.rununex import rununex_model_spec
from lucciola_amd.parts import BuildContext
from lucciola_amd.parts.position import Rotary
from lucciola_amd.sampling.sampler import SamplingParams
from lucciola_amd.weights.loader import DictSource

LENGTHS = {"A": [1, 12, 45], "B": [2, 40, 21], "C": [30, 9]}


def plain_weights(weights):
    return {k: v.to(torch.float64) for k, v in weights.items()}


def plain_logits(cfg, weights, prompts):
    w = plain_weights(weights)
    return {n: plain_rununex.forward(cfg, w, ids) for n, ids in prompts.items()}


def greedy(cfg, weights, prompt, count):
    w = plain_weights(weights)
    ids = list(prompt)
    for _ in range(count):
        ids.append(int(torch.argmax(plain_rununex.forward(cfg, w, ids)[-1])))
    return ids[len(prompt):]


def test_configuration_is_read_layer_by_layer():
    cfg = RununexConfig.from_dict(rununex_configs.R_B)
    assert (cfg.vocab, cfg.width, cfg.norm_eps) == (131, 50, 3e-6)
    assert (cfg.embedding_scale, cfg.residual_mult, cfg.logit_scale) == (1.0, 1.0, 1.0)
    assert [l.type for l in cfg.layers] == ["attention", "parallel", "attention", "parallel"]
    a, c = cfg.layers[0].mixer, cfg.layers[2].mixer
    assert (a.heads, a.kv_heads, a.dim, a.vdim, a.conv, a.chunk, a.diff) == (3, 3, 10, 7, 2, None, 0.4)
    assert a.rot.dims == 10 and a.rot.scaling is None and c.rot.base == 77.0
    assert (c.rot.scaling.factor, c.rot.scaling.low, c.rot.scaling.high, c.rot.scaling.original) == (8.0, 1.0, 4.0, 64.0)
    assert (c.conv, c.chunk) == (5, 11)
    p = cfg.layers[1].mixer
    assert (p.left.heads, p.left.kv_heads, p.left.dim, p.left.vdim, p.left.chunk) == (3, 1, 7, 9, 6)
    assert (p.right.heads, p.right.vdim, p.right.state, p.right.groups, p.right.conv, p.right.norm_groups) == (3, 5, 7, 3, 5, 3)
    assert (p.left_scale, p.right_scale) == (0.7, 0.9) and cfg.layers[3].mixer.left.chunk is None
    assert cfg.layers[0].mlp is None
    assert (cfg.layers[1].mlp.experts, cfg.layers[1].mlp.top, cfg.layers[1].mlp.shared_ff) == (3, 3, 22)
    assert cfg.layers[2].mlp.shared_ff == 0
    top = RununexConfig.from_dict(rununex_configs.R_A)
    assert (top.embedding_scale, top.residual_mult, top.logit_scale) == (3.0, 0.5, 0.5)
    assert architecture_for(rununex_configs.R_B).name == "Rununex"


@pytest.mark.parametrize("change,message", [
    (lambda c: c["layers"][0].update(type="convolution"), "not a mixer"),
    (lambda c: c["layers"][0]["mixer"].pop("diff"), "diff"),
    (lambda c: c["layers"][0]["mixer"].update(kv_heads=2), "multiple"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=5), "even"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=12), "at most"),
    (lambda c: c["layers"][2]["mixer"]["rot"]["scaling"].update(high=1.0), "high > low"),
    (lambda c: c["layers"][1]["mixer"]["right"].update(groups=2), "multiple of groups"),
    (lambda c: c["layers"][1]["mixer"]["right"].update(norm_groups=4), "must divide"),
    (lambda c: c["layers"][1]["mixer"].pop("left_scale"), "left_scale"),
    (lambda c: c["layers"][1]["mixer"]["left"].pop("scale"), "scale"),
    (lambda c: c["layers"][2]["mlp"]["router"].update(top=7), "exceeds"),
    (lambda c: c["layers"][1]["mlp"].update(kind="dense"), "not a feed-forward"),
    (lambda c: c.pop("width"), "width"),
    (lambda c: c["norm"].update(eps=0.0), "eps"),
])
def test_configuration_refuses(change, message):
    cfg = copy.deepcopy(rununex_configs.R_B)
    change(cfg)
    with pytest.raises(ConfigError, match=message):
        RununexConfig.from_dict(cfg)


def test_tensors_and_blocks():
    spec = rununex_model_spec(RununexConfig.from_dict(rununex_configs.R_B))
    assert [e.layer for e in spec.run_order] == [0, 1, 2, 3]
    assert [l.block for l in spec.layers] == ["prenorm_mixer", "prenorm_residual", "prenorm_residual", "prenorm_residual"]
    names = declared_tensors(spec)
    assert names["embed"].shape == (131, 50) and names["head"].shape == (131, 50) and names["final.norm"].shape == (50,)
    assert names["l0.mix.q"].shape == (3 * 2 * 10, 50) and names["l0.mix.k"].shape == (3 * 2 * 10, 50)
    assert names["l0.mix.v"].shape == (3 * 7, 50) and names["l0.mix.o"].shape == (50, 3 * 7)
    assert names["l0.mix.q.conv"].shape == (60, 2) and names["l0.mix.v.conv"].shape == (21, 2) and names["l0.mix.lk2"].shape == (10,)
    assert "l0.norm2" not in names and "l0.mlp.router" not in names and "l0.norm1.bias" not in names
    assert names["l1.mix.left.q"].shape == (21, 50) and names["l1.mix.left.k"].shape == (7, 50)
    assert names["l1.mix.left.v"].shape == (9, 50) and names["l1.mix.left.g"].shape == (27, 50)
    assert names["l1.mix.left.r1"].shape == (3,) and names["l1.mix.left.sink"].shape == (3,)
    assert names["l1.mix.right.in"].shape == (2 * 15 + 2 * 3 * 7 + 3, 50) and names["l1.mix.right.conv"].shape == (15 + 42, 5)
    assert names["l1.mix.right.conv.b"].shape == (57,) and names["l1.mix.right.A_log"].shape == (3,)
    assert names["l1.mix.right.norm"].shape == (15,) and names["l1.mix.right.o"].shape == (50, 15)
    assert names["l1.mlp.e2.gate"].shape == (30, 50) and names["l1.mlp.shared.down"].shape == (50, 22)
    assert "l2.mlp.shared.up" not in names and names["l2.mlp.router"].shape == (6, 50)


def test_what_the_layers_keep(monkeypatch):
    reference_ops.install(monkeypatch)
    cfg, page, seed = rununex_configs.ALL["B"]
    runner = make_runner(cfg, random_weights(cfg, seed, std=rununex_configs.STD), page, 8, "float32", "cpu", max_seqs=3)
    needs = runner.model.site_needs()
    assert needs[0] == (PagedRows(60, 21, None), FixedStates(((1, 141),)))
    assert needs[1] == (PagedRows(7, 9, None), FixedStates(((3, 5, 7), (4, 57))))
    assert needs[2] == (PagedRows(28, 11, None), FixedStates(((4, 67),)))
    assert needs[3] == (PagedRows(30, 25, None), FixedStates(((1, 9, 11),)))      # one tap: no inputs to keep
    assert len(runner.cache.groups) == 4


def test_frequencies_scaled_by_wavelength():
    """Every branch of the rule by hand: kept, divided, blended."""
    scaling = {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 64}
    f = plain_rununex.scaled_frequencies(12, 100.0, scaling)
    plain = [100.0 ** (-2.0 * i / 12) for i in range(6)]
    kinds = []
    for fi, pi in zip(f.tolist(), plain):
        wavelength = 2 * math.pi / pi
        if wavelength < 16:
            assert fi == pytest.approx(pi)
            kinds.append("kept")
        elif wavelength > 64:
            assert fi == pytest.approx(pi / 8)
            kinds.append("divided")
        else:
            s = (64 / wavelength - 1.0) / 3.0
            assert fi == pytest.approx((1 - s) * pi / 8 + s * pi)
            kinds.append("blended")
    assert set(kinds) == {"kept", "divided", "blended"}
    part = Rotary(rotary_dim=12, theta=100.0, pairing="interleaved", scaling=dict(scaling, kind="wavelength"))
    part.bind({}, BuildContext(dtype=torch.float32, device=torch.device("cpu")))
    table = part.rotary_table(40)
    angle = torch.arange(table.shape[0], dtype=torch.float64)[:, None] * f[None, :]
    assert torch.allclose(table[:, :6].double(), torch.cos(angle), atol=1e-6)
    assert torch.allclose(table[:, 6:].double(), torch.sin(angle), atol=1e-6)


def test_the_sink_and_the_distance_bias_by_hand():
    """One head, one value entry: with keys of zero every score is the bias alone, so the weights are
    (1 + r2 n)^(-r1) over the distances n and the sink's exp(s) joins the denominator only."""
    T = 5
    w = {"q": torch.zeros(2, 3), "k": torch.zeros(2, 3), "v": torch.tensor([[1.0, 0.0, 0.0]]), "g": torch.zeros(1, 3),
         "o": torch.ones(1, 1), "r1": torch.tensor([2.0]), "r2": torch.tensor([0.5]),
         "sink": torch.tensor([math.log(3.0)], dtype=torch.float64)}
    w = {"x." + k: v.double() for k, v in w.items()}
    m = {"heads": 1, "kv_heads": 1, "dim": 2, "vdim": 1, "scale": 1.0, "mask": {"size": 4}}
    h = torch.zeros(T, 3, dtype=torch.float64)
    h[:, 0] = torch.arange(1, T + 1)
    out = plain_rununex.biased_sink_attention(h, w, "x.", m, 1e-6)[:, 0] * 2       # the gate is sigmoid(0)
    for i in range(T):
        lo = i - i % 4
        weights = [(1 + 0.5 * (i - j)) ** -2.0 for j in range(lo, i + 1)]
        want = sum(wt * (j + 1) for wt, j in zip(weights, range(lo, i + 1))) / (sum(weights) + 3.0)
        assert float(out[i]) == pytest.approx(want, rel=1e-12)


def test_the_experts_get_their_weighted_input_by_hand():
    """One expert whose gate and up rows are ones: silu(w s) (w s) with s the sum of the input, not w silu(s) s."""
    h = torch.tensor([[0.5, 1.5]], dtype=torch.float64)
    w = {"x.router": torch.tensor([[1.0, 0.0]]), "x.e0.gate": torch.ones(1, 2), "x.e0.up": torch.ones(1, 2),
         "x.e0.down": torch.ones(2, 1)}
    w = {k: v.double() for k, v in w.items()}
    out = plain_rununex.routed_experts(h, w, "x.", {"router": {"experts": 1, "top": 1}})
    score = 1 / (1 + math.exp(-0.5))
    z = score * 2.0
    assert float(out[0, 0]) == pytest.approx(z / (1 + math.exp(-z)) * z, rel=1e-6)      # the router is float32


@pytest.mark.parametrize("key", ["A", "B", "C"])
@pytest.mark.parametrize("family", ["whole", "tail", "chunked", "mixed"])
def test_step_function_matches_plain(monkeypatch, key, family):
    reference_ops.install(monkeypatch)
    cfg, page, seed = rununex_configs.ALL[key]
    weights = random_weights(cfg, seed, std=rununex_configs.STD)
    prompts = prompts_for({"vocab_size": cfg["vocab"]}, LENGTHS[key], seed)
    steps = {"whole": traces.whole, "tail": traces.tail_decode, "chunked": traces.chunked,
             "mixed": traces.mixed}[family](prompts)
    blocks = traces.max_live_tokens(steps, page) // page
    runner = make_runner(cfg, weights, page, blocks, "float32", "cpu")
    got = replay(runner, steps)
    compare(got, cfg, weights, prompts, 2e-5, plain_logits(cfg, weights, prompts))
    assert not runner.cache.requests
    for g in runner.cache.groups:
        assert g.pool.num_free() == blocks


def test_stream_after_every_layer(monkeypatch):
    reference_ops.install(monkeypatch)
    cfg, page, seed = rununex_configs.ALL["A"]
    weights = random_weights(cfg, seed, std=rununex_configs.STD)
    ids = prompts_for({"vocab_size": cfg["vocab"]}, [19], seed)["r0"]
    _, want = plain_rununex.forward(cfg, plain_weights(weights), ids, keep_layers=True)
    runner = make_runner(cfg, weights, page, 8, "float32", "cpu")
    seen = []
    for layer in runner.model.layers:
        block, inner = layer.block, layer.block.forward

        def spy(stream, site, inner=inner):
            inner(stream, site)
            seen.append((stream.h.double() + cfg.get("residual_mult", 1.0) * stream.pending.double()).clone())
        block.forward = spy
    runner.step([StepEntry("r", ids[:7], [])])
    runner.step([StepEntry("r", ids[7:], [len(ids) - 8])])
    assert len(seen) == 2 * len(want)
    for k, ref in enumerate(want):
        got = torch.cat([seen[k], seen[len(want) + k]], dim=0)
        assert float((got - ref).abs().max()) < 1e-5 * float(ref.abs().max())


def test_a_slot_that_is_used_again_starts_from_zeros(monkeypatch):
    """With one slot, the second request finds the first one's state and last inputs there."""
    reference_ops.install(monkeypatch)
    cfg, page, seed = rununex_configs.ALL["B"]
    weights = random_weights(cfg, seed, std=rununex_configs.STD)
    prompts = prompts_for({"vocab_size": cfg["vocab"]}, [25, 14], seed)
    runner = make_runner(cfg, weights, page, 8, "float32", "cpu", max_seqs=1)
    got = replay(runner, traces.chunked(prompts, sizes=(9, 2, 30)))
    compare(got, cfg, weights, prompts, 2e-5, plain_logits(cfg, weights, prompts))


def test_greedy_generation_through_the_scheduler(monkeypatch):
    reference_ops.install(monkeypatch)
    cfg, page, seed = rununex_configs.ALL["A"]
    weights = random_weights(cfg, seed, std=0.2)
    arch = architecture_for(cfg)
    config = arch.read_config(cfg)
    model = _build(arch.model_spec(config), DictSource(weights), "float32", "cpu")
    engine = LLMEngine(model, config, EngineConfig(dtype="float32", block_size=page, max_blocks=40, max_seqs=3,
                                                   max_tokens_per_step=9, device="cpu", run_ahead=False))
    prompts = list(prompts_for({"vocab_size": cfg["vocab"]}, [4, 13, 27], seed + 1).values())
    got = engine.generate(prompts, SamplingParams(max_new_tokens=5))
    assert got == [greedy(cfg, weights, p, 5) for p in prompts]
    engine.runner.cache.check()
    assert not engine.runner.cache.requests


@pytest.mark.parametrize("seed", [0, 1, 2, 3, 4, 5, 6, 7])
def test_random_configurations_on_the_host(monkeypatch, seed):
    reference_ops.install(monkeypatch)
    cfg, page = rununex_configs.random_configuration(seed)
    weights = random_weights(cfg, 100 + seed, std=rununex_configs.STD)
    prompts = prompts_for({"vocab_size": cfg["vocab"]}, [3, 35, 18], seed)
    steps = traces.mixed(prompts, seed=seed)
    runner = make_runner(cfg, weights, page, traces.max_live_tokens(steps, page) // page, "float32", "cpu")
    compare(replay(runner, steps), cfg, weights, prompts, 2e-5, plain_logits(cfg, weights, prompts))
