"""The Kikunex design on the CPU: its configuration and what is refused, the run order of a repeated
stack, what its layers need of the cache, and the engine's host logic (step function, cache, state
slots, batches) with the plain torch versions of the kernels put in their place, against the plain
whole-sequence implementation."""
import copy

import pytest
import torch

import kikunex_configs
import plain_kikunex
import reference_ops
import traces
from helpers import compare, make_runner, prompts_for, random_weights, replay
from lucciola_amd import models  # noqa: F401  (registers the architectures)
from lucciola_amd.cache.specs import FixedState, FixedStates, PagedLatent
from lucciola_amd.config.engine_config import EngineConfig
from lucciola_amd.config.kikunex_config import KikunexConfig
from lucciola_amd.config.model_config import ConfigError
from lucciola_amd.config.registry import architecture_for
from lucciola_amd.engine.batch import StepEntry
from lucciola_amd.engine.llm_engine import LLMEngine
from lucciola_amd.engine.loading import _build
from lucciola_amd.models.causal_lm import declared_tensors
from lucciola_amd.models.kikunex import kikunex_model_spec
from lucciola_amd.sampling.sampler import SamplingParams
from lucciola_amd.weights.loader import DictSource

LENGTHS = {"A": [1, 12, 45], "B": [2, 40, 21], "C": [30, 9]}


def test_configuration_is_read_layer_by_layer():
    cfg = KikunexConfig.from_dict(kikunex_configs.K_B)
    assert (cfg.vocab, cfg.width, cfg.norm_eps, cfg.logit_scale) == (131, 50, 3e-6, 1.0)
    assert [l.type for l in cfg.layers] == ["lightning", "latent_attention", "lightning", "latent_attention", "lightning"]
    assert [l.mixer.heads for l in cfg.layers] == [3, 3, 1, 1, 5]
    assert cfg.layers[0].mixer.decay == (1.0, 0.5, 0.02) and cfg.layers[0].mixer.vdim == 9
    assert [cfg.layers[i].mixer.window for i in (1, 3)] == [17, None]
    assert cfg.layers[1].mixer.rot.dims == 10 and cfg.layers[3].mixer.rot.base == 77.0
    assert (cfg.layers[1].mixer.q_rank, cfg.layers[1].mixer.kv_rank) == (13, 21)
    assert cfg.layers[1].mlp is None and cfg.layers[0].mlp.kind == "dense"
    assert (cfg.layers[2].mlp.experts, cfg.layers[2].mlp.top, cfg.layers[2].mlp.groups, cfg.layers[2].mlp.scale) == (5, 1, 1, 1.0)
    assert (cfg.layers[3].mlp.groups, cfg.layers[3].mlp.keep, cfg.layers[3].mlp.scale) == (2, 1, 2.5)
    assert (cfg.loop.start, cfg.loop.stop, cfg.loop.times) == (1, 4, 2)
    assert KikunexConfig.from_dict(kikunex_configs.K_A).logit_scale == 0.5
    assert architecture_for(kikunex_configs.K_B).name == "Kikunex"


@pytest.mark.parametrize("change,message", [
    (lambda c: c["layers"][0].update(type="convolution"), "not a mixer"),
    (lambda c: c["layers"][1]["mixer"].pop("kv_rank"), "kv_rank"),
    (lambda c: c["layers"][1]["mixer"].pop("q_rank"), "q_rank"),
    (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=5), "even"),
    (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=12), "at most"),
    (lambda c: c["layers"][0]["mixer"].update(decay=[0.5, 0.5]), "one number for each"),
    (lambda c: c["layers"][0]["mixer"].update(decay=[0.5, 0.5, 1.5]), "between 0 and 1"),
    (lambda c: c["layers"][2]["mlp"]["router"].update(top=6), "exceeds"),
    (lambda c: c["layers"][3]["mlp"]["router"].update(top=4), "exceeds"),          # one group of three is kept
    (lambda c: c["layers"][3]["mlp"]["router"]["groups"].update(count=4), "do not fit"),
    (lambda c: c["layers"][0]["mlp"].update(kind="gated"), "neither"),
    (lambda c: c["loop"].update(stop=6), "does not lie"),
    (lambda c: c.pop("width"), "width"),
    (lambda c: c["norm"].update(eps=0.0), "eps"),
])
def test_configuration_refuses(change, message):
    cfg = copy.deepcopy(kikunex_configs.K_B)
    change(cfg)
    with pytest.raises(ConfigError, match=message):
        KikunexConfig.from_dict(cfg)


def test_run_order_and_tensors_of_a_repeated_stack():
    spec = kikunex_model_spec(KikunexConfig.from_dict(kikunex_configs.K_B))
    assert [e.layer for e in spec.run_order] == [0, 1, 2, 3, 1, 2, 3, 4]
    marks = [(i, e.before.params["row"], e.before.params["add_origin"]) for i, e in enumerate(spec.run_order)
             if e.before is not None]
    assert marks == [(1, 0, False), (4, 1, True)]      # once a pass; the embedding's output again from the second on
    assert [l.block for l in spec.layers] == ["prenorm_shift_residual", "prenorm_shift_mixer"] + ["prenorm_shift_residual"] * 3
    names = declared_tensors(spec)
    assert names["loop.step"].shape == (2, 50) and names["embed"].shape == (131, 50) and names["head"].shape == (131, 50)
    assert names["embed.norm"].shape == () and names["final.norm"].shape == () and names["l3.norm2"].shape == ()
    assert names["l0.shift"].shape == (50,) and names["l0.mix.norm"].shape == (27,) and names["l0.mix.g"].shape == (27, 50)
    assert names["l0.mix.q"].shape == (21, 50) and names["l0.mix.v"].shape == (27, 50) and names["l0.mlp.act"].shape == (2,)
    assert names["l1.mix.dq"].shape == (13, 50) and names["l1.mix.uq"].shape == (3 * 17, 13)
    assert names["l1.mix.dkv"].shape == (21 + 10, 50) and names["l1.mix.dkv.norm"].shape == (21,)
    assert names["l1.mix.uk"].shape == (3 * 7, 21) and names["l1.mix.uv"].shape == (3 * 9, 21)
    assert names["l1.mix.sink"].shape == (3,) and names["l1.mix.g"].shape == (3, 50)
    assert "l1.norm2" not in names and "l1.mlp.up" not in names
    assert names["l3.mlp.e5.down"].shape == (50, 22) and names["l3.mlp.correction"].shape == (6,)
    no_loop = kikunex_model_spec(KikunexConfig.from_dict(kikunex_configs.K_C))
    assert [e.layer for e in no_loop.run_order] == [0, 1, 2, 3] and "loop.step" not in declared_tensors(no_loop)


def test_what_the_layers_keep(monkeypatch):
    """Every run of a layer is a site with a cache of its own: pages of latent rows or a matrix of state
    per head, and beside either the token shift's last row."""
    reference_ops.install(monkeypatch)
    cfg, page, seed = kikunex_configs.ALL["B"]
    runner = make_runner(cfg, random_weights(cfg, seed, std=kikunex_configs.STD), page, 8, "float32", "cpu", max_seqs=3)
    needs = runner.model.site_needs()
    assert len(needs) == 8
    assert needs[0] == (FixedStates(((3, 9, 7),)), FixedState((50,)))
    assert needs[1] == (PagedLatent(31, 17), FixedState((50,))) and needs[4] == needs[1]
    assert needs[3] == (PagedLatent(19, None), FixedState((50,)))
    assert len(runner.cache.groups) == 2                       # the windowed sites and the two without a window


@pytest.mark.parametrize("key", ["A", "B", "C"])
@pytest.mark.parametrize("family", ["whole", "tail", "chunked", "mixed"])
def test_step_function_matches_plain(monkeypatch, key, family):
    reference_ops.install(monkeypatch)
    cfg, page, seed = kikunex_configs.ALL[key]
    weights = random_weights(cfg, seed, std=kikunex_configs.STD)
    prompts = prompts_for({"vocab_size": cfg["vocab"]}, LENGTHS[key], seed)
    steps = {"whole": traces.whole, "tail": traces.tail_decode, "chunked": traces.chunked,
             "mixed": traces.mixed}[family](prompts)
    blocks = traces.max_live_tokens(steps, page) // page
    runner = make_runner(cfg, weights, page, blocks, "float32", "cpu")
    got = replay(runner, steps)
    refs = {n: plain_kikunex.forward(cfg, weights, ids) for n, ids in prompts.items()}
    compare(got, cfg, weights, prompts, 2e-5, refs)
    assert not runner.cache.requests
    for g in runner.cache.groups:
        assert g.pool.num_free() == blocks


@pytest.mark.parametrize("fused", [True, False])
def test_stream_after_every_layer_run(monkeypatch, fused):
    """The residual stream after each site of the run order, a repeated layer counted each time; with
    the norm and the shift in one kernel and as two."""
    reference_ops.install(monkeypatch)
    cfg, page, seed = kikunex_configs.ALL["B"]
    weights = random_weights(cfg, seed, std=kikunex_configs.STD)
    ids = prompts_for({"vocab_size": cfg["vocab"]}, [19], seed)["r0"]
    want = []
    plain_kikunex.forward(cfg, weights, ids, trace=want)
    runner = make_runner(cfg, weights, page, 8, "float32", "cpu")
    seen = []
    for layer in runner.model.layers:
        block, inner = layer.block, layer.block.forward
        layer.mixer_shift.fused = fused

        def spy(stream, site, inner=inner):
            inner(stream, site)
            seen.append((stream.h + stream.pending.to(torch.float32)).double().clone())
        block.forward = spy
    runner.step([StepEntry("r", ids[:7], []), ])
    runner.step([StepEntry("r", ids[7:], [len(ids) - 8])])
    assert len(seen) == 2 * len(want) == 16
    for k, ref in enumerate(want):
        got = torch.cat([seen[k], seen[8 + k]], dim=0)
        assert float((got - ref).abs().max()) < 1e-5 * float(ref.abs().max())


def test_a_slot_that_is_used_again_starts_from_zeros(monkeypatch):
    """With one slot, the second request finds the first one's state and last row there: both must be
    cleared when it starts."""
    reference_ops.install(monkeypatch)
    cfg, page, seed = kikunex_configs.ALL["B"]
    weights = random_weights(cfg, seed, std=kikunex_configs.STD)
    prompts = prompts_for({"vocab_size": cfg["vocab"]}, [25, 14], seed)
    runner = make_runner(cfg, weights, page, 8, "float32", "cpu", max_seqs=1)
    got = replay(runner, traces.chunked(prompts, sizes=(9, 2, 30)))
    refs = {n: plain_kikunex.forward(cfg, weights, ids) for n, ids in prompts.items()}
    compare(got, cfg, weights, prompts, 2e-5, refs)


def test_greedy_generation_through_the_scheduler(monkeypatch):
    reference_ops.install(monkeypatch)
    cfg, page, seed = kikunex_configs.ALL["A"]
    weights = random_weights(cfg, seed, std=0.2)
    arch = architecture_for(cfg)
    config = arch.read_config(cfg)
    model = _build(arch.model_spec(config), DictSource(weights), "float32", "cpu")
    engine = LLMEngine(model, config, EngineConfig(dtype="float32", block_size=page, max_blocks=40, max_seqs=3,
                                                   max_tokens_per_step=9, device="cpu", run_ahead=False))
    prompts = list(prompts_for({"vocab_size": cfg["vocab"]}, [4, 13, 27], seed + 1).values())
    got = engine.generate(prompts, SamplingParams(max_new_tokens=5))
    assert got == [plain_kikunex.greedy(cfg, weights, p, 5) for p in prompts]
    engine.runner.cache.check()
    assert not engine.runner.cache.requests


def test_the_choice_of_experts_by_hand():
    """Two groups of three; the corrections put the second group ahead although the first holds the
    largest plain score; a negative corrected score inside the kept group still beats every expert
    outside it; the weights are the plain scores times the scale."""
    logits = torch.tensor([[4.0, -9.0, -9.0, 0.5, 0.0, -3.0]])
    correction = torch.tensor([0.0, 0.0, 0.0, 0.6, 0.6, -2.0])
    router = {"experts": 6, "top": 3, "groups": {"count": 2, "keep": 1}, "scale": 2.0}
    chosen, weights = plain_kikunex.route(logits, correction, router)
    assert chosen.tolist() == [[3, 4, 5]]
    want = torch.sigmoid(torch.tensor([0.5, 0.0, -3.0], dtype=torch.float64)) * 2.0
    assert torch.allclose(weights[0], want)
    r = reference_ops.moe_route_sigmoid(logits, 3, correction, 2, 1, 2.0)
    assert r.ids.tolist() == [[3, 4, 5]] and torch.allclose(r.weights[0].double(), want, atol=1e-6)
    # without groups the largest corrected scores win wherever they lie
    chosen, _ = plain_kikunex.route(logits, correction, {"experts": 6, "top": 3})
    assert chosen.tolist() == [[3, 4, 0]]


@pytest.mark.parametrize("seed", [0, 1, 2, 3, 4, 5, 6, 7])
def test_random_configurations_on_the_host(monkeypatch, seed):
    reference_ops.install(monkeypatch)
    cfg, page = kikunex_configs.random_configuration(seed)
    weights = random_weights(cfg, 100 + seed, std=kikunex_configs.STD)
    prompts = prompts_for({"vocab_size": cfg["vocab"]}, [3, 35, 18], seed)
    steps = traces.mixed(prompts, seed=seed)
    runner = make_runner(cfg, weights, page, traces.max_live_tokens(steps, page) // page, "float32", "cpu")
    refs = {n: plain_kikunex.forward(cfg, weights, ids) for n, ids in prompts.items()}
    compare(replay(runner, steps), cfg, weights, prompts, 2e-5, refs)
