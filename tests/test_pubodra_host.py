"""The Pubodra design on the CPU: its configuration and what is refused, the run order of a
repeated stack, the cache need of latent attention, and the engine's host logic (step function,
cache, batches) with the plain torch versions of the kernels put in their place, against the
plain whole-sequence implementation."""
import copy

import pytest
import torch

import plain_pubodra
import pubodra_configs
import reference_ops
import traces
from helpers import compare, make_runner, prompts_for, random_weights, replay
from lucciola_amd import models  # noqa: F401  (registers the architectures)
from lucciola_amd.cache.manager import CacheManager
from lucciola_amd.cache.specs import PagedLatent
from lucciola_amd.config.engine_config import EngineConfig
from lucciola_amd.config.model_config import ConfigError
from lucciola_amd.config.pubodra_config import PubodraConfig
from lucciola_amd.config.registry import architecture_for
from lucciola_amd.engine.llm_engine import LLMEngine
from lucciola_amd.engine.loading import _build
from lucciola_amd.models.causal_lm import declared_tensors
from lucciola_amd.models.pubodra import pubodra_model_spec
from lucciola_amd.sampling.sampler import SamplingParams
from lucciola_amd.weights.loader import DictSource


def test_configuration_is_read_layer_by_layer():
    cfg = PubodraConfig.from_dict(pubodra_configs.P_B)
    assert (cfg.vocab, cfg.width, cfg.norm_eps) == (131, 50, 3e-6)
    assert [l.mixer.heads for l in cfg.layers] == [3, 1, 5, 2]
    assert [l.mixer.window for l in cfg.layers] == [17, None, 33, 9]
    assert cfg.layers[0].mixer.rot.dims == 6 and cfg.layers[0].mixer.rot.scaling is None
    assert cfg.layers[3].mixer.rot.scaling.factor == 2.0
    assert cfg.layers[1].mlp is None and cfg.layers[0].mlp.kind == "dense"
    assert (cfg.layers[2].mlp.experts, cfg.layers[2].mlp.top, cfg.layers[2].mlp.ff) == (5, 1, 30)
    assert (cfg.loop.start, cfg.loop.stop, cfg.loop.times) == (1, 3, 2)
    assert architecture_for(pubodra_configs.P_B).name == "Pubodra"


@pytest.mark.parametrize("change,message", [
    (lambda c: c["layers"][0].update(type="convolution"), "not a mixer"),
    (lambda c: c["layers"][0]["mixer"].pop("kv_rank"), "kv_rank"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=5), "even"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=12), "at most"),
    (lambda c: c["layers"][2]["mlp"]["router"].update(top=6), "exceeds"),
    (lambda c: c["layers"][0]["mlp"].update(kind="gated"), "neither"),
    (lambda c: c["loop"].update(stop=5), "does not lie"),
    (lambda c: c.pop("width"), "width"),
    (lambda c: c["norm"].update(eps=0.0), "eps"),
])
def test_configuration_refuses(change, message):
    cfg = copy.deepcopy(pubodra_configs.P_B)
    change(cfg)
    with pytest.raises(ConfigError, match=message):
        PubodraConfig.from_dict(cfg)


def test_run_order_and_tensors_of_a_repeated_stack():
    spec = pubodra_model_spec(PubodraConfig.from_dict(pubodra_configs.P_B))
    assert [e.layer for e in spec.run_order] == [0, 1, 2, 1, 2, 3]
    marks = [(i, e.before.params["row"]) for i, e in enumerate(spec.run_order) if e.before is not None]
    assert marks == [(1, 0), (3, 1)]                       # once a pass, right before its first layer
    assert [l.block for l in spec.layers] == ["prenorm_residual", "prenorm_mixer", "prenorm_residual", "prenorm_residual"]
    names = declared_tensors(spec)
    assert names["loop.step"].shape == (2, 50) and names["embed"].shape == (131, 50)
    assert names["l0.mix.q"].shape == (3 * 17, 50) and names["l0.mix.dkv"].shape == (21 + 10, 50)
    assert names["l0.mix.uk"].shape == (3 * 7, 21) and names["l0.mix.uv"].shape == (3 * 9, 21)
    assert names["l0.norm1.alpha"].shape == () and "l1.norm2" not in names and "l1.mlp.up" not in names
    assert names["l2.mlp.e4.down"].shape == (50, 30) and names["l2.mlp.router"].shape == (5, 50)
    assert "lm_head.weight" not in names and names["final.norm.b"].shape == (50,)
    no_loop = pubodra_model_spec(PubodraConfig.from_dict(pubodra_configs.P_C))
    assert [e.layer for e in no_loop.run_order] == [0, 1] and "loop.step" not in declared_tensors(no_loop)


def test_latent_pages_follow_the_window():
    """Every pass of a layer is a site of its own; sites with the same row width and window share a
    block table, and pages that the window has passed go back."""
    need_a, need_b = PagedLatent(40, 24), PagedLatent(40, None)
    cache = CacheManager([need_a, need_b, need_a], block_size=8, num_blocks=16, max_seqs=2)
    assert len(cache.groups) == 2 and cache.groups[0].sites == [0, 2]
    assert cache.bytes_per_block(torch.bfloat16) == 3 * 8 * 40 * 2
    cache.admit("r")
    cache.reserve("r", 50)
    cache.commit("r")
    # the next query, at position 50, reads positions 27 .. 50: pages 0 to 2 (positions 0 .. 23) are free
    assert list(cache.groups[0].tables["r"])[:3] == [-1, -1, -1] and cache.groups[0].tables["r"][3] >= 0
    assert all(p >= 0 for p in cache.groups[1].tables["r"])
    cache.release("r")
    cache.check()
    assert all(g.pool.num_free() == 16 for g in cache.groups)


@pytest.mark.parametrize("key", ["A", "B", "C"])
@pytest.mark.parametrize("family", ["whole", "tail", "chunked", "mixed"])
def test_step_function_matches_plain(monkeypatch, key, family):
    reference_ops.install(monkeypatch)
    cfg, page, seed = pubodra_configs.ALL[key]
    weights = random_weights(cfg, seed, std=pubodra_configs.STD)
    prompts = prompts_for({"vocab_size": cfg["vocab"]}, {"A": [1, 12, 45], "B": [2, 40, 21], "C": [30, 9]}[key], seed)
    steps = {"whole": traces.whole, "tail": traces.tail_decode, "chunked": traces.chunked,
             "mixed": traces.mixed}[family](prompts)
    blocks = traces.max_live_tokens(steps, page) // page
    runner = make_runner(cfg, weights, page, blocks, "float32", "cpu")
    got = replay(runner, steps)
    refs = {n: plain_pubodra.forward(cfg, weights, ids) for n, ids in prompts.items()}
    compare(got, cfg, weights, prompts, 2e-5, refs)
    assert not runner.cache.requests
    for g in runner.cache.groups:
        assert g.pool.num_free() == blocks


def test_stream_after_every_layer_run(monkeypatch):
    """The residual stream after each site of the run order, a repeated layer counted each time."""
    reference_ops.install(monkeypatch)
    cfg, page, seed = pubodra_configs.ALL["B"]
    weights = random_weights(cfg, seed, std=pubodra_configs.STD)
    ids = prompts_for({"vocab_size": cfg["vocab"]}, [19], seed)["r0"]
    want = []
    plain_pubodra.forward(cfg, weights, ids, trace=want)
    runner = make_runner(cfg, weights, page, 8, "float32", "cpu")
    seen = []
    for layer in runner.model.layers:
        block, inner = layer.block, layer.block.forward

        def spy(stream, site, inner=inner):
            inner(stream, site)
            seen.append((stream.h + stream.pending.to(torch.float32)).double().clone())
        block.forward = spy
    from lucciola_amd.engine.batch import StepEntry
    runner.step([StepEntry("r", ids, [len(ids) - 1])])
    assert len(seen) == len(want) == 6
    for got, ref in zip(seen, want):
        assert float((got - ref).abs().max()) < 1e-5 * float(ref.abs().max())


def test_greedy_generation_through_the_scheduler(monkeypatch):
    reference_ops.install(monkeypatch)
    cfg, page, seed = pubodra_configs.ALL["A"]
    weights = random_weights(cfg, seed, std=0.2)
    arch = architecture_for(cfg)
    config = arch.read_config(cfg)
    model = _build(arch.model_spec(config), DictSource(weights), "float32", "cpu")
    engine = LLMEngine(model, config, EngineConfig(dtype="float32", block_size=page, max_blocks=40, max_seqs=3,
                                                   max_tokens_per_step=9, device="cpu", run_ahead=False))
    prompts = list(prompts_for({"vocab_size": cfg["vocab"]}, [4, 13, 27], seed + 1).values())
    got = engine.generate(prompts, SamplingParams(max_new_tokens=5))
    assert got == [plain_pubodra.greedy(cfg, weights, p, 5) for p in prompts]
    engine.runner.cache.check()
    assert not engine.runner.cache.requests


def test_latent_attention_planner():
    """Tiles of up to 16 tokens of one request, a lone token a tile of its own, the tiles that see the
    most keys first; sizes follow from the batch's make-up alone."""
    from lucciola_amd.engine.batch import HostLayout
    from lucciola_amd.kernels import ops
    layout = HostLayout(num_requests=4, num_tokens=1 + 40 + 1 + 16, q_start=[0, 1, 41, 42, 58],
                        first_position=[299, 0, 7, 100], block_size=16, single=False)
    arrays, info = ops.plan_latent_attention(layout)
    tiles = arrays["tiles"].tolist()
    assert info == {"any_portion": True, "any_lone": True, "num_tiles": 6}
    assert sorted(tiles) == sorted([[0, 1, 0, 299], [1, 16, 1, 0], [17, 16, 1, 16], [33, 8, 1, 32], [41, 1, 2, 7],
                                    [42, 16, 3, 100]])
    ends = [t[3] + t[1] for t in tiles]
    assert ends == sorted(ends, reverse=True) and tiles[0] == [0, 1, 0, 299]
    single = HostLayout(3, 3, [0, 1, 2, 3], [5, 50, 9], 16, True)
    arrays, info = ops.plan_latent_attention(single)
    assert info["any_portion"] is False and arrays["tiles"].shape == (3, 4)


@pytest.mark.parametrize("seed", [0, 1, 2, 3, 4, 5])
def test_random_configurations_on_the_host(monkeypatch, seed):
    reference_ops.install(monkeypatch)
    cfg, page = pubodra_configs.random_configuration(seed)
    weights = random_weights(cfg, 100 + seed, std=pubodra_configs.STD)
    prompts = prompts_for({"vocab_size": cfg["vocab"]}, [3, 35, 18], seed)
    steps = traces.mixed(prompts, seed=seed)
    runner = make_runner(cfg, weights, page, traces.max_live_tokens(steps, page) // page, "float32", "cpu")
    refs = {n: plain_pubodra.forward(cfg, weights, ids) for n, ids in prompts.items()}
    compare(replay(runner, steps), cfg, weights, prompts, 2e-5, refs)
