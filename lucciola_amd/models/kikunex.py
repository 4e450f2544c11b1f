"""The Kikunex decoder as data: how its configuration becomes a :class:`ModelSpec`.

The embedding's row passes an RMS norm whose weight is one number; so do the stream before each
branch of a layer and before the head, whose logits are scaled by ``logit_scale``.  Every layer is a
pre-norm residual block; what its mixer reads is first blended with the previous token's normed row
(token shift, a learned rate per coordinate).  The mixer is lightning attention (linear attention with a
fixed decay per head and a matrix of state per head and request) or latent attention (queries through a
latent of their own, a small cached latent per token, a rotated key part shared by all heads, a sliding
window, a learned sink in every head's softmax, one output gate per head); the feed-forward is dense
(xIELU), routed (sigmoid router with a correction for the choice, experts in groups, squared-ReLU
experts) or absent.  A stretch of the layers may run several times in a row with the same weights: each
run of a layer is a site of the run order with a cache and state of its own; before every pass a learned
vector is added to the stream, and before every pass but the first also the embedding's output.

Tensor names: ``embed``, ``embed.norm``, ``loop.step``, ``final.norm``, ``head`` and, for layer i,
``l<i>.norm1|norm2|shift``, ``l<i>.mix.{q,k,v,g,o,norm}`` (lightning) or
``l<i>.mix.{dq,dq.norm,uq,dkv,dkv.norm,uk,uv,sink,g,o}`` (latent attention), ``l<i>.mlp.{up,down,act}`` or
``l<i>.mlp.{router,correction}`` with ``l<i>.mlp.e<k>.{up,down}``.
"""
from __future__ import annotations

from ..config.kikunex_config import ARCHITECTURE, KikunexConfig, LayerConfig
from ..config.registry import ARCHITECTURES, Architecture
from ..config.specs import ModelSpec, PartSpec, RunEntry, shifted_layer


def kikunex_layer(cfg: KikunexConfig, i: int, layer: LayerConfig):
    p = f"l{i}."
    m = layer.mixer
    norm = PartSpec("rms", {"size": cfg.width, "eps": cfg.norm_eps, "scalar": True})
    shift = PartSpec("token_shift", {"size": cfg.width})
    names = {"mixer_norm.weight": p + "norm1", "mixer_shift.mix": p + "shift"}
    if layer.type == "lightning":
        mixer = PartSpec("lightning", {"hidden_size": cfg.width, "num_heads": m.heads, "key_dim": m.dim,
                                       "value_dim": m.vdim, "decays": tuple(m.decay), "norm_eps": cfg.norm_eps})
        names.update({"mixer.q": p + "mix.q", "mixer.k": p + "mix.k", "mixer.v": p + "mix.v",
                      "mixer.gate": p + "mix.g", "mixer.norm": p + "mix.norm", "mixer.o": p + "mix.o"})
    else:
        position = None
        if m.rot is not None:
            position = PartSpec("rotary", {"rotary_dim": m.rot.dims, "theta": m.rot.base, "pairing": "half"})
        mixer = PartSpec("latent_attention", {
            "hidden_size": cfg.width, "num_heads": m.heads, "dim": m.dim, "rot_dim": m.rot_dim,
            "vdim": m.vdim, "kv_rank": m.kv_rank, "scale": m.scale, "eps": cfg.norm_eps,
            "position": position, "window": m.window, "gate": True, "gate_per_head": True,
            "q_rank": m.q_rank, "sink": True})
        names.update({"mixer.dq": p + "mix.dq", "mixer.dq_norm": p + "mix.dq.norm", "mixer.uq": p + "mix.uq",
                      "mixer.dkv": p + "mix.dkv", "mixer.dkv_norm": p + "mix.dkv.norm",
                      "mixer.uk": p + "mix.uk", "mixer.uv": p + "mix.uv", "mixer.sink": p + "mix.sink",
                      "mixer.g": p + "mix.g", "mixer.o": p + "mix.o"})
    if layer.mlp is None:
        return shifted_layer(mixer, None, norm, None, shift, names)
    names["feed_forward_norm.weight"] = p + "norm2"
    if layer.mlp.kind == "dense":
        feed_forward = PartSpec("mlp", {"hidden_size": cfg.width, "intermediate_size": layer.mlp.ff,
                                        "activation": "xielu"})
        names.update({"feed_forward.up": p + "mlp.up", "feed_forward.down": p + "mlp.down",
                      "feed_forward.act": p + "mlp.act"})
    else:
        feed_forward = PartSpec("routed_mlp", {
            "hidden_size": cfg.width, "intermediate_size": layer.mlp.ff, "experts": layer.mlp.experts,
            "top": layer.mlp.top, "activation": "relu_squared", "scores": "sigmoid", "renormalise": False,
            "correction": True, "groups": layer.mlp.groups, "keep_groups": layer.mlp.keep,
            "weight_scale": layer.mlp.scale})
        names.update({"feed_forward.router": p + "mlp.router", "feed_forward.correction": p + "mlp.correction"})
        for k in range(layer.mlp.experts):
            names[f"feed_forward.experts.{k}.up"] = p + f"mlp.e{k}.up"
            names[f"feed_forward.experts.{k}.down"] = p + f"mlp.e{k}.down"
    return shifted_layer(mixer, feed_forward, norm, norm, shift, names)


def kikunex_run_order(cfg: KikunexConfig):
    n = len(cfg.layers)
    if cfg.loop is None:
        return [RunEntry(i) for i in range(n)]
    loop = cfg.loop
    order = [RunEntry(i) for i in range(loop.start)]
    for turn in range(loop.times):
        for i in range(loop.start, loop.stop):
            if i == loop.start:
                # the pass's own vector, and from the second pass on the embedding's output once more
                step = PartSpec("row_offset", {"size": cfg.width, "rows": loop.times, "row": turn,
                                               "add_origin": turn > 0})
                order.append(RunEntry(i, before=step, before_names={"table": "loop.step"}))
            else:
                order.append(RunEntry(i))
    return order + [RunEntry(i) for i in range(loop.stop, n)]


def kikunex_model_spec(cfg: KikunexConfig) -> ModelSpec:
    layers = [kikunex_layer(cfg, i, layer) for i, layer in enumerate(cfg.layers)]
    sizes = {"vocab_size": cfg.vocab, "hidden_size": cfg.width}
    return ModelSpec(
        hidden_size=cfg.width, vocab_size=cfg.vocab, embedding_name="embed", layers=layers,
        run_order=kikunex_run_order(cfg),
        final_norm=PartSpec("rms", {"size": cfg.width, "eps": cfg.norm_eps, "scalar": True}),
        final_norm_names={"weight": "final.norm"},
        head_name="head", init_std=cfg.initializer_range, max_positions=0,
        embedding=PartSpec("normed_token_embedding", {**sizes, "eps": cfg.norm_eps}),
        embedding_names={"norm": "embed.norm"},
        head=PartSpec("linear_head", {**sizes, "scale": cfg.logit_scale}))


ARCHITECTURES.register(ARCHITECTURE, Architecture(
    name=ARCHITECTURE, read_config=KikunexConfig.from_dict, model_spec=kikunex_model_spec))
