"""The Rununex decoder as data: how its configuration becomes a :class:`ModelSpec`.

The embedding's row is multiplied by a number.  Every layer is x + m mixer(LN(x)), then x + m ff(LN(x)) with
layer norms that have a weight and no bias and one number m for the model; the same norm stands before the
untied head, whose logits are scaled.  The mixer is differential attention (two score maps a head over the
same values, short convolutions on q, k and v, interleaved rotary pairs with frequencies scaled by wavelength,
a mask of chunks) or two mixers side by side on the same input: attention with unit q and k, a bias that grows
with the logarithm of the distance, a sink and an output gate, beside a state-space mixer; their outputs are
added with a scale each.  The feed-forward is a mixture of gated experts chosen by sigmoid scores, each fed its
score times the input, plus a shared expert; or none.

Tensor names: ``embed``, ``final.norm``, ``head`` and, for layer i, ``l<i>.norm1|norm2``,
``l<i>.mix.{q,k,v,o}``, ``l<i>.mix.{q,k,v}.conv``, ``l<i>.mix.{lq1,lk1,lq2,lk2}`` (attention) or
``l<i>.mix.left.{q,k,v,g,o,r1,r2,sink}`` and ``l<i>.mix.right.{in,conv,conv.b,dt_bias,A_log,D,norm,o}``
(parallel), ``l<i>.mlp.router``, ``l<i>.mlp.e<k>.{gate,up,down}``, ``l<i>.mlp.shared.{gate,up,down}``.
"""
from __future__ import annotations

from ..config.registry import ARCHITECTURES, Architecture
from ..config.rununex_config import ARCHITECTURE, LayerConfig, RununexConfig
from ..config.specs import ModelSpec, PartSpec, RunEntry, mixer_only_layer, prenorm_layer


def _norm(cfg: RununexConfig) -> PartSpec:
    return PartSpec("layer_norm", {"size": cfg.width, "eps": cfg.norm_eps, "bias": False,
                                   "branch_scale": cfg.residual_mult})


def rununex_layer(cfg: RununexConfig, i: int, layer: LayerConfig):
    p = f"l{i}."
    m = layer.mixer
    names = {"mixer_norm.weight": p + "norm1"}
    if layer.type == "attention":
        position = None
        if m.rot is not None:
            scaling = None
            if m.rot.scaling is not None:
                s = m.rot.scaling
                scaling = {"kind": "wavelength", "factor": s.factor, "original": s.original, "low": s.low,
                           "high": s.high}
            position = PartSpec("rotary", {"rotary_dim": m.rot.dims, "theta": m.rot.base, "pairing": "interleaved",
                                           "scaling": scaling})
        mixer = PartSpec("masked_attention", {
            "hidden_size": cfg.width, "num_heads": m.heads, "num_kv_heads": m.kv_heads, "head_dim": m.dim,
            "value_dim": m.vdim, "scale": m.scale, "eps": cfg.norm_eps, "maps": 2, "difference": m.diff,
            "conv_taps": m.conv, "position": position, "chunk": m.chunk})
        names.update({"mixer." + k: p + "mix." + k for k in ("q", "k", "v", "o", "lq1", "lk1", "lq2", "lk2")})
        if m.conv:
            names.update({f"mixer.{k}_conv": p + f"mix.{k}.conv" for k in ("q", "k", "v")})
    else:
        left = PartSpec("masked_attention", {
            "hidden_size": cfg.width, "num_heads": m.left.heads, "num_kv_heads": m.left.kv_heads,
            "head_dim": m.left.dim, "value_dim": m.left.vdim, "scale": m.left.scale, "eps": cfg.norm_eps,
            "unit_qk": True, "distance_bias": True, "sink": True, "gate": True, "chunk": m.left.chunk})
        right = PartSpec("state_space", {
            "hidden_size": cfg.width, "num_heads": m.right.heads, "value_dim": m.right.vdim,
            "state_size": m.right.state, "groups": m.right.groups, "conv_taps": m.right.conv,
            "norm_groups": m.right.norm_groups, "norm_eps": cfg.norm_eps})
        mixer = PartSpec("parallel", {"left": left, "right": right, "left_scale": m.left_scale,
                                      "right_scale": m.right_scale})
        names.update({"mixer.left." + k: p + "mix.left." + k for k in ("q", "k", "v", "g", "o", "r1", "r2", "sink")})
        names.update({"mixer.right." + k: p + "mix.right." + k
                      for k in ("in", "conv", "dt_bias", "A_log", "D", "norm", "o")})
        names["mixer.right.conv_bias"] = p + "mix.right.conv.b"
    if layer.mlp is None:
        return mixer_only_layer(mixer, _norm(cfg), names)
    mlp = layer.mlp
    feed_forward = PartSpec("routed_gated_mlp", {
        "hidden_size": cfg.width, "intermediate_size": mlp.ff, "experts": mlp.experts, "top": mlp.top,
        "activation": "silu", "scores": "sigmoid", "weigh": "input", "shared_size": mlp.shared_ff,
        "shared_gate": False})
    names["feed_forward_norm.weight"] = p + "norm2"
    names["feed_forward.router"] = p + "mlp.router"
    for k in range(mlp.experts):
        for which in ("gate", "up", "down"):
            names[f"feed_forward.experts.{k}.{which}"] = p + f"mlp.e{k}.{which}"
    if mlp.shared_ff:
        for which in ("gate", "up", "down"):
            names[f"feed_forward.shared.{which}"] = p + f"mlp.shared.{which}"
    return prenorm_layer(mixer, feed_forward, _norm(cfg), _norm(cfg), names)


def rununex_model_spec(cfg: RununexConfig) -> ModelSpec:
    layers = [rununex_layer(cfg, i, layer) for i, layer in enumerate(cfg.layers)]
    sizes = {"vocab_size": cfg.vocab, "hidden_size": cfg.width}
    return ModelSpec(
        hidden_size=cfg.width, vocab_size=cfg.vocab, embedding_name="embed", layers=layers,
        run_order=[RunEntry(i) for i in range(len(layers))],
        final_norm=_norm(cfg), final_norm_names={"weight": "final.norm"},
        head_name="head", init_std=cfg.initializer_range, max_positions=0,
        embedding=PartSpec("token_embedding", {**sizes, "scale": cfg.embedding_scale}),
        head=PartSpec("linear_head", {**sizes, "scale": cfg.logit_scale}))


ARCHITECTURES.register(ARCHITECTURE, Architecture(
    name=ARCHITECTURE, read_config=RununexConfig.from_dict, model_spec=rununex_model_spec))
