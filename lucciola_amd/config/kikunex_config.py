"""Typed configuration of the Kikunex decoder, read from the keys of its config.json.

The file lists the layers one by one (``layers``: each with the ``type`` of its mixer, "lightning" or
"latent_attention", the mixer's sizes under ``mixer`` and its feed-forward under ``mlp``, which may be
null), the model's ``width`` and ``vocab``, the norms' ``eps`` under ``norm``, ``logit_scale`` and,
optionally, a ``loop``: the layers ``start`` .. ``stop - 1`` run ``times`` times in a row with the same
weights.  Every size and constant is a field read from the file; nothing is assumed equal between
layers.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple, Union

from .model_config import ConfigError, read_config_json
from .pubodra_config import LoopConfig, RotaryConfig, _get, _int

ARCHITECTURE = "Kikunex"


@dataclass(frozen=True)
class LightningConfig:
    heads: int
    dim: int                    # query/key entries of a head
    vdim: int
    decay: Tuple[float, ...]    # one per head


@dataclass(frozen=True)
class LatentAttentionConfig:
    heads: int
    dim: int            # unrotated query/key entries of a head
    rot_dim: int        # rotated query/key entries of a head; the key's are shared by all heads
    vdim: int
    kv_rank: int        # size of the cached latent
    q_rank: int         # size of the queries' latent
    scale: float
    rot: Optional[RotaryConfig]
    window: Optional[int]


@dataclass(frozen=True)
class MlpConfig:
    kind: str           # "dense" or "moe"
    ff: int             # inner size (of one expert, for "moe")
    experts: int = 0
    top: int = 0
    groups: int = 1     # the experts form this many equal groups of neighbours
    keep: int = 1       # of which this many can be chosen from
    scale: float = 1.0  # on the chosen experts' weights


@dataclass(frozen=True)
class LayerConfig:
    type: str
    mixer: Union[LightningConfig, LatentAttentionConfig]
    mlp: Optional[MlpConfig]


@dataclass(frozen=True)
class KikunexConfig:
    vocab: int
    width: int
    norm_eps: float
    logit_scale: float
    layers: Tuple[LayerConfig, ...]
    loop: Optional[LoopConfig] = None
    initializer_range: float = 0.02
    eos_token_ids: Tuple[int, ...] = ()
    raw: Optional[Dict[str, Any]] = None    # the dict it was read from, for writing it out again

    @staticmethod
    def from_dict(data: Dict[str, Any]) -> "KikunexConfig":
        layers = _get(data, "layers", "the model")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json: 'layers' must be a list with at least one layer")
        parsed = tuple(_read_layer(entry, i) for i, entry in enumerate(layers))
        loop = data.get("loop")
        loop_cfg = None
        if loop:
            loop_cfg = LoopConfig(_int(loop, "start", "loop", 0), _int(loop, "stop", "loop", 0),
                                  _int(loop, "times", "loop", 1))
            if not 0 <= loop_cfg.start < loop_cfg.stop <= len(parsed):
                raise ConfigError(f"config.json: loop {loop_cfg.start}..{loop_cfg.stop} does not lie "
                                  f"inside the {len(parsed)} layers")
        eos = data.get("eos_token_id")
        eos_ids = () if eos is None else tuple(int(e) for e in eos) if isinstance(eos, (list, tuple)) else (int(eos),)
        eps = float(_get(_get(data, "norm", "the model"), "eps", "norm"))
        if not eps > 0:
            raise ConfigError("config.json: norm.eps must be positive")
        logit_scale = data.get("logit_scale")
        return KikunexConfig(vocab=_int(data, "vocab", "the model"), width=_int(data, "width", "the model"),
                             norm_eps=eps, logit_scale=1.0 if logit_scale is None else float(logit_scale),
                             layers=parsed, loop=loop_cfg,
                             initializer_range=float(data.get("initializer_range", 0.02)),
                             eos_token_ids=eos_ids, raw=dict(data))

    @staticmethod
    def from_folder(folder: str) -> "KikunexConfig":
        return KikunexConfig.from_dict(read_config_json(folder))

    def to_dict(self) -> Dict[str, Any]:
        return dict(self.raw) if self.raw is not None else {}


def _read_lightning(m: Dict[str, Any], mw: str) -> LightningConfig:
    heads = _int(m, "heads", mw)
    decay = _get(m, "decay", mw)
    if not isinstance(decay, (list, tuple)) or len(decay) != heads:
        raise ConfigError(f"config.json: {mw}.decay must list one number for each of the {heads} heads")
    decays = tuple(float(d) for d in decay)
    if any(not 0.0 <= d <= 1.0 for d in decays):
        raise ConfigError(f"config.json: {mw}.decay must lie between 0 and 1")
    return LightningConfig(heads=heads, dim=_int(m, "dim", mw), vdim=_int(m, "vdim", mw), decay=decays)


def _read_latent(m: Dict[str, Any], mw: str) -> LatentAttentionConfig:
    rot = m.get("rot")
    rot_dim = _int(m, "rot_dim", mw, 0)
    rot_cfg = None
    if rot and rot_dim:
        rot_cfg = RotaryConfig(float(_get(rot, "base", mw + ".rot")), _int(rot, "dims", mw + ".rot", 2), None)
        if rot_cfg.dims % 2 or rot_cfg.dims > rot_dim:
            raise ConfigError(f"config.json: {mw}.rot.dims ({rot_cfg.dims}) must be even and at most "
                              f"rot_dim ({rot_dim})")
        if not rot_cfg.base > 1:
            raise ConfigError(f"config.json: {mw}.rot.base must be above 1")
    mask = m.get("mask")
    window = None
    if mask and mask.get("size") is not None:
        window = _int(mask, "size", mw + ".mask")
    mixer = LatentAttentionConfig(heads=_int(m, "heads", mw), dim=_int(m, "dim", mw, 0), rot_dim=rot_dim,
                                  vdim=_int(m, "vdim", mw), kv_rank=_int(m, "kv_rank", mw),
                                  q_rank=_int(m, "q_rank", mw), scale=float(_get(m, "scale", mw)), rot=rot_cfg,
                                  window=window)
    if mixer.dim + mixer.rot_dim <= 0:
        raise ConfigError(f"config.json: {mw}: a head needs query/key entries (dim + rot_dim > 0)")
    return mixer


def _read_mlp(mlp: Dict[str, Any], lw: str) -> MlpConfig:
    mkind = str(_get(mlp, "kind", lw))
    if mkind == "dense":
        return MlpConfig("dense", _int(mlp, "ff", lw))
    if mkind != "moe":
        raise ConfigError(f"config.json: {lw}.kind '{mkind}' is neither 'dense' nor 'moe'")
    router = _get(mlp, "router", lw)
    rw = lw + ".router"
    experts, top = _int(router, "experts", rw), _int(router, "top", rw)
    groups = router.get("groups")
    count, keep = 1, 1
    if groups:
        count, keep = _int(groups, "count", rw + ".groups"), _int(groups, "keep", rw + ".groups")
        if experts % count or keep > count:
            raise ConfigError(f"config.json: {rw}.groups: {count} groups of which {keep} are kept do not fit "
                              f"{experts} experts")
    if top > keep * (experts // count):
        raise ConfigError(f"config.json: {rw}.top ({top}) exceeds the {keep * (experts // count)} experts that "
                          f"can be chosen from")
    scale = router.get("scale")
    return MlpConfig("moe", _int(_get(mlp, "expert", lw), "ff", lw + ".expert"), experts, top, count, keep,
                     1.0 if scale is None else float(scale))


def _read_layer(entry: Dict[str, Any], i: int) -> LayerConfig:
    where = f"layers[{i}]"
    kind = str(_get(entry, "type", where))
    m = _get(entry, "mixer", where)
    if kind == "lightning":
        mixer = _read_lightning(m, where + ".mixer")
    elif kind == "latent_attention":
        mixer = _read_latent(m, where + ".mixer")
    else:
        raise ConfigError(f"config.json: {where}.type '{kind}' is not a mixer of this design "
                          f"(lightning, latent_attention)")
    mlp = entry.get("mlp")
    return LayerConfig(kind, mixer, _read_mlp(mlp, where + ".mlp") if mlp else None)
