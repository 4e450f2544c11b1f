"""Typed configuration of the Rununex decoder, read from the keys of its config.json.

The file lists the layers one by one (``layers``: each with its ``type``, "attention" or "parallel", the
mixer's sizes under ``mixer`` and its feed-forward under ``mlp``, which may be null), the model's ``width`` and
``vocab``, the norms' ``eps`` under ``norm``, the embedding's ``scale`` under ``embedding``, ``residual_mult``
and ``logit_scale``.  Every size and constant is a field read from the file; nothing is assumed equal between
layers.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

from .model_config import ConfigError, read_config_json
from .pubodra_config import _get, _int

ARCHITECTURE = "Rununex"


def _float(data, key, where) -> float:
    value = _get(data, key, where)
    if isinstance(value, bool) or not isinstance(value, (int, float)):
        raise ConfigError(f"config.json: {where}.{key} must be a number, got {value!r}")
    return float(value)


@dataclass(frozen=True)
class WavelengthScaling:
    """Rotary frequencies by wavelength l against the ``original`` context: kept where l < original / high,
    divided by ``factor`` where l > original / low, blended in between."""

    factor: float
    low: float
    high: float
    original: float


@dataclass(frozen=True)
class RotaryConfig:
    base: float
    dims: int
    scaling: Optional[WavelengthScaling] = None


@dataclass(frozen=True)
class DifferentialAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    diff: float
    conv: int                       # taps of the convolutions on q, k and v (0: none)
    chunk: Optional[int]
    rot: Optional[RotaryConfig]


@dataclass(frozen=True)
class BiasedAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    chunk: Optional[int]


@dataclass(frozen=True)
class StateSpaceConfig:
    heads: int
    vdim: int
    state: int
    groups: int
    conv: int
    norm_groups: int


@dataclass(frozen=True)
class ParallelConfig:
    left: BiasedAttentionConfig
    right: StateSpaceConfig
    left_scale: float
    right_scale: float


@dataclass(frozen=True)
class MoeConfig:
    ff: int
    experts: int
    top: int
    shared_ff: int                  # 0: no shared expert


@dataclass(frozen=True)
class LayerConfig:
    type: str                       # "attention" or "parallel"
    mixer: Any                      # DifferentialAttentionConfig or ParallelConfig
    mlp: Optional[MoeConfig]


@dataclass(frozen=True)
class RununexConfig:
    vocab: int
    width: int
    norm_eps: float
    embedding_scale: float
    residual_mult: float
    logit_scale: float
    layers: Tuple[LayerConfig, ...]
    initializer_range: float = 0.02
    eos_token_ids: Tuple[int, ...] = ()
    raw: Optional[Dict[str, Any]] = None    # the dict it was read from, for writing it out again

    @staticmethod
    def from_dict(data: Dict[str, Any]) -> "RununexConfig":
        layers = _get(data, "layers", "the model")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json: 'layers' must be a list with at least one layer")
        parsed = tuple(_read_layer(entry, i) for i, entry in enumerate(layers))
        eps = _float(_get(data, "norm", "the model"), "eps", "norm")
        if not eps > 0:
            raise ConfigError("config.json: norm.eps must be positive")
        embedding = data.get("embedding") or {}
        eos = data.get("eos_token_id")
        eos_ids = () if eos is None else tuple(int(e) for e in eos) if isinstance(eos, (list, tuple)) else (int(eos),)
        return RununexConfig(
            vocab=_int(data, "vocab", "the model"), width=_int(data, "width", "the model"), norm_eps=eps,
            embedding_scale=float(embedding.get("scale", 1.0)),
            residual_mult=float(data.get("residual_mult", 1.0)), logit_scale=float(data.get("logit_scale", 1.0)),
            layers=parsed, initializer_range=float(data.get("initializer_range", 0.02)), eos_token_ids=eos_ids,
            raw=dict(data))

    @staticmethod
    def from_folder(folder: str) -> "RununexConfig":
        return RununexConfig.from_dict(read_config_json(folder))

    def to_dict(self) -> Dict[str, Any]:
        return dict(self.raw) if self.raw is not None else {}


def _heads(m, where) -> Tuple[int, int]:
    heads, kv_heads = _int(m, "heads", where), _int(m, "kv_heads", where)
    if heads % kv_heads:
        raise ConfigError(f"config.json: {where}.heads ({heads}) must be a multiple of kv_heads ({kv_heads})")
    return heads, kv_heads


def _chunk(m, where) -> Optional[int]:
    mask = m.get("mask")
    if mask and mask.get("size") is not None:
        return _int(mask, "size", where + ".mask")
    return None


def _read_rotary(m, where, dim: int) -> Optional[RotaryConfig]:
    rot = m.get("rot")
    if not rot or not rot.get("dims"):
        return None
    rw = where + ".rot"
    dims = _int(rot, "dims", rw, 2)
    if dims % 2 or dims > dim:
        raise ConfigError(f"config.json: {rw}.dims ({dims}) must be even and at most dim ({dim})")
    base = _float(rot, "base", rw)
    if not base > 1:
        raise ConfigError(f"config.json: {rw}.base must be above 1")
    scaling = rot.get("scaling")
    scaled = None
    if scaling:
        sw = rw + ".scaling"
        scaled = WavelengthScaling(_float(scaling, "factor", sw), _float(scaling, "low", sw),
                                   _float(scaling, "high", sw), _float(scaling, "original", sw))
        if scaled.factor <= 0 or scaled.original <= 0 or scaled.low <= 0 or scaled.high <= scaled.low:
            raise ConfigError(f"config.json: {sw} needs factor > 0, original > 0 and high > low > 0")
    return RotaryConfig(base, dims, scaled)


def _read_attention(m, where) -> DifferentialAttentionConfig:
    heads, kv_heads = _heads(m, where)
    dim = _int(m, "dim", where)
    diff = _float(m, "diff", where)
    return DifferentialAttentionConfig(
        heads=heads, kv_heads=kv_heads, dim=dim, vdim=_int(m, "vdim", where), scale=_float(m, "scale", where),
        diff=diff, conv=_int(m, "conv", where, 0) if m.get("conv") is not None else 0, chunk=_chunk(m, where),
        rot=_read_rotary(m, where, dim))


def _read_parallel(m, where) -> ParallelConfig:
    left = _get(m, "left", where)
    lw = where + ".left"
    heads, kv_heads = _heads(left, lw)
    left_cfg = BiasedAttentionConfig(heads=heads, kv_heads=kv_heads, dim=_int(left, "dim", lw),
                                     vdim=_int(left, "vdim", lw), scale=_float(left, "scale", lw),
                                     chunk=_chunk(left, lw))
    right = _get(m, "right", where)
    rw = where + ".right"
    right_cfg = StateSpaceConfig(heads=_int(right, "heads", rw), vdim=_int(right, "vdim", rw),
                                 state=_int(right, "state", rw), groups=_int(right, "groups", rw),
                                 conv=_int(right, "conv", rw), norm_groups=_int(right, "norm_groups", rw))
    if right_cfg.heads % right_cfg.groups:
        raise ConfigError(f"config.json: {rw}.heads ({right_cfg.heads}) must be a multiple of groups "
                          f"({right_cfg.groups})")
    if (right_cfg.heads * right_cfg.vdim) % right_cfg.norm_groups:
        raise ConfigError(f"config.json: {rw}.norm_groups ({right_cfg.norm_groups}) must divide heads * vdim")
    return ParallelConfig(left_cfg, right_cfg, _float(m, "left_scale", where), _float(m, "right_scale", where))


def _read_layer(entry: Dict[str, Any], i: int) -> LayerConfig:
    where = f"layers[{i}]"
    kind = str(_get(entry, "type", where))
    m = _get(entry, "mixer", where)
    mw = where + ".mixer"
    if kind == "attention":
        mixer = _read_attention(m, mw)
    elif kind == "parallel":
        mixer = _read_parallel(m, mw)
    else:
        raise ConfigError(f"config.json: {where}.type '{kind}' is not a mixer of this design (attention, parallel)")
    mlp = entry.get("mlp")
    mlp_cfg = None
    if mlp:
        lw = where + ".mlp"
        mkind = str(mlp.get("kind", "moe"))
        if mkind != "moe":
            raise ConfigError(f"config.json: {lw}.kind '{mkind}' is not a feed-forward of this design (moe)")
        router = _get(mlp, "router", lw)
        shared = mlp.get("shared")
        mlp_cfg = MoeConfig(ff=_int(_get(mlp, "expert", lw), "ff", lw + ".expert"),
                            experts=_int(router, "experts", lw + ".router"), top=_int(router, "top", lw + ".router"),
                            shared_ff=_int(shared, "ff", lw + ".shared") if shared else 0)
        if mlp_cfg.top > mlp_cfg.experts:
            raise ConfigError(f"config.json: {lw}.router.top ({mlp_cfg.top}) exceeds its {mlp_cfg.experts} experts")
    return LayerConfig(kind, mixer, mlp_cfg)
