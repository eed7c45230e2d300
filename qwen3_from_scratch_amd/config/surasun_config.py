"""Typed configuration of the Surasun decoder, read from its own config.json keys.

Its config.json is nested like Kodisun's: `layers` lists the layers in their order; each entry
names its mixer under `type` ("mamba2", "rglru" or "parallel"), gives the mixer's sizes and
constants under `mixer` and its feed-forward under `mlp` (null for none). `norm.eps` is every
norm's epsilon, `residual_mult` multiplies what a sublayer adds to the residual, and `streams`,
if present, is the number of copies the residual is held in (hyper-connections); without it the
residual is the ordinary single one. Every size is required.
"""

import copy
import json
from dataclasses import dataclass

from .kodisun_config import NO_POSITION_LIMIT, _get, _positive
from .model_config import ConfigError

NAME = "Surasun"


@dataclass(frozen=True)
class Turning:
    """A rotary encoding of the first `dims` numbers of a head by base^(-2i / dims); dims 0: none."""

    dims: int = 0
    base: float = 1.0

    @classmethod
    def read(cls, data, where, most):
        if data is None:
            return cls()
        dims = _positive(data, "dims", where)
        base = _get(data, "base", float, where)
        if dims % 2 or dims > most:
            raise ConfigError("config.json: %s.dims must be even and at most the head's size %d" % (where, most))
        if base <= 0:
            raise ConfigError("config.json: %s.base must be positive" % where)
        return cls(dims, base)


@dataclass(frozen=True)
class Mamba2Sizes:
    heads: int
    vdim: int
    state: int
    groups: int
    conv: int
    norm_groups: int

    @classmethod
    def read(cls, data, where):
        sizes = cls(**{key: _positive(data, key, where) for key in ("heads", "vdim", "state", "groups", "conv", "norm_groups")})
        if sizes.heads % sizes.groups:
            raise ConfigError("config.json: %s.heads must be a multiple of groups" % where)
        if (sizes.heads * sizes.vdim) % sizes.norm_groups:
            raise ConfigError("config.json: %s.norm_groups must divide heads * vdim" % where)
        return sizes


@dataclass(frozen=True)
class RecurrentUnitSizes:
    width: int
    blocks: int
    conv: int

    @classmethod
    def read(cls, data, where):
        sizes = cls(**{key: _positive(data, key, where) for key in ("width", "blocks", "conv")})
        if sizes.width % sizes.blocks:
            raise ConfigError("config.json: %s.blocks must divide width" % where)
        return sizes


@dataclass(frozen=True)
class SoftmaxSideSizes:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    softcap: float          # 0: scores are not capped
    rot: Turning

    @classmethod
    def read(cls, data, where):
        dim = _positive(data, "dim", where)
        cap = _get(data, "softcap", float, where) if data.get("softcap") is not None else 0.0
        sizes = cls(heads=_positive(data, "heads", where), kv_heads=_positive(data, "kv_heads", where), dim=dim,
                    vdim=_positive(data, "vdim", where), scale=_get(data, "scale", float, where), softcap=cap,
                    rot=Turning.read(data.get("rot"), where + ".rot", dim))
        if sizes.heads % sizes.kv_heads:
            raise ConfigError("config.json: %s.heads must be a multiple of kv_heads" % where)
        if cap < 0:
            raise ConfigError("config.json: %s.softcap must not be negative" % where)
        return sizes


@dataclass(frozen=True)
class RetentionSideSizes:
    heads: int
    dim: int
    vdim: int
    decay: tuple
    rot: Turning

    @classmethod
    def read(cls, data, where):
        heads, dim = _positive(data, "heads", where), _positive(data, "dim", where)
        decay = _get(data, "decay", list, where)
        if len(decay) != heads or not all(isinstance(v, (int, float)) and not isinstance(v, bool) for v in decay):
            raise ConfigError("config.json: %s.decay must hold one number per head" % where)
        return cls(heads=heads, dim=dim, vdim=_positive(data, "vdim", where), decay=tuple(float(v) for v in decay),
                   rot=Turning.read(data.get("rot"), where + ".rot", dim))


@dataclass(frozen=True)
class ParallelSizes:
    left: SoftmaxSideSizes
    right: RetentionSideSizes
    left_scale: float
    right_scale: float

    @classmethod
    def read(cls, data, where):
        return cls(left=SoftmaxSideSizes.read(_get(data, "left", dict, where), where + ".left"),
                   right=RetentionSideSizes.read(_get(data, "right", dict, where), where + ".right"),
                   left_scale=_get(data, "left_scale", float, where), right_scale=_get(data, "right_scale", float, where))


MIXERS = {"mamba2": Mamba2Sizes, "rglru": RecurrentUnitSizes, "parallel": ParallelSizes}


@dataclass(frozen=True)
class SurasunLayer:
    type: str
    mixer: object
    ff: int = 0             # the dense feed-forward's inner size; 0: the layer has none


@dataclass(frozen=True)
class SurasunConfig:
    architecture: str
    vocab: int
    width: int
    eps: float
    residual_mult: float
    streams: int            # 0: one ordinary residual
    layers: tuple
    raw: str
    eos_token_ids: tuple = ()
    max_position_embeddings: int = NO_POSITION_LIMIT

    @classmethod
    def from_dict(cls, data):
        listed = _get(data, "layers", list, "config")
        if not listed:
            raise ConfigError("config.json: 'layers' is empty")
        layers = []
        for i, entry in enumerate(listed):
            where = "layers[%d]" % i
            kind = _get(entry, "type", str, where)
            if kind not in MIXERS:
                raise ConfigError("config.json: %s.type %r is not known (%s)" % (where, kind, ", ".join(sorted(MIXERS))))
            mixer = MIXERS[kind].read(_get(entry, "mixer", dict, where), where + ".mixer")
            mlp, ff = entry.get("mlp"), 0
            if mlp is not None:
                if _get(mlp, "kind", str, where + ".mlp") != "dense":
                    raise ConfigError("config.json: %s.mlp.kind %r is not known (only 'dense')" % (where, mlp["kind"]))
                ff = _positive(mlp, "ff", where + ".mlp")
            layers.append(SurasunLayer(kind, mixer, ff))
        eps = _get(_get(data, "norm", dict, "config"), "eps", float, "norm")
        if not eps >= 0.0:
            raise ConfigError("config.json: norm.eps must not be negative")
        mult = _get(data, "residual_mult", float, "config") if data.get("residual_mult") is not None else 1.0
        streams = _positive(data, "streams", "config") if data.get("streams") is not None else 0
        return cls(architecture=NAME, vocab=_positive(data, "vocab", "config"), width=_positive(data, "width", "config"),
                   eps=eps, residual_mult=mult, streams=streams, layers=tuple(layers),
                   raw=json.dumps(data, sort_keys=True))

    def to_dict(self):
        return copy.deepcopy(json.loads(self.raw))
