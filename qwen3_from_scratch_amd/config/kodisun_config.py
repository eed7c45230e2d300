"""Typed configuration of the Kodisun decoder, read from its own config.json keys.

Its config.json is nested: `layers` is a list with one entry per layer (`type` names the mixer,
`mixer` holds the mixer's sizes and constants, `mlp` the feed-forward's or null), `loop` names a
run of layers that is passed several times with the same weights, `norm.eps` is every norm's
epsilon. The architecture is named by the string `architecture`. Nothing has a default: a size
that is missing is an error; what may be absent (a window, a frequency scaling, a shared expert,
a feed-forward, a loop) is absent as a whole.
"""

import copy
import json
from dataclasses import dataclass

from .model_config import ConfigError

NAME = "Kodisun"
# the engine asks every architecture how long a request may become; this one has rotations that
# are computed from the position itself and no table that could end
NO_POSITION_LIMIT = 1 << 30


def _get(data, key, kind, where):
    if not isinstance(data, dict) or key not in data:
        raise ConfigError("config.json: %s lacks %r" % (where, key))
    value = data[key]
    if kind is float and isinstance(value, int) and not isinstance(value, bool):
        value = float(value)
    if isinstance(value, bool) or not isinstance(value, kind):
        raise ConfigError("config.json: %s.%s must be %s, found %r" % (where, key, kind.__name__, value))
    return value


def _positive(data, key, where):
    value = _get(data, key, int, where)
    if value <= 0:
        raise ConfigError("config.json: %s.%s must be positive" % (where, key))
    return value


@dataclass(frozen=True)
class Rotation:
    """Rotary position over the first `dims` numbers of a vector, pairs (2i, 2i + 1), frequency
    base^(-2i / dims); `scaling` = (factor, original, fast, slow) or None."""

    dims: int
    base: float
    scaling: tuple = None

    @classmethod
    def read(cls, data, where):
        dims = _positive(data, "dims", where)
        if dims % 2:
            raise ConfigError("config.json: %s.dims must be even" % where)
        base = _get(data, "base", float, where)
        scaling = data.get("scaling")
        if scaling is not None:
            s = where + ".scaling"
            scaling = tuple(_get(scaling, k, float, s) for k in ("factor", "original", "fast", "slow"))
            if scaling[0] <= 0 or scaling[1] <= 0 or scaling[2] <= 0 or scaling[3] <= 0:
                raise ConfigError("config.json: %s must hold positive numbers" % s)
        if base <= 0:
            raise ConfigError("config.json: %s.base must be positive" % where)
        return cls(dims, base, scaling)


@dataclass(frozen=True)
class LatentAttentionSizes:
    heads: int
    dim: int            # unrotated query/key numbers per head
    rot_dim: int        # rotated ones
    vdim: int
    q_rank: int
    kv_rank: int
    scale: float
    window: int         # 0: every earlier token is seen
    rot: Rotation

    @classmethod
    def read(cls, data, where):
        mask = data.get("mask")
        window = 0
        if mask is not None:
            window = _positive(mask, "size", where + ".mask")
        rot = Rotation.read(_get(data, "rot", dict, where), where + ".rot")
        sizes = cls(heads=_positive(data, "heads", where), dim=_positive(data, "dim", where),
                    rot_dim=_positive(data, "rot_dim", where), vdim=_positive(data, "vdim", where),
                    q_rank=_positive(data, "q_rank", where), kv_rank=_positive(data, "kv_rank", where),
                    scale=_get(data, "scale", float, where), window=window, rot=rot)
        if rot.dims > sizes.rot_dim:
            raise ConfigError("config.json: %s.rot.dims (%d) exceeds rot_dim (%d)" % (where, rot.dims, sizes.rot_dim))
        return sizes


@dataclass(frozen=True)
class RoutedFeedForwardSizes:
    experts: int
    top: int
    expert_ff: int
    shared_ff: int      # 0: no shared expert

    @classmethod
    def read(cls, data, where):
        kind = _get(data, "kind", str, where)
        if kind != "moe":
            raise ConfigError("config.json: %s.kind %r is not known (only 'moe')" % (where, kind))
        router = _get(data, "router", dict, where)
        shared = data.get("shared")
        sizes = cls(experts=_positive(router, "experts", where + ".router"), top=_positive(router, "top", where + ".router"),
                    expert_ff=_positive(_get(data, "expert", dict, where), "ff", where + ".expert"),
                    shared_ff=_positive(shared, "ff", where + ".shared") if shared is not None else 0)
        if sizes.top > sizes.experts:
            raise ConfigError("config.json: %s.router.top exceeds the number of experts" % where)
        return sizes


@dataclass(frozen=True)
class KodisunLayer:
    type: str
    mixer: LatentAttentionSizes
    mlp: RoutedFeedForwardSizes = None


@dataclass(frozen=True)
class KodisunConfig:
    architecture: str
    vocab: int
    width: int
    eps: float
    layers: tuple
    loop: tuple                 # (start, stop, times); (0, 0, 1) without a loop
    raw: str                    # config.json as it was read, for `to_dict`
    eos_token_ids: tuple = ()
    max_position_embeddings: int = NO_POSITION_LIMIT

    @classmethod
    def from_dict(cls, data):
        layers = []
        listed = _get(data, "layers", list, "config")
        if not listed:
            raise ConfigError("config.json: 'layers' is empty")
        for i, entry in enumerate(listed):
            where = "layers[%d]" % i
            kind = _get(entry, "type", str, where)
            if kind != "latent_attention":
                raise ConfigError("config.json: %s.type %r is not known (only 'latent_attention')" % (where, kind))
            mixer = LatentAttentionSizes.read(_get(entry, "mixer", dict, where), where + ".mixer")
            mlp = entry.get("mlp")
            layers.append(KodisunLayer(kind, mixer, RoutedFeedForwardSizes.read(mlp, where + ".mlp") if mlp is not None
                                       else None))
        loop = data.get("loop")
        if loop is None:
            loop = (0, 0, 1)
        else:
            loop = (_get(loop, "start", int, "loop"), _get(loop, "stop", int, "loop"), _positive(loop, "times", "loop"))
            if not 0 <= loop[0] <= loop[1] <= len(layers):
                raise ConfigError("config.json: loop %d..%d does not lie within the %d layers" % (loop[0], loop[1], len(layers)))
        eps = _get(_get(data, "norm", dict, "config"), "eps", float, "norm")
        if not eps >= 0.0:
            raise ConfigError("config.json: norm.eps must not be negative")
        return cls(architecture=NAME, vocab=_positive(data, "vocab", "config"), width=_positive(data, "width", "config"),
                   eps=eps, layers=tuple(layers), loop=loop, raw=json.dumps(data, sort_keys=True))

    def to_dict(self):
        return copy.deepcopy(json.loads(self.raw))
