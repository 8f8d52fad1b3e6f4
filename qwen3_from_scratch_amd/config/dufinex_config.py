"""Typed configuration of the Dufinex decoder, read from its own config.json keys.

Its config.json is nested like Kodisun's and Surasun's: `layers` lists the layers in their order;
each entry names its mixer under `type` ("attention" or "channel_delta"), gives the mixer's sizes
and constants under `mixer` and its feed-forward under `mlp` (null for none; `kind` "dense" or
"moe"). `norm.eps` is every norm's epsilon, `embedding.scale` multiplies the embedded rows. An
attention layer whose mixer says `kv_from: j` has no keys and values of its own and reads those of
layer j. Every size is required.
"""

import copy
import json
from dataclasses import dataclass

from .kodisun_config import NO_POSITION_LIMIT, _get, _positive
from .model_config import ConfigError

NAME = "Dufinex"


@dataclass(frozen=True)
class SinkAttentionSizes:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    kv_from: int = None         # the layer whose keys and values this one reads; None: its own

    @classmethod
    def read(cls, data, where):
        sizes = cls(heads=_positive(data, "heads", where), kv_heads=_positive(data, "kv_heads", where),
                    dim=_positive(data, "dim", where), vdim=_positive(data, "vdim", where),
                    scale=_get(data, "scale", float, where),
                    kv_from=_get(data, "kv_from", int, where) if data.get("kv_from") is not None else None)
        if sizes.heads % sizes.kv_heads:
            raise ConfigError("config.json: %s.heads must be a multiple of kv_heads" % where)
        return sizes


@dataclass(frozen=True)
class ChannelDeltaSizes:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int

    @classmethod
    def read(cls, data, where):
        sizes = cls(**{key: _positive(data, key, where) for key in ("heads", "kv_heads", "dim", "vdim", "conv")})
        if sizes.heads % sizes.kv_heads:
            raise ConfigError("config.json: %s.heads must be a multiple of kv_heads" % where)
        return sizes


MIXERS = {"attention": SinkAttentionSizes, "channel_delta": ChannelDeltaSizes}


@dataclass(frozen=True)
class DenseSizes:
    ff: int
    limit: float

    @classmethod
    def read(cls, data, where):
        return cls(ff=_positive(data, "ff", where), limit=_limit(data, where))


@dataclass(frozen=True)
class ExpertSizes:
    experts: int
    top: int
    ff: int
    limit: float

    @classmethod
    def read(cls, data, where):
        router = _get(data, "router", dict, where)
        expert = _get(data, "expert", dict, where)
        sizes = cls(experts=_positive(router, "experts", where + ".router"), top=_positive(router, "top", where + ".router"),
                    ff=_positive(expert, "ff", where + ".expert"), limit=_limit(expert, where + ".expert"))
        if sizes.top > sizes.experts:
            raise ConfigError("config.json: %s.router.top must not exceed experts" % where)
        return sizes


def _limit(data, where):
    limit = _get(data, "limit", float, where)
    if not limit > 0:
        raise ConfigError("config.json: %s.limit must be positive" % where)
    return limit


FEED_FORWARDS = {"dense": DenseSizes, "moe": ExpertSizes}


@dataclass(frozen=True)
class DufinexLayer:
    type: str
    mixer: object
    mlp_kind: str = None        # "dense", "moe" or None: the layer has no feed-forward
    mlp: object = None


@dataclass(frozen=True)
class DufinexConfig:
    architecture: str
    vocab: int
    width: int
    eps: float
    embedding_scale: float
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
            mlp, mlp_kind, sizes = entry.get("mlp"), None, None
            if mlp is not None:
                mlp_kind = _get(mlp, "kind", str, where + ".mlp")
                if mlp_kind not in FEED_FORWARDS:
                    raise ConfigError("config.json: %s.mlp.kind %r is not known (%s)"
                                      % (where, mlp_kind, ", ".join(sorted(FEED_FORWARDS))))
                sizes = FEED_FORWARDS[mlp_kind].read(mlp, where + ".mlp")
            layers.append(DufinexLayer(kind, mixer, mlp_kind, sizes))
        for i, layer in enumerate(layers):
            j = getattr(layer.mixer, "kv_from", None)
            if j is None:
                continue
            where = "layers[%d].mixer.kv_from" % i
            if not 0 <= j < i or layers[j].type != "attention" or layers[j].mixer.kv_from is not None:
                raise ConfigError("config.json: %s must name an earlier attention layer with keys of its own" % where)
            theirs, mine = layers[j].mixer, layer.mixer
            if (theirs.kv_heads, theirs.dim, theirs.vdim) != (mine.kv_heads, mine.dim, mine.vdim):
                raise ConfigError("config.json: %s: the two layers' key heads, key and value sizes differ" % where)
        eps = _get(_get(data, "norm", dict, "config"), "eps", float, "norm")
        if not eps >= 0.0:
            raise ConfigError("config.json: norm.eps must not be negative")
        scale = _get(_get(data, "embedding", dict, "config"), "scale", float, "embedding")
        return cls(architecture=NAME, vocab=_positive(data, "vocab", "config"), width=_positive(data, "width", "config"),
                   eps=eps, embedding_scale=scale, layers=tuple(layers), raw=json.dumps(data, sort_keys=True))

    def to_dict(self):
        return copy.deepcopy(json.loads(self.raw))
