"""Typed configuration of the Fidevik decoder, read from its own config.json keys.

Its config.json is nested like Kodisun's: `layers` lists the layers (`type` names the mixer, `mixer`
holds its sizes and constants, `mlp` the feed-forward's or null), `loop` names a run of layers that is
passed several times with the same weights, `norm.eps` is every norm's epsilon, `logit_scale`
multiplies the logits. The architecture is named by the string `architecture`. No size has a
default: one that is missing is an error; what may be absent (a rotation, groups of experts, a
shared expert, a feed-forward, a loop) is absent as a whole.
"""

import copy
import json
from dataclasses import dataclass

from .kodisun_config import NO_POSITION_LIMIT, Rotation, _get, _positive
from .model_config import ConfigError

NAME = "Fidevik"


@dataclass(frozen=True)
class GroupedAttentionSizes:
    """Softmax attention with `kv_heads` key/value heads for `heads` query heads."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot: Rotation       # None: positions do not turn queries and keys

    @classmethod
    def read(cls, data, where):
        rot = data.get("rot")
        sizes = cls(heads=_positive(data, "heads", where), kv_heads=_positive(data, "kv_heads", where),
                    dim=_positive(data, "dim", where), vdim=_positive(data, "vdim", where),
                    scale=_get(data, "scale", float, where),
                    rot=Rotation.read(rot, where + ".rot") if rot is not None else None)
        if sizes.heads % sizes.kv_heads:
            raise ConfigError("config.json: %s.kv_heads (%d) must divide heads (%d)" % (where, sizes.kv_heads, sizes.heads))
        if sizes.rot is not None:
            if sizes.rot.scaling is not None:
                raise ConfigError("config.json: %s.rot.scaling is not part of this architecture" % where)
            if sizes.rot.dims > sizes.dim:
                raise ConfigError("config.json: %s.rot.dims (%d) exceeds dim (%d)" % (where, sizes.rot.dims, sizes.dim))
        return sizes


@dataclass(frozen=True)
class PositionlessLatentSizes:
    """Latent attention without positions: queries through a latent of `q_rank`, keys and values
    from one of `kv_rank` numbers per token."""

    heads: int
    dim: int
    vdim: int
    q_rank: int
    kv_rank: int
    scale: float

    @classmethod
    def read(cls, data, where):
        return cls(heads=_positive(data, "heads", where), dim=_positive(data, "dim", where),
                   vdim=_positive(data, "vdim", where), q_rank=_positive(data, "q_rank", where),
                   kv_rank=_positive(data, "kv_rank", where), scale=_get(data, "scale", float, where))


@dataclass(frozen=True)
class DenseFeedForwardSizes:
    ff: int

    @classmethod
    def read(cls, data, where):
        return cls(ff=_positive(data, "ff", where))


@dataclass(frozen=True)
class GroupedExpertsSizes:
    experts: int
    top: int
    groups: int         # 1 without groups
    keep: int
    expert_ff: int
    shared_ff: int      # 0: no shared expert

    @classmethod
    def read(cls, data, where):
        router = _get(data, "router", dict, where)
        r = where + ".router"
        groups = router.get("groups")
        count = keep = 1
        if groups is not None:
            count, keep = _positive(groups, "count", r + ".groups"), _positive(groups, "keep", r + ".groups")
        shared = data.get("shared")
        sizes = cls(experts=_positive(router, "experts", r), top=_positive(router, "top", r), groups=count, keep=keep,
                    expert_ff=_positive(_get(data, "expert", dict, where), "ff", where + ".expert"),
                    shared_ff=_positive(shared, "ff", where + ".shared") if shared is not None else 0)
        if sizes.top > sizes.experts:
            raise ConfigError("config.json: %s.top exceeds the number of experts" % r)
        if sizes.experts % sizes.groups:
            raise ConfigError("config.json: %s.groups.count (%d) must divide the experts (%d)" % (r, sizes.groups, sizes.experts))
        if sizes.keep > sizes.groups:
            raise ConfigError("config.json: %s.groups.keep exceeds groups.count" % r)
        if sizes.top > sizes.keep * (sizes.experts // sizes.groups):
            raise ConfigError("config.json: %s.top (%d) exceeds the experts of the %d groups that are kept"
                              % (r, sizes.top, sizes.keep))
        return sizes


MIXERS = {"attention": GroupedAttentionSizes, "latent_attention": PositionlessLatentSizes}
FEED_FORWARDS = {"dense": DenseFeedForwardSizes, "moe": GroupedExpertsSizes}


@dataclass(frozen=True)
class FidevikLayer:
    type: str
    mixer: object
    mlp_kind: str = None
    mlp: object = None


@dataclass(frozen=True)
class FidevikConfig:
    architecture: str
    vocab: int
    width: int
    eps: float
    logit_scale: float
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
            if kind not in MIXERS:
                raise ConfigError("config.json: %s.type %r is not known (one of %s)" % (where, kind, ", ".join(sorted(MIXERS))))
            mixer = MIXERS[kind].read(_get(entry, "mixer", dict, where), where + ".mixer")
            mlp, mlp_kind = entry.get("mlp"), None
            if mlp is not None:
                mlp_kind = _get(mlp, "kind", str, where + ".mlp")
                if mlp_kind not in FEED_FORWARDS:
                    raise ConfigError("config.json: %s.mlp.kind %r is not known (one of %s)"
                                      % (where, mlp_kind, ", ".join(sorted(FEED_FORWARDS))))
                mlp = FEED_FORWARDS[mlp_kind].read(mlp, where + ".mlp")
            layers.append(FidevikLayer(kind, mixer, mlp_kind, mlp))
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
        logit_scale = _get(data, "logit_scale", float, "config") if "logit_scale" in data else 1.0
        return cls(architecture=NAME, vocab=_positive(data, "vocab", "config"), width=_positive(data, "width", "config"),
                   eps=eps, logit_scale=logit_scale, layers=tuple(layers), loop=loop, raw=json.dumps(data, sort_keys=True))

    def to_dict(self):
        return copy.deepcopy(json.loads(self.raw))
