"""The Dufinex decoder as a ModelSpec: a scaled token embedding; layers in the order the
configuration lists them, each a mixer and, where the layer has one, a feed-forward, both reading
the residual stream as it is, with a norm only on what they return; the mixers are softmax
attention with a sink per head and a gate per head (a layer may read an earlier layer's keys and
values instead of making its own) or the gated delta rule with a decay per key channel; the
feed-forwards are a clamped gated unit with biases or a choice among many small ones. The model's
last norm reads the stream and the head is the embedding table without its scale. Every size and
constant is the configuration's."""

from ..config.dufinex_config import NAME, DufinexConfig
from ..config.registry import register_architecture
from ..parts.base import PartSpec
from .spec import LayerSpec, ModelSpec, RunStep, Slot

GLU_SLOPE = 1.702       # the sigmoid's slope in the feed-forwards' activation, fixed by the design
UNIT_EPS = 1e-6         # inside the root of the delta rule's unit norms, fixed by the design


def _mixer(kind, m, width, eps):
    if kind == "attention":
        return PartSpec.of("mixer", "sink_attention", hidden_size=width, heads=m.heads, kv_heads=m.kv_heads, dim=m.dim,
                           vdim=m.vdim, scale=m.scale, eps=eps, own_keys=m.kv_from is None)
    return PartSpec.of("mixer", "channel_delta", hidden_size=width, heads=m.heads, kv_heads=m.kv_heads, dim=m.dim,
                       vdim=m.vdim, conv=m.conv, eps=eps, unit_eps=UNIT_EPS)


def _feed_forward(kind, f, width):
    if kind == "dense":
        return PartSpec.of("feed_forward", "clamped_glu", hidden_size=width, intermediate_size=f.ff, limit=f.limit,
                           slope=GLU_SLOPE)
    return PartSpec.of("feed_forward", "gated_experts", hidden_size=width, experts=f.experts, top=f.top, expert_ff=f.ff,
                       limit=f.limit, slope=GLU_SLOPE)


def dufinex_spec(config):
    width = config.width
    norm = PartSpec.of("norm", "rms", size=width, eps=config.eps, leaf="")
    reader = PartSpec.of("norm", "none", size=width)
    layers, order = [], []
    for i, layer in enumerate(config.layers):
        slots = [Slot("mixer", _mixer(layer.type, layer.mixer, width, config.eps), "mix"),
                 Slot("mixer_norm", reader, "in1"), Slot("mixer_out_norm", norm, "norm1")]
        if layer.mlp is not None:
            slots += [Slot("feed_forward", _feed_forward(layer.mlp_kind, layer.mlp, width), "mlp"),
                      Slot("feed_forward_norm", reader, "in2"), Slot("feed_forward_out_norm", norm, "norm2")]
        layers.append(LayerSpec(prefix="l%d" % i, slots=tuple(slots), block=PartSpec.of("block", "sandwich")))
        order.append(RunStep(i, reads_cache_of=getattr(layer.mixer, "kv_from", None)))
    return ModelSpec(
        hidden_size=width, vocab_size=config.vocab,
        embedding=PartSpec.of("embedding", "token", vocab_size=config.vocab, hidden_size=width, leaf="",
                              scale=config.embedding_scale),
        embedding_prefix="embed",
        position=PartSpec.of("position", "none"),
        layers=tuple(layers), order=tuple(order),
        final_norm=norm, final_norm_prefix="final.norm",
        head=PartSpec.of("head", "linear", hidden_size=width, vocab_size=config.vocab, weight_name="embed"))


register_architecture(NAME, DufinexConfig, dufinex_spec)
