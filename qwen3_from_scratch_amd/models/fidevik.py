"""The Fidevik decoder as a ModelSpec: a token embedding; pre-norm layers in the order the
configuration lists them, each a mixer behind a layer norm with a weight and a bias and, where
the layer has one, a feed-forward behind another; the mixers are softmax attention over grouped
key heads, with queries and keys normalised over their whole projections and turned by the
position in neighbouring pairs, or latent attention without positions, with a sink in the softmax
and a gate per head; the feed-forwards are a gated unit with the tanh form of gelu, or experts
chosen by corrected sigmoid scores within the best groups, with a gated shared expert. A run of
the layers may be passed several times with the same weights, every pass with a cache of its own;
each pass begins with its own vector added to the stream and, from the second on, with the
embedding's output added once more. The model's norm, an untied head and a scale on the logits
end it. Every size and constant is the configuration's."""

from ..config.fidevik_config import NAME, FidevikConfig
from ..config.registry import register_architecture
from ..parts.base import PartSpec
from .kodisun import run_order
from .spec import LayerSpec, ModelSpec, Slot

DENSE_ACTIVATION = "gelu_tanh"      # the dense feed-forward's gate, fixed by the design
EXPERT_ACTIVATION = "silu"          # the experts' and the shared expert's


def _mixer(kind, m, width, eps):
    if kind == "attention":
        return PartSpec.of("mixer", "softcap_attention", hidden_size=width, heads=m.heads, kv_heads=m.kv_heads, dim=m.dim,
                           vdim=m.vdim, scale=m.scale, eps=eps, rot_dims=m.rot.dims if m.rot else 0,
                           rot_base=m.rot.base if m.rot else 1.0, biases=False, gated=False)
    return PartSpec.of("mixer", "latent_attention", hidden_size=width, heads=m.heads, dim=m.dim, rot_dim=0, vdim=m.vdim,
                       q_rank=m.q_rank, kv_rank=m.kv_rank, scale=m.scale, eps=eps, sink=True, gated=True)


def _feed_forward(kind, f, width):
    if kind == "dense":
        return PartSpec.of("feed_forward", "swiglu", hidden_size=width, intermediate_size=f.ff,
                           names=("gate", "up", "down"), activation=DENSE_ACTIVATION)
    return PartSpec.of("feed_forward", "grouped_experts", hidden_size=width, experts=f.experts, top=f.top,
                       expert_ff=f.expert_ff, groups=f.groups, keep=f.keep, shared_ff=f.shared_ff,
                       activation=EXPERT_ACTIVATION)


def fidevik_spec(config):
    width = config.width
    norm = PartSpec.of("norm", "layer_bias", size=width, eps=config.eps, leaf="")
    layers = []
    for i, layer in enumerate(config.layers):
        slots = [Slot("mixer", _mixer(layer.type, layer.mixer, width, config.eps), "mix"), Slot("mixer_norm", norm, "norm1")]
        if layer.mlp is not None:
            slots += [Slot("feed_forward", _feed_forward(layer.mlp_kind, layer.mlp, width), "mlp"),
                      Slot("feed_forward_norm", norm, "norm2")]
        layers.append(LayerSpec(prefix="l%d" % i, slots=tuple(slots), block=PartSpec.of("block", "pre_norm")))
    start, stop, times = config.loop
    looped = stop > start
    return ModelSpec(
        hidden_size=width, vocab_size=config.vocab,
        embedding=PartSpec.of("embedding", "token", vocab_size=config.vocab, hidden_size=width, leaf=""),
        embedding_prefix="embed",
        position=PartSpec.of("position", "none"),
        layers=tuple(layers), order=run_order(len(layers), config.loop),
        final_norm=norm, final_norm_prefix="final.norm",
        head=PartSpec.of("head", "linear", hidden_size=width, vocab_size=config.vocab, weight_name="head",
                         scale=config.logit_scale),
        pass_vectors=PartSpec.of("embedding", "pass_vectors", passes=times, hidden_size=width, leaf="step",
                                 restart=True) if looped else None,
        pass_vectors_prefix="loop",
        # a loop over no layers at all still has its table of vectors in the file; nothing reads it
        ignorable_tensors=() if looped else ("loop.step",))


register_architecture(NAME, FidevikConfig, fidevik_spec)
