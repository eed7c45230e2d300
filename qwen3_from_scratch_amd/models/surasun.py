"""The Surasun decoder as a ModelSpec: a token embedding into a residual held in several streams
(hyper-connections; or the ordinary single residual), layers in the order the configuration
lists them, each a mixer behind a layer norm and, where the layer has one, a dense gated
feed-forward behind another; the mixers are Mamba-2, Griffin's recurrent unit, or softmax
attention and retention side by side. The model's last norm reads the streams' sum and the head
is the embedding table. Every size and constant is the configuration's."""

from ..config.registry import register_architecture
from ..config.surasun_config import NAME, SurasunConfig
from ..parts.base import PartSpec
from .spec import LayerSpec, ModelSpec, RunStep, Slot


def _mixer(kind, m, width, eps):
    if kind == "mamba2":
        return PartSpec.of("mixer", "mamba2", hidden_size=width, heads=m.heads, vdim=m.vdim, state=m.state,
                           groups=m.groups, conv=m.conv, norm_groups=m.norm_groups, eps=eps)
    if kind == "rglru":
        return PartSpec.of("mixer", "rglru", hidden_size=width, width=m.width, blocks=m.blocks, conv=m.conv)
    left = PartSpec.of("mixer", "softcap_attention", hidden_size=width, heads=m.left.heads, kv_heads=m.left.kv_heads,
                       dim=m.left.dim, vdim=m.left.vdim, scale=m.left.scale, softcap=m.left.softcap, eps=eps,
                       rot_dims=m.left.rot.dims, rot_base=m.left.rot.base)
    right = PartSpec.of("mixer", "retention", hidden_size=width, heads=m.right.heads, dim=m.right.dim,
                        vdim=m.right.vdim, decay=m.right.decay, eps=eps, rot_dims=m.right.rot.dims,
                        rot_base=m.right.rot.base)
    return PartSpec.of("mixer", "parallel", left=left, right=right, left_scale=m.left_scale, right_scale=m.right_scale)


def surasun_spec(config):
    width = config.width
    norm = PartSpec.of("norm", "layer", size=width, eps=config.eps, leaf="")
    block = PartSpec.of("block", "hyper_connections", streams=config.streams, mult=config.residual_mult)
    layers = []
    for i, layer in enumerate(config.layers):
        slots = [Slot("mixer", _mixer(layer.type, layer.mixer, width, config.eps), "mix"), Slot("mixer_norm", norm, "norm1")]
        if layer.ff:
            slots += [Slot("feed_forward", PartSpec.of("feed_forward", "swiglu", hidden_size=width,
                                                       intermediate_size=layer.ff, names=("gate", "up", "down")), "mlp"),
                      Slot("feed_forward_norm", norm, "norm2")]
        layers.append(LayerSpec(prefix="l%d" % i, slots=tuple(slots), block=block))
    return ModelSpec(
        hidden_size=width, vocab_size=config.vocab,
        embedding=PartSpec.of("embedding", "token", vocab_size=config.vocab, hidden_size=width, leaf="",
                              copies=max(config.streams, 1)),
        embedding_prefix="embed",
        position=PartSpec.of("position", "none"),
        layers=tuple(layers), order=tuple(RunStep(i) for i in range(len(layers))),
        final_norm=norm, final_norm_prefix="final.norm",
        head=PartSpec.of("head", "linear", hidden_size=width, vocab_size=config.vocab, weight_name="embed"))


register_architecture(NAME, SurasunConfig, surasun_spec)
