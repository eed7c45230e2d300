"""The Kodisun decoder as a ModelSpec: a token embedding; layers of latent attention with a
sliding window, each with a norm before and behind the mixer and before and behind a routed
feed-forward (or no feed-forward); a run of the layers that is passed several times with the
same weights, every pass with a cache of its own and a vector of its own added to the stream
before it; a final norm and an untied linear head. Every size and constant is the
configuration's; layers may differ from one another in all of them."""

from ..config.kodisun_config import NAME, KodisunConfig
from ..config.registry import register_architecture
from ..parts.base import PartSpec
from .spec import LayerSpec, ModelSpec, RunStep, Slot


def run_order(num_layers, loop):
    """The layers before the loop once, the loop's layers `times` times in a row, the rest once."""
    start, stop, times = loop
    if stop <= start:
        return tuple(RunStep(i) for i in range(num_layers))
    order = [RunStep(i) for i in range(start)]
    for number in range(times):
        order += [RunStep(i, enters=number if i == start else None) for i in range(start, stop)]
    return tuple(order + [RunStep(i) for i in range(stop, num_layers)])


def kodisun_spec(config):
    width = config.width
    norm = PartSpec.of("norm", "rms", size=width, eps=config.eps, leaf="")
    layers = []
    for i, layer in enumerate(config.layers):
        m = layer.mixer
        mixer = PartSpec.of("mixer", "latent_attention", hidden_size=width, heads=m.heads, dim=m.dim, rot_dim=m.rot_dim,
                            vdim=m.vdim, q_rank=m.q_rank, kv_rank=m.kv_rank, scale=m.scale, eps=config.eps,
                            window=m.window)
        position = PartSpec.of("position", "rotary_pairs", dims=m.rot.dims, base=m.rot.base, scaling=m.rot.scaling)
        slots = [Slot("mixer", mixer, "mix"), Slot("mixer_norm", norm, "norm1"), Slot("mixer_out_norm", norm, "norm1b")]
        if layer.mlp is not None:
            f = layer.mlp
            slots += [Slot("feed_forward", PartSpec.of("feed_forward", "routed_experts", hidden_size=width,
                                                       experts=f.experts, top=f.top, expert_ff=f.expert_ff,
                                                       shared_ff=f.shared_ff, activation="erf"), "mlp"),
                      Slot("feed_forward_norm", norm, "norm2"), Slot("feed_forward_out_norm", norm, "norm2b")]
        layers.append(LayerSpec(prefix="l%d" % i, slots=tuple(slots), block=PartSpec.of("block", "sandwich"),
                                position=position))
    start, stop, times = config.loop
    looped = stop > start
    return ModelSpec(
        hidden_size=width, vocab_size=config.vocab,
        embedding=PartSpec.of("embedding", "token", vocab_size=config.vocab, hidden_size=width, leaf=""),
        embedding_prefix="embed",
        position=PartSpec.of("position", "none"),
        layers=tuple(layers), order=run_order(len(layers), config.loop),
        final_norm=norm, final_norm_prefix="final.norm",
        head=PartSpec.of("head", "linear", hidden_size=width, vocab_size=config.vocab, weight_name="head"),
        pass_vectors=PartSpec.of("embedding", "pass_vectors", passes=times, hidden_size=width, leaf="step") if looped else None,
        pass_vectors_prefix="loop")


register_architecture(NAME, KodisunConfig, kodisun_spec)
