"""Tadolix as a `ModelSpec`: which parts, with which sizes, under which tensor names.

Tensor names: `embed`, `final.norm`, `head`; layer i's start with `l<i>.`: the norms `norm1`, `norm2` (weights
stored around zero), the convolution before the mixer `canon1`, the stream weights `hc1.{in, out, mix}` and
`hc2.{in, out, mix}`, the mixer's `mix.*` (a pair: `left.{q, k, v, g, o, rel}` and `right.{z, x, g, o}`; the
recurrent block: `y`, `x`, `conv`, `ra`, `ri`, `lam`, `o`; a bias being its matrix's name with `.b`), the
feed-forward's `mlp.{gate, up, down}`. Matrix names carry no suffix.
"""
from .config import TadolixConfig
from ..config.registry import register_architecture
from ..parts.spec import LayerCall, LayerSpec, ModelSpec, PartSpec


def tadolix_spec(cfg: TadolixConfig) -> ModelSpec:
    d = cfg.width
    norm = PartSpec("rms_norm", dict(width=d, eps=cfg.eps, weight_suffix="", unit_offset=True))
    no_norm = PartSpec("layer_norm", dict(width=d, eps=cfg.eps, affine=False))
    layers = []
    for i, layer in enumerate(cfg.layers):
        m = layer["mixer"]
        if layer["type"] == "parallel":
            left, right = m["left"], m["right"]
            attention = PartSpec("attention", dict(
                width=d, num_heads=left["heads"], num_kv_heads=left.get("kv_heads", left["heads"]),
                head_size=left["dim"], value_size=left["vdim"], names=("q", "k", "v", "o"), weight_suffix="",
                bias=False, scale=left.get("scale", left["dim"] ** -0.5),
                qk_norm=dict(eps=cfg.eps, per_head=True, weighted=False), softcap=left.get("softcap"),
                distance_bias=dict(name="rel", max_distance=left["bias_max"], rows=left.get("bias_rows")),
                chunk=(left.get("mask") or {}).get("size"), out_gate="g"))
            recurrence = PartSpec("min_gru", dict(width=d, inner=right["width"], names=("z", "x", "g", "o"),
                                                  bias_suffix=".b"))
            mixer = PartSpec("side_by_side", dict(left=attention, right=recurrence, left_name="left.",
                                                  right_name="right.", left_scale=m.get("left_scale", 1.0),
                                                  right_scale=m.get("right_scale", 1.0)))
        else:
            mixer = PartSpec("rglru", dict(width=d, inner=m["width"], blocks=m["blocks"], taps=m["conv"],
                                           names=("y", "x", "conv", "ra", "ri", "lam", "o"), bias_suffix=".b"))
        mlp = layer.get("mlp")
        if mlp is not None:
            ffn = PartSpec("gated", dict(width=d, inner=mlp["ff"], activation="gelu_new",
                                         names=("gate", "up", "down")))
        else:
            ffn = PartSpec("none", {})
        block = PartSpec("hyper", dict(streams=cfg.streams or 0, taps=cfg.taps, conv_name="canon1",
                                       names=("hc1.", "hc2."), parts=("in", "out", "mix")))
        layers.append(LayerSpec(prefix=f"l{i}.", block=block, mixer=mixer, feed_forward=ffn, mixer_norm=norm,
                                feed_forward_norm=norm if mlp is not None else no_norm, mixer_name="mix.",
                                feed_forward_name="mlp.", mixer_norm_name="norm1", feed_forward_norm_name="norm2"))
    embedding = PartSpec("token_table", dict(vocab=cfg.vocab, embed_width=d, width=d,
                                             position=PartSpec("sinusoidal", dict(width=d, base=10000.0)),
                                             table_name="embed", projection_name=None, position_name=None,
                                             scale=cfg.embedding_scale))
    head = PartSpec("vocab_projection", dict(vocab=cfg.vocab, embed_width=d, width=d, norm=norm, weight_name="head",
                                             tied_to=None, projection_name=None, norm_name="final.norm"))
    # every pass through a layer of the loop keeps a cache and a state of its own
    schedule = tuple(LayerCall(i) for i in cfg.run_order())
    return ModelSpec(hidden_size=d, vocab_size=cfg.vocab, max_positions=cfg.max_positions, embedding=embedding,
                     layers=tuple(layers), schedule=schedule, head=head, init_std=cfg.init_std)


ARCHITECTURE = register_architecture("Tadolix", "tadolix", TadolixConfig, tadolix_spec,
                                     model_class="transformers_neuronx_amd.tadolix.model:TadolixForSampling")
