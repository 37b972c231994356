"""Zotunex as a `ModelSpec`: which parts, with which sizes, under which tensor names.

Tensor names: `embed`, `final.norm`, `head`; layer i's start with `l<i>.`: the norms `norm1` and `norm2` (one number
each), the mixer's `mix.*` (attention: `q`, `k`, `q.norm`, `k.norm`, `temp`, `g`, `o`; latent attention: `q`, `dkv`,
`dkv.norm`, `uk`, `uv`, `sink`, `g`, `o`), the feed-forward's `mlp.*` (dense: `up`, `down`; experts: `router`,
`correction`, `e<j>.{gate, up, down}`, `shared.{gate, up, down}`). Matrix names carry no suffix.
"""
from .config import ZotunexConfig
from ..config.registry import register_architecture
from ..parts.spec import LayerSpec, ModelSpec, PartSpec


def _rotary(rot, interleaved: bool) -> PartSpec:
    return PartSpec("rotary", dict(base=rot["base"], dims=rot["dims"], interleaved=interleaved,
                                   scaling=rot.get("scaling")))


def zotunex_spec(cfg: ZotunexConfig) -> ModelSpec:
    d = cfg.width
    norm = PartSpec("rms_norm", dict(width=d, eps=cfg.eps, weight_suffix="", scalar=True))
    no_norm = PartSpec("layer_norm", dict(width=d, eps=cfg.eps, affine=False))       # before a feed-forward that is not there
    layers, unread = [], []
    for i, layer in enumerate(cfg.layers):
        m = layer["mixer"]
        if layer["type"] == "attention":
            mixer = PartSpec("attention", dict(
                width=d, num_heads=m["heads"], num_kv_heads=m.get("kv_heads", m["heads"]), head_size=m["dim"],
                value_size=m["dim"], names=("q", "k", None, "o"), weight_suffix="", bias=False, scale=m["scale"],
                rotation=_rotary(m["rot"], True) if m.get("rot") is not None else None,
                qk_norm=dict(eps=cfg.eps, suffix=".norm", shared=True), values_from_keys=True, head_scale="temp",
                out_gate="g", out_gate_per_head=True))
        else:
            mixer = PartSpec("latent_attention", dict(
                width=d, num_heads=m["heads"], head_size=m["dim"], rot_size=m["rot_dim"], value_size=m["vdim"],
                kv_rank=m["kv_rank"], q_rank=None, scale=m["scale"], eps=cfg.eps, rotation=_rotary(m["rot"], False),
                names=(None, "q", "dkv", "uk", "uv", "o"), sink="sink", out_gate="g"))
        mlp = layer.get("mlp")
        if mlp is None:
            ffn = PartSpec("none", {})
            unread.append(f"l{i}.norm2")
        elif mlp["kind"] == "dense":
            ffn = PartSpec("dense", dict(width=d, inner=mlp["ff"], activation="relu2", up_name="up", down_name="down",
                                         bias=False, weight_suffix=""))
        else:
            shared = mlp.get("shared")
            ffn = PartSpec("mixture", dict(
                width=d, experts=mlp["router"]["experts"], top=mlp["router"]["top"], inner=mlp["expert"]["ff"],
                shared_inner=shared["ff"] if shared else 0, score="sigmoid", renormalize=False, weight_on="output",
                activation="clamped_swiglu", limit=mlp["expert"]["limit"], shared_limit=shared["limit"] if shared else None,
                router_name="router", correction_name="correction", route_scale=mlp["router"].get("scale", 1.0),
                expert_name="e{}.", shared_name="shared.", names=("gate", "up", "down")))
        layers.append(LayerSpec(prefix=f"l{i}.", block="pre_norm", mixer=mixer, feed_forward=ffn, mixer_norm=norm,
                                feed_forward_norm=norm if mlp is not None else no_norm, mixer_name="mix.", feed_forward_name="mlp.",
                                mixer_norm_name="norm1", feed_forward_norm_name="norm2"))
    embedding = PartSpec("token_table", dict(vocab=cfg.vocab, embed_width=d, width=d, position=PartSpec("none", {}),
                                             table_name="embed", projection_name=None, position_name=None,
                                             scale=cfg.embedding_scale))
    head = PartSpec("vocab_projection", dict(vocab=cfg.vocab, embed_width=d, width=d, norm=norm, weight_name="head",
                                             tied_to=None, projection_name=None, norm_name="final.norm"))
    return ModelSpec(hidden_size=d, vocab_size=cfg.vocab, max_positions=cfg.max_positions, embedding=embedding,
                     layers=tuple(layers), schedule=ModelSpec.sequential(len(layers)), head=head,
                     init_std=cfg.init_std, unread=tuple(unread))


ARCHITECTURE = register_architecture("Zotunex", "zotunex", ZotunexConfig, zotunex_spec,
                                     model_class="transformers_neuronx_amd.zotunex.model:ZotunexForSampling")
