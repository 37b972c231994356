"""Small Zotunex configurations of the tests' own, their random weights, and the runner that serves them.
The sizes differ between the cases in everything that can differ: head counts of 1 and more, grouped and
ungrouped key/value heads, heads that are turned wholly, partly and not at all, with and without stretched
positions, latents smaller and larger than a head, rotated parts of 2 elements and more, value heads smaller and
larger than query heads, either kind of layer first and last, dense and routed feed-forwards and layers without
one, one expert a token and several, with and without a shared expert, widths that are multiples of nothing."""
import random

import torch

from transformers_neuronx_amd.config import EngineConfig
from transformers_neuronx_amd.engine.factory import build_runner
from transformers_neuronx_amd.engine.model import model_param_decls
from transformers_neuronx_amd.weights.loader import TensorDict
from transformers_neuronx_amd.weights.random_init import random_tensors
from transformers_neuronx_amd.zotunex import ZotunexConfig, zotunex_spec


def attention(heads, kv_heads, dim, scale, rot_dims=None, base=10000.0, factor=None):
    m = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=dim, scale=scale)
    if rot_dims is not None:
        m["rot"] = dict(base=base, dims=rot_dims)
        if factor:
            m["rot"]["scaling"] = dict(factor=factor)
    return "attention", m


def latent(heads, dim, rot_dim, vdim, kv_rank, scale, base=10000.0, factor=None):
    m = dict(heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, kv_rank=kv_rank, scale=scale,
             rot=dict(base=base, dims=rot_dim))
    if factor:
        m["rot"]["scaling"] = dict(factor=factor)
    return "latent_attention", m


def dense(ff):
    return dict(kind="dense", ff=ff)


def moe(experts, top, ff, limit, scale, shared=None):
    d = dict(kind="moe", router=dict(experts=experts, top=top, scale=scale), expert=dict(ff=ff, limit=limit))
    if shared:
        d["shared"] = dict(ff=shared[0], limit=shared[1])
    return d


def layer(mixer, mlp):
    return dict(type=mixer[0], mixer=mixer[1], mlp=mlp)


CASES = {
    # attention first, latent attention last; grouped heads; a layer without a feed-forward
    "a": dict(architecture="Zotunex", vocab=211, width=96, norm=dict(eps=1e-4), embedding=dict(scale=3.0),
              layers=[layer(attention(4, 2, 16, 0.3, 8, 1000.0, 2.0), moe(5, 2, 40, 1.5, 1.25, (24, 0.8))),
                      layer(latent(3, 16, 8, 24, 32, 0.2, 500.0), dense(72)),
                      layer(attention(3, 3, 32, 0.15, 32, 77.0), None),
                      layer(attention(8, 1, 16, 0.4), moe(7, 3, 24, 7.0, 0.5)),
                      layer(latent(2, 8, 2, 8, 16, 0.35, 10.0, 8.0), moe(3, 1, 56, 0.6, 2.0, (8, 5.0)))]),
    # latent attention at both ends; one head; sizes that are multiples of nothing
    "b": dict(architecture="Zotunex", vocab=77, width=50, norm=dict(eps=1e-6),
              layers=[layer(latent(1, 10, 6, 14, 12, 0.25, 123.0), moe(4, 4, 16, 2.0, 1.0)),
                      layer(attention(3, 1, 10, 0.2, 6, 123.0, 3.0), dense(30)),
                      layer(attention(2, 2, 20, 0.1, 20, 9.0), moe(9, 2, 26, 1.0, 3.0, (34, 1.0))),
                      layer(latent(5, 6, 4, 6, 40, 0.4, 300.0, 2.5), None)]),
    # sizes the matrix-unit kernels take: multiples of 16, latents of 64 and 128, pages of keys in 64s
    "c": dict(architecture="Zotunex", vocab=320, width=128, norm=dict(eps=1e-5), embedding=dict(scale=8.0),
              layers=[layer(latent(4, 32, 16, 32, 64, 0.17, 20000.0), dense(256)),
                      layer(attention(4, 2, 64, 0.12, 16, 20000.0, 4.0), moe(8, 2, 64, 1.0, 1.5, (128, 1.0))),
                      layer(latent(16, 16, 8, 48, 128, 0.14, 50000.0, 2.0), moe(16, 4, 32, 3.0, 0.75)),
                      layer(attention(8, 1, 32, 0.1, 32, 500.0), dense(128)),
                      layer(attention(2, 2, 128, 0.09, 64, 1e6), moe(4, 1, 128, 0.5, 2.5))]),
    # one layer of each kind, values the other cases make equal or 1: a scale of 1, a factor of 1, one expert of one
    "d": dict(architecture="Zotunex", vocab=130, width=64, norm=dict(eps=1e-3), embedding=dict(scale=1.0),
              layers=[layer(attention(1, 1, 16, 1.0, 2, 10.0, 1.0), moe(1, 1, 48, 100.0, 1.0)),
                      layer(latent(2, 16, 16, 16, 16, 1.0, 10.0, 1.0), dense(8))]),
}


def config(name) -> ZotunexConfig:
    return ZotunexConfig.from_dict(dict(CASES[name], init_std=0.35))


def weights(cfg, seed, storage=torch.float32):
    """Random tensors by checkpoint name (matrices in `storage`), made lively: wide enough that no part drowns,
    norms' numbers away from 1, numbers on the scores that differ between heads, sinks that weigh about as much as
    a key, corrections that change which experts are chosen, clamps that are met."""
    w = random_tensors(model_param_decls(zotunex_spec(cfg)), cfg.init_std, seed, storage)
    g = torch.Generator().manual_seed(seed + 1000)
    for k in list(w):
        last = k.rsplit(".", 1)[-1]
        if last in ("q", "k", "o", "dkv", "uk", "uv", "gate", "up", "down", "head"):
            w[k] = (w[k].float() * (1.5 / w[k].shape[1] ** 0.5 / cfg.init_std)).to(w[k].dtype)
        elif last in ("g", "router"):
            w[k] = (w[k].float() * (4.0 / w[k].shape[1] ** 0.5 / cfg.init_std)).to(w[k].dtype)
        elif last in ("norm1", "norm2") or k == "final.norm":
            w[k] = torch.rand((), generator=g) * 1.5 + 0.5
        elif last == "temp":
            w[k] = torch.rand(w[k].shape, generator=g) * 1.5 + 0.5
        elif last == "sink":
            w[k] = torch.randn(w[k].shape, generator=g) * 1.5
        elif last == "correction":
            w[k] = torch.randn(w[k].shape, generator=g) * 0.3
    return w


def runner(cfg, w, dtype="float32", kernels="reference", device="cpu", page_size=16, max_tokens=256, max_seqs=4,
           use_graphs=True):
    ecfg = EngineConfig(dtype=dtype, page_size=page_size, max_tokens=max_tokens, max_num_seqs=max_seqs, device=device,
                        kernels=kernels, use_graphs=use_graphs)
    return build_runner(cfg, TensorDict({k: v.clone() for k, v in w.items()}), ecfg)


def requests(cfg, lengths, seed):
    g = torch.Generator().manual_seed(seed)
    return {f"r{i}": torch.randint(0, cfg.vocab, (n,), generator=g).tolist() for i, n in enumerate(lengths)}


def drawn(seed: int) -> ZotunexConfig:
    """A configuration drawn from a seed: any sizes, any order of the two kinds of layers, any feed-forward or
    none."""
    rnd = random.Random(seed)
    width = rnd.choice([24, 36, 64, 100, 128, 256])
    n_layers = rnd.randint(1, 5)
    layers = []
    for i in range(n_layers):
        factor = rnd.choice([None, None, 2.0, 4.0, 16.0])
        base = rnd.choice([10.0, 500.0, 10000.0, 1e6])
        if rnd.random() < 0.5:
            groups = rnd.choice([1, 2, 3])
            dim = rnd.choice([4, 8, 10, 16, 32, 64, 96])
            rot = rnd.choice([None] + [d for d in (2, 4, 8, 10, 16, 32, 64) if d <= dim])
            mixer = attention(groups * rnd.choice([1, 2, 4, 6]), groups, dim, rnd.uniform(0.05, 0.4), rot, base, factor)
        else:
            mixer = latent(rnd.choice([1, 2, 3, 6, 16, 20]), rnd.choice([4, 8, 10, 16, 64]), rnd.choice([2, 4, 8, 16, 64]),
                           rnd.choice([4, 6, 16, 24, 48, 64]), rnd.choice([8, 12, 16, 48, 64, 128]), rnd.uniform(0.05, 0.4),
                           base, factor)
        kind = rnd.random()
        if kind < 0.15 and n_layers > 1:
            mlp = None
        elif kind < 0.5:
            mlp = dense(rnd.choice([8, 20, 64, 200]))
        else:
            experts = rnd.choice([1, 2, 5, 12, 33, 70])
            shared = rnd.choice([None, None, (16, 0.7), (40, 4.0)])
            mlp = moe(experts, rnd.randint(1, min(experts, 4)), rnd.choice([8, 20, 64, 72]), rnd.choice([0.5, 1.0, 7.0]),
                      rnd.choice([0.5, 1.0, 2.5]), shared)
        layers.append(layer(mixer, mlp))
    raw = dict(architecture="Zotunex", vocab=rnd.choice([50, 97, 256, 300]), width=width,
               norm=dict(eps=rnd.choice([1e-6, 1e-5, 1e-3])), layers=layers, init_std=0.35)
    if rnd.random() < 0.8:
        raw["embedding"] = dict(scale=rnd.choice([0.25, 1.0, 4.0, 11.0]))
    return ZotunexConfig.from_dict(raw)
