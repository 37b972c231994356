"""Small Tadolix configurations of the tests' own, their random weights, and the runner that serves them.
The sizes differ between the cases in everything that can differ: 1, 2, 4 copies of the stream and the plain
residual; convolutions of 1 to 4 taps and none; loops over the first layers, the last ones, one layer, once, and
none; pairs and recurrent blocks in any order, with and without a feed-forward; head counts of 1 and more, grouped
and not; value heads smaller and larger than query heads; chunks of 1 token, of less and of more than a page, of
exactly a page, and none; bias tables of 2 to 32 rows with an odd count among them; recurrences of one part and
of several; widths that are multiples of nothing."""
import random

import torch

from transformers_neuronx_amd.config import EngineConfig
from transformers_neuronx_amd.engine.factory import build_runner
from transformers_neuronx_amd.engine.model import model_param_decls
from transformers_neuronx_amd.tadolix import TadolixConfig, tadolix_spec
from transformers_neuronx_amd.weights.loader import TensorDict
from transformers_neuronx_amd.weights.random_init import random_tensors


def pair(heads, kv_heads, dim, vdim, chunk, scale, cap, rows, far, right, left_scale=1.0, right_scale=1.0):
    left = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale, bias_max=far, bias_rows=rows)
    if cap is not None:
        left["softcap"] = cap
    if chunk is not None:
        left["mask"] = dict(size=chunk)
    return "parallel", dict(left=left, right=dict(width=right), left_scale=left_scale, right_scale=right_scale)


def recurrent(width, blocks, conv):
    return "rglru", dict(width=width, blocks=blocks, conv=conv)


def layer(mixer, ff):
    return dict(type=mixer[0], mixer=mixer[1], mlp=dict(kind="dense", ff=ff) if ff else None)


CASES = {
    # three copies, a loop over the middle, pairs and recurrent blocks mixed
    "a": dict(architecture="Tadolix", vocab=211, width=96, norm=dict(eps=1e-4), embedding=dict(scale=3.0),
              canon=dict(taps=3), streams=3, loop=dict(start=1, stop=3, times=2),
              layers=[layer(pair(4, 2, 16, 24, 20, 0.3, 5.0, 8, 40, 40, 1.3, 0.6), 72),
                      layer(recurrent(64, 4, 4), None),
                      layer(pair(3, 3, 32, 16, 7, 0.2, 30.0, 6, 100, 56, 0.7, 1.1), 40),
                      layer(recurrent(48, 1, 2), 24)]),
    # the plain residual (no copies), no convolution, no loop; chunks of one token, of a page, none; no cap
    "b": dict(architecture="Tadolix", vocab=130, width=64, norm=dict(eps=1e-6),
              layers=[layer(pair(1, 1, 16, 16, 1, 0.25, None, 2, 5, 16), 48),
                      layer(pair(2, 1, 16, 32, 16, 0.5, 2.0, 32, 64, 80), None),
                      layer(recurrent(32, 2, 1), 16),
                      layer(pair(4, 4, 8, 12, None, 0.4, 50.0, 7, 33, 8, 2.0, 0.25), 40)]),
    # sizes that are multiples of nothing; one copy; two taps; a loop over the last layers; an odd table
    "c": dict(architecture="Tadolix", vocab=77, width=50, norm=dict(eps=1e-5), embedding=dict(scale=0.5),
              canon=dict(taps=2), streams=1, loop=dict(start=2, stop=4, times=3),
              layers=[layer(recurrent(30, 3, 3), 26),
                      layer(pair(3, 1, 10, 14, 33, 0.2, 8.0, 9, 70, 22), None),
                      layer(pair(2, 2, 20, 6, 5, 0.1, 1.0, 4, 9, 34, 0.3, 3.0), 30),
                      layer(recurrent(26, 2, 4), None)]),
    # sizes the matrix-unit kernels take; four copies; four taps; the loop runs the first layer alone, once more
    "d": dict(architecture="Tadolix", vocab=320, width=128, norm=dict(eps=1e-5), embedding=dict(scale=8.0),
              canon=dict(taps=4), streams=4, loop=dict(start=0, stop=1, times=2),
              layers=[layer(pair(4, 2, 32, 32, 48, 0.17, 20.0, 16, 96, 128), 256),
                      layer(recurrent(128, 4, 4), 128),
                      layer(pair(8, 2, 16, 32, 64, 0.14, 12.0, 16, 128, 64), None),
                      layer(pair(2, 2, 64, 64, 100, 0.1, 40.0, 32, 200, 256), 128)]),
}


def config(name) -> TadolixConfig:
    return TadolixConfig.from_dict(dict(CASES[name], init_std=0.35))


def weights(cfg, seed, storage=torch.float32):
    """Random tensors by checkpoint name (matrices in `storage`), made lively: wide enough that no part drowns,
    gates that open and close, decays all over (0, 1), stream weights that mix."""
    w = random_tensors(model_param_decls(tadolix_spec(cfg)), cfg.init_std, seed, storage)
    g = torch.Generator().manual_seed(seed + 1000)
    for k in list(w):
        last = k.rsplit(".", 1)[-1]
        if last in ("q", "k", "v", "o", "g", "gate", "up", "down", "head", "y", "x", "z"):
            w[k] = (w[k].float() * (1.5 / w[k].shape[1] ** 0.5 / cfg.init_std)).to(w[k].dtype)
        elif last in ("ra", "ri"):
            w[k] = (w[k].float() * (3.0 / w[k].shape[2] ** 0.5 / cfg.init_std)).to(w[k].dtype)
        elif last == "lam":
            w[k] = torch.rand(w[k].shape, generator=g) * 6.0 - 5.0
        elif last == "rel":
            w[k] = torch.randn(w[k].shape, generator=g) * 1.5
        elif last == "mix":
            s = w[k].shape[0]
            w[k] = torch.eye(s) * 0.8 + torch.randn(s, s, generator=g) * 0.15
        elif last == "in":
            w[k] = torch.rand(w[k].shape, generator=g) * 0.8 + 0.2
    return w


def runner(cfg, w, dtype="float32", kernels="reference", device="cpu", page_size=16, max_tokens=256, max_seqs=4,
           use_graphs=True):
    ecfg = EngineConfig(dtype=dtype, page_size=page_size, max_tokens=max_tokens, max_num_seqs=max_seqs, device=device,
                        kernels=kernels, use_graphs=use_graphs)
    return build_runner(cfg, TensorDict({k: v.clone() for k, v in w.items()}), ecfg)


def requests(cfg, lengths, seed):
    g = torch.Generator().manual_seed(seed)
    return {f"r{i}": torch.randint(0, cfg.vocab, (n,), generator=g).tolist() for i, n in enumerate(lengths)}


def drawn(seed: int) -> TadolixConfig:
    """A configuration drawn from a seed: any sizes, any order of the two kinds of layers, with and without a
    feed-forward, copies, taps and loop of any kind, chunks from 1 token to none."""
    rnd = random.Random(seed)
    width = rnd.choice([24, 36, 64, 100, 128, 256])
    n_layers = rnd.randint(1, 5)
    layers = []
    for _ in range(n_layers):
        if rnd.random() < 0.6:
            groups = rnd.choice([1, 2, 3])
            rows = rnd.choice([2, 3, 4, 8, 16, 32])
            mixer = pair(groups * rnd.choice([1, 2, 4]), groups, rnd.choice([4, 8, 10, 16, 32, 64]),
                         rnd.choice([4, 6, 16, 24, 48, 64]), rnd.choice([None, 1, 2, 15, 16, 17, 40, 64]),
                         rnd.choice([0.1, 0.25, 0.5]), rnd.choice([None, 1.0, 10.0, 30.0]), rows,
                         rows // 2 + rnd.choice([1, 5, 30, 200]), rnd.choice([8, 20, 64, 100]),
                         rnd.choice([0.5, 1.0, 1.2]), rnd.choice([0.5, 1.0, 2.0]))
        else:
            blocks = rnd.choice([1, 2, 4])
            mixer = recurrent(blocks * rnd.choice([4, 10, 16, 32]), blocks, rnd.choice([1, 2, 3, 4, 5]))
        layers.append(layer(mixer, rnd.choice([None, 16, 40, 64, 130])))
    raw = dict(architecture="Tadolix", vocab=rnd.choice([50, 128, 300]), width=width, layers=layers,
               norm=dict(eps=rnd.choice([1e-6, 1e-5, 1e-3])), init_std=0.35)
    if rnd.random() < 0.7:
        raw["embedding"] = dict(scale=rnd.choice([0.5, 4.0, 11.0]))
    if rnd.random() < 0.8:
        raw["canon"] = dict(taps=rnd.choice([1, 2, 3, 4, 5]))
    if rnd.random() < 0.8:
        raw["streams"] = rnd.choice([1, 2, 3, 4, 6])
    if rnd.random() < 0.7:
        start = rnd.randint(0, n_layers - 1)
        raw["loop"] = dict(start=start, stop=rnd.randint(start, n_layers), times=rnd.choice([1, 2, 3]))
    return TadolixConfig.from_dict(raw)
