"""Tadolix on the host: the plain implementation pinned by what its mechanisms must do, the configuration's
reader, and the engine (registry, loader, cache and state manager, step function, scheduler, entry point) on the
torch rendition of the kernels against the plain implementation, for configurations of the tests' own."""
import json
import math
import os

import pytest
import torch

import plain_tadolix as P
import tadolix_cases as tc
import schedules
from transformers_neuronx_amd.config import EngineConfig, read_config
from transformers_neuronx_amd.config.model_config import ConfigError
from transformers_neuronx_amd.engine import StepEntry
from transformers_neuronx_amd.engine.engine import LLMEngine
from transformers_neuronx_amd.sampling import SamplingParams
from transformers_neuronx_amd.tadolix import TadolixConfig, tadolix_spec
from transformers_neuronx_amd.weights import WeightsError, write_random_model

F64 = torch.float64
# float32 against the plain implementation's float64, as a share of the logits' range
TOL = 4e-5


# ---------------------------------------------------------------- the plain implementation, pinned

def test_plain_buckets_of_distances():
    # below half the rows a distance is its own row; then logarithmic steps that reach the last row at `far`
    assert [P.bucket(n, 16, 240) for n in range(8)] == list(range(8))
    assert P.bucket(8, 16, 240) == 8 and P.bucket(239, 16, 240) == 15 and P.bucket(240, 16, 240) == 15
    assert P.bucket(10 ** 6, 16, 240) == 15
    rows = [P.bucket(n, 16, 240) for n in range(300)]
    assert rows == sorted(rows) and set(rows) == set(range(16))
    # the first distance of row 8 + k is the first n with 8 * 30^(k / 8) <= n
    for k in range(1, 8):
        first = rows.index(8 + k)
        assert 8 * 30 ** (k / 8) <= first < 8 * 30 ** (k / 8) + 1
    assert [P.bucket(n, 2, 5) for n in range(7)] == [0, 1, 1, 1, 1, 1, 1]
    assert [P.bucket(n, 7, 33) for n in (0, 2, 3, 32, 33)] == [0, 2, 3, 6, 6]
    # the engine's table by distance is these rows of the tensor, head by head
    from transformers_neuronx_amd.parts.mixer import bias_by_distance
    table = torch.randn(9, 3)
    by = bias_by_distance(table, 70)
    assert by.shape == (3, 71)
    for n in (0, 3, 4, 5, 17, 40, 69, 70):
        assert torch.equal(by[:, n], table[P.bucket(n, 9, 70)])


def test_plain_convolution_and_recurrences_by_hand():
    h = torch.tensor([[1.0, 10.0], [2.0, 20.0], [4.0, 40.0]], dtype=F64)
    w = torch.tensor([[0.5, 2.0, 3.0], [0.0, 0.0, 1.0]], dtype=F64)     # the last column is the current token's
    got = P.causal_conv(h, w)
    assert torch.allclose(got[:, 0], torch.tensor([3.0, 2.0 + 6.0, 0.5 + 4.0 + 12.0], dtype=F64))
    assert torch.equal(got[:, 1], h[:, 1])
    # the minimal recurrence with one channel, in plain numbers
    one = lambda v: torch.tensor([[v]], dtype=F64)
    w = {"p.z": one(1.0), "p.z.b": torch.tensor([0.5], dtype=F64), "p.x": one(-1.0), "p.x.b": torch.tensor([1.0], dtype=F64),
         "p.g": one(2.0), "p.o": one(3.0)}
    x = torch.tensor([[0.5], [3.0]], dtype=F64)
    s, want = 0.0, []
    for v in (0.5, 3.0):
        z = 1 / (1 + math.exp(-(v + 0.5)))
        u = 1.0 - v
        c = u + 0.5 if u >= 0 else 1 / (1 + math.exp(-u))
        s = (1 - z) * s + z * c
        g = 2 * v
        want.append(3.0 * s * g / (1 + math.exp(-g)))
    assert torch.allclose(P.min_gru(w, "p.", x)[:, 0], torch.tensor(want, dtype=F64), atol=1e-12)
    # the gated linear recurrence with one channel and one tap; the first token is no special case
    m = dict(width=1, blocks=1, conv=1)
    w = {"p.y": one(1.0), "p.y.b": torch.zeros(1, dtype=F64), "p.x": one(2.0), "p.x.b": torch.tensor([0.25], dtype=F64),
         "p.conv": one(0.5), "p.conv.b": torch.tensor([0.1], dtype=F64), "p.ra": one(1.5).view(1, 1, 1),
         "p.ra.b": torch.tensor([[0.2]], dtype=F64), "p.ri": one(-1.0).view(1, 1, 1), "p.ri.b": torch.tensor([[0.3]], dtype=F64),
         "p.lam": torch.tensor([0.7], dtype=F64), "p.o": one(1.0)}
    s, want = 0.0, []
    for v in (0.5, 3.0):
        u = 0.5 * (2 * v + 0.25) + 0.1
        r, i = 1 / (1 + math.exp(-(1.5 * u + 0.2))), 1 / (1 + math.exp(-(-u + 0.3)))
        a = math.exp(-8 * r * math.log(1 + math.exp(0.7)))
        s = a * s + math.sqrt(1 - a * a) * i * u
        y = 0.5 * v * (1 + math.tanh(math.sqrt(2 / math.pi) * (v + 0.044715 * v ** 3)))
        want.append(s * y)
    assert torch.allclose(P.rglru(m, w, "p.", x)[:, 0], torch.tensor(want, dtype=F64), atol=1e-12)


def test_plain_chunks_cap_and_gate():
    cfg = tc.config("a")
    raw, w = cfg.to_dict(), P.widen(tc.weights(cfg, 0))
    m = raw["layers"][0]["mixer"]["left"]
    size, T = m["mask"]["size"], 50
    h = torch.randn(T, cfg.width, dtype=F64)
    full = P.chunk_attention(m, w, "l0.mix.left.", h, cfg.eps)
    # the last query (position 49, chunk 40..59) sees position 40 and not 39
    out_of, inside = h.clone(), h.clone()
    out_of[size * 2 - 1] += 1.0
    inside[size * 2] += 1.0
    assert torch.equal(P.chunk_attention(m, w, "l0.mix.left.", out_of, cfg.eps)[-1], full[-1])
    assert not torch.allclose(P.chunk_attention(m, w, "l0.mix.left.", inside, cfg.eps)[-1], full[-1])
    # a chunk's first token sees itself alone: its value through the gate and the output matrix
    per = m["heads"] // m["kv_heads"]
    val = (h[size] @ w["l0.mix.left.v"].T).view(m["kv_heads"], m["vdim"]).repeat_interleave(per, dim=0).reshape(-1)
    assert torch.allclose(full[size], (val * torch.sigmoid(h[size] @ w["l0.mix.left.g"].T)) @ w["l0.mix.left.o"].T)
    # queries and keys are normed head by head: scaling one head's rows changes nothing (eps aside)
    w2 = dict(w)
    w2["l0.mix.left.q"] = w["l0.mix.left.q"].clone()
    w2["l0.mix.left.q"][:m["dim"]] *= 7.0
    assert torch.allclose(P.chunk_attention(m, w2, "l0.mix.left.", h, cfg.eps), full, atol=1e-4)
    # a tiny cap flattens the scores: what is left is the bias by distance
    flat = P.chunk_attention(dict(m, softcap=1e-9), w, "l0.mix.left.", h, cfg.eps)
    w3 = dict(w, **{"l0.mix.left.q": torch.zeros_like(w["l0.mix.left.q"])})
    assert torch.allclose(flat, P.chunk_attention(m, w3, "l0.mix.left.", h, cfg.eps), atol=1e-6)


def test_plain_copies_of_the_stream():
    # an identity mix, ones into every copy and a read of one copy is the plain residual sum
    y = torch.randn(4, 6, dtype=F64)
    x = torch.randn(4, 6, dtype=F64)
    copies = P.hyper([x.clone(), x.clone()], y, torch.eye(2, dtype=F64), torch.ones(2, dtype=F64))
    assert torch.equal(copies[0], x + y) and torch.equal(copies[1], x + y)
    # every new copy is made from the old ones: [from, to]
    mix = torch.tensor([[0.0, 1.0], [2.0, 0.0]], dtype=F64)
    a, b = torch.randn(3, dtype=F64), torch.randn(3, dtype=F64)
    got = P.hyper([a, b], torch.zeros(3, dtype=F64), mix, torch.zeros(2, dtype=F64))
    assert torch.equal(got[0], 2.0 * b) and torch.equal(got[1], a)
    assert P.run_order(dict(layers=[0] * 5, loop=dict(start=1, stop=3, times=3))) == [0, 1, 2, 1, 2, 1, 2, 3, 4]
    assert P.run_order(dict(layers=[0] * 3)) == [0, 1, 2]
    s = P.sinusoid(3, 6, 100.0)
    assert torch.allclose(s[0], torch.tensor([0.0, 1.0] * 3, dtype=F64))
    assert abs(float(s[2, 2]) - math.sin(2 * 100.0 ** (-2 / 6))) < 1e-12 and abs(float(s[1, 1]) - math.cos(1.0)) < 1e-12


# ---------------------------------------------------------------- configuration and weights

def test_the_configuration_is_read_from_nested_keys_and_names_what_is_wrong(tmp_path):
    cfg = tc.config("a")
    assert cfg.run_order() == [0, 1, 2, 1, 2, 3] and cfg.taps == 3 and cfg.streams == 3
    assert tc.config("b").streams is None and tc.config("b").taps == 0 and tc.config("b").run_order() == [0, 1, 2, 3]
    folder = write_random_model(cfg, str(tmp_path / "m"), 0, dtype="float32")
    arch, read = read_config(folder)
    assert arch.name == "Tadolix" and read.layers == cfg.layers and read.to_dict() == dict(cfg.to_dict(), torch_dtype="float32")
    raw = json.load(open(os.path.join(folder, "config.json")))

    def broken(change):
        r = json.loads(json.dumps(raw))
        change(r)
        return r
    for change, text in ((lambda r: r["norm"].pop("eps"), "norm.eps"),
                         (lambda r: r["layers"][1].update(type="other"), r"layers\[1\].type"),
                         (lambda r: r["layers"][0]["mixer"]["left"].pop("heads"), r"layers\[0\].mixer.left.heads"),
                         (lambda r: r["layers"][0]["mixer"]["left"].update(kv_heads=3), r"layers\[0\].mixer.left.heads"),
                         (lambda r: r["layers"][0]["mixer"]["left"].pop("bias_max"), "left.bias_max"),
                         (lambda r: r["layers"][0]["mixer"]["right"].pop("width"), "right.width"),
                         (lambda r: r["layers"][1]["mixer"].update(blocks=5), r"layers\[1\].mixer.width"),
                         (lambda r: r["layers"][1]["mixer"].pop("conv"), r"layers\[1\].mixer.conv"),
                         (lambda r: r["layers"][0]["mlp"].update(kind="moe"), r"layers\[0\].mlp.kind"),
                         (lambda r: r["loop"].update(stop=9), "loop"),
                         (lambda r: r["canon"].update(taps=0), "canon.taps"),
                         (lambda r: r.update(streams=0), "streams"),
                         (lambda r: r.pop("width"), "width")):
        with pytest.raises(ConfigError, match=text):
            TadolixConfig.from_dict(broken(change))


def test_the_loader_names_what_is_missing_and_takes_the_bias_rows_from_the_file(tmp_path):
    from safetensors.torch import load_file, save_file
    from transformers_neuronx_amd.engine.factory import runner_from_folder
    cfg = tc.config("a")
    folder = write_random_model(cfg, str(tmp_path / "m"), 0, dtype="float32")
    tensors = load_file(os.path.join(folder, "model.safetensors"))
    assert tensors["l0.mix.left.rel"].shape == (8, 4) and tensors["l0.mix.left.g"].shape == (96, 96)
    assert tensors["l0.mix.left.o"].shape == (96, 96) and tensors["l0.mix.right.z.b"].shape == (40,)
    assert tensors["l1.mix.ra"].shape == (4, 16, 16) and tensors["l1.mix.conv"].shape == (64, 4)
    assert "l1.norm2" not in tensors and "l1.hc2.in" not in tensors and tensors["l1.hc1.mix"].shape == (3, 3)
    assert tensors["l0.canon1"].shape == (96, 3) and "head" in tensors and "final.norm" in tensors
    ecfg = EngineConfig(dtype="float32", kernels="reference", device="cpu", max_tokens=64)
    # a configuration that does not say how many rows the bias table has: the tensor does
    raw = json.load(open(os.path.join(folder, "config.json")))
    for l in raw["layers"]:
        if l["type"] == "parallel":
            l["mixer"]["left"].pop("bias_rows")
    json.dump(raw, open(os.path.join(folder, "config.json"), "w"))
    toks = list(range(30))
    a = runner_from_folder(folder, ecfg).step([StepEntry("r", toks, [29])])
    want = P.forward(raw, P.widen(tensors), toks)[-1]
    assert float((a[0].double() - want).abs().max() / want.abs().max()) < TOL
    bad = dict(tensors)
    del bad["l1.mix.ra.b"]
    bad["l0.mix.surplus"] = torch.zeros(2)
    save_file(bad, os.path.join(folder, "model.safetensors"))
    with pytest.raises(WeightsError) as e:
        runner_from_folder(folder, ecfg)
    assert "l1.mix.ra.b" in str(e.value) and "l0.mix.surplus" in str(e.value)


# ---------------------------------------------------------------- the engine on the host

def _expected(cfg, w, requests):
    raw, wide = cfg.to_dict(), P.widen(w)
    return {rid: P.forward(raw, wide, toks) for rid, toks in requests.items()}


def step_through(runner, expected, made, tol, few_over=0.0):
    steps, place = made
    over, seen = [], 0
    for rec in steps:
        logits = runner.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in rec["entries"]])
        for row in range(0 if logits is None else logits.shape[0]):
            rid, pos = place[(rec["step"], row)]
            want = expected[rid][pos]
            err = float((logits[row].double().cpu() - want).abs().max() / expected[rid].abs().max())
            seen += 1
            if not err < tol:
                over.append((rec["step"], rid, pos, err))
            assert few_over or err < tol, (rec["step"], rid, pos, err)
        for rid in rec["end"]:
            runner.finish(rid)
        runner.cache.check()
    assert len(over) <= few_over * seen, over[:5]
    assert not runner.cache.requests


@pytest.mark.parametrize("name", sorted(tc.CASES))
def test_schedules_on_the_host(name):
    cfg = tc.config(name)
    w = tc.weights(cfg, 3)
    runner = tc.runner(cfg, w, max_tokens=208)
    requests = tc.requests(cfg, [70, 33, 5, 100, 1], 1)
    expected = _expected(cfg, w, requests)
    for made in (schedules.whole(requests), schedules.head_then_singles(requests, tail=12), schedules.portions(requests),
                 schedules.portions(requests, sizes=(2, 2, 3, 2, 16, 2, 15, 17, 2)),
                 schedules.mixed(requests, max_tokens=208, page=16, seed=5, tail=8, max_live=3),
                 schedules.only_last(schedules.mixed(requests, max_tokens=208, page=16, seed=6, tail=20, max_live=4))):
        step_through(runner, expected, made, TOL)


def test_the_stream_after_every_run_of_a_layer():
    """What a debug context taps after each call of the run order is the sum of the copies."""
    from transformers_neuronx_amd import debug
    cfg = tc.config("a")
    w = tc.weights(cfg, 8)
    toks = tc.requests(cfg, [27], 4)["r0"]
    after = []
    P.forward(cfg.to_dict(), P.widen(w), toks, after)
    runner = tc.runner(cfg, w)
    with debug.debug_context() as taps:
        runner.step([StepEntry("r", toks, [0])])
    names = [k for k in taps if k.startswith("call")]
    assert len(names) == len(after) == 6
    for name, want in zip(names, after):
        assert float((taps[name].double() - want).abs().max() / want.abs().max()) < 1e-5


def test_a_slot_that_is_used_again_starts_afresh():
    """The state a request leaves in its slot (recurrences, convolution inputs) is not the next one's."""
    cfg = tc.config("c")
    w = tc.weights(cfg, 4)
    runner = tc.runner(cfg, w, max_tokens=64, max_seqs=1)
    requests = tc.requests(cfg, [37, 20, 3, 45], 2)
    expected = _expected(cfg, w, requests)
    for rid, toks in requests.items():
        assert runner.cache.slots.num_free == 1
        got = runner.step([StepEntry(rid, toks[:2], [0, 1])])
        got = torch.cat([got, runner.step([StepEntry(rid, toks[2:], list(range(len(toks) - 2)))])])
        assert float((got.double() - expected[rid]).abs().max() / expected[rid].abs().max()) < TOL
        runner.finish(rid)


def test_long_decoding_across_many_chunks():
    cfg = tc.config("b")
    w = tc.weights(cfg, 5)
    runner = tc.runner(cfg, w, max_tokens=160, max_seqs=2)
    toks = tc.requests(cfg, [150], 3)["r0"]
    expected = _expected(cfg, w, {"r0": toks})["r0"]
    got = [runner.step([StepEntry("r0", toks[:21], list(range(21)))])]
    for t in toks[21:]:
        got.append(runner.step([StepEntry("r0", [t], [0])]))
    got = torch.cat(got)
    assert float((got.double() - expected).abs().max() / expected.abs().max()) < TOL


def _greedy(cfg, w, prompt, new):
    raw, wide = cfg.to_dict(), P.widen(w)
    toks = list(prompt)
    for _ in range(new):
        toks.append(int(P.forward(raw, wide, toks)[-1].argmax()))
    return toks[len(prompt):]


@pytest.mark.parametrize("run_ahead", [False, True])
def test_greedy_generation_through_the_scheduler(run_ahead):
    cfg = tc.config("c")
    w = tc.weights(cfg, 6)
    ecfg = EngineConfig(dtype="float32", kernels="reference", device="cpu", page_size=16, max_tokens=96, max_num_seqs=3,
                        max_num_batched_tokens=24, chunk_size=9, run_ahead=run_ahead)
    from transformers_neuronx_amd.engine.factory import build_runner
    from transformers_neuronx_amd.weights.loader import TensorDict
    engine = LLMEngine(build_runner(cfg, TensorDict(w), ecfg), ecfg)
    prompts = list(tc.requests(cfg, [30, 3, 17, 1, 22], 7).values())
    out = engine.generate(prompts, SamplingParams(temperature=0.0, max_new_tokens=12, ignore_eos=True))
    for prompt, tokens in zip(prompts, out):
        assert tokens == _greedy(cfg, w, prompt, 12)
    engine.runner.cache.check()
    assert not engine.runner.cache.requests


def test_generation_through_the_entry_point_on_the_host(tmp_path):
    from safetensors.torch import load_file
    from transformers_neuronx_amd import NeuronAutoModelForCausalLM
    from transformers_neuronx_amd.tadolix.model import TadolixForSampling
    cfg = tc.config("a")
    folder = write_random_model(cfg, str(tmp_path / "m"), 11, dtype="float32")
    w = load_file(os.path.join(folder, "model.safetensors"))
    model = NeuronAutoModelForCausalLM.from_pretrained(folder, batch_size=2, amp="f32", n_positions=64, page_size=16,
                                                       kernels="reference", device="cpu")
    assert type(model) is TadolixForSampling
    model.to_neuron()
    ids = torch.tensor([[5, 200, 17, 3], [9, 9, 100, 42]])
    out = model.sample(ids, sequence_length=14, top_k=1)
    for row in range(2):
        assert out[row, 4:].tolist() == _greedy(cfg, w, ids[row].tolist(), 10)


@pytest.mark.parametrize("seed", range(10))
def test_configurations_drawn_from_a_seed_on_the_host(seed):
    cfg = tc.drawn(seed)
    w = tc.weights(cfg, seed)
    runner = tc.runner(cfg, w, max_tokens=176)
    requests = tc.requests(cfg, [70, 33, 5, 1], seed)
    step_through(runner, _expected(cfg, w, requests), schedules.mixed(requests, max_tokens=176, page=16, seed=5, tail=8, max_live=3), TOL)
