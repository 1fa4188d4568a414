"""Sunatar on the host: the plain implementation pinned by what its mechanisms must do, the configuration's
reader, and the engine (registry, loader, cache and state manager, step function, scheduler, entry point) on the
torch rendition of the kernels against the plain implementation, for configurations of the tests' own."""
import json
import math
import os

import pytest
import torch

import plain_sunatar as P
import sunatar_cases as sc
import schedules
from transformers_neuronx_amd.config import EngineConfig, read_config
from transformers_neuronx_amd.config.model_config import ConfigError
from transformers_neuronx_amd.engine import StepEntry
from transformers_neuronx_amd.engine.engine import LLMEngine
from transformers_neuronx_amd.sampling import SamplingParams
from transformers_neuronx_amd.sunatar import SunatarConfig, sunatar_spec
from transformers_neuronx_amd.weights import WeightsError, write_random_model

F64 = torch.float64
# float32 against the plain implementation's float64, as a share of the logits' range: the memory's result is a
# quotient whose denominator can come close to its floor, which spreads a rounding over a few more bits
TOL = 6e-5


# ---------------------------------------------------------------- the plain implementation, pinned

def test_plain_rotation_by_halves_counts_distances_only():
    g = torch.Generator().manual_seed(0)
    q, k = torch.randn(5, 3, 12, generator=g, dtype=F64), torch.randn(5, 3, 12, generator=g, dtype=F64)
    pos = torch.tensor([0, 3, 4, 9, 20])
    f = P.rotary_frequencies(50.0, 8)
    a = torch.einsum("ihd,jhd->hij", P.rotate_halves(q, pos, f), P.rotate_halves(k, pos, f))
    b = torch.einsum("ihd,jhd->hij", P.rotate_halves(q, pos + 1000, f), P.rotate_halves(k, pos + 1000, f))
    assert torch.allclose(a, b, atol=1e-9)
    # elements beyond `dims` pass, position 0 turns nothing, a pair (i, i + half) keeps its length
    turned = P.rotate_halves(q, pos, f)
    assert torch.equal(turned[..., 8:], q[..., 8:]) and torch.allclose(turned[0], q[0])
    assert torch.allclose(turned[..., 1] ** 2 + turned[..., 5] ** 2, q[..., 1] ** 2 + q[..., 5] ** 2)
    # the first pair turns by the position itself (frequency 1)
    one = P.rotate_halves(torch.tensor([[[1.0, 0.0]]], dtype=F64), torch.tensor([1]), P.rotary_frequencies(7.0, 2))
    assert torch.allclose(one[0, 0], torch.tensor([math.cos(1.0), math.sin(1.0)], dtype=F64))


def test_plain_scaled_frequencies():
    plain = P.rotary_frequencies(5000.0, 24)
    scaled = P.rotary_frequencies(5000.0, 24, dict(factor=8.0, low=1.0, high=4.0, original=100))
    wavelength = 2 * math.pi / plain
    fast, slow = wavelength < 100 / 4.0, wavelength > 100 / 1.0
    assert fast.any() and slow.any() and (~fast & ~slow).any()
    assert torch.equal(scaled[fast], plain[fast]) and torch.allclose(scaled[slow], plain[slow] / 8.0)
    between = ~fast & ~slow
    assert ((scaled[between] > plain[between] / 8.0) & (scaled[between] < plain[between])).all()
    # the blend is linear in turns per `original` tokens: halfway between low and high it is the mean of the two
    turns = 100 * plain[between] / (2 * math.pi)
    share = (turns - 1.0) / 3.0
    assert torch.allclose(scaled[between], (1 - share) * plain[between] / 8.0 + share * plain[between])
    # the engine's own frequencies are these
    from transformers_neuronx_amd.parts.position import RotaryPositions
    for base, dims, scaling in ((5000.0, 24, dict(factor=8.0, low=1.0, high=4.0, original=100)), (77.0, 6, None),
                                (1e6, 64, dict(factor=2.0, low=0.5, high=3.0, original=4096))):
        part = RotaryPositions(base, dims, interleaved=False, scaling=scaling)
        assert torch.allclose(part.frequencies().double(), P.rotary_frequencies(base, dims, scaling), rtol=1e-6, atol=0)


def test_plain_gates_and_memory_by_hand():
    assert abs(float(P.log_sigmoid(torch.tensor(0.0, dtype=F64))) + math.log(2.0)) < 1e-12
    assert abs(float(P.log_sigmoid(torch.tensor(-800.0, dtype=F64))) + 800.0) < 1e-9
    assert abs(float(P.soft_cap(torch.tensor(1e6, dtype=F64), 7.0)) - 7.0) < 1e-9
    assert abs(float(P.silu(torch.tensor(1.0, dtype=F64))) - 1.0 / (1.0 + math.exp(-1.0))) < 1e-12
    # one head, one query/key element, one value element: the recurrence in plain numbers
    m = dict(heads=1, dim=1, vdim=1, gate_cap=100.0)
    w = {k: torch.tensor([[v]], dtype=F64) for k, v in dict(q=1.0, k=1.0, v=2.0, g=0.0, o=1.0, i=1.0, f=-1.0).items()}
    w = {"p." + k: v for k, v in w.items()}
    w.update({"p.i.b": torch.tensor([0.5], dtype=F64), "p.f.b": torch.tensor([0.25], dtype=F64), "p.norm": torch.ones(1, dtype=F64)})
    h = torch.tensor([[1.0], [2.0]], dtype=F64)
    got = P.mlstm(m, w, "p.", h, 0.0)
    peak, mem, norm, want = 0.0, 0.0, 0.0, []
    for x in (1.0, 2.0):
        gi, gf = 100.0 * math.tanh((x + 0.5) / 100.0), -math.log1p(math.exp(-100.0 * math.tanh((0.25 - x) / 100.0)))
        new = max(gf + peak, gi)
        mem = math.exp(gf + peak - new) * mem + math.exp(gi - new) * x * (2 * x)
        norm = math.exp(gf + peak - new) * norm + math.exp(gi - new) * x
        peak = new
        o = mem * x / (max(abs(norm * x), math.exp(-peak)) + 1e-6)
        want.append(o / math.sqrt(o * o) * 0.5 * 1.0)       # unit root mean square of one element is its sign
    assert torch.allclose(got[:, 0], torch.tensor(want, dtype=F64), atol=1e-12)


def test_plain_window_and_value_blend():
    cfg = sc.config("a")
    raw, w = cfg.to_dict(), P.widen(sc.weights(cfg, 0))
    m = raw["layers"][4]["mixer"]
    T = 40
    h = torch.randn(T, cfg.width, dtype=F64)
    first = torch.randn(T, m["kv_heads"], m["vdim"], dtype=F64)
    full, own = P.attention(m, w, "l4.mix.", h, cfg.eps, first)
    size = m["mask"]["size"]
    # a token outside the window of the last query changes nothing there; one just inside does
    far, near = h.clone(), h.clone()
    far[T - 1 - size] += 1.0
    near[T - size] += 1.0
    assert torch.equal(P.attention(m, w, "l4.mix.", far, cfg.eps, first)[0][-1], full[-1])
    assert not torch.allclose(P.attention(m, w, "l4.mix.", near, cfg.eps, first)[0][-1], full[-1])
    # a window of one token and a blend weight of 1: the first layer's values through the output matrix
    w1 = dict(w, **{"l4.mix.vmix": torch.tensor(1.0, dtype=F64)})
    alone = P.attention(dict(m, mask=dict(size=1)), w1, "l4.mix.", h, cfg.eps, first)[0]
    per = m["heads"] // m["kv_heads"]
    assert torch.allclose(alone, first.repeat_interleave(per, dim=1).reshape(T, -1) @ w["l4.mix.o"].T)
    # the norm runs over all heads at once: scaling one head's rows changes the others' queries
    w2 = dict(w)
    w2["l4.mix.q"] = w["l4.mix.q"].clone()
    w2["l4.mix.q"][:m["dim"]] *= 10.0
    assert not torch.allclose(P.attention(m, w2, "l4.mix.", h, cfg.eps, first)[0], full)


def test_plain_router_takes_the_largest_scores_as_they_are():
    z = torch.tensor([[0.0, 2.0, 2.0, -1.0], [5.0, -5.0, 0.0, 0.0]], dtype=F64)
    chosen, score = P.route(z, 2)
    assert chosen.tolist() == [[1, 2], [0, 2]]
    assert torch.allclose(score, torch.sigmoid(torch.tensor([[2.0, 2.0], [5.0, 0.0]], dtype=F64)))
    # the weight is on what the expert reads: expert(s h), not s expert(h)
    cfg = sc.config("b")
    w = P.widen(sc.weights(cfg, 1))
    mlp = cfg.to_dict()["layers"][1]["mlp"]
    h = torch.randn(3, cfg.width, dtype=F64)
    got = P.mixture(mlp, w, "l1.mlp.", h)
    chosen, score = P.route(h @ w["l1.mlp.router"].T, 1)
    want = torch.stack([P.gated_expert(w, f"l1.mlp.e{int(chosen[t, 0])}.", score[t, 0] * h[t]) for t in range(3)])
    assert torch.allclose(got, want + P.gated_expert(w, "l1.mlp.shared.", h))
    outside = torch.stack([score[t, 0] * P.gated_expert(w, f"l1.mlp.e{int(chosen[t, 0])}.", h[t]) for t in range(3)])
    assert not torch.allclose(want, outside)


# ---------------------------------------------------------------- configuration and weights

def test_config_reads_the_nested_keys_and_names_the_one_at_fault(tmp_path):
    cfg = sc.config("a")
    assert (cfg.eps, cfg.embedding_scale, len(cfg.layers)) == (1e-4, 3.0, 5)
    spec = sunatar_spec(cfg)
    kinds = [l.mixer.kind for l in spec.layers]
    assert kinds == ["attention", "attention", "mlstm", "attention", "attention"]
    # the first layer blends nothing; the second is the first that does, and the later ones blend with it
    assert spec.layers[0].mixer.params["value_mix"] is None
    assert [spec.layers[i].mixer.params["value_mix"]["first"] for i in (1, 3, 4)] == [True, False, False]
    assert spec.unread == ("l1.mix.vmix",)
    assert spec.layers[3].feed_forward.kind == "none" and spec.layers[2].feed_forward.params["shared_inner"] == 0
    folder = write_random_model(cfg, str(tmp_path / "m"), 0, dtype="float32")
    arch, read = read_config(folder)
    assert arch.name == "Sunatar" and read.layers == cfg.layers and read.to_dict() == dict(cfg.to_dict(), torch_dtype="float32")
    raw = json.load(open(os.path.join(folder, "config.json")))

    def broken(change):
        r = json.loads(json.dumps(raw))
        change(r)
        return r
    for change, text in ((lambda r: r["norm"].pop("eps"), "norm.eps"),
                         (lambda r: r["layers"][2].update(type="other"), r"layers\[2\].type"),
                         (lambda r: r["layers"][0]["mixer"].pop("heads"), r"layers\[0\].mixer.heads"),
                         (lambda r: r["layers"][1]["mixer"].update(kv_heads=3), r"layers\[1\].mixer.heads"),
                         (lambda r: r["layers"][1]["mixer"]["rot"].update(dims=7), "rot.dims"),
                         (lambda r: r["layers"][1]["mixer"]["rot"]["scaling"].pop("low"), "rot.scaling.low"),
                         (lambda r: r["layers"][2]["mixer"].pop("gate_cap"), r"layers\[2\].mixer.gate_cap"),
                         (lambda r: r["layers"][3]["mixer"].update(vdim=8), r"layers\[3\].mixer"),
                         (lambda r: r["layers"][0]["mlp"]["router"].update(top=6), "router.top"),
                         (lambda r: r["layers"][0]["mlp"].update(kind="dense"), r"layers\[0\].mlp.kind"),
                         (lambda r: r.pop("width"), "width")):
        with pytest.raises(ConfigError, match=text):
            SunatarConfig.from_dict(broken(change))


def test_the_loader_names_what_is_missing_and_passes_over_the_first_blend_weight(tmp_path):
    from safetensors.torch import load_file, save_file
    from transformers_neuronx_amd.engine.factory import runner_from_folder
    cfg = sc.config("a")
    folder = write_random_model(cfg, str(tmp_path / "m"), 0, dtype="float32")
    tensors = load_file(os.path.join(folder, "model.safetensors"))
    assert "l1.mix.vmix" not in tensors and tensors["l3.mix.vmix"].shape == () and "l3.mlp.router" not in tensors
    assert tensors["l2.mix.i"].shape == (3, 96) and tensors["l0.mlp.e4.down"].shape == (96, 40)
    assert tensors["l1.mix.q.norm"].shape == (128,) and tensors["l1.mix.o"].shape == (96, 64)
    assert tensors["l3.mix.o"].shape == (96, 32) and tensors["l3.mix.v.b"].shape == (32,)
    ecfg = EngineConfig(dtype="float32", kernels="reference", device="cpu", max_tokens=64)
    # the blend weight of the first blending layer, which nothing reads, may lie in the file
    save_file(dict(tensors, **{"l1.mix.vmix": torch.tensor(0.5)}), os.path.join(folder, "model.safetensors"))
    runner_from_folder(folder, ecfg)
    bad = dict(tensors)
    del bad["l2.mix.f.b"]
    bad["l0.mix.surplus"] = torch.zeros(2)
    save_file(bad, os.path.join(folder, "model.safetensors"))
    with pytest.raises(WeightsError) as e:
        runner_from_folder(folder, ecfg)
    assert "l2.mix.f.b" in str(e.value) and "l0.mix.surplus" in str(e.value)


# ---------------------------------------------------------------- the engine on the host

def _expected(cfg, w, requests):
    raw, wide = cfg.to_dict(), P.widen(w)
    return {rid: P.forward(raw, wide, toks) for rid, toks in requests.items()}


def step_through(runner, expected, made, tol, few_over=0.0):
    """`few_over`: the share of positions that may lie over `tol`, by any distance: in bfloat16 a rounding of the
    router's input changes which expert a token takes where two scores are close, and that token's result is
    another expert's (the plain implementation in bfloat16 arithmetic is as far off there). float32 allows none."""
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


@pytest.mark.parametrize("name", sorted(sc.CASES))
def test_schedules_on_the_host(name):
    cfg = sc.config(name)
    w = sc.weights(cfg, 3)
    runner = sc.runner(cfg, w, max_tokens=208)
    requests = sc.requests(cfg, [70, 33, 5, 100, 1], 1)
    expected = _expected(cfg, w, requests)
    for made in (schedules.whole(requests), schedules.head_then_singles(requests, tail=12), schedules.portions(requests),
                 schedules.portions(requests, sizes=(2, 2, 3, 2, 16, 2, 15, 17, 2)),
                 schedules.mixed(requests, max_tokens=208, page=16, seed=5, tail=8, max_live=3),
                 schedules.only_last(schedules.mixed(requests, max_tokens=208, page=16, seed=6, tail=20, max_live=4))):
        step_through(runner, expected, made, TOL)


def test_a_slot_that_is_used_again_starts_afresh():
    """The memory a request leaves in its slot is not the next one's."""
    cfg = sc.config("b")
    w = sc.weights(cfg, 4)
    runner = sc.runner(cfg, w, max_tokens=64, max_seqs=1)
    requests = sc.requests(cfg, [37, 20, 3, 45], 2)
    expected = _expected(cfg, w, requests)
    for rid, toks in requests.items():
        assert runner.cache.slots.num_free == 1
        got = runner.step([StepEntry(rid, toks[:2], [0, 1])])
        got = torch.cat([got, runner.step([StepEntry(rid, toks[2:], list(range(len(toks) - 2)))])])
        assert float((got.double() - expected[rid]).abs().max() / expected[rid].abs().max()) < TOL
        runner.finish(rid)


def test_pages_of_a_window_go_back_and_long_decoding_stays_right():
    """Case b's windows are 1, 16 and 17 tokens: a request of 150 tokens never holds more than three pages of 16
    in any of its groups, and its memories run on through all of them."""
    cfg = sc.config("b")
    w = sc.weights(cfg, 5)
    runner = sc.runner(cfg, w, max_tokens=64, max_seqs=2)
    toks = sc.requests(cfg, [150], 3)["r0"]
    expected = _expected(cfg, w, {"r0": toks})["r0"]
    got = [runner.step([StepEntry("r0", toks[:21], list(range(21)))])]
    for t in toks[21:]:
        got.append(runner.step([StepEntry("r0", [t], [0])]))
        for g in runner.cache.groups.values():
            assert g.pool.num_pages - g.pool.num_free <= 3
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
    cfg = sc.config("c")
    w = sc.weights(cfg, 6)
    ecfg = EngineConfig(dtype="float32", kernels="reference", device="cpu", page_size=16, max_tokens=96, max_num_seqs=3,
                        max_num_batched_tokens=24, chunk_size=9, run_ahead=run_ahead)
    from transformers_neuronx_amd.engine.factory import build_runner
    from transformers_neuronx_amd.weights.loader import TensorDict
    engine = LLMEngine(build_runner(cfg, TensorDict(w), ecfg), ecfg)
    prompts = list(sc.requests(cfg, [30, 3, 17, 1, 22], 7).values())
    out = engine.generate(prompts, SamplingParams(temperature=0.0, max_new_tokens=12, ignore_eos=True))
    for prompt, tokens in zip(prompts, out):
        assert tokens == _greedy(cfg, w, prompt, 12)
    engine.runner.cache.check()
    assert not engine.runner.cache.requests


def test_generation_through_the_entry_point_on_the_host(tmp_path):
    from safetensors.torch import load_file
    from transformers_neuronx_amd import NeuronAutoModelForCausalLM
    from transformers_neuronx_amd.sunatar.model import SunatarForSampling
    cfg = sc.config("a")
    folder = write_random_model(cfg, str(tmp_path / "m"), 11, dtype="float32")
    w = load_file(os.path.join(folder, "model.safetensors"))
    model = NeuronAutoModelForCausalLM.from_pretrained(folder, batch_size=2, amp="f32", n_positions=64, page_size=16,
                                                       kernels="reference", device="cpu")
    assert type(model) is SunatarForSampling
    model.to_neuron()
    ids = torch.tensor([[5, 200, 17, 3], [9, 9, 100, 42]])
    out = model.sample(ids, sequence_length=14, top_k=1)
    for row in range(2):
        assert out[row, 4:].tolist() == _greedy(cfg, w, ids[row].tolist(), 10)


@pytest.mark.parametrize("seed", range(10))
def test_configurations_drawn_from_a_seed_on_the_host(seed):
    cfg = sc.drawn(seed)
    w = sc.weights(cfg, seed)
    runner = sc.runner(cfg, w, max_tokens=176)
    requests = sc.requests(cfg, [70, 33, 5, 1], seed)
    step_through(runner, _expected(cfg, w, requests), schedules.mixed(requests, max_tokens=176, page=16, seed=5, tail=8, max_live=3), TOL)
