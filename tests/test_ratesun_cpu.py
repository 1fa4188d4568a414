"""Ratesun on the host: the plain implementation pinned by what its mechanisms must do, the configuration's
reader, and the engine (registry, loader, cache and state manager, step function, scheduler, entry point) on the
torch rendition of the kernels against the plain implementation, for configurations of the tests' own."""
import json
import os

import pytest
import torch

import plain_ratesun as P
import ratesun_cases as rc
import schedules
from transformers_neuronx_amd.config import EngineConfig, read_config
from transformers_neuronx_amd.config.model_config import ConfigError
from transformers_neuronx_amd.engine import StepEntry
from transformers_neuronx_amd.engine.engine import LLMEngine
from transformers_neuronx_amd.ratesun import RatesunConfig, ratesun_spec
from transformers_neuronx_amd.sampling import SamplingParams
from transformers_neuronx_amd.weights import WeightsError, write_random_model


# ---------------------------------------------------------------- the plain implementation, pinned

def test_plain_rotation_counts_distances_only():
    g = torch.Generator().manual_seed(0)
    q, k = torch.randn(5, 3, 12, generator=g, dtype=torch.float64), torch.randn(5, 12, generator=g, dtype=torch.float64)
    pos = torch.tensor([0, 3, 4, 9, 20])
    a = torch.einsum("ihd,jd->hij", P.rotate_pairs(q, pos, 50.0, 8), P.rotate_pairs(k, pos, 50.0, 8))
    b = torch.einsum("ihd,jd->hij", P.rotate_pairs(q, pos + 1000, 50.0, 8), P.rotate_pairs(k, pos + 1000, 50.0, 8))
    assert torch.allclose(a, b, atol=1e-9)
    # elements beyond `dims` pass, position 0 turns nothing, and a pair keeps its length
    assert torch.equal(P.rotate_pairs(q, pos, 50.0, 8)[..., 8:], q[..., 8:])
    assert torch.allclose(P.rotate_pairs(q, pos, 50.0, 8)[0], q[0])
    turned = P.rotate_pairs(q, pos, 50.0, 12)
    assert torch.allclose(turned[..., 0] ** 2 + turned[..., 1] ** 2, q[..., 0] ** 2 + q[..., 1] ** 2)
    # the first pair turns by the position itself (frequency 1): a quarter turn at pi / 2 ... checked by hand
    one = P.rotate_pairs(torch.tensor([[1.0, 0.0]], dtype=torch.float64), torch.tensor([1]), 7.0, 2)
    assert torch.allclose(one, torch.tensor([[torch.cos(torch.tensor(1.0)), torch.sin(torch.tensor(1.0))]], dtype=torch.float64))


def test_plain_convolution_norms_and_rows():
    h = torch.arange(12, dtype=torch.float64).reshape(6, 2) + 1
    w = torch.tensor([[0.5, 0.25, 2.0], [1.0, 0.0, -1.0]], dtype=torch.float64)
    out = P.input_conv(h, w)
    # token 0 sees itself alone (the last tap), token 2 all three
    assert torch.allclose(out[0], h[0] + w[:, 2] * h[0])
    assert torch.allclose(out[2], h[2] + w[:, 0] * h[0] + w[:, 1] * h[1] + w[:, 2] * h[2])
    assert torch.allclose(P.input_conv(h, w[:, :1]), h * (1 + w[:, 0]))
    z = torch.full((1, 7), 3.0, dtype=torch.float64)
    assert torch.allclose(P.poly_norm(z, torch.tensor([1.0, 10.0, 100.0, 0.5]), 1e-12), torch.full((1, 7), 111.5, dtype=torch.float64))
    x = torch.randn(4, 9, dtype=torch.float64)
    assert torch.allclose(P.layer_norm(x, torch.ones(9), torch.zeros(9), 1e-5),
                          torch.nn.functional.layer_norm(x, (9,), eps=1e-5))
    assert P.bigram_rows([5, 6, 5], 11, 3, 2) == [11, (5 * 3 + 6 * 2) % 11, (6 * 3 + 5 * 2) % 11]
    assert abs(float(P.gelu_tanh(torch.tensor(1.0, dtype=torch.float64))) - 0.8411919906) < 1e-9


def test_plain_window_and_borrowed_latent():
    cfg = rc.config("a")
    raw, w = cfg.to_dict(), P.widen(rc.weights(cfg, 0))
    m = raw["layers"][0]["mixer"]
    T = 40
    h = torch.randn(T, cfg.width, dtype=torch.float64)
    pos = torch.arange(T)
    c, kr = P.kv_latent(h, w, "l0.mix.", m, cfg.eps, pos)
    full = P.latent_attention(h, w, "l0.mix.", m, cfg.eps, pos, c, kr)
    # a latent outside the window of every query that is asked for changes nothing; one just inside does
    far, near = c.clone(), c.clone()
    far[T - 1 - m["mask"]["size"]] += 5.0
    near[T - m["mask"]["size"]] += 5.0
    assert torch.equal(P.latent_attention(h, w, "l0.mix.", m, cfg.eps, pos, far, kr)[-1], full[-1])
    assert not torch.allclose(P.latent_attention(h, w, "l0.mix.", m, cfg.eps, pos, near, kr)[-1], full[-1])
    # a window of one token: the token's own value through the output matrix
    one = dict(m, mask=dict(size=1))
    own = (c @ w["l0.mix.uv"].T) @ w["l0.mix.o"].T
    assert torch.allclose(P.latent_attention(h, w, "l0.mix.", one, cfg.eps, pos, c, kr), own)


# ---------------------------------------------------------------- configuration and weights

def test_config_reads_the_nested_keys_and_names_the_one_at_fault(tmp_path):
    cfg = rc.config("a")
    assert (cfg.eps, cfg.taps, cfg.side_dim, cfg.bigram["buckets"]) == (1e-4, 4, 8, 97)
    spec = ratesun_spec(cfg)
    assert [(c.layer, c.cache, c.writes) for c in spec.schedule] == [(0, 0, True), (1, 0, False), (2, 2, True), (3, 2, False)]
    # the latent of layer 0 is kept for the wider window of its reader, that of layer 2 for good
    assert spec.layers[0].mixer.params["keep"] == 50 and spec.layers[0].mixer.params["window"] == 24
    assert spec.layers[2].mixer.params["keep"] == "all"
    # a writer with a window whose reader sees everything keeps everything (seed 1 of the drawn configurations)
    drawn = ratesun_spec(rc.drawn(1))
    assert drawn.layers[0].mixer.params["window"] == 1 and drawn.layers[0].mixer.params["keep"] == "all"
    folder = write_random_model(cfg, str(tmp_path / "m"), 0, dtype="float32")
    arch, read = read_config(folder)
    assert arch.name == "Ratesun" and read.layers == cfg.layers and read.to_dict() == dict(cfg.to_dict(), torch_dtype="float32")
    raw = json.load(open(os.path.join(folder, "config.json")))

    def broken(change):
        r = json.loads(json.dumps(raw))
        change(r)
        return r
    for change, text in ((lambda r: r["norm"].pop("eps"), "norm.eps"),
                         (lambda r: r["layers"][1]["mixer"].update(kv_from=1), "kv_from"),
                         (lambda r: r["layers"][1]["mixer"].update(kv_rank=16), r"layers\[1\].mixer.kv_rank"),
                         (lambda r: r["layers"][2].update(type="other"), r"layers\[2\].type"),
                         (lambda r: r["layers"][0]["mixer"].pop("heads"), r"layers\[0\].mixer.heads"),
                         (lambda r: r["layers"][0]["mixer"]["rot"].update(dims=7), "rot.dims"),
                         (lambda r: r["canon"].update(taps=0), "canon.taps"),
                         (lambda r: r.pop("width"), "width")):
        with pytest.raises(ConfigError, match=text):
            RatesunConfig.from_dict(broken(change))


def test_the_loader_names_what_is_missing_and_passes_over_what_an_absent_part_left(tmp_path):
    from safetensors.torch import load_file, save_file
    from transformers_neuronx_amd.engine.factory import runner_from_folder
    cfg = rc.config("a")
    folder = write_random_model(cfg, str(tmp_path / "m"), 0, dtype="float32")
    tensors = load_file(os.path.join(folder, "model.safetensors"))
    assert "l1.mlp.up" not in tensors and "l1.canon2" not in tensors and "l1.mix.dkv" not in tensors
    assert tensors["l3.dwa"].shape == (5,) and tensors["side.embed"].shape == (211, 32) and tensors["bigram"].shape == (98, 96)
    ecfg = EngineConfig(dtype="float32", kernels="reference", device="cpu", max_tokens=64)
    # vectors of the feed-forward that layer 1 does not have may lie in the file
    save_file(dict(tensors, **{"l1.norm2": torch.ones(96), "l1.canon2": torch.ones(96, 4)}), os.path.join(folder, "model.safetensors"))
    runner_from_folder(folder, ecfg)
    bad = dict(tensors)
    del bad["l2.mix.dkv.norm"]
    bad["l0.mix.surplus"] = torch.zeros(2)
    save_file(bad, os.path.join(folder, "model.safetensors"))
    with pytest.raises(WeightsError) as e:
        runner_from_folder(folder, ecfg)
    assert "l2.mix.dkv.norm" in str(e.value) and "l0.mix.surplus" in str(e.value)


# ---------------------------------------------------------------- the engine on the host

def _expected(cfg, w, requests):
    raw, wide = cfg.to_dict(), P.widen(w)
    return {rid: P.forward(raw, wide, toks) for rid, toks in requests.items()}


def step_through(runner, expected, made, tol, few_over=0.0):
    """`few_over`: the share of positions that may lie over `tol` (none by more than ten times): bfloat16 at a
    place where the model itself is ill-conditioned, such as a token-keyed input of one element, whose sign a
    rounding can turn; the plain implementation in bfloat16 arithmetic is as far off there."""
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
            assert err < tol * (10 if few_over else 1), (rec["step"], rid, pos, err)
        for rid in rec["end"]:
            runner.finish(rid)
        runner.cache.check()
    assert len(over) <= few_over * seen, over[:5]
    assert not runner.cache.requests


@pytest.mark.parametrize("name", sorted(rc.CASES))
def test_schedules_on_the_host(name):
    cfg = rc.config(name)
    w = rc.weights(cfg, 3)
    runner = rc.runner(cfg, w, max_tokens=208)
    requests = rc.requests(cfg, [70, 33, 5, 100, 1], 1)
    expected = _expected(cfg, w, requests)
    for made in (schedules.whole(requests), schedules.head_then_singles(requests, tail=12), schedules.portions(requests),
                 schedules.portions(requests, sizes=(2, 2, 3, 2, 16, 2, 15, 17, 2)),
                 schedules.mixed(requests, max_tokens=208, page=16, seed=5, tail=8, max_live=3),
                 schedules.only_last(schedules.mixed(requests, max_tokens=208, page=16, seed=6, tail=20, max_live=4))):
        step_through(runner, expected, made, 2e-5)


def test_a_slot_that_is_used_again_starts_afresh():
    """The state a request leaves (its last token, the inputs of its convolutions) is not the next one's."""
    cfg = rc.config("a")
    w = rc.weights(cfg, 4)
    runner = rc.runner(cfg, w, max_tokens=64, max_seqs=1)
    requests = rc.requests(cfg, [37, 20, 3, 45], 2)
    expected = _expected(cfg, w, requests)
    for rid, toks in requests.items():
        assert runner.cache.slots.num_free == 1
        got = runner.step([StepEntry(rid, toks[:2], [0, 1])])
        got = torch.cat([got, runner.step([StepEntry(rid, toks[2:], list(range(len(toks) - 2)))])])
        assert float((got.double() - expected[rid]).abs().max() / expected[rid].abs().max()) < 2e-5
        runner.finish(rid)


def test_pages_of_a_window_go_back_and_long_decoding_stays_right():
    """Case b's widest window is 17 tokens: a request of 150 tokens never holds more than three pages of 16."""
    cfg = rc.config("b")
    w = rc.weights(cfg, 5)
    runner = rc.runner(cfg, w, max_tokens=64, max_seqs=2)
    toks = rc.requests(cfg, [150], 3)["r0"]
    expected = _expected(cfg, w, {"r0": toks})["r0"]
    got = [runner.step([StepEntry("r0", toks[:21], list(range(21)))])]
    for t in toks[21:]:
        got.append(runner.step([StepEntry("r0", [t], [0])]))
        for g in runner.cache.groups.values():
            assert g.pool.num_pages - g.pool.num_free <= 3
    got = torch.cat(got)
    assert float((got.double() - expected).abs().max() / expected.abs().max()) < 2e-5


def _greedy(cfg, w, prompt, new):
    raw, wide = cfg.to_dict(), P.widen(w)
    toks = list(prompt)
    for _ in range(new):
        toks.append(int(P.forward(raw, wide, toks)[-1].argmax()))
    return toks[len(prompt):]


@pytest.mark.parametrize("run_ahead", [False, True])
def test_greedy_generation_through_the_scheduler(run_ahead):
    cfg = rc.config("c")
    w = rc.weights(cfg, 6)
    ecfg = EngineConfig(dtype="float32", kernels="reference", device="cpu", page_size=16, max_tokens=96, max_num_seqs=3,
                        max_num_batched_tokens=24, chunk_size=9, run_ahead=run_ahead)
    from transformers_neuronx_amd.engine.factory import build_runner
    from transformers_neuronx_amd.weights.loader import TensorDict
    engine = LLMEngine(build_runner(cfg, TensorDict(w), ecfg), ecfg)
    prompts = list(rc.requests(cfg, [30, 3, 17, 1, 22], 7).values())
    out = engine.generate(prompts, SamplingParams(temperature=0.0, max_new_tokens=12, ignore_eos=True))
    for prompt, tokens in zip(prompts, out):
        assert tokens == _greedy(cfg, w, prompt, 12)
    engine.runner.cache.check()
    assert not engine.runner.cache.requests


def test_generation_through_the_entry_point_on_the_host(tmp_path):
    from safetensors.torch import load_file
    from transformers_neuronx_amd import NeuronAutoModelForCausalLM
    from transformers_neuronx_amd.ratesun.model import RatesunForSampling
    cfg = rc.config("a")
    folder = write_random_model(cfg, str(tmp_path / "m"), 11, dtype="float32")
    w = load_file(os.path.join(folder, "model.safetensors"))
    model = NeuronAutoModelForCausalLM.from_pretrained(folder, batch_size=2, amp="f32", n_positions=64, page_size=16,
                                                       kernels="reference", device="cpu")
    assert type(model) is RatesunForSampling
    model.to_neuron()
    ids = torch.tensor([[5, 200, 17, 3], [9, 9, 100, 42]])
    out = model.sample(ids, sequence_length=14, top_k=1)
    for row in range(2):
        assert out[row, 4:].tolist() == _greedy(cfg, w, ids[row].tolist(), 10)


def test_bindings_pass_as_many_arguments_as_the_entry_points_take():
    """Every C entry point of the package's kernel modules is declared with as many argument types as its source
    has parameters (a call with one too many would hand the launch a stream cut to 32 bits)."""
    import re
    from transformers_neuronx_amd.kernels import build, hip
    for module in build.MODULES:
        source = open(os.path.join(build.CSRC, f"{module}.hip")).read()
        for name, types in hip._SIGNATURES[module].items():
            found = re.search(r'extern "C" int ' + name + r"\(([^)]*)\)", source)
            assert found, f"{module}.hip has no entry point {name}"
            assert len([a for a in found.group(1).split(",") if a.strip()]) == len(types), name


@pytest.mark.parametrize("seed", range(10))
def test_configurations_drawn_from_a_seed_on_the_host(seed):
    cfg = rc.drawn(seed)
    w = rc.weights(cfg, seed)
    runner = rc.runner(cfg, w, max_tokens=176)
    requests = rc.requests(cfg, [70, 33, 5, 1], seed)
    step_through(runner, _expected(cfg, w, requests), schedules.mixed(requests, max_tokens=176, page=16, seed=5, tail=8, max_live=3), 2e-5)
