"""Sunatar on the GPU: every kernel of its parts alone against the plain implementation's function of the same
mechanism (float32 and bfloat16), attention with a key made to stand out far away, at page borders, at the first
token and just inside and outside the window, memories and pages that change hands, the engine under every way
of cutting, recorded decoding, generation through the entry point, and the replay program."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_sunatar as P
import sunatar_cases as sc
import schedules
from test_sunatar_cpu import TOL, _expected, _greedy, step_through
from transformers_neuronx_amd.engine import StepEntry
from transformers_neuronx_amd.engine.batch import build_context

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DTYPES = [("float32", torch.float32, 5e-6), ("bfloat16", torch.bfloat16, 1.2e-2)]
F64 = torch.float64


def _ops(dtype):
    from transformers_neuronx_amd.kernels import make_ops
    return make_ops("hip", dtype, DEV)


def _ctx(runs, cached, slots, tables=None, page_size=16, planners=None):
    entries = [StepEntry(i, [0] * n, []) for i, n in enumerate(runs)]
    tables = tables if tables is not None else {}
    return build_context(entries, cached, slots, {k: np.asarray(v, dtype=np.int32) for k, v in tables.items()},
                         page_size, DEV, planners)


def _close(got, want, tol):
    want = want.to(F64)
    err = float((got.double().cpu() - want).abs().max() / max(1e-30, float(want.abs().max())))
    assert err < tol, err


# ---------------------------------------------------------------- each mechanism alone

@pytest.mark.parametrize("name,dtype,tol", DTYPES)
@pytest.mark.parametrize("sizes", [
    # heads, kv heads, n, v, cached head, turned elements, scaling, blended
    (3, 1, 10, 14, 16, 6, None, True), (4, 2, 32, 16, 32, 32, (8.0, 1.0, 4.0, 64), True), (2, 2, 16, 40, 48, 4, None, False),
    (8, 2, 128, 128, 128, 64, (8.0, 1.0, 4.0, 512), True), (1, 1, 8, 8, 16, 2, (2.0, 0.5, 3.0, 16), False)])
def test_projections_are_normed_turned_blended_and_stored(name, dtype, tol, sizes):
    """Queries and keys: one norm over all heads, halves turned by the position, the scale; values blended with
    another layer's; both into pages in heads filled up with zeros. Two steps: a portion, then a portion beside a
    single token of another request."""
    heads, groups, n, v, d, dims, scaling, blended = sizes
    ops = _ops(dtype)
    g = torch.Generator().manual_seed(3)
    ps, eps, scale, lam = 16, 1e-5, 0.37, 0.3
    total = heads * n + groups * (n + v)
    lens = {0: 41, 1: 19}
    proj = {r: torch.randn(t, total, generator=g) * 2 for r, t in lens.items()}
    first = {r: torch.randn(t, groups * v, generator=g) for r, t in lens.items()}
    qw, kw = torch.rand(heads * n, generator=g) + 0.5, torch.rand(groups * n, generator=g) + 0.5
    from transformers_neuronx_amd.parts.position import RotaryPositions
    rotation = RotaryPositions(500.0, dims, interleaved=False, scaling=dict(zip(("factor", "low", "high", "original"), scaling)) if scaling else None)
    rotation.device = DEV
    freqs = rotation.frequencies()
    plain_f = P.rotary_frequencies(500.0, dims, dict(zip(("factor", "low", "high", "original"), scaling)) if scaling else None)
    _close(freqs, plain_f, 1e-6)
    want = {}
    for r, t in lens.items():
        x = proj[r].double()
        q = P.unit_rms(x[:, :heads * n], eps) * qw.double()
        k = P.unit_rms(x[:, heads * n:heads * n + groups * n], eps) * kw.double()
        pos = torch.arange(t)
        q = P.rotate_halves(q.view(t, heads, n), pos, plain_f) * scale
        k = P.rotate_halves(k.view(t, groups, n), pos, plain_f)
        val = x[:, heads * n + groups * n:]
        if blended:
            val = (1 - lam) * val + lam * first[r].double()
        want[r] = (q, k, val.view(t, groups, v))
    k_pages = torch.full((12, groups, ps, d), 7.0, dtype=dtype, device=DEV)      # what former holders left
    v_pages = torch.full((12, groups, d, ps), 7.0, dtype=dtype, device=DEV)
    tables = {0: [5, 2, 9], 1: [4, 11]}
    steps = [[(0, 0, 30)], [(0, 30, 41), (1, 0, 18)], [(1, 18, 19)]]
    mixw = torch.tensor([lam], device=DEV)
    for step in steps:
        rows = torch.cat([proj[r][a:b] for r, a, b in step]).to(DEV)
        # the values to blend with are a view into a wider tensor, as the first layer's projections are
        wide = torch.cat([torch.cat([torch.zeros(b - a, 3), first[r][a:b]], dim=1) for r, a, b in step]).to(DEV)
        table = np.full((len(step), 3), -1, dtype=np.int32)
        for i, (r, _, _) in enumerate(step):
            table[i, :len(tables[r])] = tables[r]
        ctx = _ctx([b - a for _, a, b in step], [a for _, a, _ in step], [r for r, _, _ in step], {"g": table}, ps)
        q = ops.qkv_prepare(rows, heads, groups, n, v, d, qw.to(DEV), kw.to(DEV), eps, freqs, False, scale, mixw,
                            wide[:, 3:] if blended else None, ctx, ctx.groups["g"], k_pages, v_pages)
        at = 0
        for r, a, b in step:
            got = q[at:at + b - a].view(b - a, heads, d)
            _close(got[:, :, :n], want[r][0][a:b], tol)
            assert not got[:, :, n:].any()
            at += b - a
    for r, t in lens.items():
        pages = torch.tensor(tables[r])
        keys = k_pages[pages].permute(0, 2, 1, 3).reshape(-1, groups, d)[:t]
        vals = v_pages[pages].permute(0, 3, 1, 2).reshape(-1, groups, d)[:t]
        _close(keys[:, :, :n], want[r][1], tol)
        _close(vals[:, :, :v], want[r][2], tol)
        assert not keys[:, :, n:].any() and not vals[:, :, v:].any()
    assert float(k_pages[0].float().min()) == 7.0       # a page of no one is not touched


@pytest.mark.parametrize("name,dtype,tol", DTYPES)
@pytest.mark.parametrize("sizes", [(1, 1, 1), (3, 8, 40), (5, 32, 48), (2, 6, 10), (2, 128, 128), (1, 100, 272), (2, 12, 600)])
def test_matrix_memory_across_steps_cut_anywhere(name, dtype, tol, sizes):
    """The recurrence over steps of 1, 2 and more tokens, two requests side by side in slots that former holders
    left full, every step of single tokens run twice (a recorded step is), against the whole sequence at once."""
    heads, n, v = sizes
    ops = _ops(dtype)
    g = torch.Generator().manual_seed(4)
    cap, eps = 9.0, 1e-5
    total = 2 * heads * n + 2 * heads * v + 2 * heads
    lens = {0: 45, 1: 12}
    proj = {r: torch.randn(t, total, generator=g) for r, t in lens.items()}
    for r in proj:
        proj[r][:, -2 * heads:] *= 4.0        # gates that open and close
    nw = torch.rand(heads * v, generator=g) + 0.5
    want = {}
    for r, t in lens.items():
        x = proj[r].double()
        hn, hv = heads * n, heads * v
        # the plain function takes a mixer's input and its matrices: identity matrices hand it the projections
        m = dict(heads=heads, dim=n, vdim=v, gate_cap=cap)
        eye = torch.eye(total, dtype=F64)
        w = {"p.q": eye[:hn], "p.k": eye[hn:2 * hn], "p.v": eye[2 * hn:2 * hn + hv], "p.g": eye[2 * hn + hv:2 * hn + 2 * hv],
             "p.i": eye[-2 * heads:-heads], "p.f": eye[-heads:], "p.i.b": torch.zeros(heads, dtype=F64),
             "p.f.b": torch.zeros(heads, dtype=F64), "p.norm": nw.double(), "p.o": torch.eye(hv, dtype=F64)}
        want[r] = P.mlstm(m, w, "p.", x, eps)
    state = [torch.full((3, 2, heads, v, n), 3.0, device=DEV), torch.full((3, 2, heads, n), -2.0, device=DEV),
             torch.full((3, 2, heads), 5.0, device=DEV)]
    # request 0 in slot 2, request 1 in slot 0 from the third step on
    cuts0 = [0, 1, 2, 4, 5, 6, 30, 32, 45]
    cuts1 = [None, None, 0, 1, 2, 9, 11, 12, None]
    for s in range(len(cuts0) - 1):
        step = [(0, cuts0[s], cuts0[s + 1], 2)]
        if cuts1[s] is not None and cuts1[s + 1] is not None:
            step.append((1, cuts1[s], cuts1[s + 1], 0))
        rows = torch.cat([proj[r][a:b] for r, a, b, _ in step]).to(DEV)
        ctx = _ctx([b - a for _, a, b, _ in step], [a for _, a, _, _ in step], [slot for _, _, _, slot in step])
        single = all(b - a == 1 for _, a, b, _ in step)
        for _ in range(2 if single else 1):
            got = ops.matrix_memory(rows, heads, n, v, cap, eps, nw.to(DEV), ctx, *state)
        at = 0
        for r, a, b, _ in step:
            _close(got[at:at + b - a], want[r][a:b], max(tol, 2e-5))
            at += b - a
    assert float(state[0][1].min()) == 3.0       # a slot of no one is not touched


@pytest.mark.parametrize("name,dtype,tol", DTYPES)
@pytest.mark.parametrize("sizes", [
    # tokens, experts, a token's experts, width, inner size, shared inner size
    (1, 4, 1, 64, 16, 0), (37, 5, 2, 96, 40, 24), (130, 10, 1, 192, 72, 88), (9, 3, 3, 50, 30, 10), (300, 70, 4, 128, 24, 0)])
def test_router_and_experts(name, dtype, tol, sizes):
    from transformers_neuronx_amd.parts.feed_forward import ExpertMixture
    tokens, experts, top, width, inner, shared = sizes
    ops = _ops(dtype)
    g = torch.Generator().manual_seed(5)
    part = ExpertMixture(width, experts, top, inner, "router", "e{}.", ("gate", "up", "down"), shared_inner=shared,
                         score="sigmoid", weight_on="input")
    w = {}
    for d in part.param_decls("p."):
        w[d.name] = (torch.randn(d.shape, generator=g) * (1.5 / d.shape[1] ** 0.5)).to(dtype)
    w["p.router"] = (w["p.router"].float() * 2).to(dtype)
    part.load({k: v.to(DEV) for k, v in w.items()}, "p.", ops, dtype)
    h = torch.randn(tokens, width, generator=g).to(dtype)
    residual = torch.randn(tokens, width, generator=g)
    mlp = dict(router=dict(experts=experts, top=top), expert=dict(ff=inner), shared=dict(ff=shared) if shared else None)
    wide = P.widen(w)
    got = part.forward(h.to(DEV), None, residual.to(DEV))
    # the router's choice alone: to the number wherever the plain scores leave no doubt about it
    s = torch.sigmoid(h.double() @ wide["p.router"].T)
    ranked = torch.sort(s, dim=-1, descending=True, stable=True).values
    gaps = (ranked[:, :-1] - ranked[:, 1:])[:, :top].min(-1).values if experts > 1 else torch.ones(tokens, dtype=F64)
    # (the kernel sees the same rounded inputs as the plain function; scores that float32 cannot tell apart, such
    # as two that are 1 to its last bit, are the doubt)
    clear = gaps > 1e-5
    assert int(clear.sum()) >= tokens // 3
    chosen, score = P.route(h.double() @ wide["p.router"].T, top)
    got_chosen, got_score = ops.route(ops.linear(h.to(DEV), part.w_router, None, out_f32=True), top, "sigmoid", False)
    assert got_chosen.cpu()[clear].tolist() == chosen[clear].tolist()
    _close(got_score.cpu()[clear], score[clear], 1e-5 if dtype == torch.float32 else 1e-2)
    # the experts' sum for the tokens whose choice is clear
    want = residual.double() + P.mixture(mlp, wide, "p.", h.double())
    _close(got.cpu()[clear], want[clear], tol)


@pytest.mark.parametrize("weight_on,score,renormalize", [("input", "sigmoid", False), ("output", "softmax", True)])
@pytest.mark.parametrize("forced", [None, "ours", "plain"])
def test_experts_of_a_step_of_many_tokens(weight_on, score, renormalize, forced):
    """Many pairs an expert: the experts' products go to the vendor library over rows in expert order (the host
    reads where each expert's rows begin); `forced`: the same step held on our own kernels, with and without the
    matrix unit. All against sums made token by token, with the router's own choice."""
    from transformers_neuronx_amd.parts.feed_forward import ExpertMixture
    tokens, experts, top, width, inner = 700, 4, 2, 128, 72
    ops = _ops(torch.bfloat16)
    ops.expert_library_rows = 0 if forced else 96
    ops.expert_plain_products = forced == "plain"
    g = torch.Generator().manual_seed(6)
    part = ExpertMixture(width, experts, top, inner, "router", "e{}.", ("gate", "up", "down"), score=score,
                         renormalize=renormalize, weight_on=weight_on)
    w = {d.name: (torch.randn(d.shape, generator=g) * (1.5 / d.shape[1] ** 0.5)).to(torch.bfloat16) for d in part.param_decls("p.")}
    part.load({k: v.to(DEV) for k, v in w.items()}, "p.", ops, torch.bfloat16)
    h = torch.randn(tokens, width, generator=g).to(torch.bfloat16)
    residual = torch.randn(tokens, width, generator=g)
    ctx = _ctx([tokens], [0], [0])
    got = part.forward(h.to(DEV), ctx, residual.to(DEV))
    chosen, weights = ops.route(ops.linear(h.to(DEV), part.w_router, None, out_f32=True), top, score, renormalize)
    chosen, weights = chosen.cpu(), weights.cpu().double()
    wide = P.widen(w)
    want = residual.double().clone()
    for t in range(tokens):
        for c in range(top):
            e, s = int(chosen[t, c]), weights[t, c]
            if weight_on == "input":
                want[t] += P.gated_expert(wide, f"p.e{e}.", s * h[t].double())
            else:
                want[t] += s * P.gated_expert(wide, f"p.e{e}.", h[t].double())
    _close(got, want, 1.2e-2)


def _standout(dtype, heads, groups, n, v, d, window, length, run, ps, standout, seed):
    """A request of `length` tokens whose last `run` are the step's: projections such that for the last query the
    key at position `standout` scores far above the rest in every head. Returns the projections of all tokens
    and the plain result for the last `run` queries."""
    g = torch.Generator().manual_seed(seed)
    total = heads * n + groups * (n + v)
    proj = torch.randn(length, total, generator=g) * 0.3
    mark = torch.randn(n, generator=g)
    mark = mark / mark.norm() * 9.0
    for gi in range(groups):
        proj[standout, heads * n + gi * n:heads * n + (gi + 1) * n] = mark
    for h in range(heads):
        proj[length - 1, h * n:(h + 1) * n] = mark
    proj = proj.to(dtype).float()
    x = proj.double()
    q = x[:, :heads * n].view(length, heads, n)
    k = x[:, heads * n:heads * n + groups * n].view(length, groups, n).repeat_interleave(heads // groups, dim=1)
    val = x[:, heads * n + groups * n:].view(length, groups, v).repeat_interleave(heads // groups, dim=1)
    prob = P.window_softmax(torch.einsum("ihd,jhd->hij", q, k), window)
    want = torch.einsum("hij,jhd->ihd", prob, val)[length - run:]
    return proj, want, prob


@pytest.mark.parametrize("name,dtype,tol", DTYPES)
@pytest.mark.parametrize("case", [
    # query heads, kv heads, n, v, cached head, window, length, run, page, standout (back from the last query)
    dict(h=4, g=2, n=16, v=24, d=32, window=40, length=300, run=1, ps=16, back=39),      # just inside the window
    dict(h=4, g=2, n=16, v=24, d=32, window=40, length=300, run=1, ps=16, back=40),      # just outside
    dict(h=2, g=1, n=64, v=64, d=64, window=0, length=700, run=1, ps=16, back=697),      # far away, no window
    dict(h=2, g=2, n=32, v=16, d=32, window=0, length=700, run=37, ps=16, back=699),     # the very first token, in a portion
    dict(h=6, g=3, n=16, v=16, d=16, window=17, length=64, run=64, ps=16, back=16),      # a whole prompt, edge of the window
    dict(h=6, g=3, n=16, v=16, d=16, window=17, length=64, run=64, ps=16, back=17),
    dict(h=1, g=1, n=64, v=32, d=64, window=33, length=129, run=2, ps=64, back=32),      # a page border
    dict(h=4, g=1, n=16, v=16, d=16, window=1, length=50, run=3, ps=16, back=0),         # a window of one token
    dict(h=2, g=2, n=128, v=128, d=128, window=300, length=280, run=5, ps=16, back=279), # a window wider than the request
    dict(h=6, g=2, n=48, v=80, d=80, window=70, length=390, run=1, ps=64, back=69),       # values wider than keys
    dict(h=6, g=2, n=48, v=80, d=80, window=70, length=390, run=200, ps=64, back=70),
])
def test_attention_finds_the_key_that_stands_out(name, dtype, tol, case):
    """Through the kernel that stores and the attention kernels, no norm and no turning, so that the step's
    projections are the queries and keys themselves."""
    from transformers_neuronx_amd.kernels.attention_plan import attention_plan
    ops = _ops(dtype)
    h, g, n, v, d, window, length, run, ps = (case[k] for k in ("h", "g", "n", "v", "d", "window", "length", "run", "ps"))
    standout = length - 1 - case["back"]
    proj, want, prob = _standout(dtype, h, g, n, v, d, window, length, run, ps, standout, 7)
    visible = not window or case["back"] < window
    if case["back"] > 0 or window == 1:
        assert (float(prob[:, -1, standout].min()) > 0.9) == visible
    blocks = -(-length // ps)
    order = torch.randperm(blocks + 3, generator=torch.Generator().manual_seed(1))[:blocks].tolist()
    k_pages = torch.zeros(blocks + 3, g, ps, d, dtype=dtype, device=DEV)
    v_pages = torch.zeros(blocks + 3, g, d, ps, dtype=dtype, device=DEV)
    head = length - run
    got = None
    for a, b in ((0, head), (head, length)):
        if b == a:
            continue
        ctx = _ctx([b - a], [a], [0], {"g": [order]}, ps, {"attention": attention_plan})
        q = ops.qkv_prepare(proj[a:b].to(DEV), h, g, n, v, d, None, None, 0.0, None, False, 1.0, None, None, ctx,
                            ctx.groups["g"], k_pages, v_pages)
        got = ops.attention(q, h, g, d, ctx, ctx.groups["g"], k_pages, v_pages, window or None)
    _close(got.view(run, h, d)[:, :, :v], want, tol)


# ---------------------------------------------------------------- the engine

@pytest.mark.parametrize("dtype,tol", [("float32", TOL), ("bfloat16", 6e-2)])
@pytest.mark.parametrize("name", sorted(sc.CASES))
def test_schedules_on_the_gpu(name, dtype, tol):
    cfg = sc.config(name)
    w = sc.weights(cfg, 3, torch.bfloat16 if dtype == "bfloat16" else torch.float32)
    runner = sc.runner(cfg, w, dtype=dtype, kernels="hip", device=DEV, max_tokens=208)
    requests = sc.requests(cfg, [70, 33, 5, 100, 1], 1)
    expected = _expected(cfg, w, requests)
    few = 0.15 if dtype == "bfloat16" else 0.0
    for made in (schedules.whole(requests), schedules.head_then_singles(requests, tail=12), schedules.portions(requests),
                 schedules.portions(requests, sizes=(2, 2, 3, 2, 16, 2, 15, 17, 2)),
                 schedules.mixed(requests, max_tokens=208, page=16, seed=5, tail=8, max_live=3),
                 schedules.only_last(schedules.mixed(requests, max_tokens=208, page=16, seed=6, tail=20, max_live=4))):
        step_through(runner, expected, made, tol, few)
    from transformers_neuronx_amd.kernels import hip
    assert {"prepare", "memory", "experts", "gemm", "attention"} <= set(hip.loaded_libraries())


@pytest.mark.parametrize("graphs", [True, False])
def test_long_decoding_recorded_and_not(graphs):
    """300 tokens one by one beside requests that join and leave: windows pass over decoded tokens, pages go
    back, memories run on, the batch size changes (a recorded step is made for each), slots change hands."""
    cfg = sc.config("d")
    w = sc.weights(cfg, 8)
    runner = sc.runner(cfg, w, dtype="float32", kernels="hip", device=DEV, max_tokens=512, page_size=16, use_graphs=graphs)
    requests = sc.requests(cfg, [320, 90, 60], 9)
    expected = _expected(cfg, w, requests)
    a, b, c = requests["r0"], requests["r1"], requests["r2"]
    got = {"r0": [runner.step([StepEntry("r0", a[:20], list(range(20)))])], "r1": [], "r2": []}
    for i in range(20, 320):
        entries = [StepEntry("r0", [a[i]], [0])]
        if 50 <= i < 140:
            entries.append(StepEntry("r1", [b[i - 50]], [0]))
        if 200 <= i < 260:
            entries.append(StepEntry("r2", [c[i - 200]], [0]))
        out = runner.step(entries)
        for row, e in enumerate(entries):
            got[e.req].append(out[row:row + 1].clone())
        if i == 139:
            runner.finish("r1")
        if i == 259:
            runner.finish("r2")
    assert (runner.graph_replays > 0) == graphs
    for rid in requests:
        have = torch.cat(got[rid])
        assert float((have.double().cpu() - expected[rid]).abs().max() / expected[rid].abs().max()) < TOL, rid


@pytest.mark.parametrize("amp,tol", [("f32", TOL), ("bf16", 6e-2)])
def test_generation_through_the_entry_point(tmp_path, amp, tol):
    from safetensors.torch import load_file
    from transformers_neuronx_amd import NeuronAutoModelForCausalLM
    from transformers_neuronx_amd.weights import write_random_model
    cfg = sc.config("a")
    folder = write_random_model(cfg, str(tmp_path / "m"), 11, dtype="float32" if amp == "f32" else "bfloat16")
    w = load_file(os.path.join(folder, "model.safetensors"))
    model = NeuronAutoModelForCausalLM.from_pretrained(folder, batch_size=2, amp=amp, n_positions=64, page_size=16,
                                                       device=DEV).load()
    ids = torch.tensor([[5, 200, 17, 3], [9, 9, 100, 42]])
    logits = model(ids)
    raw, wide = cfg.to_dict(), P.widen(w)
    for row in range(2):
        want = P.forward(raw, wide, ids[row].tolist())[-1]
        assert float((logits[row].double().cpu() - want).abs().max() / want.abs().max()) < tol
    if amp == "f32":
        out = model.sample(ids, sequence_length=14, top_k=1)
        for row in range(2):
            assert out[row, 4:].tolist() == _greedy(cfg, w, ids[row].tolist(), 10)


def test_generation_through_the_scheduler_with_few_pages():
    from transformers_neuronx_amd.config import EngineConfig
    from transformers_neuronx_amd.engine.engine import LLMEngine
    from transformers_neuronx_amd.engine.factory import build_runner
    from transformers_neuronx_amd.sampling import SamplingParams
    from transformers_neuronx_amd.weights.loader import TensorDict
    cfg = sc.config("c")
    w = sc.weights(cfg, 6)
    ecfg = EngineConfig(dtype="float32", kernels="hip", device=DEV, page_size=16, max_tokens=96, max_num_seqs=3,
                        max_num_batched_tokens=24, chunk_size=9)
    engine = LLMEngine(build_runner(cfg, TensorDict(w), ecfg), ecfg)
    prompts = list(sc.requests(cfg, [30, 3, 17, 1, 22], 7).values())
    out = engine.generate(prompts, SamplingParams(temperature=0.0, max_new_tokens=12, ignore_eos=True))
    for prompt, tokens in zip(prompts, out):
        assert tokens == _greedy(cfg, w, prompt, 12)
    engine.runner.cache.check()
    assert not engine.runner.cache.requests


def test_the_replay_program_serves_a_folder(tmp_path):
    from transformers_neuronx_amd.weights import write_random_model
    cfg = sc.config("c")
    folder = write_random_model(cfg, str(tmp_path / "m"), 12, dtype="bfloat16")
    from safetensors.torch import load_file
    w = load_file(os.path.join(folder, "model.safetensors"))
    requests = sc.requests(cfg, [40, 9, 70, 3, 25], 13)
    expected = _expected(cfg, w, requests)
    steps, place = schedules.mixed(requests, max_tokens=192, page=64, seed=1, tail=6, max_live=4)
    out_dir = tmp_path / "out"
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", "float32",
                           "--out", str(out_dir), "--max-tokens", "192"], input="\n".join(json.dumps(s) for s in steps),
                          capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [l for l in proc.stdout.splitlines() if l.startswith("done")] == [f"done {s['step']}" for s in steps]
    for (step, row), (rid, pos) in place.items():
        got = np.fromfile(out_dir / f"{step}.f32", dtype="<f4").reshape(-1, cfg.vocab)[row]
        want = expected[rid][pos].numpy()
        assert np.abs(got - want).max() / np.abs(expected[rid].numpy()).max() < TOL


def test_the_command_line_serves_the_folder(tmp_path, capsys):
    """`opt_demo save --random --config` writes a folder of whatever architecture the config.json names, and
    `run --benchmark --profile` generates from it and times its kernels."""
    from transformers_neuronx_amd.opt import demo
    with open(tmp_path / "config.json", "w") as fp:
        json.dump(dict(sc.CASES["d"], init_std=0.3), fp)
    folder = str(tmp_path / "model")
    assert demo.main(["--amp", "bf16", "save", folder, "--random", "--config", str(tmp_path / "config.json")]) in (0, None)
    assert demo.main(["--amp", "bf16", "run", folder, "--batch_size", "2", "--n_positions", "40", "--prompt_len", "9",
                      "--top_k", "1", "--benchmark", "--profile", "--page_size", "16"]) in (0, None)
    text = capsys.readouterr().out
    assert "running SunatarForSampling.from_pretrained" in text
    report = json.loads(next(line for line in text.splitlines() if line.startswith("{")))
    assert report["inferences"] == 10 and report["e2e_output_token_throughput"] > 0
    for kernel in ("tnx_qkv_prepare", "tnx_matrix_memory", "tnx_expert_mixture", "tnx_route", "tnx_gated_activation"):
        assert kernel in text, kernel


@pytest.mark.parametrize("dtype,tol", [("float32", TOL), ("bfloat16", 6e-2)])
@pytest.mark.parametrize("seed", range(12))
def test_configurations_drawn_from_a_seed(seed, dtype, tol):
    cfg = sc.drawn(seed)
    w = sc.weights(cfg, seed, torch.bfloat16 if dtype == "bfloat16" else torch.float32)
    runner = sc.runner(cfg, w, dtype=dtype, kernels="hip", device=DEV, max_tokens=176)
    requests = sc.requests(cfg, [70, 33, 5, 1], seed)
    expected = _expected(cfg, w, requests)
    few = 0.15 if dtype == "bfloat16" else 0.0
    step_through(runner, expected, schedules.mixed(requests, max_tokens=176, page=16, seed=5, tail=8, max_live=3), tol, few)
    step_through(runner, expected, schedules.head_then_singles(requests, tail=20), tol, few)
