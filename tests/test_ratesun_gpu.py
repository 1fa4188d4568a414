"""Ratesun on the GPU: every kernel of its parts alone against the plain implementation's function of the same
mechanism (float32 and bfloat16), attention with keys made to stand out far away, at page borders and just
inside and outside the window, state and pages that change hands, the engine under every way of cutting,
recorded decoding, generation through the entry point, and the replay program."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_ratesun as P
import ratesun_cases as rc
import schedules
from test_ratesun_cpu import _expected, _greedy, step_through
from transformers_neuronx_amd.engine import StepEntry
from transformers_neuronx_amd.engine.batch import build_context

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DTYPES = [("float32", torch.float32, 3e-6), ("bfloat16", torch.bfloat16, 1.2e-2)]


def _ops(dtype):
    from transformers_neuronx_amd.kernels import make_ops
    return make_ops("hip", dtype, DEV)


def _ctx(runs, cached, slots, tables=None, page_size=16):
    """A step of runs of `runs` tokens for requests that hold `cached` tokens, in state slots `slots`."""
    entries = [StepEntry(i, [0] * n, []) for i, n in enumerate(runs)]
    tables = tables if tables is not None else {}
    return build_context(entries, cached, slots, {k: np.asarray(v, dtype=np.int32) for k, v in tables.items()},
                         page_size, DEV)


def _close(got, want, tol):
    want = want.to(torch.float64)
    err = float((got.double().cpu() - want).abs().max() / max(1e-30, float(want.abs().max())))
    assert err < tol, err


# ---------------------------------------------------------------- each mechanism alone

@pytest.mark.parametrize("name,dtype,tol", DTYPES)
def test_pair_table_rows_and_the_token_kept_between_steps(name, dtype, tol):
    ops = _ops(dtype)
    g = torch.Generator().manual_seed(0)
    vocab, width, buckets, mp, mc = 50, 36, 7, 1000003, 999983        # multipliers that overflow 32 bits with the ids
    table = torch.randn(vocab, width, generator=g).to(dtype)
    pairs = torch.randn(buckets + 1, width, generator=g).to(dtype)
    seqs = {0: torch.randint(0, vocab, (9,), generator=g).tolist(), 1: torch.randint(0, vocab, (4,), generator=g).tolist()}
    want = {k: table.double()[torch.tensor(s)] + pairs.double()[torch.tensor(P.bigram_rows(s, buckets, mp, mc))] for k, s in seqs.items()}
    state = torch.full((3, 2), 12345, dtype=torch.int32, device=DEV)          # what a former holder left
    # request 0 in slot 2: 3 tokens, then 1, then 5; request 1 in slot 0 joins at the second step, whole
    cuts = [([(0, 0, 3)]), ([(0, 3, 4), (1, 0, 4)]), ([(0, 4, 9)])]
    for step in cuts:
        ids = torch.tensor(sum((seqs[r][a:b] for r, a, b in step), []), dtype=torch.int32, device=DEV)
        ctx = _ctx([b - a for _, a, b in step], [a for _, a, _ in step], [2 if r == 0 else 0 for r, _, _ in step])
        out = ops.embed_pairs(ids, table.to(DEV), pairs.to(DEV), buckets, mp, mc, ctx, state)
        at = 0
        for r, a, b in step:
            _close(out[at:at + b - a], want[r][a:b], 1e-6)
            at += b - a
    # a token id -1 - k stands for the token kept on the device for slot k
    kept = torch.tensor([0, 0, seqs[0][4]], dtype=torch.int32, device=DEV)
    state[2] = torch.tensor([0, seqs[0][3]], dtype=torch.int32)
    out = ops.embed_pairs(torch.tensor([-3], dtype=torch.int32, device=DEV), table.to(DEV), pairs.to(DEV), buckets, mp, mc,
                          _ctx([1], [4], [2]), state, kept)
    _close(out, want[0][4:5], 1e-6)


@pytest.mark.parametrize("center", [True, False])
@pytest.mark.parametrize("width", [50, 256, 1031])
def test_norm_that_joins_a_part_to_the_stream(width, center):
    ops = _ops(torch.float32)
    g = torch.Generator().manual_seed(1)
    y, x = torch.randn(7, width, generator=g) * 3 + 1, torch.randn(7, width, generator=g)
    w, b = torch.randn(width, generator=g), torch.randn(width, generator=g)
    if center:
        want = x.double() + 0.3 * P.layer_norm(y.double(), w.double(), b.double(), 1e-5)
    else:
        want = x.double() + 0.3 * P.rms_norm(y.double(), w.double(), 1e-5)
    out = torch.empty(7, width, device=DEV)
    got = ops.norm_add(y.to(DEV), w.to(DEV), b.to(DEV) if center else None, 1e-5, center, x.to(DEV), 0.3, out)
    assert got.data_ptr() == out.data_ptr()
    _close(got, want, 2e-6)


@pytest.mark.parametrize("name,dtype,tol", DTYPES)
@pytest.mark.parametrize("taps", [1, 2, 3, 5])
def test_input_convolution_across_steps_of_any_length(name, dtype, tol, taps):
    ops = _ops(dtype)
    g = torch.Generator().manual_seed(2)
    width = 70
    w = torch.randn(width, taps, generator=g)
    h = {0: torch.randn(23, width, generator=g), 1: torch.randn(6, width, generator=g)}
    want = {k: P.input_conv(v.double(), w.double()) for k, v in h.items()}
    state = torch.full((3, 2, taps, width), 7.0, device=DEV) if taps > 1 else None
    if state is not None:
        state[1].zero_()       # a request's slot is cleared when it gets it
        state[2].zero_()
    # request 0 (slot 1, convolution 1 of 2): 1, 1, 2, 4, 1, 14 tokens; request 1 (slot 2) beside it from the third step
    cuts0 = [0, 1, 2, 4, 8, 9, 23]
    cuts1 = [None, None, 0, 5, 6]
    for s in range(len(cuts0) - 1):
        step = [(0, cuts0[s], cuts0[s + 1], 1)]
        if s + 1 < len(cuts1) and cuts1[s] is not None:
            step.append((1, cuts1[s], cuts1[s + 1], 2))
        rows = torch.cat([h[r][a:b] for r, a, b, _ in step]).to(DEV)
        ctx = _ctx([b - a for _, a, b, _ in step], [a for _, a, _, _ in step], [slot for _, _, _, slot in step])
        out = ops.input_conv(rows, w.to(DEV), state, 1, ctx, dtype)
        # a single-token step run again reads the same (what a recorded step does before its first replay)
        if all(b - a == 1 for _, a, b, _ in step):
            again = ops.input_conv(rows, w.to(DEV), state, 1, ctx, dtype)
            assert torch.equal(out, again)
        at = 0
        for r, a, b, _ in step:
            _close(out[at:at + b - a], want[r][a:b], tol)
            at += b - a
    if state is not None:
        assert float(state[0].min()) == 7.0 and float(state[1, 0].abs().max()) == 0.0     # nobody else's places


@pytest.mark.parametrize("name,dtype,tol", DTYPES)
@pytest.mark.parametrize("taps,width,joined", [(1, 64, True), (2, 72, False), (3, 2052, True), (4, 128, True), (5, 70, True),
                                               (4, 4100, False)])
def test_norm_and_convolution_in_one_launch(name, dtype, tol, taps, width, joined):
    """The part before joins the stream, the norm and the convolution follow, across steps cut anywhere; widths
    that the one-launch kernel takes and one that it does not."""
    ops = _ops(dtype)
    g = torch.Generator().manual_seed(6)
    w = torch.randn(width, taps, generator=g)
    pre_w, pre_b, post_w = torch.randn(width, generator=g), torch.randn(width, generator=g), torch.randn(width, generator=g)
    lens = {0: 23, 1: 6}
    x = {k: torch.randn(n, width, generator=g) for k, n in lens.items()}
    y = {k: torch.randn(n, width, generator=g) * 3 for k, n in lens.items()}
    want_x = {k: (x[k].double() + 0.3 * P.rms_norm(y[k].double(), post_w.double(), 1e-5)) if joined else x[k].double() for k in x}
    want = {k: P.input_conv(P.layer_norm(want_x[k], pre_w.double(), pre_b.double(), 1e-5), w.double()) for k in x}
    state = torch.full((3, 2, taps, width), 7.0, device=DEV) if taps > 1 else None
    if state is not None:
        state[1:].zero_()
    cuts0, cuts1 = [0, 1, 2, 4, 8, 9, 23], [None, None, 0, 5, 6]
    for s_ in range(len(cuts0) - 1):
        step = [(0, cuts0[s_], cuts0[s_ + 1], 1)]
        if s_ + 1 < len(cuts1) and cuts1[s_] is not None:
            step.append((1, cuts1[s_], cuts1[s_ + 1], 2))
        xs = torch.cat([x[r][a:b] for r, a, b, _ in step]).to(DEV)
        ys = torch.cat([y[r][a:b] for r, a, b, _ in step]).to(DEV)
        ctx = _ctx([b - a for _, a, b, _ in step], [a for _, a, _, _ in step], [slot for _, _, _, slot in step])
        join = (ys, post_w.to(DEV), None, False, 0.3) if joined else None
        got_x, out = ops.join_norm_conv(xs, join, (pre_w.to(DEV), pre_b.to(DEV), True, 1e-5), w.to(DEV), state, 0, ctx, dtype)
        if all(b - a == 1 for _, a, b, _ in step):          # run again, as a recorded step is: the same
            _, again = ops.join_norm_conv(xs, join, (pre_w.to(DEV), pre_b.to(DEV), True, 1e-5), w.to(DEV), state, 0, ctx, dtype)
            assert torch.equal(out, again)
        at = 0
        for r, a, b, _ in step:
            _close(out[at:at + b - a], want[r][a:b], max(tol, 3e-6))
            _close(got_x[at:at + b - a], want_x[r][a:b], 3e-6)
            at += b - a
    if state is not None:
        assert float(state[0].min()) == 7.0 and float(state[1, 1].abs().max()) == 0.0


def test_norm_that_joins_leaves_a_copy_for_the_next_product():
    ops = _ops(torch.bfloat16)
    g = torch.Generator().manual_seed(1)
    for width in (64, 1028, 4096, 30):
        y, x, w = torch.randn(5, width, generator=g), torch.randn(5, width, generator=g), torch.randn(width, generator=g)
        out, copy = ops.norm_add(y.to(DEV), w.to(DEV), None, 1e-5, False, x.to(DEV), 0.5, None, want_compute=True)
        _close(out, x.double() + 0.5 * P.rms_norm(y.double(), w.double(), 1e-5), 3e-6)
        assert copy.dtype == torch.bfloat16 and torch.equal(copy, out.to(torch.bfloat16))


@pytest.mark.parametrize("name,dtype,tol", DTYPES)
def test_normed_powers_columns_and_the_average_over_depth(name, dtype, tol):
    ops = _ops(dtype)
    g = torch.Generator().manual_seed(3)
    coeffs = torch.tensor([0.7, -1.3, 0.4, 0.25])
    for inner in (333, 320, 5000, 16384, 16388):
        z = torch.randn(5, inner, generator=g) * 2
        _close(ops.poly_norm(z.to(DEV), coeffs.to(DEV), 1e-5), P.poly_norm(z.double(), coeffs.double(), 1e-5), tol)
    gate, rows = torch.randn(5, 6, generator=g).to(dtype), torch.randn(5, 30, generator=g).to(dtype)
    _close(ops.mul_columns(gate.to(DEV), rows.to(DEV), 18), gate.double() * rows.double()[:, 18:24], tol)
    hist = torch.randn(6, 5, 77, generator=g)
    wts = torch.randn(6, generator=g)
    _close(ops.weighted_sum(hist.to(DEV), wts.to(DEV), 4), sum(wts[j].double() * hist[j].double() for j in range(4)), 2e-6)


@pytest.mark.parametrize("name,dtype,tol", DTYPES)
@pytest.mark.parametrize("sizes", [(3, 10, 18, 7), (4, 64, 128, 33), (1, 128, 48, 130), (16, 32, 512, 1)])
def test_product_per_head(name, dtype, tol, sizes):
    heads, k, n, tokens = sizes
    ops = _ops(dtype)
    g = torch.Generator().manual_seed(4)
    x = torch.randn(tokens, heads, k + 5, generator=g).to(dtype)
    w = torch.randn(heads, n, k, generator=g).to(dtype)
    got = ops.batched_linear(x.to(DEV)[:, :, :k], w.to(DEV), alpha=0.37)
    _close(got, 0.37 * torch.einsum("thk,hnk->thn", x.double()[:, :, :k], w.double()), tol)


@pytest.mark.parametrize("name,dtype,tol", DTYPES)
def test_latent_norms_and_their_pages(name, dtype, tol):
    ops = _ops(dtype)
    g = torch.Generator().manual_seed(5)
    Q, R, r, pairs, ps = 22, 18, 6, 2, 16
    down = torch.randn(9, Q + R + r, generator=g) * 2
    qw, kw = torch.randn(Q, generator=g), torch.randn(R, generator=g)
    freqs = (50.0 ** (-2.0 * torch.arange(pairs, dtype=torch.float64) / (2 * pairs))).float()
    lat = torch.zeros(5, ps, R, dtype=dtype, device=DEV)
    rot = torch.zeros(5, ps, r, dtype=dtype, device=DEV)
    across = torch.zeros(5, R, ps, dtype=dtype, device=DEV)
    # one request of 9 tokens from position 12 on: crosses from page 3 into page 1
    ctx = _ctx([9], [12], [0], {"g": [[3, 1, 4]]}, ps)
    c_q = ops.latent_norms(down.to(DEV), Q, R, r, qw.to(DEV), kw.to(DEV), 1e-5, freqs.to(DEV), ctx, ctx.groups["g"], lat, rot, across)
    _close(c_q, P.rms_norm(down.double()[:, :Q], qw.double(), 1e-5), tol)
    stored = torch.cat([lat[3, 12:], lat[1, :5]])
    _close(stored, P.rms_norm(down.double()[:, Q:Q + R], kw.double(), 1e-5), tol)
    turned = P.rotate_pairs(down.double()[:, Q + R:], torch.arange(12, 21), 50.0, 2 * pairs)
    _close(torch.cat([rot[3, 12:], rot[1, :5]]), turned, tol)
    assert float(lat[[0, 2, 4]].abs().max()) == 0 and float(lat[1, 5:].abs().max()) == 0
    assert torch.equal(across.transpose(1, 2), lat)          # the same latents, a page's tokens side by side


def _attention_case(dtype, heads, n, r, R, window, length, run, ps, standout, seed):
    """Queries of the last `run` tokens of a request of `length` tokens over pages in a scrambled order. Key
    `standout` (a position) is made to dominate the scores of the last query, if it can see it."""
    g = torch.Generator().manual_seed(seed)
    c = torch.randn(length, R, generator=g).to(dtype)
    kr = torch.randn(length, r, generator=g).to(dtype)
    q = torch.randn(run, heads, n + r, generator=g).to(dtype)
    q_lat = torch.randn(run, heads, R, generator=g).to(dtype) * 0.3
    if standout is not None:
        direction = torch.nn.functional.normalize(torch.randn(R, generator=g), dim=0)
        c[standout] = (direction * 6).to(dtype)
        q_lat[-1] = (direction * 20).to(dtype)
    blocks = -(-length // ps)
    order = torch.randperm(blocks + 3, generator=g)[:blocks].tolist()
    lat = torch.randn(blocks + 3, ps, R, generator=g).to(dtype).to(DEV) * 50          # what others left in the pages
    rot = torch.randn(blocks + 3, ps, r, generator=g).to(dtype).to(DEV) * 50
    for j in range(length):
        lat[order[j // ps], j % ps] = c[j]
        rot[order[j // ps], j % ps] = kr[j]
    return c, kr, q, q_lat, lat, rot, order, lat.transpose(1, 2).contiguous()


def _plain_attention(c, kr, q, q_lat, n, window, first, freqs_base, dims, scale):
    """The mechanism restated: scores scale * (q_lat . c + turn(q_r) . k_r) under the window, softmax, sum of c."""
    c, kr, q, q_lat = c.double(), kr.double(), q.double(), q_lat.double()
    run, length = q.shape[0], c.shape[0]
    pos = torch.arange(first, first + run)
    q_r = P.rotate_pairs(q[..., n:], pos, freqs_base, dims)
    scores = (torch.einsum("ihd,jd->hij", q_lat, c) + torch.einsum("ihd,jd->hij", q_r, kr)) * scale
    i, j = pos[:, None], torch.arange(length)[None, :]
    seen = (j <= i) & ((i - j < window) if window else torch.ones_like(j <= i))
    prob = torch.softmax(scores.masked_fill(~seen[None], float("-inf")), dim=-1)
    return torch.einsum("hij,jd->ihd", prob, c), prob


@pytest.mark.parametrize("name,dtype,tol", DTYPES)
@pytest.mark.parametrize("case", [
    # heads, n, r, R, window, length, run, page, standout position (relative to the last query: 0 is itself)
    dict(heads=3, n=8, r=6, R=18, window=40, length=300, run=1, ps=16, back=39),     # just inside the window
    dict(heads=3, n=8, r=6, R=18, window=40, length=300, run=1, ps=16, back=40),     # just outside
    dict(heads=2, n=16, r=4, R=24, window=0, length=700, run=1, ps=16, back=697),    # far away, no window
    dict(heads=2, n=16, r=4, R=24, window=0, length=700, run=37, ps=16, back=699),   # the very first token, in a portion
    dict(heads=5, n=4, r=2, R=10, window=17, length=64, run=64, ps=16, back=16),     # a whole prompt, edge of the window
    dict(heads=1, n=32, r=16, R=64, window=33, length=129, run=2, ps=64, back=32),   # a page border: position 96 = 128 - 32
    dict(heads=4, n=8, r=8, R=300, window=1, length=50, run=3, ps=16, back=0),       # a window of one token
    dict(heads=2, n=8, r=4, R=20, window=300, length=280, run=5, ps=16, back=279),   # a window wider than the request
    # sizes the matrix unit takes (in bfloat16): latents in 16s, rotated parts in 8s
    dict(heads=3, n=8, r=8, R=48, window=40, length=300, run=1, ps=16, back=39),
    dict(heads=3, n=8, r=8, R=48, window=40, length=300, run=1, ps=16, back=40),
    dict(heads=20, n=16, r=16, R=80, window=0, length=700, run=1, ps=64, back=697),  # 20 heads: two blocks of columns
    dict(heads=2, n=16, r=24, R=160, window=0, length=700, run=37, ps=16, back=699),
    dict(heads=5, n=8, r=8, R=16, window=17, length=64, run=64, ps=16, back=16),
    dict(heads=2, n=32, r=16, R=64, window=33, length=300, run=200, ps=64, back=32),  # several tiles of queries
    dict(heads=1, n=32, r=64, R=512, window=33, length=129, run=2, ps=64, back=32),
    dict(heads=17, n=8, r=8, R=272, window=100, length=290, run=1, ps=32, back=99),
])
@pytest.mark.parametrize("kernel", ["shared", "alone", "any"])
def test_attention_finds_the_key_that_stands_out(name, dtype, tol, case, kernel):
    """`kernel`: bfloat16 on the matrix unit with a block's waves sharing a tile, or each walking the keys alone
    (prompt runs), or the kernel for any sizes, which is also float32's."""
    if kernel != "any" and dtype == torch.float32:
        pytest.skip("float32 has the one kernel")
    ops = _ops(dtype)
    ops.latent_matrix_unit = kernel != "any"
    ops.latent_prompt_kind = 1 if kernel == "alone" else 0
    heads, n, r, R, window, length, run, ps = (case[k] for k in ("heads", "n", "r", "R", "window", "length", "run", "ps"))
    standout = length - 1 - case["back"]
    c, kr, q, q_lat, lat, rot, order, across = _attention_case(dtype, heads, n, r, R, window, length, run, ps, standout, 7)
    dims, base, scale = r - 2 if r > 2 else r, 321.0, 0.4
    from transformers_neuronx_amd.kernels.attention_plan import attention_plan
    freqs = (base ** (-2.0 * torch.arange(dims // 2, dtype=torch.float64) / dims)).float().to(DEV)
    want, prob = _plain_attention(c, kr, q, q_lat, n, window, length - run, base, dims, scale)
    visible = not window or case["back"] < window
    if case["back"] > 0 or window == 1:
        assert (float(prob[:, -1, standout].min()) > 0.9) == visible
    entries = [StepEntry(0, [0] * run, [])]
    ctx = build_context(entries, [length - run], [0], {"g": np.asarray([order], dtype=np.int32)}, ps, DEV,
                        {"attention": attention_plan})
    got = ops.latent_attention(q.reshape(run, -1).to(DEV), q_lat.to(DEV), heads, n, r, R, freqs, scale, ctx,
                               ctx.groups["g"], lat, rot, across, window or None)
    # float32: an angle is position * frequency in float32, which at position 700 is 4e-5 of a turn's radian off
    # the float64 angle, and the scores here are large
    _close(got, want, max(tol, 4e-5))


# ---------------------------------------------------------------- the engine

@pytest.mark.parametrize("dtype,tol", [("float32", 2e-5), ("bfloat16", 6e-2)])
@pytest.mark.parametrize("name", sorted(rc.CASES))
def test_schedules_on_the_gpu(name, dtype, tol):
    cfg = rc.config(name)
    w = rc.weights(cfg, 3, torch.bfloat16 if dtype == "bfloat16" else torch.float32)
    runner = rc.runner(cfg, w, dtype=dtype, kernels="hip", device=DEV, max_tokens=208)
    requests = rc.requests(cfg, [70, 33, 5, 100, 1], 1)
    expected = _expected(cfg, w, requests)
    for made in (schedules.whole(requests), schedules.head_then_singles(requests, tail=12), schedules.portions(requests),
                 schedules.portions(requests, sizes=(2, 2, 3, 2, 16, 2, 15, 17, 2)),
                 schedules.mixed(requests, max_tokens=208, page=16, seed=5, tail=8, max_live=3),
                 schedules.only_last(schedules.mixed(requests, max_tokens=208, page=16, seed=6, tail=20, max_live=4))):
        step_through(runner, expected, made, tol)
    from transformers_neuronx_amd.kernels import hip
    assert {"stream", "latent", "gemm"} <= set(hip.loaded_libraries())


@pytest.mark.parametrize("graphs", [True, False])
def test_long_decoding_recorded_and_not(graphs):
    """300 tokens one by one beside a second request that joins and leaves: windows pass over decoded tokens,
    pages go back, the batch size changes (a recorded step is made for each), slots change hands."""
    cfg = rc.config("d")
    w = rc.weights(cfg, 8)
    runner = rc.runner(cfg, w, dtype="float32", kernels="hip", device=DEV, max_tokens=512, page_size=16, use_graphs=graphs)
    requests = rc.requests(cfg, [320, 90, 60], 9)
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
        assert float((have.double().cpu() - expected[rid]).abs().max() / expected[rid].abs().max()) < 2e-5, rid


@pytest.mark.parametrize("amp,tol", [("f32", 2e-5), ("bf16", 6e-2)])
def test_generation_through_the_entry_point(tmp_path, amp, tol):
    from safetensors.torch import load_file
    from transformers_neuronx_amd import NeuronAutoModelForCausalLM
    from transformers_neuronx_amd.weights import write_random_model
    cfg = rc.config("a")
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


def test_the_replay_program_serves_a_folder(tmp_path):
    from transformers_neuronx_amd.weights import write_random_model
    cfg = rc.config("c")
    folder = write_random_model(cfg, str(tmp_path / "m"), 12, dtype="bfloat16")
    from safetensors.torch import load_file
    w = load_file(os.path.join(folder, "model.safetensors"))
    requests = rc.requests(cfg, [40, 9], 13)
    expected = _expected(cfg, w, requests)
    steps, place = schedules.mixed(requests, max_tokens=128, page=64, seed=1, tail=6, max_live=2)
    out_dir = tmp_path / "out"
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", "float32",
                           "--out", str(out_dir), "--max-tokens", "128"], input="\n".join(json.dumps(s) for s in steps),
                          capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [l for l in proc.stdout.splitlines() if l.startswith("done")] == [f"done {s['step']}" for s in steps]
    for (step, row), (rid, pos) in place.items():
        got = np.fromfile(out_dir / f"{step}.f32", dtype="<f4").reshape(-1, cfg.vocab)[row]
        want = expected[rid][pos].numpy()
        assert np.abs(got - want).max() / np.abs(expected[rid].numpy()).max() < 2e-5


def test_the_command_line_serves_the_folder(tmp_path, capsys):
    """`opt_demo save --random --config` writes a folder of whatever architecture the config.json names, and
    `run --benchmark --profile` generates from it and times its kernels."""
    from transformers_neuronx_amd.opt import demo
    with open(tmp_path / "config.json", "w") as fp:
        json.dump(dict(rc.CASES["d"], init_std=0.3), fp)
    folder = str(tmp_path / "model")
    assert demo.main(["--amp", "bf16", "save", folder, "--random", "--config", str(tmp_path / "config.json")]) in (0, None)
    assert demo.main(["--amp", "bf16", "run", folder, "--batch_size", "2", "--n_positions", "40", "--prompt_len", "9",
                      "--top_k", "1", "--benchmark", "--profile", "--page_size", "16"]) in (0, None)
    text = capsys.readouterr().out
    assert "running RatesunForSampling.from_pretrained" in text
    report = json.loads(next(line for line in text.splitlines() if line.startswith("{")))
    assert report["inferences"] == 10 and report["e2e_output_token_throughput"] > 0
    for kernel in ("tnx_join_norm_conv", "tnx_latent_attention_mfma", "tnx_batched_linear", "tnx_poly_norm", "tnx_embed_pairs"):
        assert kernel in text, kernel


@pytest.mark.parametrize("dtype,tol", [("float32", 2e-5), ("bfloat16", 6e-2)])
@pytest.mark.parametrize("seed", range(12))
def test_configurations_drawn_from_a_seed(seed, dtype, tol):
    cfg = rc.drawn(seed)
    w = rc.weights(cfg, seed, torch.bfloat16 if dtype == "bfloat16" else torch.float32)
    runner = rc.runner(cfg, w, dtype=dtype, kernels="hip", device=DEV, max_tokens=176)
    requests = rc.requests(cfg, [70, 33, 5, 1], seed)
    expected = _expected(cfg, w, requests)
    few = 0.03 if dtype == "bfloat16" else 0.0
    step_through(runner, expected, schedules.mixed(requests, max_tokens=176, page=16, seed=5, tail=8, max_live=3), tol, few)
    step_through(runner, expected, schedules.head_then_singles(requests, tail=20), tol, few)


@pytest.mark.parametrize("case", [
    dict(heads=3, n=16, r=8, v=32, R=48, window=40, length=300, run=150, ps=16, back=39),
    dict(heads=3, n=16, r=8, v=32, R=48, window=40, length=300, run=150, ps=16, back=40),
    dict(heads=2, n=64, r=32, v=64, R=128, window=0, length=700, run=300, ps=64, back=699),
    dict(heads=5, n=8, r=8, v=16, R=24, window=17, length=64, run=64, ps=16, back=16),
    dict(heads=1, n=128, r=64, v=128, R=512, window=100, length=400, run=130, ps=64, back=99),
    dict(heads=2, n=24, r=16, v=48, R=40, window=300, length=280, run=2, ps=16, back=279),
])
def test_prompt_attention_with_keys_and_values_made_explicitly(case):
    """bfloat16 steps of prompts' runs alone: keys W_uk c and values W_uv c of what a run can see are made from
    the cached latents and attention runs on them. One key is made to stand out for the last query."""
    from transformers_neuronx_amd.kernels.attention_plan import attention_plan
    dtype = torch.bfloat16
    ops = _ops(dtype)
    heads, n, r, v, R, window, length, run, ps = (case[k] for k in ("heads", "n", "r", "v", "R", "window", "length", "run", "ps"))
    standout = length - 1 - case["back"]
    g = torch.Generator().manual_seed(9)
    w_uk = (torch.randn(heads * n, R, generator=g) / R ** 0.5).to(dtype)
    w_uv = (torch.randn(heads * v, R, generator=g) / R ** 0.5).to(dtype)
    c = torch.randn(length, R, generator=g).to(dtype)
    kr = torch.randn(length, r, generator=g).to(dtype)
    q = torch.randn(run, heads, n + r, generator=g).to(dtype) * 0.3
    keys = (c.double() @ w_uk.double().T).view(length, heads, n)
    q[-1, :, :n] = (keys[standout] / keys[standout].norm(dim=-1, keepdim=True) * 12).to(dtype)
    c[standout] = c[standout] * 4
    blocks = -(-length // ps)
    order = torch.randperm(blocks + 3, generator=g)[:blocks].tolist()
    lat = torch.randn(blocks + 3, ps, R, generator=g).to(dtype).to(DEV) * 50
    rot = torch.randn(blocks + 3, ps, r, generator=g).to(dtype).to(DEV) * 50
    for j in range(length):
        lat[order[j // ps], j % ps] = c[j]
        rot[order[j // ps], j % ps] = kr[j]
    dims, base, scale = r - 2, 321.0, 0.4
    freqs = (base ** (-2.0 * torch.arange(dims // 2, dtype=torch.float64) / dims)).float().to(DEV)
    # the mechanism restated with keys and values made explicitly, in float64
    cd, pos = c.double(), torch.arange(length - run, length)
    keys = (cd @ w_uk.double().T).view(length, heads, n)
    vals = (cd @ w_uv.double().T).view(length, heads, v)
    q_r = P.rotate_pairs(q.double()[..., n:], pos, base, dims)
    scores = (torch.einsum("ihd,jhd->hij", q.double()[..., :n], keys) + torch.einsum("ihd,jd->hij", q_r, kr.double())) * scale
    i, j = pos[:, None], torch.arange(length)[None, :]
    seen = (j <= i) & ((i - j < window) if window else torch.ones_like(j <= i))
    prob = torch.softmax(scores.masked_fill(~seen[None], float("-inf")), dim=-1)
    want = torch.einsum("hij,jhd->ihd", prob, vals).reshape(run, heads * v)
    visible = not window or case["back"] < window
    assert (float(prob[:, -1, standout].min()) > 0.9) == visible
    ctx = build_context([StepEntry(0, [0] * run, [])], [length - run], [0], {"g": np.asarray([order], dtype=np.int32)}, ps, DEV,
                        {"attention": attention_plan})
    ops.expand_rows = 2
    assert ops.latent_expands(ctx, n, r, v, R)
    got = ops.latent_attention_expanded(q.reshape(run, -1).to(DEV), w_uk.to(DEV), w_uv.to(DEV), heads, n, r, v, R, freqs, scale,
                                        ctx, ctx.groups["g"], lat, rot, window or None)
    _close(got, want, 2e-2)


@pytest.mark.parametrize("name", ["d"])
def test_schedules_with_expanded_prompt_steps(name):
    """The engine in bfloat16 with every step of prompts' runs alone on the expanded keys and values."""
    cfg = rc.config(name)
    w = rc.weights(cfg, 3, torch.bfloat16)
    runner = rc.runner(cfg, w, dtype="bfloat16", kernels="hip", device=DEV, max_tokens=400)
    runner.ops.expand_rows = 2
    requests = rc.requests(cfg, [170, 33, 5, 100, 2], 1)
    expected = _expected(cfg, w, requests)
    for made in (schedules.whole(requests), schedules.portions(requests),
                 schedules.mixed(requests, max_tokens=400, page=16, seed=5, tail=8, max_live=3)):
        step_through(runner, expected, made, 6e-2)
