"""Small Sunatar configurations of the tests' own, their random weights, and the runner that serves them.
The sizes differ between the cases in everything that can differ: head counts of 1 and more, grouped and
ungrouped key/value heads, value heads smaller and larger than query heads, windows of 1, of less and of more than
a page and none, rotations of a part of a head and of all of it with and without scaled frequencies, layers that
blend values and layers that do not (the first blending layer not the first layer), matrix memories first, last
and side by side, one expert a token and several, with and without a shared expert, layers without a
feed-forward, widths that are multiples of nothing."""
import random

import torch

from transformers_neuronx_amd.config import EngineConfig
from transformers_neuronx_amd.engine.factory import build_runner
from transformers_neuronx_amd.engine.model import model_param_decls
from transformers_neuronx_amd.sunatar import SunatarConfig, sunatar_spec
from transformers_neuronx_amd.weights.loader import TensorDict
from transformers_neuronx_amd.weights.random_init import random_tensors


def attention(heads, kv_heads, dim, vdim, window, scale, rot_dims, base, scaling=None, v_mix=False):
    m = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale, v_mix=v_mix,
             rot=dict(base=base, dims=rot_dims))
    if scaling:
        m["rot"]["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    if window is not None:
        m["mask"] = dict(size=window)
    return "attention", m


def memory(heads, dim, vdim, cap):
    return "mlstm", dict(heads=heads, dim=dim, vdim=vdim, gate_cap=cap)


def moe(experts, top, ff, shared):
    d = dict(kind="moe", router=dict(experts=experts, top=top), expert=dict(ff=ff))
    if shared:
        d["shared"] = dict(ff=shared)
    return d


def layer(mixer, mlp):
    return dict(type=mixer[0], mixer=mixer[1], mlp=mlp)


CASES = {
    # a memory between attention layers; values blended from the second layer on; two experts a token
    "a": dict(architecture="Sunatar", vocab=211, width=96, norm=dict(eps=1e-4), embedding=dict(scale=3.0),
              layers=[layer(attention(3, 3, 16, 24, None, 0.3, 8, 1000.0), moe(5, 2, 40, 24)),
                      layer(attention(4, 2, 32, 16, 24, 0.2, 32, 1000.0, (8.0, 1.0, 4.0, 64), v_mix=True), moe(5, 2, 40, 24)),
                      layer(memory(3, 8, 40, 6.0), moe(7, 3, 24, 0)),
                      layer(attention(2, 2, 16, 16, 50, 0.15, 4, 77.0, v_mix=True), None),
                      layer(attention(8, 2, 8, 16, 9, 0.4, 8, 77.0, (2.0, 0.5, 3.0, 16), v_mix=True), moe(3, 1, 56, 8))]),
    # memories alone at both ends; windows of 1, of exactly a page and of one more; no scale at the input
    "b": dict(architecture="Sunatar", vocab=130, width=64, norm=dict(eps=1e-6),
              layers=[layer(memory(1, 16, 16, 15.0), moe(4, 4, 16, 0)),
                      layer(attention(1, 1, 16, 16, 1, 0.25, 2, 10.0, v_mix=True), moe(2, 1, 48, 48)),
                      layer(attention(2, 1, 16, 16, 16, 0.11, 16, 50000.0, v_mix=True), moe(9, 2, 72, 0)),
                      layer(attention(4, 4, 8, 12, 17, 0.4, 6, 300.0), None),
                      layer(memory(4, 4, 8, 1.5), moe(6, 1, 40, 16))]),
    # sizes that are multiples of nothing; memories side by side
    "c": dict(architecture="Sunatar", vocab=77, width=50, norm=dict(eps=1e-5), embedding=dict(scale=0.5),
              layers=[layer(attention(3, 1, 10, 14, 33, 0.2, 6, 123.0, (3.0, 2.0, 9.0, 40)), moe(3, 2, 30, 10)),
                      layer(memory(2, 6, 10, 30.0), moe(5, 1, 26, 0)),
                      layer(memory(5, 10, 6, 8.0), None),
                      layer(attention(2, 2, 20, 6, 5, 0.1, 20, 9.0, v_mix=True), moe(8, 8, 12, 34))]),
    # sizes the matrix-unit kernels take: multiples of 16 and 128
    "d": dict(architecture="Sunatar", vocab=320, width=128, norm=dict(eps=1e-5), embedding=dict(scale=8.0),
              layers=[layer(attention(4, 2, 32, 32, 70, 0.17, 16, 20000.0, (6.0, 1.0, 8.0, 32), v_mix=True), moe(8, 2, 64, 128)),
                      layer(memory(2, 64, 64, 12.0), moe(8, 2, 64, 128)),
                      layer(attention(8, 2, 16, 32, 40, 0.14, 16, 20000.0, v_mix=True), moe(16, 4, 32, 64)),
                      layer(attention(2, 2, 64, 32, None, 0.1, 32, 500.0, v_mix=True), moe(4, 1, 128, 0))]),
}


def config(name) -> SunatarConfig:
    return SunatarConfig.from_dict(dict(CASES[name], init_std=0.35))


def weights(cfg, seed, storage=torch.float32):
    """Random tensors by checkpoint name (matrices in `storage`), made lively: wide enough that no part drowns,
    blending weights that are neither 0 nor 1, gates that open and close."""
    w = random_tensors(model_param_decls(sunatar_spec(cfg)), cfg.init_std, seed, storage)
    g = torch.Generator().manual_seed(seed + 1000)
    for k in list(w):
        last = k.rsplit(".", 1)[-1]
        if last in ("q", "k", "v", "o", "g", "gate", "up", "down", "head"):
            w[k] = (w[k].float() * (1.5 / w[k].shape[1] ** 0.5 / cfg.init_std)).to(w[k].dtype)
        elif last in ("i", "f", "router"):
            w[k] = (w[k].float() * (4.0 / w[k].shape[1] ** 0.5 / cfg.init_std)).to(w[k].dtype)
        elif last == "vmix":
            w[k] = torch.rand((), generator=g) * 0.6 + 0.2
    return w


def runner(cfg, w, dtype="float32", kernels="reference", device="cpu", page_size=16, max_tokens=256, max_seqs=4,
           use_graphs=True):
    ecfg = EngineConfig(dtype=dtype, page_size=page_size, max_tokens=max_tokens, max_num_seqs=max_seqs, device=device,
                        kernels=kernels, use_graphs=use_graphs)
    return build_runner(cfg, TensorDict({k: v.clone() for k, v in w.items()}), ecfg)


def requests(cfg, lengths, seed):
    g = torch.Generator().manual_seed(seed)
    return {f"r{i}": torch.randint(0, cfg.vocab, (n,), generator=g).tolist() for i, n in enumerate(lengths)}


def drawn(seed: int) -> SunatarConfig:
    """A configuration drawn from a seed: any sizes, any order of the two kinds of layers, with and without a
    feed-forward, windows from 1 token to none."""
    rnd = random.Random(seed)
    width = rnd.choice([24, 36, 64, 100, 128, 256])
    n_layers = rnd.randint(1, 5)
    layers = []
    blended = None        # (kv_heads, vdim) of the layers that blend
    for i in range(n_layers):
        if rnd.random() < 0.65:
            groups = rnd.choice([1, 2, 3])
            heads = groups * rnd.choice([1, 2, 4])
            dim = rnd.choice([4, 8, 10, 16, 32, 64])
            vdim = rnd.choice([4, 6, 16, 24, 48, 64])
            mix = rnd.random() < 0.7
            if mix:
                if blended is None:
                    blended = (groups, vdim)
                else:
                    groups, vdim = blended
                    heads = groups * rnd.choice([1, 2, 4])
            rot = rnd.choice([d for d in (2, 4, 8, 10, 16, 32, 64) if d <= dim and d % 2 == 0] or [dim - dim % 2])
            scaling = rnd.choice([None, (rnd.choice([2.0, 4.0, 8.0]), rnd.choice([0.5, 1.0]), rnd.choice([2.0, 4.0]), rnd.choice([8, 32, 2048]))])
            mixer = attention(heads, groups, dim, vdim, rnd.choice([None, 1, 2, 7, 16, 17, 31, 48, 64, 65, 90]),
                              rnd.uniform(0.05, 0.4), rot, rnd.choice([10.0, 500.0, 10000.0, 1e6]), scaling, v_mix=mix)
        else:
            mixer = memory(rnd.randint(1, 5), rnd.choice([4, 6, 16, 32, 40]), rnd.choice([4, 10, 16, 48, 80]),
                           rnd.choice([1.0, 5.0, 12.0, 30.0]))
        mlp = None
        if rnd.random() < 0.8 or n_layers == 1:
            experts = rnd.choice([1, 2, 5, 12, 33, 70])
            mlp = moe(experts, rnd.randint(1, min(experts, 4)), rnd.choice([8, 20, 64, 72]), rnd.choice([0, 0, 16, 40]))
        layers.append(layer(mixer, mlp))
    raw = dict(architecture="Sunatar", vocab=rnd.choice([50, 97, 256, 300]), width=width,
               norm=dict(eps=rnd.choice([1e-6, 1e-5, 1e-3])), layers=layers, init_std=0.35)
    if rnd.random() < 0.8:
        raw["embedding"] = dict(scale=rnd.choice([0.25, 1.0, 4.0, 11.0]))
    return SunatarConfig.from_dict(raw)
