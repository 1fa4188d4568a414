"""Small Ratesun configurations of the tests' own, their random weights, and the runner that serves them.
The sizes differ between the cases in everything that can differ: head counts of 1 and more, windows of 1, of
less and of more than a page, a reader whose window is wider than that of the layer whose latent it reads,
layers without a feed-forward, convolutions of 1, 2, 3 and 4 taps, widths that are no multiple of 4, a rotation
that turns fewer elements than the rotated part has."""
import torch

from transformers_neuronx_amd.config import EngineConfig
from transformers_neuronx_amd.engine.factory import build_runner
from transformers_neuronx_amd.engine.model import model_param_decls
from transformers_neuronx_amd.ratesun import RatesunConfig, ratesun_spec
from transformers_neuronx_amd.weights.loader import TensorDict
from transformers_neuronx_amd.weights.random_init import random_tensors


def _mixer(heads, dim, rot_dim, vdim, kv_rank, q_rank, window, base, scale, kv_from=None, dims=None):
    m = dict(heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, kv_rank=kv_rank, q_rank=q_rank,
             rot=dict(base=base, dims=rot_dim if dims is None else dims), scale=scale)
    if window is not None:
        m["mask"] = dict(size=window)
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def _layer(mixer, ff):
    return dict(type="latent_attention", mixer=mixer, mlp=dict(kind="dense", ff=ff) if ff else None)


CASES = {
    # four layers, two latents: a reader with a wider window than its writer, a layer that sees everything
    "a": dict(architecture="Ratesun", vocab=211, width=96, norm=dict(eps=1e-4), residual_mult=0.5, logit_scale=0.7,
              canon=dict(taps=4), embedding=dict(bigram=dict(buckets=97, mul_prev=31, mul_cur=7)),
              token_side=dict(dim=8),
              layers=[_layer(_mixer(3, 16, 8, 24, 32, 40, 24, 1000.0, 0.2), 120),
                      _layer(_mixer(2, 32, 8, 16, 32, 24, 50, 1000.0, 0.15, kv_from=0), None),
                      _layer(_mixer(5, 8, 4, 8, 20, 16, None, 77.0, 0.3), 64),
                      _layer(_mixer(1, 24, 4, 40, 20, 12, 9, 77.0, 0.25, kv_from=2), 56)]),
    # no pair table, no token input, one tap; windows of 1, of exactly a page and of one more
    "b": dict(architecture="Ratesun", vocab=130, width=64, norm=dict(eps=1e-6), residual_mult=1.0, logit_scale=1.0,
              canon=dict(taps=1),
              layers=[_layer(_mixer(1, 16, 2, 16, 16, 16, 1, 10.0, 0.25), 48),
                      _layer(_mixer(2, 16, 16, 8, 48, 32, 16, 50000.0, 0.11), 72),
                      _layer(_mixer(4, 8, 6, 12, 24, 20, 17, 300.0, 0.4, dims=4), 40)]),
    # sizes that are multiples of nothing; two taps; a reader right behind its writer and another far behind
    "c": dict(architecture="Ratesun", vocab=77, width=50, norm=dict(eps=1e-5), residual_mult=0.3, logit_scale=2.0,
              canon=dict(taps=2), embedding=dict(bigram=dict(buckets=13, mul_prev=5, mul_cur=1)),
              token_side=dict(dim=3),
              layers=[_layer(_mixer(3, 10, 6, 14, 18, 10, 33, 123.0, 0.2), 30),
                      _layer(_mixer(2, 6, 6, 10, 18, 14, 33, 123.0, 0.3, kv_from=0), 26),
                      _layer(_mixer(2, 12, 2, 6, 10, 22, 5, 9.0, 0.2), None),
                      _layer(_mixer(1, 20, 6, 20, 18, 8, 20, 123.0, 0.1, kv_from=0), 34)]),
    # sizes the matrix-unit kernels take: multiples of 16 and 128, three taps
    "d": dict(architecture="Ratesun", vocab=320, width=128, norm=dict(eps=1e-5), residual_mult=0.4, logit_scale=0.5,
              canon=dict(taps=3), embedding=dict(bigram=dict(buckets=251, mul_prev=3, mul_cur=11)),
              token_side=dict(dim=16),
              layers=[_layer(_mixer(4, 32, 32, 32, 128, 128, 70, 10000.0, 0.125), 256),
                      _layer(_mixer(8, 16, 32, 16, 128, 64, 40, 10000.0, 0.14, kv_from=0), 128),
                      _layer(_mixer(2, 64, 16, 64, 64, 128, None, 500.0, 0.1), 256)]),
}


def config(name) -> RatesunConfig:
    return RatesunConfig.from_dict(dict(CASES[name], init_std=0.35))


def weights(cfg, seed, storage=torch.float32):
    """Random tensors by checkpoint name (matrices in `storage`), made lively: wide enough that no part drowns."""
    w = random_tensors(model_param_decls(ratesun_spec(cfg)), cfg.init_std, seed, storage)
    for k in w:
        if k.endswith((".up", ".down", ".o", ".uq", ".uk", ".uv", ".dq", ".dkv", ".gate", ".proj")):
            w[k] = (w[k].float() * (2.0 / w[k].shape[1] ** 0.5 / cfg.init_std)).to(w[k].dtype)
    return w


def runner(cfg, w, dtype="float32", kernels="reference", device="cpu", page_size=16, max_tokens=256, max_seqs=4,
           use_graphs=True):
    ecfg = EngineConfig(dtype=dtype, page_size=page_size, max_tokens=max_tokens, max_num_seqs=max_seqs, device=device,
                        kernels=kernels, use_graphs=use_graphs)
    return build_runner(cfg, TensorDict({k: v.clone() for k, v in w.items()}), ecfg)


def requests(cfg, lengths, seed):
    g = torch.Generator().manual_seed(seed)
    return {f"r{i}": torch.randint(0, cfg.vocab, (n,), generator=g).tolist() for i, n in enumerate(lengths)}


def drawn(seed: int) -> RatesunConfig:
    """A configuration drawn from a seed: any sizes, any order of layers with and without a latent of their own,
    with and without a feed-forward, windows from 1 token to none."""
    import random
    rnd = random.Random(seed)
    width = rnd.choice([24, 36, 64, 100, 128, 256])
    n_layers = rnd.randint(1, 5)
    layers, own = [], []
    for i in range(n_layers):
        window = rnd.choice([None, 1, 2, 7, 16, 17, 31, 48, 64, 65, 90])
        base = rnd.choice([10.0, 500.0, 10000.0, 1e6])
        if own and rnd.random() < 0.45:
            src = rnd.choice(own)
            of = layers[src]["mixer"]
            m = _mixer(rnd.randint(1, 6), rnd.choice([4, 8, 10, 16, 32]), of["rot_dim"], rnd.choice([4, 6, 16, 24]),
                       of["kv_rank"], rnd.choice([8, 12, 32, 40]), window, of["rot"]["base"], rnd.uniform(0.05, 0.4),
                       kv_from=src, dims=of["rot"]["dims"])
        else:
            rot = rnd.choice([2, 4, 8, 16])
            m = _mixer(rnd.randint(1, 6), rnd.choice([4, 8, 10, 16, 32]), rot, rnd.choice([4, 6, 16, 24]),
                       rnd.choice([8, 16, 20, 32, 48, 64]), rnd.choice([8, 12, 32, 40]), window, base,
                       rnd.uniform(0.05, 0.4), dims=rnd.choice([rot, max(2, rot - 2)]))
            own.append(i)
        layers.append(_layer(m, rnd.choice([None, 16, 40, 72, 130]) if n_layers > 1 else 40))
    raw = dict(architecture="Ratesun", vocab=rnd.choice([50, 97, 256, 300]), width=width, norm=dict(eps=rnd.choice([1e-6, 1e-5, 1e-3])),
               residual_mult=rnd.uniform(0.2, 1.0), logit_scale=rnd.uniform(0.25, 2.0), layers=layers, init_std=0.35)
    if rnd.random() < 0.8:
        raw["canon"] = dict(taps=rnd.randint(1, 5))
    if rnd.random() < 0.8:
        raw["embedding"] = dict(bigram=dict(buckets=rnd.choice([1, 7, 64, 1021]), mul_prev=rnd.randint(0, 2000), mul_cur=rnd.randint(1, 50)))
    if rnd.random() < 0.8:
        raw["token_side"] = dict(dim=rnd.choice([1, 4, 5, 16]))
    return RatesunConfig.from_dict(raw)
