"""Ratesun as a `ModelSpec`: which parts, with which sizes, under which tensor names.

Tensor names: `embed`, `bigram`, `side.embed`, `final.norm`; layer i's start with `l<i>.`: the norms `norm1`,
`norm2` (before the mixer and the feed-forward) and `norm1b`, `norm2b` (after them), a bias being the weight's
name with `.b`; the convolutions `canon1`, `canon2`; the mixer's `mix.*`, the feed-forward's `mlp.*`, the
token-keyed input's `side.*` and the depth weights `dwa`. Matrix names carry no suffix.
"""
from .config import RatesunConfig
from ..config.registry import register_architecture
from ..parts.spec import LayerCall, LayerSpec, ModelSpec, PartSpec

MIX_NAMES = ("dq", "uq", "dkv", "uk", "uv", "o")


def ratesun_spec(cfg: RatesunConfig) -> ModelSpec:
    d, n_layers = cfg.width, len(cfg.layers)
    norm = PartSpec("layer_norm", dict(width=d, eps=cfg.eps, affine=True, weight_suffix="", bias_suffix=".b"))
    no_norm = PartSpec("layer_norm", dict(width=d, eps=cfg.eps, affine=False))
    # a latent that several layers read is kept for the widest window among them (all of it, if one sees all)
    keeps = {}
    for i, layer in enumerate(cfg.layers):
        m = layer["mixer"]
        src = m["kv_from"] if m.get("kv_from") is not None else i
        size = (m.get("mask") or {}).get("size") or "all"
        if src not in keeps:
            keeps[src] = size
        elif keeps[src] != "all":
            keeps[src] = "all" if size == "all" else max(keeps[src], size)
    layers, schedule, unread = [], [], []
    for i, layer in enumerate(cfg.layers):
        m = layer["mixer"]
        own = m.get("kv_from") is None
        mixer = PartSpec("latent_attention", dict(
            width=d, num_heads=m["heads"], head_size=m["dim"], rot_size=m["rot_dim"], value_size=m["vdim"],
            kv_rank=m["kv_rank"], q_rank=m["q_rank"], eps=cfg.eps,
            # a mixer that names no scale gets the usual one for its query/key size; one that names no number of
            # turned elements turns the whole rotated part
            scale=m.get("scale", (m["dim"] + m["rot_dim"]) ** -0.5),
            rotation=PartSpec("rotary", dict(base=m["rot"]["base"], dims=m["rot"].get("dims", m["rot_dim"]),
                                             interleaved=True)),
            names=MIX_NAMES, window=(m.get("mask") or {}).get("size"), keep=keeps[i] if own else None, own_kv=own))
        mlp = layer.get("mlp")
        if mlp is not None:
            ffn = PartSpec("dense", dict(width=d, inner=mlp["ff"], activation="poly_norm", bias=False, up_name="up",
                                         down_name="down", weight_suffix="", act_name="act", eps=cfg.eps))
        else:
            ffn = PartSpec("none", {})
            unread += [f"l{i}.{name}" for name in ("norm2", "norm2.b", "norm2b", "norm2b.b", "canon2")]
        side = None
        if cfg.token_side:
            side = dict(table="side.embed", rows=cfg.vocab, columns=n_layers * cfg.side_dim, dim=cfg.side_dim,
                        offset=i * cfg.side_dim, gate="side.gate", proj="side.proj", norm="side.norm", eps=cfg.eps)
        block = PartSpec("sandwich", dict(
            mixer_post_norm=norm, feed_forward_post_norm=norm, names=("norm1b", "norm2b"), mult=cfg.residual_mult,
            taps=cfg.taps, conv_names=("canon1", "canon2"), side=side, depth_average=i + 2, depth_name="dwa",
            depth_slots=n_layers + 1))
        layers.append(LayerSpec(prefix=f"l{i}.", block=block, mixer=mixer, feed_forward=ffn, mixer_norm=norm,
                                feed_forward_norm=norm if mlp is not None else no_norm, mixer_name="mix.",
                                feed_forward_name="mlp.", mixer_norm_name="norm1", feed_forward_norm_name="norm2"))
        # cache ids are layer numbers: a layer without a latent of its own reads the cache of the one it names
        schedule.append(LayerCall(i, cache=i if own else m["kv_from"], writes=own))
    pair = cfg.bigram
    if pair:
        embedding = PartSpec("token_pair_table", dict(vocab=cfg.vocab, width=d, buckets=pair["buckets"],
                                                      mul_prev=pair["mul_prev"], mul_cur=pair["mul_cur"],
                                                      table_name="embed", pairs_name="bigram"))
    else:
        embedding = PartSpec("token_table", dict(vocab=cfg.vocab, embed_width=d, width=d, position=PartSpec("none", {}),
                                                 table_name="embed", projection_name=None, position_name=None))
    head = PartSpec("vocab_projection", dict(vocab=cfg.vocab, embed_width=d, width=d, norm=norm, weight_name="head",
                                             tied_to="embed", projection_name=None, norm_name="final.norm",
                                             logit_scale=cfg.logit_scale))
    return ModelSpec(hidden_size=d, vocab_size=cfg.vocab, max_positions=cfg.max_positions, embedding=embedding,
                     layers=tuple(layers), schedule=tuple(schedule), head=head, init_std=cfg.init_std,
                     unread=tuple(unread))


ARCHITECTURE = register_architecture("Ratesun", "ratesun", RatesunConfig, ratesun_spec,
                                     model_class="transformers_neuronx_amd.ratesun.model:RatesunForSampling")
