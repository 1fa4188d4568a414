"""Sunatar as a `ModelSpec`: which parts, with which sizes, under which tensor names.

Tensor names: `embed`, `final.norm`, `head`; layer i's start with `l<i>.`: the norm `norm1`, the mixer's `mix.*`
(`q`, `k`, `v`, `o`, a bias being the weight's name with `.b`; attention's `q.norm`, `k.norm`, `vmix`; the matrix
memory's `g`, `i`, `f`, `norm`), the feed-forward's `mlp.*` (`router`, `e<j>.{gate, up, down}`,
`shared.{gate, up, down}`). Matrix names carry no suffix.
"""
from .config import SunatarConfig
from ..config.registry import register_architecture
from ..parts.spec import LayerSpec, ModelSpec, PartSpec


def sunatar_spec(cfg: SunatarConfig) -> ModelSpec:
    d = cfg.width
    norm = PartSpec("layer_norm", dict(width=d, eps=cfg.eps, affine=True, bias=False, weight_suffix=""))
    no_norm = PartSpec("layer_norm", dict(width=d, eps=cfg.eps, affine=False))
    layers, unread = [], []
    first_mixing = None
    for i, layer in enumerate(cfg.layers):
        m = layer["mixer"]
        if layer["type"] == "attention":
            rot = m.get("rot")
            rotation = None
            if rot is not None:
                rotation = PartSpec("rotary", dict(base=rot["base"], dims=rot.get("dims", m["dim"]), interleaved=False,
                                                   scaling=rot.get("scaling")))
            mixing = None
            if m.get("v_mix"):
                if first_mixing is None:
                    first_mixing = i
                    unread.append(f"l{i}.mix.vmix")        # the first such layer blends nothing
                mixing = dict(key="sunatar values", first=first_mixing == i, name="vmix")
            mixer = PartSpec("attention", dict(
                width=d, num_heads=m["heads"], num_kv_heads=m.get("kv_heads", m["heads"]), head_size=m["dim"],
                value_size=m["vdim"], names=("q", "k", "v", "o"), weight_suffix="", bias_suffix=".b", bias=True,
                out_bias=False, window=(m.get("mask") or {}).get("size"), scale=m.get("scale", m["dim"] ** -0.5),
                rotation=rotation, qk_norm=dict(eps=cfg.eps, suffix=".norm"), value_mix=mixing))
        else:
            mixer = PartSpec("mlstm", dict(
                width=d, num_heads=m["heads"], head_size=m["dim"], value_size=m["vdim"], gate_cap=m["gate_cap"],
                eps=cfg.eps, names=("q", "k", "v", "g", "o", "i", "f", "norm"), bias_suffix=".b"))
        mlp = layer.get("mlp")
        if mlp is not None:
            shared = mlp.get("shared")
            ffn = PartSpec("mixture", dict(
                width=d, experts=mlp["router"]["experts"], top=mlp["router"]["top"], inner=mlp["expert"]["ff"],
                shared_inner=shared["ff"] if shared else 0, score="sigmoid", renormalize=False, weight_on="input",
                activation="silu", router_name="router", expert_name="e{}.", shared_name="shared.",
                names=("gate", "up", "down")))
        else:
            ffn = PartSpec("none", {})
        layers.append(LayerSpec(prefix=f"l{i}.", block="parallel", mixer=mixer, feed_forward=ffn, mixer_norm=norm,
                                feed_forward_norm=no_norm, mixer_name="mix.", feed_forward_name="mlp.",
                                mixer_norm_name="norm1", feed_forward_norm_name="norm2"))
    embedding = PartSpec("token_table", dict(vocab=cfg.vocab, embed_width=d, width=d, position=PartSpec("none", {}),
                                             table_name="embed", projection_name=None, position_name=None,
                                             scale=cfg.embedding_scale))
    head = PartSpec("vocab_projection", dict(vocab=cfg.vocab, embed_width=d, width=d, norm=norm, weight_name="head",
                                             tied_to=None, projection_name=None, norm_name="final.norm"))
    return ModelSpec(hidden_size=d, vocab_size=cfg.vocab, max_positions=cfg.max_positions, embedding=embedding,
                     layers=tuple(layers), schedule=ModelSpec.sequential(len(layers)), head=head,
                     init_std=cfg.init_std, unread=tuple(unread))


ARCHITECTURE = register_architecture("Sunatar", "sunatar", SunatarConfig, sunatar_spec,
                                     model_class="transformers_neuronx_amd.sunatar.model:SunatarForSampling")
