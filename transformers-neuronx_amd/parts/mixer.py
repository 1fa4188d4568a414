"""Token mixers."""
import math
from typing import Dict, List, Optional

import torch

from .base import POSITIONS, CacheNeed, Mixer, register_mixer
from .spec import ParamDecl


@register_mixer("attention")
class Attention(Mixer):
    """Softmax attention over a paged key/value cache.

    `Q = (h Wq^T + bq) * scale`, keys and values of the step's tokens are stored
    into the request's pages, each query attends to the keys of its own request
    at positions `<=` its own (and `> position - window` when a window is set),
    softmax in float32, then the output projection (reference:
    opt/model.py:444-523; scale layers/attention.py:428-437; masks
    hlo.py:1030-1042 and the bottom-right block-diagonal form hlo.py:3211-3309;
    cache scatter by slot hlo.py:3665-3704).

    `num_kv_heads < num_heads` groups query heads over shared key/value heads.
    `own_kv=False` builds a mixer without key/value projections that reads the
    cache another call of the run order writes. `rotation` names a position
    encoding (a `PartSpec` of the position registry) that turns the queries and
    keys before they are scaled and stored: through its `pair_tables`, inside the
    projection's launch, or else through its `on_query_key`; OPT has none.
    """

    recordable = True

    def __init__(self, width: int, num_heads: int, head_size: int, names, num_kv_heads: Optional[int] = None,
                 bias: bool = True, window: Optional[int] = None, scale: Optional[float] = None,
                 own_kv: bool = True, rotation=None):
        """`names`: the checkpoint's names of the query, key, value and output projections, relative to
        the mixer's prefix (the architecture's spec gives them)."""
        self.width, self.num_heads, self.head_size = width, num_heads, head_size
        self.num_kv_heads = num_kv_heads if num_kv_heads is not None else num_heads
        if self.num_heads % self.num_kv_heads:
            raise ValueError(f"num_heads ({num_heads}) must be a multiple of num_kv_heads ({self.num_kv_heads})")
        if head_size % 16 or not 16 <= head_size <= 256:
            raise ValueError(f"head_size must be a multiple of 16 between 16 and 256, got {head_size}")
        self.has_bias, self.window, self.own_kv = bias, window, own_kv
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(head_size)
        self.names = tuple(names)
        self.rotation = POSITIONS.build(rotation) if rotation is not None else None
        if self.rotation is not None and not getattr(self.rotation, "recordable", False):
            self.recordable = False
        if len(self.names) != 4:
            raise ValueError("names: the query, key, value and output projections, four names")

    def cache_need(self) -> Optional[CacheNeed]:
        return CacheNeed("paged", kv_heads=self.num_kv_heads, head_size=self.head_size, window=self.window)

    def param_decls(self, prefix: str) -> List[ParamDecl]:
        qn, kn, vn, on = self.names
        q_out = self.num_heads * self.head_size
        kv_out = self.num_kv_heads * self.head_size
        outs = [(qn, q_out)] + ([(kn, kv_out), (vn, kv_out)] if self.own_kv else [])
        d = []
        for n, out in outs:
            d.append(ParamDecl(f"{prefix}{n}.weight", (out, self.width)))
            if self.has_bias:
                d.append(ParamDecl(f"{prefix}{n}.bias", (out,), "vector"))
        d.append(ParamDecl(f"{prefix}{on}.weight", (self.width, q_out)))
        if self.has_bias:
            d.append(ParamDecl(f"{prefix}{on}.bias", (self.width,), "vector"))
        if self.rotation is not None:
            d += self.rotation.param_decls(prefix + "rotation")
        return d

    def load(self, tensors: Dict, prefix: str, ops, dtype) -> None:
        super().load(tensors, prefix, ops, dtype)
        qn, kn, vn, on = self.names
        ins = [qn] + ([kn, vn] if self.own_kv else [])
        # One fused projection: a plain concatenation of the rows (the reference's
        # fused form interleaves per tensor-parallel shard, utils.py:189-242).
        self.w_qkv = ops.prepare_weight(torch.cat([tensors[f"{prefix}{n}.weight"] for n in ins], dim=0).contiguous())
        self.b_qkv = (torch.cat([tensors[f"{prefix}{n}.bias"] for n in ins], dim=0).contiguous()
                      if self.has_bias else None)
        self.w_out = ops.prepare_weight(tensors[f"{prefix}{on}.weight"])
        self.b_out = tensors[f"{prefix}{on}.bias"] if self.has_bias else None
        self.turn = None
        if self.rotation is not None:
            self.rotation.load(tensors, prefix + "rotation", ops, dtype)
            self.turn = self.rotation.pair_tables(self.head_size)     # the pairwise form: applied by the projection

    def first_weight(self):
        return self.w_qkv

    def step_planners(self):
        from ..kernels.attention_plan import attention_plan
        return {"attention": attention_plan}

    def launch_shape(self, step):
        shape = getattr(self.ops, "attention_launch_shape", None)
        return shape(step, self.num_heads, self.window, self.head_size, self.num_kv_heads) if shape is not None else None

    def flops_per_token(self, keys: float = 0.0) -> float:
        seen = min(keys, self.window) if self.window else keys
        return super().flops_per_token(keys) + 4.0 * self.num_heads * self.head_size * seen   # q k^T and p v

    def forward(self, h, ctx, cache, residual):
        if cache.writes != self.own_kv:
            raise ValueError("an attention mixer with own_kv writes its cache; one without reads another's")
        view = ctx.groups[cache.group]
        kv_write = self.num_kv_heads if self.own_kv else 0
        if self.rotation is not None and self.turn is None:
            # the projections with their bias, turned by the encoding, then scaled and stored
            qkv = self.ops.linear(h, self.w_qkv, self.b_qkv)
            qkv = self.rotation.on_query_key(qkv, ctx, self.num_heads, kv_write, self.head_size)
            q = self.ops.qkv_write(qkv, None, self.num_heads, kv_write, self.head_size, self.scale, ctx, view,
                                   cache.k_pages, cache.v_pages)
            c = self.ops.attention(q, self.num_heads, self.num_kv_heads, self.head_size, ctx, view,
                                   cache.k_pages, cache.v_pages, self.window)
            return self.ops.linear(c, self.w_out, self.b_out, residual=residual, out_f32=True)
        q = self.ops.qkv_project(h, self.w_qkv, self.b_qkv, self.num_heads,
                                 self.num_kv_heads if self.own_kv else 0, self.head_size, self.scale, ctx, view,
                                 cache.k_pages, cache.v_pages, **({"turn": self.turn} if self.turn is not None else {}))
        c = self.ops.attention(q, self.num_heads, self.num_kv_heads, self.head_size, ctx, view,
                               cache.k_pages, cache.v_pages, self.window)
        return self.ops.linear(c, self.w_out, self.b_out, residual=residual, out_f32=True)


@register_mixer("latent_attention")
class LatentAttention(Mixer):
    """Softmax attention whose keys and values are made from one small vector a token, and only that vector
    is cached.

    With H heads, per head n unrotated and r rotated query/key elements and v value elements, a key/value
    latent of R and a query latent of Q elements:
        c_q = rms_norm(W_dq h),  q = W_uq c_q  laid out head by head as [n | r]
        [c' | k_r'] = W_dkv h,   c = rms_norm(c'),  k_r = turn(k_r')      (R and r elements; k_r is shared by the heads)
        score(i, j, head) = scale * (q_n[i] . (W_uk c[j]) + turn(q_r[i]) . k_r[j]),   value = W_uv c[j]
    over the keys of the query's own request at positions j <= i (and i - j < window with a window), softmax
    in float32, then W_o on the heads side by side. `turn` is the `rotation` (a `rotary` position part).

    The cache holds c and k_r, in pages of their own shapes. The products with W_uk and W_uv are moved to the
    query's side, so that a cached token is read as it lies: q_lat = W_uk^T q_n (R elements a head),
    score = scale * (q_lat . c + q_r . k_r), and the weighted sum of the c[j] goes through W_uv afterwards.
    c is kept twice, the second time with a page's tokens side by side (`across`), as the other designs'
    values are: the weighted sum contracts over tokens, and the matrix unit wants them next to each other.
    That order is the one for decoding, where what is read counts. A step of prompts' runs alone may take the
    other (`ops.latent_expands`): the keys W_uk c and values W_uv c of what the runs can see are made once for
    the step, and a (query, key) pair costs 2 (n + r + v) multiply-adds a head instead of 2 (2R + r).

    `own_kv=False`: no W_dkv; the mixer reads the cache of another call of the run order, whose R, r and
    rotation are its own. `keep`: the tokens the cache keeps: a number, "all", or None for the mixer's own window;
    a cache that is read by mixers of different windows keeps the most any of them sees.
    """

    recordable = True

    def __init__(self, width: int, num_heads: int, head_size: int, rot_size: int, value_size: int, kv_rank: int,
                 q_rank: int, scale: float, eps: float, rotation, names, window: Optional[int] = None,
                 keep=None, own_kv: bool = True, norm_suffix: str = ".norm", weight_suffix: str = ""):
        """`names`: the checkpoint's names, relative to the mixer's prefix, of W_dq, W_uq, W_dkv, W_uk, W_uv and
        W_o; a latent's norm weight is its down-projection's name with `norm_suffix`."""
        self.width, self.num_heads, self.head_size, self.rot_size = width, num_heads, head_size, rot_size
        self.value_size, self.kv_rank, self.q_rank = value_size, kv_rank, q_rank
        self.scale, self.eps, self.window, self.own_kv = float(scale), float(eps), window, own_kv
        self.keep = keep if own_kv else None
        if keep is not None and keep != "all" and (not isinstance(keep, int) or keep < 1):
            raise ValueError(f"keep is a number of tokens, \"all\" or None, got {keep!r}")
        if own_kv and isinstance(keep, int) and (window is None or keep < window):
            raise ValueError(f"a cache that keeps {keep} tokens cannot serve a window of {window}")
        self.names = tuple(names)
        if len(self.names) != 6:
            raise ValueError("names: W_dq, W_uq, W_dkv, W_uk, W_uv, W_o, six names")
        self.norm_suffix, self.weight_suffix = norm_suffix, weight_suffix
        self.rotation = POSITIONS.build(rotation)
        if rot_size % 2 or self.rotation.dims > rot_size:
            raise ValueError(f"the rotated part has {rot_size} elements; the rotation turns {self.rotation.dims}")

    def cache_need(self) -> Optional[CacheNeed]:
        keep = None if self.keep == "all" else (self.keep if self.keep is not None else self.window)
        return CacheNeed("paged", window=keep,
                         page_tensors=(("latent", ("page", self.kv_rank)), ("rotated", ("page", self.rot_size)),
                                       ("across", (self.kv_rank, "page"))))

    def step_planners(self):
        from ..kernels.attention_plan import attention_plan
        return {"attention": attention_plan}

    def param_decls(self, prefix: str) -> List[ParamDecl]:
        dq, uq, dkv, uk, uv, o = (prefix + n for n in self.names)
        s, h = self.weight_suffix, self.num_heads
        d = [ParamDecl(dq + s, (self.q_rank, self.width)),
             ParamDecl(dq + self.norm_suffix, (self.q_rank,), "vector", "around_one"),
             ParamDecl(uq + s, (h * (self.head_size + self.rot_size), self.q_rank))]
        if self.own_kv:
            d += [ParamDecl(dkv + s, (self.kv_rank + self.rot_size, self.width)),
                  ParamDecl(dkv + self.norm_suffix, (self.kv_rank,), "vector", "around_one")]
        d += [ParamDecl(uk + s, (h * self.head_size, self.kv_rank)),
              ParamDecl(uv + s, (h * self.value_size, self.kv_rank)),
              ParamDecl(o + s, (self.width, h * self.value_size))]
        return d

    def load(self, tensors: Dict, prefix: str, ops, dtype) -> None:
        super().load(tensors, prefix, ops, dtype)
        dq, uq, dkv, uk, uv, o = (prefix + n for n in self.names)
        s, h = self.weight_suffix, self.num_heads
        # one product for both latents: the rows of W_dq, then those of W_dkv
        down = [tensors[dq + s]] + ([tensors[dkv + s]] if self.own_kv else [])
        self.w_down = ops.prepare_weight(torch.cat(down, dim=0).contiguous())
        self.q_norm = tensors[dq + self.norm_suffix]
        self.kv_norm = tensors[dkv + self.norm_suffix] if self.own_kv else None
        self.w_uq = ops.prepare_weight(tensors[uq + s])
        # W_uk a head, transposed: [H, R, n], the matrix that takes a head's q_n to its q_lat
        self.w_uk_t = tensors[uk + s].view(h, self.head_size, self.kv_rank).transpose(1, 2).contiguous()
        self.w_uv = tensors[uv + s].view(h, self.value_size, self.kv_rank).contiguous()
        # the whole matrices, for steps whose keys and values are made explicitly
        self.w_uk_whole = ops.prepare_weight(tensors[uk + s])
        self.w_uv_whole = tensors[uv + s]
        self.w_o = ops.prepare_weight(tensors[o + s])
        self.rotation.load(tensors, prefix + "rotation", ops, dtype)
        self.freqs = self.rotation.frequencies()
        if not self.rotation.interleaved:
            raise ValueError("latent attention turns neighbouring pairs (the interleaved layout)")

    def first_weight(self):
        return None          # the product's float32 result goes to two norms: the norm before it stays a kernel

    def flops_per_token(self, keys: float = 0.0) -> float:
        seen = min(keys, self.window) if self.window else keys
        return super().flops_per_token(keys) + 2.0 * self.num_heads * (2 * self.kv_rank + self.rot_size) * seen

    def forward(self, h, ctx, cache, residual):
        if cache.writes != self.own_kv:
            raise ValueError("a latent-attention mixer with own_kv writes its cache; one without reads another's")
        ops, view = self.ops, ctx.groups[cache.group]
        heads, n, r = self.num_heads, self.head_size, self.rot_size
        latent, rotated, across = cache.pages["latent"], cache.pages["rotated"], cache.pages["across"]
        if latent.shape[-1] != self.kv_rank or rotated.shape[-1] != r:
            raise ValueError(f"the cache holds latents of {latent.shape[-1]} + {rotated.shape[-1]} elements, "
                             f"this mixer reads {self.kv_rank} + {r}")
        down = ops.linear(h, self.w_down, None, out_f32=True, f32_by_library=True)
        c_q = ops.latent_norms(down, self.q_rank, self.kv_rank if self.own_kv else 0, r if self.own_kv else 0,
                               self.q_norm, self.kv_norm, self.eps, self.freqs, ctx, view, latent, rotated, across)
        q = ops.linear(c_q, self.w_uq, None)
        if ops.latent_expands(ctx, n, r, self.value_size, self.kv_rank):
            # a step of prompts' runs alone: keys and values made from the latents, attention on them
            values = ops.latent_attention_expanded(q, self.w_uk_whole, self.w_uv_whole, heads, n, r, self.value_size,
                                                   self.kv_rank, self.freqs, self.scale, ctx, view, latent, rotated,
                                                   self.window)
            return ops.linear(values, self.w_o, None, residual=residual, out_f32=True, f32_by_library=residual is None)
        q_lat = ops.batched_linear(q.view(-1, heads, n + r)[:, :, :n], self.w_uk_t)
        o_lat = ops.latent_attention(q, q_lat, heads, n, r, self.kv_rank, self.freqs, self.scale, ctx, view,
                                     latent, rotated, across, self.window)
        values = ops.batched_linear(o_lat, self.w_uv)
        return ops.linear(values.view(-1, heads * self.value_size), self.w_o, None, residual=residual, out_f32=True,
                          f32_by_library=residual is None)
