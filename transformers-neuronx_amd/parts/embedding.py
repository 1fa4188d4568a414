"""Input and output ends of the decoder."""
from typing import Dict, List, Optional

import torch

from .base import (EMBEDDINGS, HEADS, NORMS, POSITIONS, Part, Stream, register_embedding, register_head)
from .spec import ParamDecl, PartSpec


@register_embedding("token_table")
class TokenEmbedding(Part):
    """Token rows `[vocab, embed_width]`, a projection to the hidden width when the
    two differ (no bias), then the position encoding's input step (reference:
    opt/model.py:162-166; the projection is read by no reference code path,
    opt/config.py:34)."""

    recordable = True

    def __init__(self, vocab: int, embed_width: int, width: int, position: PartSpec,
                 table_name: str, projection_name: Optional[str], position_name: str, scale: float = 1.0):
        """`scale`: the token's row times this number (in float32, where the row joins the stream)."""
        self.vocab, self.embed_width, self.width = vocab, embed_width, width
        self.scale = float(scale)
        self.table_name, self.projection_name, self.position_name = table_name, projection_name, position_name
        self.position = POSITIONS.build(position)
        self.projects = embed_width != width

    def param_decls(self, prefix: str = "") -> List[ParamDecl]:
        d = [ParamDecl(self.table_name, (self.vocab, self.embed_width), "table")]
        if self.projects:
            d.append(ParamDecl(self.projection_name, (self.width, self.embed_width)))
        return d + self.position.param_decls(self.position_name)

    def load(self, tensors: Dict, prefix: str, ops, dtype) -> None:
        super().load(tensors, prefix, ops, dtype)
        self.table = tensors[self.table_name]
        self.projection = ops.prepare_weight(tensors[self.projection_name]) if self.projects else None
        self.position.load(tensors, self.position_name, ops, dtype)

    def forward(self, ctx, want_compute: bool) -> Stream:
        x = self.ops.embed(ctx.token_ids, self.table, self.dtype, ctx.kept_tokens)
        if self.projects:
            x = self.ops.linear(x, self.projection, None)
        if self.scale != 1.0:
            xf, xc = self.position.at_input(x, ctx.positions, want_compute, scale=self.scale)
        else:
            xf, xc = self.position.at_input(x, ctx.positions, want_compute)
        return Stream(xf, xc)


@register_embedding("token_pair_table")
class TokenPairEmbedding(Part):
    """Token rows plus a row that depends on the token and the one before it in its request:
    `x = table[token] + pairs[(previous * mul_prev + token * mul_cur) mod buckets]`, and for the first token of
    a request the row after the buckets (the table has buckets + 1 rows). The sum is float32. A request's last
    token is per-request state (two places, by the parity of its position): a step's first token of a request
    pairs with it."""

    recordable = True

    def __init__(self, vocab: int, width: int, buckets: int, mul_prev: int, mul_cur: int, table_name: str,
                 pairs_name: str):
        self.vocab, self.width, self.buckets = vocab, width, buckets
        self.mul_prev, self.mul_cur = mul_prev, mul_cur
        self.table_name, self.pairs_name = table_name, pairs_name
        self.position = POSITIONS.build(PartSpec("none", {}))
        if buckets <= 0:
            raise ValueError(f"a pair table needs buckets, got {buckets}")

    def state_need(self):
        from .base import CacheNeed
        return CacheNeed("state", state_shapes=(("last_token", (2,)),), state_dtype="int32")

    def param_decls(self, prefix: str = "") -> List[ParamDecl]:
        return [ParamDecl(self.table_name, (self.vocab, self.width), "table"),
                ParamDecl(self.pairs_name, (self.buckets + 1, self.width), "table")]

    def load(self, tensors: Dict, prefix: str, ops, dtype) -> None:
        super().load(tensors, prefix, ops, dtype)
        self.table, self.pairs = tensors[self.table_name], tensors[self.pairs_name]
        self.position.load(tensors, "", ops, dtype)

    def forward(self, ctx, want_compute: bool) -> Stream:
        x = self.ops.embed_pairs(ctx.token_ids, self.table, self.pairs, self.buckets, self.mul_prev, self.mul_cur,
                                 ctx, ctx.input_state.state["last_token"], ctx.kept_tokens)
        return Stream(x, self.ops.cast(x, self.dtype) if want_compute else None)


@register_head("vocab_projection")
class VocabHead(Part):
    """Rows that need logits are picked first, then an optional norm, an optional
    projection to the embedding width (no bias) and the `[vocab, width]` matrix,
    which is the token table when the checkpoint holds no head of its own
    (reference: layers/transformer.py:196-208, row selection :298-333; tie
    opt/model.py:204-205). Logits are float32."""

    recordable = True

    def __init__(self, vocab: int, embed_width: int, width: int, norm: Optional[PartSpec],
                 weight_name: str, tied_to: Optional[str], projection_name: Optional[str], norm_name: str,
                 logit_scale: float = 1.0):
        """`logit_scale`: the logits are the product times this number (folded into the matrix's float32
        result, not into the matrix)."""
        self.logit_scale = float(logit_scale)
        self.vocab, self.embed_width, self.width = vocab, embed_width, width
        self.norm = NORMS.build(norm) if norm is not None else None
        self.weight_name, self.tied_to = weight_name, tied_to
        self.projection_name, self.norm_name = projection_name, norm_name
        self.projects = embed_width != width

    def param_decls(self, prefix: str = "") -> List[ParamDecl]:
        d = [ParamDecl(self.weight_name, (self.vocab, self.embed_width), "matrix", tied_to=self.tied_to)]
        if self.projects:
            d.append(ParamDecl(self.projection_name, (self.embed_width, self.width)))
        if self.norm is not None:
            d += self.norm.param_decls(self.norm_name)
        return d

    def load(self, tensors: Dict, prefix: str, ops, dtype) -> None:
        super().load(tensors, prefix, ops, dtype)
        self.weight = ops.prepare_weight(tensors[self.weight_name])
        self.projection = ops.prepare_weight(tensors[self.projection_name]) if self.projects else None
        if self.norm is not None:
            self.norm.load(tensors, self.norm_name, ops, dtype)

    def forward(self, stream: Stream, ctx):
        if ctx.logits_rows.numel() == 0:      # a step of prompt portions alone: nothing is asked of the head
            return torch.empty(0, self.vocab, dtype=torch.float32, device=stream.x.device)
        rows = self.ops.gather_rows(stream.x, ctx.logits_rows)
        if self.norm is not None:
            _, h = self.norm.forward(rows, False, True)
        else:
            h = self.ops.cast(rows, self.dtype)
        if self.projects:
            h = self.ops.linear(h, self.projection, None)
        logits = self.ops.linear(h, self.weight, None, out_f32=True)
        return logits if self.logit_scale == 1.0 else logits.mul_(self.logit_scale)
