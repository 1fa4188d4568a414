"""Feed-forward parts."""
from typing import Dict, List

from .base import FeedForward, register_feed_forward
from .spec import ParamDecl


@register_feed_forward("dense")
class DenseFeedForward(FeedForward):
    """`act(h W1^T + b1) W2^T + b2`, the activation applied to the float32
    accumulator (reference: hlo.py:550-559; activations.py:20-48)."""

    recordable = True

    def __init__(self, width: int, inner: int, activation: str, up_name: str, down_name: str, bias: bool = True,
                 weight_suffix: str = ".weight", act_name: str = None, eps: float = 1e-5):
        """`up_name`, `down_name`: the checkpoint's names of the two matrices, relative to the part's prefix;
        `weight_suffix`: what a matrix's name adds to them.

        `activation="poly_norm"` is no function of one element: with N(v) = v / sqrt(mean(v^2) + eps) over a
        token's inner values, act(z) = a N(z) + b N(z^2) + c N(z^3) + e, powers element by element, the four
        numbers being the tensor `act_name`. Sums and roots are float32."""
        self.width, self.inner, self.activation, self.has_bias = width, inner, activation, bias
        self.up_name, self.down_name, self.weight_suffix = up_name, down_name, weight_suffix
        self.act_name, self.eps = act_name, float(eps)
        if activation == "poly_norm" and not act_name:
            raise ValueError("activation 'poly_norm' needs `act_name`, the tensor of its four numbers")

    def param_decls(self, prefix: str) -> List[ParamDecl]:
        d = [ParamDecl(f"{prefix}{self.up_name}{self.weight_suffix}", (self.inner, self.width)),
             ParamDecl(f"{prefix}{self.down_name}{self.weight_suffix}", (self.width, self.inner))]
        if self.has_bias:
            d += [ParamDecl(f"{prefix}{self.up_name}.bias", (self.inner,), "vector"),
                  ParamDecl(f"{prefix}{self.down_name}.bias", (self.width,), "vector")]
        if self.activation == "poly_norm":
            d.append(ParamDecl(f"{prefix}{self.act_name}", (4,), "vector", "around_one"))
        return d

    def load(self, tensors: Dict, prefix: str, ops, dtype) -> None:
        super().load(tensors, prefix, ops, dtype)
        self.w1 = ops.prepare_weight(tensors[f"{prefix}{self.up_name}{self.weight_suffix}"])
        self.w2 = ops.prepare_weight(tensors[f"{prefix}{self.down_name}{self.weight_suffix}"])
        self.b1 = tensors.get(f"{prefix}{self.up_name}.bias") if self.has_bias else None
        self.b2 = tensors.get(f"{prefix}{self.down_name}.bias") if self.has_bias else None
        self.coeffs = tensors[f"{prefix}{self.act_name}"] if self.activation == "poly_norm" else None

    def first_weight(self):
        return self.w1

    def forward(self, h, ctx, residual):
        """`residual` None: f(h) alone, in float32 (for an arrangement that norms it before the sum)."""
        if self.activation == "poly_norm":
            inner = self.ops.poly_norm(self.ops.linear(h, self.w1, self.b1, out_f32=True, f32_by_library=True),
                                       self.coeffs, self.eps)
        else:
            inner = self.ops.linear(h, self.w1, self.b1, act=self.activation)
        return self.ops.linear(inner, self.w2, self.b2, residual=residual, out_f32=True, f32_by_library=residual is None)


@register_feed_forward("none")
class NoFeedForward(FeedForward):
    """A layer without a feed-forward: the stream passes."""

    recordable = True
    absent = True

    def __init__(self, **_):
        pass

    def forward(self, h, ctx, residual):
        return residual
