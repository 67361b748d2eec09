"""Operations on the whole residual stream between runs of layers.

``remix``: ``x <- J [x; x0]`` with ``J [hidden, 2 hidden]`` (the columns that meet ``x`` first) and ``x0`` the
embedding output of the same tokens: the stream is mixed with what the tokens were before any layer.  A design that
walks a run of its layers several times does this at the start of every walk.  The two streams are lowered to the
compute dtype side by side, the product sums in float and its result is the new float32 residual.
"""

from __future__ import annotations

from .plan import TensorSpec
from .registry import register_stream_op


@register_stream_op("remix")
class Remix:
    """params: hidden_size."""

    def __init__(self, params, env):
        self.hidden = int(params["hidden_size"])
        self.env = env
        self.weight = None

    def weight_specs(self):
        return {"weight": TensorSpec((self.hidden, 2 * self.hidden))}

    def bind(self, tensors):
        self.weight = tensors["weight"].contiguous()

    def forward(self, stream, ctx, first):
        k = self.env.kernels
        x = stream.settle(k)
        both = k.side_by_side(x, first, self.env.dtype)
        stream.residual = k.linear(both, self.weight, out_float32=True)
        stream.lowered = None
