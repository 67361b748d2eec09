"""Gates on a sublayer's result on its way into the residual stream.

``sigmoid_linear``: the result is multiplied element by element by ``sigmoid(G h + g)``, ``h`` being the sublayer's
own input.  The part computes the logits ``G h``; the bias, the sigmoid and the product are the business of the kernel
that adds the result into the residual (the block hands logits and bias to the stream with the result).
"""

from __future__ import annotations

from .plan import TensorSpec
from .registry import register_gate


@register_gate("sigmoid_linear")
class SigmoidLinearGate:
    """params: hidden_size, and optionally bias (default True)."""

    def __init__(self, params, env):
        self.hidden = int(params["hidden_size"])
        self.has_bias = bool(params.get("bias", True))
        self.env = env
        self.weight = None
        self.bias = None

    def weight_specs(self):
        specs = {"weight": TensorSpec((self.hidden, self.hidden))}
        if self.has_bias:
            specs["bias"] = TensorSpec((self.hidden,), "vector")
        return specs

    def bind(self, tensors):
        self.weight = tensors["weight"].contiguous()
        self.bias = tensors["bias"].contiguous() if self.has_bias else None

    def logits(self, h):
        return self.env.kernels.linear(h, self.weight)
