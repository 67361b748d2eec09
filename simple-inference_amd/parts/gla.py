"""Gated linear attention: a mixer whose memory is a matrix state per head instead of keys and values.

For a token with input ``h`` (``H`` heads, key width ``D``, value width ``Dv``):

    q = Wq h * D^(-1/2),  k = Wk h            [H, D]
    v = Wv h                                  [H, Dv]
    alpha = sigmoid(A2 (A1 h) + a)^(1/tau)    [H, D]    a decay per key channel, through a low-rank pair
    S <- diag(alpha) S + k v^T                per head, S [D, Dv]
    o = S^T q                                 the state already holds this token
    y = Wo (concat_h(o_h / rms(o_h) * w) * silu(Wg h))

A request's state is all zeros before its first token, float32 in both modes, and kept in the request's state slot
(one per run of the layer); the cache manager hands it in as ``cache.state``.  A sequence's tokens must arrive in
order, which the step function guarantees.  All input projections (q, k, v, g and the low-rank ``A1``) are one
stacked matrix; the decays (``A2``, bias, log-sigmoid, the power) are the kernels' business, in float.

The rank of the low-rank pair is whatever the checkpoint's tensors have, unless ``decay_rank`` names it.
"""

from __future__ import annotations

import torch

from .plan import StateNeed, TensorSpec
from .registry import register_mixer


@register_mixer("gla")
class GatedLinearAttention:
    """params: hidden_size, num_heads, key_dim, value_dim, tau, norm_eps, and optionally decay_rank."""

    def __init__(self, params, env):
        self.hidden = int(params["hidden_size"])
        self.num_heads = int(params["num_heads"])
        self.key_dim = int(params["key_dim"])
        self.value_dim = int(params["value_dim"])
        self.tau = float(params["tau"])
        if not self.tau > 0:
            raise ValueError(f"tau must be positive, got {self.tau}")
        self.eps = float(params["norm_eps"])
        rank = params.get("decay_rank")
        self.rank = int(rank) if rank else -1      # -1: read from the checkpoint
        check = getattr(env.kernels, "check_recurrent_geometry", None)
        if check is not None:
            check(self.key_dim, self.value_dim)
        self.env = env
        self.w_in = self.w_a2 = self.b_a2 = self.norm = self.w_o = None
        self.columns = None

    takes_scaled_rows = False

    def weight_specs(self):
        qk, v = self.num_heads * self.key_dim, self.num_heads * self.value_dim
        return {
            "q": TensorSpec((qk, self.hidden)), "k": TensorSpec((qk, self.hidden)),
            "v": TensorSpec((v, self.hidden)), "g": TensorSpec((v, self.hidden)),
            "a1": TensorSpec((self.rank, self.hidden)), "a2": TensorSpec((qk, self.rank)),
            "a2_bias": TensorSpec((qk,), "vector"), "norm": TensorSpec((self.value_dim,), "vector"),
            "o": TensorSpec((self.hidden, v)),
        }

    def bind(self, tensors):
        rank = tensors["a1"].shape[0]
        if tensors["a2"].shape[1] != rank or (self.rank > 0 and rank != self.rank):
            raise ValueError(f"the low-rank pair of the decay does not fit: a1 {tuple(tensors['a1'].shape)}, "
                             f"a2 {tuple(tensors['a2'].shape)}, expected rank {self.rank if self.rank > 0 else 'any'}")
        self.rank = rank
        qk, v = self.num_heads * self.key_dim, self.num_heads * self.value_dim
        # the low-rank input last, filled up with zero rows so that a projected row keeps its alignment
        pad = -(-rank // 8) * 8 - rank
        stacked = [tensors["q"], tensors["k"], tensors["v"], tensors["g"], tensors["a1"]]
        if pad:
            stacked.append(tensors["a1"].new_zeros((pad, self.hidden)))
        self.w_in = torch.cat(stacked, dim=0).contiguous()
        self.columns = (0, qk, 2 * qk, 2 * qk + v, 2 * qk + 2 * v)
        self.w_a2 = tensors["a2"].contiguous()
        self.b_a2 = tensors["a2_bias"].contiguous()
        self.norm = tensors["norm"].contiguous()
        self.w_o = tensors["o"].contiguous()
        prepare = getattr(self.env.kernels, "prepare_pending_weight", None)
        if prepare is not None:
            prepare(self.w_o)

    def cache_need(self):
        return None

    def state_need(self):
        return StateNeed((self.num_heads, self.key_dim, self.value_dim), "float32", 0.0)

    def forward(self, h, ctx, cache):
        k = self.env.kernels
        proj = k.linear(h, self.w_in)
        out = k.gla_recurrent(proj, self.columns, self.w_a2, self.b_a2, self.norm, self.num_heads, self.key_dim,
                              self.value_dim, self.tau, self.key_dim ** -0.5, self.eps, ctx, cache)
        return k.pending_linear(out, self.w_o)
