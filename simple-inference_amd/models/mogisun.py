"""``Mogisun``: a decoder of gated pre-norm layers whose mixers are softmax attention or gated linear attention,
whose feed-forwards are dense or mixtures of experts, and which walks a run of its layers several times.

All that is particular to the design is here: which parts a layer has, in which order layers run, and what the
tensors are called in the checkpoint.

* A layer is a gated pre-norm block: ``h = norm1(x); x += sigmoid(R1 h + r1) * mixer(h)`` and the same with the
  feed-forward, if it has one.
* ``attention``: grouped-query softmax attention without a rotation; biased q, k, v and o; q and k divided by their
  root mean square per head (no gains); a query temperature that grows with the position; an explicit score scale;
  a sigmoid gate per head on the output.
* ``gla``: gated linear attention (a decaying matrix state per head, kept in the request's state slot).
* ``dense``: SwiGLU.  ``moe``: routed SwiGLU experts with an optional shared expert behind a scalar sigmoid gate.
* ``loop``: layers ``start .. stop-1`` run ``times`` times with the same weights; every walk keeps keys, values and
  states of its own (the plan's ``order`` names those layers once per walk) and begins with a re-mix of the stream
  with the embedding output (``loop.in``), the first walk too.
* The head multiplies its logits by ``logit_scale`` and caps them softly at ``logit_softcap``.

Checkpoint names: ``embed``, ``loop.in``, ``final.norm``, ``head``; layer ``i``: ``l<i>.norm1``, ``l<i>.norm2``,
``l<i>.rg1``, ``l<i>.rg2`` (``.b`` for their biases), ``l<i>.mix.*`` and ``l<i>.mlp.*``.
"""

from __future__ import annotations

from ..config.mogisun_config import DenseMlp, LinearAttention, MogisunConfig, MoeMlp, SoftmaxAttention
from ..config.registry import register_architecture
from ..parts.plan import LayerSpec, ModelPlan, PartSpec


def _mixer(cfg: MogisunConfig, m, p: str) -> PartSpec:
    if isinstance(m, SoftmaxAttention):
        return PartSpec("attention", {
            "hidden_size": cfg.width, "num_heads": m.heads, "num_kv_heads": m.kv_heads, "head_dim": m.dim,
            "value_head_dim": m.vdim, "scale": m.scale, "bias": True, "o_bias": True, "out_gate": True,
            "qk_norm": {"eps": cfg.norm_eps, "gain": False},
            "q_temp": m.q_temp.to_dict() if m.q_temp is not None else None,
            "position": {"kind": "none", "params": {}},
        }, {
            "q": f"{p}.q", "k": f"{p}.k", "v": f"{p}.v", "o": f"{p}.o", "gate": f"{p}.g",
            "q_bias": f"{p}.q.b", "k_bias": f"{p}.k.b", "v_bias": f"{p}.v.b", "o_bias": f"{p}.o.b",
        }, role="mixer")
    assert isinstance(m, LinearAttention)
    return PartSpec("gla", {
        "hidden_size": cfg.width, "num_heads": m.heads, "key_dim": m.dim, "value_dim": m.vdim, "tau": m.tau,
        "norm_eps": cfg.norm_eps, "decay_rank": m.rank,
    }, {
        "q": f"{p}.q", "k": f"{p}.k", "v": f"{p}.v", "g": f"{p}.g", "o": f"{p}.o", "norm": f"{p}.norm",
        "a1": f"{p}.a1", "a2": f"{p}.a2", "a2_bias": f"{p}.a2.b",
    }, role="mixer")


def _feed_forward(cfg: MogisunConfig, mlp, p: str) -> PartSpec:
    if isinstance(mlp, DenseMlp):
        return PartSpec("swiglu", {"hidden_size": cfg.width, "intermediate_size": mlp.ff},
                        {"gate": f"{p}.gate", "up": f"{p}.up", "down": f"{p}.down"}, role="feed_forward")
    assert isinstance(mlp, MoeMlp)
    names = {"router": f"{p}.router"}
    for e in range(mlp.experts):
        names.update({f"gate{e}": f"{p}.e{e}.gate", f"up{e}": f"{p}.e{e}.up", f"down{e}": f"{p}.e{e}.down"})
    if mlp.shared_ff is not None:
        names.update({"shared_gate": f"{p}.shared.gate", "shared_up": f"{p}.shared.up",
                      "shared_down": f"{p}.shared.down", "shared_scale": f"{p}.shared.sg"})
    return PartSpec("moe", {"hidden_size": cfg.width, "experts": mlp.experts, "top": mlp.top, "expert_size": mlp.ff,
                            "shared_size": mlp.shared_ff}, names, role="feed_forward")


def mogisun_plan(cfg: MogisunConfig) -> ModelPlan:
    norm = lambda name: PartSpec("rmsnorm", {"size": cfg.width, "eps": cfg.norm_eps}, {"weight": name}, role="norm")
    gate = lambda name: PartSpec("sigmoid_linear", {"hidden_size": cfg.width}, {"weight": name, "bias": name + ".b"},
                                 role="gate")
    layers = []
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}"
        parts = {"mixer_norm": norm(f"{p}.norm1"), "mixer": _mixer(cfg, layer.mixer, f"{p}.mix"),
                 "mixer_gate": gate(f"{p}.rg1")}
        if layer.mlp is not None:
            parts.update({"feed_forward_norm": norm(f"{p}.norm2"),
                          "feed_forward": _feed_forward(cfg, layer.mlp, f"{p}.mlp"),
                          "feed_forward_gate": gate(f"{p}.rg2")})
        layers.append(LayerSpec(block="gated_prenorm", parts=parts))
    runs = cfg.run_order()
    stream_ops, entries = [], {}
    if cfg.loop is not None:
        stream_ops.append(PartSpec("remix", {"hidden_size": cfg.width}, {"weight": "loop.in"}))
        entries = {e: 0 for e, (_, enters) in enumerate(runs) if enters}
    return ModelPlan(
        hidden_size=cfg.width,
        vocab_size=cfg.vocab,
        embedding=PartSpec("embedding", {"vocab_size": cfg.vocab, "hidden_size": cfg.width}, {"weight": "embed"}),
        layers=layers,
        final_norm=PartSpec("rmsnorm", {"size": cfg.width, "eps": cfg.norm_eps}, {"weight": "final.norm"}),
        head=PartSpec("head", {"vocab_size": cfg.vocab, "hidden_size": cfg.width, "tied": False,
                               "scale": cfg.logit_scale, "softcap": cfg.logit_softcap}, {"weight": "head"}),
        order=[i for i, _ in runs],
        stream_ops=stream_ops,
        entries=entries,
    )


register_architecture("Mogisun", MogisunConfig.from_dict, mogisun_plan, replace=True)
