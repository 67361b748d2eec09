"""``Feduzen``: a decoder whose layers add the *norm of a sublayer's output* to the residual stream.

All that is particular to the design is here: which parts a layer has, in which order layers run, and what the
tensors are called in the checkpoint.  A layer is an output-norm block (``x += norm1(mixer(x))``, then
``x += norm2(ff(x))`` if it has a feed-forward).  Its mixer is grouped-query attention with biased projections,
a per-head RMS norm of q and k before a rotation of the first ``rot.dims`` dimensions, an explicit score scale,
a mask of blocks of ``mask.size`` positions, and a per-head sink in the softmax; its feed-forward is dense with
the square of relu.  The embedding is multiplied by ``embedding.scale``; the head has a matrix of its own.

A layer with ``weights_of`` is a further run of the parts of the layer it names, and its keys and values go to
pages that only this run uses: in the plan it is a second entry of ``order`` for that layer, not a second copy of
its tensors.

Checkpoint names: ``embed``, ``final.norm``, ``head``; layer ``i``: ``l<i>.norm1``, ``l<i>.norm2``,
``l<i>.mix.{q,k,v}`` with ``.b`` for the biases, ``l<i>.mix.{q,k}.norm``, ``l<i>.mix.sink``, ``l<i>.mix.o``,
``l<i>.mlp.{up,down}``.
"""

from __future__ import annotations

from ..config.feduzen_config import FeduzenConfig
from ..config.registry import register_architecture
from ..parts.plan import LayerSpec, ModelPlan, PartSpec


def feduzen_plan(cfg: FeduzenConfig) -> ModelPlan:
    norm = lambda name: PartSpec("rmsnorm", {"size": cfg.width, "eps": cfg.norm_eps}, {"weight": name})
    layers, index_of, order = [], {}, []
    for i, layer in enumerate(cfg.layers):
        owner = cfg.owner_of(i)
        if owner != i:
            continue
        p, m = f"l{i}", layer.mixer
        position = {"kind": "none", "params": {}}
        if m.rot is not None:
            position = {"kind": "rope", "params": {
                "rotary_dim": m.rot.dims, "theta": m.rot.base,
                "scaling": m.rot.scaling.as_rope_scaling() if m.rot.scaling is not None else None}}
        parts = {
            "mixer": PartSpec("attention", {
                "hidden_size": cfg.width, "num_heads": m.heads, "num_kv_heads": m.kv_heads, "head_dim": m.dim,
                "value_head_dim": m.vdim, "scale": m.scale, "chunk": m.chunk, "bias": True,
                "qk_norm": {"eps": cfg.norm_eps}, "sink": True, "position": position,
            }, {
                "q": f"{p}.mix.q", "k": f"{p}.mix.k", "v": f"{p}.mix.v", "o": f"{p}.mix.o",
                "q_bias": f"{p}.mix.q.b", "k_bias": f"{p}.mix.k.b", "v_bias": f"{p}.mix.v.b",
                "q_norm": f"{p}.mix.q.norm", "k_norm": f"{p}.mix.k.norm", "sink": f"{p}.mix.sink",
            }, role="mixer"),
            "mixer_norm": norm(f"{p}.norm1"),
        }
        if layer.mlp is not None:
            parts["feed_forward"] = PartSpec("dense", {
                "hidden_size": cfg.width, "intermediate_size": layer.mlp.ff, "activation": "relu2",
            }, {"up": f"{p}.mlp.up", "down": f"{p}.mlp.down"}, role="feed_forward")
            parts["feed_forward_norm"] = norm(f"{p}.norm2")
        index_of[i] = len(layers)
        layers.append(LayerSpec(block="output_norm", parts=parts))
    for i in range(len(cfg.layers)):
        order.append(index_of[cfg.owner_of(i)])
    return ModelPlan(
        hidden_size=cfg.width,
        vocab_size=cfg.vocab,
        embedding=PartSpec("embedding", {"vocab_size": cfg.vocab, "hidden_size": cfg.width,
                                         "scale": cfg.embedding_scale}, {"weight": "embed"}),
        layers=layers,
        final_norm=norm("final.norm"),
        head=PartSpec("head", {"vocab_size": cfg.vocab, "hidden_size": cfg.width, "tied": False}, {"weight": "head"}),
        order=order,
    )


register_architecture("Feduzen", FeduzenConfig.from_dict, feduzen_plan, replace=True)
