"""The Mumusun decoder as a plan of parts.

A token's row is looked up in ``embed``; every layer then adds two normed sub-block outputs to the stream,
x <- x + norm1(mixer(x)) and, where the layer has a feed-forward, x <- x + norm2(ffn(x)), the sub-blocks reading the
stream itself (the "outnorm" arrangement); the norms are layer norms with a weight and no bias; after the last
layer the same norm (``final.norm``) and the output matrix ``head``.  The mixer is attention through a latent with a
sliding window and a partly rotated query/key, the feed-forward a mixture of experts with a sigmoid router whose
choice is limited to the best groups of experts and whose weights are the scores as they are.  Layers carry their
own sizes and constants, so each layer's parts are built from that layer's entry of the config.

Tensor names: ``embed``, ``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.mix.*``, ``l<i>.mlp.*``, ``final.norm``, ``head``.
"""
from __future__ import annotations

from ..config.mumusun import MumusunConfig
from ..config.registry import register_architecture
from ..parts.plan import LayerSpec, ModelPlan, PartSpec, ScheduleEntry

GROUP_SCORE_TOP = 2       # a group of experts is scored by the sum of this many of its highest scores


def mumusun_plan(cfg: MumusunConfig) -> ModelPlan:
    layers = []
    for i, L in enumerate(cfg.layers):
        p, m = f"l{i}", L.mixer
        mixer = PartSpec(L.type, {
            "name": f"{p}.mix", "n_heads": m.heads, "dim": m.dim, "rot_dim": m.rot_dim, "v_dim": m.vdim,
            "q_rank": m.q_rank, "kv_rank": m.kv_rank, "scale": m.scale, "eps": cfg.norm_eps, "window": m.window,
            "position": PartSpec("rotary", {"head_dim": m.rot_dim, "rotary_dim": m.rot_dims, "theta": m.rot_base,
                                            "style": "split_half"}),
        })
        ffn = norm_post = None
        if L.mlp is not None:
            ffn = PartSpec("moe", {"name": f"{p}.mlp", "n_experts": L.mlp.experts, "top": L.mlp.top, "ff": L.mlp.ff,
                                   "groups": L.mlp.groups, "keep_groups": L.mlp.keep_groups, "group_top": GROUP_SCORE_TOP,
                                   "scoring": "sigmoid", "renormalize": False})
            norm_post = PartSpec("layernorm", {"name": f"{p}.norm2", "tensor": f"{p}.norm2", "eps": cfg.norm_eps})
        layers.append(LayerSpec(prefix=p, block=PartSpec("outnorm"),
                                norm_in=PartSpec("layernorm", {"name": f"{p}.norm1", "tensor": f"{p}.norm1", "eps": cfg.norm_eps}),
                                mixer=mixer, norm_post=norm_post, ffn=ffn))
    return ModelPlan(
        vocab_size=cfg.vocab, hidden_size=cfg.width, max_position=cfg.max_positions,
        embedding=PartSpec("token_embedding", {"name": "embed", "tensor": "embed", "vocab_size": cfg.vocab}),
        layers=tuple(layers), schedule=tuple(ScheduleEntry(i) for i in range(len(layers))),
        final_norm=PartSpec("layernorm", {"name": "final.norm", "tensor": "final.norm", "eps": cfg.norm_eps}),
        lm_head=PartSpec("linear_head", {"name": "head", "tensor": "head", "vocab_size": cfg.vocab}),
    )


register_architecture(MumusunConfig, mumusun_plan)
