"""The Podurax decoder as a plan of parts.

A token's row of ``embed`` times a scale starts the stream; every layer adds x <- x + m * mixer(norm1(x)) and, where
it has a feed-forward, x <- x + m * ff(norm2(x)) (RMS norms, the "prenorm" arrangement with the model's factor m);
after the last layer the model's norm (``final.norm``) and the output matrix ``head``.  A layer's mixer is either

  attention   grouped-query attention with biased projections, a rotation of the first dimensions of every head with
              frequencies stretched for long contexts, q and k brought to unit root mean square after the rotation, a
              sliding window that also keeps the request's first tokens, a softmax with one added to its denominator,
              values mixed with those of the first such layer, and a sigmoid gate per head on the output; or
  mamba1      a selective state-space recurrence behind a short causal convolution,

and its feed-forward is gated with the tanh form of gelu.  Layers carry their own sizes and constants, so each layer's
parts are built from that layer's entry of the config.

Tensor names: ``embed``, ``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.mix.*``, ``l<i>.mlp.*``, ``final.norm``, ``head``; a
bias is its matrix's name with ``.b``.
"""
from __future__ import annotations

from ..config.podurax import PoduraxConfig
from ..config.registry import register_architecture
from ..parts.plan import LayerSpec, ModelPlan, PartSpec, ScheduleEntry

SINK_SCORE = 0.0        # the key without value that every softmax of the design has: exp(0) = 1 added to the denominator


def _attention(p: str, m, cfg: PoduraxConfig, role) -> PartSpec:
    names = {"q": f"{p}.q", "k": f"{p}.k", "v": f"{p}.v", "o": f"{p}.o", "q_bias": f"{p}.q.b", "k_bias": f"{p}.k.b",
             "v_bias": f"{p}.v.b", "gate": f"{p}.g", "mix": f"{p}.vmix"}
    position = PartSpec("rotary", {"head_dim": m.dim, "rotary_dim": m.rot_dims, "theta": m.rot_base, "style": "split_half",
                                   "scaling": m.rot_scaling.to_dict() if m.rot_scaling is not None else None})
    return PartSpec("paged_attention", {
        "name": p, "n_heads": m.heads, "n_kv_heads": m.kv_heads, "head_dim": m.dim, "v_head_dim": m.vdim, "bias": True,
        "scale": m.scale, "window": m.window, "keep_first": m.keep_first, "sink": SINK_SCORE, "unit_norm_eps": cfg.norm_eps,
        "output_gate": True, "value_mix": role, "position": position, "tensors": names})


def _mamba1(p: str, m) -> PartSpec:
    names = {"in": f"{p}.in", "conv": f"{p}.conv", "conv_bias": f"{p}.conv.b", "x": f"{p}.x", "dt": f"{p}.dt",
             "dt_bias": f"{p}.dt.b", "A_log": f"{p}.A_log", "D": f"{p}.D", "out": f"{p}.o"}
    return PartSpec("selective_ssm", {"name": p, "inner": m.inner, "state": m.state, "dt_rank": m.dt_rank, "conv": m.conv,
                                      "tensors": names})


def podurax_plan(cfg: PoduraxConfig) -> ModelPlan:
    layers, mixing_seen = [], False
    norm = lambda name: PartSpec("rmsnorm", {"name": name, "tensor": name, "eps": cfg.norm_eps})
    for i, L in enumerate(cfg.layers):
        p = f"l{i}"
        if L.type == "attention":
            role = None
            if L.mixer.v_mix:          # the first such layer hands its values on, the others mix them in
                role, mixing_seen = ("mix" if mixing_seen else "source"), True
            mixer = _attention(f"{p}.mix", L.mixer, cfg, role)
        else:
            mixer = _mamba1(f"{p}.mix", L.mixer)
        ffn = norm_post = None
        if L.mlp is not None:
            ffn = PartSpec("gated_ffn", {"name": f"{p}.mlp", "intermediate_size": L.mlp.ff, "activation": "gelu_tanh",
                                         "tensors": {"gate": f"{p}.mlp.gate", "up": f"{p}.mlp.up", "down": f"{p}.mlp.down"}})
            norm_post = norm(f"{p}.norm2")
        layers.append(LayerSpec(prefix=p, block=PartSpec("prenorm", {"residual_scale": cfg.residual_mult}),
                                norm_in=norm(f"{p}.norm1"), mixer=mixer, norm_post=norm_post, ffn=ffn))
    return ModelPlan(
        vocab_size=cfg.vocab, hidden_size=cfg.width, max_position=cfg.max_positions,
        embedding=PartSpec("token_embedding", {"name": "embed", "tensor": "embed", "vocab_size": cfg.vocab,
                                               "scale": cfg.embedding_scale}),
        layers=tuple(layers), schedule=tuple(ScheduleEntry(i) for i in range(len(layers))),
        final_norm=norm("final.norm"),
        lm_head=PartSpec("linear_head", {"name": "head", "tensor": "head", "vocab_size": cfg.vocab}),
    )


register_architecture(PoduraxConfig, podurax_plan)
