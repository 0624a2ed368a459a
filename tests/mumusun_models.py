"""Small Mumusun configurations for the tests and the folders they are written to: random weights made sharp, so that
a misplaced key, a wrong expert or a norm left out moves the logits by far more than rounding does."""
import copy
import json
import os

import torch


def _mixer(heads, dim, rot_dim, vdim, q_rank, kv_rank, scale, base, dims=None, window=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank, "scale": scale,
         "rot": {"base": base, "dims": rot_dim if dims is None else dims}}
    if window:
        m["mask"] = {"size": window}
    return m


def _moe(experts, top, ff, count=1, keep=1):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top, "groups": {"count": count, "keep": keep}}}


def _layer(mixer, mlp):
    return {"type": "latent_attention", "mixer": mixer, "mlp": mlp}


CONFIGS = {
    # layers that differ in everything: windows of 20 and 33 and none (three cache groups), a rotation over part of the
    # rotated dimensions, a layer without feed-forward, one expert of six, groups 4 -> 2
    "P": {"architecture": "Mumusun", "vocab": 300, "width": 64, "norm": {"eps": 1e-5}, "layers": [
        _layer(_mixer(3, 16, 8, 24, 40, 32, 0.2, 10000.0, window=20), _moe(8, 3, 48, 4, 2)),
        _layer(_mixer(2, 8, 16, 8, 16, 48, 0.25, 500.0, dims=8, window=33), None),
        _layer(_mixer(4, 24, 4, 12, 24, 40, 0.19, 300000.0), _moe(6, 1, 40)),
    ]},
    # one head, one group kept of three, top 2, widths that are no multiples of 8 or 16, a window shorter than a page
    "Q": {"architecture": "Mumusun", "vocab": 131, "width": 88, "norm": {"eps": 1e-6}, "layers": [
        _layer(_mixer(1, 20, 12, 28, 36, 44, 0.18, 1000.0, window=7), _moe(9, 2, 56, 3, 1)),
        _layer(_mixer(5, 12, 6, 10, 20, 26, 0.24, 2000.0, dims=4, window=40), _moe(4, 4, 24, 2, 2)),
    ]},
    # sizes the matrix-core kernels take: multiples of 16 throughout, a window of 48
    "R": {"architecture": "Mumusun", "vocab": 512, "width": 128, "norm": {"eps": 1e-5}, "layers": [
        _layer(_mixer(4, 32, 16, 32, 64, 48, 0.144, 10000.0, window=48), _moe(8, 2, 64, 2, 1)),
        _layer(_mixer(4, 32, 16, 32, 64, 48, 0.144, 10000.0), _moe(8, 2, 64, 4, 3)),
    ]},
    # nothing a multiple of 8: every product takes its general path (the vector loads and matrix-core tiles do not apply)
    "S": {"architecture": "Mumusun", "vocab": 99, "width": 100, "norm": {"eps": 1e-5}, "layers": [
        _layer(_mixer(3, 10, 6, 14, 30, 27, 0.25, 3000.0, dims=6, window=19), _moe(5, 2, 50)),
        _layer(_mixer(2, 18, 2, 9, 21, 35, 0.22, 100.0, window=1000), _moe(6, 3, 22, 3, 2)),
    ]},
}


def config(name):
    return copy.deepcopy(CONFIGS[name])


def router_values(n):
    """n distinct router logits between -2.3 and 2.9, unevenly spaced (no two pairs of them have nearly the same sum of
    sigmoids, as values that mirror each other around zero would)."""
    import math
    return [-2.3 + 5.2 * k / max(n - 1, 1) + 0.11 * math.sin(1.7 * k + 0.3) for k in range(n)]


def write_model(folder, cfg, seed, gain=4.0, decisive_router=False):
    """config.json and model.safetensors with seeded weights, bfloat16-representable, shaped so that faults show:
    large query and key projections (peaked attention), large routers (clear choices), norm weights away from 1.

    With ``decisive_router`` no choice of experts is a close call, so that an engine that rounds its activations to
    bfloat16 makes the choices of the exact model: expert e's router row reads channel e of the stream alone, a
    token's embedding holds a permutation of ``router_values`` on those channels, and the layers' norms have weight 0
    there, so the channels keep the embedding's values through every layer."""
    from safetensors.torch import save_file
    from inferflux_amd.config import config_from_dict
    from inferflux_amd.engine.model import Model
    g = torch.Generator().manual_seed(seed)
    specs = Model.param_specs_for(config_from_dict(cfg))
    tensors = {}
    for name, spec in specs.items():
        if name.endswith(("norm", "norm1", "norm2")):
            t = 1.0 + 0.3 * torch.randn(spec.shape, generator=g)
        else:
            t = torch.randn(spec.shape, generator=g) / (spec.shape[-1] ** 0.5)
            if name.endswith((".uq", ".dkv", ".uk")):
                t = t * gain ** 0.5
            elif name.endswith(".router"):
                t = t * 3.0
            elif name == "embed":
                t = t * spec.shape[-1] ** 0.5
        tensors[name] = t.to(torch.bfloat16).contiguous()
    if decisive_router:
        n = max([L["mlp"]["router"]["experts"] for L in cfg["layers"] if L["mlp"] is not None], default=0)
        values = torch.tensor(router_values(n))
        for tok in range(cfg["vocab"]):
            tensors["embed"][tok, :n] = values[torch.randperm(n, generator=g)].to(torch.bfloat16)
        for i, L in enumerate(cfg["layers"]):
            tensors[f"l{i}.norm1"][:n] = 0
            if L["mlp"] is not None:
                tensors[f"l{i}.norm2"][:n] = 0
                E = L["mlp"]["router"]["experts"]
                tensors[f"l{i}.mlp.router"] = torch.eye(E, cfg["width"]).to(torch.bfloat16)
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file(tensors, os.path.join(folder, "model.safetensors"))
    return folder
