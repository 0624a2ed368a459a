"""Small Podurax configurations for the tests and the folders they are written to: random weights made sharp, so that
a misplaced key, a window one token off, a lost state or a sink left out moves the logits by far more than rounding."""
import copy
import json
import math
import os

import torch


def attention(heads, kv_heads, dim, vdim, scale, base, dims, window=None, keep_first=0, v_mix=True, scaling=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "v_mix": v_mix,
         "rot": {"base": base, "dims": dims}}
    if scaling:
        m["rot"]["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    if window or keep_first:
        m["mask"] = {"size": window, "keep_first": keep_first}
    return {"type": "attention", "mixer": m}


def mamba1(inner, state, dt_rank, conv):
    return {"type": "mamba1", "mixer": {"inner": inner, "state": state, "dt_rank": dt_rank, "conv": conv}}


def layer(mixer, ff):
    return {**mixer, "mlp": {"kind": "dense", "ff": ff} if ff else None}


def model(vocab, width, eps, emb_scale, mult, layers):
    return {"architecture": "Podurax", "vocab": vocab, "width": width, "norm": {"eps": eps}, "embedding": {"scale": emb_scale},
            "residual_mult": mult, "layers": layers}


CONFIGS = {
    # layers that differ in everything: grouped heads with values wider than keys, windows of 20 and 33 with 3 and 5 kept
    # first tokens (two cache groups) and a layer that sees everything and does not mix values, stretched and plain
    # frequencies, a recurrence between them, a layer without feed-forward
    "A": model(300, 64, 1e-5, 2.0, 0.5, [
        layer(attention(4, 2, 16, 24, 0.6, 10000.0, 8, window=20, keep_first=3, scaling=(4.0, 64, 8.0, 1.0)), 96),
        layer(mamba1(96, 6, 5, 4), 80),
        layer(attention(4, 2, 16, 24, 0.55, 500.0, 16, window=33, keep_first=5), None),
        layer(attention(2, 1, 32, 8, 0.3, 300000.0, 4, v_mix=False), 72),
        layer(attention(6, 2, 8, 24, 1.1, 1000.0, 8, window=33, keep_first=5, scaling=(8.0, 32, 4.0, 0.5)), 64),
    ]),
    # a recurrence first and last, values that the design's one model happens to make equal or 1 made otherwise and back:
    # factors of 1, as many kv heads as heads, a rotation over the whole head, a convolution of one tap, one mixing layer
    "B": model(131, 88, 1e-6, 1.0, 1.0, [
        layer(mamba1(40, 17, 3, 2), 56),
        layer(attention(3, 3, 12, 12, 0.7, 2000.0, 12, window=7, keep_first=0), 40),
        layer(mamba1(56, 4, 9, 1), None),
    ]),
    # sizes the matrix-core kernels take: multiples of 16 throughout
    "C": model(512, 128, 1e-5, 0.5, 0.7, [
        layer(attention(4, 2, 64, 64, 0.16, 10000.0, 32, window=48, keep_first=4, scaling=(8.0, 256, 32.0, 1.0)), 192),
        layer(mamba1(256, 16, 8, 4), 192),
        layer(attention(8, 2, 32, 64, 0.3, 10000.0, 16, window=48, keep_first=4), 128),
    ]),
    # a size at which the products take their other kernels (weights in tiles, K in slices, the library for prompts), heads of
    # 96 and 48, a recurrence of 1,024 channels
    "E": model(1000, 512, 1e-5, 1.0, 0.6, [
        layer(attention(8, 2, 96, 96, 0.12, 50000.0, 32, window=128, keep_first=8, scaling=(4.0, 512, 16.0, 2.0)), 1536),
        layer(mamba1(1024, 16, 32, 4), 1536),
        layer(attention(16, 2, 48, 96, 0.2, 50000.0, 48, window=40, keep_first=2), None),
        layer(mamba1(768, 8, 24, 3), 1024),
    ]),
    # nothing a multiple of 8; more kept first tokens than the window is long, and nearly as many
    "D": model(99, 100, 1e-5, 1.5, 0.8, [
        layer(attention(3, 1, 10, 14, 0.9, 3000.0, 6, window=9, keep_first=40), 50),
        layer(mamba1(50, 5, 7, 3), 30),
        layer(attention(2, 1, 18, 14, 0.5, 100.0, 18, window=19, keep_first=17), 22),
    ]),
}


def config(name):
    return copy.deepcopy(CONFIGS[name])


def write_model(folder, cfg, seed, gain=1.0):
    """config.json and model.safetensors with seeded weights, bfloat16-representable, shaped so that faults show: norm
    weights away from 1, query/key projections with a gain (peaked attention), biases that matter, step sizes and
    decays over the range a trained recurrence has."""
    from safetensors.torch import save_file
    from inferflux_amd.config import config_from_dict
    from inferflux_amd.engine.model import Model
    g = torch.Generator().manual_seed(seed)
    specs = Model.param_specs_for(config_from_dict(cfg))
    tensors = {}
    for name, spec in specs.items():
        shape = tuple(spec.shape)
        if name.endswith(("norm", "norm1", "norm2")):
            t = 1.0 + 0.3 * torch.randn(shape, generator=g)
        elif name.endswith(".vmix"):
            t = 0.25 + 0.5 * torch.rand(shape, generator=g)
        elif name.endswith(".A_log"):
            t = torch.log(1.0 + 15.0 * torch.rand(shape, generator=g))
        elif name.endswith(".dt.b"):
            t = -4.0 + 3.5 * torch.rand(shape, generator=g)
        elif name.endswith(".D"):
            t = 1.0 + 0.5 * torch.randn(shape, generator=g)
        elif name.endswith(".conv"):
            t = torch.randn(shape, generator=g) * 0.6
        elif name.endswith(".b"):
            t = torch.randn(shape, generator=g) * 0.3
        else:
            t = torch.randn(shape, generator=g) / (shape[-1] ** 0.5)
            if name.endswith((".mix.q", ".mix.k")):
                t = t * gain
            elif name.endswith(".mix.dt"):
                t = t * 2.0
            elif name == "embed":
                t = t * shape[-1] ** 0.5
        tensors[name] = t.to(torch.bfloat16).contiguous()
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file(tensors, os.path.join(folder, "model.safetensors"))
    return folder


def load_plain(folder):
    """(config, tensors as float64 arrays) for the plain implementation."""
    from safetensors.torch import load_file
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    return cfg, {k: v.to(torch.float64).numpy() for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}
