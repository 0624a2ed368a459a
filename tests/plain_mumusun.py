"""A plain, slow implementation of the Mumusun decoder: whole sequences, no cache, one function per mechanism, on the
CPU.  It shares no code with the engine: config.json is read with json, model.safetensors with the safetensors
package, and every size and constant comes from the config dict.

    layer         x <- x + LN1(mixer(x));  x <- x + LN2(moe(x)) where the layer has a feed-forward
    LN            (x - mean) / sqrt(mean((x - mean)^2) + eps) * w, no bias
    mixer         attention through a latent (see ``latent_attention``)
    feed-forward  mixture of experts with a sigmoid router limited to the best groups (see ``route`` and ``moe``)
    output        LN_final(x) W_head^T
"""
import json
import math
import os

import torch


def load_folder(folder, dtype=torch.float64):
    from safetensors.torch import load_file
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    W = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}
    return cfg, W


def layer_norm(x, w, eps):
    mean = x.mean(-1, keepdim=True)
    var = ((x - mean) ** 2).mean(-1, keepdim=True)
    return (x - mean) / torch.sqrt(var + eps) * w


def rms_norm(x, w, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w


def rotate(x, positions, dims, base):
    """x [S, heads, d]: of each head's first ``dims`` elements, i and i + dims/2 are a pair (u, v) that becomes
    (u cos a - v sin a, v cos a + u sin a) with a = position * base^(-2i/dims); the other elements stay."""
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=x.dtype)
    a = torch.as_tensor(positions, dtype=x.dtype)[:, None] * f[None, :]
    cos, sin = torch.cos(a)[:, None, :], torch.sin(a)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * cos - v * sin, v * cos + u * sin, x[..., dims:]], dim=-1)


def visible(positions, window):
    """[S, S] booleans: query i sees key j when 0 <= i - j, and i - j < window if there is one."""
    p = torch.as_tensor(positions)
    d = p[:, None] - p[None, :]
    ok = d >= 0
    if window:
        ok &= d < window
    return ok


def latent_attention(h, W, p, m, eps, positions):
    """h [S, width].  Queries through a latent of q_rank, keys and values through one of kv_rank; every head's key is
    [W_uk c | the one rotated part] and its value W_uv c, formed here for every position."""
    S = h.shape[0]
    H, d, r, dv, kr = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    cq = rms_norm(h @ W[p + "dq"].T, W[p + "dq.norm"], eps)
    q = (cq @ W[p + "uq"].T).view(S, H, d + r)
    down = h @ W[p + "dkv"].T
    c = rms_norm(down[:, :kr], W[p + "dkv.norm"], eps)
    k_rot = rotate(down[:, None, kr:], positions, m["rot"]["dims"], m["rot"]["base"])[:, 0]        # [S, r], shared by the heads
    k_n = (c @ W[p + "uk"].T).view(S, H, d)
    v = (c @ W[p + "uv"].T).view(S, H, dv)
    q_n, q_r = q[..., :d], rotate(q[..., d:], positions, m["rot"]["dims"], m["rot"]["base"])
    scores = (torch.einsum("ihd,jhd->hij", q_n, k_n) + torch.einsum("ihd,jd->hij", q_r, k_rot)) * m["scale"]
    window = (m.get("mask") or {}).get("size")
    scores = scores.masked_fill(~visible(positions, window), -math.inf)
    a = torch.softmax(scores, dim=-1)
    out = torch.einsum("hij,jhd->ihd", a, v).reshape(S, H * dv)
    return out @ W[p + "o"].T


def route(h, w_router, r):
    """(chosen [S, top] expert indices, s [S, experts] scores).  s = sigmoid(W_r h); the experts form ``count`` equal
    groups of neighbours, a group scores the sum of its two highest s, and the ``top`` highest s are taken among the
    experts of the ``keep`` best groups."""
    E, top = r["experts"], r["top"]
    groups = r.get("groups") or {}
    G, keep = groups.get("count", 1), groups.get("keep", 1)
    s = torch.sigmoid(h @ w_router.T)
    per = E // G
    chosen = []
    for t in range(h.shape[0]):
        gscore = []
        for g in range(G):
            best = sorted((float(x) for x in s[t, g * per:(g + 1) * per]), reverse=True)
            gscore.append(sum(best[:2]))
        kept = sorted(range(G), key=lambda g: -gscore[g])[:keep] if keep < G else list(range(G))
        allowed = [e for e in range(E) if e // per in kept]
        chosen.append(sorted(allowed, key=lambda e: -float(s[t, e]))[:top])
    return torch.tensor(chosen), s


def expert(h, w_gate, w_up, w_down):
    g = h @ w_gate.T
    return ((g * torch.sigmoid(g)) * (h @ w_up.T)) @ w_down.T


def moe(h, W, p, m):
    """sum over the chosen experts of s_e * expert_e(h): the scores as they are, not renormalised."""
    chosen, s = route(h, W[p + "router"], m["router"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e in chosen[t].tolist():
            out[t] += s[t, e] * expert(h[t], W[f"{p}e{e}.gate"], W[f"{p}e{e}.up"], W[f"{p}e{e}.down"])
    return out


def forward(cfg, W, ids, streams=None):
    """Logits [S, vocab]; ``streams`` (a list) receives the stream after every layer."""
    eps = cfg["norm"]["eps"]
    positions = list(range(len(ids)))
    x = W["embed"][torch.as_tensor(ids, dtype=torch.long)]
    for i, L in enumerate(cfg["layers"]):
        assert L["type"] == "latent_attention"
        x = x + layer_norm(latent_attention(x, W, f"l{i}.mix.", L["mixer"], eps, positions), W[f"l{i}.norm1"], eps)
        if L.get("mlp") is not None:
            x = x + layer_norm(moe(x, W, f"l{i}.mlp.", L["mlp"]), W[f"l{i}.norm2"], eps)
        if streams is not None:
            streams.append(x.clone())
    return layer_norm(x, W["final.norm"], eps) @ W["head"].T


def greedy_generate(cfg, W, prompt, n_new):
    ids = list(prompt)
    for _ in range(n_new):
        ids.append(int(forward(cfg, W, ids)[-1].argmax()))
    return ids[len(prompt):]
