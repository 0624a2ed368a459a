"""The Podurax decoder written out plainly, in float64 on the CPU: one function per mechanism, no cache, no batching,
nothing shared with the engine.  What the engine's kernels are compared with.

A model is (config, tensors): ``config`` the parsed config.json (a dict), ``tensors`` a dict of float64 arrays by the
names the model file uses.  Everything works on one whole sequence [T, ...].
"""
from __future__ import annotations

import math

import numpy as np


def rms(x, eps):
    """x divided by its root mean square over the last axis, eps inside the root."""
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def rms_norm(x, w, eps):
    return rms(x, eps) * w


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z / (1.0 + np.exp(-z))


def softplus(z):
    return np.logaddexp(0.0, z)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def yarn_frequencies(dims, base, scaling):
    """(frequency per pair [dims / 2], the factor on cos and sin).  ``scaling`` None: plain rotary frequencies."""
    i = np.arange(dims // 2, dtype=np.float64)
    f = base ** (-2.0 * i / dims)
    if not scaling:
        return f, 1.0
    factor, original = float(scaling["factor"]), float(scaling["original"])

    def dim_of(turns):
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(dim_of(float(scaling["fast"]))), 0)
    hi = min(math.ceil(dim_of(float(scaling["slow"]))), dims - 1)
    ramp = np.clip((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate(x, positions, dims, base, scaling):
    """x [T, heads, d]: the first ``dims`` dimensions of every head turned, pair (i, i + dims/2) by position * f_i."""
    f, mag = yarn_frequencies(dims, base, scaling)
    a = positions.astype(np.float64)[:, None] * f[None, :]            # [T, dims/2]
    c, s = (np.cos(a) * mag)[:, None, :], (np.sin(a) * mag)[:, None, :]
    h = dims // 2
    u, v = x[..., :h], x[..., h:dims]
    out = x.copy()
    out[..., :h] = u * c - v * s
    out[..., h:dims] = v * c + u * s
    return out


def visible(i, j, size, keep_first):
    """Whether position i sees position j: causal, within the last ``size`` positions (None: all) or among the first
    ``keep_first``."""
    if j > i:
        return False
    return size is None or i - j < size or j < keep_first


def sink_softmax_attention(q, k, v, scale, size, keep_first, sink=True):
    """q [T, H, d], k [T, G, d], v [T, G, dv] -> [T, H, dv].  Weights exp(s_j) / (1 + sum_j exp(s_j)) with ``sink``."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = np.zeros((T, H, v.shape[2]))
    i, j = np.arange(T)[:, None], np.arange(T)[None, :]
    mask = (j <= i) & ((i - j < size if size is not None else True) | (j < keep_first))      # ``visible`` for all pairs
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale                     # [T, T]
        s = np.where(mask, s, -np.inf)
        m = np.maximum(s.max(axis=1, keepdims=True), 0.0 if sink else -np.inf)
        e = np.exp(s - m)
        den = e.sum(axis=1, keepdims=True) + (np.exp(-m) if sink else 0.0)
        out[:, h] = (e / den) @ v[:, g]
    return out


def attention_mixer(h, W, p, m, eps, v_first=None, is_first=False):
    """The attention mixer of layer prefix ``p`` with sizes ``m`` on input h [T, width].  Returns (output, the values
    before mixing, for the layers after the first that mixes)."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ W[p + "q"].T + W[p + "q.b"]).reshape(T, H, d)
    k = (h @ W[p + "k"].T + W[p + "k.b"]).reshape(T, G, d)
    v = (h @ W[p + "v"].T + W[p + "v.b"]).reshape(T, G, dv)
    pos = np.arange(T)
    rot = m["rot"]
    q = rms(rotate(q, pos, rot["dims"], rot["base"], rot.get("scaling")), eps)
    k = rms(rotate(k, pos, rot["dims"], rot["base"], rot.get("scaling")), eps)
    v_own = v
    if m.get("v_mix") and v_first is not None and not is_first:
        lam = float(W[p + "vmix"])
        v = (1.0 - lam) * v + lam * v_first
    mask = m.get("mask") or {}
    o = sink_softmax_attention(q, k, v, m["scale"], mask.get("size"), mask.get("keep_first", 0))
    gate = sigmoid(h @ W[p + "g"].T)                          # [T, H]
    o = o * gate[:, :, None]
    return o.reshape(T, H * dv) @ W[p + "o"].T, v_own


def causal_conv(x, w, b):
    """x [T, C], w [C, taps] (last column the current token's), zeros before the start."""
    T, C = x.shape
    taps = w.shape[1]
    xp = np.concatenate([np.zeros((taps - 1, C)), x])
    y = np.zeros((T, C))
    for j in range(taps):
        y += xp[j:j + T] * w[:, j]
    return y + b


def selective_scan(x, dt, A, B, C, D):
    """x, dt [T, C]; A [C, N]; B, C [T, N]; D [C].  S <- exp(dt A) S + dt x B; y = S C + D x."""
    T, Cn = x.shape
    S = np.zeros(A.shape)
    y = np.zeros((T, Cn))
    for t in range(T):
        S = np.exp(dt[t][:, None] * A) * S + (dt[t] * x[t])[:, None] * B[t][None, :]
        y[t] = S @ C[t] + D * x[t]
    return y


def mamba1_mixer(h, W, p, m):
    inner, N, R = m["inner"], m["state"], m["dt_rank"]
    xz = h @ W[p + "in"].T
    x, z = xz[:, :inner], xz[:, inner:]
    x = silu(causal_conv(x, W[p + "conv"], W[p + "conv.b"]))
    proj = x @ W[p + "x"].T
    dt, B, C = proj[:, :R], proj[:, R:R + N], proj[:, R + N:R + 2 * N]
    dt = softplus(dt @ W[p + "dt"].T + W[p + "dt.b"])
    y = selective_scan(x, dt, -np.exp(W[p + "A_log"]), B, C, W[p + "D"])
    return (y * silu(z)) @ W[p + "o"].T


def dense_ff(h, W, p):
    return (gelu_tanh(h @ W[p + "gate"].T) * (h @ W[p + "up"].T)) @ W[p + "down"].T


def forward(config, W, tokens, return_layers=False):
    """Logits [T, vocab] of one whole sequence (and the stream after every layer)."""
    eps, mult = config["norm"]["eps"], config.get("residual_mult", 1.0)
    x = W["embed"][np.asarray(tokens)] * config.get("embedding", {}).get("scale", 1.0)
    v_first, seen_mix, layers = None, False, []
    for i, L in enumerate(config["layers"]):
        p = f"l{i}."
        h = rms_norm(x, W[p + "norm1"], eps)
        if L["type"] == "attention":
            mixes = bool(L["mixer"].get("v_mix"))
            y, v_own = attention_mixer(h, W, p + "mix.", L["mixer"], eps, v_first, is_first=mixes and not seen_mix)
            if mixes and not seen_mix:
                v_first, seen_mix = v_own, True
        elif L["type"] == "mamba1":
            y = mamba1_mixer(h, W, p + "mix.", L["mixer"])
        else:
            raise ValueError(L["type"])
        x = x + mult * y
        if L.get("mlp") is not None:
            x = x + mult * dense_ff(rms_norm(x, W[p + "norm2"], eps), W, p + "mlp.")
        layers.append(x.copy())
    logits = rms_norm(x, W["final.norm"], eps) @ W["head"].T
    return (logits, np.stack(layers)) if return_layers else logits


def greedy_generate(config, W, prompt, n_new):
    """``n_new`` tokens, each the first maximum of the last position's logits of the whole sequence so far."""
    ids = list(prompt)
    for _ in range(n_new):
        ids.append(int(np.argmax(forward(config, W, ids)[-1])))
    return ids[len(prompt):]
