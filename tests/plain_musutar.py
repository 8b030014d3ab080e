"""A plain, slow implementation of the Musutar decoder, one function per mechanism, in float64 on the CPU.

It is the oracle of the tests: written from the design's equations, it shares no code with the
package. A model is a dict of a configuration (the keys of its config.json) and a dict of tensors
by checkpoint name; a sequence is run whole, token by token where the mechanism is a recurrence.

Notation: T tokens, C = width, S = streams, H query heads, G key/value heads, D = per-head size of
queries and keys, E = per-head size of values.
"""

from __future__ import annotations

import math

import torch

F = torch.float64


def layer_norm(x, weight, eps):
    """(x - mean) / sqrt(var + eps) * w, var = mean of the squared deviations; no bias."""
    mean = x.mean(-1, keepdim=True)
    var = ((x - mean) ** 2).mean(-1, keepdim=True)
    return (x - mean) / torch.sqrt(var + eps) * weight


def rms_norm(x, weight, eps):
    return x / torch.sqrt((x ** 2).mean(-1, keepdim=True) + eps) * weight


def causal_conv(u, w):
    """u [T, N], w [N, taps] -> y_t = sum_j w[:, j] * u_(t - taps + 1 + j), zeros before the start."""
    T, N = u.shape
    taps = w.shape[1]
    y = torch.zeros_like(u)
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                y[t] += w[:, j] * u[s]
    return y


def rotary_frequencies(rot):
    """-> (frequency of each pair [dims / 2], factor on cosine and sine). With `scaling`
    (factor, original, fast, slow) the frequencies between the two corrections are blended
    towards f / factor and both cosine and sine are scaled by 0.1 ln(factor) + 1."""
    dims, base = int(rot["dims"]), float(rot["base"])
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=F)
    scaling = rot.get("scaling")
    if not scaling:
        return f, 1.0
    factor, original = float(scaling["factor"]), float(scaling["original"])

    def dim_of(turns):
        return dims * math.log(original / (2 * math.pi * turns)) / (2 * math.log(base))

    lo = max(math.floor(dim_of(float(scaling["fast"]))), 0)
    hi = min(math.ceil(dim_of(float(scaling["slow"]))), dims - 1)
    ramp = torch.tensor([min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0) for i in range(half)], dtype=F)
    return f / factor * ramp + f * (1 - ramp), 0.1 * math.log(factor) + 1.0


def rotate(x, positions, rot):
    """x [T, heads, D]: the first rot.dims dimensions of each head are rotated, pair (i, i + dims/2)."""
    if not rot:
        return x
    dims = int(rot["dims"])
    half = dims // 2
    f, mag = rotary_frequencies(rot)
    ang = positions.to(F)[:, None] * f[None, :]
    cos, sin = (ang.cos() * mag)[:, None, :], (ang.sin() * mag)[:, None, :]
    a, b = x[..., :half], x[..., half:dims]
    return torch.cat([a * cos - b * sin, b * cos + a * sin, x[..., dims:]], -1)


def windowed_attention(q, k, v, scale, window):
    """q [T, H, D], k [T, G, D], v [T, G, E] -> [T, H, E]; query i sees keys j with 0 <= i - j < window
    (all j <= i without a window); query head h uses key/value head h // (H / G)."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[2], dtype=F)
    for i in range(T):
        first = 0 if window is None else max(0, i - window + 1)
        for h in range(H):
            g = h // (H // G)
            s = (k[first:i + 1, g] @ q[i, h]) * scale
            out[i, h] = torch.softmax(s, 0) @ v[first:i + 1, g]
    return out


def decayed_state_scan(q, k, v, decay):
    """S_t = decay_h S_(t-1) + k_t v_t^T, o_t = S_t^T q_t per head. q, k [T, H, D], v [T, H, E]."""
    T, H, D = q.shape
    E = v.shape[2]
    out = torch.zeros(T, H, E, dtype=F)
    state = torch.zeros(H, D, E, dtype=F)
    rate = torch.tensor([float(d) for d in decay], dtype=F)
    for t in range(T):
        state = rate[:, None, None] * state + k[t][:, :, None] * v[t][:, None, :]
        out[t] = torch.einsum("hde,hd->he", state, q[t])
    return out


def silu(x):
    return x * torch.sigmoid(x)


def attention_mixer(h, w, prefix, cfg, positions, borrowed=None):
    """-> (output [T, C], (keys after convolution and rotation, values after convolution))."""
    T = h.shape[0]
    H, G, D, E = int(cfg["heads"]), int(cfg["kv_heads"]), int(cfg["dim"]), int(cfg["vdim"])

    def projected(name):
        u = h @ w[prefix + name].T
        conv = w.get(prefix + name + ".conv")
        return causal_conv(u, conv) if conv is not None else u

    q = rotate(projected("q").view(T, H, D), positions, cfg.get("rot"))
    if borrowed is None:
        k = rotate(projected("k").view(T, G, D), positions, cfg.get("rot"))
        v = projected("v").view(T, G, E)
    else:
        k, v = borrowed
    window = (cfg.get("mask") or {}).get("size")
    mixed = windowed_attention(q, k, v, float(cfg["scale"]), None if window is None else int(window))
    gated = mixed.reshape(T, H * E) * torch.sigmoid(h @ w[prefix + "g"].T)
    return gated @ w[prefix + "o"].T, (k, v)


def lightning_mixer(h, w, prefix, cfg, eps):
    T = h.shape[0]
    H, D, E = int(cfg["heads"]), int(cfg["dim"]), int(cfg["vdim"])
    q = silu(h @ w[prefix + "q"].T).view(T, H, D)
    k = silu(h @ w[prefix + "k"].T).view(T, H, D)
    v = silu(h @ w[prefix + "v"].T).view(T, H, E)
    mixed = decayed_state_scan(q, k, v, cfg["decay"]).reshape(T, H * E)
    normed = rms_norm(mixed, w[prefix + "norm"], eps)
    return (normed * torch.sigmoid(h @ w[prefix + "g"].T)) @ w[prefix + "o"].T


def squared_relu_mlp(h, w, prefix):
    return (torch.relu(h @ w[prefix + "up"].T) ** 2) @ w[prefix + "down"].T


def forward(config, weights, tokens):
    """-> (logits [T, vocab], the sum of the streams after every layer [layers, T, C])."""
    w = {k: (v.to(F) if v.dtype.is_floating_point else v) for k, v in weights.items()}
    eps = float(config["norm"]["eps"])
    taps = int(config["canon"]["taps"]) if config.get("canon") else 0
    S = int(config.get("streams", 1))
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    T = tokens.shape[0]
    positions = torch.arange(T)
    x = [w["embed"][tokens].clone() for _ in range(S)]
    kept = {}
    after = []
    for i, layer in enumerate(config["layers"]):
        p = f"l{i}."
        for q_index, sub in ((1, "mixer"), (2, "mlp")):
            if sub == "mlp" and not layer.get("mlp"):
                continue
            hc = p + f"hc{q_index}."
            u = sum(w[hc + "in"][s] * x[s] for s in range(S))
            h = layer_norm(u, w[p + f"norm{q_index}"], eps)
            gate = torch.sigmoid(h @ w[p + f"rg{q_index}"].T + w[p + f"rg{q_index}.b"])
            if sub == "mixer":
                m = layer["mixer"]
                if taps:
                    h = h + causal_conv(h, w[p + "canon1"])
                if layer["type"] == "attention":
                    source = m.get("kv_from")
                    y, kv = attention_mixer(h, w, p + "mix.", m, positions, None if source is None else kept[int(source)])
                    kept[i] = kv
                elif layer["type"] == "lightning":
                    y = lightning_mixer(h, w, p + "mix.", m, eps)
                else:
                    raise ValueError(layer["type"])
            else:
                if layer["mlp"]["kind"] != "dense":
                    raise ValueError(layer["mlp"]["kind"])
                y = squared_relu_mlp(h, w, p + "mlp.")
            y = y * gate
            x = [sum(w[hc + "mix"][s, t] * x[s] for s in range(S)) + w[hc + "out"][t] * y for t in range(S)]
        after.append(sum(x))
    final = layer_norm(sum(x), w["final.norm"], eps)
    return final @ w["head"].T, torch.stack(after)
