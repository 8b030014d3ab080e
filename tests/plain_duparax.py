"""A plain, slow implementation of the Duparax decoder, one function per mechanism, in float64 on the CPU.

It is the oracle of the tests: written from the design's equations, it shares no code with the
package. A model is a dict of a configuration (the keys of its config.json) and a dict of tensors
by checkpoint name; a sequence is run whole, token by token where the mechanism is a recurrence.

Notation: T tokens, C = model width, H query heads, G key/value heads, D = per-head size of queries
and keys, E = per-head size of values, R = channels of the recurrent unit, B = its blocks.
"""

from __future__ import annotations

import math

import torch

F = torch.float64


def rms_norm(x, weight, eps):
    """x / sqrt(mean(x^2) + eps) * w over the last dimension."""
    return x / torch.sqrt((x ** 2).mean(-1, keepdim=True) + eps) * weight


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def query_temperature(positions, coef, every):
    """1 + coef * ln(floor((p + 1) / every) + 1) for each position p."""
    steps = torch.div(positions + 1, every, rounding_mode="floor")
    return 1.0 + coef * torch.log(steps.to(F) + 1.0)


def softmax_attention(q, k, v, scale):
    """q [T, H, D], k [T, G, D], v [T, G, E] -> [T, H, E]; query i sees keys j <= i; query head h uses
    key/value head h // (H / G)."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[2], dtype=F)
    for h in range(H):
        g = h // (H // G)
        for i in range(T):
            s = (k[: i + 1, g] @ q[i, h]) * scale
            p = torch.softmax(s, 0)
            out[i, h] = p @ v[: i + 1, g]
    return out


def left_mixer(h, w, p, m):
    """Grouped-query softmax attention with biases, no rotation, a query temperature by position."""
    T = h.shape[0]
    H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w[p + "q"].T + w[p + "q.b"]).view(T, H, D)
    k = (h @ w[p + "k"].T + w[p + "k.b"]).view(T, G, D)
    v = (h @ w[p + "v"].T + w[p + "v.b"]).view(T, G, E)
    temp = m.get("q_temp")
    if temp:
        q = q * query_temperature(torch.arange(T), float(temp["coef"]), int(temp["every"]))[:, None, None]
    o = softmax_attention(q, k, v, float(m["scale"]))
    return o.reshape(T, H * E) @ w[p + "o"].T


def gated_linear_recurrence(q, k, v, alpha):
    """q, k, alpha [T, H, D], v [T, H, E]: S_t = diag(alpha_t) S_(t-1) + k_t v_t^T, o_t = S_t^T q_t, S_0 = 0."""
    T, H, D = q.shape
    E = v.shape[2]
    S = torch.zeros(H, D, E, dtype=F)
    out = torch.zeros(T, H, E, dtype=F)
    for t in range(T):
        S = alpha[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        out[t] = torch.einsum("hde,hd->he", S, q[t])
    return out


def right_mixer(h, w, p, m, eps):
    """Gated linear attention: a decay per key channel from a low-rank projection."""
    T = h.shape[0]
    H, D, E = m["heads"], m["dim"], m["vdim"]
    q = (h @ w[p + "q"].T).view(T, H, D) * D ** -0.5
    k = (h @ w[p + "k"].T).view(T, H, D)
    v = (h @ w[p + "v"].T).view(T, H, E)
    z = (h @ w[p + "a1"].T) @ w[p + "a2"].T + w[p + "a2.b"]
    alpha = torch.sigmoid(z).pow(1.0 / float(m["tau"])).view(T, H, D)
    o = gated_linear_recurrence(q, k, v, alpha)
    o = rms_norm(o, w[p + "norm"], eps).reshape(T, H * E)
    return (o * silu(h @ w[p + "g"].T)) @ w[p + "o"].T


def parallel_mixer(h, w, p, m, eps):
    """Both mixers read h; the result is half the sum of their outputs, each RMS-normed over C first."""
    left = rms_norm(left_mixer(h, w, p + "left.", m["left"]), w[p + "left.out"], eps)
    right = rms_norm(right_mixer(h, w, p + "right.", m["right"], eps), w[p + "right.out"], eps)
    return 0.5 * (left + right)


def causal_conv(u, w, b):
    """u [T, N], w [N, taps], b [N] -> y_t = b + sum_j w[:, j] * u_(t - taps + 1 + j), zeros before the start."""
    T, N = u.shape
    taps = w.shape[1]
    y = b.expand(T, N).clone()
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                y[t] += w[:, j] * u[s]
    return y


def block_diagonal(u, w, b):
    """u [T, R] in B equal parts, w [B, R/B, R/B] ([out, in] each), b [B, R/B] -> [T, R]."""
    T, R = u.shape
    B = w.shape[0]
    parts = u.view(T, B, R // B)
    return (torch.einsum("tbi,boi->tbo", parts, w) + b).reshape(T, R)


def real_gated_recurrence(u, r, i, lam):
    """log a = -8 r softplus(lam); S_t = a S_(t-1) + sqrt(1 - a^2) i u from S = 0, the first token included."""
    T, R = u.shape
    a = torch.exp(-8.0 * r * torch.nn.functional.softplus(lam))
    S = torch.zeros(R, dtype=F)
    out = torch.zeros(T, R, dtype=F)
    for t in range(T):
        S = a[t] * S + torch.sqrt(1.0 - a[t] ** 2) * i[t] * u[t]
        out[t] = S
    return out


def rglru_mixer(h, w, p, m):
    y = gelu_tanh(h @ w[p + "y"].T + w[p + "y.b"])
    u = causal_conv(h @ w[p + "x"].T + w[p + "x.b"], w[p + "conv"], w[p + "conv.b"])
    r = torch.sigmoid(block_diagonal(u, w[p + "ra"], w[p + "ra.b"]))
    i = torch.sigmoid(block_diagonal(u, w[p + "ri"], w[p + "ri.b"]))
    S = real_gated_recurrence(u, r, i, w[p + "lam"])
    return (S * y) @ w[p + "o"].T


def gated_mlp(h, w, p):
    return (silu(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def routed_mlp(h, w, p, mlp):
    """Every token uses the `top` experts with the largest router logits, weighted by the softmax over those
    logits alone; a shared expert, if there is one, is added for every token."""
    top = int(mlp["router"]["top"])
    z = h @ w[p + "router"].T + w[p + "router.b"]
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        chosen = torch.topk(z[t], top).indices
        weight = torch.softmax(z[t][chosen], 0)
        for e, g in zip(chosen.tolist(), weight):
            out[t] += g * gated_mlp(h[t:t + 1], w, p + f"e{e}.")[0]
    if mlp.get("shared"):
        out = out + gated_mlp(h, w, p + "shared.")
    return out


def feed_forward(h, w, p, mlp):
    if mlp["kind"] == "dense":
        return gated_mlp(h, w, p)
    return routed_mlp(h, w, p, mlp)


def forward(cfg, weights, ids):
    """ids (list of T token ids) -> (logits [T, vocab], residual stream after every layer [L, T, C]), float64."""
    w = {n: t.to(F) for n, t in weights.items()}
    eps = float(cfg["norm"]["eps"])
    x = w["embed"][torch.tensor(ids, dtype=torch.long)]
    after = []
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = rms_norm(x, w[p + "norm1"], eps)
        if layer["type"] == "parallel":
            y = parallel_mixer(h, w, p + "mix.", layer["mixer"], eps)
        elif layer["type"] == "rglru":
            y = rglru_mixer(h, w, p + "mix.", layer["mixer"])
        else:
            raise ValueError(layer["type"])
        x = x + rms_norm(y, w[p + "norm1b"], eps)
        if layer.get("mlp"):
            h = rms_norm(x, w[p + "norm2"], eps)
            x = x + rms_norm(feed_forward(h, w, p + "mlp.", layer["mlp"]), w[p + "norm2b"], eps)
        after.append(x)
    logits = rms_norm(x, w["final.norm"], eps) @ w["head"].T * float(cfg.get("logit_scale", 1.0))
    return logits, torch.stack(after)
