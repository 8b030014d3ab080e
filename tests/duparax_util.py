"""Small Duparax models for the tests: configurations, random weights by tensor name, model folders. The names and
shapes of the tensors are written out here from the design, not taken from the package."""

from __future__ import annotations

import json
import math
from pathlib import Path

import torch

import plain_duparax as plain
from distie_amd.weights.safetensors_io import write_safetensors

RANK = "rank"        # the decay's rank is not a key of the design's config.json: the tensors tell it


def dense(ff=80):
    return {"kind": "dense", "ff": ff}


def moe(experts=6, top=2, ff=24, shared=40):
    out = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff}}
    if shared:
        out["shared"] = {"ff": shared}
    return out


def parallel_layer(heads=4, kv_heads=2, dim=16, vdim=24, scale=0.3, coef=0.7, every=5, r_heads=2, r_dim=8, r_vdim=16,
                   tau=4.0, rank=6, mlp="dense"):
    left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if every:
        left["q_temp"] = {"coef": coef, "every": every}
    right = {"heads": r_heads, "dim": r_dim, "vdim": r_vdim, "tau": tau, RANK: rank}
    return {"type": "parallel", "mixer": {"left": left, "right": right}, "mlp": dense() if mlp == "dense" else mlp}


def rglru_layer(width=64, blocks=4, conv=4, mlp="dense"):
    return {"type": "rglru", "mixer": {"width": width, "blocks": blocks, "conv": conv},
            "mlp": dense() if mlp == "dense" else mlp}


def make_config(layers, vocab=61, width=48, eps=1e-5, logit_scale=0.4):
    cfg = {"architecture": "Duparax", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}
    if logit_scale is not None:
        cfg["logit_scale"] = logit_scale
    return cfg


def file_config(cfg):
    """The config.json of a model folder: without the rank, which a folder's reader takes from the tensors."""
    out = json.loads(json.dumps(cfg))
    for layer in out["layers"]:
        if layer["type"] == "parallel":
            layer["mixer"]["right"].pop(RANK, None)
    return out


def mlp_shapes(p, mlp, C):
    if mlp is None:
        return {}
    if mlp["kind"] == "dense":
        return {p + "gate": (mlp["ff"], C), p + "up": (mlp["ff"], C), p + "down": (C, mlp["ff"])}
    E, F = mlp["router"]["experts"], mlp["expert"]["ff"]
    out = {p + "router": (E, C), p + "router.b": (E,)}
    sizes = [(f"e{e}.", F) for e in range(E)] + ([("shared.", mlp["shared"]["ff"])] if mlp.get("shared") else [])
    for name, size in sizes:
        out.update({p + name + "gate": (size, C), p + name + "up": (size, C), p + name + "down": (C, size)})
    return out


def tensor_shapes(cfg):
    """Checkpoint name -> shape, from the design."""
    C = cfg["width"]
    out = {"embed": (cfg["vocab"], C), "final.norm": (C,), "head": (cfg["vocab"], C)}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        out.update({p + "norm1": (C,), p + "norm1b": (C,)})
        if layer.get("mlp"):
            out.update({p + "norm2": (C,), p + "norm2b": (C,)})
        if layer["type"] == "parallel":
            a, b = m["left"], m["right"]
            H, G, D, E = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
            q = p + "mix.left."
            out.update({q + "q": (H * D, C), q + "q.b": (H * D,), q + "k": (G * D, C), q + "k.b": (G * D,),
                        q + "v": (G * E, C), q + "v.b": (G * E,), q + "o": (C, H * E)})
            H, D, E, r = b["heads"], b["dim"], b["vdim"], b[RANK]
            q = p + "mix.right."
            out.update({q + "q": (H * D, C), q + "k": (H * D, C), q + "v": (H * E, C), q + "g": (H * E, C),
                        q + "o": (C, H * E), q + "norm": (E,), q + "a1": (r, C), q + "a2": (H * D, r), q + "a2.b": (H * D,)})
            out.update({p + "mix.left.out": (C,), p + "mix.right.out": (C,)})
        else:
            R, B = m["width"], m["blocks"]
            q = p + "mix."
            out.update({q + "y": (R, C), q + "y.b": (R,), q + "x": (R, C), q + "x.b": (R,), q + "conv": (R, m["conv"]),
                        q + "conv.b": (R,), q + "ra": (B, R // B, R // B), q + "ra.b": (B, R // B),
                        q + "ri": (B, R // B, R // B), q + "ri.b": (B, R // B), q + "lam": (R,), q + "o": (C, R)})
        out.update(mlp_shapes(p + "mlp.", layer.get("mlp"), C))
    return out


def random_weights(cfg, seed=0, dtype=torch.float32):
    """Values that keep every mechanism alive: projections ~ N(0, 1/in), norm weights near 1, decays spread between
    fast and slow, filters with a strong newest tap, router logits far apart. Rounded to `dtype` (the oracle then
    computes with what the file holds)."""
    g = torch.Generator().manual_seed(seed)
    rnd = lambda *shape: torch.randn(*shape, generator=g)
    w = {}
    for name, shape in tensor_shapes(cfg).items():
        last = name.split(".")[-1]
        parts = name.split(".")
        if "norm" in last or last == "out":
            t = 1.0 + 0.2 * rnd(*shape)
        elif name.endswith("a2.b"):
            t = 1.0 + 1.5 * rnd(*shape)
        elif name.endswith("router.b"):
            t = 0.5 * rnd(*shape)
        elif last == "b":
            t = 0.5 * rnd(*shape)
        elif last == "conv":
            t = 0.3 * rnd(*shape)
            t[:, -1] += 1.0
        elif last == "lam":
            t = rnd(*shape) - 1.0
        elif last == "router":
            t = 3.0 * rnd(*shape) / math.sqrt(shape[-1])
        elif name == "embed":
            t = rnd(*shape)
        elif last in ("ra", "ri"):
            t = 1.5 * rnd(*shape) / math.sqrt(shape[-1])
        else:
            t = rnd(*shape) / math.sqrt(shape[-1])
            if last in ("q", "k") and "left" in parts:
                t = t * 1.5
        w[name] = t.to(dtype)
    return w


def write_model(folder, cfg, weights) -> Path:
    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    (folder / "config.json").write_text(json.dumps(file_config(cfg)))
    names = list(weights)
    write_safetensors(folder / "model.safetensors", [(n, weights[n].dtype, tuple(weights[n].shape)) for n in names],
                      ((n, weights[n].contiguous()) for n in names), {"format": "pt"})
    return folder


def oracle(cfg, weights, ids):
    """float64 logits of the plain implementation as float32 [T, vocab]."""
    return plain.forward(cfg, weights, ids)[0].float()


def close_calls(cfg, weights, ids):
    """For every position, two measures of how much rounding can change what the token computes (both 1.0 where the
    model has nothing of the kind): the smallest gap between the last chosen and the first unchosen router logit over
    the routed layers, relative to the largest logit of its row; and the smallest size of a gated linear attention
    head's output in front of its norm, relative to the root of the sum of its terms' squares (what terms of random
    signs would leave; an output that is what is left of a cancellation, as the first token's is when its query and key are
    nearly orthogonal, comes out of the norm with a size and sign that rounding decides). A token that is large in
    both is computed the same way in bfloat16."""
    w = {n: t.double() for n, t in weights.items()}
    eps = float(cfg["norm"]["eps"])
    T = len(ids)
    gaps, sizes = torch.ones(T, dtype=torch.float64), torch.ones(T, dtype=torch.float64)
    x = w["embed"][torch.tensor(ids)]
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = plain.rms_norm(x, w[p + "norm1"], eps)
        if layer["type"] == "parallel":
            m, r = layer["mixer"]["right"], p + "mix.right."
            H, D, E = m["heads"], m["dim"], m["vdim"]
            q = (h @ w[r + "q"].T).view(T, H, D) * D ** -0.5
            k, v = (h @ w[r + "k"].T).view(T, H, D), (h @ w[r + "v"].T).view(T, H, E)
            z = (h @ w[r + "a1"].T) @ w[r + "a2"].T + w[r + "a2.b"]
            o = plain.gated_linear_recurrence(q, k, v, torch.sigmoid(z).pow(1.0 / float(m["tau"])).view(T, H, D))
            alpha = torch.sigmoid(z).pow(1.0 / float(m["tau"])).view(T, H, D)
            spread = plain.gated_linear_recurrence(q ** 2, k ** 2, v ** 2, alpha ** 2)     # the terms' squares, summed
            sizes = torch.minimum(sizes, (o.pow(2).mean(-1) / spread.mean(-1)).sqrt().min(-1).values)
            right = (plain.rms_norm(o, w[r + "norm"], eps).reshape(T, H * E) * plain.silu(h @ w[r + "g"].T)) @ w[r + "o"].T
            left = plain.left_mixer(h, w, p + "mix.left.", layer["mixer"]["left"])
            y = 0.5 * (plain.rms_norm(left, w[p + "mix.left.out"], eps) + plain.rms_norm(right, w[p + "mix.right.out"], eps))
        else:
            y = plain.rglru_mixer(h, w, p + "mix.", layer["mixer"])
        x = x + plain.rms_norm(y, w[p + "norm1b"], eps)
        mlp = layer.get("mlp")
        if not mlp:
            continue
        h = plain.rms_norm(x, w[p + "norm2"], eps)
        if mlp["kind"] == "moe" and mlp["router"]["top"] < mlp["router"]["experts"]:
            z = h @ w[p + "mlp.router"].T + w[p + "mlp.router.b"]
            s = torch.sort(z, dim=-1, descending=True).values
            k = mlp["router"]["top"]
            gaps = torch.minimum(gaps, (s[:, k - 1] - s[:, k]) / z.abs().max(-1).values)
        x = x + plain.rms_norm(plain.feed_forward(h, w, p + "mlp.", mlp), w[p + "norm2b"], eps)
    return gaps, sizes


def random_ids(cfg, n, seed):
    return torch.randint(0, cfg["vocab"], (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def clear_ids(cfg, weights, n, seed, margin=0.12, size=0.15):
    """`n` random token ids none of which hangs on a close call (`close_calls`): the first token that does is drawn
    again (what stands before it stays as it is, being causal), until none is left."""
    g = torch.Generator().manual_seed(seed)
    ids = torch.randint(0, cfg["vocab"], (n,), generator=g).tolist()
    for _ in range(40 * n):
        gaps, sizes = close_calls(cfg, weights, ids)
        close = ((gaps < margin) | (sizes < size)).nonzero()
        if not len(close):
            return ids
        ids[int(close[0])] = int(torch.randint(0, cfg["vocab"], (1,), generator=g))
    raise AssertionError("no sequence without a close call found")


def logit_error(got, want):
    """Per row: root mean square of the difference (its mean taken off), over that of the wanted logits."""
    d = got.double() - want.double()
    d = d - d.mean(-1, keepdim=True)
    ref = want.double() - want.double().mean(-1, keepdim=True)
    return (d.pow(2).mean(-1).sqrt() / ref.pow(2).mean().sqrt()).float()


TOL = {torch.float32: 5e-5, torch.bfloat16: 6e-2}
