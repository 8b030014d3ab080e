"""Small Musutar models for the tests: configurations, random weights by tensor name, model folders, and replays
of requests through the step function under different ways of cutting. The names and shapes of the tensors are
written out here from the design, not taken from the package."""

from __future__ import annotations

import json
import math
from pathlib import Path

import torch

import plain_musutar as plain
from distie_amd.weights.safetensors_io import write_safetensors


def attention_layer(heads=4, kv_heads=2, dim=16, vdim=16, conv=4, window=12, rot_dims=8, base=100.0, scaling=True,
                    scale=0.3, kv_from=None, ff=80):
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if conv:
        mixer["conv"] = conv
    if window:
        mixer["mask"] = {"size": window}
    if rot_dims:
        mixer["rot"] = {"base": base, "dims": rot_dims}
        if scaling:
            mixer["rot"]["scaling"] = {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 1.0}
    if kv_from is not None:
        mixer["kv_from"] = kv_from
    return {"type": "attention", "mixer": mixer, "mlp": {"kind": "dense", "ff": ff} if ff else None}


def lightning_layer(heads=2, dim=8, vdim=16, decay=(0.7, 0.97), ff=80):
    return {"type": "lightning", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay)},
            "mlp": {"kind": "dense", "ff": ff} if ff else None}


def make_config(layers, vocab=61, width=48, streams=2, taps=3, eps=1e-5):
    cfg = {"architecture": "Musutar", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}
    if streams is not None:
        cfg["streams"] = streams
    if taps:
        cfg["canon"] = {"taps": taps}
    return cfg


def tensor_shapes(cfg):
    """Checkpoint name -> shape, from the design."""
    C, S = cfg["width"], cfg.get("streams")
    taps = (cfg.get("canon") or {}).get("taps", 0)
    out = {"embed": (cfg["vocab"], C), "final.norm": (C,), "head": (cfg["vocab"], C)}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        subs = (1, 2) if layer.get("mlp") else (1,)
        for q in subs:
            out[p + f"norm{q}"] = (C,)
            out[p + f"rg{q}"] = (C, C)
            out[p + f"rg{q}.b"] = (C,)
            if S is not None:
                out[p + f"hc{q}.in"], out[p + f"hc{q}.out"], out[p + f"hc{q}.mix"] = (S,), (S,), (S, S)
        if taps:
            out[p + "canon1"] = (C, taps)
        H, D, E = m["heads"], m["dim"], m["vdim"]
        if layer["type"] == "attention":
            G = m["kv_heads"]
            rows = {"q": H * D}
            if m.get("kv_from") is None:
                rows.update({"k": G * D, "v": G * E})
            for name, n in rows.items():
                out[p + "mix." + name] = (n, C)
                if m.get("conv"):
                    out[p + "mix." + name + ".conv"] = (n, m["conv"])
            out[p + "mix.g"], out[p + "mix.o"] = (H * E, C), (C, H * E)
        else:
            out.update({p + "mix.q": (H * D, C), p + "mix.k": (H * D, C), p + "mix.v": (H * E, C),
                        p + "mix.g": (H * E, C), p + "mix.o": (C, H * E), p + "mix.norm": (H * E,)})
        if layer.get("mlp"):
            out[p + "mlp.up"], out[p + "mlp.down"] = (layer["mlp"]["ff"], C), (C, layer["mlp"]["ff"])
    return out


def random_weights(cfg, seed=0, dtype=torch.float32):
    """Values that keep every mechanism alive: projections ~ N(0, 1/in), norm weights near 1, stream weights near
    an even read, a near-identity mix and a full write, filters with a strong newest tap, gates around one half.
    Rounded to `dtype` (the oracle then computes with what the file holds)."""
    g = torch.Generator().manual_seed(seed)
    rnd = lambda *shape: torch.randn(*shape, generator=g)
    S = cfg.get("streams")
    w = {}
    for name, shape in tensor_shapes(cfg).items():
        last = name.split(".")[-1]
        if "norm" in last:
            t = 1.0 + 0.2 * rnd(*shape)
        elif last == "in":
            t = 1.0 / S + 0.2 * rnd(*shape)
        elif last == "out":
            t = 1.0 + 0.2 * rnd(*shape)
        elif last == "mix":
            t = torch.eye(S) + 0.15 * rnd(*shape)
        elif last == "conv" or last == "canon1":
            t = 0.3 * rnd(*shape)
            t[:, -1] += 1.0 if last == "conv" else 0.0
        elif last == "b":
            t = 0.5 * rnd(*shape)
        elif name == "embed":
            t = rnd(*shape)
        else:
            t = rnd(*shape) / math.sqrt(shape[-1])
            if last in ("q", "k"):
                t = t * 1.5
        w[name] = t.to(dtype)
    return w


def write_model(folder, cfg, weights) -> Path:
    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    (folder / "config.json").write_text(json.dumps(cfg))
    names = list(weights)
    write_safetensors(folder / "model.safetensors", [(n, weights[n].dtype, tuple(weights[n].shape)) for n in names],
                      ((n, weights[n].contiguous()) for n in names), {"format": "pt"})
    return folder


def oracle(cfg, weights, ids):
    """float64 logits of the plain implementation as float32 [T, vocab]."""
    return plain.forward(cfg, weights, ids)[0].float()


def logit_error(got, want):
    """Per row: root mean square of the difference (its mean taken off), over that of the wanted logits."""
    d = got.double() - want.double()
    d = d - d.mean(-1, keepdim=True)
    ref = want.double() - want.double().mean(-1, keepdim=True)
    return (d.pow(2).mean(-1).sqrt() / ref.pow(2).mean().sqrt()).float()


TOL = {torch.float32: 5e-5, torch.bfloat16: 6e-2}


def random_ids(cfg, n, seed):
    return torch.randint(0, cfg["vocab"], (n,), generator=torch.Generator().manual_seed(seed)).tolist()
