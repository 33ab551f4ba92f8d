"""Small Fosulix configurations and weights for the tests, made here from the design's naming alone (the product's
list of tensors is checked against this, not used to make it)."""
from __future__ import annotations

import json
import math
import os
from typing import Dict

import numpy as np
import torch


def latent(heads, dim, rot_dim, vdim, q_rank, kv_rank, base=10000.0, scaling=None, mask=None, kv_from=None, scale=None,
           dims=None):
    rot = {"dims": rot_dim if dims is None else dims, "base": base}
    if scaling is not None:
        rot["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank,
         "scale": scale if scale is not None else (dim + rot_dim) ** -0.5, "rot": rot}
    if mask is not None:
        m["mask"] = {"size": mask}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": m}


def memory(heads, dim, vdim):
    return {"type": "hgrn2", "mixer": {"heads": heads, "dim": dim, "vdim": vdim}}


def moe(experts, top, ff, limit=2.0, scale=1.0, groups=None):
    router = {"experts": experts, "top": top, "scale": scale}
    if groups is not None:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": router}


def layer(mixer, mlp=None):
    return {**mixer, "mlp": mlp}


def config(width, vocab, layers, eps=1e-5, mult=0.5, embed_scale=1.0, taps=4, max_positions=1024):
    return {"architecture": "Fosulix", "vocab": vocab, "width": width, "norm": {"eps": eps}, "residual_mult": mult,
            "embedding": {"scale": embed_scale}, "canon": {"taps": taps}, "max_positions": max_positions, "layers": layers}


# Sizes unlike one another: one head and several; plain, rotated and value parts of a head all of different sizes;
# latents narrower and wider than the heads; rotation with and without stretched frequencies, of the whole rotated
# part and of a piece of it; windows below, at and above a page of 16, and none; readers of another layer's latents
# with a wider and with a narrower window than the owner's, next to it and layers away; the matrix memory first,
# last and between, with one head and several, key channels that fill no lane evenly; layers without feed-forward;
# routers with and without groups, groups of one, two and more, one expert chosen and several, scale 1 and not;
# 2, 3 and 5 taps; widths that are no multiples of 64.
SMALL = {
    "A": config(64, 211, [
        layer(latent(4, 8, 8, 12, 20, 24, base=10000.0, scaling=(8.0, 64, 32.0, 1.0), mask=20), moe(6, 2, 24, groups=(3, 2), scale=1.5)),
        layer(memory(3, 12, 20), moe(4, 1, 16, limit=1.0)),
        layer(latent(4, 8, 8, 12, 20, 24, base=10000.0, scaling=(8.0, 64, 32.0, 1.0), mask=33, kv_from=0), None),
        layer(latent(2, 16, 4, 8, 12, 40, base=500.0), moe(8, 3, 12, groups=(4, 3), scale=0.7, limit=3.0)),
        layer(latent(3, 16, 4, 24, 30, 40, base=500.0, mask=7, kv_from=3), moe(5, 5, 8)),
    ], mult=0.35, embed_scale=4.0, taps=4),
    "B": config(96, 130, [
        layer(memory(1, 40, 48), moe(9, 4, 8, groups=(9, 5), scale=2.0)),
        layer(latent(1, 24, 16, 40, 48, 16, base=77.0, scaling=(4.0, 32, 8.0, 2.0), mask=16, dims=8), moe(4, 2, 40, groups=(2, 1))),
        layer(memory(5, 8, 8), None),
        layer(latent(3, 8, 16, 8, 16, 16, base=77.0, scaling=(4.0, 32, 8.0, 2.0), mask=40, kv_from=1, dims=8), moe(6, 2, 20, groups=(1, 1))),
        layer(latent(2, 32, 32, 32, 24, 64, base=30000.0, scaling=(16.0, 128, 32.0, 1.0)), moe(7, 3, 16, limit=0.5)),
    ], eps=1e-6, mult=1.0, embed_scale=1.0, taps=2),
    "C": config(128, 257, [
        layer(latent(8, 16, 16, 16, 64, 32, base=1000.0, mask=24), moe(16, 4, 32, groups=(8, 3), scale=2.5)),
        layer(latent(2, 64, 16, 48, 32, 32, base=1000.0, mask=50, kv_from=0), moe(8, 2, 64, groups=(2, 2))),
        layer(latent(4, 32, 64, 32, 96, 128, base=1000.0, scaling=(2.0, 16, 4.0, 1.0), mask=5), None),
        layer(memory(2, 64, 32), moe(4, 4, 32, scale=0.25)),
    ], mult=0.7, embed_scale=11.0, taps=5),
    # latents of 128, 256 and 576 elements in multiples of 32 with parts in multiples of 16: in bfloat16 and pages of 32
    # tokens attention goes to the matrix-core kernel, with 3, 4 and 16 heads (16 heads fill a tile of 16 columns, fewer
    # heads put several rows, in steps of single tokens several requests, into one).  Its mixtures take all their
    # experts, so that no rounded router input changes a choice at an early position and, through attention and memory,
    # every later position with it: what differs from the plain results in bfloat16 is then attention's rounding.
    "D": config(128, 300, [
        layer(latent(4, 16, 64, 16, 32, 64, base=1000.0, scaling=(8.0, 64, 32.0, 1.0), mask=40), moe(4, 4, 32, groups=(2, 2), scale=1.5)),
        layer(latent(16, 8, 64, 8, 64, 64, base=1000.0, scaling=(8.0, 64, 32.0, 1.0), mask=70, kv_from=0), None),
        layer(memory(2, 32, 32), moe(3, 3, 32)),
        layer(latent(3, 32, 32, 24, 48, 224, base=500.0), moe(2, 2, 48, limit=1.0)),
        layer(latent(2, 16, 64, 16, 32, 512, base=10000.0, mask=33), None),
    ], mult=0.5, embed_scale=6.0, taps=3),
}


def tensor_shapes(raw: dict) -> Dict[str, tuple]:
    w, shapes = raw["width"], {}
    shapes["embed"] = (raw["vocab"], w)
    for i, entry in enumerate(raw["layers"]):
        p, m, f = f"l{i}.", entry["mixer"], entry["mlp"]
        shapes[p + "norm1"] = (w,)
        shapes[p + "canon1"] = (w, raw["canon"]["taps"])
        shapes[p + "dwa"] = (i + 2,)
        x = p + "mix."
        if entry["type"] == "hgrn2":
            qk, vv = m["heads"] * m["dim"], m["heads"] * m["vdim"]
            shapes.update({x + "q": (qk, w), x + "f": (qk, w), x + "f.b": (qk,), x + "lower": (qk,), x + "v": (vv, w),
                           x + "norm": (m["vdim"],), x + "o": (w, vv)})
        else:
            shapes.update({x + "dq": (m["q_rank"], w), x + "dq.norm": (m["q_rank"],),
                           x + "uq": (m["heads"] * (m["dim"] + m["rot_dim"]), m["q_rank"]),
                           x + "uk": (m["heads"] * m["dim"], m["kv_rank"]), x + "uv": (m["heads"] * m["vdim"], m["kv_rank"]),
                           x + "o": (w, m["heads"] * m["vdim"])})
            if m.get("kv_from") is None:
                shapes.update({x + "dkv": (m["kv_rank"] + m["rot_dim"], w), x + "dkv.norm": (m["kv_rank"],)})
        if f is None:
            continue
        shapes[p + "norm2"] = (w,)
        y = p + "mlp."
        shapes[y + "router"] = (f["router"]["experts"], w)
        for e in range(f["router"]["experts"]):
            ff = f["expert"]["ff"]
            shapes.update({f"{y}e{e}.gate": (ff, w), f"{y}e{e}.up": (ff, w), f"{y}e{e}.down": (w, ff)})
    shapes["final.norm"] = (w,)
    return shapes


def make_weights(raw: dict, seed: int, dtype=torch.bfloat16, sharpen: float = 1.0) -> Dict[str, torch.Tensor]:
    """Weights at which every mechanism matters: projections that keep activations of order 1, gains around 1, a
    router whose scores spread, gate and up values that reach the experts' limit, lower bounds of the forget gate spread
    over (0, 1) with some close to 1 so that the memory reaches far back, depth weights of both signs.  ``sharpen``
    scales the gain of the query latent's norm, so that scores spread and a misplaced key moves the logits.  Rounded
    to ``dtype``."""
    gen = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(raw).items():
        last = name.split(".")[-1]
        if name.endswith("dq.norm"):
            t = (1.0 + 0.2 * torch.randn(shape, generator=gen)) * sharpen
        elif last in ("norm1", "norm2", "norm"):
            t = 1.0 + 0.2 * torch.randn(shape, generator=gen)
        elif name == "embed":
            t = torch.randn(shape, generator=gen) / raw["embedding"]["scale"]
        elif last == "router":
            t = torch.randn(shape, generator=gen) * (3.0 / math.sqrt(shape[-1]))
        elif last == "lower":
            t = torch.rand(shape, generator=gen) ** 0.3
        elif last == "b":
            t = torch.randn(shape, generator=gen)
        elif last == "canon1":
            t = 0.4 * torch.randn(shape, generator=gen)
        elif last == "dwa":
            t = torch.randn(shape, generator=gen) * (0.5 / math.sqrt(shape[0]))
            t[-1] = 1.0
        elif last in ("gate", "up"):
            t = torch.randn(shape, generator=gen) * (2.5 / math.sqrt(shape[-1]))
        else:
            t = torch.randn(shape, generator=gen) * (1.5 / math.sqrt(shape[-1]))
        out[name] = t.to(dtype)
    return out


def write_dir(path: str, raw: dict, weights: Dict[str, torch.Tensor]) -> str:
    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as handle:
        json.dump(raw, handle)
    save_file({k: v.contiguous() for k, v in weights.items()}, os.path.join(path, "model.safetensors"))
    return path


def relative_error(have: np.ndarray, want: np.ndarray) -> np.ndarray:
    """Per row: root mean square of the difference (its mean taken off, as a logit's shift means nothing) over
    the root mean square of the expected logits."""
    d = have.astype(np.float64) - want.astype(np.float64)
    d = d - d.mean(axis=-1, keepdims=True)
    scale = np.sqrt((want.astype(np.float64) ** 2).mean()) + 1e-30
    return np.sqrt((d * d).mean(axis=-1)) / scale
