"""Small Nogidra configurations and weights for the tests, made here from the design's naming alone (the product's
list of tensors is checked against this, not used to make it)."""
from __future__ import annotations

import json
import math
import os
from typing import Dict

import numpy as np
import torch


def attention(heads, kv_heads, dim, vdim, taps=4, mask=None, q_temp=(0.5, 16), scale=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale if scale is not None else dim ** -0.5}
    if taps is not None:
        m["conv"] = taps
    if q_temp is not None:
        m["q_temp"] = {"coef": q_temp[0], "every": q_temp[1]}
    if mask is not None:
        m["mask"] = {"size": mask}
    return {"type": "attention", "mixer": m}


def latent(heads, dim, rot_dim, vdim, kv_rank, base=10000.0, mask=None, scale=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank,
         "scale": scale if scale is not None else (dim + rot_dim) ** -0.5, "rot": {"dims": rot_dim, "base": base}}
    if mask is not None:
        m["mask"] = {"size": mask}
    return {"type": "latent_attention", "mixer": m}


def parallel(left, right, left_scale=0.5, right_scale=0.5):
    """``left`` = (heads, kv_heads, dim, vdim, rotated elements, base, mask), ``right`` = (heads, vdim, state, groups,
    norm_groups, taps)."""
    heads, kv_heads, dim, vdim, dims, base, mask = left
    l = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": dim ** -0.5, "rot": {"dims": dims, "base": base}}
    if mask is not None:
        l["mask"] = {"size": mask}
    r = dict(zip(("heads", "vdim", "state", "groups", "norm_groups", "conv"), right))
    return {"type": "parallel", "mixer": {"left": l, "right": r, "left_scale": left_scale, "right_scale": right_scale}}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def layer(mixer, mlp=None):
    return {**mixer, "mlp": mlp}


def config(width, vocab, layers, eps=1e-5, cap=20.0, max_positions=1024):
    out = {"architecture": "Nogidra", "vocab": vocab, "width": width, "norm": {"eps": eps}, "max_positions": max_positions,
           "layers": layers}
    if cap is not None:
        out["logit_softcap"] = cap
    return out


# Sizes unlike one another: one key/value head and several; keys and values of different sizes; convolutions of 2, 3 and
# 5 taps and none; query factors whose period is passed many times within a test, and none; windows below, at and above
# a page of 16, and none; rotated parts that are a piece of a head and the whole; state-space layers with one group and
# with a group a head, one norm run and several, states that fill no lane evenly; every mixer first, last and between;
# layers without feed-forward; routers that take one expert, several and all; widths that are no multiples of 64; a
# model without a cap on its logits.
SMALL = {
    "A": config(64, 211, [
        layer(attention(4, 2, 16, 24, taps=3, mask=20, q_temp=(0.7, 8)), dense(40)),
        layer(parallel((4, 2, 16, 16, 8, 100.0, 33), (3, 8, 12, 3, 1, 2), 0.8, -0.6), moe(6, 2, 24)),
        layer(latent(3, 8, 8, 12, 24, base=500.0, mask=7), None),
        layer(attention(2, 1, 8, 8, taps=None, mask=None, q_temp=None), moe(4, 1, 16)),
        layer(parallel((2, 1, 24, 8, 24, 10000.0, None), (4, 12, 20, 1, 4, 5), 1.3, 0.4), dense(72)),
    ], cap=12.0),
    "B": config(96, 130, [
        layer(parallel((6, 3, 16, 16, 16, 77.0, 16), (2, 24, 40, 2, 2, 4), 0.7, 1.25), dense(24)),
        layer(latent(1, 24, 16, 40, 16, base=77.0, mask=16), moe(5, 5, 8)),
        layer(attention(6, 6, 8, 16, taps=5, mask=40, q_temp=(-0.2, 3)), None),
        layer(latent(2, 32, 32, 32, 64, base=30000.0), moe(7, 3, 16)),
        layer(attention(3, 1, 32, 8, taps=2, mask=5, q_temp=(1.5, 50)), dense(100)),
    ], eps=1e-6, cap=None),
    "C": config(128, 257, [
        layer(latent(8, 16, 16, 16, 32, base=1000.0, mask=24), moe(16, 4, 32)),
        layer(attention(8, 2, 32, 32, taps=4, mask=50, q_temp=(0.5, 32)), moe(8, 2, 64)),
        layer(parallel((8, 1, 32, 32, 16, 1000.0, 24), (8, 16, 64, 4, 2, 4), 1.0, 1.0), None),
        layer(latent(4, 32, 64, 32, 128, base=1000.0, mask=5), dense(96)),
    ], cap=50.0),
}


def tensor_shapes(raw: dict) -> Dict[str, tuple]:
    w, shapes = raw["width"], {}
    shapes["embed"] = (raw["vocab"], w)
    for i, entry in enumerate(raw["layers"]):
        p, m, f = f"l{i}.", entry["mixer"], entry["mlp"]
        shapes[p + "norm1"] = (w,)
        x = p + "mix."
        if entry["type"] == "attention":
            qw, kw, vw = m["heads"] * m["dim"], m["kv_heads"] * m["dim"], m["kv_heads"] * m["vdim"]
            shapes.update({x + "q": (qw, w), x + "k": (kw, w), x + "v": (vw, w), x + "g": (m["heads"], w),
                           x + "o": (w, m["heads"] * m["vdim"])})
            if m.get("conv"):
                shapes.update({x + "q.conv": (qw, m["conv"]), x + "k.conv": (kw, m["conv"]), x + "v.conv": (vw, m["conv"])})
        elif entry["type"] == "latent_attention":
            shapes.update({x + "q": (m["heads"] * (m["dim"] + m["rot_dim"]), w), x + "dkv": (m["kv_rank"] + m["rot_dim"], w),
                           x + "dkv.norm": (m["kv_rank"],), x + "uk": (m["heads"] * m["dim"], m["kv_rank"]),
                           x + "uv": (m["heads"] * m["vdim"], m["kv_rank"]), x + "o": (w, m["heads"] * m["vdim"])})
        else:
            l, r = m["left"], m["right"]
            qw, kw, vw = l["heads"] * l["dim"], l["kv_heads"] * l["dim"], l["kv_heads"] * l["vdim"]
            y = x + "left."
            shapes.update({y + "q": (qw, w), y + "q.b": (qw,), y + "k": (kw, w), y + "k.b": (kw,), y + "v": (vw, w),
                           y + "v.b": (vw,), y + "q.norm": (qw,), y + "k.norm": (kw,), y + "o": (w, l["heads"] * l["vdim"])})
            inner, bc = r["heads"] * r["vdim"], r["groups"] * r["state"]
            y = x + "right."
            shapes.update({y + "in": (2 * inner + 2 * bc + r["heads"], w), y + "conv": (inner + 2 * bc, r["conv"]),
                           y + "conv.b": (inner + 2 * bc,), y + "dt_bias": (r["heads"],), y + "A_log": (r["heads"],),
                           y + "D": (r["heads"],), y + "norm": (inner,), y + "o": (w, inner)})
        if f is None:
            continue
        shapes[p + "norm2"] = (w,)
        y = p + "mlp."
        if f["kind"] == "dense":
            shapes.update({y + "gate": (f["ff"], w), y + "gate.b": (f["ff"],), y + "up": (f["ff"], w), y + "up.b": (f["ff"],),
                           y + "down": (w, f["ff"]), y + "down.b": (w,)})
        else:
            shapes[y + "router"] = (f["router"]["experts"], w)
            for e in range(f["router"]["experts"]):
                ff = f["expert"]["ff"]
                shapes.update({f"{y}e{e}.gate": (ff, w), f"{y}e{e}.up": (ff, w), f"{y}e{e}.down": (w, ff)})
    shapes["final.norm"] = (w,)
    shapes["head"] = (raw["vocab"], w)
    return shapes


def make_weights(raw: dict, seed: int, dtype=torch.bfloat16, sharpen: float = 1.0) -> Dict[str, torch.Tensor]:
    """Weights at which every mechanism matters: projections that keep activations of order 1, norm weights around zero,
    biases of order 1/2, filters whose taps all count, a router whose outputs spread, decays that reach from a few tokens
    to hundreds back, step sizes on both sides of 1.  ``sharpen`` scales the query projections, so that scores spread and
    a misplaced key moves the logits.  Rounded to ``dtype``."""
    gen = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(raw).items():
        parts = name.split(".")
        last = parts[-1]
        if last in ("norm1", "norm2") or name == "final.norm":
            t = 0.2 * torch.randn(shape, generator=gen)                      # the gain is 1 + this
        elif last == "norm":
            t = 1.0 + 0.2 * torch.randn(shape, generator=gen)                # plain gains
        elif last == "conv":
            t = 0.5 * torch.randn(shape, generator=gen)
            t[:, -1] += 1.0
        elif last == "b":
            t = 0.5 * torch.randn(shape, generator=gen)
        elif last == "router":
            t = torch.randn(shape, generator=gen) * (3.0 / math.sqrt(shape[-1]))
        elif last == "A_log":
            t = torch.rand(shape, generator=gen) * 5.0 - 4.0                 # rates from 0.02 to 2.7 a unit of step size
        elif last == "dt_bias":
            t = torch.randn(shape, generator=gen) - 0.5
        elif last == "D":
            t = 1.0 + 0.5 * torch.randn(shape, generator=gen)
        elif last == "q":
            t = torch.randn(shape, generator=gen) * (1.5 * sharpen / math.sqrt(shape[-1]))
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
