"""Nogidra: how its configuration becomes parts.

A small decoder-only design whose config.json lists its layers one by one.  A layer is pre-norm (``prenorm`` block):
x <- x + mixer(norm1(x)), x <- x + ff(norm2(x)), with RMS norms whose stored weights lie around zero (the gain is
1 + weight).  Three mixers:

* ``attention``: grouped-query softmax attention without rotation.  q, k and v each pass a short causal convolution
  behind the projection; the queries at position p count times 1 + coef ln(floor((p + 1) / every) + 1); head h's score for
  a key at distance d is lowered by 2^(-8 (h + 1) / H) d; a sliding window; a sigmoid gate a head on the result.
* ``latent_attention``: queries straight from the input; keys and values out of one normed latent a token and one
  rotated key part that all heads share, which is all the cache holds; rotation in half-split pairs; a sliding window.
* ``parallel``: softmax attention (projections with biases, q and k normed over the whole projection, neighbouring
  pairs rotated on a head's first elements, a window) and a state-space layer with one decay a head (Mamba-2) side by
  side, summed with a weight each.

The feed-forward is gated with silu, dense with biases on all three projections, or a mixture of experts without
biases whose router takes the ``top`` largest outputs and weighs them by the softmax over those alone.  A final norm, an
untied head, logits capped by cap tanh(logits / cap).  Tensor names: ``embed``, ``head``, ``final.norm`` and per layer
``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.mix.*``, ``l<i>.mlp.*``.
"""
from __future__ import annotations

from ..config.nogidra import (BiasedAttentionConfig, DenseConfig, LatentAttentionConfig, NogidraConfig)
from ..parts.base import PartSpec
from ..parts.model import ModelSpec, default_schedule
from .registry import register_architecture


def _norm(config: NogidraConfig, name: str) -> PartSpec:
    return PartSpec("rmsnorm", {"size": config.width, "eps": config.eps, "weight": name, "weight_offset": 1.0})


def _rope(kind: str, dims: int, base: float, positions: dict) -> str:
    name = f"{kind}_{dims}_{base!r}"
    positions.setdefault(name, PartSpec(kind, {"rotary_dim": dims, "theta": base}))
    return name


def distance_slopes(heads: int) -> list:
    """The design's slopes: head h's scores fall by 2^(-8 (h + 1) / heads) a position of distance."""
    return [2.0 ** (-8.0 * (h + 1) / heads) for h in range(heads)]


def _mixer(config: NogidraConfig, i: int, positions: dict) -> PartSpec:
    m, p = config.layers[i].mixer, f"l{i}.mix."
    if isinstance(m, BiasedAttentionConfig):
        params = {"hidden": config.width, "q_heads": m.heads, "kv_heads": m.kv_heads, "head_dim": m.dim,
                  "value_dim": m.vdim, "qk_norm_eps": None, "window": m.window, "scale": m.scale, "position": None,
                  "float_output": True, "q": p + "q", "k": p + "k", "v": p + "v", "o": p + "o", "gate": p + "g",
                  "distance_slopes": distance_slopes(m.heads)}
        if m.taps is not None:
            params["conv"] = {"taps": m.taps, "q": p + "q.conv", "k": p + "k.conv", "v": p + "v.conv"}
        if m.temp_every is not None:
            params["query_factor"] = (m.temp_coef, m.temp_every)
        return PartSpec("gqa_attention", params)
    if isinstance(m, LatentAttentionConfig):
        return PartSpec("latent_attention", {
            "hidden": config.width, "heads": m.heads, "dim": m.dim, "rot_dim": m.rot_dim, "vdim": m.vdim, "q_rank": None,
            "kv_rank": m.kv_rank, "scale": m.scale, "eps": config.eps, "window": m.window,
            "position": _rope("rope_half_split", m.rot_dims, m.rot_base, positions), "q": p + "q", "uk": p + "uk",
            "uv": p + "uv", "o": p + "o", "dkv": p + "dkv", "dkv_norm": p + "dkv.norm"})
    l, r = m.left, m.right
    x, y = p + "left.", p + "right."
    left = PartSpec("gqa_attention", {
        "hidden": config.width, "q_heads": l.heads, "kv_heads": l.kv_heads, "head_dim": l.dim, "value_dim": l.vdim,
        "qk_norm_eps": config.eps, "norm_span": "projection", "window": l.window, "scale": l.scale,
        "position": _rope("rope_adjacent", l.rot_dims, l.rot_base, positions), "float_output": True,
        "q": x + "q", "k": x + "k", "v": x + "v", "o": x + "o", "q_norm": x + "q.norm", "k_norm": x + "k.norm",
        "bias": {"q": x + "q.b", "k": x + "k.b", "v": x + "v.b"}})
    right = PartSpec("state_space", {
        "hidden": config.width, "heads": r.heads, "vdim": r.vdim, "state": r.state, "groups": r.groups,
        "norm_groups": r.norm_groups, "taps": r.taps, "eps": config.eps, "in": y + "in", "conv": y + "conv",
        "conv_bias": y + "conv.b", "dt_bias": y + "dt_bias", "A_log": y + "A_log", "D": y + "D", "norm": y + "norm",
        "o": y + "o"})
    return PartSpec("parallel", {"hidden": config.width, "eps": config.eps, "branches": {"left": left, "right": right},
                                 "weights": {"left": m.left_scale, "right": m.right_scale}})


def _feed_forward(config: NogidraConfig, i: int):
    f, p = config.layers[i].mlp, f"l{i}.mlp."
    if f is None:
        return None
    if isinstance(f, DenseConfig):
        return PartSpec("swiglu", {"hidden": config.width, "intermediate": f.ff, "gate": p + "gate", "up": p + "up",
                                   "down": p + "down", "float_output": True,
                                   "bias": {"gate": p + "gate.b", "up": p + "up.b", "down": p + "down.b"}})
    # softmax over all outputs, the best taken, their scores over the winners' sum: the softmax over the winners alone
    return PartSpec("routed_glu", {"hidden": config.width, "experts": f.experts, "identity": 0, "top": f.top,
                                   "group_count": 1, "group_keep": 1, "intermediate": f.expert_ff, "activation": "silu",
                                   "score": "softmax", "renormalize": True, "router": p + "router", "correction": None,
                                   "expert": p + "e{e}", "shared": None})


def nogidra_model_spec(config: NogidraConfig) -> ModelSpec:
    positions: dict = {}
    layers, unused = [], []
    for i in range(len(config.layers)):
        p = f"l{i}."
        params = {"norm1": _norm(config, p + "norm1"), "mixer": _mixer(config, i, positions)}
        feed_forward = _feed_forward(config, i)
        if feed_forward is not None:
            params.update(norm2=_norm(config, p + "norm2"), feed_forward=feed_forward)
        else:
            unused.append(p + "norm2")          # a file may hold the second norm of a layer that has no second sublayer
        layers.append(PartSpec("prenorm", params))
    return ModelSpec(hidden_size=config.width, vocab_size=config.vocab, max_positions=config.max_positions,
                     embedding="embed", layers=layers, schedule=default_schedule(len(layers)),
                     final_norm=_norm(config, "final.norm"), head="head", positions=positions,
                     logit_cap=config.logit_softcap, ignore_tensors=tuple(unused))


register_architecture(NogidraConfig.ARCHITECTURE, NogidraConfig.from_dict, nogidra_model_spec)
