"""Fosulix: how its configuration becomes parts.

A small decoder-only design whose config.json lists its layers one by one.  The stream starts as the token's vector
times a factor.  A layer is pre-norm with a factor m on what each sublayer adds (``scaled_prenorm`` block):
x <- x + m mixer(conv(norm1(x))), x <- x + m ff(norm2(x)), where conv is a short causal convolution over time in residual
form on what the mixer reads.  Two mixers: attention through latents (queries through a normed latent; keys and values
from one normed latent and one rotated key part that all heads share, which is all the cache holds; rotation of
neighbouring pairs with frequencies stretched for longer sequences; a sliding window; a layer may read the latents an
earlier layer cached), and a matrix memory whose forget gate per key channel also says what is written (``hgrn2``).  The
feed-forward is a mixture of experts with sigmoid scores, groups scored by their two best, weights that are the scores
times a factor, and experts whose gate and up values are held to a limit.  Behind every layer the stream is re-mixed
from the embedding's output and all layers' own results with the layer's weights (``ModelSpec.depth_weights``).  A final
RMS norm; the head is the token table.  Tensor names: ``embed``, ``final.norm`` and per layer ``l<i>.norm1``,
``l<i>.norm2``, ``l<i>.canon1``, ``l<i>.dwa``, ``l<i>.mix.{dq,dq.norm,uq,dkv,dkv.norm,uk,uv,o}`` or
``l<i>.mix.{q,f,f.b,lower,v,norm,o}``, ``l<i>.mlp.{router,e<j>.{gate,up,down}}``.
"""
from __future__ import annotations

from ..config.fosulix import FosulixConfig, LatentAttentionConfig
from ..parts.base import PartSpec
from ..parts.model import LayerRun, ModelSpec
from .registry import register_architecture


def _norm(config: FosulixConfig, name: str) -> PartSpec:
    return PartSpec("rmsnorm", {"size": config.width, "eps": config.eps, "weight": name})


def _position(m: LatentAttentionConfig, positions: dict) -> str:
    s = m.rot_scaling
    if s is None:
        name = f"rope_{m.rot_dims}_{m.rot_base!r}"
        positions.setdefault(name, PartSpec("rope_adjacent", {"rotary_dim": m.rot_dims, "theta": m.rot_base}))
        return name
    name = f"rope_{m.rot_dims}_{m.rot_base!r}_x{s.factor!r}_{s.original!r}_{s.fast!r}_{s.slow!r}"
    positions.setdefault(name, PartSpec("rope_scaled_adjacent", {"rotary_dim": m.rot_dims, "theta": m.rot_base,
                                                                "factor": s.factor, "original": s.original,
                                                                "fast": s.fast, "slow": s.slow}))
    return name


def _mixer(config: FosulixConfig, i: int, positions: dict) -> PartSpec:
    m, p = config.layers[i].mixer, f"l{i}.mix."
    if not isinstance(m, LatentAttentionConfig):
        return PartSpec("hgrn2", {"hidden": config.width, "heads": m.heads, "dim": m.dim, "vdim": m.vdim, "eps": config.eps,
                                  "q": p + "q", "f": p + "f", "f_bias": p + "f.b", "lower": p + "lower", "v": p + "v",
                                  "norm": p + "norm", "o": p + "o"})
    params = {"hidden": config.width, "heads": m.heads, "dim": m.dim, "rot_dim": m.rot_dim, "vdim": m.vdim,
              "q_rank": m.q_rank, "kv_rank": m.kv_rank, "scale": m.scale, "eps": config.eps, "window": m.window,
              "position": _position(m, positions), "dq": p + "dq", "dq_norm": p + "dq.norm", "uq": p + "uq",
              "uk": p + "uk", "uv": p + "uv", "o": p + "o"}
    if m.kv_from is None:
        params.update(dkv=p + "dkv", dkv_norm=p + "dkv.norm", retain_window=config.latent_retention(i))
    else:
        params.update(shared_kv=True, retain_window=config.latent_retention(m.kv_from))
    return PartSpec("latent_attention", params)


def _feed_forward(config: FosulixConfig, i: int):
    f, p = config.layers[i].mlp, f"l{i}.mlp."
    if f is None:
        return None
    return PartSpec("routed_glu", {"hidden": config.width, "experts": f.experts, "identity": 0, "top": f.top,
                                   "group_count": f.group_count, "group_keep": f.group_keep, "intermediate": f.expert_ff,
                                   "activation": "clamped_swish", "limit": f.limit, "score": "sigmoid", "group_best": 2,
                                   "renormalize": False, "weight_scale": f.scale, "router": p + "router",
                                   "correction": None, "expert": p + "e{e}", "shared": None})


def fosulix_model_spec(config: FosulixConfig) -> ModelSpec:
    positions: dict = {}
    layers, schedule, depth = [], [], []
    for i, layer in enumerate(config.layers):
        p = f"l{i}."
        params = {"norm1": _norm(config, p + "norm1"), "mixer": _mixer(config, i, positions), "scale": config.residual_mult,
                  "conv1": PartSpec("causal_conv", {"channels": config.width, "taps": config.taps, "weights": [p + "canon1"],
                                                    "add_input": True})}
        feed_forward = _feed_forward(config, i)
        if feed_forward is not None:
            params.update(feed_forward=feed_forward, norm2=_norm(config, p + "norm2"))
        layers.append(PartSpec("scaled_prenorm", params))
        # a layer without latents of its own reads the mixer cache of the layer that makes them; its convolution's
        # inputs are its own
        source = getattr(layer.mixer, "kv_from", None)
        schedule.append(LayerRun(i, i, True, borrow=None if source is None else {"mixer": source}))
        depth.append(p + "dwa")
    return ModelSpec(hidden_size=config.width, vocab_size=config.vocab, max_positions=config.max_positions,
                     embedding="embed", layers=layers, schedule=schedule, final_norm=_norm(config, "final.norm"),
                     head=None, positions=positions, embedding_scale=config.embedding_scale, depth_weights=depth)


register_architecture(FosulixConfig.ARCHITECTURE, FosulixConfig.from_dict, fosulix_model_spec)
