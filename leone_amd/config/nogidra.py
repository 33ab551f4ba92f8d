"""Nogidra configuration: a list of pre-norm layers, each with one of three mixers (softmax attention whose scores fall
with the distance, attention through a latent, softmax attention and a state-space layer side by side) and a dense or
routed feed-forward (or none), a capped output.

config.json keys: ``architecture`` ("Nogidra"), ``vocab``, ``width``, ``norm.eps``, ``logit_softcap`` (optional) and
``layers``: a list of ``{"type", "mixer", "mlp"}``.  ``type`` names the mixer:

  ``attention``         ``mixer`` = {heads, kv_heads, dim, vdim, scale, conv, mask: {size}, q_temp: {coef, every}}
                        ``conv``: taps of the convolutions behind the q, k and v projections.
  ``latent_attention``  ``mixer`` = {heads, dim, rot_dim, vdim, kv_rank, scale, rot: {dims, base}, mask: {size}}
  ``parallel``          ``mixer`` = {left: {heads, kv_heads, dim, vdim, scale, rot: {dims, base}, mask: {size}},
                                     right: {heads, vdim, state, groups, norm_groups, conv}, left_scale, right_scale}

``mask`` may be absent (every earlier key is seen), and so may ``conv`` and ``q_temp`` of an ``attention`` mixer,
``kv_heads`` (as many as ``heads``), ``vdim`` (``dim``) and ``scale`` (one over the root of a key's size).
``mlp`` is null, {kind: "dense", ff} or {kind: "moe", expert: {ff}, router: {experts, top}}.  ``max_positions``
(optional) bounds the rotary tables and a request's length.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Any, Dict, Mapping, Optional, Tuple, Union

from .base import ConfigError, FieldReader

DEFAULT_MAX_POSITIONS = 32768


def _sub(raw: Mapping[str, Any], key: str, where: str, optional: bool = False) -> Optional[FieldReader]:
    value = raw.get(key)
    if value is None and optional:
        return None
    if not isinstance(value, dict):
        raise ConfigError(f"{where}{key}", f"expected an object, found {value!r}")
    return FieldReader(value)


def _relabel(error: ConfigError, where: str) -> ConfigError:
    if error.field.startswith(where) or error.field.startswith("layers["):
        return error
    return ConfigError(where + error.field, str(error).split(": ", 2)[-1])


def _number(reader: FieldReader, key: str) -> float:
    """A finite number of either sign (a coefficient, a branch's weight)."""
    value = reader.optional(key)
    if isinstance(value, bool) or not isinstance(value, (int, float)) or not math.isfinite(float(value)):
        raise ConfigError(key, f"expected a finite number, found {value!r}")
    return float(value)


def _window(m: FieldReader, where: str) -> Optional[int]:
    mask = _sub(m.raw, "mask", where, optional=True)
    if mask is None:
        return None
    try:
        return mask.positive_int("size")
    except ConfigError as error:
        raise _relabel(error, where + "mask.") from None


def _rotation(m: FieldReader, where: str, most: int) -> Tuple[int, float]:
    rot = _sub(m.raw, "rot", where)
    try:
        dims, base = rot.positive_int("dims"), rot.positive_float("base")
    except ConfigError as error:
        raise _relabel(error, where + "rot.") from None
    if dims % 2 or dims > most:
        raise ConfigError(where + "rot.dims", f"must be even and at most {most}, found {dims}")
    if base <= 1.0:
        raise ConfigError(where + "rot.base", f"must be above 1, found {base}")
    return dims, base


@dataclass(frozen=True)
class BiasedAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    taps: Optional[int]           # taps of the convolutions behind q, k and v; None: none
    window: Optional[int]         # None: every earlier key is seen
    temp_coef: Optional[float]    # the queries at position p count times 1 + coef * ln(floor((p + 1) / every) + 1)
    temp_every: Optional[int]


@dataclass(frozen=True)
class LatentAttentionConfig:
    heads: int
    dim: int                      # elements of a head's query and key that are not rotated
    rot_dim: int                  # elements that are; the key's are shared by the heads
    vdim: int
    kv_rank: int
    scale: float
    rot_dims: int
    rot_base: float
    window: Optional[int]


@dataclass(frozen=True)
class NormedAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot_dims: int
    rot_base: float
    window: Optional[int]


@dataclass(frozen=True)
class StateSpaceConfig:
    heads: int
    vdim: int
    state: int
    groups: int
    norm_groups: int
    taps: int


@dataclass(frozen=True)
class ParallelConfig:
    left: NormedAttentionConfig
    right: StateSpaceConfig
    left_scale: float
    right_scale: float


@dataclass(frozen=True)
class DenseConfig:
    ff: int


@dataclass(frozen=True)
class MixtureConfig:
    experts: int
    top: int
    expert_ff: int


@dataclass(frozen=True)
class LayerConfig:
    kind: str                     # "attention", "latent_attention" or "parallel"
    mixer: Union[BiasedAttentionConfig, LatentAttentionConfig, ParallelConfig]
    mlp: Union[None, DenseConfig, MixtureConfig]


def _grouped(heads: int, kv_heads: int, where: str) -> None:
    if heads % kv_heads:
        raise ConfigError(where + "kv_heads", f"{heads} query heads cannot be grouped over {kv_heads} key/value heads")


def _biased_attention(raw: Mapping[str, Any], where: str) -> BiasedAttentionConfig:
    m = _sub(raw, "mixer", where)
    w = where + "mixer."
    try:
        heads, dim = m.positive_int("heads"), m.positive_int("dim")
        kv_heads, vdim = m.positive_int("kv_heads", heads), m.positive_int("vdim", dim)
        scale = m.positive_float("scale", dim ** -0.5)
        taps = m.positive_int("conv", None)
        coef = every = None
        temp = _sub(m.raw, "q_temp", w, optional=True)
        if temp is not None:
            try:
                coef, every = _number(temp, "coef"), temp.positive_int("every")
            except ConfigError as error:
                raise _relabel(error, w + "q_temp.") from None
        window = _window(m, w)
    except ConfigError as error:
        raise _relabel(error, w) from None
    _grouped(heads, kv_heads, w)
    if taps is not None and taps < 2:
        raise ConfigError(w + "conv", f"a convolution has at least 2 taps, found {taps}")
    return BiasedAttentionConfig(heads, kv_heads, dim, vdim, scale, taps, window, coef, every)


def _latent(raw: Mapping[str, Any], where: str) -> LatentAttentionConfig:
    m = _sub(raw, "mixer", where)
    w = where + "mixer."
    try:
        heads, dim, rot_dim, vdim, kv_rank = (m.positive_int(k) for k in ("heads", "dim", "rot_dim", "vdim", "kv_rank"))
        scale = m.positive_float("scale", (dim + rot_dim) ** -0.5)
        rot_dims, rot_base = _rotation(m, w, rot_dim)
        window = _window(m, w)
    except ConfigError as error:
        raise _relabel(error, w) from None
    return LatentAttentionConfig(heads, dim, rot_dim, vdim, kv_rank, scale, rot_dims, rot_base, window)


def _parallel(raw: Mapping[str, Any], where: str) -> ParallelConfig:
    m = _sub(raw, "mixer", where)
    w = where + "mixer."
    try:
        left, right = _sub(m.raw, "left", w), _sub(m.raw, "right", w)
        try:
            heads, dim = left.positive_int("heads"), left.positive_int("dim")
            kv_heads, vdim = left.positive_int("kv_heads", heads), left.positive_int("vdim", dim)
            scale = left.positive_float("scale", dim ** -0.5)
            rot_dims, rot_base = _rotation(left, w + "left.", dim)
            window = _window(left, w + "left.")
            _grouped(heads, kv_heads, w + "left.")
        except ConfigError as error:
            raise _relabel(error, w + "left.") from None
        try:
            s_heads, s_vdim, state, groups, norm_groups, taps = (
                right.positive_int(k) for k in ("heads", "vdim", "state", "groups", "norm_groups", "conv"))
        except ConfigError as error:
            raise _relabel(error, w + "right.") from None
        left_scale, right_scale = _number(m, "left_scale"), _number(m, "right_scale")
    except ConfigError as error:
        raise _relabel(error, w) from None
    if s_heads % groups:
        raise ConfigError(w + "right.groups", f"{s_heads} heads do not share {groups} groups evenly")
    if (s_heads * s_vdim) % norm_groups:
        raise ConfigError(w + "right.norm_groups", f"{s_heads * s_vdim} columns cannot be normed in {norm_groups} equal runs")
    if taps < 2:
        raise ConfigError(w + "right.conv", f"a convolution has at least 2 taps, found {taps}")
    return ParallelConfig(NormedAttentionConfig(heads, kv_heads, dim, vdim, scale, rot_dims, rot_base, window),
                          StateSpaceConfig(s_heads, s_vdim, state, groups, norm_groups, taps), left_scale, right_scale)


def _mlp(raw: Mapping[str, Any], where: str):
    if raw.get("mlp") is None:
        return None
    f = _sub(raw, "mlp", where)
    w = where + "mlp."
    kind = f.optional("kind")
    try:
        if kind == "dense":
            return DenseConfig(f.positive_int("ff"))
        if kind != "moe":
            raise ConfigError(w + "kind", f"expected \"dense\" or \"moe\", found {kind!r}")
        expert, router = _sub(f.raw, "expert", w), _sub(f.raw, "router", w)
        try:
            ff = expert.positive_int("ff")
        except ConfigError as error:
            raise _relabel(error, w + "expert.") from None
        try:
            experts, top = router.positive_int("experts"), router.positive_int("top")
        except ConfigError as error:
            raise _relabel(error, w + "router.") from None
    except ConfigError as error:
        raise _relabel(error, w) from None
    if top > experts:
        raise ConfigError(w + "router.top", f"{top} of {experts} experts cannot be chosen")
    return MixtureConfig(experts, top, ff)


_MIXERS = {"attention": _biased_attention, "latent_attention": _latent, "parallel": _parallel}


@dataclass(frozen=True)
class NogidraConfig:
    vocab: int
    width: int
    eps: float
    layers: Tuple[LayerConfig, ...]
    logit_softcap: Optional[float] = None
    max_positions: int = DEFAULT_MAX_POSITIONS
    architecture: str = "Nogidra"

    ARCHITECTURE = "Nogidra"

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any]) -> "NogidraConfig":
        top = FieldReader(raw)
        vocab, width = top.positive_int("vocab"), top.positive_int("width")
        eps = _sub(raw, "norm", "").positive_float("eps")
        cap = top.positive_float("logit_softcap", None) if top.has("logit_softcap") else None
        listed = raw.get("layers")
        if not isinstance(listed, list) or not listed:
            raise ConfigError("layers", f"expected a list of layers, found {listed!r}")
        layers = []
        for i, entry in enumerate(listed):
            where = f"layers[{i}]."
            if not isinstance(entry, dict):
                raise ConfigError(f"layers[{i}]", f"expected an object, found {entry!r}")
            kind = entry.get("type")
            if kind not in _MIXERS:
                raise ConfigError(where + "type", f"expected one of {', '.join(sorted(_MIXERS))}, found {kind!r}")
            layers.append(LayerConfig(kind, _MIXERS[kind](entry, where), _mlp(entry, where)))
        return cls(vocab, width, eps, tuple(layers), logit_softcap=cap,
                   max_positions=top.positive_int("max_positions", DEFAULT_MAX_POSITIONS))

    def to_dict(self) -> Dict[str, Any]:
        def masked(mixer: Dict[str, Any], window: Optional[int]) -> Dict[str, Any]:
            if window is not None:
                mixer["mask"] = {"size": window}
            return mixer

        layers = []
        for layer in self.layers:
            m = layer.mixer
            if isinstance(m, BiasedAttentionConfig):
                mixer: Dict[str, Any] = {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim, "scale": m.scale}
                if m.taps is not None:
                    mixer["conv"] = m.taps
                if m.temp_every is not None:
                    mixer["q_temp"] = {"coef": m.temp_coef, "every": m.temp_every}
                masked(mixer, m.window)
            elif isinstance(m, LatentAttentionConfig):
                mixer = masked({"heads": m.heads, "dim": m.dim, "rot_dim": m.rot_dim, "vdim": m.vdim, "kv_rank": m.kv_rank,
                                "scale": m.scale, "rot": {"dims": m.rot_dims, "base": m.rot_base}}, m.window)
            else:
                l, r = m.left, m.right
                mixer = {"left": masked({"heads": l.heads, "kv_heads": l.kv_heads, "dim": l.dim, "vdim": l.vdim, "scale": l.scale,
                                         "rot": {"dims": l.rot_dims, "base": l.rot_base}}, l.window),
                         "right": {"heads": r.heads, "vdim": r.vdim, "state": r.state, "groups": r.groups,
                                   "norm_groups": r.norm_groups, "conv": r.taps},
                         "left_scale": m.left_scale, "right_scale": m.right_scale}
            f = layer.mlp
            if f is None:
                mlp = None
            elif isinstance(f, DenseConfig):
                mlp = {"kind": "dense", "ff": f.ff}
            else:
                mlp = {"kind": "moe", "expert": {"ff": f.expert_ff}, "router": {"experts": f.experts, "top": f.top}}
            layers.append({"type": layer.kind, "mixer": mixer, "mlp": mlp})
        out: Dict[str, Any] = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
                               "norm": {"eps": self.eps}, "layers": layers}
        if self.logit_softcap is not None:
            out["logit_softcap"] = self.logit_softcap
        if self.max_positions != DEFAULT_MAX_POSITIONS:
            out["max_positions"] = self.max_positions
        return out

    # what the generic entry points ask a configuration for
    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def max_position_embeddings(self) -> int:
        return self.max_positions

    eos_token_id = None
