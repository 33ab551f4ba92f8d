"""Fosulix configuration: a list of layers, each with a latent-attention or a gated-memory mixer and a mixture of
experts (or no feed-forward), a stream that is re-mixed from all earlier layers' results after every layer.

config.json keys: ``architecture`` ("Fosulix"), ``vocab``, ``width``, ``norm.eps``, ``residual_mult`` (factor on what
every sublayer adds), ``embedding.scale``, ``canon.taps`` (taps of the input convolution ahead of every mixer), and
``layers``: a list of ``{"type", "mixer", "mlp"}``.  ``type`` names the mixer:

  ``latent_attention``  ``mixer`` = {heads, dim, rot_dim, vdim, q_rank, kv_rank, scale,
                                     rot: {dims, base, scaling: {factor, original, fast, slow}}, mask: {size}, kv_from}
                        ``rot.scaling`` may be absent (plain frequencies), ``mask`` may be absent (every earlier key is
                        seen), ``kv_from`` (absent or a layer's index): the layer has no down-projection for keys and
                        values and reads the latents that layer caches.
  ``hgrn2``             ``mixer`` = {heads, dim, vdim}

``mlp`` is null or {kind: "moe", expert: {ff, limit}, router: {experts, top, scale, groups: {count, keep}}}
(``groups`` may be absent: one group).  ``max_positions`` (optional) bounds the rotary tables and a request's length.
"""
from __future__ import annotations

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


@dataclass(frozen=True)
class RotationScaling:
    factor: float
    original: float
    fast: float
    slow: float


@dataclass(frozen=True)
class LatentAttentionConfig:
    heads: int
    dim: int                      # elements of a head's query and key that are not rotated
    rot_dim: int                  # elements that are; the key's are shared by the heads
    vdim: int
    q_rank: int
    kv_rank: int
    scale: float
    rot_dims: int                 # how many of the rot_dim elements turn (the design has them equal)
    rot_base: float
    rot_scaling: Optional[RotationScaling]
    window: Optional[int]         # None: every earlier key is seen
    kv_from: Optional[int]        # the layer whose cached latents this one reads; None: its own


@dataclass(frozen=True)
class GatedMemoryConfig:
    heads: int
    dim: int
    vdim: int


@dataclass(frozen=True)
class MixtureConfig:
    experts: int
    top: int
    group_count: int
    group_keep: int
    scale: float                  # multiplies the chosen experts' scores
    expert_ff: int
    limit: float                  # bound on an expert's gate and up values


@dataclass(frozen=True)
class LayerConfig:
    kind: str                     # "latent_attention" or "hgrn2"
    mixer: Union[LatentAttentionConfig, GatedMemoryConfig]
    mlp: Optional[MixtureConfig]


def _latent(raw: Mapping[str, Any], where: str, index: int) -> LatentAttentionConfig:
    m = _sub(raw, "mixer", where)
    w = where + "mixer."
    try:
        heads, dim, rot_dim, vdim = (m.positive_int(k) for k in ("heads", "dim", "rot_dim", "vdim"))
        q_rank, kv_rank = m.positive_int("q_rank"), m.positive_int("kv_rank")
        scale = m.positive_float("scale")
        rot = _sub(m.raw, "rot", w)
        try:
            rot_dims, rot_base = rot.positive_int("dims"), rot.positive_float("base")
            scaling = None
            s = _sub(rot.raw, "scaling", w + "rot.", optional=True)
            if s is not None:
                try:
                    scaling = RotationScaling(s.positive_float("factor"), s.positive_float("original"),
                                              s.positive_float("fast"), s.positive_float("slow"))
                except ConfigError as error:
                    raise _relabel(error, w + "rot.scaling.") from None
        except ConfigError as error:
            raise _relabel(error, w + "rot.") from None
        if rot_dims % 2 or rot_dims > rot_dim:
            raise ConfigError(w + "rot.dims", f"must be even and at most rot_dim {rot_dim}, found {rot_dims}")
        if rot_base <= 1.0:
            raise ConfigError(w + "rot.base", f"must be above 1, found {rot_base}")
        window = None
        mask = _sub(m.raw, "mask", w, optional=True)
        if mask is not None:
            try:
                window = mask.positive_int("size")
            except ConfigError as error:
                raise _relabel(error, w + "mask.") from None
    except ConfigError as error:
        raise _relabel(error, w) from None
    kv_from = m.optional("kv_from")
    if kv_from is not None and (isinstance(kv_from, bool) or not isinstance(kv_from, int) or not 0 <= kv_from < index):
        raise ConfigError(w + "kv_from", f"layer {index} can only read the latents of an earlier layer, found {kv_from!r}")
    return LatentAttentionConfig(heads, dim, rot_dim, vdim, q_rank, kv_rank, scale, rot_dims, rot_base, scaling, window, kv_from)


def _gated_memory(raw: Mapping[str, Any], where: str) -> GatedMemoryConfig:
    m = _sub(raw, "mixer", where)
    try:
        return GatedMemoryConfig(m.positive_int("heads"), m.positive_int("dim"), m.positive_int("vdim"))
    except ConfigError as error:
        raise _relabel(error, where + "mixer.") from None


def _mlp(raw: Mapping[str, Any], where: str) -> Optional[MixtureConfig]:
    if raw.get("mlp") is None:
        return None
    f = _sub(raw, "mlp", where)
    w = where + "mlp."
    kind = f.optional("kind")
    if kind != "moe":
        raise ConfigError(w + "kind", f"expected \"moe\", found {kind!r}")
    try:
        expert, router = _sub(f.raw, "expert", w), _sub(f.raw, "router", w)
        try:
            ff, limit = expert.positive_int("ff"), expert.positive_float("limit")
        except ConfigError as error:
            raise _relabel(error, w + "expert.") from None
        try:
            experts, top, scale = router.positive_int("experts"), router.positive_int("top"), router.positive_float("scale")
            groups = _sub(router.raw, "groups", w + "router.", optional=True)
            try:
                count, keep = (groups.positive_int("count"), groups.positive_int("keep")) if groups is not None else (1, 1)
            except ConfigError as error:
                raise _relabel(error, w + "router.groups.") from None
        except ConfigError as error:
            raise _relabel(error, w + "router.") from None
    except ConfigError as error:
        raise _relabel(error, w) from None
    if top > experts:
        raise ConfigError(w + "router.top", f"{top} of {experts} experts cannot be chosen")
    if experts % count or keep > count:
        raise ConfigError(w + "router.groups", f"{experts} experts in {count} equal groups of which {keep} stay open")
    if top > keep * (experts // count):
        raise ConfigError(w + "router.groups", f"{keep} groups of {experts // count} cannot give {top} choices")
    return MixtureConfig(experts, top, count, keep, scale, ff, limit)


@dataclass(frozen=True)
class FosulixConfig:
    vocab: int
    width: int
    eps: float
    residual_mult: float
    embedding_scale: float
    taps: int
    layers: Tuple[LayerConfig, ...]
    max_positions: int = DEFAULT_MAX_POSITIONS
    architecture: str = "Fosulix"

    ARCHITECTURE = "Fosulix"

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any]) -> "FosulixConfig":
        top = FieldReader(raw)
        vocab, width = top.positive_int("vocab"), top.positive_int("width")
        eps = _sub(raw, "norm", "").positive_float("eps")
        mult = top.positive_float("residual_mult")
        try:
            embedding_scale = _sub(raw, "embedding", "").positive_float("scale")
        except ConfigError as error:
            raise _relabel(error, "embedding.") from None
        try:
            taps = _sub(raw, "canon", "").positive_int("taps")
        except ConfigError as error:
            raise _relabel(error, "canon.") from None
        if taps < 2:
            raise ConfigError("canon.taps", f"an input convolution has at least 2 taps, found {taps}")
        listed = raw.get("layers")
        if not isinstance(listed, list) or not listed:
            raise ConfigError("layers", f"expected a list of layers, found {listed!r}")
        layers = []
        for i, entry in enumerate(listed):
            where = f"layers[{i}]."
            if not isinstance(entry, dict):
                raise ConfigError(f"layers[{i}]", f"expected an object, found {entry!r}")
            kind = entry.get("type")
            if kind == "latent_attention":
                mixer = _latent(entry, where, i)
            elif kind == "hgrn2":
                mixer = _gated_memory(entry, where)
            else:
                raise ConfigError(where + "type", f"expected \"latent_attention\" or \"hgrn2\", found {kind!r}")
            layers.append(LayerConfig(kind, mixer, _mlp(entry, where)))
        for i, layer in enumerate(layers):
            source = getattr(layer.mixer, "kv_from", None)
            if source is None:
                continue
            other, mine = layers[source].mixer, layer.mixer
            if not isinstance(other, LatentAttentionConfig) or other.kv_from is not None:
                raise ConfigError(f"layers[{i}].mixer.kv_from", f"layer {source} caches no latents of its own")
            if (other.kv_rank, other.rot_dim, other.rot_dims, other.rot_base, other.rot_scaling) != \
                    (mine.kv_rank, mine.rot_dim, mine.rot_dims, mine.rot_base, mine.rot_scaling):
                raise ConfigError(f"layers[{i}].mixer.kv_from", f"layer {source}'s latent or rotation differ from this layer's")
        return cls(vocab, width, eps, mult, embedding_scale, taps, tuple(layers),
                   max_positions=top.positive_int("max_positions", DEFAULT_MAX_POSITIONS))

    def to_dict(self) -> Dict[str, Any]:
        layers = []
        for layer in self.layers:
            m = layer.mixer
            if isinstance(m, LatentAttentionConfig):
                rot: Dict[str, Any] = {"dims": m.rot_dims, "base": m.rot_base}
                if m.rot_scaling is not None:
                    s = m.rot_scaling
                    rot["scaling"] = {"factor": s.factor, "original": s.original, "fast": s.fast, "slow": s.slow}
                mixer: Dict[str, Any] = {"heads": m.heads, "dim": m.dim, "rot_dim": m.rot_dim, "vdim": m.vdim,
                                         "q_rank": m.q_rank, "kv_rank": m.kv_rank, "scale": m.scale, "rot": rot}
                if m.window is not None:
                    mixer["mask"] = {"size": m.window}
                if m.kv_from is not None:
                    mixer["kv_from"] = m.kv_from
            else:
                mixer = {"heads": m.heads, "dim": m.dim, "vdim": m.vdim}
            f = layer.mlp
            mlp = None if f is None else {
                "kind": "moe", "expert": {"ff": f.expert_ff, "limit": f.limit},
                "router": {"experts": f.experts, "top": f.top, "scale": f.scale,
                           "groups": {"count": f.group_count, "keep": f.group_keep}}}
            layers.append({"type": layer.kind, "mixer": mixer, "mlp": mlp})
        out = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.eps},
               "residual_mult": self.residual_mult, "embedding": {"scale": self.embedding_scale},
               "canon": {"taps": self.taps}, "layers": layers}
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

    def latent_retention(self, layer: int) -> Optional[int]:
        """The window that the cache of ``layer`` must keep: the widest of its own mask and of the masks of the
        layers that read its latents (None: everything)."""
        masks = [self.layers[layer].mixer] + [l.mixer for l in self.layers if getattr(l.mixer, "kv_from", None) == layer]
        if any(m.window is None for m in masks):
            return None
        return max(m.window for m in masks)
