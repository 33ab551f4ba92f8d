"""How norm, mixer and feed-forward are arranged in one layer."""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..weights.loader import TensorSpec
from .. import ops
from .base import BLOCKS, CONVS, FEED_FORWARDS, MIXERS, NORMS, Part, PartSpec
from .context import CacheView, StepContext


@BLOCKS.register("prenorm")
class PreNormBlock(Part):
    """x1 = x + mixer(norm1(x)); x2 = x1 + feed_forward(norm2(x1)).

    Reference layer order: crates/leone/src/runtime.rs:9019-9050.
    Parameters: ``norm1``, ``mixer``, ``norm2``, ``feed_forward`` (part specs); the second sublayer is there
    only if ``feed_forward`` is given.
    The residual stream is float32; each delta is added by the following norm's
    kernel, so the block returns its last delta instead of adding it.
    """

    def __init__(self, spec: PartSpec, **context):
        self.norm1 = NORMS.build(spec["norm1"], **context)
        self.mixer = MIXERS.build(spec["mixer"], **context)
        self.feed_forward = FEED_FORWARDS.build(spec["feed_forward"], **context) if spec.get("feed_forward") is not None else None
        self.norm2 = NORMS.build(spec["norm2"], **context) if spec.get("norm2") is not None else None
        if self.feed_forward is not None and self.norm2 is None:
            raise ValueError("a prenorm block with a feed-forward needs norm2")

    def parts(self):
        return tuple(part for part in (self.norm1, self.mixer, self.norm2, self.feed_forward) if part is not None)

    @property
    def graph_safe(self) -> bool:
        return all(getattr(part, "graph_safe", False) for part in self.parts())

    def tensor_specs(self) -> List[TensorSpec]:
        return [s for part in self.parts() for s in part.tensor_specs()]

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        for part in self.parts():
            part.bind(tensors)

    def streamed_weights(self) -> List[torch.Tensor]:
        return [w for part in self.parts() if hasattr(part, "streamed_weights") for w in part.streamed_weights()]

    def cache_need(self):
        return self.mixer.cache_need()

    def row_tilings(self):
        """The tilings its parts declare (``RowTiling``), also those of mixers inside a mixer."""
        found = []
        for part in self.parts():
            if hasattr(part, "row_tiling"):
                found.append(part.row_tiling())
            if hasattr(part, "row_tilings"):
                found += part.row_tilings()
        return found

    prepares_next = True

    def entry_norm(self, out_dtype):
        """What the block before may prepare for this block's first norm (``RmsNorm.folded``), or None."""
        if getattr(self.mixer, "fused_io", False) and hasattr(self.norm1, "folded"):
            return self.norm1.folded(out_dtype)
        return None

    def forward(self, x: torch.Tensor, pending, step: StepContext, cache: Optional[CacheView], next_norm=None):
        """Returns the delta that is still to be added to ``x``, None if everything has been added, or, if
        ``next_norm`` (the next block's ``entry_norm``) was given and the last product could do it, that
        norm's operand (``ops.PreparedRows``; everything has been added then)."""
        y = self._normed(self.norm1, x, pending, step, self.mixer)
        if getattr(self.mixer, "fused_io", False):
            inner = None
            if getattr(self.mixer, "prepares_next", False) and getattr(self.feed_forward, "fused_io", False) \
                    and hasattr(self.norm2, "folded"):
                inner = self.norm2.folded(step.dtype)
            delta = (self.mixer.forward(y, step, cache, residual=x, next_norm=inner) if inner is not None
                     else self.mixer.forward(y, step, cache, residual=x))
        else:
            delta = self.mixer.forward(y, step, cache)
        if self.feed_forward is None:
            return delta
        y = self._normed(self.norm2, x, delta, step, self.feed_forward)
        if getattr(self.feed_forward, "fused_io", False):
            if next_norm is not None and getattr(self.feed_forward, "prepares_next", False):
                return self.feed_forward.forward(y, step, residual=x, next_norm=next_norm)
            return self.feed_forward.forward(y, step, residual=x)
        return self.feed_forward.forward(y, step)

    @staticmethod
    def _normed(norm, x, delta, step, consumer):
        # A consumer with fused_io takes a norm that is only described and may fold it into its first
        # product; any other gets the normalised rows.
        if getattr(consumer, "fused_io", False) and hasattr(norm, "lazy"):
            return norm.lazy(x, delta, step.dtype)
        return norm.add_norm(x, delta, step.dtype)


@BLOCKS.register("sandwich")
class SandwichBlock(Part):
    """A norm before and one behind each sublayer, and a short causal convolution on what a sublayer reads:

        x <- x + norm1b(mixer(conv1(norm1(x))));   x <- x + norm2b(feed_forward(conv2(norm2(x))))

    The second sublayer is there only if ``feed_forward`` is given; a ``conv`` may be None (the sublayer reads
    the norm's result as it is).  The convolutions keep their last inputs per request, so the block's cache need
    is a dict: ``mixer`` (the mixer's own), ``conv1``, ``conv2``.

    Parameters: ``norm1``, ``conv1``, ``mixer``, ``norm1b`` and optionally ``norm2``, ``conv2``,
    ``feed_forward``, ``norm2b`` (part specs).  The norm behind a sublayer is not carried out here: the block
    hands on ``ops.NormedDelta`` and the norm that runs next does it together with the residual sum and its own.
    """

    def __init__(self, spec: PartSpec, **context):
        def optional(registry, key):
            return registry.build(spec[key], **context) if spec.get(key) is not None else None
        self.norm1 = NORMS.build(spec["norm1"], **context)
        self.conv1 = optional(CONVS, "conv1")
        self.mixer = MIXERS.build(spec["mixer"], **context)
        self.norm1b = NORMS.build(spec["norm1b"], **context)
        self.feed_forward = optional(FEED_FORWARDS, "feed_forward")
        self.norm2 = optional(NORMS, "norm2")
        self.conv2 = optional(CONVS, "conv2")
        self.norm2b = optional(NORMS, "norm2b")
        if self.feed_forward is not None and (self.norm2 is None or self.norm2b is None):
            raise ValueError("a sandwich block with a feed-forward needs norm2 and norm2b")

    def parts(self):
        return tuple(part for part in (self.norm1, self.conv1, self.mixer, self.norm1b, self.norm2, self.conv2,
                                       self.feed_forward, self.norm2b) if part is not None)

    @property
    def graph_safe(self) -> bool:
        return all(getattr(part, "graph_safe", False) for part in self.parts())

    def tensor_specs(self) -> List[TensorSpec]:
        return [s for part in self.parts() for s in part.tensor_specs()]

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        for part in self.parts():
            part.bind(tensors)

    def streamed_weights(self) -> List[torch.Tensor]:
        return [w for part in self.parts() if hasattr(part, "streamed_weights") for w in part.streamed_weights()]

    def cache_need(self):
        need = {"mixer": self.mixer.cache_need()}
        if self.conv1 is not None:
            need["conv1"] = self.conv1.cache_need()
        if self.conv2 is not None and self.feed_forward is not None:
            need["conv2"] = self.conv2.cache_need()
        return need

    def row_tilings(self):
        found = []
        for part in self.parts():
            if hasattr(part, "row_tiling"):
                found.append(part.row_tiling())
            if hasattr(part, "row_tilings"):
                found += part.row_tilings()
        return found

    @staticmethod
    def _read(norm, conv, x, pending, step, cache):
        """What a sublayer reads: the norm of the stream (which first takes in what is pending), through the
        convolution if there is one."""
        if conv is None:
            return norm.add_norm(x, pending, step.dtype)
        if step.decode_only and getattr(norm, "folds_conv", False) and conv.add_input and conv.activation is None:
            # single decoded tokens: norm, convolution and the move of its state in one launch
            return norm.add_norm(x, pending, step.dtype, conv=(conv.weight, cache.state, step, cache.writes))
        return conv.forward(norm.add_norm(x, pending, torch.float32), step, cache, step.dtype)

    def forward(self, x: torch.Tensor, pending, step: StepContext, cache):
        cache = cache or {}
        h = self._read(self.norm1, self.conv1, x, pending, step, cache.get("conv1"))
        pending = ops.NormedDelta(self.mixer.forward(h, step, cache.get("mixer")), self.norm1b)
        if self.feed_forward is None:
            return pending
        h = self._read(self.norm2, self.conv2, x, pending, step, cache.get("conv2"))
        return ops.NormedDelta(self.feed_forward.forward(h, step), self.norm2b)


@BLOCKS.register("postnorm")
class PostNormBlock(Part):
    """The norms stand behind the sublayers, which read the stream itself:

        x <- x + norm1(mixer(x));   x <- x + norm2(feed_forward(x))

    The second sublayer is there only if ``feed_forward`` is given.  Parameters: ``mixer``, ``norm1`` and optionally
    ``feed_forward``, ``norm2`` (part specs); the norms are RMS norms.  The sublayers hand back float32.  A norm
    behind a sublayer, the residual sum and the rows of the stream in the type the next sublayer's products read
    are one kernel (``ops.add_normed``); the block's last norm is left to whoever runs next (``ops.NormedDelta``):
    the next block of this kind, or the model's final norm, which does both norms and the sum in one kernel.
    """

    def __init__(self, spec: PartSpec, **context):
        self.mixer = MIXERS.build(spec["mixer"], **context)
        self.norm1 = NORMS.build(spec["norm1"], **context)
        self.feed_forward = FEED_FORWARDS.build(spec["feed_forward"], **context) if spec.get("feed_forward") is not None else None
        self.norm2 = NORMS.build(spec["norm2"], **context) if spec.get("norm2") is not None else None
        if self.feed_forward is not None and self.norm2 is None:
            raise ValueError("a postnorm block with a feed-forward needs norm2")
        for norm in (self.norm1, self.norm2):
            if norm is not None and not hasattr(norm, "add_behind"):
                raise ValueError("the norms of a postnorm block must be able to stand behind a sublayer (add_behind)")

    def parts(self):
        return tuple(part for part in (self.mixer, self.norm1, self.feed_forward, self.norm2) if part is not None)

    @property
    def graph_safe(self) -> bool:
        return all(getattr(part, "graph_safe", False) for part in self.parts())

    def tensor_specs(self) -> List[TensorSpec]:
        return [s for part in self.parts() for s in part.tensor_specs()]

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        for part in self.parts():
            part.bind(tensors)

    def streamed_weights(self) -> List[torch.Tensor]:
        return [w for part in self.parts() if hasattr(part, "streamed_weights") for w in part.streamed_weights()]

    def cache_need(self):
        return self.mixer.cache_need()

    def row_tilings(self):
        return [part.row_tiling() for part in self.parts() if hasattr(part, "row_tiling")]

    @staticmethod
    def _take_in(x: torch.Tensor, pending, step: StepContext) -> torch.Tensor:
        """Adds what the block before left to be added and returns the stream's rows as the products read them."""
        if isinstance(pending, ops.PreparedRows):
            pending = None                        # its product has added into the stream already
        if isinstance(pending, ops.NormedDelta) and hasattr(pending.norm, "add_behind"):
            return pending.norm.add_behind(x, pending.rows, step.dtype)
        if pending is not None:
            delta = pending.materialize() if isinstance(pending, ops.NormedDelta) else pending
            x.add_(delta.sum(dim=0) if delta.dim() == 3 else delta)
        return ops.add_normed(x, None, None, 0.0, out_dtype=step.dtype)

    def forward(self, x: torch.Tensor, pending, step: StepContext, cache: Optional[CacheView]):
        h = self._take_in(x, pending, step)
        mixed = self.mixer.forward(h, step, cache)
        if self.feed_forward is None:
            return ops.NormedDelta(mixed, self.norm1)
        h = self.norm1.add_behind(x, mixed, step.dtype)
        return ops.NormedDelta(self.feed_forward.forward(h, step), self.norm2)


@BLOCKS.register("scaled_prenorm")
class ScaledPreNormBlock(Part):
    """Pre-norm sublayers whose results enter the stream times a factor, the mixer reading through a short convolution:

        x <- x + scale * mixer(conv1(norm1(x)));   x <- x + scale * feed_forward(norm2(x))

    The second sublayer is there only if ``feed_forward`` is given; ``conv1`` may be None (the mixer reads the norm's
    result as it is).  The convolution keeps its last inputs per request, so the block's cache need is a dict:
    ``mixer`` (the mixer's own) and ``conv1``.  Parameters: ``norm1``, ``conv1``, ``mixer``, ``scale`` and optionally
    ``norm2``, ``feed_forward`` (part specs).  The sublayers hand back float32.  The block's last sum is left to
    whoever runs next (``ops.ScaledDelta``): a norm adds it in its own kernel, and a model that re-mixes the stream
    over depth takes it into that kernel.
    """

    def __init__(self, spec: PartSpec, **context):
        self.norm1 = NORMS.build(spec["norm1"], **context)
        self.conv1 = CONVS.build(spec["conv1"], **context) if spec.get("conv1") is not None else None
        self.mixer = MIXERS.build(spec["mixer"], **context)
        self.feed_forward = FEED_FORWARDS.build(spec["feed_forward"], **context) if spec.get("feed_forward") is not None else None
        self.norm2 = NORMS.build(spec["norm2"], **context) if spec.get("norm2") is not None else None
        self.scale = float(spec.get("scale", 1.0))
        if self.feed_forward is not None and self.norm2 is None:
            raise ValueError("a scaled_prenorm block with a feed-forward needs norm2")

    def parts(self):
        return tuple(part for part in (self.norm1, self.conv1, self.mixer, self.norm2, self.feed_forward) if part is not None)

    @property
    def graph_safe(self) -> bool:
        return all(getattr(part, "graph_safe", False) for part in self.parts())

    def tensor_specs(self) -> List[TensorSpec]:
        return [s for part in self.parts() for s in part.tensor_specs()]

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        for part in self.parts():
            part.bind(tensors)

    def streamed_weights(self) -> List[torch.Tensor]:
        return [w for part in self.parts() if hasattr(part, "streamed_weights") for w in part.streamed_weights()]

    def cache_need(self):
        need = {"mixer": self.mixer.cache_need()}
        if self.conv1 is not None:
            need["conv1"] = self.conv1.cache_need()
        return need

    def row_tilings(self):
        return [part.row_tiling() for part in self.parts() if hasattr(part, "row_tiling")]

    def forward(self, x: torch.Tensor, pending, step: StepContext, cache):
        cache = cache or {}
        if self.conv1 is None:
            h = self.norm1.add_norm(x, pending, step.dtype)
        else:
            h = self.conv1.forward(self.norm1.add_norm(x, pending, torch.float32), step, cache.get("conv1"), step.dtype)
        delta = ops.ScaledDelta(self.mixer.forward(h, step, cache.get("mixer")), self.scale)
        if self.feed_forward is None:
            return delta
        h = self.norm2.add_norm(x, delta, step.dtype)
        return ops.ScaledDelta(self.feed_forward.forward(h, step), self.scale)
