"""Normalisation parts."""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from .. import ops
from ..weights.loader import TensorSpec, VECTOR
from .base import NORMS, Part, PartSpec


@NORMS.register("rmsnorm")
class RmsNorm(Part):
    """y = (x * gain) / sqrt(mean(x^2) + eps); the gain multiplies directly (not 1 + gain).

    Reference: crates/leone/src/cpu.rs:1642-1663.  Parameters: ``size``, ``eps``, ``weight`` (tensor name).
    Optional: ``weight_offset`` (a number): the stored weight lies around zero and the gain is offset + weight; the
    sum is made once, in float32, when the weights are bound, and the kernels see an ordinary gain.
    """

    graph_safe = True

    def __init__(self, spec: PartSpec, **_):
        self.size = int(spec["size"])
        self.eps = float(spec["eps"])
        self.weight_name = spec["weight"]
        self.weight_offset = float(spec["weight_offset"]) if spec.get("weight_offset") is not None else None
        self.gain: Optional[torch.Tensor] = None

    def tensor_specs(self) -> List[TensorSpec]:
        if self.weight_offset is not None:      # random weights of such a norm lie around zero, so that the gain lies around the offset
            return [TensorSpec(self.weight_name, (self.size,), VECTOR, init=("normal", 0.0, 0.02))]
        return [TensorSpec(self.weight_name, (self.size,), VECTOR)]

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.gain = tensors[self.weight_name].contiguous()
        if self.weight_offset is not None:
            self.gain = (self.gain.float() + self.weight_offset).contiguous()

    def add_norm(self, x: torch.Tensor, delta: Optional[torch.Tensor], out_dtype: torch.dtype,
                 rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        if isinstance(delta, ops.PreparedRows):
            delta = None                      # the product that made it has added into the stream already
        if isinstance(delta, ops.ScaledDelta):
            # a sublayer's result that enters the stream times a factor: sum and norm in one kernel
            return ops.residual_norm(x, delta.rows, delta.scale, self.gain, self.eps, out_dtype, rows)
        if isinstance(delta, ops.NormedDelta):
            behind = delta.norm
            if isinstance(behind, RmsNorm) and behind.gain.dtype == self.gain.dtype:
                # the norm behind the last sublayer, the residual sum and this norm in one kernel
                return ops.add_normed(x, delta.rows, behind.gain, behind.eps, then=(self.gain, self.eps, out_dtype), rows=rows)
            delta = delta.materialize()       # a delta that another kind of norm is still to be applied to
        return ops.add_rmsnorm(x, delta, self.gain, self.eps, out_dtype, rows)

    def apply(self, rows: torch.Tensor, out_dtype: torch.dtype = torch.float32) -> torch.Tensor:
        """The norm of float32 rows that are no stream (nothing is added, nothing written back)."""
        return ops.add_rmsnorm(rows, None, self.gain, self.eps, out_dtype)

    def add_behind(self, x: torch.Tensor, delta: Optional[torch.Tensor], out_dtype: Optional[torch.dtype]):
        """For a norm that stands behind its sublayer: x += norm(delta) in the float32 stream, and the new rows of
        the stream come back in ``out_dtype`` (what the next sublayer's products read; None: nothing comes back)."""
        return ops.add_normed(x, delta, self.gain, self.eps, out_dtype=out_dtype)

    def folded(self, out_dtype: torch.dtype):
        """(gain, eps, type) for a product that can leave this norm's operand behind when it adds into the
        stream (``ops.linear(..., next_norm=)``)."""
        return (self.gain, self.eps, out_dtype)

    def lazy(self, x: torch.Tensor, delta: Optional[torch.Tensor], out_dtype: torch.dtype,
             rows: Optional[torch.Tensor] = None):
        """The same, but if there is nothing to add the norm is only described (``ops.NormedRows``), so
        that the product that consumes it can carry it out itself."""
        if isinstance(delta, ops.PreparedRows):
            if rows is None and delta.gain is self.gain and delta.eps == self.eps and delta.dtype == out_dtype:
                return delta
            delta = None                      # made for another norm: the stream itself is up to date
        if delta is not None:
            return self.add_norm(x, delta, out_dtype, rows)
        return ops.NormedRows(x, self.gain, self.eps, out_dtype, rows)


@NORMS.register("layernorm")
class LayerNorm(Part):
    folds_conv = True      # add_norm(..., conv=) takes the residual-form convolution of single rows into its kernel

    """y = (x - mean) / sqrt(var + eps) * weight + bias, var the mean squared deviation; mean and variance in float.

    Parameters: ``size``, ``eps``, ``weight``, ``bias`` (tensor names).  ``add_norm`` also takes a delta that
    is still to go through another layer norm (``ops.NormedDelta``: the norm behind a sublayer) and does that
    norm, the residual sum and its own in one kernel.
    """

    graph_safe = True

    def __init__(self, spec: PartSpec, **_):
        self.size = int(spec["size"])
        self.eps = float(spec["eps"])
        self.weight_name, self.bias_name = spec["weight"], spec["bias"]
        self.gain: Optional[torch.Tensor] = None
        self.bias: Optional[torch.Tensor] = None

    def tensor_specs(self) -> List[TensorSpec]:
        return [TensorSpec(self.weight_name, (self.size,), VECTOR), TensorSpec(self.bias_name, (self.size,), VECTOR)]

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.gain = tensors[self.weight_name].contiguous()
        self.bias = tensors[self.bias_name].contiguous()
        if self.gain.dtype != self.bias.dtype:
            self.gain, self.bias = self.gain.float(), self.bias.float()

    def add_norm(self, x: torch.Tensor, delta, out_dtype: torch.dtype, rows: Optional[torch.Tensor] = None,
                 conv: Optional[tuple] = None) -> torch.Tensor:
        """``conv`` = (weight, state, step, write_state): in a step of single rows the input convolution of the
        sublayer that reads this norm is done in the same kernel (``ops.add_layernorm``)."""
        if isinstance(delta, ops.PreparedRows):
            delta = None
        delta_norm = None
        if isinstance(delta, ops.ScaledDelta):
            delta = delta.materialize()
        if isinstance(delta, ops.NormedDelta):
            behind = delta.norm
            if isinstance(behind, LayerNorm) and behind.gain.dtype == self.gain.dtype:
                delta, delta_norm = delta.rows, (behind.gain, behind.bias, behind.eps)
            else:
                delta = delta.materialize()
        elif delta is not None and delta.dim() == 3:
            delta = delta.sum(dim=0)          # planes of a product cut along its inner dimension
        return ops.add_layernorm(x, delta, self.gain, self.bias, self.eps, out_dtype, rows, delta_norm, conv)

    def apply(self, rows: torch.Tensor, out_dtype: torch.dtype = torch.float32) -> torch.Tensor:
        """The norm of float32 rows that are no stream (nothing is added, nothing written back)."""
        return ops.add_layernorm(rows, None, self.gain, self.bias, self.eps, out_dtype)
