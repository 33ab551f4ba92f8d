"""Token mixers."""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

from .. import ops
from ..weights.loader import MATRIX, VECTOR, TensorSpec
from .base import CONVS, MIXERS, KvNeed, Part, PartSpec, RowTiling
from .context import KvCacheView, StepContext
from .position import rotation_of


@MIXERS.register("gqa_attention")
class GqaAttention(Part):
    """Grouped-query causal attention over a paged key/value cache.

    q = Wq y, k = Wk y, v = Wv y (no bias); optional per-head RMSNorm of q and
    k over head_dim, then the position encoding on q and k; k and v go into the
    cache; each row attends the keys of its own request up to its position
    (within ``window`` if set) with scale 1/sqrt(head_dim); out = Wo o.
    Reference: crates/leone/src/runtime.rs:9104-9157 (decode order),
    crates/leone/src/backend.rs:2182-2208 (per-head norm),
    crates/leone/src/cpu.rs:2299-2357 (attention).

    Parameters: ``hidden``, ``q_heads``, ``kv_heads``, ``head_dim``, ``qk_norm_eps``
    (None: no q/k norm), ``window`` (None: all keys), ``position`` (name of a
    position part) and tensor names ``q``, ``k``, ``v``, ``o``, ``q_norm``, ``k_norm``.
    Optional: ``scale`` (the scores' factor, 1/sqrt(head_dim) if absent), ``value_dim`` (values and the output
    of a head have this size instead of ``head_dim``), ``gate`` (tensor name ``[q_heads, hidden]``: head h's
    result is multiplied by sigmoid(gate y)_h before the output projection), ``float_output`` (the output
    projection's result comes in float32 whatever the engine's type).
    ``gate_each`` (with ``gate``): the gate is ``[q_heads * value_dim, hidden]``, one value for every element of
    the heads' results.  ``keep_first`` (with ``window``): keys at positions below it stay in sight whatever the
    window, at their own positions.  ``shared_kv``: the layer has no key and value projections (and no key norm)
    and reads the cache another layer writes (its run names that layer's cache slot and does not write).
    ``retain_window`` / ``retain_first``: what the cache must keep if other layers with wider masks read it too
    (by default this layer's own ``window`` and ``keep_first``; ``retain_window`` 0: everything).
    ``bias``: a dict with tensor names ``q``, ``k``, ``v`` of biases that the projections add.  ``norm_span``
    "projection" (with ``qk_norm_eps``): q and k are each divided by their root mean square over the whole projection,
    all heads at once, and ``q_norm`` / ``k_norm`` have the projections' sizes (default "head": every head by itself,
    one gain for all heads).  ``conv``: a dict ``taps``, ``q``, ``k``, ``v`` (tensor names ``[channels, taps]``): q, k
    and v each pass a short causal convolution over time directly behind the projection; the layer then also keeps a
    request's last ``taps - 1`` projected rows.  ``distance_slopes`` (one number a query head): head h's score for a
    key at distance d is lowered by slopes[h] * d.  ``query_factor`` = (coef, every): the queries at position p count
    times 1 + coef * ln(floor((p + 1) / every) + 1).
    """

    graph_safe = True

    def __init__(self, spec: PartSpec, positions: Optional[dict] = None, **_):
        p = spec.params
        self.hidden = int(p["hidden"])
        self.q_heads = int(p["q_heads"])
        self.kv_heads = int(p["kv_heads"])
        self.head_dim = int(p["head_dim"])
        if self.q_heads % self.kv_heads:
            raise ValueError(f"{self.q_heads} query heads cannot be grouped over {self.kv_heads} kv heads")
        self.qk_norm_eps = p.get("qk_norm_eps")
        self.window = p.get("window")
        self.scale = float(p.get("scale", 1.0 / math.sqrt(self.head_dim)))
        self.shared_kv = bool(p.get("shared_kv", False))
        self.names = {k: p[k] for k in (("q", "o") if self.shared_kv else ("q", "k", "v", "o"))}
        self.keep_first = int(p.get("keep_first") or 0) if self.window else 0
        self.gate_each = bool(p.get("gate_each", False))
        self.retain_window = self.window if "retain_window" not in p else (p["retain_window"] or None)
        self.retain_first = int(p.get("retain_first", self.keep_first) or 0)
        self.value_dim = int(p.get("value_dim") or self.head_dim)
        self.float_output = bool(p.get("float_output", False))
        # The cache packs keys in runs of 8 elements and the kernels take values in pairs: heads of other sizes are
        # filled up with zero rows of the projections (and zero columns of the output projection) when the weights are
        # bound, which changes no score and no result.  ``file_*`` are the sizes the tensors have.
        self.file_head_dim, self.file_value_dim = self.head_dim, self.value_dim
        self.head_dim, self.value_dim = -(-self.head_dim // 8) * 8, -(-self.value_dim // 2) * 2
        self.padded = (self.head_dim, self.value_dim) != (self.file_head_dim, self.file_value_dim)
        if p.get("gate"):
            self.names["gate"] = p["gate"]
        self.bias_names = dict(p["bias"]) if p.get("bias") else None
        self.norm_span = str(p.get("norm_span") or "head")
        if self.norm_span not in ("head", "projection"):
            raise ValueError(f"attention: norm_span {self.norm_span!r} is neither 'head' nor 'projection'")
        self.wide_norm = self.qk_norm_eps is not None and self.norm_span == "projection"
        self.slope_values = [float(v) for v in p["distance_slopes"]] if p.get("distance_slopes") is not None else None
        if self.slope_values is not None and len(self.slope_values) != self.q_heads:
            raise ValueError(f"attention: {len(self.slope_values)} distance slopes for {self.q_heads} query heads")
        self.query_factor = (float(p["query_factor"][0]), int(p["query_factor"][1])) if p.get("query_factor") else None
        if self.query_factor is not None and self.query_factor[1] <= 0:
            raise ValueError(f"attention: the query factor's period must be positive, found {self.query_factor[1]}")
        self.conv = None
        if p.get("conv"):
            if self.shared_kv or self.bias_names:
                raise ValueError("attention: convolutions behind the projections go with keys of the layer's own and no biases")
            c = p["conv"]
            self.conv = CONVS.build(PartSpec("causal_conv", {
                "channels": [self.q_heads * self.head_dim, self.kv_heads * self.head_dim, self.kv_heads * self.value_dim],
                "taps": int(c["taps"]), "weights": [c["q"], c["k"], c["v"]]}))
        if (self.bias_names or self.wide_norm) and self.shared_kv:
            raise ValueError("attention: biases and norms over a whole projection go with keys of the layer's own")
        # a value size of its own, a gate, or anything between the projection and the heads: the projection carries
        # more than q, k and v of one size, or passes through kernels of its own
        self.general = (self.value_dim != self.head_dim or "gate" in self.names or self.shared_kv or bool(self.bias_names)
                        or self.wide_norm or self.conv is not None or self.slope_values is not None
                        or self.query_factor is not None or self.padded)
        if self.padded and (self.shared_kv or self.gate_each or (self.qk_norm_eps is not None and not self.wide_norm)):
            raise ValueError(f"attention: heads of {self.file_head_dim} and values of {self.file_value_dim} elements are filled up "
                             f"to multiples of 8 and 2, which a norm a head, a gate an element and a borrowed cache do not allow")
        if self.qk_norm_eps is not None:
            self.names.update(q_norm=p["q_norm"])
            if not self.shared_kv:
                self.names.update(k_norm=p["k_norm"])
        self.position = (positions or {}).get(p.get("position")) if p.get("position") else None
        if p.get("position") and self.position is None:
            raise ValueError(f"attention names position part {p.get('position')!r}, which the model does not define")
        self.w_qkv = self.w_o = self.q_gain = self.k_gain = self.bias = self.slopes = None

    def cache_need(self):
        keys = KvNeed(self.kv_heads, self.head_dim, self.retain_window,
                      value_dim=self.value_dim if self.value_dim != self.head_dim else None,
                      keep_first=self.retain_first if self.retain_window else 0)
        if self.conv is None:
            return keys
        return {"kv": keys, "conv": self.conv.cache_need()}

    def row_tiling(self) -> RowTiling:
        """The tiles of the prompt-attention kernel."""
        return RowTiling(ops.PREFILL_TILE_ROWS, ops.PREFILL_GROUP_TILES, ops.PREFILL_MIN_ROWS)

    def tensor_specs(self) -> List[TensorSpec]:
        qw, kvw, vw = self.q_heads * self.file_head_dim, self.kv_heads * self.file_head_dim, self.kv_heads * self.file_value_dim
        specs = [TensorSpec(self.names["q"], (qw, self.hidden), MATRIX)]
        if not self.shared_kv:
            specs += [TensorSpec(self.names["k"], (kvw, self.hidden), MATRIX),
                      TensorSpec(self.names["v"], (vw, self.hidden), MATRIX)]
        specs.append(TensorSpec(self.names["o"], (self.hidden, self.q_heads * self.file_value_dim), MATRIX))
        if "gate" in self.names:
            gates = self.q_heads * self.file_value_dim if self.gate_each else self.q_heads
            specs.append(TensorSpec(self.names["gate"], (gates, self.hidden), MATRIX))
        if self.qk_norm_eps is not None:
            q_size, k_size = ((qw, kvw) if self.wide_norm else (self.file_head_dim, self.file_head_dim))
            specs.append(TensorSpec(self.names["q_norm"], (q_size,), VECTOR))
            if not self.shared_kv:
                specs.append(TensorSpec(self.names["k_norm"], (k_size,), VECTOR))
        if self.bias_names:
            small = ("normal", 0.0, 0.02)
            specs += [TensorSpec(self.bias_names["q"], (qw,), VECTOR, init=small),
                      TensorSpec(self.bias_names["k"], (kvw,), VECTOR, init=small),
                      TensorSpec(self.bias_names["v"], (vw,), VECTOR, init=small)]
        if self.conv is not None:       # the filters as the file has them: one row a channel of the heads' own sizes
            specs += [TensorSpec(name, (width, self.conv.taps), VECTOR) for name, width in zip(self.conv.names, (qw, kvw, vw))]
        return specs

    def _filled(self, rows: torch.Tensor, heads: int, size: int, to: int) -> torch.Tensor:
        """``rows`` ``[heads * size, ...]`` with every head's rows filled up with zero rows to ``to``."""
        if size == to:
            return rows
        shaped = rows.reshape(heads, size, -1)
        shaped = torch.nn.functional.pad(shaped, (0, 0, 0, to - size))
        return shaped.reshape(heads * to, *rows.shape[1:])

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        # One product for q, k and v: a pure re-layout of the three matrices.
        d, e = self.file_head_dim, self.file_value_dim
        fused = [self._filled(tensors.pop(self.names["q"]), self.q_heads, d, self.head_dim)]
        if not self.shared_kv:
            fused += [self._filled(tensors.pop(self.names["k"]), self.kv_heads, d, self.head_dim),
                      self._filled(tensors.pop(self.names["v"]), self.kv_heads, e, self.value_dim)]
        if "gate" in self.names:
            fused.append(tensors.pop(self.names["gate"]))      # the heads' gates ride along as further columns
        self.w_qkv = torch.cat(fused, dim=0).contiguous()
        w_o = tensors.pop(self.names["o"])
        # zero columns of the output projection meet what the values' zero rows give
        self.w_o = self._filled(w_o.t(), self.q_heads, e, self.value_dim).t().contiguous()
        if self.qk_norm_eps is not None:
            self.q_gain = tensors.pop(self.names["q_norm"]).contiguous()
            # a layer without keys of its own never normalises one; the kernels want the two gains together
            self.k_gain = self.q_gain if self.shared_kv else tensors.pop(self.names["k_norm"]).contiguous()
            if self.q_gain.dtype != self.k_gain.dtype:
                self.q_gain, self.k_gain = self.q_gain.float(), self.k_gain.float()
            if self.wide_norm:
                self.q_gain = self._filled(self.q_gain, self.q_heads, d, self.head_dim).contiguous()
                self.k_gain = self._filled(self.k_gain, self.kv_heads, d, self.head_dim).contiguous()
        if self.bias_names:
            self.bias = torch.cat([self._filled(tensors.pop(self.bias_names["q"]), self.q_heads, d, self.head_dim),
                                   self._filled(tensors.pop(self.bias_names["k"]), self.kv_heads, d, self.head_dim),
                                   self._filled(tensors.pop(self.bias_names["v"]), self.kv_heads, e, self.value_dim)]).contiguous()
        if self.conv is not None:
            for name, heads, size, to in zip(self.conv.names, (self.q_heads, self.kv_heads, self.kv_heads), (d, d, e),
                                             (self.head_dim, self.head_dim, self.value_dim)):
                tensors[name] = self._filled(tensors[name], heads, size, to)
            self.conv.bind(tensors)
        if self.slope_values is not None:
            self.slopes = torch.tensor(self.slope_values, dtype=torch.float32, device=self.w_o.device)

    def streamed_weights(self) -> List[torch.Tensor]:
        return [self.w_qkv, self.w_o]

    fused_io = True
    prepares_next = True

    def forward(self, y, step: StepContext, cache,
                residual: Optional[torch.Tensor] = None, next_norm=None):
        """``y`` may be a norm still to be done; with ``residual`` the result may be added there (None returned),
        and with ``next_norm`` the norm that follows may come back prepared (see ``ops.linear``)."""
        out_dtype = torch.float32 if self.float_output else None
        rotation = rotation_of(self.position)
        if rotation.cos is not None and step.max_position >= rotation.cos.shape[0]:
            raise ValueError(f"position {step.max_position} is beyond the rotary table of {rotation.cos.shape[0]} positions")
        conv_state = None
        if isinstance(cache, dict):
            cache, conv_state = cache["kv"], cache.get("conv")
        if self.general:
            proj = ops.linear(y, self.w_qkv, out_dtype=torch.float32)
            if proj.dim() == 3:
                proj = proj.sum(dim=0)
            heads = proj
            qw, kw, vw = self.q_heads * self.head_dim, self.kv_heads * self.head_dim, self.kv_heads * self.value_dim
            if self.conv is not None:
                # q, k and v pass their filters side by side in one launch; the gates' columns stay where they are
                heads = self.conv.forward(proj[:, :qw + kw + vw], step, conv_state, torch.float32)
            if self.bias is not None or self.wide_norm:
                # a span's mean is taken over the elements the projection has in the file, not over what fills it up
                spans = [(0, qw, self.q_gain, self.q_heads * self.file_head_dim),
                         (qw, kw, self.k_gain, self.kv_heads * self.file_head_dim)] if self.wide_norm else []
                ops.bias_span_norm(heads, self.bias, spans, self.qk_norm_eps if self.wide_norm else 1.0, round_to=step.dtype)
            head_gains = (None, None) if self.wide_norm else (self.q_gain, self.k_gain)
            q = ops.qk_norm_rope_write(heads, self.q_heads, self.kv_heads, self.head_dim, head_gains[0], head_gains[1],
                                       self.qk_norm_eps if self.qk_norm_eps is not None else 1.0, rotation.cos, rotation.sin,
                                       step.positions, step.row_entry, cache.block_table, cache.k_pool, cache.v_pool,
                                       write_cache=cache.writes and not self.shared_kv, out_dtype=step.dtype,
                                       pairing=rotation.pairing, value_dim=self.value_dim, queries_only=self.shared_kv)
            gate = None
            if "gate" in self.names:
                gate = proj[:, self.q_heads * self.head_dim:] if self.shared_kv else \
                    proj[:, (self.q_heads + self.kv_heads) * self.head_dim + self.kv_heads * self.value_dim:]
            attended = self._attend(q, step, cache, gate)
            return ops.linear(attended, self.w_o, out_dtype=out_dtype, residual=residual, next_norm=next_norm)
        qkv = ops.linear(y, self.w_qkv, planes_ok=True)
        # How much of a head is rotated and in which pairs is the position part's affair; the kernels are told.
        rotation = rotation_of(self.position)
        cos, sin = rotation.cos, rotation.sin
        if cos is not None and step.max_position >= cos.shape[0]:
            raise ValueError(f"position {step.max_position} is beyond the rotary table of {cos.shape[0]} positions")
        kernels = self.attention_kernels(step.dtype, cache.page_tokens, cache.block_table.shape[1])
        if step.decode_only and kernels["decode"] == "projected":
            # Single decoded tokens, every row another request: the attention kernel makes the heads itself.
            attended = ops.attention_decode_projected(
                qkv, self.q_heads, self.kv_heads, self.head_dim, self.q_gain, self.k_gain,
                self.qk_norm_eps if self.qk_norm_eps is not None else 1.0, cos, sin, cache.k_pool, cache.v_pool,
                step.positions, step.row_entry, cache.block_table, self.scale, int(self.window or 0),
                max_context=step.max_position + 1, write_cache=cache.writes, pairing=rotation.pairing)
            return ops.linear(attended, self.w_o, out_dtype=out_dtype, residual=residual, next_norm=next_norm)
        q = ops.qk_norm_rope_write(qkv, self.q_heads, self.kv_heads, self.head_dim, self.q_gain, self.k_gain,
                                   self.qk_norm_eps if self.qk_norm_eps is not None else 1.0, cos, sin,
                                   step.positions, step.row_entry, cache.block_table, cache.k_pool, cache.v_pool,
                                   write_cache=cache.writes, out_dtype=step.dtype, pairing=rotation.pairing)
        attended = self._attend(q, step, cache)
        return ops.linear(attended, self.w_o, out_dtype=out_dtype, residual=residual, next_norm=next_norm)

    def attention_kernels(self, dtype: torch.dtype, page_tokens: int, max_blocks: int = 0) -> Dict[str, str]:
        """Which kernels this shape gets, by kind of work: ``decode`` (steps of single tokens): "projected" (the
        split-KV matrix-core kernel that also makes the heads and writes the cache), "split_kv" (the same
        kernel behind the norm/rotation/write kernel) or "rows" (the float kernel for any shape and type);
        ``prompt`` (portions of at least ``ops.PREFILL_MIN_ROWS`` rows): "flash" (the matrix-core prompt
        kernel), else what single tokens get."""
        group = self.q_heads // self.kv_heads
        if self._rows_only() or not ops.decode_attention_supported(dtype, self.head_dim, page_tokens, group, max_blocks):
            return {"decode": "rows", "prompt": "rows"}
        rotation = rotation_of(self.position)
        projected = not self.general and ops.decode_projected_supported(self.head_dim, rotation.rotary_dim, rotation.pairing)
        return {"decode": "projected" if projected else "split_kv",
                "prompt": "flash" if ops.prefill_attention_supported(dtype, self.head_dim, page_tokens, max_blocks) else "split_kv"}

    def _rows_only(self) -> bool:
        """What the matrix-core kernels are not built for: values of another size than the keys."""
        return self.value_dim != self.head_dim

    def _attend(self, q: torch.Tensor, step: StepContext, cache: KvCacheView, gate: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Long prompt portions through the prompt kernel, the other rows through the split-KV kernel; the
        row kernel takes what the matrix-core kernels refuse (float32, odd sizes, values of another size than
        the keys).  ``gate``: the heads' gates (float32 ``[rows, q_heads]``), applied to the result."""
        window = int(self.window or 0)
        group = self.q_heads // self.kv_heads
        max_blocks = cache.block_table.shape[1]
        if self._rows_only() or \
                not ops.decode_attention_supported(q.dtype, self.head_dim, cache.page_tokens, group, max_blocks):
            return ops.attention_rows(q, cache.k_pool, cache.v_pool, step.positions, step.row_entry,
                                      cache.block_table, self.q_heads, self.scale, window, gate=gate,
                                      keep_first=self.keep_first, gate_each=self.gate_each, slopes=self.slopes,
                                      query_factor=self.query_factor)
        first = 0
        out = torch.empty_like(q)
        tiled = step.tiled.get(self.row_tiling())
        if (tiled is not None and tiled.rows
                and ops.prefill_attention_supported(q.dtype, self.head_dim, cache.page_tokens, max_blocks)):
            ops.attention_prefill(q, out, cache.k_pool, cache.v_pool, step.positions, tiled.tiles,
                                  cache.block_table, self.q_heads, self.scale, window,
                                  mean_keys=tiled.mean_keys or step.max_position + 1, covered_rows=tiled.rows,
                                  keep_first=self.keep_first, slopes=self.slopes, query_factor=self.query_factor)
            first = tiled.rows
        if first < step.rows:
            ops.attention_decode(q[first:], cache.k_pool, cache.v_pool, step.positions[first:],
                                 step.row_entry[first:], cache.block_table, self.q_heads, self.scale, window,
                                 max_context=step.max_position + 1, out=out[first:], keep_first=self.keep_first,
                                 slopes=self.slopes, query_factor=self.query_factor)
        if gate is None:
            return out
        # a gate for every element is a gate a head of one element
        return ops.head_gate(out, gate, self.q_heads * self.value_dim, 1) if self.gate_each else \
            ops.head_gate(out, gate, self.q_heads, self.value_dim)
