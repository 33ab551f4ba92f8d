"""Attention whose keys and values come out of a small latent that is all the cache holds."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional

import torch

from .. import ops
from ..weights.loader import MATRIX, VECTOR, TensorSpec
from .base import MIXERS, Part, PartSpec
from .context import CacheView, StepContext
from .position import rotation_of


@dataclass
class LatentCacheView(CacheView):
    k_pool: torch.Tensor = None        # [pages, ceil((rank + rot) / 8), page_tokens, 8]: a token's vector as a key
    v_pool: torch.Tensor = None        # [pages, page_tokens / 8, rank, 8]: its latent once more, as a value
    block_table: torch.Tensor = None   # int32 [entries, max_blocks] of the layer's group
    page_tokens: int = 0


@dataclass(frozen=True)
class LatentNeed:
    """A mixer that caches, per token, one latent of ``rank`` elements and a rotated key part of ``rot`` elements that
    all its heads share, in the engine's type.  The vector is kept twice, packed in runs of 8 in the order each of
    attention's two products reads it: as a key ``[pages, ceil((rank + rot) / 8), page_tokens, 8]`` and, its latent
    alone, as a value ``[pages, page_tokens / 8, rank, 8]``."""
    rank: int
    rot: int
    window: Optional[int] = None        # only the last `window` positions are ever read
    page_tokens: Optional[int] = None
    keep_first: int = 0

    paged = True

    def group_key(self):
        return self

    def allocate(self, pages: int, page_tokens: int, dtype: torch.dtype, device):
        if page_tokens % 8:
            raise ValueError(f"the cache packs runs of 8 tokens: page_tokens {page_tokens} must be a multiple of 8")
        return (torch.zeros((pages, -(-(self.rank + self.rot) // 8), page_tokens, 8), dtype=dtype, device=device),
                torch.zeros((pages, page_tokens // 8, self.rank, 8), dtype=dtype, device=device))

    def view(self, storage, block_table, page_tokens: int):
        return LatentCacheView(writes=True, k_pool=storage[0], v_pool=storage[1], block_table=block_table,
                               page_tokens=page_tokens)

    def poison(self, storage, index: torch.Tensor) -> None:
        for pool in storage:
            pool.index_fill_(0, index, float("nan"))

    def bytes_per_token(self, element_size: int) -> int:
        return (-(-(self.rank + self.rot) // 8) * 8 + self.rank) * element_size


@MIXERS.register("latent_attention")
class LatentAttention(Part):
    """Causal softmax attention with queries, keys and values that pass through latents.

    Queries: c_q = rmsnorm(W_dq y) * gain, q = W_uq c_q, head by head ``dim`` plain elements and ``rot_dim`` rotated
    ones.  Keys and values: W_dkv y gives ``kv_rank`` elements, RMS-normed times a gain (the latent c), and ``rot_dim``
    more that are rotated and serve every head as the rotated part of its key.  Head h's plain key is W_uk[h] c, its
    value W_uv[h] c; score = (q_plain . k_plain + q_rot . k_rot) * ``scale``; a row sees its request's keys at positions
    pos - window < j <= pos (``window`` None: all); softmax; out = W_o on the heads side by side.

    The cache holds c and the rotated part only (``LatentNeed``).  The up-projections are never applied to cached
    tokens: W_uk goes to the query's side (q_plain W_uk[h], a product a head) and W_uv to the result's side (W_uv[h]
    on the weighted sum of the latents), so attention runs over the latents themselves, shared by all heads.

    Parameters: ``hidden``, ``heads``, ``dim``, ``rot_dim``, ``vdim``, ``q_rank``, ``kv_rank``, ``scale``, ``eps``,
    ``window``, ``position`` (name of a position part; its width may be less than ``rot_dim``), tensor names ``dq``,
    ``dq_norm``, ``uq``, ``uk``, ``uv``, ``o`` and, unless ``shared_kv``, ``dkv`` and ``dkv_norm``.  With ``q_rank`` None
    the queries come straight from the input, q = W_q y, and the tensor name ``q`` stands for ``dq``, ``dq_norm`` and
    ``uq``.  The kernels rotate neighbouring pairs (2i, 2i + 1); a position part that pairs element i with element
    i + R/2 is served by putting the rows of W_q's (W_uq's) rotated part and of W_dkv's last ``rot_dim`` rows in the order
    (0, R/2, 1, R/2 + 1, ...) when the weights are bound: the rotated parts only ever meet each other in a dot product,
    which no common reordering of its two sides changes.  ``shared_kv``: the layer has no W_dkv and reads the cache another layer writes (its run names that
    layer's cache slot and does not write).  ``retain_window``: what the cache must keep if layers with wider windows
    read it too (by default this layer's ``window``; 0: everything).
    """

    graph_safe = True

    def __init__(self, spec: PartSpec, positions: Optional[dict] = None, **_):
        p = spec.params
        self.hidden, self.heads, self.dim, self.rot_dim, self.vdim, self.kv_rank = (
            int(p[k]) for k in ("hidden", "heads", "dim", "rot_dim", "vdim", "kv_rank"))
        self.q_rank = int(p["q_rank"]) if p.get("q_rank") else None
        self.scale, self.eps = float(p["scale"]), float(p["eps"])
        self.window = int(p["window"]) if p.get("window") else None
        self.retain_window = self.window if "retain_window" not in p else (p["retain_window"] or None)
        self.shared_kv = bool(p.get("shared_kv", False))
        keys = (("q",) if self.q_rank is None else ("dq", "dq_norm", "uq")) + ("uk", "uv", "o") + \
            (() if self.shared_kv else ("dkv", "dkv_norm"))
        self.names = {k: p[k] for k in keys}
        self.position = (positions or {}).get(p.get("position")) if p.get("position") else None
        if p.get("position") and self.position is None:
            raise ValueError(f"latent attention names position part {p.get('position')!r}, which the model does not define")
        self.w_down = self.w_uq = self.w_uk = self.w_uv = self.w_o = self.q_gain = self.kv_gain = None

    def cache_need(self) -> LatentNeed:
        return LatentNeed(self.kv_rank, self.rot_dim, self.retain_window)

    def tensor_specs(self) -> List[TensorSpec]:
        n = self.names
        if self.q_rank is None:
            specs = [TensorSpec(n["q"], (self.heads * (self.dim + self.rot_dim), self.hidden), MATRIX)]
        else:
            specs = [TensorSpec(n["dq"], (self.q_rank, self.hidden), MATRIX), TensorSpec(n["dq_norm"], (self.q_rank,), VECTOR),
                     TensorSpec(n["uq"], (self.heads * (self.dim + self.rot_dim), self.q_rank), MATRIX)]
        if not self.shared_kv:
            specs += [TensorSpec(n["dkv"], (self.kv_rank + self.rot_dim, self.hidden), MATRIX),
                      TensorSpec(n["dkv_norm"], (self.kv_rank,), VECTOR)]
        return specs + [TensorSpec(n["uk"], (self.heads * self.dim, self.kv_rank), MATRIX),
                        TensorSpec(n["uv"], (self.heads * self.vdim, self.kv_rank), MATRIX),
                        TensorSpec(n["o"], (self.hidden, self.heads * self.vdim), MATRIX)]

    def _paired(self, rows: torch.Tensor, first: int) -> torch.Tensor:
        """``rows`` with rows first .. first + R of a part that a half-split rotation turns put in the order the
        kernels' neighbouring pairs need: (0, R/2, 1, R/2 + 1, ...)."""
        rotation = rotation_of(self.position)
        if rotation.pairing != "half_split" or not rotation.rotary_dim:
            return rows
        half = rotation.rotary_dim // 2
        order = torch.arange(rows.shape[0], device=rows.device)
        turned = torch.stack([torch.arange(half), torch.arange(half) + half], dim=1).reshape(-1).to(rows.device)
        order[first:first + 2 * half] = first + turned
        return rows.index_select(0, order)

    def _paired_heads(self, rows: torch.Tensor) -> torch.Tensor:
        """The same for the queries' projection: the rotated part of every head."""
        size = self.dim + self.rot_dim
        heads = [self._paired(rows[h * size:(h + 1) * size], self.dim) for h in range(self.heads)]
        return torch.cat(heads, dim=0)

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        n = self.names
        rotation = rotation_of(self.position)
        if rotation.rotary_dim > self.rot_dim:
            raise ValueError(f"latent attention: a rotation of {rotation.rotary_dim} elements on a part of {self.rot_dim}")
        dkv = [] if self.shared_kv else [self._paired(tensors.pop(n["dkv"]), self.kv_rank)]
        if self.q_rank is None:
            down = [self._paired_heads(tensors.pop(n["q"]))] + dkv
            self.w_uq = None
        else:
            down = [tensors.pop(n["dq"])] + dkv
            self.w_uq = self._paired_heads(tensors.pop(n["uq"])).contiguous()
        self.w_down = torch.cat(down, dim=0).contiguous()             # one product for everything that reads the input
        # a product a head: [heads, inner, outer]; W_uk as stored is [heads, dim, rank] already, W_uv is turned
        self.w_uk = tensors.pop(n["uk"]).view(self.heads, self.dim, self.kv_rank).contiguous()
        self.w_uv = tensors.pop(n["uv"]).view(self.heads, self.vdim, self.kv_rank).transpose(1, 2).contiguous()
        self.w_o = tensors.pop(n["o"]).contiguous()
        self.q_gain = tensors.pop(n["dq_norm"]).contiguous() if self.q_rank is not None else None
        self.kv_gain = self.q_gain if self.shared_kv else tensors.pop(n["dkv_norm"]).contiguous()
        if self.q_gain is not None and self.q_gain.dtype != self.kv_gain.dtype:
            self.q_gain, self.kv_gain = self.q_gain.float(), self.kv_gain.float()

    def streamed_weights(self) -> List[torch.Tensor]:
        return [w for w in (self.w_down, self.w_uq, self.w_o) if w is not None]

    def forward(self, y: torch.Tensor, step: StepContext, cache: LatentCacheView) -> torch.Tensor:
        rotation = rotation_of(self.position)
        if rotation.cos is not None and step.max_position >= rotation.cos.shape[0]:
            raise ValueError(f"position {step.max_position} is beyond the rotary table of {rotation.cos.shape[0]} positions")
        writes = cache.writes and not self.shared_kv
        down = ops.linear(ops.materialize(y), self.w_down, out_dtype=torch.float32)
        if down.dim() == 3:
            down = down.sum(dim=0)
        direct = self.q_rank is None
        q_width = self.heads * (self.dim + self.rot_dim)
        if not direct or writes:
            c_q = ops.latent_prepare(down, step.dtype, self.eps, q_column=None if direct else 0, q_rank=self.q_rank or 0,
                                     q_gain=self.q_gain, kv_column=(q_width if direct else self.q_rank) if writes else None,
                                     rank=self.kv_rank, rot=self.rot_dim, kv_gain=self.kv_gain, cos=rotation.cos,
                                     sin=rotation.sin, positions=step.positions, row_entry=step.row_entry,
                                     block_table=cache.block_table, k_pool=cache.k_pool, v_pool=cache.v_pool)
        if direct:
            q = down[:, :q_width]               # the queries came out of the same product, a slice of its rows
        else:
            q = ops.linear(c_q, self.w_uq, out_dtype=torch.float32)
            if q.dim() == 3:
                q = q.sum(dim=0)
        # W_uk on the query's side; the rotated query part behind it.  The matrix-core kernel reads its queries in bfloat16.
        cores = ops.latent_cores_supported(step.dtype, self.kv_rank, self.rot_dim, cache.page_tokens)
        q = ops.head_product(q, self.w_uk, self.heads, step.dtype if cores else torch.float32, tail=self.rot_dim,
                             cos=rotation.cos, sin=rotation.sin, positions=step.positions)
        mixed = ops.latent_attention(q, cache.k_pool, cache.v_pool, step.positions, step.row_entry, cache.block_table,
                                     self.heads, self.kv_rank, self.rot_dim, self.scale, int(self.window or 0),
                                     max_position=step.max_position)
        values = ops.head_product(mixed, self.w_uv, self.heads, step.dtype)
        return ops.linear(values, self.w_o, out_dtype=torch.float32)
