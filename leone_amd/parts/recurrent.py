"""Mixers that carry a matrix memory per request and head from token to token, and a mixer made of several
side by side.  Their recurrences run in float32 whatever the engine's type; the state lives in the request's
state slot and starts at zero."""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

from .. import ops
from ..weights.loader import MATRIX, VECTOR, TensorSpec
from .base import CONVS, MIXERS, Part, PartSpec, StateNeed
from .context import StepContext
from .position import rotation_of


SCAN_MAX_DIM = 256      # key channels a head may have: 32 a lane over at most 8 lanes (csrc/recurrent.hip)


def _check_dim(kind: str, dim: int) -> None:
    if dim > SCAN_MAX_DIM:
        raise ValueError(f"{kind}: heads of {dim} key channels; the recurrence kernels take up to {SCAN_MAX_DIM}")


@MIXERS.register("mlstm")
class MlstmMixer(Part):
    """Matrix memory with exponential gates (the mLSTM cell of xLSTM).

    Per head, with q = Wq h / sqrt(dim), k = Wk h, v = Wv h, log gates i = soft_cap(Wi h + bi) and
    f = logsigmoid(soft_cap(Wf h + bf)), soft_cap(z) = cap * tanh(z / cap), and a running maximum m that starts
    at 0:  m' = max(f + m, i);  S' = exp(f + m - m') S + exp(i - m') k v^T;  n' likewise with k alone;
    o = S'^T q / (max(|n' . q|, exp(-m')) + 1e-6).  Each head's o over its root mean square, times ``norm``
    (all heads' size), times sigmoid(Wg h), then Wo.

    Parameters: ``hidden``, ``heads``, ``dim``, ``vdim``, ``gate_cap``, ``eps`` and tensor names ``q``, ``k``,
    ``v``, ``g``, ``o``, ``norm``, ``i``, ``i_bias``, ``f``, ``f_bias``.
    """

    graph_safe = True

    def __init__(self, spec: PartSpec, **_):
        p = spec.params
        self.hidden, self.heads, self.dim, self.vdim = (int(p[k]) for k in ("hidden", "heads", "dim", "vdim"))
        self.cap, self.eps = float(p["gate_cap"]), float(p["eps"])
        _check_dim("mlstm", self.dim)
        self.names = {k: p[k] for k in ("q", "k", "v", "g", "o", "norm", "i", "i_bias", "f", "f_bias")}
        qk, vv = self.heads * self.dim, self.heads * self.vdim
        self.columns = {"q": 0, "k": qk, "v": 2 * qk, "g": 2 * qk + vv, "i": 2 * qk + 2 * vv, "f": 2 * qk + 2 * vv + self.heads}
        self.w_in = self.w_o = self.norm = self.i_bias = self.f_bias = None

    def tensor_specs(self) -> List[TensorSpec]:
        n, qk, vv = self.names, self.heads * self.dim, self.heads * self.vdim
        return [TensorSpec(n["q"], (qk, self.hidden), MATRIX), TensorSpec(n["k"], (qk, self.hidden), MATRIX),
                TensorSpec(n["v"], (vv, self.hidden), MATRIX), TensorSpec(n["g"], (vv, self.hidden), MATRIX),
                TensorSpec(n["o"], (self.hidden, vv), MATRIX), TensorSpec(n["norm"], (vv,), VECTOR),
                TensorSpec(n["i"], (self.heads, self.hidden), MATRIX), TensorSpec(n["i_bias"], (self.heads,), VECTOR),
                TensorSpec(n["f"], (self.heads, self.hidden), MATRIX), TensorSpec(n["f_bias"], (self.heads,), VECTOR)]

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        # one product for everything that reads h: q, k, v, the output gate and the two cell gates
        self.w_in = torch.cat([tensors.pop(self.names[k]) for k in ("q", "k", "v", "g", "i", "f")], dim=0).contiguous()
        self.w_o = tensors.pop(self.names["o"]).contiguous()
        self.norm = tensors.pop(self.names["norm"]).contiguous()
        self.i_bias = tensors.pop(self.names["i_bias"]).contiguous()
        self.f_bias = tensors.pop(self.names["f_bias"]).contiguous()
        if self.i_bias.dtype != self.f_bias.dtype:
            self.i_bias, self.f_bias = self.i_bias.float(), self.f_bias.float()

    def streamed_weights(self) -> List[torch.Tensor]:
        return [self.w_in, self.w_o]

    def cache_need(self) -> StateNeed:
        # S [dim, vdim], then n [dim], then m, head by head
        return StateNeed((self.heads, self.dim * self.vdim + self.dim + 1), torch.float32)

    def forward(self, h: torch.Tensor, step: StepContext, cache) -> torch.Tensor:
        proj = ops.linear(h, self.w_in, out_dtype=torch.float32)
        o, under = ops.outer_scan(proj, self.columns, cache.state, step, self.heads, self.dim, self.vdim,
                                  gates={"i_bias": self.i_bias, "f_bias": self.f_bias, "cap": self.cap},
                                  q_scale=1.0 / math.sqrt(self.dim), write_state=cache.writes)
        gate = proj[:, self.columns["g"]:self.columns["i"]]
        y = ops.head_norm_gate(o, self.heads, self.vdim, self.eps, step.dtype, gain=self.norm, gate=gate,
                               activation="sigmoid", denominator=under)
        return ops.linear(y, self.w_o, out_dtype=torch.float32)


@MIXERS.register("retention")
class RetentionMixer(Part):
    """Linear attention with one fixed decay a head, no softmax and no denominator.

    q = Wq h, k = Wk h / sqrt(dim) (after the rotation), v = Wv h; rotary positions on q and k as the
    position part says; per head S' = decay S + k v^T, o = S'^T q; each head's o over its root mean square (no
    gain), times silu(Wg h), then Wo.

    Parameters: ``hidden``, ``heads``, ``dim``, ``vdim``, ``decay`` (one number a head), ``eps``, ``position``
    (name of a position part, or None) and tensor names ``q``, ``k``, ``v``, ``g``, ``o``.
    """

    graph_safe = True

    def __init__(self, spec: PartSpec, positions: Optional[dict] = None, **_):
        p = spec.params
        self.hidden, self.heads, self.dim, self.vdim = (int(p[k]) for k in ("hidden", "heads", "dim", "vdim"))
        self.eps = float(p["eps"])
        _check_dim("retention", self.dim)
        self.decay_values = [float(d) for d in p["decay"]]
        if len(self.decay_values) != self.heads:
            raise ValueError(f"retention: {len(self.decay_values)} decays for {self.heads} heads")
        self.names = {k: p[k] for k in ("q", "k", "v", "g", "o")}
        self.position = (positions or {}).get(p.get("position")) if p.get("position") else None
        if p.get("position") and self.position is None:
            raise ValueError(f"retention names position part {p.get('position')!r}, which the model does not define")
        qk, vv = self.heads * self.dim, self.heads * self.vdim
        self.columns = {"q": 0, "k": qk, "v": 2 * qk, "g": 2 * qk + vv}
        self.w_in = self.w_o = self.decay = None

    def tensor_specs(self) -> List[TensorSpec]:
        n, qk, vv = self.names, self.heads * self.dim, self.heads * self.vdim
        return [TensorSpec(n["q"], (qk, self.hidden), MATRIX), TensorSpec(n["k"], (qk, self.hidden), MATRIX),
                TensorSpec(n["v"], (vv, self.hidden), MATRIX), TensorSpec(n["g"], (vv, self.hidden), MATRIX),
                TensorSpec(n["o"], (self.hidden, vv), MATRIX)]

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.w_in = torch.cat([tensors.pop(self.names[k]) for k in ("q", "k", "v", "g")], dim=0).contiguous()
        self.w_o = tensors.pop(self.names["o"]).contiguous()
        self.decay = torch.tensor(self.decay_values, dtype=torch.float32, device=self.w_o.device)

    def streamed_weights(self) -> List[torch.Tensor]:
        return [self.w_in, self.w_o]

    def cache_need(self) -> StateNeed:
        return StateNeed((self.heads, self.dim * self.vdim), torch.float32)

    def forward(self, h: torch.Tensor, step: StepContext, cache) -> torch.Tensor:
        proj = ops.linear(h, self.w_in, out_dtype=torch.float32)
        rotation = rotation_of(self.position)
        if rotation.cos is not None:
            if rotation.pairing != "half_split":
                raise ValueError("retention rotates in half-split pairs only")
            if step.max_position >= rotation.cos.shape[0]:
                raise ValueError(f"position {step.max_position} is beyond the rotary table of {rotation.cos.shape[0]} positions")
        o, _ = ops.outer_scan(proj, self.columns, cache.state, step, self.heads, self.dim, self.vdim, decay=self.decay,
                              k_scale=1.0 / math.sqrt(self.dim), cos=rotation.cos, sin=rotation.sin,
                              write_state=cache.writes)
        y = ops.head_norm_gate(o, self.heads, self.vdim, self.eps, step.dtype, gate=proj[:, self.columns["g"]:],
                               activation="silu")
        return ops.linear(y, self.w_o, out_dtype=torch.float32)


@MIXERS.register("channel_delta")
class ChannelDeltaMixer(Part):
    """The gated delta rule with one decay per head and key channel.

    q = Wq h, k = Wk h (``kv_heads`` heads of ``dim``; head h of the memory uses q/k head h // (heads / kv_heads)),
    v = Wv h (``heads`` of ``vdim``); each through a short causal convolution and silu; q and k made unit vectors
    per head (x / sqrt(sum x^2 + 1e-6)), q times dim^-1/2; beta = sigmoid(Wb h) a head;
    g = exp(-exp(A_log) * softplus(Wa2 (Wa1 h) + dt_bias)) per head and key channel.  Per head:
    S <- g * S (rows of S are key channels); u = beta (v - S^T k); S <- S + k u^T; o = S^T q.  Each head's o over
    its root mean square, times ``norm`` (size vdim, shared by the heads), times sigmoid(Wg2 (Wg1 h)), then Wo.

    Parameters: ``hidden``, ``heads``, ``kv_heads``, ``dim``, ``vdim``, ``taps``, ``eps`` and tensor names ``q``,
    ``k``, ``v``, ``q_conv``, ``k_conv``, ``v_conv``, ``b``, ``A_log``, ``dt_bias``, ``a1``, ``a2``, ``g1``, ``g2``,
    ``norm``, ``o``.  The ranks of the two low-rank pairs come with ``a_rank`` and ``g_rank``.
    """

    graph_safe = True
    UNIT_EPS = 1e-6

    def __init__(self, spec: PartSpec, **context):
        p = spec.params
        self.hidden, self.heads, self.kv_heads, self.dim, self.vdim = (
            int(p[k]) for k in ("hidden", "heads", "kv_heads", "dim", "vdim"))
        if self.heads % self.kv_heads:
            raise ValueError(f"channel_delta: {self.heads} heads cannot be grouped over {self.kv_heads} q/k heads")
        _check_dim("channel_delta", self.dim)
        self.eps, self.a_rank, self.g_rank = float(p["eps"]), int(p["a_rank"]), int(p["g_rank"])
        self.names = {k: p[k] for k in ("q", "k", "v", "b", "A_log", "dt_bias", "a1", "a2", "g1", "g2", "norm", "o")}
        qk, vv = self.kv_heads * self.dim, self.heads * self.vdim
        self.conv = CONVS.build(PartSpec("causal_conv", {"channels": [qk, qk, vv], "taps": int(p["taps"]),
                                                         "weights": [p["q_conv"], p["k_conv"], p["v_conv"]],
                                                         "activation": "silu"}), **context)
        self.columns = {"q": 0, "k": qk, "v": 2 * qk, "b": 2 * qk + vv, "a1": 2 * qk + vv + self.heads,
                        "g1": 2 * qk + vv + self.heads + self.a_rank}
        self.conv_width = 2 * qk + vv
        self.w_in = self.w_a2 = self.w_g2 = self.w_o = self.norm = self.rate_log = self.step_bias = None

    def tensor_specs(self) -> List[TensorSpec]:
        n, qk, vv = self.names, self.kv_heads * self.dim, self.heads * self.vdim
        return [TensorSpec(n["q"], (qk, self.hidden), MATRIX), TensorSpec(n["k"], (qk, self.hidden), MATRIX),
                TensorSpec(n["v"], (vv, self.hidden), MATRIX), TensorSpec(n["b"], (self.heads, self.hidden), MATRIX),
                TensorSpec(n["A_log"], (self.heads,), VECTOR), TensorSpec(n["dt_bias"], (self.heads * self.dim,), VECTOR),
                TensorSpec(n["a1"], (self.a_rank, self.hidden), MATRIX),
                TensorSpec(n["a2"], (self.heads * self.dim, self.a_rank), MATRIX),
                TensorSpec(n["g1"], (self.g_rank, self.hidden), MATRIX), TensorSpec(n["g2"], (vv, self.g_rank), MATRIX),
                TensorSpec(n["norm"], (self.vdim,), VECTOR), TensorSpec(n["o"], (self.hidden, vv), MATRIX)] \
            + self.conv.tensor_specs()

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.w_in = torch.cat([tensors.pop(self.names[k]) for k in ("q", "k", "v", "b", "a1", "g1")], dim=0).contiguous()
        self.w_a2 = tensors.pop(self.names["a2"]).contiguous()
        self.w_g2 = tensors.pop(self.names["g2"]).contiguous()
        self.w_o = tensors.pop(self.names["o"]).contiguous()
        self.norm = tensors.pop(self.names["norm"]).contiguous()
        self.rate_log = tensors.pop(self.names["A_log"]).contiguous()
        self.step_bias = tensors.pop(self.names["dt_bias"]).contiguous()
        if self.rate_log.dtype != self.step_bias.dtype:
            self.rate_log, self.step_bias = self.rate_log.float(), self.step_bias.float()
        self.conv.bind(tensors)

    def streamed_weights(self) -> List[torch.Tensor]:
        return [self.w_in, self.w_o]

    def cache_need(self):
        return {"conv": self.conv.cache_need(), "memory": StateNeed((self.heads, self.dim, self.vdim), torch.float32)}

    def forward(self, h: torch.Tensor, step: StepContext, cache) -> torch.Tensor:
        c = self.columns
        proj = ops.linear(h, self.w_in, out_dtype=torch.float32)
        qkv = self.conv.forward(proj[:, :self.conv_width], step, cache["conv"], torch.float32)
        # the two low-rank pairs: their narrow halves came out of the fused product
        step_size = ops.linear(proj[:, c["a1"]:c["g1"]].to(step.dtype).contiguous(), self.w_a2, out_dtype=torch.float32)
        gate = ops.linear(proj[:, c["g1"]:].to(step.dtype).contiguous(), self.w_g2, out_dtype=torch.float32)
        memory = cache["memory"]
        o = ops.delta_scan(qkv, {"q": c["q"], "k": c["k"], "v": c["v"]}, proj[:, c["b"]:c["a1"]], step_size,
                           self.rate_log, self.step_bias, memory.state, step, self.heads, self.kv_heads, self.dim,
                           self.vdim, q_scale=1.0 / math.sqrt(self.dim), unit_eps=self.UNIT_EPS, write_state=memory.writes)
        y = ops.head_norm_gate(o, self.heads, self.vdim, self.eps, step.dtype, gain=self.norm, gate=gate,
                               activation="sigmoid")
        return ops.linear(y, self.w_o, out_dtype=torch.float32)


@MIXERS.register("hgrn2")
class GatedMemoryMixer(Part):
    """Linear attention whose forget gate also decides what is written (HGRN2): there is no key projection.

    q = silu(Wq h) (``heads`` of ``dim``), v = Wv h (``heads`` of ``vdim``), forget gate per head and key channel
    f = lower + (1 - lower) * sigmoid(Wf h + f_bias) with a stored lower bound.  Per head S' = diag(f) S + (1 - f) v^T
    (f on the rows of S that belong to q's channels), o = S'^T q; each head's o over its root mean square times ``norm``
    (size vdim, shared by the heads), then Wo.  The state is float32 and starts at zero.

    Parameters: ``hidden``, ``heads``, ``dim``, ``vdim``, ``eps`` and tensor names ``q``, ``f``, ``f_bias``, ``lower``,
    ``v``, ``norm``, ``o``.
    """

    graph_safe = True

    def __init__(self, spec: PartSpec, **_):
        p = spec.params
        self.hidden, self.heads, self.dim, self.vdim = (int(p[k]) for k in ("hidden", "heads", "dim", "vdim"))
        self.eps = float(p["eps"])
        _check_dim("hgrn2", self.dim)
        self.names = {k: p[k] for k in ("q", "f", "f_bias", "lower", "v", "norm", "o")}
        qk = self.heads * self.dim
        self.columns = {"q": 0, "f": qk, "v": 2 * qk}
        self.w_in = self.w_o = self.norm = self.f_bias = self.lower = None

    def tensor_specs(self) -> List[TensorSpec]:
        n, qk, vv = self.names, self.heads * self.dim, self.heads * self.vdim
        return [TensorSpec(n["q"], (qk, self.hidden), MATRIX), TensorSpec(n["f"], (qk, self.hidden), MATRIX),
                TensorSpec(n["f_bias"], (qk,), VECTOR, init=("normal", 0.0, 1.0)),
                TensorSpec(n["lower"], (qk,), VECTOR, init=("uniform", 0.0, 1.0)),      # a lower bound of a gate in (0, 1)
                TensorSpec(n["v"], (vv, self.hidden), MATRIX), TensorSpec(n["norm"], (self.vdim,), VECTOR),
                TensorSpec(n["o"], (self.hidden, vv), MATRIX)]

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.w_in = torch.cat([tensors.pop(self.names[k]) for k in ("q", "f", "v")], dim=0).contiguous()
        self.w_o = tensors.pop(self.names["o"]).contiguous()
        self.norm = tensors.pop(self.names["norm"]).contiguous()
        self.f_bias = tensors.pop(self.names["f_bias"]).contiguous()
        self.lower = tensors.pop(self.names["lower"]).contiguous()
        if self.f_bias.dtype != self.lower.dtype:
            self.f_bias, self.lower = self.f_bias.float(), self.lower.float()

    def streamed_weights(self) -> List[torch.Tensor]:
        return [self.w_in, self.w_o]

    def cache_need(self) -> StateNeed:
        return StateNeed((self.heads, self.dim * self.vdim), torch.float32)

    def forward(self, h: torch.Tensor, step: StepContext, cache) -> torch.Tensor:
        proj = ops.linear(h, self.w_in, out_dtype=torch.float32)
        o = ops.gated_scan(proj, self.columns, self.f_bias, self.lower, cache.state, step, self.heads, self.dim, self.vdim,
                           q_activation="silu", write_state=cache.writes)
        y = ops.head_norm_gate(o, self.heads, self.vdim, self.eps, step.dtype, gain=self.norm)
        return ops.linear(y, self.w_o, out_dtype=torch.float32)


@MIXERS.register("state_space")
class StateSpaceMixer(Part):
    """A selective state-space layer with one decay a head (Mamba-2).

    One input projection gives, side by side, z (``heads * vdim``), x (``heads * vdim``), B and C (``groups * state``
    each) and a step size a head.  x, B and C together pass a short causal convolution per channel (with a bias) and
    silu.  dt = softplus(step + dt_bias); per head, with group g = head // (heads / groups):
    S <- exp(-exp(A_log) dt) S + dt B_g x^T (S is ``state`` x ``vdim``, float32, from zero), y = S^T C_g + D x.
    y times silu(z), then normed in ``norm_groups`` equal runs of columns, each by its own root mean square, times
    ``norm`` (all columns' size), then the output projection.  The gate stands ahead of the norm.

    Parameters: ``hidden``, ``heads``, ``vdim``, ``state``, ``groups``, ``norm_groups``, ``taps``, ``eps`` and tensor
    names ``in``, ``conv``, ``conv_bias``, ``dt_bias``, ``A_log``, ``D``, ``norm``, ``o``.
    """

    graph_safe = True

    def __init__(self, spec: PartSpec, **context):
        p = spec.params
        self.hidden, self.heads, self.vdim, self.state, self.groups, self.norm_groups = (
            int(p[k]) for k in ("hidden", "heads", "vdim", "state", "groups", "norm_groups"))
        self.eps = float(p["eps"])
        _check_dim("state_space", self.state)
        self.inner = self.heads * self.vdim
        if self.heads % self.groups:
            raise ValueError(f"state_space: {self.heads} heads do not share {self.groups} groups evenly")
        if self.inner % self.norm_groups:
            raise ValueError(f"state_space: {self.inner} columns cannot be normed in {self.norm_groups} equal runs")
        self.names = {k: p[k] for k in ("in", "conv_bias", "dt_bias", "A_log", "D", "norm", "o")}
        bc = self.groups * self.state
        self.conv_width = self.inner + 2 * bc
        self.conv = CONVS.build(PartSpec("causal_conv", {"channels": self.conv_width, "taps": int(p["taps"]),
                                                         "weights": [p["conv"]], "activation": "silu"}), **context)
        # the projection's columns, and x, B and C within what the convolution hands on
        self.columns = {"z": 0, "xbc": self.inner, "dt": self.inner + self.conv_width}
        self.scan_columns = {"x": 0, "b": self.inner, "c": self.inner + bc}
        self.w_in = self.w_o = self.norm = self.conv_bias = self.step_bias = self.rate_log = self.skip = None

    def tensor_specs(self) -> List[TensorSpec]:
        n = self.names
        return [TensorSpec(n["in"], (self.inner + self.conv_width + self.heads, self.hidden), MATRIX),
                TensorSpec(n["conv_bias"], (self.conv_width,), VECTOR, init=("normal", 0.0, 0.02)),
                # step sizes around softplus(-2 .. 0) and rates exp(0 .. 1.5): memories that reach tens of tokens back
                TensorSpec(n["dt_bias"], (self.heads,), VECTOR, init=("uniform", -2.0, 0.0)),
                TensorSpec(n["A_log"], (self.heads,), VECTOR, init=("uniform", 0.0, 1.5)),
                TensorSpec(n["D"], (self.heads,), VECTOR), TensorSpec(n["norm"], (self.inner,), VECTOR),
                TensorSpec(n["o"], (self.hidden, self.inner), MATRIX)] + self.conv.tensor_specs()

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        n = self.names
        self.w_in = tensors.pop(n["in"]).contiguous()
        self.w_o = tensors.pop(n["o"]).contiguous()
        self.norm = tensors.pop(n["norm"]).contiguous()
        self.conv.bind(tensors)
        self.conv_bias = tensors.pop(n["conv_bias"]).to(self.conv.weight.dtype).contiguous()
        self.step_bias, self.rate_log, self.skip = (tensors.pop(n[k]).contiguous() for k in ("dt_bias", "A_log", "D"))
        if len({self.step_bias.dtype, self.rate_log.dtype, self.skip.dtype}) > 1:
            self.step_bias, self.rate_log, self.skip = self.step_bias.float(), self.rate_log.float(), self.skip.float()

    def streamed_weights(self) -> List[torch.Tensor]:
        return [self.w_in, self.w_o]

    def cache_need(self):
        return {"conv": self.conv.cache_need(), "memory": StateNeed((self.heads, self.state * self.vdim), torch.float32)}

    def forward(self, h: torch.Tensor, step: StepContext, cache) -> torch.Tensor:
        c = self.columns
        proj = ops.linear(ops.materialize(h), self.w_in, out_dtype=torch.float32)
        if proj.dim() == 3:
            proj = proj.sum(dim=0)
        conv_cache = cache["conv"]
        xbc = ops.causal_conv(proj[:, c["xbc"]:c["dt"]], self.conv.weight, conv_cache.state, step, torch.float32,
                              activation="silu", write_state=conv_cache.writes, bias=self.conv_bias)
        memory = cache["memory"]
        y = ops.state_space_scan(xbc, self.scan_columns, self.groups, proj[:, c["dt"]:], self.step_bias, self.rate_log,
                                 self.skip, memory.state, step, self.heads, self.state, self.vdim, write_state=memory.writes)
        y = ops.head_norm_gate(y, self.norm_groups, self.inner // self.norm_groups, self.eps, step.dtype, gain=self.norm,
                               gate=proj[:, c["z"]:c["xbc"]], activation="silu", gate_first=True)
        return ops.linear(y, self.w_o, out_dtype=torch.float32)


@MIXERS.register("parallel")
class ParallelMixer(Part):
    """Several mixers side by side on the same input: each result is divided by its root mean square over the
    model width and multiplied by a plain gain of its own; the mixer's result is ``scale`` times their sum (the
    mean for ``scale`` = 1 / branches, the default).  With ``weights`` (a dict name -> number) instead of ``gains``
    nothing is normed: the result is the sum of the branches' results, each times its weight.

    Parameters: ``hidden``, ``eps``, ``branches`` (a dict name -> mixer spec), ``gains`` (a dict name -> tensor
    name) or ``weights``, ``scale`` (optional, with ``gains``).
    """

    def __init__(self, spec: PartSpec, **context):
        p = spec.params
        self.hidden, self.eps = int(p["hidden"]), float(p["eps"])
        self.branches = {name: MIXERS.build(inner, **context) for name, inner in p["branches"].items()}
        self.weights = {name: float(v) for name, v in p["weights"].items()} if p.get("weights") is not None else None
        self.gain_names = dict(p.get("gains") or {})
        if (self.weights is None) == (not self.gain_names):
            raise ValueError("parallel: either a gain or a weight for every branch")
        if set(self.gain_names if self.weights is None else self.weights) != set(self.branches) or not 1 <= len(self.branches) <= 4:
            raise ValueError("parallel: one gain, or one weight, for each of 1 to 4 branches")
        self.scale = float(p.get("scale") or 1.0 / len(self.branches))
        self.gains: Dict[str, torch.Tensor] = {}

    @property
    def graph_safe(self) -> bool:
        return all(getattr(b, "graph_safe", False) for b in self.branches.values())

    def tensor_specs(self) -> List[TensorSpec]:
        specs = [s for b in self.branches.values() for s in b.tensor_specs()]
        return specs + [TensorSpec(name, (self.hidden,), VECTOR) for name in self.gain_names.values()]

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        for branch in self.branches.values():
            branch.bind(tensors)
        self.gains = {name: tensors.pop(tensor).contiguous() for name, tensor in self.gain_names.items()}
        if len({g.dtype for g in self.gains.values()}) > 1:
            self.gains = {name: g.float() for name, g in self.gains.items()}

    def streamed_weights(self) -> List[torch.Tensor]:
        return [w for b in self.branches.values() if hasattr(b, "streamed_weights") for w in b.streamed_weights()]

    def row_tilings(self):
        return [b.row_tiling() for b in self.branches.values() if hasattr(b, "row_tiling")]

    def cache_need(self):
        return {name: b.cache_need() for name, b in self.branches.items()}

    def forward(self, h: torch.Tensor, step: StepContext, cache) -> torch.Tensor:
        h = ops.materialize(h)
        results = [b.forward(h, step, cache.get(name)) for name, b in self.branches.items()]
        results = [r.sum(dim=0) if r.dim() == 3 else r for r in results]
        results = [r if r.dtype == torch.float32 else r.float() for r in results]
        if self.weights is not None:
            return ops.weighted_mix(results, [self.weights[name] for name in self.branches])
        return ops.rms_mix(results, [self.gains[name] for name in self.branches], self.eps, self.scale)
