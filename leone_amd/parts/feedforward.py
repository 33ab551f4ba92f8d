"""Feed-forward parts."""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from .. import ops
from ..weights.loader import MATRIX, VECTOR, TensorSpec
from .base import FEED_FORWARDS, Part, PartSpec
from .context import StepContext


@FEED_FORWARDS.register("swiglu")
class SwiGluMlp(Part):
    """down(silu(gate y) * (up y)), no bias, silu(g) = g / (1 + exp(-g)).

    Reference: crates/leone/src/runtime.rs:9283-9319, crates/leone/src/cpu.rs:892-907.
    Parameters: ``hidden``, ``intermediate`` and tensor names ``gate``, ``up``, ``down``.
    Optional: ``activation`` (what stands on the gate instead of silu, a key of ``ops.GATE_ACTIVATIONS``),
    ``float_output`` (what is handed back comes in float32 whatever the engine's type), ``bias`` (a dict with tensor
    names ``gate``, ``up``, ``down``: all three projections add a bias; the products then hand on float32, the biases
    are added there, and the result comes in float32).
    """

    graph_safe = True

    def __init__(self, spec: PartSpec, **_):
        p = spec.params
        self.hidden = int(p["hidden"])
        self.intermediate = int(p["intermediate"])
        self.names = {k: p[k] for k in ("gate", "up", "down")}
        self.bias_names = dict(p["bias"]) if p.get("bias") else None
        self.bias_in = self.bias_out = None
        if self.bias_names:
            self.fused_io = self.prepares_next = False      # its products hand on float32 for the biases to be added
        self.activation = str(p.get("activation") or "silu")
        if self.activation not in ops.GATE_ACTIVATIONS:
            raise ValueError(f"unknown gate activation {self.activation!r}; known: {', '.join(ops.GATE_ACTIVATIONS)}")
        self.float_output = bool(p.get("float_output", False))
        self.w_gate_up = self.w_down = None

    def tensor_specs(self) -> List[TensorSpec]:
        specs = [TensorSpec(self.names["gate"], (self.intermediate, self.hidden), MATRIX),
                 TensorSpec(self.names["up"], (self.intermediate, self.hidden), MATRIX),
                 TensorSpec(self.names["down"], (self.hidden, self.intermediate), MATRIX)]
        if self.bias_names:
            small = ("normal", 0.0, 0.02)
            specs += [TensorSpec(self.bias_names["gate"], (self.intermediate,), VECTOR, init=small),
                      TensorSpec(self.bias_names["up"], (self.intermediate,), VECTOR, init=small),
                      TensorSpec(self.bias_names["down"], (self.hidden,), VECTOR, init=small)]
        return specs

    fused_io = True
    prepares_next = True

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        # One product for gate and up: 8 gate rows, their 8 up rows, and so on (a pure re-layout), which
        # lets the activation be applied where the product is finished.  An intermediate size that is no
        # multiple of 8 is filled up with zero rows; they give silu(0) * 0 = 0 and meet zero columns of
        # the down projection, so the result is unchanged.
        gate, up, down = (tensors.pop(self.names[k]) for k in ("gate", "up", "down"))
        if self.bias_names:
            # gate rows, then up rows: the biases are added behind the product, which therefore folds nothing in
            self.w_gate_up = torch.cat([gate, up], dim=0).contiguous()
            self.w_down = down.contiguous()
            self.bias_in = torch.cat([tensors.pop(self.bias_names["gate"]), tensors.pop(self.bias_names["up"])]).contiguous()
            self.bias_out = tensors.pop(self.bias_names["down"]).contiguous()
            return
        pad = -self.intermediate % 8
        if pad:
            gate = torch.nn.functional.pad(gate, (0, 0, 0, pad))
            up = torch.nn.functional.pad(up, (0, 0, 0, pad))
            down = torch.nn.functional.pad(down, (0, pad))
        self.w_gate_up = ops.interleave_gate_up(gate, up).contiguous()
        self.w_down = down.contiguous()

    def streamed_weights(self) -> List[torch.Tensor]:
        return [self.w_gate_up, self.w_down]

    def forward(self, y, step: StepContext, residual: Optional[torch.Tensor] = None, next_norm=None):
        """``y`` may be a norm still to be done; with ``residual`` the result may be added there (None returned),
        and with ``next_norm`` the norm that follows may come back prepared (see ``ops.linear``)."""
        if self.bias_in is not None:
            both = ops.linear(ops.materialize(y), self.w_gate_up, out_dtype=torch.float32)
            if both.dim() == 3:
                both = both.sum(dim=0)
            activated = ops.bias_glu(both, self.bias_in, step.dtype, self.activation)
            out = ops.linear(activated, self.w_down, out_dtype=torch.float32)
            if out.dim() == 3:
                out = out.sum(dim=0)
            return ops.add_bias(out, self.bias_out)
        activated = ops.linear(y, self.w_gate_up, gated=True, activation=self.activation)
        return ops.linear(activated, self.w_down, residual=residual, next_norm=next_norm,
                          out_dtype=torch.float32 if self.float_output else None)


@FEED_FORWARDS.register("relu2")
class ReluSquaredMlp(Part):
    """down(relu(up y)^2), no bias.  Parameters: ``hidden``, ``intermediate`` and tensor names ``up``, ``down``."""

    graph_safe = True

    def __init__(self, spec: PartSpec, **_):
        p = spec.params
        self.hidden, self.intermediate = int(p["hidden"]), int(p["intermediate"])
        self.names = {k: p[k] for k in ("up", "down")}
        self.w_up = self.w_down = None

    def tensor_specs(self) -> List[TensorSpec]:
        return [TensorSpec(self.names["up"], (self.intermediate, self.hidden), MATRIX),
                TensorSpec(self.names["down"], (self.hidden, self.intermediate), MATRIX)]

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.w_up = tensors.pop(self.names["up"]).contiguous()
        self.w_down = tensors.pop(self.names["down"]).contiguous()

    def streamed_weights(self) -> List[torch.Tensor]:
        return [self.w_up, self.w_down]

    def forward(self, y: torch.Tensor, step: StepContext) -> torch.Tensor:
        return ops.linear(ops.relu_squared(ops.linear(y, self.w_up)), self.w_down, out_dtype=torch.float32)


@FEED_FORWARDS.register("routed_glu")
class RoutedGluMlp(Part):
    """A mixture of small gated feed-forwards of which a router picks ``top`` for every row.

    Router logits z = W_router y in float; scores s = softmax(z) over all router outputs; a row's choice scores are
    s + ``correction``; the outputs form ``group_count`` equal groups of neighbours, a group's score is its best
    choice score, and only outputs of the ``group_keep`` best groups can be chosen; the ``top`` best choice scores
    win and weigh in with s over the winners' sum.  The first ``experts`` outputs are experts
    down_e(act(gate_e y) * (up_e y)); the ``identity`` outputs behind them hand y itself on.  A ``shared`` feed-forward
    (a part spec, optional) runs for every row and is added.  The result is float32.

    Parameters: ``hidden``, ``experts``, ``identity``, ``top``, ``group_count``, ``group_keep``, ``intermediate``,
    ``activation`` (a key of ``ops.GATE_ACTIVATIONS``), tensor names ``router`` ``[experts + identity, hidden]``,
    ``correction`` ``[experts + identity]`` (None: no correction) and ``expert`` (a pattern with ``{e}``:
    ``expert.format(e=3) + ".gate"`` and so on), ``shared``.

    Optional, for routers of another rule: ``score`` ("softmax", or "sigmoid": every output's own sigmoid), ``group_best``
    (a group's score is the sum of its so many best choice scores, 1 by default), ``renormalize`` (False: the weights
    are the winners' scores themselves), ``weight_scale`` (multiplies the weights), and ``activation`` "clamped_swish"
    with ``limit`` (``ops.EXPERT_ACTIVATIONS``): g = min(gate, limit), u = clamp(up, -limit, limit),
    g sigmoid(1.702 g) (u + 1).

    The choice lives on the device only: which rows go to which expert is worked out there, and the grids do not
    depend on it, so a recorded step replays with other choices.
    """

    graph_safe = True

    def __init__(self, spec: PartSpec, **context):
        p = spec.params
        self.hidden, self.intermediate = int(p["hidden"]), int(p["intermediate"])
        self.experts, self.identity, self.top = int(p["experts"]), int(p.get("identity") or 0), int(p["top"])
        self.group_count, self.group_keep = int(p.get("group_count") or 1), int(p.get("group_keep") or 1)
        self.activation = str(p.get("activation") or "silu")
        self.total = self.experts + self.identity
        if self.top > self.total or self.total % self.group_count or not 1 <= self.group_keep <= self.group_count:
            raise ValueError(f"a router of {self.total} outputs cannot choose {self.top} from {self.group_keep} of "
                             f"{self.group_count} equal groups")
        if self.activation not in ops.EXPERT_ACTIVATIONS:
            raise ValueError(f"unknown expert activation {self.activation!r}; known: {', '.join(ops.EXPERT_ACTIVATIONS)}")
        self.limit = float(p["limit"]) if p.get("limit") is not None else None
        if self.activation == "clamped_swish" and not (self.limit and self.limit > 0.0):
            raise ValueError(f"the clamped activation needs a positive limit, found {self.limit!r}")
        self.rule = ops.RouterRule(str(p.get("score") or "softmax"), int(p.get("group_best") or 1),
                                   bool(p.get("renormalize", True)), float(p.get("weight_scale", 1.0)))
        self.router_name, self.correction_name, self.expert_name = p["router"], p.get("correction"), p["expert"]
        self.shared = FEED_FORWARDS.build(p["shared"], **context) if p.get("shared") is not None else None
        self.w_router = self.correction = self.w_gate_up = self.w_down = self.w_gate_up_all = self.w_down_all = None
        self.always = 0

    def tensor_specs(self) -> List[TensorSpec]:
        specs = [TensorSpec(self.router_name, (self.total, self.hidden), MATRIX)]
        if self.correction_name:
            specs.append(TensorSpec(self.correction_name, (self.total,), VECTOR))
        for e in range(self.experts):
            name = self.expert_name.format(e=e)
            specs += [TensorSpec(name + ".gate", (self.intermediate, self.hidden), MATRIX),
                      TensorSpec(name + ".up", (self.intermediate, self.hidden), MATRIX),
                      TensorSpec(name + ".down", (self.hidden, self.intermediate), MATRIX)]
        return specs + (self.shared.tensor_specs() if self.shared is not None else [])

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.w_router = tensors.pop(self.router_name).contiguous()
        self.correction = tensors.pop(self.correction_name).contiguous() if self.correction_name else None
        names = [self.expert_name.format(e=e) for e in range(self.experts)]
        # all experts side by side: [experts, 2, ff, hidden] (gate rows, then up rows) and [experts, hidden, ff]
        gate_up = torch.stack([torch.stack([tensors.pop(n + ".gate"), tensors.pop(n + ".up")]) for n in names])
        down = torch.stack([tensors.pop(n + ".down") for n in names])
        # A shared expert of the experts' kind rides along in the experts' launches of short steps: cut into pieces of
        # the experts' size (the last filled up with zero rows, which add nothing), they stand behind the experts as
        # experts that every row takes with weight 1.
        self.always = 0
        if isinstance(self.shared, SwiGluMlp) and self.shared.activation == self.activation:
            shared = {k: tensors[self.shared.names[k]] for k in ("gate", "up", "down")}
            pieces = -(-self.shared.intermediate // self.intermediate)
            pad = pieces * self.intermediate - self.shared.intermediate
            rows = [torch.nn.functional.pad(shared[k], (0, 0, 0, pad)).view(pieces, self.intermediate, self.hidden) for k in ("gate", "up")]
            cols = torch.nn.functional.pad(shared["down"], (0, pad)).view(self.hidden, pieces, self.intermediate).permute(1, 0, 2)
            gate_up = torch.cat([gate_up, torch.stack(rows, dim=1).to(gate_up.dtype)])
            down = torch.cat([down, cols.to(down.dtype)])
            self.always = pieces
        self.w_gate_up_all, self.w_down_all = gate_up.contiguous(), down.contiguous()
        self.w_gate_up, self.w_down = self.w_gate_up_all[:self.experts], self.w_down_all[:self.experts]
        if self.shared is not None:
            self.shared.bind(tensors)

    def streamed_weights(self) -> List[torch.Tensor]:
        return self.shared.streamed_weights() if self.shared is not None else []

    def forward(self, y: torch.Tensor, step: StepContext) -> torch.Tensor:
        y = ops.materialize(y)
        logits = ops.linear(y, self.w_router, out_dtype=torch.float32)
        if self.always and y.shape[0] <= ops.ROUTE_PLAN_ROWS:
            return ops.routed_feed_forward(y, logits, self.correction, self.top, self.group_count, self.group_keep,
                                           self.w_gate_up_all, self.w_down_all, self.activation, always=self.always,
                                           rule=self.rule, limit=self.limit)
        extra = None
        if self.shared is not None:
            extra = self.shared.forward(y, step)
            if extra.dim() == 3:
                extra = extra.sum(dim=0)
            if extra.dtype != torch.float32:
                extra = extra.float()
        return ops.routed_feed_forward(y, logits, self.correction, self.top, self.group_count, self.group_keep,
                                       self.w_gate_up, self.w_down, self.activation, extra=extra, rule=self.rule,
                                       limit=self.limit)
