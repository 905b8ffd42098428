"""Gated feed-forward: ``down(act(gate(x)) * up(x))`` without biases
(miniserve/model/qwen3.py:128-131). Gate and up are one matrix product over one weight that holds
both (the reference concatenates them, miniserve/model/fused.py:41,195; here their rows alternate in
runs of 16 where the width allows, so that a matrix kernel's lane holds gate and up of the same output
and can finish the activation itself); the activation product is evaluated in float32 and rounded
once; the down projection adds into the residual stream in its epilogue.

``names`` (optional) maps ``gate`` / ``up`` / ``down`` to the tensors' names behind the prefix (default
``<x>_proj.weight``); ``limit`` belongs to the activations that bound their inputs (``swiglu_clamped``).
``none`` is the feed-forward of a layer that has none. ``dense_mlp`` (no counterpart in the reference) is
``down(act(up(x)))`` without a gate: tensors ``up`` / ``down`` (``names``), the activation in float32 on the float32
result of the first product, rounded once.

``moe_mlp`` (no counterpart in the reference) is a mixture of ``num_experts`` gated feed-forwards of which every token
runs ``top``: router logits ``router x (+ router_bias)`` in float32, the ``top`` largest chosen (ties: the lower index),
weights the softmax over the chosen logits alone, the output the weighted sum of the chosen experts' outputs. ``shared``
(optional) is the ``PartSpec`` of any registered feed-forward that runs for every token and is added. ``names`` maps
``router``, ``router_bias``, ``expert`` (a pattern with ``{}`` for the expert's number, behind the prefix) and ``gate`` /
``up`` / ``down`` (behind the expert's own prefix).

Further parameters of ``moe_mlp`` (the defaults give the mixture above): ``gated=False`` (an expert is
``down(act(up x))``, no ``gate`` tensors; ``activation`` may then be any that has an ungated form, ``relu_squared``
among them); ``scoring="softmax"`` (the router's softmax runs over all its outputs; the choice goes by the softmax
value plus ``router_bias``, a correction that only the choice sees; the weights are the chosen outputs' softmax values
as they stand, not renormalised); ``groups`` / ``keep_groups`` (with that scoring: the router's outputs form ``groups``
equal groups of neighbours, a group's score is the largest choice score in it, and only outputs of the ``keep_groups``
best groups can be chosen); ``identity`` (the router has that many outputs more than there are experts with weights; a
token that chooses one of them gets its own input back, times the weight)."""

from __future__ import annotations

import torch

from ..config.spec import PartSpec
from .base import FeedForward, TensorSpec
from .registry import part_class, register

def _names(spec: PartSpec) -> dict[str, str]:
    p = spec.get("prefix", "")
    given = spec.get("names") or {}
    return {k: p + given.get(k, f"{k}_proj.weight") for k in ("gate", "up", "down")}


@register("feed_forward", "none")
class NoFeedForward(FeedForward):
    """A layer without a feed-forward: nothing is added."""

    def forward(self, x, residual):
        return None


@register("feed_forward", "gated_mlp")
class GatedMLP(FeedForward):
    def __init__(self, spec: PartSpec, rt):
        super().__init__(spec, rt)
        self.prefix = spec.get("prefix", "")
        self.hidden = int(spec["hidden_size"])
        self.inter = int(spec["intermediate_size"])
        self.activation = spec.get("activation", "silu")
        self.limit = float(spec["limit"]) if spec.get("limit") is not None else None
        if self.activation not in rt.ops.ACTIVATIONS or self.activation in rt.ops.ACTIVATIONS_UNGATED_ONLY:
            raise NotImplementedError(f"activation {self.activation!r} is not supported, expected one of "
                                      f"{sorted(set(rt.ops.ACTIVATIONS) - set(rt.ops.ACTIVATIONS_UNGATED_ONLY))}")
        if self.activation in rt.ops.ACTIVATIONS_WITH_LIMIT and not (self.limit is not None and self.limit > 0):
            raise ValueError(f"activation {self.activation!r} needs a positive limit, got {self.limit!r}")
        self.names = _names(spec)
        self.gate_up = self.down = None
        self.block = 0  # rows per run of gate / up rows in gate_up (0: all gates, then all ups)

    @classmethod
    def tensors(cls, spec: PartSpec) -> dict[str, TensorSpec]:
        h, i = int(spec["hidden_size"]), int(spec["intermediate_size"])
        n = _names(spec)
        return {n["gate"]: TensorSpec((i, h)), n["up"]: TensorSpec((i, h)), n["down"]: TensorSpec((h, i))}

    def bind(self, tensors) -> None:
        g, u = tensors[self.names["gate"]], tensors[self.names["up"]]
        if g.dtype != u.dtype:
            raise ValueError(f"{self.prefix}gate/up projections are stored in different dtypes")
        ops = self.rt.ops
        self.block = ops.GATE_BLOCK if self.inter % ops.GATE_BLOCK == 0 else 0
        self.gate_up = ops.interleave_gate_up(g, u) if self.block else torch.cat((g, u), dim=0).contiguous()
        self.down = tensors[self.names["down"]]

    def forward(self, x, residual):
        ops = self.rt.ops
        m = ops.gated_linear(x, self.gate_up, self.activation, out_dtype=self.rt.dtype, block=self.block, limit=self.limit)
        return ops.linear(m, self.down, accumulate_into=residual, defer=True)

    def parameters_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in (self.gate_up, self.down))

    def flops(self, rows) -> int:
        return 2 * sum(n for n, _ in rows) * 3 * self.hidden * self.inter


@register("feed_forward", "dense_mlp")
class DenseMLP(FeedForward):
    def __init__(self, spec: PartSpec, rt):
        super().__init__(spec, rt)
        self.prefix = spec.get("prefix", "")
        self.hidden = int(spec["hidden_size"])
        self.inter = int(spec["intermediate_size"])
        self.activation = spec.get("activation", "gelu_tanh")
        if rt is not None and (self.activation not in rt.ops.ACTIVATIONS or self.activation in rt.ops.ACTIVATIONS_WITH_LIMIT):
            raise NotImplementedError(f"activation {self.activation!r} has no ungated form")
        given = spec.get("names") or {}
        self.names = {k: self.prefix + given.get(k, f"{k}_proj.weight") for k in ("up", "down")}
        self.up = self.down = None

    @classmethod
    def tensors(cls, spec: PartSpec) -> dict[str, TensorSpec]:
        h, i, p = int(spec["hidden_size"]), int(spec["intermediate_size"]), spec.get("prefix", "")
        given = spec.get("names") or {}
        return {p + given.get("up", "up_proj.weight"): TensorSpec((i, h)), p + given.get("down", "down_proj.weight"): TensorSpec((h, i))}

    def bind(self, tensors) -> None:
        self.up, self.down = tensors[self.names["up"]], tensors[self.names["down"]]

    def forward(self, x, residual):
        ops = self.rt.ops
        m = ops.activate(ops.linear(x, self.up, out_dtype=torch.float32), self.activation, self.rt.dtype)
        return ops.linear(m, self.down, accumulate_into=residual, defer=True)

    def parameters_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in (self.up, self.down))

    def flops(self, rows) -> int:
        return 2 * sum(n for n, _ in rows) * 2 * self.hidden * self.inter


def _moe_names(spec: PartSpec) -> dict[str, str]:
    given = spec.get("names") or {}
    default = {"router": "router.weight", "router_bias": "router.bias", "expert": "experts.{}.", "gate": "gate_proj.weight",
               "up": "up_proj.weight", "down": "down_proj.weight"}
    return {k: given.get(k, d) for k, d in default.items()}


@register("feed_forward", "moe_mlp")
class MixtureMLP(FeedForward):
    def __init__(self, spec: PartSpec, rt):
        super().__init__(spec, rt)
        self.prefix = spec.get("prefix", "")
        self.hidden = int(spec["hidden_size"])
        self.inter = int(spec["intermediate_size"])
        self.num_experts = int(spec["num_experts"])
        self.top = int(spec["top"])
        self.activation = spec.get("activation", "silu")
        self.router_bias = bool(spec.get("router_bias", False))
        self.gated = bool(spec.get("gated", True))
        self.scoring = spec.get("scoring", "chosen_softmax")
        self.groups = int(spec.get("groups") or 1)
        self.keep_groups = int(spec.get("keep_groups") or self.groups)
        self.identity = int(spec.get("identity") or 0)
        self.outputs = self.num_experts + self.identity  # what the router tells apart
        if self.scoring not in ("chosen_softmax", "softmax"):
            raise ValueError(f"router scoring {self.scoring!r}: 'chosen_softmax' or 'softmax'")
        if self.identity < 0 or self.num_experts < 1:
            raise ValueError(f"{self.num_experts} experts and {self.identity} identity experts")
        if self.groups != 1 and self.scoring != "softmax":
            raise NotImplementedError("groups of experts go with scoring='softmax'")
        if self.groups < 1 or self.outputs % self.groups or not 1 <= self.keep_groups <= self.groups:
            raise ValueError(f"{self.outputs} router outputs in {self.groups} groups of which {self.keep_groups} are kept")
        if not 1 <= self.top <= (self.outputs // self.groups) * self.keep_groups:
            raise ValueError(f"top {self.top} of {self.outputs} router outputs in {self.groups} groups of which {self.keep_groups} are kept")
        if rt is not None:
            ops = rt.ops
            if self.activation not in ops.ACTIVATIONS or self.activation in ops.ACTIVATIONS_WITH_LIMIT or (
                    self.gated and self.activation in ops.ACTIVATIONS_UNGATED_ONLY):
                raise NotImplementedError(f"activation {self.activation!r} is not of the form "
                                          f"{'act(gate) * up' if self.gated else 'act(up)'}")
            if self.outputs > ops.MOE_MAX_EXPERTS or self.top > ops.MOE_MAX_TOP:
                raise ValueError(f"{self.outputs} experts / top {self.top}: the kernels take up to {ops.MOE_MAX_EXPERTS} "
                                 f"experts and {ops.MOE_MAX_TOP} choices")
        self.names = _moe_names(spec)
        sh = spec.get("shared")
        self.shared = part_class("feed_forward", sh)(sh, rt) if sh is not None else None
        self.router = self.bias = self.gate = self.up = self.down = None

    @classmethod
    def _expert_names(cls, spec: PartSpec, j: int) -> dict[str, str]:
        n, p = _moe_names(spec), spec.get("prefix", "")
        return {k: p + n["expert"].format(j) + n[k] for k in ("gate", "up", "down")}

    @classmethod
    def tensors(cls, spec: PartSpec) -> dict[str, TensorSpec]:
        n, p = _moe_names(spec), spec.get("prefix", "")
        h, i, e = int(spec["hidden_size"]), int(spec["intermediate_size"]), int(spec["num_experts"])
        outputs = e + int(spec.get("identity") or 0)
        out = {p + n["router"]: TensorSpec((outputs, h))}
        if spec.get("router_bias", False):
            out[p + n["router_bias"]] = TensorSpec((outputs,), init="uniform")
        for j in range(e):
            en = cls._expert_names(spec, j)
            out[en["up"]], out[en["down"]] = TensorSpec((i, h)), TensorSpec((h, i))
            if spec.get("gated", True):
                out[en["gate"]] = TensorSpec((i, h))
        sh = spec.get("shared")
        if sh is not None:
            out.update(part_class("feed_forward", sh).tensors(sh))
        return out

    def bind(self, tensors) -> None:
        n, p = self.names, self.prefix
        self.router = tensors[p + n["router"]]
        self.bias = tensors[p + n["router_bias"]] if self.router_bias else None
        kinds = ("gate", "up", "down") if self.gated else ("up", "down")
        per = [{k: v for k, v in self._expert_names(self.spec, j).items() if k in kinds} for j in range(self.num_experts)]
        if len({tensors[en[k]].dtype for en in per for k in en}) != 1:
            raise ValueError(f"{p}: the experts' projections are stored in different dtypes")
        # one tensor per projection, [experts, rows, columns]: a kernel finds an expert's weights by its number
        stacked = {k: torch.stack([tensors[en[k]] for en in per]).contiguous() for k in kinds}
        self.gate, self.up, self.down = stacked.get("gate"), stacked["up"], stacked["down"]
        if self.shared is not None:
            self.shared.bind(tensors)

    def forward(self, x, residual):
        ops = self.rt.ops
        pending = self.shared.forward(x, residual) if self.shared is not None else None
        logits = ops.linear(x, self.router, out_dtype=torch.float32, defer=True)  # few rows: partial sums, added by the routing
        ids, weights = ops.moe_route(logits, self.bias, self.top, self.scoring, self.groups, self.keep_groups)
        xe = ops.cast(x, self.up.dtype)  # experts stored in 32-bit compute in 32-bit
        ops.moe_experts(xe, ids, weights, self.gate, self.up, self.down, self.activation, residual)
        return pending

    def parameters_bytes(self) -> int:
        """What one token reads: the router, its ``top`` experts and the shared expert (a step of several tokens reads up
        to ``top`` experts more per token)."""
        per_expert = sum(t[0].numel() * t.element_size() for t in (self.gate, self.up, self.down) if t is not None)
        own = self.router.numel() * self.router.element_size() + self.top * per_expert
        return own + (self.shared.parameters_bytes() if self.shared is not None else 0)

    def step_read_bytes(self, tokens: int) -> int:
        """The router, the shared expert and the experts that ``tokens`` tokens are expected to choose between them when
        every choice of ``top`` is as likely as any other: ``E (1 - (1 - top / E) ** tokens)`` experts."""
        per_expert = sum(t[0].numel() * t.element_size() for t in (self.gate, self.up, self.down) if t is not None)
        distinct = self.num_experts * (1.0 - (1.0 - self.top / self.outputs) ** max(1, tokens))
        own = self.router.numel() * self.router.element_size() + int(round(distinct * per_expert))
        return own + (self.shared.parameters_bytes() if self.shared is not None else 0)

    def flops(self, rows) -> int:
        tokens = sum(n for n, _ in rows)
        products = 3 if self.gated else 2
        chosen = self.top * self.num_experts / self.outputs  # identity experts multiply nothing
        own = 2 * tokens * self.hidden * self.outputs + int(2 * tokens * chosen * products * self.hidden * self.inter)
        return own + (self.shared.flops(rows) if self.shared is not None else 0)
