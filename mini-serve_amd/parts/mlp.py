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
result of the first product, rounded once."""

from __future__ import annotations

import torch

from ..config.spec import PartSpec
from .base import FeedForward, TensorSpec
from .registry import register

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
        if self.activation not in rt.ops.ACTIVATIONS:
            raise NotImplementedError(f"activation {self.activation!r} is not supported, expected one of {sorted(rt.ops.ACTIVATIONS)}")
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
