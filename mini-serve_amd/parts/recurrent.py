"""Mixers that keep a matrix state of fixed size per request and head instead of keys and values per token,
and the mixer that runs two mixers side by side. None has a counterpart in the reference.

Both recurrent mixers are ``S_t = a_t S_(t-1) + b_t k_t v_t^T``, ``o_t = S_t^T q_t`` per head (``S: [dim, value_dim]``),
computed in float32 by one kernel family (``ops.gated_recurrence``) whose state lives in the cache manager's state
slots; they differ in where ``a`` and ``b`` come from and in what happens to ``o``:

* ``decay_linear_attention``: ``q, k, v = silu(W h)``; ``a`` is a constant per head (``decay``), ``b = 1``; the
  concatenated heads are RMS-normed together (weight ``norm``), multiplied by ``sigmoid(W_g h)`` and projected.
* ``mlstm``: ``q = W_q h / sqrt(dim)``, ``k``, ``v`` plain; a log input gate and a log forget gate per head, each
  bounded by a soft cap (``cap tanh(z / cap)``, the forget gate then through a log-sigmoid), a running maximum that
  keeps the exponentials in range, and a normaliser vector ``n``; each head's output is divided by its root mean
  square, the heads are concatenated, multiplied by a weight and by ``sigmoid(W_g h)`` and projected.

All projections of a mixer are one matrix product over row-concatenated weights whose float32 result the recurrence
kernel reads in place (activation, scale and gates are applied on the way in).
"""

from __future__ import annotations

import torch

from ..config.spec import PartSpec
from .base import KVNeed, Mixer, StateNeed, StateTensor, TensorSpec
from .registry import part_class, register


def _named(spec: PartSpec, default: dict) -> dict[str, str]:
    p = spec.get("prefix", "")
    given = spec.get("names") or {}
    return {k: p + given.get(k, d) for k, d in default.items()}


class _RecurrentMixer(Mixer):
    """What the two recurrent mixers share: sizes, the fused projection and the gated output norm."""

    NAMES: dict = {}

    def __init__(self, spec: PartSpec, rt):
        super().__init__(spec, rt)
        self.hidden = int(spec["hidden_size"])
        self.heads = int(spec["num_heads"])
        self.dim = int(spec["head_dim"])
        self.value_dim = int(spec.get("value_dim") or self.dim)
        self.eps = float(spec["eps"])
        self.names = _named(spec, self.NAMES)
        if min(self.heads, self.dim, self.value_dim) < 1 or max(self.dim, self.value_dim) > 256:
            raise ValueError(f"{self.heads} heads of sizes {self.dim} / {self.value_dim}: the recurrence kernels take sizes 1..256")
        self.proj = self.o = self.norm = None
        self.columns: dict[str, int] = {}

    def _fuse(self, tensors, order) -> None:
        parts = [tensors[self.names[k]] for k in order]
        if len({t.dtype for t in parts}) != 1:
            raise ValueError(f"{self.names[order[0]]} and its neighbours are stored in different dtypes")
        at = 0
        for k, t in zip(order, parts):
            self.columns[k] = at
            at += t.shape[0]
        self.proj = torch.cat(parts, dim=0).contiguous()
        self.o = tensors[self.names["o"]]
        self.norm = tensors[self.names["norm"]]

    def _finish(self, o, x32, group, residual):
        ops = self.rt.ops
        n = self.heads * self.value_dim
        gate = x32[:, self.columns["g"] : self.columns["g"] + n]
        y = ops.group_rmsnorm_gate(o, group, self.norm, gate, self.eps, self.rt.dtype)
        return ops.linear(y, self.o, accumulate_into=residual, defer=True)

    def parameters_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in (self.proj, self.o, self.norm))

    def flops(self, rows) -> int:
        tokens = sum(n for n, _ in rows)
        qk, vo = self.heads * self.dim, self.heads * self.value_dim
        linear = 2 * tokens * self.hidden * (self.proj.shape[0] if self.proj is not None else 2 * qk + 2 * vo) + 2 * tokens * vo * self.hidden
        return linear + 4 * tokens * self.heads * self.dim * self.value_dim  # the state's update and its product with q


@register("mixer", "decay_linear_attention")
class DecayLinearAttention(_RecurrentMixer):
    NAMES = {"q": "q", "k": "k", "v": "v", "g": "g", "o": "o", "norm": "norm"}

    def __init__(self, spec: PartSpec, rt):
        super().__init__(spec, rt)
        decay = [float(d) for d in spec["decay"]]
        if len(decay) != self.heads:
            raise ValueError(f"{len(decay)} decays for {self.heads} heads")
        if not all(0.0 <= d <= 1.0 for d in decay):
            raise ValueError(f"decays must lie in [0, 1], got {decay}")
        self.decay = torch.tensor(decay, dtype=torch.float32, device=rt.device) if rt is not None else None
        self.chunks = min(decay) > 1e-30  # the chunked kernels work with the decays' logarithms

    @classmethod
    def tensors(cls, spec: PartSpec) -> dict[str, TensorSpec]:
        n = _named(spec, cls.NAMES)
        w, h, d = int(spec["hidden_size"]), int(spec["num_heads"]), int(spec["head_dim"])
        e = int(spec.get("value_dim") or d)
        return {n["q"]: TensorSpec((h * d, w)), n["k"]: TensorSpec((h * d, w)), n["v"]: TensorSpec((h * e, w)),
                n["g"]: TensorSpec((h * e, w)), n["o"]: TensorSpec((w, h * e)), n["norm"]: TensorSpec((h * e,), init="ones")}

    def bind(self, tensors) -> None:
        self._fuse(tensors, ("q", "k", "v", "g"))

    def state_need(self) -> StateNeed:
        return StateNeed((StateTensor("S", (self.heads, self.dim, self.value_dim), "float32"),))

    def forward(self, x, batch, cache, state, residual):
        ops = self.rt.ops
        x32 = ops.linear(x, self.proj, out_dtype=torch.float32)
        o = ops.gated_recurrence(x32, self.columns, self.heads, self.dim, self.value_dim, batch, state, mode="decay",
                                 activation="silu", decay=self.decay, chunks=self.chunks)
        return self._finish(o, x32, self.heads * self.value_dim, residual)


@register("mixer", "mlstm")
class MLSTM(_RecurrentMixer):
    NAMES = {"q": "q", "k": "k", "v": "v", "g": "g", "i": "i", "f": "f", "i_bias": "i.b", "f_bias": "f.b", "o": "o",
             "norm": "norm"}

    def __init__(self, spec: PartSpec, rt):
        super().__init__(spec, rt)
        self.cap = float(spec["gate_cap"])
        if not self.cap > 0:
            raise ValueError(f"gate_cap must be positive, not {self.cap}")
        self.i_bias = self.f_bias = None

    @classmethod
    def tensors(cls, spec: PartSpec) -> dict[str, TensorSpec]:
        n = _named(spec, cls.NAMES)
        w, h, d = int(spec["hidden_size"]), int(spec["num_heads"]), int(spec["head_dim"])
        e = int(spec.get("value_dim") or d)
        return {n["q"]: TensorSpec((h * d, w)), n["k"]: TensorSpec((h * d, w)), n["v"]: TensorSpec((h * e, w)),
                n["g"]: TensorSpec((h * e, w)), n["i"]: TensorSpec((h, w)), n["f"]: TensorSpec((h, w)),
                n["i_bias"]: TensorSpec((h,), init="uniform"), n["f_bias"]: TensorSpec((h,), init="uniform"),
                n["o"]: TensorSpec((w, h * e)), n["norm"]: TensorSpec((h * e,), init="ones")}

    def bind(self, tensors) -> None:
        self._fuse(tensors, ("q", "k", "v", "g", "i", "f"))
        self.i_bias, self.f_bias = tensors[self.names["i_bias"]], tensors[self.names["f_bias"]]

    def state_need(self) -> StateNeed:
        return StateNeed((StateTensor("S", (self.heads, self.dim, self.value_dim), "float32"),
                          StateTensor("n", (self.heads, self.dim), "float32"), StateTensor("m", (self.heads,), "float32")))

    def forward(self, x, batch, cache, state, residual):
        ops = self.rt.ops
        x32 = ops.linear(x, self.proj, out_dtype=torch.float32)
        o = ops.gated_recurrence(x32, self.columns, self.heads, self.dim, self.value_dim, batch, state, mode="exp_gates",
                                 q_scale=self.dim ** -0.5, cap=self.cap, i_bias=self.i_bias, f_bias=self.f_bias)
        return self._finish(o, x32, self.value_dim, residual)

    def parameters_bytes(self) -> int:
        return super().parameters_bytes() + sum(t.numel() * t.element_size() for t in (self.i_bias, self.f_bias))


@register("mixer", "normed_pair")
class NormedPair(Mixer):
    """Two mixers side by side on the same input: ``coef * (rmsnorm(left(h)) w_left + rmsnorm(right(h)) w_right)`` with
    the norms over the model width. The sub-mixers are any registered mixers (``left`` / ``right``: their ``PartSpec``);
    at most one of them may keep keys and values per token, both may keep state."""

    SIDES = ("left", "right")

    def __init__(self, spec: PartSpec, rt):
        super().__init__(spec, rt)
        self.hidden = int(spec["hidden_size"])
        self.eps = float(spec["eps"])
        self.coef = float(spec.get("coef", 0.5))
        self.subs = [part_class("mixer", spec[s])(spec[s], rt) for s in self.SIDES]
        self.out_names = [spec.get(f"{s}_norm", f"{s}.out") for s in self.SIDES]
        self.out_weights = None
        if sum(m.kv_need() is not None for m in self.subs) > 1:
            raise NotImplementedError("only one of two mixers side by side may keep keys and values per token")

    @classmethod
    def tensors(cls, spec: PartSpec) -> dict[str, TensorSpec]:
        out = {}
        for s in cls.SIDES:
            out.update(part_class("mixer", spec[s]).tensors(spec[s]))
            out[spec.get(f"{s}_norm", f"{s}.out")] = TensorSpec((int(spec["hidden_size"]),), init="ones")
        return out

    @classmethod
    def aliases(cls, spec: PartSpec) -> dict[str, str]:
        out = {}
        for s in cls.SIDES:
            out.update(part_class("mixer", spec[s]).aliases(spec[s]))
        return out

    def bind(self, tensors) -> None:
        for m in self.subs:
            names = list(type(m).tensors(m.spec)) + list(type(m).aliases(m.spec))
            m.bind({n: tensors[n] for n in names})
        self.out_weights = [tensors[n] for n in self.out_names]

    def kv_need(self) -> KVNeed | None:
        return next((n for n in (m.kv_need() for m in self.subs) if n is not None), None)

    def state_need(self) -> StateNeed | None:
        tensors = []
        for side, m in zip(self.SIDES, self.subs):
            need = m.state_need()
            if need is not None:
                tensors += [StateTensor(f"{side}.{t.name}", t.shape, t.dtype) for t in need.tensors]
        return StateNeed(tuple(tensors)) if tensors else None

    def forward(self, x, batch, cache, state, residual):
        ops = self.rt.ops
        streams = []
        for side, m in zip(self.SIDES, self.subs):
            # each mixer adds into a stream of its own, which starts at zero
            own = torch.zeros_like(residual)
            sub_state = {k[len(side) + 1:]: v for k, v in (state or {}).items() if k.startswith(side + ".")}
            pending = m.forward(x, batch, cache if m.kv_need() is not None else None, sub_state or None, own)
            ops.add_pending(own, pending)
            streams.append(own)
        ops.normed_mean_add(residual, streams, self.out_weights, self.eps, self.coef)
        return None

    def parameters_bytes(self) -> int:
        return sum(m.parameters_bytes() for m in self.subs) + sum(w.numel() * w.element_size() for w in self.out_weights)

    def flops(self, rows) -> int:
        return sum(m.flops(rows) for m in self.subs)
