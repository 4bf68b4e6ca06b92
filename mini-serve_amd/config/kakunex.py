"""Typed configuration of the Kakunex decoder, read from its own ``config.json`` keys. The reference has no
such architecture.

``config.json``: ``architecture`` (the name), ``vocab``, ``width``, ``norm.eps``, ``logit_scale`` and ``layers``, a list
in which every entry names its mixer (``type``), the mixer's sizes and constants (``mixer``) and its feed-forward
(``mlp``, or null for none). Layer ``i``'s tensors start with ``l<i>.``.

A layer is ``x += mixer(h) + ff(h)`` with ``h = layer_norm(x)`` (weight ``norm1``, bias ``norm1.b``). Mixers:

* ``mlstm`` (``heads``, ``dim``, ``vdim``, ``gate_cap``; tensors ``mix.q k v g o norm i i.b f f.b``): a matrix memory
  per head with capped exponential gates.
* ``parallel`` (``left``, ``right``): half the sum of two mixers on the same input, each RMS-normed over the width
  (weights ``mix.left.out`` / ``mix.right.out``). Left (``heads``, ``kv_heads``, ``dim``, ``vdim``, ``scale``, ``rot``,
  ``mask``; tensors ``mix.left.q k v o q.norm k.norm``): grouped-query softmax attention with an RMS norm over the
  whole query and the whole key projection, rotation of adjacent pairs of the first ``rot.dims`` elements of every
  head by frequencies ``rot.base ** (-2i / rot.dims)`` (slowed down in wavelength bands by ``rot.scaling``: ``factor``,
  ``low``, ``high``, ``original``), and a window of ``mask.size`` keys that also keeps the sequence's first
  ``mask.keep_first``. Right (``heads``, ``dim``, ``vdim``, ``decay``; tensors ``mix.right.q k v g o norm``): linear
  attention with a constant decay per head.

Feed-forward (``kind: dense``, ``ff``, ``limit``; tensors ``mlp.gate up down``): gated, with gate and up bounded by
``limit``. The final layer norm is ``final.norm`` / ``final.norm.b``; the head is the embedding table ``embed``,
its logits multiplied by ``logit_scale``.
"""

from __future__ import annotations

import copy
from dataclasses import dataclass

from .registry import register_architecture
from .spec import LayerSpec, ModelSpec, PartSpec, RunEntry

MIXER_TYPES = ("mlstm", "parallel")


def _need(d: dict, keys, where: str) -> None:
    if not isinstance(d, dict):
        raise ValueError(f"{where} must be an object, got {d!r}")
    missing = [k for k in keys if k not in d]
    if missing:
        raise KeyError(f"config.json lacks {missing} in {where}")


def _positive_int(d: dict, key: str, where: str) -> int:
    v = d[key]
    if not isinstance(v, int) or isinstance(v, bool) or v < 1:
        raise ValueError(f"{where}.{key} must be a positive integer, got {v!r}")
    return v


@register_architecture("Kakunex")
@dataclass(frozen=True)
class KakunexConfig:
    vocab: int
    width: int
    eps: float
    logit_scale: float
    layers: tuple  # of dicts as in config.json: {"type", "mixer", "mlp"}

    @classmethod
    def from_dict(cls, cfg: dict) -> "KakunexConfig":
        _need(cfg, ("vocab", "width", "norm", "layers"), "config.json")
        _need(cfg["norm"], ("eps",), "norm")
        if not isinstance(cfg["layers"], (list, tuple)) or not cfg["layers"]:
            raise ValueError("layers must be a non-empty list")
        out = cls(
            vocab=_positive_int(cfg, "vocab", "config.json"),
            width=_positive_int(cfg, "width", "config.json"),
            eps=float(cfg["norm"]["eps"]),
            logit_scale=float(cfg.get("logit_scale", 1.0)),
            layers=tuple(copy.deepcopy(layer) for layer in cfg["layers"]),
        )
        out.validate()
        return out

    def validate(self) -> None:
        if not self.eps >= 0:
            raise ValueError(f"norm.eps must not be negative, got {self.eps}")
        for i, layer in enumerate(self.layers):
            where = f"layers[{i}]"
            _need(layer, ("type", "mixer"), where)
            kind, m = layer["type"], layer["mixer"]
            if kind not in MIXER_TYPES:
                raise NotImplementedError(f"{where}.type {kind!r} is not supported, expected one of {MIXER_TYPES}")
            if kind == "mlstm":
                _need(m, ("heads", "dim", "vdim", "gate_cap"), f"{where}.mixer")
                for k in ("heads", "dim", "vdim"):
                    _positive_int(m, k, f"{where}.mixer")
                if not float(m["gate_cap"]) > 0:
                    raise ValueError(f"{where}.mixer.gate_cap must be positive")
            else:
                _need(m, ("left", "right"), f"{where}.mixer")
                left, right = m["left"], m["right"]
                _need(left, ("heads", "kv_heads", "dim", "vdim", "scale"), f"{where}.mixer.left")
                for k in ("heads", "kv_heads", "dim", "vdim"):
                    _positive_int(left, k, f"{where}.mixer.left")
                if left["heads"] % left["kv_heads"]:
                    raise ValueError(f"{where}.mixer.left: {left['heads']} heads are no multiple of {left['kv_heads']} kv_heads")
                if not float(left["scale"]) > 0:
                    raise ValueError(f"{where}.mixer.left.scale must be positive")
                rot = left.get("rot")
                if rot:
                    _need(rot, ("base", "dims"), f"{where}.mixer.left.rot")
                    if rot["dims"] % 2 or not 2 <= rot["dims"] <= left["dim"]:
                        raise ValueError(f"{where}.mixer.left.rot.dims must be even and at most dim, got {rot['dims']}")
                    if rot.get("scaling"):
                        _need(rot["scaling"], ("factor", "low", "high", "original"), f"{where}.mixer.left.rot.scaling")
                mask = left.get("mask")
                if mask:
                    _need(mask, ("size",), f"{where}.mixer.left.mask")
                    _positive_int(mask, "size", f"{where}.mixer.left.mask")
                    if int(mask.get("keep_first", 0)) < 0:
                        raise ValueError(f"{where}.mixer.left.mask.keep_first must not be negative")
                _need(right, ("heads", "dim", "vdim", "decay"), f"{where}.mixer.right")
                for k in ("heads", "dim", "vdim"):
                    _positive_int(right, k, f"{where}.mixer.right")
                if len(right["decay"]) != right["heads"]:
                    raise ValueError(f"{where}.mixer.right: {len(right['decay'])} decays for {right['heads']} heads")
            mlp = layer.get("mlp")
            if mlp:
                _need(mlp, ("kind", "ff"), f"{where}.mlp")
                if mlp["kind"] != "dense":
                    raise NotImplementedError(f"{where}.mlp.kind {mlp['kind']!r} is not supported, expected 'dense'")
                _need(mlp, ("limit",), f"{where}.mlp")
                _positive_int(mlp, "ff", f"{where}.mlp")
                if not float(mlp["limit"]) > 0:
                    raise ValueError(f"{where}.mlp.limit must be positive")

    def to_dict(self) -> dict:
        """The ``config.json`` that reads back as this configuration."""
        return {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.eps},
                "logit_scale": self.logit_scale, "layers": [copy.deepcopy(layer) for layer in self.layers]}

    # ------------------------------------------------------------------ lowering

    def _mixer(self, kind: str, m: dict) -> PartSpec:
        w, eps = self.width, self.eps
        if kind == "mlstm":
            return PartSpec("mlstm", {"prefix": "mix.", "hidden_size": w, "num_heads": m["heads"], "head_dim": m["dim"],
                                      "value_dim": m["vdim"], "gate_cap": float(m["gate_cap"]), "eps": eps})
        left, right = m["left"], m["right"]
        rot, mask = left.get("rot"), left.get("mask")
        position = None
        if rot:
            scaling = dict(rot["scaling"], kind="wavelength_bands") if rot.get("scaling") else None
            position = PartSpec("rotary", {"dim": int(rot["dims"]), "theta": float(rot["base"]), "pairing": "adjacent",
                                           "scaling": scaling})
        attention = PartSpec("gqa_attention", {
            "prefix": "mix.left.", "hidden_size": w, "num_heads": left["heads"], "num_kv_heads": left["kv_heads"],
            "head_dim": left["dim"], "value_dim": left["vdim"], "scale": float(left["scale"]),
            "qk_norm": "projection", "qk_norm_eps": eps,
            "window": int(mask["size"]) if mask else 0, "keep_first": int(mask.get("keep_first", 0)) if mask else 0,
            "exact_weights": True, "position": position,
            "names": {"q": "q", "k": "k", "v": "v", "o": "o", "q_norm": "q.norm", "k_norm": "k.norm"},
        })
        linear = PartSpec("decay_linear_attention", {
            "prefix": "mix.right.", "hidden_size": w, "num_heads": right["heads"], "head_dim": right["dim"],
            "value_dim": right["vdim"], "decay": tuple(float(d) for d in right["decay"]), "eps": eps})
        return PartSpec("normed_pair", {"hidden_size": w, "eps": eps, "coef": 0.5, "left": attention, "right": linear,
                                        "left_norm": "mix.left.out", "right_norm": "mix.right.out"})

    def to_spec(self) -> ModelSpec:
        w = self.width
        layers = []
        for i, layer in enumerate(self.layers):
            mlp = layer.get("mlp")
            ffn = PartSpec("none") if not mlp else PartSpec("gated_mlp", {
                "prefix": "mlp.", "hidden_size": w, "intermediate_size": int(mlp["ff"]), "activation": "swiglu_clamped",
                "limit": float(mlp["limit"]), "names": {"gate": "gate", "up": "up", "down": "down"}})
            block = PartSpec("parallel", {"norm": PartSpec("layernorm", {"width": w, "eps": self.eps, "tensor": "norm1",
                                                                         "bias_tensor": "norm1.b"})})
            layers.append(LayerSpec(f"l{i}.", block, self._mixer(layer["type"], layer["mixer"]), ffn))
        return ModelSpec(
            architecture=self.architecture,
            vocab_size=self.vocab,
            hidden_size=w,
            embedding=PartSpec("token_embedding", {"vocab_size": self.vocab, "width": w, "tensor": "embed"}),
            layers=tuple(layers),
            run_order=tuple(RunEntry(i, i) for i in range(len(layers))),
            final_norm=PartSpec("layernorm", {"width": w, "eps": self.eps, "tensor": "final.norm", "bias_tensor": "final.norm.b"}),
            head=PartSpec("linear_head", {"vocab_size": self.vocab, "width": w, "tensor": "head", "tied_to": "embed",
                                          "logit_scale": self.logit_scale}),
            max_position=None,
        )
