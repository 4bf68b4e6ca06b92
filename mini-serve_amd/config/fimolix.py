"""Typed configuration of the Fimolix decoder, read from its own ``config.json`` keys. The reference has no such
architecture.

``config.json``: ``architecture`` (the name), ``vocab``, ``width``, ``norm.eps`` and ``layers``, a list in which every
entry names its mixer (``type``), the mixer's sizes and constants (``mixer``) and its feed-forward (``mlp``, or null for
none). Layer ``i``'s tensors start with ``l<i>.``.

A layer is ``x += N1(mixer(x))``, then ``x += N2(ff(x))``: the sublayers read the stream itself and their output is
RMS-normed with a weight stored around zero, ``y / rms(y) * (1 + w)`` (``norm1``, ``norm2``). Mixers:

* ``attention`` (``heads``, ``kv_heads``, ``dim``, ``vdim``, ``scale``, ``softcap``, ``conv``, ``diff``; tensors ``mix.q k v o
  q.conv k.conv v.conv q.norm k.norm lq1 lk1 lq2 lk2``): two softmax maps per head over the same values, rows of ``q`` and
  ``k`` laid out (head, map, element); a causal convolution of ``conv`` taps over time behind each projection; an RMS
  norm per head and map; scores ``softcap tanh(scale q.k / softcap)``, every earlier key visible, no positions. The
  second map is subtracted with the weight ``exp(lq1.lk1) - exp(lq2.lk2) + diff``; the difference is divided by its root
  mean square over the head and multiplied by ``1 - diff``.
* ``latent_attention`` (``heads``, ``dim``, ``rot_dim``, ``vdim``, ``kv_rank``, ``scale``, ``rot``, ``mask``, optional
  ``kv_from``; tensors ``mix.q dkv dkv.norm uk uv sink g o``): ``dkv`` projects to ``kv_rank`` latent elements (RMS-normed,
  weight ``dkv.norm``) and ``rot_dim`` elements of a key part shared by all heads; ``uk`` / ``uv`` make each head's
  plain key part (``dim``) and value (``vdim``) from the latent; query heads are ``[dim plain, rot_dim rotated]``. The
  rotation turns adjacent pairs of the first ``rot.dims`` rotated elements by ``position * rot.base ** (-2i / rot.dims)``.
  A query sees the last ``mask.size`` tokens, itself included; ``exp(sink_h)`` joins head ``h``'s softmax denominator;
  head ``h``'s output is multiplied by ``sigmoid(g x)_h``. With ``kv_from: j`` the layer has no ``dkv`` and reads what
  layer ``j`` keeps.

Feed-forward (``kind: dense``, ``ff``; tensors ``mlp.up down``): ``down(gelu_tanh(up(x)))``. The final norm is
``final.norm`` (one plus weight); the head is the embedding table ``embed``.
"""

from __future__ import annotations

import copy
from dataclasses import dataclass

from .registry import register_architecture
from .spec import LayerSpec, ModelSpec, PartSpec, RunEntry

MIXER_TYPES = ("attention", "latent_attention")


def _need(d, keys, where: str) -> None:
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


@register_architecture("Fimolix")
@dataclass(frozen=True)
class FimolixConfig:
    vocab: int
    width: int
    eps: float
    layers: tuple  # of dicts as in config.json: {"type", "mixer", "mlp"}

    @classmethod
    def from_dict(cls, cfg: dict) -> "FimolixConfig":
        _need(cfg, ("vocab", "width", "norm", "layers"), "config.json")
        _need(cfg["norm"], ("eps",), "norm")
        if not isinstance(cfg["layers"], (list, tuple)) or not cfg["layers"]:
            raise ValueError("layers must be a non-empty list")
        out = cls(
            vocab=_positive_int(cfg, "vocab", "config.json"),
            width=_positive_int(cfg, "width", "config.json"),
            eps=float(cfg["norm"]["eps"]),
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
            mw = f"{where}.mixer"
            if kind == "attention":
                _need(m, ("heads", "kv_heads", "dim", "vdim", "scale", "diff", "conv"), mw)
                for k in ("heads", "kv_heads", "dim", "vdim", "conv"):
                    _positive_int(m, k, mw)
                if m["heads"] % m["kv_heads"]:
                    raise ValueError(f"{mw}: {m['heads']} heads are no multiple of {m['kv_heads']} kv_heads")
                if m.get("softcap") is not None and not float(m["softcap"]) > 0:
                    raise ValueError(f"{mw}.softcap must be positive")
            else:
                _need(m, ("heads", "dim", "rot_dim", "vdim", "kv_rank", "scale", "rot"), mw)
                for k in ("heads", "dim", "rot_dim", "vdim", "kv_rank"):
                    _positive_int(m, k, mw)
                _need(m["rot"], ("base", "dims"), f"{mw}.rot")
                dims = m["rot"]["dims"]
                if not isinstance(dims, int) or dims % 2 or not 2 <= dims <= m["rot_dim"]:
                    raise ValueError(f"{mw}.rot.dims must be even and at most rot_dim, got {dims!r}")
                if not float(m["rot"]["base"]) > 0:
                    raise ValueError(f"{mw}.rot.base must be positive")
                if m.get("mask"):
                    _need(m["mask"], ("size",), f"{mw}.mask")
                    _positive_int(m["mask"], "size", f"{mw}.mask")
                src = m.get("kv_from")
                if src is not None:
                    if not isinstance(src, int) or isinstance(src, bool) or not 0 <= src < i:
                        raise ValueError(f"{mw}.kv_from must name an earlier layer, got {src!r}")
                    other = self.layers[src]
                    if other["type"] != "latent_attention" or other["mixer"].get("kv_from") is not None:
                        raise ValueError(f"{mw}.kv_from names layer {src}, which keeps no latent of its own")
                    for k in ("kv_rank", "rot_dim", "rot"):
                        if other["mixer"][k] != m[k]:
                            raise ValueError(f"{mw}.{k} differs from layer {src}'s, whose cache the layer reads")
            if not float(m["scale"]) > 0:
                raise ValueError(f"{mw}.scale must be positive")
            mlp = layer.get("mlp")
            if mlp:
                _need(mlp, ("kind", "ff"), f"{where}.mlp")
                if mlp["kind"] != "dense":
                    raise NotImplementedError(f"{where}.mlp.kind {mlp['kind']!r} is not supported, expected 'dense'")
                _positive_int(mlp, "ff", f"{where}.mlp")

    def to_dict(self) -> dict:
        """The ``config.json`` that reads back as this configuration."""
        return {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.eps},
                "layers": [copy.deepcopy(layer) for layer in self.layers]}

    # ------------------------------------------------------------------ lowering

    def _norm(self, tensor: str) -> PartSpec:
        return PartSpec("rmsnorm", {"width": self.width, "eps": self.eps, "tensor": tensor, "offset": 1.0})

    def _mixer(self, kind: str, m: dict) -> PartSpec:
        w, eps = self.width, self.eps
        if kind == "attention":
            return PartSpec("differential_attention", {
                "prefix": "mix.", "hidden_size": w, "num_heads": m["heads"], "num_kv_heads": m["kv_heads"], "head_dim": m["dim"],
                "value_dim": m["vdim"], "scale": float(m["scale"]), "softcap": float(m.get("softcap") or 0.0),
                "conv_taps": int(m["conv"]), "qk_norm_eps": eps, "eps": eps, "lambda_offset": float(m["diff"])})
        rot, mask = m["rot"], m.get("mask")
        position = PartSpec("rotary", {"dim": int(rot["dims"]), "theta": float(rot["base"]), "pairing": "adjacent"})
        return PartSpec("latent_attention", {
            "prefix": "mix.", "hidden_size": w, "num_heads": m["heads"], "head_dim": m["dim"], "rot_dim": m["rot_dim"],
            "value_dim": m["vdim"], "latent_dim": m["kv_rank"], "scale": float(m["scale"]),
            "window": int(mask["size"]) if mask else 0, "eps": eps, "sinks": True, "gate": True,
            "shares_cache": m.get("kv_from") is not None, "position": position})

    def to_spec(self) -> ModelSpec:
        w = self.width
        layers, order = [], []
        for i, layer in enumerate(self.layers):
            mlp = layer.get("mlp")
            ffn = PartSpec("none") if not mlp else PartSpec("dense_mlp", {
                "prefix": "mlp.", "hidden_size": w, "intermediate_size": int(mlp["ff"]), "activation": "gelu_tanh",
                "names": {"up": "up", "down": "down"}})
            block = PartSpec("outnorm", {"mixer_norm": self._norm("norm1"), "ffn_norm": self._norm("norm2") if mlp else None,
                                         "spare": None if mlp else {"norm2": w}})
            layers.append(LayerSpec(f"l{i}.", block, self._mixer(layer["type"], layer["mixer"]), ffn))
            src = layer["mixer"].get("kv_from") if layer["type"] == "latent_attention" else None
            order.append(RunEntry(i, i) if src is None else RunEntry(i, int(src), writes_cache=False))
        return ModelSpec(
            architecture=self.architecture,
            vocab_size=self.vocab,
            hidden_size=w,
            embedding=PartSpec("token_embedding", {"vocab_size": self.vocab, "width": w, "tensor": "embed"}),
            layers=tuple(layers),
            run_order=tuple(order),
            final_norm=self._norm("final.norm"),
            head=PartSpec("linear_head", {"vocab_size": self.vocab, "width": w, "tensor": "head", "tied_to": "embed"}),
            max_position=None,
        )
