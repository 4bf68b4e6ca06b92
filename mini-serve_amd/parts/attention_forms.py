"""Two further forms of softmax attention over the paged cache. Neither has a counterpart in the reference.

``differential_attention``: every head has two score maps over the same values, the second subtracted from the first
with one weight per layer. Queries and keys carry both maps (``[heads, 2, D]`` / ``[kv_heads, 2, D]`` per token), the
values one set per key/value head. Options, each with its constant as a parameter: a short causal convolution over
time behind the three projections (``conv_taps``; the last ``taps - 1`` projection rows of a request are its state),
an RMS norm per head and map with one weight shared by all (``qk_norm_eps``), a soft cap on the scaled scores
(``softcap``). The maps' difference ``a1 - lambda a2`` is divided by its root mean square over the head and
multiplied by ``1 - lambda_offset``; ``lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + lambda_offset``.
To the attention kernel the maps are heads: ``2 heads`` query heads over ``2 kv_heads`` key heads, of which two
neighbours share one value head. The query rows of the projection are reordered once, when the weights are bound, so
that the query heads of one key head lie side by side: (key/value head, map, head of the group).

``latent_attention``: a token keeps one latent vector ``c [C]`` (RMS-normed) and one rotated key part ``[R]`` that
all heads share. A head's key is ``[W_uk c, shared part]``, its value ``W_uv c``. The products with ``W_uk`` and
``W_uv`` are moved to the query's side and behind the weighted sum: ``q_plain . (W_uk c) = (W_uk^T q_plain) . c``
and ``sum_j p_j W_uv c_j = W_uv sum_j p_j c_j``. The attention kernel then sees ``heads`` query heads of ``C + R``
elements over one key head whose rows are ``[c, rotated part]`` and whose values are ``c`` again. The cache holds
those rows and, as the values, ``c`` once more with the tokens of one element side by side (the order in which the
matrix cores take the second product's operand). Options: a sliding ``window``, a learned sink per head in the softmax's
denominator (``sinks``), a sigmoid gate per head read off the mixer's input (``gate``), and ``shares_cache``: the
layer has no projection of its own for the latent and reads the cache rows another layer wrote (its run-order entry
names that layer's cache slot), with query, up-projections, window and the rest of its own.
"""

from __future__ import annotations

import torch

from ..config.spec import PartSpec
from .base import CachePlane, KVNeed, Mixer, StateNeed, StateTensor, TensorSpec
from .registry import part_class, register


def _named(spec: PartSpec, default: dict) -> dict[str, str]:
    p = spec.get("prefix", "")
    given = spec.get("names") or {}
    return {k: p + given.get(k, d) for k, d in default.items()}


@register("mixer", "differential_attention")
class DifferentialAttention(Mixer):
    NAMES = {"q": "q", "k": "k", "v": "v", "o": "o", "q_conv": "q.conv", "k_conv": "k.conv", "v_conv": "v.conv",
             "q_norm": "q.norm", "k_norm": "k.norm", "lq1": "lq1", "lk1": "lk1", "lq2": "lq2", "lk2": "lk2"}

    def __init__(self, spec: PartSpec, rt):
        super().__init__(spec, rt)
        self.hidden = int(spec["hidden_size"])
        self.heads = int(spec["num_heads"])
        self.kv_heads = int(spec["num_kv_heads"])
        self.head_dim = int(spec["head_dim"])
        self.value_dim = int(spec.get("value_dim") or self.head_dim)
        self.scale = float(spec["scale"])
        self.softcap = float(spec.get("softcap") or 0.0)
        self.taps = int(spec.get("conv_taps") or 1)
        self.qk_norm_eps = spec.get("qk_norm_eps")
        self.eps = float(spec["eps"])
        self.lambda_offset = float(spec["lambda_offset"])
        self.names = _named(spec, self.NAMES)
        if self.heads % self.kv_heads:
            raise ValueError(f"{self.heads} query heads are no multiple of {self.kv_heads} KV heads")
        if not self.scale > 0 or self.softcap < 0 or self.taps < 1:
            raise ValueError("scale must be positive, softcap not negative and conv_taps at least 1")
        if not (1 <= self.head_dim <= 1024 and 1 <= self.value_dim <= 1024):
            raise ValueError(f"head sizes {self.head_dim} / {self.value_dim}: the attention kernel takes sizes up to 1024")
        self.group = self.heads // self.kv_heads
        self.channels = 2 * (self.heads + self.kv_heads) * self.head_dim + self.kv_heads * self.value_dim
        self.proj = self.conv = self.o = self.q_norm = self.k_norm = None
        self.lam = None

    @classmethod
    def tensors(cls, spec: PartSpec) -> dict[str, TensorSpec]:
        n = _named(spec, cls.NAMES)
        w, d = int(spec["hidden_size"]), int(spec["head_dim"])
        e = int(spec.get("value_dim") or d)
        h, g = int(spec["num_heads"]), int(spec["num_kv_heads"])
        taps = int(spec.get("conv_taps") or 1)
        out = {n["q"]: TensorSpec((2 * h * d, w)), n["k"]: TensorSpec((2 * g * d, w)), n["v"]: TensorSpec((g * e, w)),
               n["o"]: TensorSpec((w, h * e))}
        out.update({n[k]: TensorSpec((d,)) for k in ("lq1", "lk1", "lq2", "lk2")})
        if spec.get("conv_taps"):
            out.update({n["q_conv"]: TensorSpec((2 * h * d, taps)), n["k_conv"]: TensorSpec((2 * g * d, taps)),
                        n["v_conv"]: TensorSpec((g * e, taps))})
        if spec.get("qk_norm_eps") is not None:
            out.update({n["q_norm"]: TensorSpec((d,), init="ones"), n["k_norm"]: TensorSpec((d,), init="ones")})
        return out

    def _query_order(self, device) -> torch.Tensor:
        """Rows of the stored query projection, (head, map, element), in the order (key/value head, map, head of the
        group, element)."""
        idx = torch.arange(2 * self.heads * self.head_dim, device=device).view(self.kv_heads, self.group, 2, self.head_dim)
        return idx.permute(0, 2, 1, 3).reshape(-1)

    def bind(self, tensors) -> None:
        n = self.names
        q, k, v = (tensors[n[x]] for x in ("q", "k", "v"))
        if len({t.dtype for t in (q, k, v)}) != 1:
            raise ValueError(f"{n['q']} and its neighbours are stored in different dtypes")
        order = self._query_order(q.device)
        self.proj = torch.cat((q[order], k, v), dim=0).contiguous()
        if self.spec.get("conv_taps"):
            parts = [tensors[n["q_conv"]][order], tensors[n["k_conv"]], tensors[n["v_conv"]]]
            self.conv = torch.cat(parts, dim=0).contiguous()
        else:
            self.conv = torch.ones((self.channels, 1), dtype=q.dtype, device=q.device)
        self.o = tensors[n["o"]]
        if self.qk_norm_eps is not None:
            self.q_norm, self.k_norm = tensors[n["q_norm"]].to(self.conv.dtype), tensors[n["k_norm"]].to(self.conv.dtype)
        # one number for the layer, formed once, in float32
        dots = [(tensors[n[a]].to(torch.float32) * tensors[n[b]].to(torch.float32)).sum() for a, b in (("lq1", "lk1"), ("lq2", "lk2"))]
        lam = torch.exp(dots[0]) - torch.exp(dots[1]) + torch.tensor(self.lambda_offset, dtype=torch.float32, device=dots[0].device)
        self.lam = float(lam.item())

    def kv_need(self) -> KVNeed:
        return KVNeed((CachePlane("k", 2 * self.kv_heads, self.head_dim),
                       CachePlane("v", self.kv_heads, self.value_dim, token_minor=True)), 0)

    def state_need(self) -> StateNeed | None:
        if self.taps == 1:
            return None
        return StateNeed((StateTensor("conv", (self.taps - 1, self.channels), "float32"),))

    def forward(self, x, batch, cache, state, residual):
        ops = self.rt.ops
        if not cache.writes:
            raise NotImplementedError("differential attention keeps keys and values of its own")
        x32 = ops.linear(x, self.proj, out_dtype=torch.float32)
        eps = 0.0 if self.qk_norm_eps is None else float(self.qk_norm_eps)
        q = ops.conv_norm_store(x32, self.conv, self.taps, state["conv"] if self.taps > 1 else None, batch, self.q_norm, self.k_norm,
                                eps, cache.slots, cache.k, cache.v, 2 * self.heads, 2 * self.kv_heads, self.kv_heads, self.head_dim,
                                self.value_dim, self.rt.dtype)
        a = ops.paged_attention(q, cache.k, cache.v, cache.block_table, batch, 2 * self.heads, 2 * self.kv_heads, self.head_dim,
                                self.scale, 0, self.value_dim, softcap=self.softcap, value_share=2, out_dtype=torch.float32)
        o = ops.map_difference_norm(a, self.kv_heads, self.group, self.value_dim, self.lam, self.eps, 1.0 - self.lambda_offset,
                                    self.rt.dtype)
        return ops.linear(o, self.o, accumulate_into=residual, defer=True)

    def parameters_bytes(self) -> int:
        ts = [self.proj, self.conv, self.o] + ([self.q_norm, self.k_norm] if self.q_norm is not None else [])
        return sum(t.numel() * t.element_size() for t in ts)

    def flops(self, rows) -> int:
        tokens = sum(n for n, _ in rows)
        pairs = sum(n * cached + n * (n + 1) // 2 for n, cached in rows)
        linear = 2 * tokens * self.hidden * (self.channels + self.heads * self.value_dim)
        return linear + 2 * pairs * 2 * self.heads * (self.head_dim + self.value_dim) + 2 * tokens * self.channels * self.taps


@register("mixer", "latent_attention")
class LatentAttention(Mixer):
    NAMES = {"q": "q", "dkv": "dkv", "dkv_norm": "dkv.norm", "uk": "uk", "uv": "uv", "sink": "sink", "g": "g", "o": "o"}

    def __init__(self, spec: PartSpec, rt):
        super().__init__(spec, rt)
        self.hidden = int(spec["hidden_size"])
        self.heads = int(spec["num_heads"])
        self.plain_dim = int(spec["head_dim"])
        self.rot_dim = int(spec["rot_dim"])
        self.value_dim = int(spec["value_dim"])
        self.latent_dim = int(spec["latent_dim"])
        self.scale = float(spec["scale"])
        self.window = int(spec.get("window") or 0)
        self.eps = float(spec["eps"])
        self.sinks = bool(spec.get("sinks", False))
        self.gate = bool(spec.get("gate", False))
        self.shares_cache = bool(spec.get("shares_cache", False))
        self.names = _named(spec, self.NAMES)
        self.key_dim = self.latent_dim + self.rot_dim
        if min(self.heads, self.plain_dim, self.value_dim, self.latent_dim) < 1 or self.rot_dim < 0 or self.window < 0:
            raise ValueError("heads and sizes must be positive, rot_dim and window not negative")
        if self.key_dim > 1024:
            raise ValueError(f"latent and rotated sizes {self.latent_dim} + {self.rot_dim}: the attention kernel takes up to 1024 together")
        if not self.scale > 0:
            raise ValueError(f"the attention scale must be positive, not {self.scale}")
        pos = spec.get("position") or PartSpec("none")
        self.position = part_class("position", pos)(pos, rt)
        self.q_col = 0
        self.kv_col = None if self.shares_cache else self.heads * (self.plain_dim + self.rot_dim)
        self.g_col = self.heads * (self.plain_dim + self.rot_dim) + (0 if self.shares_cache else self.key_dim)
        self.proj = self.o = self.dkv_norm = self.uk_t = self.uv = self.sink = None

    @classmethod
    def tensors(cls, spec: PartSpec) -> dict[str, TensorSpec]:
        n = _named(spec, cls.NAMES)
        w, h = int(spec["hidden_size"]), int(spec["num_heads"])
        d, r, e, c = (int(spec[k]) for k in ("head_dim", "rot_dim", "value_dim", "latent_dim"))
        out = {n["q"]: TensorSpec((h * (d + r), w)), n["uk"]: TensorSpec((h * d, c)), n["uv"]: TensorSpec((h * e, c)),
               n["o"]: TensorSpec((w, h * e))}
        if not spec.get("shares_cache", False):
            out[n["dkv"]] = TensorSpec((c + r, w))
            out[n["dkv_norm"]] = TensorSpec((c,), init="ones")
        if spec.get("sinks", False):
            out[n["sink"]] = TensorSpec((h,), init="uniform")
        if spec.get("gate", False):
            out[n["g"]] = TensorSpec((h, w))
        return out

    def bind(self, tensors) -> None:
        n = self.names
        parts = [tensors[n["q"]]] + ([] if self.shares_cache else [tensors[n["dkv"]]]) + ([tensors[n["g"]]] if self.gate else [])
        if len({t.dtype for t in parts}) != 1:
            raise ValueError(f"{n['q']} and its neighbours are stored in different dtypes")
        self.proj = torch.cat(parts, dim=0).contiguous()
        h, d, e, c = self.heads, self.plain_dim, self.value_dim, self.latent_dim
        self.uk_t = tensors[n["uk"]].view(h, d, c).transpose(1, 2).contiguous()  # per head [C, D]: q_plain -> the latent's space
        self.uv = tensors[n["uv"]].view(h, e, c).contiguous()
        self.o = tensors[n["o"]]
        if not self.shares_cache:
            self.dkv_norm = tensors[n["dkv_norm"]]
        if self.sinks:
            self.sink = tensors[n["sink"]].to(torch.float32).contiguous()

    def kv_need(self) -> KVNeed:
        return KVNeed((CachePlane("k", 1, self.key_dim), CachePlane("v", 1, self.latent_dim, token_minor=True)), self.window)

    def forward(self, x, batch, cache, state, residual):
        ops = self.rt.ops
        if cache.writes == self.shares_cache:
            raise ValueError("a latent attention writes the cache exactly when it has a latent projection of its own")
        x32 = ops.linear(x, self.proj, out_dtype=torch.float32)
        rot = self.position.rotation(batch)
        if rot is not None and rot.dim > self.rot_dim:
            raise ValueError(f"{rot.dim} rotated elements in a part of {self.rot_dim}")
        q_plain, q_full = ops.latent_prepare(
            x32, self.q_col, self.kv_col, rot.table if rot is not None else None, rot.dim if rot is not None else 0,
            rot.pairing if rot is not None else "halves", self.dkv_norm, self.eps, cache.slots, cache.k, cache.v, self.heads,
            self.plain_dim, self.rot_dim, self.latent_dim, self.rt.dtype)
        ops.head_linear(q_plain, self.uk_t, q_full, 0)
        a = ops.paged_attention(q_full, cache.k, cache.v, cache.block_table, batch, self.heads, 1, self.key_dim, self.scale,
                                self.window, self.latent_dim, sinks=self.sink)
        o = torch.empty((x.shape[0], self.heads * self.value_dim), dtype=self.rt.dtype, device=x.device)
        ops.head_linear(a, self.uv, o, 0, gate=(x32, self.g_col) if self.gate else None)
        return ops.linear(o, self.o, accumulate_into=residual, defer=True)

    def parameters_bytes(self) -> int:
        ts = [self.proj, self.uk_t, self.uv, self.o] + [t for t in (self.dkv_norm, self.sink) if t is not None]
        return sum(t.numel() * t.element_size() for t in ts)

    def flops(self, rows) -> int:
        tokens = sum(n for n, _ in rows)
        pairs = 0
        for n, cached in rows:
            if self.window:
                pairs += sum(min(p + 1, self.window) for p in range(cached, cached + n))
            else:
                pairs += n * cached + n * (n + 1) // 2
        linear = 2 * tokens * self.hidden * (self.proj.shape[0] if self.proj is not None else 0) + 2 * tokens * self.hidden * self.heads * self.value_dim
        per_head = 2 * tokens * self.heads * self.latent_dim * (self.plain_dim + self.value_dim)
        return linear + per_head + 2 * pairs * self.heads * (self.key_dim + self.latent_dim)
