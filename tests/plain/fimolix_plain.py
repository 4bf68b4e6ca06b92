"""Fimolix, whole sequences, no cache, float64 numpy: one function per mechanism. It shares no code with
the product path.

A Fimolix layer norms what a sublayer puts out, not what it reads: ``x += N1(mixer(x))``, then ``x += N2(ff(x))``,
with ``N(y) = y / rms(y) * (1 + w)``. Mixers: ``attention`` (two softmax maps per head over the same values, the
second subtracted with one learned weight per layer; a short causal convolution over time behind each of the three
projections; soft-capped scores; no positions) and ``latent_attention`` (keys and values of all heads are read off
one small vector per token; a part of every query and one shared key part carry a rotation; a sliding window; a
learned sink in the softmax's denominator; a gate per head). The feed-forward is ``down(gelu_tanh(up(x)))``. The head
is the embedding table.

Notation: T tokens, W width, H heads, G key/value heads, D query/key size, E value size, R rotated size,
C latent size.
"""

from __future__ import annotations

import math

import numpy as np


# ---------------------------------------------------------------- norms and activations


def unit_rms(x, eps):
    return x / np.sqrt((x * x).mean(axis=-1, keepdims=True) + eps)


def rms_norm(x, w, eps):
    return unit_rms(x, eps) * w


def one_plus_norm(x, w, eps):
    """The layers' and the model's norm: the stored weight lies around zero."""
    return unit_rms(x, eps) * (1.0 + w)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


# ---------------------------------------------------------------- short convolution over time


def short_conv(u, w):
    """``u [T, channels]``, ``w [channels, taps]``: ``y_t = sum_j w[:, j] u_(t - taps + 1 + j)``, zeros before the start."""
    T, taps = u.shape[0], w.shape[1]
    padded = np.concatenate([np.zeros((taps - 1, u.shape[1])), u], axis=0)
    y = np.zeros_like(u)
    for j in range(taps):
        y += padded[j : j + T] * w[:, j]
    return y


# ---------------------------------------------------------------- rotation


def rotate_adjacent(x, positions, dims, base):
    """Turns the pairs (2i, 2i + 1), i < dims / 2, of the last axis of ``x [T, ..., >= dims]`` by ``p base^(-2i/dims)``."""
    i = np.arange(dims // 2, dtype=np.float64)
    ang = positions.astype(np.float64)[:, None] * base ** (-2.0 * i / dims)  # [T, dims/2]
    shape = (x.shape[0],) + (1,) * (x.ndim - 2) + (dims // 2,)
    cos, sin = np.cos(ang).reshape(shape), np.sin(ang).reshape(shape)
    out = x.copy()
    a, b = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = a * cos - b * sin
    out[..., 1:dims:2] = b * cos + a * sin
    return out


# ---------------------------------------------------------------- softmax over visible keys


def masked_softmax(scores, visible, sink=None):
    """``scores [T, T]``, ``visible`` boolean of the same shape; ``sink``: a number whose exponential joins the
    denominator (it has neither key nor value)."""
    s = np.where(visible, scores, -np.inf)
    m = s.max(axis=-1, keepdims=True)
    if sink is not None:
        m = np.maximum(m, sink)
    e = np.where(visible, np.exp(s - m), 0.0)
    den = e.sum(axis=-1, keepdims=True)
    if sink is not None:
        den = den + np.exp(sink - m)
    return e / den


def causal(T):
    i = np.arange(T)
    return i[None, :] <= i[:, None]


def sliding(T, size):
    i = np.arange(T)
    d = i[:, None] - i[None, :]
    return (d >= 0) & (d < size)


# ---------------------------------------------------------------- mixers


def differential_attention(h, w, m, eps):
    """``w``: the mixer's tensors by their names behind ``mix.``; ``m``: its entry of the configuration."""
    T = h.shape[0]
    H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = short_conv(h @ w["q"].T, w["q.conv"]).reshape(T, H, 2, D)
    k = short_conv(h @ w["k"].T, w["k.conv"]).reshape(T, G, 2, D)
    v = short_conv(h @ w["v"].T, w["v.conv"]).reshape(T, G, E)
    q = rms_norm(q, w["q.norm"], eps)
    k = rms_norm(k, w["k.norm"], eps)
    lam = math.exp(float((w["lq1"] * w["lk1"]).sum())) - math.exp(float((w["lq2"] * w["lk2"]).sum())) + m["diff"]
    cap = m.get("softcap")  # absent: the scores are not capped
    seen = causal(T)
    out = np.zeros((T, H, E))
    for head in range(H):
        g = head // (H // G)
        maps = []
        for which in range(2):
            s = (q[:, head, which] @ k[:, g, which].T) * m["scale"]
            if cap:
                s = cap * np.tanh(s / cap)
            maps.append(masked_softmax(s, seen) @ v[:, g])
        o = maps[0] - lam * maps[1]
        out[:, head] = unit_rms(o, eps) * (1.0 - m["diff"])
    return out.reshape(T, H * E) @ w["o"].T


def latent_of(h, w, m, eps, positions):
    """What a latent-attention layer keeps per token: the normed latent ``[T, C]`` and the rotated shared key part ``[T, R]``."""
    C, R = m["kv_rank"], m["rot_dim"]
    both = h @ w["dkv"].T
    c = rms_norm(both[:, :C], w["dkv.norm"], eps)
    kr = rotate_adjacent(both[:, C:], positions, m["rot"]["dims"], m["rot"]["base"])
    return c, kr


def latent_attention(h, w, m, eps, positions, kept):
    """``kept``: ``(c, kr)`` of this layer or of the layer it borrows them from."""
    T = h.shape[0]
    H, D, R, E = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
    c, kr = kept
    q = (h @ w["q"].T).reshape(T, H, D + R)
    q_plain = q[:, :, :D]
    q_turned = rotate_adjacent(q[:, :, D:], positions, m["rot"]["dims"], m["rot"]["base"])
    k_plain = (c @ w["uk"].T).reshape(T, H, D)
    v = (c @ w["uv"].T).reshape(T, H, E)
    gate = sigmoid(h @ w["g"].T)  # [T, H]
    seen = sliding(T, m["mask"]["size"]) if m.get("mask") else causal(T)  # absent: every earlier token is seen
    out = np.zeros((T, H, E))
    for head in range(H):
        s = (q_plain[:, head] @ k_plain[:, head].T + q_turned[:, head] @ kr.T) * m["scale"]
        p = masked_softmax(s, seen, sink=float(w["sink"][head]))
        out[:, head] = (p @ v[:, head]) * gate[:, head : head + 1]
    return out.reshape(T, H * E) @ w["o"].T


def dense_ff(h, w):
    return gelu_tanh(h @ w["up"].T) @ w["down"].T


# ---------------------------------------------------------------- the model


def _sub(weights, prefix):
    return {k[len(prefix):]: v for k, v in weights.items() if k.startswith(prefix)}


def forward(cfg, weights, tokens, return_layers=False):
    """Logits ``[T, vocab]`` of one sequence (and, asked for, the stream after every layer ``[layers, T, W]``)."""
    eps = cfg["norm"]["eps"]
    tokens = np.asarray(tokens)
    positions = np.arange(len(tokens))
    x = weights["embed"][tokens].astype(np.float64)
    kept, after = {}, []
    for i, layer in enumerate(cfg["layers"]):
        w, m = _sub(weights, f"l{i}.mix."), layer["mixer"]
        if layer["type"] == "attention":
            y = differential_attention(x, w, m, eps)
        elif layer["type"] == "latent_attention":
            source = m.get("kv_from")
            if source is None:
                kept[i] = latent_of(x, w, m, eps, positions)
                source = i
            y = latent_attention(x, w, m, eps, positions, kept[source])
        else:
            raise ValueError(f"layer {i}: unknown mixer {layer['type']!r}")
        x = x + one_plus_norm(y, weights[f"l{i}.norm1"], eps)
        if layer.get("mlp"):
            x = x + one_plus_norm(dense_ff(x, _sub(weights, f"l{i}.mlp.")), weights[f"l{i}.norm2"], eps)
        after.append(x.copy())
    logits = one_plus_norm(x, weights["final.norm"], eps) @ weights["embed"].T
    return (logits, np.stack(after)) if return_layers else logits


def greedy(cfg, weights, prompt, new_tokens):
    """The ``new_tokens`` tokens that greedy decoding appends to ``prompt`` (the whole sequence is run again each time)."""
    toks = list(prompt)
    for _ in range(new_tokens):
        toks.append(int(np.argmax(forward(cfg, weights, toks)[-1])))
    return toks[len(prompt):]
