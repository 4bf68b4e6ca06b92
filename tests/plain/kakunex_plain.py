"""Kakunex, whole sequences, no cache, float64 numpy: one function per mechanism, token by token
where the design is a recurrence. It shares no code with the product path.

A Kakunex layer is ``x += mixer(h) + ff(h)`` with ``h = layer_norm(x)`` (one norm, both sublayers read it).
Mixers: ``mlstm`` (matrix memory with exponential gates and a running maximum) and ``parallel`` (a softmax
attention with a sliding window that also keeps the first tokens, beside a linear attention with a fixed
decay per head; the two outputs are RMS-normed over the width and averaged). The feed-forward is gated with
clamped inputs. The head is the embedding table, scaled.

Notation: T tokens, W width, H heads, G key/value heads, D query/key size, E value size.
"""

from __future__ import annotations

import math

import numpy as np


# ---------------------------------------------------------------- norms and activations


def layer_norm(x, w, b, eps):
    mu = x.mean(axis=-1, keepdims=True)
    var = ((x - mu) ** 2).mean(axis=-1, keepdims=True)
    return (x - mu) / np.sqrt(var + eps) * w + b


def unit_rms(x, eps):
    return x / np.sqrt((x * x).mean(axis=-1, keepdims=True) + eps)


def rms_norm(x, w, eps):
    return unit_rms(x, eps) * w


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def log_sigmoid(z):
    return -np.logaddexp(0.0, -z)


# ---------------------------------------------------------------- rotation


def rotary_frequencies(dims: int, base: float, scaling: dict | None) -> np.ndarray:
    """``f_i = base^(-2i/dims)``, i < dims/2; with ``scaling`` the long wavelengths are slowed down:
    wavelength ``l = 2 pi / f``; ``l < original/high`` keeps f, ``l > original/low`` takes ``f/factor``,
    between the two a straight blend in ``s = (original/l - low) / (high - low)``."""
    i = np.arange(dims // 2, dtype=np.float64)
    f = base ** (-2.0 * i / dims)
    if not scaling:
        return f
    factor, low, high, orig = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
    out = np.empty_like(f)
    for n, fi in enumerate(f):
        wl = 2 * math.pi / fi
        if wl < orig / high:
            out[n] = fi
        elif wl > orig / low:
            out[n] = fi / factor
        else:
            s = (orig / wl - low) / (high - low)
            out[n] = (1 - s) * fi / factor + s * fi
    return out


def rotate_adjacent(x, positions, freqs):
    """``x [T, heads, D]``: elements (2i, 2i+1) of the first ``2 len(freqs)`` of every head are turned by
    ``positions[t] * freqs[i]``; the rest pass."""
    out = x.copy()
    r = 2 * len(freqs)
    ang = positions[:, None].astype(np.float64) * freqs[None, :]
    c, s = np.cos(ang)[:, None, :], np.sin(ang)[:, None, :]
    u, v = x[..., 0:r:2], x[..., 1:r:2]
    out[..., 0:r:2] = u * c - v * s
    out[..., 1:r:2] = v * c + u * s
    return out


# ---------------------------------------------------------------- softmax attention with window and kept first tokens


def visible(i: int, j: int, size: int, keep_first: int) -> bool:
    return j <= i and (i - j < size or j < keep_first)


def window_attention(h, w, m, eps):
    """``m``: the left mixer's config (dim, vdim, heads, kv_heads, mask, rot, scale); ``w``: its tensors
    by short name (q, k, v, o, q.norm, k.norm)."""
    T = h.shape[0]
    H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rms_norm(h @ w["q"].T, w["q.norm"], eps).reshape(T, H, D)  # over the whole projection, before the split
    k = rms_norm(h @ w["k"].T, w["k.norm"], eps).reshape(T, G, D)
    v = (h @ w["v"].T).reshape(T, G, E)
    rot = m.get("rot")
    pos = np.arange(T)
    if rot:
        f = rotary_frequencies(int(rot["dims"]), float(rot["base"]), rot.get("scaling"))
        q, k = rotate_adjacent(q, pos, f), rotate_adjacent(k, pos, f)
    mask = m.get("mask") or {}
    size, keep = int(mask.get("size", 0)) or T + 1, int(mask.get("keep_first", 0))
    out = np.zeros((T, H, E))
    for i in range(T):
        js = [j for j in range(i + 1) if visible(i, j, size, keep)]
        for a in range(H):
            g = a // (H // G)
            s = (k[js, g] @ q[i, a]) * m["scale"]
            p = np.exp(s - s.max())
            out[i, a] = (p / p.sum()) @ v[js, g]
    return out.reshape(T, H * E) @ w["o"].T


# ---------------------------------------------------------------- linear attention with a fixed decay per head


def lightning_attention(h, w, m, eps):
    T = h.shape[0]
    H, D, E = m["heads"], m["dim"], m["vdim"]
    q = silu(h @ w["q"].T).reshape(T, H, D)
    k = silu(h @ w["k"].T).reshape(T, H, D)
    v = silu(h @ w["v"].T).reshape(T, H, E)
    out = np.zeros((T, H, E))
    for a in range(H):
        S = np.zeros((D, E))
        for t in range(T):
            S = m["decay"][a] * S + np.outer(k[t, a], v[t, a])
            out[t, a] = S.T @ q[t, a]
    y = rms_norm(out.reshape(T, H * E), w["norm"], eps) * sigmoid(h @ w["g"].T)
    return y @ w["o"].T


def parallel_mixer(h, w, m, eps):
    """Half the sum of the two mixers' outputs, each RMS-normed over the width first."""
    left = {k[len("left."):]: v for k, v in w.items() if k.startswith("left.") and k != "left.out"}
    right = {k[len("right."):]: v for k, v in w.items() if k.startswith("right.") and k != "right.out"}
    a = rms_norm(window_attention(h, left, m["left"], eps), w["left.out"], eps)
    b = rms_norm(lightning_attention(h, right, m["right"], eps), w["right.out"], eps)
    return 0.5 * (a + b)


# ---------------------------------------------------------------- matrix memory with exponential gates


def mlstm(h, w, m, eps):
    T = h.shape[0]
    H, D, E, cap = m["heads"], m["dim"], m["vdim"], float(m["gate_cap"])
    q = (h @ w["q"].T).reshape(T, H, D) * D ** -0.5
    k = (h @ w["k"].T).reshape(T, H, D)
    v = (h @ w["v"].T).reshape(T, H, E)
    gi = cap * np.tanh((h @ w["i"].T + w["i.b"]) / cap)  # log input gate
    gf = log_sigmoid(cap * np.tanh((h @ w["f"].T + w["f.b"]) / cap))  # log forget gate
    out = np.zeros((T, H, E))
    for a in range(H):
        S, n, mx = np.zeros((D, E)), np.zeros(D), 0.0
        for t in range(T):
            m_new = max(gf[t, a] + mx, gi[t, a])
            fs, is_ = math.exp(gf[t, a] + mx - m_new), math.exp(gi[t, a] - m_new)
            S = fs * S + is_ * np.outer(k[t, a], v[t, a])
            n = fs * n + is_ * k[t, a]
            mx = m_new
            o = S.T @ q[t, a] / (max(abs(n @ q[t, a]), math.exp(-mx)) + 1e-6)
            out[t, a] = unit_rms(o, eps)
    y = out.reshape(T, H * E) * w["norm"] * sigmoid(h @ w["g"].T)
    return y @ w["o"].T


# ---------------------------------------------------------------- feed-forward


def dense_ff(h, w, m):
    lim = float(m["limit"])
    g = np.minimum(h @ w["gate"].T, lim)
    u = np.clip(h @ w["up"].T, -lim, lim)
    return (g * sigmoid(1.702 * g) * (u + 1)) @ w["down"].T


# ---------------------------------------------------------------- the model


def _sub(weights, prefix):
    return {k[len(prefix):]: v for k, v in weights.items() if k.startswith(prefix)}


MIXERS = {"mlstm": mlstm, "parallel": parallel_mixer}


def forward(cfg: dict, weights: dict, tokens, return_layers: bool = False):
    """Logits ``[T, vocab]`` of one sequence (and the residual stream after every layer)."""
    eps = float(cfg["norm"]["eps"])
    x = weights["embed"][np.asarray(tokens)]
    after = []
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = layer_norm(x, weights[p + "norm1"], weights[p + "norm1.b"], eps)
        y = MIXERS[layer["type"]](h, _sub(weights, p + "mix."), layer["mixer"], eps)
        if layer.get("mlp"):
            y = y + dense_ff(h, _sub(weights, p + "mlp."), layer["mlp"])
        x = x + y
        after.append(x)
    z = layer_norm(x, weights["final.norm"], weights["final.norm.b"], eps)
    logits = z @ weights["embed"].T * float(cfg["logit_scale"])
    return (logits, np.stack(after)) if return_layers else logits


def greedy(cfg: dict, weights: dict, prompt, max_new: int) -> list[int]:
    """One token per pass over the whole sequence so far, first maximal index."""
    ids, out = list(prompt), []
    for _ in range(max_new):
        nxt = int(np.argmax(forward(cfg, weights, ids)[-1]))
        out.append(nxt)
        ids.append(nxt)
    return out
