"""Kakunex on the CPU: its configuration and lowering, the cache manager's kept first pages in both
implementations, the slowed-down rotation frequencies, and the plain implementation held against closed forms
that do not share its loops."""

from __future__ import annotations

import copy
import math
import random

import numpy as np
import pytest

from kakunex_models import KAKUNEX
from miniserve_amd.cache import NO_PAGE, CacheLayout, CacheManager, PageAllocator
from miniserve_amd.cache.backend import allocator_class
from miniserve_amd.cache.native import NativePageAllocator
from miniserve_amd.config import config_from_dict
from miniserve_amd.parts.model import CacheSlotNeed, expected_tensors
from miniserve_amd.parts.registry import part_class
from plain import kakunex_plain as K

BACKENDS = [PageAllocator, NativePageAllocator]


# ---------------------------------------------------------------- configuration


@pytest.mark.parametrize("name", sorted(KAKUNEX))
def test_config_reads_back_and_names_its_tensors(name):
    cfg = KAKUNEX[name][0]
    c = config_from_dict(cfg)
    assert config_from_dict(c.to_dict()).to_dict() == c.to_dict()
    names = expected_tensors(c.to_spec())
    assert names["embed"].shape == (cfg["vocab"], cfg["width"]) and "final.norm.b" in names
    for i, layer in enumerate(cfg["layers"]):
        assert (f"l{i}.mlp.down" in names) == bool(layer["mlp"])
        if layer["type"] == "mlstm":
            m = layer["mixer"]
            assert names[f"l{i}.mix.i"].shape == (m["heads"], cfg["width"]) and names[f"l{i}.mix.f.b"].shape == (m["heads"],)
            assert names[f"l{i}.mix.o"].shape == (cfg["width"], m["heads"] * m["vdim"])
        else:
            left, right = layer["mixer"]["left"], layer["mixer"]["right"]
            assert names[f"l{i}.mix.left.q.norm"].shape == (left["heads"] * left["dim"],)
            assert names[f"l{i}.mix.left.v"].shape == (left["kv_heads"] * left["vdim"], cfg["width"])
            assert names[f"l{i}.mix.right.g"].shape == (right["heads"] * right["vdim"], cfg["width"])
            assert names[f"l{i}.mix.left.out"].shape == names[f"l{i}.mix.right.out"].shape == (cfg["width"],)
    assert "head" not in names  # the head reads the embedding's table


def test_config_refusals():
    base = KAKUNEX["kxA"][0]

    def changed(fn):
        c = copy.deepcopy(base)
        fn(c)
        return c

    with pytest.raises(NotImplementedError):
        config_from_dict(changed(lambda c: c["layers"][0].update(type="conv")))
    with pytest.raises(NotImplementedError):
        config_from_dict(changed(lambda c: c["layers"][0]["mlp"].update(kind="routed")))
    with pytest.raises(ValueError):
        config_from_dict(changed(lambda c: c["layers"][0]["mixer"]["left"].update(kv_heads=3)))
    with pytest.raises(ValueError):
        config_from_dict(changed(lambda c: c["layers"][0]["mixer"]["right"].update(decay=[0.5])))
    with pytest.raises(ValueError):
        config_from_dict(changed(lambda c: c["layers"][0]["mixer"]["left"]["rot"].update(dims=7)))
    with pytest.raises(KeyError):
        config_from_dict(changed(lambda c: c["layers"][1]["mixer"].pop("gate_cap")))
    with pytest.raises(KeyError):
        config_from_dict(changed(lambda c: c.pop("width")))
    with pytest.raises(ValueError, match="architecture"):
        config_from_dict({"vocab": 3})


def needs_of(cfg):
    spec = config_from_dict(cfg).to_spec()
    out = []
    for e in spec.run_order:
        mixer = part_class("mixer", spec.layers[e.layer].mixer)(spec.layers[e.layer].mixer, None)
        out.append(CacheSlotNeed(e.cache, mixer.kv_need(), mixer.state_need()))
    return out


def test_lowering_groups_the_cache_by_window_and_kept_keys():
    layout = CacheLayout.from_needs(needs_of(KAKUNEX["kxA"][0]))
    assert sorted((g.window, g.keep_first, g.slots) for g in layout.groups) == [(12, 5, (0,)), (33, 0, (2,))]
    planes = {g.window: {p.name: (p.heads, p.width, p.token_minor) for p in g.planes} for g in layout.groups}
    assert planes[12] == {"k": (2, 16, False), "v": (2, 24, True)}
    states = {s.slot: {t.name: t.shape for t in s.tensors} for s in layout.states}
    assert states[0] == {"right.S": (3, 8, 16)} and states[1] == {"S": (2, 24, 16), "n": (2, 24), "m": (2,)}
    layout = CacheLayout.from_needs(needs_of(KAKUNEX["kxC"][0]))
    assert sorted((g.window, g.keep_first) for g in layout.groups) == [(0, 0), (7, 0)]  # no mask: every key is kept


# ---------------------------------------------------------------- kept first pages


@pytest.mark.parametrize("A", BACKENDS)
def test_release_before_keeps_the_first_pages(A):
    a = A(10, 4)
    t = a.new_table()
    t.append(30)  # pages 0..7
    assert t.release_before(7, 2) == 0  # page 1 is kept, nothing else is wholly passed
    assert t.release_before(18, 2) == 2 and t.pages == [0, 1, NO_PAGE, NO_PAGE, 4, 5, 6, 7]
    assert t.num_held == 6 and a.num_free == 4
    assert t.slot(5) == 5 and t.slot(17) == 4 * 4 + 1
    with pytest.raises(IndexError):
        t.slot(9)
    assert t.release_before(18, 2) == 0 and t.release_before(25, 2) == 2 and t.num_held == 4
    assert t.append(4) == [5]  # the newest freed page comes back first
    t.release()
    assert a.num_free == 10
    a.check_invariants()
    # more kept pages than the table has yet: nothing goes until the window has passed them all
    t = a.new_table()
    t.append(6)
    assert t.release_before(6, 3) == 0
    t.append(20)
    assert t.release_before(17, 3) == 1 and t.pages[:4] == t.pages[:3] + [NO_PAGE] and t.num_held == 6
    t.release()
    assert a.num_free == 10
    a.check_invariants()


def test_backends_agree_with_kept_pages_under_random_operations():
    rng = random.Random(5)
    for keep in (0, 1, 3):
        a, b = PageAllocator(40, 4), NativePageAllocator(40, 4)
        ta, tb = a.new_table(), b.new_table()
        for _ in range(200):
            op = rng.random()
            if op < 0.6:
                n = rng.randint(1, 9)
                if ta.pages_needed(n) <= a.num_free:
                    assert ta.append(n) == tb.append(n)
            elif op < 0.95:
                pos = rng.randint(0, ta.num_tokens + 3)
                assert ta.release_before(pos, keep) == tb.release_before(pos, keep)
            else:
                ta.release(), tb.release()
            assert ta.pages == tb.pages and ta.num_held == tb.num_held and a.num_free == b.num_free
            a.check_invariants(), b.check_invariants()


@pytest.mark.parametrize("backend", ["python", "cpp"])
def test_a_window_that_keeps_first_keys_holds_their_pages(backend):
    layout = CacheLayout.from_needs(needs_of(KAKUNEX["kxB"][0]))  # one group: window 16, the first 17 keys kept
    m = CacheManager(layout, 4, [64], 2, allocator_class=allocator_class(backend))
    assert m.keep_pages(layout.groups[0]) == 5
    rc = m.acquire()
    for _ in range(30):
        m.extend(rc, 3)
        m.advance(rc)
    (t,) = rc.tables
    live = [i for i, p in enumerate(t.pages) if p != NO_PAGE]
    first_window_page = (90 - 16 + 1) // 4
    assert live == list(range(5)) + list(range(first_window_page, 23))
    assert m.peak_pages(10_000, 3) == [(16 - 1 + 3 + 3) // 4 + 1 + 5]
    m.release(rc)
    assert m.idle


# ---------------------------------------------------------------- rotation frequencies


def test_scaled_frequencies_follow_their_bands():
    import torch

    from miniserve_amd.parts.rotary import scale_frequencies

    for dims, base, scaling in ((48, 5e5, {"factor": 6.0, "low": 1.0, "high": 5.0, "original": 2048}),
                                (8, 100.0, {"factor": 4.0, "low": 1.0, "high": 3.0, "original": 64}),
                                (6, 8.0, {"factor": 2.0, "low": 0.5, "high": 3.0, "original": 16})):
        plain = K.rotary_frequencies(dims, base, None)
        mine = scale_frequencies(torch.tensor(plain, dtype=torch.float32), scaling).double().numpy()
        want = K.rotary_frequencies(dims, base, scaling)
        assert np.allclose(mine, want, rtol=2e-7, atol=0)
        kept = (2 * math.pi / plain) < scaling["original"] / scaling["high"]
        slowed = (2 * math.pi / plain) > scaling["original"] / scaling["low"]
        assert np.allclose(want[kept], plain[kept]) and np.allclose(want[slowed], plain[slowed] / scaling["factor"])
        between = ~kept & ~slowed
        assert ((want[between] <= plain[between]) & (want[between] >= plain[between] / scaling["factor"])).all()


# ---------------------------------------------------------------- the plain implementation against closed forms


def test_plain_rotation_is_a_complex_product():
    rng = np.random.default_rng(0)
    x = rng.normal(size=(5, 2, 10))
    f = np.array([0.7, 0.05, 1.3])
    pos = np.array([0, 1, 7, 100, 3])
    got = K.rotate_adjacent(x, pos, f)
    z = (x[..., 0:6:2] + 1j * x[..., 1:6:2]) * np.exp(1j * pos[:, None, None] * f[None, None, :])
    assert np.allclose(got[..., 0:6:2], z.real) and np.allclose(got[..., 1:6:2], z.imag) and (got[..., 6:] == x[..., 6:]).all()


def test_plain_mask():
    assert [j for j in range(10) if K.visible(9, j, 3, 2)] == [0, 1, 7, 8, 9]
    assert [j for j in range(10) if K.visible(2, j, 3, 2)] == [0, 1, 2]
    assert [j for j in range(10) if K.visible(6, j, 3, 0)] == [4, 5, 6]


def test_plain_decay_attention_is_a_weighted_sum():
    rng = np.random.default_rng(1)
    T, W, H, D, E = 9, 6, 2, 3, 4
    m = {"heads": H, "dim": D, "vdim": E, "decay": [0.8, 0.99]}
    w = {"q": rng.normal(size=(H * D, W)), "k": rng.normal(size=(H * D, W)), "v": rng.normal(size=(H * E, W)),
         "g": rng.normal(size=(H * E, W)), "o": np.eye(H * E), "norm": np.ones(H * E)}
    h = rng.normal(size=(T, W))
    q, k, v = (K.silu(h @ w[n].T).reshape(T, H, -1) for n in ("q", "k", "v"))
    o = np.zeros((T, H, E))
    for t in range(T):
        for a in range(H):
            for j in range(t + 1):
                o[t, a] += m["decay"][a] ** (t - j) * (q[t, a] @ k[j, a]) * v[j, a]
    want = K.rms_norm(o.reshape(T, -1), w["norm"], 1e-6) * K.sigmoid(h @ w["g"].T)
    assert np.allclose(K.lightning_attention(h, w, m, 1e-6), want)


def test_plain_mlstm_equals_the_unstabilised_sums():
    """Without the running maximum the state is a sum of terms exp(sum of later forget gates + input gate) k v^T
    (and the zero state, whose weight the maximum still counts): small gates keep that form exact in float64."""
    rng = np.random.default_rng(2)
    T, W, H, D, E, cap = 7, 5, 2, 3, 2, 4.0
    m = {"heads": H, "dim": D, "vdim": E, "gate_cap": cap}
    w = {n: rng.normal(size=(H * D, W)) for n in ("q", "k")}
    w.update({n: rng.normal(size=(H * E, W)) for n in ("v", "g")})
    w.update({"i": rng.normal(size=(H, W)), "f": rng.normal(size=(H, W)), "i.b": rng.normal(size=H), "f.b": rng.normal(size=H),
              "o": np.eye(H * E), "norm": rng.normal(size=H * E)})
    h = rng.normal(size=(T, W))
    q = (h @ w["q"].T).reshape(T, H, D) / math.sqrt(D)
    k, v = (h @ w["k"].T).reshape(T, H, D), (h @ w["v"].T).reshape(T, H, E)
    gi = cap * np.tanh((h @ w["i"].T + w["i.b"]) / cap)
    gf = np.log(K.sigmoid(cap * np.tanh((h @ w["f"].T + w["f.b"]) / cap)))
    out = np.zeros((T, H, E))
    for a in range(H):
        for t in range(T):
            logw = np.array([gf[j + 1 : t + 1, a].sum() + gi[j, a] for j in range(t + 1)])
            mt = max(gf[: t + 1, a].sum(), logw.max())  # the zero state carries the maximum's start, 0, through every forget gate
            C = sum(math.exp(lw) * np.outer(k[j, a], v[j, a]) for j, lw in enumerate(logw))
            n = sum(math.exp(lw) * k[j, a] for j, lw in enumerate(logw))
            o = (C.T @ q[t, a]) * math.exp(-mt) / (max(abs(n @ q[t, a]) * math.exp(-mt), math.exp(-mt)) + 1e-6)
            out[t, a] = K.unit_rms(o, 1e-6)
    want = out.reshape(T, -1) * w["norm"] * K.sigmoid(h @ w["g"].T)
    assert np.allclose(K.mlstm(h, w, m, 1e-6), want)


def test_plain_layer_is_one_norm_and_a_sum():
    cfg = KAKUNEX["kxA"][0]
    rng = np.random.default_rng(3)
    names = expected_tensors(config_from_dict(cfg).to_spec())
    w = {n: rng.normal(size=ts.shape) * 0.2 for n, ts in names.items()}
    tokens = [3, 1, 4, 1, 5, 9, 2, 6]
    logits, layers = K.forward(cfg, w, tokens, return_layers=True)
    x = w["embed"][tokens]
    h = K.layer_norm(x, w["l0.norm1"], w["l0.norm1.b"], 1e-5)
    mix = K.parallel_mixer(h, {k[len("l0.mix."):]: v for k, v in w.items() if k.startswith("l0.mix.")}, cfg["layers"][0]["mixer"], 1e-5)
    ff = K.dense_ff(h, {k[len("l0.mlp."):]: v for k, v in w.items() if k.startswith("l0.mlp.")}, cfg["layers"][0]["mlp"])
    assert np.allclose(layers[0], x + mix + ff)
    z = K.layer_norm(layers[-1], w["final.norm"], w["final.norm.b"], 1e-5)
    assert np.allclose(logits, z @ w["embed"].T * 1.7) and logits.shape == (8, 101)
    assert np.allclose(h.mean(-1), (w["l0.norm1"] * ((x - x.mean(-1, keepdims=True)) / x.std(-1, keepdims=True))).mean(-1)
                       + w["l0.norm1.b"].mean(), atol=1e-3)
