"""Fimolix on the CPU: its configuration and lowering (run order, borrowed cache slots, what the cache manager
makes of them), the loader's treatment of a norm a layer without feed-forward may still carry, and the plain
implementation held against forms that do not share its loops."""

from __future__ import annotations

import copy
import math

import numpy as np
import pytest
import torch

from fimolix_models import FIMOLIX, make_folder
from miniserve_amd.cache import CacheLayout
from miniserve_amd.config import config_from_dict
from miniserve_amd.config.presets import preset
from miniserve_amd.config.spec import PartSpec
from miniserve_amd.parts.model import CacheSlotNeed, expected_tensors
from miniserve_amd.parts.registry import part_class
from plain import fimolix_plain as F
from plain.model_folder import read_model_folder


# ---------------------------------------------------------------- configuration


@pytest.mark.parametrize("name", sorted(FIMOLIX))
def test_config_reads_back_and_names_its_tensors(name):
    cfg = FIMOLIX[name][0]
    c = config_from_dict(cfg)
    assert config_from_dict(c.to_dict()).to_dict() == c.to_dict()
    names = expected_tensors(c.to_spec())
    w = cfg["width"]
    assert names["embed"].shape == (cfg["vocab"], w) and names["final.norm"].shape == (w,) and "head" not in names
    for i, layer in enumerate(cfg["layers"]):
        m = layer["mixer"]
        assert (f"l{i}.mlp.down" in names) == bool(layer["mlp"])
        assert names[f"l{i}.norm2"].optional == (not layer["mlp"])
        if layer["type"] == "attention":
            assert names[f"l{i}.mix.q"].shape == (2 * m["heads"] * m["dim"], w)
            assert names[f"l{i}.mix.k.conv"].shape == (2 * m["kv_heads"] * m["dim"], m["conv"])
            assert names[f"l{i}.mix.v"].shape == (m["kv_heads"] * m["vdim"], w)
            assert names[f"l{i}.mix.q.norm"].shape == names[f"l{i}.mix.lk2"].shape == (m["dim"],)
            assert names[f"l{i}.mix.o"].shape == (w, m["heads"] * m["vdim"])
        else:
            assert names[f"l{i}.mix.q"].shape == (m["heads"] * (m["dim"] + m["rot_dim"]), w)
            assert (f"l{i}.mix.dkv" in names) == (m.get("kv_from") is None) == (f"l{i}.mix.dkv.norm" in names)
            assert names[f"l{i}.mix.uk"].shape == (m["heads"] * m["dim"], m["kv_rank"])
            assert names[f"l{i}.mix.uv"].shape == (m["heads"] * m["vdim"], m["kv_rank"])
            assert names[f"l{i}.mix.sink"].shape == (m["heads"],) and names[f"l{i}.mix.g"].shape == (m["heads"], w)


def test_run_order_and_cache_groups():
    """A layer that borrows another's latent runs over that layer's cache slot without writing it; the slot keeps the
    widest window of its readers; mixers of one kind with equal sizes share a group of pages."""
    spec = config_from_dict(FIMOLIX["fxA"][0]).to_spec()
    assert [(e.layer, e.cache, e.writes_cache) for e in spec.run_order] == [(0, 0, True), (1, 1, True), (2, 0, False)]
    for name, windows in (("fxA", {0: 33}), ("fxB", {1: 21}), ("fxC", {0: 0, 2: 64}), ("fxD", {1: 40})):
        spec = config_from_dict(FIMOLIX[name][0]).to_spec()
        mixers = [part_class("mixer", layer.mixer)(layer.mixer, None) for layer in spec.layers]
        needs = {}
        for e in spec.run_order:  # what DecoderModel.cache_slots does, without a device
            kv, st = mixers[e.layer].kv_need(), mixers[e.layer].state_need()
            if e.writes_cache:
                needs[e.cache] = CacheSlotNeed(e.cache, kv, st)
        layout = CacheLayout.from_needs([needs[s] for s in sorted(needs)])
        kinds = {i: layer["type"] for i, layer in enumerate(FIMOLIX[name][0]["layers"])}
        latent_slots = {s for g in layout.groups for s in g.slots if kinds[s] == "latent_attention"}
        assert latent_slots == set(windows), name
        for i, layer in enumerate(FIMOLIX[name][0]["layers"]):
            st = mixers[i].state_need()
            if layer["type"] == "attention" and layer["mixer"]["conv"] > 1:
                m = layer["mixer"]
                channels = 2 * (m["heads"] + m["kv_heads"]) * m["dim"] + m["kv_heads"] * m["vdim"]
                assert st.tensors[0].shape == (m["conv"] - 1, channels)
            else:
                assert st is None


def test_config_refusals():
    base = FIMOLIX["fxA"][0]

    def changed(fn):
        c = copy.deepcopy(base)
        fn(c)
        return c

    with pytest.raises(NotImplementedError):
        config_from_dict(changed(lambda c: c["layers"][0].update(type="conv")))
    with pytest.raises(KeyError):
        config_from_dict(changed(lambda c: c["layers"][1]["mixer"].pop("diff")))
    with pytest.raises(ValueError):
        config_from_dict(changed(lambda c: c["layers"][1]["mixer"].update(kv_heads=3)))
    with pytest.raises(ValueError):
        config_from_dict(changed(lambda c: c["layers"][0]["mixer"]["rot"].update(dims=10)))  # more than rot_dim
    with pytest.raises(ValueError):
        config_from_dict(changed(lambda c: c["layers"][2]["mixer"].update(kv_from=1)))  # no latent attention
    with pytest.raises(ValueError):
        config_from_dict(changed(lambda c: c["layers"][2]["mixer"].update(kv_from=2)))  # not an earlier layer
    with pytest.raises(ValueError):
        config_from_dict(changed(lambda c: c["layers"][2]["mixer"].update(kv_rank=16)))  # unlike the owner's
    with pytest.raises(NotImplementedError):
        config_from_dict(changed(lambda c: c["layers"][0]["mlp"].update(kind="routed")))
    assert config_from_dict(preset("fimolix-tiny")).to_spec().architecture == "Fimolix"


def test_the_measured_shapes_are_valid_configurations():
    from miniserve_amd.measurement.designs import SHAPES, fimolix_config

    for name, shape in SHAPES.items():
        spec = config_from_dict(fimolix_config(shape)).to_spec()
        assert len(spec.layers) == shape["layers"], name
        borrowed = [e for e in spec.run_order if not e.writes_cache]
        assert len(borrowed) == shape["layers"] // 4 and all(e.cache == e.layer - 3 for e in borrowed)


def test_a_spare_second_norm_loads_and_is_ignored(tmp_path):
    """A layer without a feed-forward has no use for a second norm; a checkpoint that carries one all the same loads."""
    from safetensors.torch import load_file, save_file

    from miniserve_amd.weights.loader import WeightsError, load_weights

    folder = make_folder(tmp_path, "fxA")
    spec = config_from_dict(FIMOLIX["fxA"][0]).to_spec()
    file = folder / "model.safetensors"
    tensors = load_file(str(file))
    assert "l1.norm2" not in tensors
    load_weights(folder, spec, torch.float32, "cpu")
    tensors["l1.norm2"] = torch.zeros(64, dtype=torch.bfloat16)
    save_file(tensors, str(file))
    assert "l1.norm2" in load_weights(folder, spec, torch.float32, "cpu")
    tensors["l1.norm3"] = torch.zeros(64, dtype=torch.bfloat16)
    save_file(tensors, str(file))
    with pytest.raises(WeightsError):
        load_weights(folder, spec, torch.float32, "cpu")


def test_query_rows_are_reordered_by_key_head_and_map():
    spec = PartSpec("differential_attention", {"hidden_size": 8, "num_heads": 4, "num_kv_heads": 2, "head_dim": 3, "value_dim": 2,
                                               "scale": 1.0, "eps": 1e-6, "lambda_offset": 0.5})
    mixer = part_class("mixer", spec)(spec, None)
    order = mixer._query_order("cpu").view(2, 2, 2, 3)  # key head, map, head of the group, element
    for g in range(2):
        for which in range(2):
            for r in range(2):
                head = g * 2 + r
                assert order[g, which, r].tolist() == [(head * 2 + which) * 3 + d for d in range(3)]


# ---------------------------------------------------------------- the plain implementation against other forms


def test_short_convolution_token_by_token():
    rng = np.random.default_rng(0)
    u, w = rng.normal(size=(9, 5)), rng.normal(size=(5, 4))
    want = np.zeros_like(u)
    for t in range(9):
        for j in range(4):
            s = t - 4 + 1 + j
            if s >= 0:
                want[t] += w[:, j] * u[s]
    assert np.allclose(F.short_conv(u, w), want)
    assert np.allclose(F.short_conv(u, w[:, 3:]), u * w[:, 3])  # one tap: the newest


def test_softmax_with_a_sink_and_the_window():
    rng = np.random.default_rng(1)
    s = rng.normal(size=(6, 6))
    p = F.masked_softmax(s, F.sliding(6, 3), sink=0.7)
    for i in range(6):
        js = [j for j in range(6) if 0 <= i - j < 3]
        den = sum(math.exp(s[i, j]) for j in js) + math.exp(0.7)
        for j in range(6):
            assert math.isclose(p[i, j], math.exp(s[i, j]) / den if j in js else 0.0, rel_tol=1e-12, abs_tol=1e-15)
    assert np.allclose(F.masked_softmax(s, F.causal(6)).sum(1), 1.0)
    assert (F.masked_softmax(s, F.causal(6), sink=-1e9).sum(1) > 1 - 1e-12).all()


def test_rotation_turns_adjacent_pairs_and_keeps_the_rest():
    x = np.arange(2 * 6, dtype=np.float64).reshape(2, 6) + 1
    out = F.rotate_adjacent(x, np.array([0, 3]), 4, 100.0)
    assert np.allclose(out[0], x[0]) and np.allclose(out[:, 4:], x[:, 4:])
    for i in range(2):
        a = 3 * 100.0 ** (-2 * i / 4)
        assert np.allclose(out[1, 2 * i : 2 * i + 2], [x[1, 2 * i] * math.cos(a) - x[1, 2 * i + 1] * math.sin(a),
                                                         x[1, 2 * i + 1] * math.cos(a) + x[1, 2 * i] * math.sin(a)])
    # scores depend on the distance only
    q, k = np.ones((1, 4)), np.ones((1, 4)) * 0.5
    d1 = F.rotate_adjacent(q, np.array([9]), 4, 100.0) @ F.rotate_adjacent(k, np.array([4]), 4, 100.0).T
    d2 = F.rotate_adjacent(q, np.array([105]), 4, 100.0) @ F.rotate_adjacent(k, np.array([100]), 4, 100.0).T
    assert np.allclose(d1, d2)


def test_latent_attention_equals_its_form_with_the_products_moved(tmp_path):
    """Keys and values made per head from the latent (the plain form), against queries taken into the latent's space and
    one up-projection behind the weighted sum."""
    cfg, w = read_model_folder(make_folder(tmp_path, "fxA"))
    m = cfg["layers"][0]["mixer"]
    sub = {k[len("l0.mix."):]: v for k, v in w.items() if k.startswith("l0.mix.")}
    rng = np.random.default_rng(2)
    T = 30
    h, pos, eps = rng.normal(size=(T, cfg["width"])), np.arange(T), cfg["norm"]["eps"]
    kept = F.latent_of(h, sub, m, eps, pos)
    want = F.latent_attention(h, sub, m, eps, pos, kept)
    H, D, R, E, C = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    c, kr = kept
    q = (h @ sub["q"].T).reshape(T, H, D + R)
    out = np.zeros((T, H, E))
    for a in range(H):
        q_lat = q[:, a, :D] @ sub["uk"][a * D : (a + 1) * D]  # [T, C]
        q_rot = F.rotate_adjacent(q[:, a, D:], pos, m["rot"]["dims"], m["rot"]["base"])
        s = (q_lat @ c.T + q_rot @ kr.T) * m["scale"]
        p = F.masked_softmax(s, F.sliding(T, m["mask"]["size"]), sink=float(sub["sink"][a]))
        out[:, a] = (p @ c) @ sub["uv"][a * E : (a + 1) * E].T * F.sigmoid(h @ sub["g"][a])[:, None]
    assert np.allclose(out.reshape(T, -1) @ sub["o"].T, want, rtol=1e-9, atol=1e-12)


def test_a_one_layer_model_in_closed_form(tmp_path):
    """One token: every softmax is over one key (and the sink), the convolution sees its newest tap alone."""
    cfg = {"architecture": "Fimolix", "vocab": 11, "width": 8, "norm": {"eps": 1e-6}, "layers": [
        {"type": "attention", "mixer": {"heads": 2, "kv_heads": 1, "dim": 4, "vdim": 3, "scale": 0.5, "conv": 3, "diff": 0.25,
                                         "softcap": 2.0}, "mlp": None}]}
    from miniserve_amd.weights.random_init import Init, write_model_folder

    _, w = read_model_folder(write_model_folder(tmp_path / "one", cfg, 3, Init(0.3, (0.5, 1.5))))
    x = w["embed"][5]
    v = (w["l0.mix.v"] @ x) * w["l0.mix.v.conv"][:, -1]  # both maps put all their weight on the one value
    lam = math.exp(w["l0.mix.lq1"] @ w["l0.mix.lk1"]) - math.exp(w["l0.mix.lq2"] @ w["l0.mix.lk2"]) + 0.25
    o = np.concatenate([F.unit_rms((1 - lam) * v, 1e-6) * 0.75] * 2)
    y = x + F.one_plus_norm(w["l0.mix.o"] @ o, w["l0.norm1"], 1e-6)
    want = w["embed"] @ F.one_plus_norm(y, w["final.norm"], 1e-6)
    assert np.allclose(F.forward(cfg, w, [5])[0], want)
