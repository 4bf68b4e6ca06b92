"""Small Kakunex configurations for the tests. They differ from one another in every size and option: heads and
key/value heads (grouped, one group, none shared), query/key sizes unlike value sizes, sizes that are no multiple
of 8, rotation over the whole head or part of it, with and without the slowed-down wavelength bands, windows
shorter and longer than a page, kept first keys (none, fewer than a page, more than a page), layers with and
without a feed-forward, every order of the two mixers, a logit scale that is and is not one."""

from __future__ import annotations

from pathlib import Path

from miniserve_amd.weights.random_init import Init, write_model_folder


def attention(heads, kv_heads, dim, vdim, scale, rot=None, mask=None):
    out = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if rot is not None:
        out["rot"] = rot
    if mask is not None:
        out["mask"] = mask
    return out


def linear(heads, dim, vdim, decay):
    return {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay)}


def parallel(left, right, ff=None, limit=2.0):
    return {"type": "parallel", "mixer": {"left": left, "right": right},
            "mlp": {"kind": "dense", "ff": ff, "limit": limit} if ff else None}


def mlstm(heads, dim, vdim, cap, ff=None, limit=2.0):
    return {"type": "mlstm", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap},
            "mlp": {"kind": "dense", "ff": ff, "limit": limit} if ff else None}


def model(vocab, width, eps, logit_scale, layers):
    return {"architecture": "Kakunex", "vocab": vocab, "width": width, "norm": {"eps": eps}, "logit_scale": logit_scale,
            "layers": layers}


BANDS = {"factor": 4.0, "low": 1.0, "high": 3.0, "original": 64}

KAKUNEX = {
    # name: (config, seed, init)
    "kxA": (model(101, 64, 1e-5, 1.7, [
        parallel(attention(4, 2, 16, 24, 0.3, {"base": 100.0, "dims": 8, "scaling": BANDS}, {"size": 12, "keep_first": 5}),
                 linear(3, 8, 16, (0.5, 0.9, 0.995)), ff=96, limit=1.0),
        mlstm(2, 24, 16, 5.0, ff=None),
        parallel(attention(3, 3, 32, 32, 0.2, {"base": 10000.0, "dims": 32}, {"size": 33, "keep_first": 0}),
                 linear(1, 16, 8, (0.97,)), ff=48, limit=3.0),
    ]), 11, Init(0.12, (0.6, 1.4))),
    "kxB": (model(257, 80, 1e-6, 1.0, [
        mlstm(5, 12, 20, 12.0, ff=112, limit=0.7),
        mlstm(1, 40, 40, 2.0, ff=None),
        parallel(attention(6, 1, 20, 12, 0.25, {"base": 50.0, "dims": 4}, {"size": 16, "keep_first": 17}),
                 linear(4, 20, 20, (1.0, 0.3, 0.8, 0.99)), ff=None),
    ]), 12, Init(0.1, (0.5, 1.5))),
    # a window with neither rotation nor kept keys, an attention that sees every key, and a head size of 64
    "kxC": (model(139, 96, 1e-6, 0.5, [
        parallel(attention(2, 1, 64, 64, 0.125, None, {"size": 7}), linear(2, 64, 32, (0.9, 0.999)), ff=64, limit=2.0),
        parallel(attention(2, 2, 8, 40, 0.5, {"base": 8.0, "dims": 6, "scaling": dict(BANDS, low=0.5, original=16)}, None),
                 linear(3, 4, 4, (0.6, 0.7, 0.8)), ff=None),
        mlstm(3, 32, 32, 8.0, ff=80, limit=1.5),
    ]), 13, Init(0.1, (0.7, 1.3))),
    # sizes that are multiples of nothing: width, feed-forward, vocabulary and every head size odd or twice an odd number
    "kxD": (model(77, 90, 1e-5, 2.5, [
        parallel(attention(3, 1, 10, 6, 0.4, {"base": 300.0, "dims": 10}, {"size": 21, "keep_first": 3}),
                 linear(2, 5, 7, (0.85, 0.99)), ff=50, limit=1.2),
        mlstm(3, 9, 11, 7.0, ff=34, limit=2.0),
    ]), 14, Init(0.1, (0.6, 1.4))),
}


def make_folder(tmp: Path, name: str) -> Path:
    cfg, seed, init = KAKUNEX[name]
    return write_model_folder(Path(tmp) / name, cfg, seed, init)
