"""Small Fimolix configurations for the tests. They differ from one another in every size and option: heads and
key/value heads (grouped, one group, none shared), query/key sizes unlike value sizes, sizes that are no multiple
of 8, rotation over the whole rotated part or a part of it, windows shorter and longer than a page and none at all,
convolutions of one to five taps, latent layers that read another layer's cache through a wider and through a
narrower window, keys wider than 256 elements, layers with and without a feed-forward, every order of the mixers."""

from __future__ import annotations

from pathlib import Path

from miniserve_amd.weights.random_init import Init, write_model_folder


def attention(heads, kv_heads, dim, vdim, scale, conv, diff, softcap=None, ff=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "conv": conv, "diff": diff}
    if softcap is not None:
        m["softcap"] = softcap
    return {"type": "attention", "mixer": m, "mlp": {"kind": "dense", "ff": ff} if ff else None}


def latent(heads, dim, rot_dim, vdim, kv_rank, scale, rot, size=None, kv_from=None, ff=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "scale": scale, "rot": rot}
    if size is not None:
        m["mask"] = {"size": size}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": m, "mlp": {"kind": "dense", "ff": ff} if ff else None}


def model(vocab, width, eps, layers):
    return {"architecture": "Fimolix", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}


FIMOLIX = {
    # name: (config, seed, init)
    # a borrowed cache read through a wider window than its owner's, a rotation over half the rotated part
    "fxA": (model(101, 64, 1e-5, [
        latent(3, 8, 8, 12, 24, 0.4, {"base": 100.0, "dims": 4}, size=12, ff=96),
        attention(4, 2, 16, 24, 0.3, 3, 0.3, softcap=5.0, ff=None),
        latent(2, 16, 8, 8, 24, 0.3, {"base": 100.0, "dims": 4}, size=33, kv_from=0, ff=48),
    ]), 21, Init(0.12, (0.6, 1.4))),
    # sizes that are multiples of nothing; one key/value head for all; a borrowed cache read through a narrower window
    "fxB": (model(77, 90, 1e-6, [
        attention(3, 1, 10, 6, 0.5, 2, 0.8, softcap=30.0, ff=50),
        latent(2, 5, 6, 7, 9, 0.6, {"base": 300.0, "dims": 6}, size=21, ff=None),
        latent(3, 7, 6, 5, 9, 0.5, {"base": 300.0, "dims": 6}, size=7, kv_from=1, ff=34),
        attention(2, 2, 7, 9, 0.6, 5, 0.2, ff=None),
    ]), 22, Init(0.12, (0.5, 1.5))),
    # keys of more than 256 elements, a latent attention that sees every token, a convolution of one tap, no cap
    "fxC": (model(139, 96, 1e-6, [
        latent(2, 24, 16, 16, 272, 0.15, {"base": 10000.0, "dims": 16}, size=None, ff=64),
        attention(2, 2, 64, 64, 0.125, 1, 0.5, ff=None),
        latent(4, 8, 2, 40, 16, 0.5, {"base": 8.0, "dims": 2}, size=64, ff=80),
    ]), 23, Init(0.1, (0.7, 1.3))),
    # sizes whose slices all start at multiples of 16 bytes: every product per head runs on strided rows in place
    "fxD": (model(160, 128, 1e-5, [
        attention(4, 1, 32, 64, 0.18, 4, 0.5, softcap=8.0, ff=192),
        latent(4, 32, 16, 40, 64, 0.2, {"base": 1000.0, "dims": 16}, size=40, ff=192),
        attention(2, 1, 64, 32, 0.12, 2, 0.1, softcap=3.0, ff=None),
        latent(2, 16, 16, 24, 64, 0.25, {"base": 1000.0, "dims": 16}, size=40, kv_from=1, ff=64),
    ]), 24, Init(0.1, (0.6, 1.4))),
}


def make_folder(tmp: Path, name: str) -> Path:
    cfg, seed, init = FIMOLIX[name]
    return write_model_folder(Path(tmp) / name, cfg, seed, init)
