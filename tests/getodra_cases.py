"""Small Getodra configurations for the tests: sizes that no fast kernel's tiling suits, sizes
that suit them, and one in which much is 1 or absent (one head, one tap, a layer without a
feed-forward, a rotation of part of the rotated numbers, no scaling of the rotation)."""
import math


def _latent(heads, dim, rot_dim, vdim, rank, dims=None, scaling=True, base=10000.0):
    rot = {"base": base, "dims": rot_dim if dims is None else dims}
    if scaling:
        rot["scaling"] = {"factor": 8.0, "original": 64, "fast": 16.0, "slow": 2.0}
    return {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": rank,
            "scale": 1.0 / math.sqrt(dim + rot_dim), "rot": rot}


def _lightning(heads, dim, vdim, decay):
    return {"heads": heads, "dim": dim, "vdim": vdim, "decay": decay}


def _layer(kind, mixer, ff, weights_of=None):
    e = {"type": kind, "mixer": mixer, "mlp": None if ff is None else {"kind": "dense", "ff": ff}}
    if weights_of is not None:
        e["weights_of"] = weights_of
    return e


def config_odd():
    la = _latent(3, 24, 8, 20, 40)
    li = _lightning(5, 12, 20, [0.5, 0.8, 0.95, 0.99, 1.0])
    return {"architecture": "Getodra", "vocab": 200, "width": 72, "max_positions": 160,
            "norm": {"eps": 1e-5}, "canon": {"taps": 3},
            "layers": [_layer("latent_attention", la, 100), _layer("lightning", li, 88),
                       _layer("latent_attention", la, 100, weights_of=0),
                       _layer("lightning", li, 88, weights_of=1)]}


def config_even():
    la = _latent(4, 64, 32, 32, 64, base=50000.0)
    li = _lightning(2, 32, 64, [0.9, 0.97])
    return {"architecture": "Getodra", "vocab": 384, "width": 128, "max_positions": 320,
            "norm": {"eps": 1e-6}, "canon": {"taps": 4},
            "layers": [_layer("lightning", li, 256), _layer("latent_attention", la, 256),
                       _layer("lightning", li, 256, weights_of=0), _layer("latent_attention", la, 192)]}


def config_ones():
    la = _latent(1, 16, 16, 16, 32, dims=8, scaling=False)
    li = _lightning(1, 16, 16, [0.7])
    return {"architecture": "Getodra", "vocab": 96, "width": 64, "max_positions": 128,
            "norm": {"eps": 1e-5}, "canon": {"taps": 1},
            "layers": [_layer("latent_attention", la, None), _layer("lightning", li, 64),
                       _layer("latent_attention", la, None, weights_of=0)]}


CASES = {"odd": (config_odd, 11), "even": (config_even, 22), "ones": (config_ones, 33)}
