"""Small Sosepel configurations for the tests: sizes that no fast kernel's tiling suits, sizes
that suit them, and one in which much is 1 or absent (one head, one expert chosen, no groups,
no shared expert, no pair table, no temperature, no caps, a loop that runs once)."""
import math


def _mixer(heads, kv_heads, dim, vdim, diff=0.4, cap=30.0, temp=(0.25, 7)):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "diff": diff,
         "scale": 1.0 / math.sqrt(dim)}
    if cap:
        m["softcap"] = cap
    if temp:
        m["q_temp"] = {"coef": temp[0], "every": temp[1]}
    return m


def _moe(ff, experts, top, groups=None, shared=None):
    r = {"experts": experts, "top": top}
    if groups:
        r["groups"] = {"count": groups[0], "keep": groups[1]}
    return {"kind": "moe", "expert": {"ff": ff}, "router": r, "shared": {"ff": shared} if shared else None}


def _layer(mixer, mlp):
    return {"type": "attention", "mixer": mixer, "mlp": mlp}


def config_odd():
    a = _mixer(6, 3, 12, 20)
    b = _mixer(3, 3, 10, 36, diff=0.7, temp=(0.5, 16))
    return {"architecture": "Sosepel", "vocab": 211, "width": 72, "norm": {"eps": 1e-5},
            "logit_softcap": 9.0,
            "embedding": {"scale": 1.5, "bigram": {"buckets": 37, "mul_prev": 31, "mul_cur": 5}},
            "layers": [_layer(a, {"kind": "dense", "ff": 100}),
                       _layer(b, _moe(24, 6, 3, groups=(3, 2), shared=40)),
                       _layer(a, _moe(40, 9, 2, groups=(3, 1))),
                       _layer(b, None)],
            "loop": {"start": 1, "stop": 3, "times": 3}}


def config_even():
    a = _mixer(4, 1, 32, 64, cap=20.0, temp=(0.3, 32))
    b = _mixer(2, 2, 16, 32, diff=0.5)
    c = _mixer(4, 2, 64, 128, diff=0.3, temp=(0.2, 64))
    return {"architecture": "Sosepel", "vocab": 384, "width": 128, "norm": {"eps": 1e-6},
            "logit_softcap": 12.0,
            "embedding": {"scale": 0.8, "bigram": {"buckets": 101, "mul_prev": 17, "mul_cur": 3}},
            "layers": [_layer(a, _moe(64, 8, 2, groups=(4, 2), shared=96)),
                       _layer(b, {"kind": "dense", "ff": 192}),
                       _layer(c, None),
                       _layer(a, _moe(32, 16, 4, groups=(2, 1), shared=64))],
            "loop": {"start": 0, "stop": 2, "times": 2}}


def config_ones():
    a = _mixer(1, 1, 16, 16, diff=0.2, cap=None, temp=None)
    return {"architecture": "Sosepel", "vocab": 96, "width": 64, "norm": {"eps": 1e-5},
            "embedding": {"scale": 1.0},
            "layers": [_layer(a, _moe(16, 2, 1)), _layer(a, {"kind": "dense", "ff": 48}),
                       _layer(a, _moe(24, 4, 4, shared=32))],
            "loop": {"start": 2, "stop": 3, "times": 1}}


def config_straight():
    """No loop at all, groups of one expert each."""
    a = _mixer(2, 1, 8, 24, cap=15.0, temp=(1.0, 1))
    cfg = config_ones()
    cfg.update(vocab=120, width=40, logit_softcap=5.0,
               layers=[_layer(a, _moe(16, 4, 2, groups=(4, 3))), _layer(a, None)])
    cfg["embedding"] = {"scale": 2.0, "bigram": {"buckets": 1, "mul_prev": 1, "mul_cur": 1}}
    del cfg["loop"]
    return cfg


def random_config(seed):
    """A seeded random configuration: head counts and groups of every kind, sizes in steps of
    8 and others, widths and vocabularies that are no power of two, layers of every kind of
    feed-forward in any order, with and without pair table, caps, temperature, loop."""
    import random
    rng = random.Random(seed)
    width = rng.choice([40, 64, 72, 96, 100, 128, 136, 192])

    def mixer():
        kv = rng.choice([1, 2, 3])
        dim = rng.choice([8, 12, 16, 24, 32, 40, 64, 80])
        return _mixer(kv * rng.choice([1, 1, 2, 3, 4, 5]), kv, dim, rng.choice([8, 16, 20, 24, 40, 64, 96, 128]),
                      diff=rng.choice([0.1, 0.35, 0.6, 0.8]), cap=rng.choice([None, 8.0, 30.0, 40.0]),
                      temp=rng.choice([None, (0.3, 32), (0.5, 8), (1.0, 1), (0.2, 17)]))

    def mlp():
        kind = rng.choice(["none", "dense", "moe", "moe", "moe"])
        if kind == "none":
            return None
        if kind == "dense":
            return {"kind": "dense", "ff": rng.choice([24, 64, 100, 160])}
        count = rng.choice([1, 2, 3, 4, 8])
        per = rng.choice([1, 2, 3, 4, 6])
        keep = rng.randint(1, count)
        top = rng.randint(1, min(keep * per, 6))
        return _moe(rng.choice([16, 24, 40, 64]), count * per, top,
                    groups=None if count == 1 and rng.random() < 0.5 else (count, keep),
                    shared=rng.choice([None, 16, 48, 72]))

    n = rng.randint(1, 5)
    cfg = {"architecture": "Sosepel", "vocab": rng.choice([97, 256, 333, 600]), "width": width,
           "norm": {"eps": rng.choice([1e-6, 1e-5])}, "embedding": {"scale": rng.choice([0.75, 1.0, 3.0])},
           "layers": [_layer(mixer(), mlp()) for _ in range(n)]}
    if rng.random() < 0.7:
        cfg["logit_softcap"] = rng.choice([5.0, 12.0, 30.0])
    if rng.random() < 0.7:
        cfg["embedding"]["bigram"] = {"buckets": rng.choice([1, 13, 521, 4099]),
                                      "mul_prev": rng.choice([1, 131, 65537]), "mul_cur": rng.choice([1, 5, 31])}
    if rng.random() < 0.7:
        start = rng.randrange(n)
        cfg["loop"] = {"start": start, "stop": rng.randint(start + 1, n), "times": rng.randint(1, 3)}
    return cfg


CASES = {"odd": (config_odd, 11), "even": (config_even, 22), "ones": (config_ones, 33),
         "straight": (config_straight, 44)}
