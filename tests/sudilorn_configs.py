"""Small Sudilorn configurations that differ from each other in every size, constant and option."""
import random

import torch


def _rot(base, dims, scaling=None):
    r = {"base": base, "dims": dims}
    if scaling is not None:
        r["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    return r


def _diff(heads, kv_heads, dim, vdim, scale, diff, conv, window, rot, mlp=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "diff": diff, "rot": rot}
    if conv:
        m["conv"] = conv
    if window is not None:
        m["mask"] = {"size": window}
    return {"type": "attention", "mixer": m, "mlp": mlp}


def _left(heads, kv_heads, dim, vdim, scale, window, keep, rot):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "rot": rot}
    if window is not None:
        m["mask"] = {"size": window, "keep_first": keep} if keep else {"size": window}
    return m


def _right(heads, kv_heads, dim, vdim, conv):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim}
    if conv:
        m["conv"] = conv
    return m


def _par(left, right, left_scale, right_scale, mlp=None):
    return {"type": "parallel", "mixer": {"left": left, "right": right, "left_scale": left_scale,
                                          "right_scale": right_scale}, "mlp": mlp}


def _moe(experts, top, ff, groups=None, keep=None):
    router = {"experts": experts, "top": top}
    if groups is not None:
        router["groups"] = {"count": groups, "keep": keep}
    return {"kind": "moe", "router": router, "expert": {"ff": ff}}


SUDILORN = {
    # the mixers in both orders, grouped kv heads, values smaller and larger than keys, windows shorter than a prompt,
    # kept first tokens that end inside a page, a stretch whose ramp lies inside the pairs, three groups of experts of
    # which two stay, a layer without a feed-forward
    "SA": {
        "seed": 3, "architecture": "Sudilorn", "vocab": 300, "width": 64, "norm": {"eps": 1e-5}, "residual_mult": 0.7,
        "layers": [
            _par(_left(4, 2, 16, 8, 0.3, 24, 3, _rot(10000.0, 8)), _right(4, 2, 12, 20, 3), 0.6, 1.3,
                 mlp=_moe(6, 2, 24, groups=3, keep=2)),
            _diff(4, 2, 16, 24, 0.35, 0.3, 4, 20, _rot(5000.0, 12, (8.0, 64, 4.0, 1.0)), mlp=_moe(4, 1, 16)),
            _diff(2, 1, 8, 8, 0.5, 0.8, 0, 33, _rot(100.0, 8), mlp=None),
            _par(_left(2, 2, 8, 24, 0.4, 40, 0, _rot(50.0, 4)), _right(2, 1, 16, 8, 2), 1.0, 0.4,
                 mlp=_moe(8, 3, 32, groups=2, keep=1)),
        ],
    },
    # sizes that fit no fast path (a width that is no multiple of 4, heads of 6 and 10 elements, a prime vocabulary),
    # one kv head, as many kv heads as heads, one group that holds every expert, groups of one expert, every expert
    # chosen, a convolution of one tap, no window at all, kept tokens beyond the window's size, a multiplier of one
    "SB": {
        "seed": 5, "architecture": "Sudilorn", "vocab": 257, "width": 54, "norm": {"eps": 1e-3}, "residual_mult": 1.0,
        "layers": [
            _diff(3, 1, 6, 10, 0.6, 0.5, 2, 7, _rot(30.0, 6, (4.0, 16, 8.0, 2.0)), mlp=_moe(2, 2, 20, groups=1, keep=1)),
            _par(_left(3, 3, 10, 6, 0.4, 5, 9, _rot(1000.0, 10)), _right(3, 3, 7, 9, 1), 0.5, 0.5,
                 mlp=_moe(3, 1, 18, groups=3, keep=2)),
            _par(_left(2, 1, 6, 6, 0.5, None, 0, _rot(70.0, 2)), _right(1, 1, 10, 6, 0), 1.5, 1.0, mlp=None),
            _diff(1, 1, 10, 6, 0.3, 0.1, 5, None, _rot(400.0, 10), mlp=_moe(5, 5, 12)),
        ],
    },
    # sharp scores: a key just inside a window, a kept first token or a key where a page ends carries most of a
    # query's weight
    "SS": {
        "seed": 13, "architecture": "Sudilorn", "vocab": 128, "width": 32, "norm": {"eps": 1e-5}, "residual_mult": 0.9,
        "layers": [
            _par(_left(2, 1, 16, 16, 1.5, 48, 2, _rot(10000.0, 4)), _right(2, 1, 16, 16, 4), 1.0, 0.7,
                 mlp=_moe(4, 2, 16, groups=2, keep=1)),
            _diff(2, 1, 16, 16, 2.0, 0.4, 3, 37, _rot(10000.0, 8, (2.0, 32, 2.0, 1.0)), mlp=_moe(4, 2, 16, groups=2, keep=2)),
        ],
    },
}

# with the sizes the vector and matrix-core paths need (GPU tests)
SUDILORN_FAST = {
    "SF": {
        "seed": 9, "architecture": "Sudilorn", "vocab": 1000, "width": 256, "norm": {"eps": 1e-5}, "residual_mult": 0.8,
        "layers": [
            _par(_left(8, 2, 64, 64, 0.125, 80, 5, _rot(10000.0, 32)), _right(4, 2, 64, 128, 4), 0.7, 0.9,
                 mlp=_moe(8, 2, 128, groups=4, keep=2)),
            _diff(4, 2, 64, 128, 0.12, 0.5, 4, 100, _rot(500000.0, 64, (16.0, 128, 16.0, 1.0)), mlp=_moe(16, 4, 64, groups=4, keep=3)),
            _diff(8, 8, 32, 32, 0.2, 0.7, 2, 64, _rot(1000.0, 16), mlp=None),
            _par(_left(4, 4, 128, 96, 0.09, 130, 17, _rot(300.0, 128)), _right(8, 2, 128, 64, 3), 1.0, 1.0,
                 mlp=_moe(6, 1, 64)),
        ],
    },
}


def sudilorn_config_json(name: str) -> dict:
    return {k: v for k, v in {**SUDILORN, **SUDILORN_FAST}[name].items() if k != "seed"}


def write_sudilorn(name: str, out_dir: str, dtype=torch.float32) -> str:
    from jax_llm_examples_amd.config import get_architecture
    from jax_llm_examples_amd.weights import write_random_model

    top = sudilorn_config_json(name)
    arch = get_architecture(top["architecture"])
    return write_random_model(arch, arch.parse_config(top), out_dir, {**SUDILORN, **SUDILORN_FAST}[name]["seed"], dtype)


def draw_sudilorn(seed: int):
    """A configuration drawn at random: ``(config.json, page size, request lengths)``."""
    rng = random.Random(seed)

    def rot(dim):
        dims = rng.choice([d for d in (2, 4, 8, 16, 32, 64) if d <= dim])
        sc = rng.choice([None, (rng.choice([2.0, 8.0]), rng.choice([16, 64]), rng.choice([4.0, 32.0]), rng.choice([0.5, 1.0]))])
        return dims, sc

    def moe():
        experts = rng.choice([2, 4, 6, 8, 12])
        groups = rng.choice([None] + [g for g in (1, 2, 3, 4) if experts % g == 0])
        keep = None if groups is None else rng.randint(1, groups)
        per = experts if groups is None else keep * (experts // groups)
        return _moe(experts, rng.randint(1, min(per, 4)), rng.choice([16, 24, 64, 96]), groups, keep)

    layers = []
    for _ in range(rng.randint(1, 4)):
        kv = rng.choice([1, 2, 3])
        heads = kv * rng.choice([1, 2, 4])
        dim, vdim = rng.choice([8, 16, 24, 32, 64, 128]), rng.choice([8, 16, 40, 64, 128])
        window = rng.choice([None, 5, 16, 31, 64, 100])
        mlp = rng.choice([None, moe(), moe()])
        if rng.random() < 0.5:
            dims, sc = rot(dim)
            layers.append(_diff(heads, kv, dim, vdim, rng.choice([0.1, 0.3]), rng.choice([0.2, 0.6]),
                                rng.choice([0, 1, 2, 4]), window, _rot(rng.choice([100.0, 250000.0]), dims, sc), mlp))
        else:
            dims, _ = rot(dim)
            rk = rng.choice([1, 2])
            layers.append(_par(_left(heads, kv, dim, vdim, rng.choice([0.1, 0.3]), window, rng.choice([0, 1, 4, 20]),
                                     _rot(rng.choice([100.0, 500000.0]), dims)),
                               _right(rk * rng.choice([1, 2]), rk, rng.choice([8, 16, 48, 64, 128]),
                                      rng.choice([8, 24, 64, 128]), rng.choice([0, 2, 4])),
                               rng.choice([0.5, 1.0]), rng.choice([0.5, 1.2]), mlp))
    top = {"architecture": "Sudilorn", "vocab": rng.choice([97, 257, 300, 512, 1001]),
           "width": rng.choice([56, 64, 72, 100, 128, 192, 256, 264]), "norm": {"eps": rng.choice([1e-5, 1e-6, 1e-3])},
           "residual_mult": rng.choice([0.5, 1.0, 1.4]), "layers": layers}
    lengths = [rng.choice([1, 2, 17, 33, 64, 65, 97, 130]) for _ in range(rng.randint(2, 5))]
    return top, rng.choice([16, 16, 32, 64]), lengths
