"""Small Mazotar configurations that differ from each other in every size, constant and option."""
import torch


def _attn(heads, kv_heads, dim, vdim, scale, rows, far, temp=None, kv_from=None, mlp=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "bias_max": far,
         "bias_rows": rows}
    if temp is not None:
        m["q_temp"] = {"coef": temp[0], "every": temp[1]}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "attention", "mixer": m, "mlp": mlp}


def _mem(heads, dim, vdim, cap, mlp=None):
    return {"type": "mlstm", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap}, "mlp": mlp}


def _dense(ff):
    return {"kind": "dense", "ff": ff}


def _moe(experts, top, ff, shared=None):
    m = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff}}
    if shared is not None:
        m["shared"] = {"ff": shared}
    return m


MAZOTAR = {
    # attention first, a layer that borrows the keys and values of the layer before it, grouped kv heads, values
    # smaller and larger than keys, two experts a token, a shared expert of another width, three streams, a layer
    # without a feed-forward, a short distance table whose last row begins inside a prompt
    "MA": {
        "seed": 3, "architecture": "Mazotar", "vocab": 300, "width": 64, "norm": {"eps": 1e-5}, "streams": 3,
        "embedding": {"scale": 0.7},
        "layers": [
            _attn(4, 2, 16, 8, 0.3, 12, 40, temp=(0.4, 16), mlp=_moe(5, 2, 24, shared=40)),
            _attn(4, 2, 16, 8, 0.2, 8, 21, temp=(0.2, 7), kv_from=0, mlp=_dense(48)),
            _mem(2, 12, 20, 8.0, mlp=_moe(3, 1, 32)),
            _attn(2, 2, 8, 24, 0.5, 16, 100, mlp=None),
            _mem(3, 8, 8, 15.0, mlp=_dense(40)),
        ],
    },
    # sizes that fit no fast path (a width that is no multiple of 4, heads of 6 and 10 elements, a value size that is
    # no multiple of 4, a prime vocabulary), one stream with its weights, one kv head, no query temperature, no
    # embedding scale, every expert chosen, a borrowed cache two layers back
    "MB": {
        "seed": 5, "architecture": "Mazotar", "vocab": 257, "width": 54, "norm": {"eps": 1e-3}, "streams": 1,
        "layers": [
            _mem(1, 10, 6, 5.0, mlp=_moe(2, 2, 20, shared=12)),
            _attn(3, 1, 6, 10, 0.6, 6, 9, mlp=_dense(28)),
            _mem(2, 7, 9, 20.0, mlp=None),
            _attn(3, 1, 6, 10, 0.4, 20, 300, temp=(1.0, 5), kv_from=1, mlp=_moe(4, 3, 18)),
        ],
    },
    # no streams at all: the plain residual sum
    "MC": {
        "seed": 7, "architecture": "Mazotar", "vocab": 128, "width": 32, "norm": {"eps": 1e-6},
        "embedding": {"scale": 2.0},
        "layers": [
            _mem(2, 8, 16, 12.0, mlp=_dense(48)),
            _attn(2, 1, 8, 8, 0.4, 10, 64, temp=(0.3, 32), mlp=_moe(4, 1, 16, shared=16)),
            _attn(2, 1, 8, 8, 0.35, 10, 50, kv_from=1, mlp=None),
        ],
    },
    # sharp scores: a key just where a page ends, or hundreds of tokens back, carries most of a query's weight
    "MS": {
        "seed": 13, "architecture": "Mazotar", "vocab": 128, "width": 32, "norm": {"eps": 1e-5}, "streams": 2,
        "layers": [
            _attn(2, 1, 16, 16, 1.5, 8, 30, temp=(0.5, 64), mlp=_dense(48)),
            _mem(2, 16, 16, 10.0, mlp=_dense(48)),
        ],
    },
}

# with the sizes the vector and matrix-core paths need (GPU tests)
MAZOTAR_FAST = {
    "MF": {
        "seed": 9, "architecture": "Mazotar", "vocab": 1000, "width": 256, "norm": {"eps": 1e-5}, "streams": 4,
        "embedding": {"scale": 0.8},
        "layers": [
            _mem(4, 32, 64, 11.0, mlp=_dense(384)),
            _attn(8, 2, 64, 64, 0.125, 32, 200, temp=(0.25, 96), mlp=_moe(8, 2, 128, shared=128)),
            _attn(4, 4, 128, 96, 0.09, 16, 90, temp=(0.2, 50), mlp=_moe(6, 1, 64, shared=192)),
            _attn(8, 2, 64, 64, 0.1, 64, 1000, kv_from=1, mlp=_dense(256)),
            _mem(2, 128, 128, 6.0, mlp=_moe(4, 1, 128)),
        ],
    },
    # values twice the keys' size at matrix-core head sizes, five query heads a kv head, a head of 32
    "MG": {
        "seed": 15, "architecture": "Mazotar", "vocab": 777, "width": 160, "norm": {"eps": 1e-6}, "streams": 2,
        "layers": [
            _attn(10, 2, 32, 64, 0.17, 24, 150, temp=(0.1, 10), mlp=_dense(288)),
            _mem(5, 24, 40, 9.0, mlp=_moe(5, 2, 64, shared=32)),
            _attn(5, 1, 96, 32, 0.1, 10, 33, mlp=_dense(200)),
        ],
    },
}


def mazotar_config_json(name: str) -> dict:
    return {k: v for k, v in {**MAZOTAR, **MAZOTAR_FAST}[name].items() if k != "seed"}


def write_mazotar(name: str, out_dir: str, dtype=torch.float32) -> str:
    from jax_llm_examples_amd.config import get_architecture
    from jax_llm_examples_amd.weights import write_random_model

    top = mazotar_config_json(name)
    arch = get_architecture(top["architecture"])
    return write_random_model(arch, arch.parse_config(top), out_dir, {**MAZOTAR, **MAZOTAR_FAST}[name]["seed"], dtype)
