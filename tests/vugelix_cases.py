"""Small Vugelix configurations, random weights for them and ways of cutting requests into steps, for the tests.

The configurations differ from each other in every size and option; among them are values that make two sizes equal
or 1 (one head, one tap, one stream, a window of one position, a window longer than any request), a layer without
feed-forward, no rotation and a rotation of the whole head, a model without stream coefficients, layers that run
another layer's weights with a cache and a state of their own, and layers of different sizes in one model. Weights are
drawn wide enough that attention is far from uniform, the cap on the scores bends them and the recurrent state matters;
they are stored in bfloat16, so runs in both element types read the same numbers.
"""
from __future__ import annotations

import json
import os

import torch

from pevazen_cases import in_portions, interleaved, peak_tokens, tokens, whole  # noqa: F401  (ways of cutting, shared)


def _left(heads, kv_heads, dim, vdim, window, rot_dims, base, scale, softcap):
    return {"dim": dim, "heads": heads, "kv_heads": kv_heads, "mask": {"size": window}, "rot": {"base": base, "dims": rot_dims},
            "scale": scale, "softcap": softcap, "vdim": vdim}


def _right(heads, kv_heads, dim, vdim, conv):
    return {"conv": conv, "dim": dim, "heads": heads, "kv_heads": kv_heads, "vdim": vdim}


def _layer(left, right, left_scale, right_scale, ff, **more):
    return dict({"type": "parallel", "mlp": None if ff is None else {"kind": "dense", "ff": ff},
                 "mixer": {"left": left, "left_scale": left_scale, "right": right, "right_scale": right_scale}}, **more)


_A0 = _layer(_left(4, 2, 8, 12, 6, 4, 50.0, 0.6, 3.0), _right(4, 2, 8, 6, 4), 0.7, 0.4, 56)
_A1 = _layer(_left(3, 1, 12, 4, 9, 12, 200.0, 0.4, 8.0), _right(3, 3, 5, 7, 2), 1.2, 0.8, None)
CONFIG_A = {
    "architecture": "Vugelix", "norm": {"eps": 1e-5}, "vocab": 97, "width": 40, "streams": 3,
    "embedding": {"scale": 3.0}, "logit_scale": 0.25,
    "layers": [_A0, _A1, dict(_A0, weights_of=0), _layer(_left(2, 2, 6, 6, 4, 6, 10.0, 0.5, 2.0), _right(2, 1, 4, 10, 3), 0.5, 0.5, 24),
               dict(_A1, weights_of=1)],
}

# sizes of one: one stream, one head, one tap, a window of one position, a window longer than any request, no rotation
_B0 = _layer(_left(1, 1, 10, 10, 1000, 0, 7.0, 0.7, 5.0), _right(1, 1, 3, 3, 1), 1.0, 1.0, 16)
CONFIG_B = {
    "architecture": "Vugelix", "norm": {"eps": 1e-6}, "vocab": 61, "width": 24, "streams": 1,
    "embedding": {"scale": 1.0}, "logit_scale": 1.0,
    "layers": [_B0, _layer(_left(1, 1, 4, 2, 1, 2, 30.0, 1.0, 1.0), _right(2, 1, 6, 2, 2), 0.3, 1.5, None),
               dict(_B0, weights_of=0), _layer(_left(6, 3, 16, 16, 8, 16, 10000.0, 0.25, 20.0), _right(2, 1, 16, 16, 3), 0.9, 0.2, 40)],
}

# no key 'streams': the plain pre-norm layer on one stream, without coefficients; no scales on embedding and logits
CONFIG_C = {
    "architecture": "Vugelix", "norm": {"eps": 1e-6}, "vocab": 50, "width": 32,
    "layers": [_layer(_left(4, 4, 8, 8, 5, 8, 100.0, 0.5, 4.0), _right(4, 4, 8, 8, 3), 0.5, 0.5, 48),
               _layer(_left(2, 1, 16, 8, 11, 4, 1000.0, 0.3, 6.0), _right(3, 1, 7, 5, 4), 0.8, 0.6, None)],
}

# sizes that the kernels on the matrix cores take (head sizes in steps of 16, equal for keys and values), with
# windows shorter and longer than a tile of keys
_R0 = _layer(_left(4, 2, 32, 32, 40, 16, 10000.0, 32 ** -0.5 * 2, 6.0), _right(2, 2, 64, 64, 4), 0.6, 0.5, 256)
CONFIG_R = {
    "architecture": "Vugelix", "norm": {"eps": 1e-6}, "vocab": 128, "width": 128, "streams": 2,
    "embedding": {"scale": 4.0}, "logit_scale": 0.5,
    "layers": [_R0, _layer(_left(8, 2, 16, 16, 24, 8, 500.0, 0.5, 10.0), _right(4, 1, 32, 16, 2), 0.4, 0.7, 256),
               dict(_R0, weights_of=0)],
}

# the same kinds of sizes with windows longer than a page of 64 tokens, one of them no multiple of it
_S0 = _layer(_left(4, 1, 32, 32, 96, 16, 10000.0, 0.3, 12.0), _right(4, 2, 32, 16, 4), 0.6, 0.5, 64)
CONFIG_S = {
    "architecture": "Vugelix", "norm": {"eps": 1e-6}, "vocab": 96, "width": 64, "streams": 4,
    "embedding": {"scale": 8.0}, "logit_scale": 0.5,
    "layers": [_S0, _layer(_left(2, 2, 48, 48, 160, 48, 1000.0, 0.25, 30.0), _right(2, 1, 32, 16, 4), 0.5, 0.6, None),
               dict(_S0, weights_of=0)],
}

# head sizes, state sizes and a width of the kind real models have (two layers and one run again)
_W0 = _layer(_left(8, 2, 128, 128, 200, 64, 10000.0, 128 ** -0.5 * 2, 20.0), _right(4, 2, 128, 128, 4), 0.6, 0.5, 2048)
CONFIG_W = {
    "architecture": "Vugelix", "norm": {"eps": 1e-6}, "vocab": 512, "width": 1024, "streams": 4,
    "embedding": {"scale": 32.0}, "logit_scale": 0.5,
    "layers": [_W0, _layer(_left(16, 4, 64, 64, 70, 64, 500000.0, 0.25, 50.0), _right(8, 8, 64, 128, 3), 0.5, 0.5, 3072),
               dict(_W0, weights_of=0)],
}

CASES = {"A": (CONFIG_A, 21), "B": (CONFIG_B, 32), "C": (CONFIG_C, 23), "R": (CONFIG_R, 24), "S": (CONFIG_S, 25)}


def random_tensors(config: dict, seed: int) -> dict[str, torch.Tensor]:
    """The stored tensors of a model of this configuration, by their names, in bfloat16."""
    gen = torch.Generator().manual_seed(seed)
    W = config["width"]
    n = config.get("streams")
    out = {}

    def normal(shape, std, mean=0.0):
        return mean + std * torch.randn(shape, generator=gen)

    def matrix(rows, cols, gain=1.0):
        return normal((rows, cols), gain / cols ** 0.5)

    out["embed"] = normal((config["vocab"], W), 1.0 / (config.get("embedding") or {}).get("scale", 1.0))
    out["final.norm"] = normal((W,), 0.1, 1.0)
    for i, layer in enumerate(config["layers"]):
        if "weights_of" in layer:
            continue
        p = f"l{i}."
        out[p + "norm1"] = normal((W,), 0.1, 1.1)
        a, r = layer["mixer"]["left"], layer["mixer"]["right"]
        H, G, D, E = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
        for name, rows in (("q", H * D), ("k", G * D), ("v", G * E)):
            out[p + "mix.left." + name] = matrix(rows, W, 3.0 if name != "v" else 1.0)
        out[p + "mix.left.g"] = matrix(H, W, 2.0)
        out[p + "mix.left.o"] = matrix(W, H * E)
        H, G, D, E, taps = r["heads"], r["kv_heads"], r["dim"], r["vdim"], r["conv"]
        for name, rows in (("q", G * D), ("k", G * D), ("v", H * E)):
            out[p + "mix.right." + name] = matrix(rows, W, 1.5)
            out[p + "mix.right." + name + ".conv"] = normal((rows, taps), 0.6)
        out[p + "mix.right.b"] = matrix(H, W, 2.0)
        out[p + "mix.right.a"] = matrix(H, W, 2.0)
        out[p + "mix.right.A_log"] = normal((H,), 0.5, -0.5)
        out[p + "mix.right.dt_bias"] = normal((H,), 1.0, -0.5)
        out[p + "mix.right.norm"] = normal((E,), 0.2, 1.0)
        out[p + "mix.right.g"] = matrix(H * E, W, 2.0)
        out[p + "mix.right.o"] = matrix(W, H * E)
        sublayers = ["hc1"]
        if layer.get("mlp") is not None:
            ff = layer["mlp"]["ff"]
            out[p + "norm2"] = normal((W,), 0.1, 0.9)
            out[p + "mlp.up"] = matrix(ff, W, 1.5)
            out[p + "mlp.down"] = matrix(W, ff, 1.0)
            sublayers.append("hc2")
        if n:
            for q in sublayers:
                out[p + q + ".in"] = normal((n,), 0.3 / n, 1.0 / n)
                out[p + q + ".out"] = normal((n,), 0.3, 0.8)
                out[p + q + ".mix"] = torch.eye(n) * 0.8 + normal((n, n), 0.3 / n, 0.2 / n)
    return {k: v.to(torch.bfloat16) for k, v in out.items()}


def write_model(folder: str, config: dict, seed: int, tensors: dict | None = None) -> str:
    from safetensors.torch import save_file

    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(config, f)
    tensors = random_tensors(config, seed) if tensors is None else tensors
    save_file({k: v.contiguous() for k, v in tensors.items()}, os.path.join(folder, "model.safetensors"))
    return folder


def random_config(seed: int) -> dict:
    """A configuration drawn at random (seeded): head sizes that the matrix-core kernels take and sizes that they do
    not, 1 to 20 query heads per key/value head, widths and vocabularies that are no multiple of 8, 1 to 8 streams or
    none, windows around the sizes of pages and tiles, layers that run earlier layers' weights in any order."""
    import random
    r = random.Random(seed)
    width = r.choice([24, 40, 52, 64, 72, 100])
    owners, layers = [], []
    for i in range(r.randint(2, 5)):
        if owners and r.random() < 0.4:
            j = r.choice(owners)
            layers.append(dict(layers[j], weights_of=j))
            continue
        kv = r.choice([1, 2, 3])
        group = r.choice([1, 2, 4, 5, 17, 20]) if kv == 1 else r.choice([1, 2, 3])
        dim = r.choice([8, 16, 20, 32, 48, 64])
        vdim = dim if r.random() < 0.6 else r.choice([4, 12, 16, 24])
        rot = r.choice([0, 2, dim // 2 // 2 * 2, dim])
        left = _left(kv * group, kv, dim, vdim, r.choice([1, 3, 15, 16, 17, 31, 32, 33, 63, 64, 65, 100, 500]), rot,
                     r.choice([10.0, 1000.0, 50000.0]), r.choice([0.5, 1.0, 2.0]) * dim ** -0.5, r.choice([2.0, 5.0, 30.0]))
        rkv = r.choice([1, 2])
        right = _right(rkv * r.choice([1, 2, 3]), rkv, r.choice([4, 7, 16, 32, 40]), r.choice([4, 6, 16, 32, 40]), r.choice([1, 2, 3, 4, 6]))
        owners.append(i)
        layers.append(_layer(left, right, r.choice([0.3, 0.6, 1.0]), r.choice([0.3, 0.5, 1.0]), r.choice([None, 24, 50, 64])))
    config = {"architecture": "Vugelix", "norm": {"eps": r.choice([1e-6, 1e-5, 1e-3])}, "vocab": r.choice([33, 64, 90, 131]),
              "width": width, "embedding": {"scale": r.choice([1.0, 4.0, 10.0])}, "logit_scale": r.choice([0.25, 1.0, 2.0]),
              "layers": layers}
    streams = r.choice([None, 1, 2, 3, 4, 8])
    if streams is not None:
        config["streams"] = streams
    return config
