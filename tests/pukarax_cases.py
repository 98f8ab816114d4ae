"""Small Pukarax configurations, random weights for them and ways of cutting requests into steps, for the tests.

The configurations differ from each other in every size and option; among them are values that make two sizes equal
or 1 (one head, one expert, all experts chosen, a chunk of one position, a chunk longer than any request, value heads
of the key heads' size and of another), layers without feed-forward, no rotation, a partial and a whole rotation,
loops at the start, in the middle and over all layers, and none. Weights are drawn wide enough that attention is far
from uniform and the router's choices are clear; they are stored in bfloat16, so runs in both element types read the
same numbers.
"""
from __future__ import annotations

import json
import os

import torch

from pevazen_cases import in_portions, interleaved, peak_tokens, tokens, whole  # noqa: F401  (ways of cutting, shared)


def two_maps(heads, kv_heads, dim, vdim, chunk, rot_dims, base, scale, diff):
    m = {"diff": diff, "dim": dim, "heads": heads, "kv_heads": kv_heads, "mask": {"size": chunk}, "scale": scale, "vdim": vdim}
    if rot_dims:
        m["rot"] = {"base": base, "dims": rot_dims}
    return {"type": "attention", "mixer": m}


def keys_as_values(heads, kv_heads, dim, chunk, rot_dims, base, factor, scale):
    m = {"dim": dim, "heads": heads, "kv_heads": kv_heads, "mask": {"size": chunk}, "scale": scale, "vdim": dim}
    if rot_dims:
        m["rot"] = {"base": base, "dims": rot_dims}
        if factor is not None:
            m["rot"]["scaling"] = {"factor": factor}
    return {"type": "attention_2", "mixer": m}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, shared=None):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top},
            "shared": {"ff": shared} if shared else None}


def model(vocab, width, eps, embed_scale, logit_scale, layers, loop=None):
    cfg = {"architecture": "Pukarax", "embedding": {"scale": embed_scale}, "layers": layers, "logit_scale": logit_scale,
           "norm": {"eps": eps}, "vocab": vocab, "width": width}
    if loop is not None:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg


def _with(entry, mlp):
    return dict(entry, mlp=mlp)


# width a multiple of 8; a loop in the middle; a layer without feed-forward; partial rotations; experts with and without a shared one
CONFIG_A = model(67, 40, 1e-5, 3.0, 0.5, [
    _with(keys_as_values(4, 2, 8, 6, 4, 100.0, 2.0, 0.6), dense(24)),
    _with(two_maps(2, 1, 6, 10, 5, 6, 1000.0, 0.5, 0.3), moe(5, 2, 12, 16)),
    _with(keys_as_values(2, 2, 12, 9, 12, 50.0, None, 0.4), None),
    _with(two_maps(4, 2, 4, 4, 7, 2, 10.0, 0.7, 0.6), moe(3, 1, 8)),
], loop=(1, 3, 3))
# a width that is no multiple of 8, one head, one expert, all experts chosen, a chunk of one position and one longer than any
# request, no rotation, no loop
CONFIG_B = model(50, 36, 1e-3, 1.0, 2.0, [
    _with(two_maps(1, 1, 8, 3, 1000, 0, 1.0, 0.35, 0.8), moe(1, 1, 10, 6)),
    _with(keys_as_values(1, 1, 10, 1, 10, 20.0, 4.0, 0.3), moe(4, 4, 6)),
    _with(keys_as_values(3, 1, 6, 1000, 0, 1.0, None, 0.5), dense(20)),
    _with(two_maps(3, 3, 2, 5, 1, 2, 7.0, 1.0, 0.1), None),
])
# head sizes that the kernels on the matrix cores take (and one that they do not), a loop over all layers
CONFIG_C = model(90, 64, 2e-6, 8.0, 0.2, [
    _with(keys_as_values(4, 2, 16, 11, 8, 10000.0, 16.0, 0.25), moe(6, 3, 16, 24)),
    _with(two_maps(2, 2, 16, 32, 13, 16, 300000.0, 0.25, 0.35), dense(40)),
    _with(two_maps(4, 1, 32, 16, 20, 8, 300.0, 0.2, 0.45), moe(8, 2, 8, 8)),
], loop=(0, 3, 2))
# recorded steps: a loop at the start
CONFIG_R = model(40, 32, 1e-5, 2.0, 1.0, [
    _with(two_maps(2, 1, 16, 16, 8, 8, 100.0, 0.3, 0.45), moe(4, 2, 8, 8)),
    _with(keys_as_values(2, 1, 16, 12, 16, 1000.0, 2.0, 0.3), dense(16)),
], loop=(0, 1, 2))
# the same kinds of sizes with chunks longer than a page of 64 tokens, one of them no multiple of it
CONFIG_S = model(120, 64, 1e-6, 4.0, 0.5, [
    _with(keys_as_values(4, 2, 32, 150, 32, 20000.0, 4.0, 0.18), moe(6, 2, 16, 32)),
    _with(two_maps(2, 1, 32, 64, 80, 32, 300000.0, 0.18, 0.55), dense(48)),
    _with(two_maps(2, 2, 16, 48, 128, 16, 300000.0, 0.25, 0.4), moe(4, 2, 16)),
], loop=(0, 2, 2))
# the sizes of a real model's layers in small number: heads of 128 and 64, a width of 1,024
CONFIG_W = model(500, 1024, 1e-6, 32.0, 0.1, [
    _with(keys_as_values(8, 2, 128, 256, 128, 20000.0, 4.0, 0.09), moe(8, 2, 256, 512)),
    _with(two_maps(8, 4, 64, 128, 192, 64, 300000.0, 0.125, 0.6), dense(2048)),
])

CASES = {"A": (CONFIG_A, 31), "B": (CONFIG_B, 42), "C": (CONFIG_C, 33), "R": (CONFIG_R, 34), "S": (CONFIG_S, 35)}


def random_tensors(config: dict, seed: int) -> dict[str, torch.Tensor]:
    g = torch.Generator().manual_seed(seed)
    W = config["width"]
    out = {}

    def normal(shape, std, mean=0.0):
        return mean + std * torch.randn(shape, generator=g)

    def matrix(rows, cols, gain=1.0):
        return normal((rows, cols), gain / cols ** 0.5)

    def gated(prefix, ff):
        out[prefix + "gate"] = matrix(ff, W, 1.5)
        out[prefix + "up"] = matrix(ff, W, 1.5)
        out[prefix + "down"] = matrix(W, ff)

    out["embed"] = normal((config["vocab"], W), 1.0 / config["embedding"]["scale"])
    out["final.norm"] = normal((W,), 0.1, 1.0)
    for i, layer in enumerate(config["layers"]):
        p = f"l{i}."
        m = layer["mixer"]
        H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        out[p + "norm1"] = normal((W,), 0.1, 1.1)
        out[p + "norm1b"] = normal((W,), 0.1, 0.6)
        if layer["type"] == "attention":
            out[p + "mix.q"] = matrix(2 * H * D, W, 3.0)
            out[p + "mix.k"] = matrix(2 * G * D, W, 3.0)
            out[p + "mix.v"] = matrix(G * E, W)
            out[p + "mix.g"] = matrix(H, W, 2.0)
            for name, n in (("q", 2 * H * D), ("k", 2 * G * D), ("v", G * E)):
                out[p + f"mix.{name}.b"] = normal((n,), 0.3)
            out[p + "mix.o.b"] = normal((W,), 0.2)
            for name in ("lq1", "lk1", "lq2", "lk2"):
                out[p + "mix." + name] = normal((D,), 0.6 / D ** 0.5)      # (lambda stays within about 0.2 of ``diff``)
        else:
            out[p + "mix.q"] = matrix(H * D, W, 3.0)
            out[p + "mix.k"] = matrix(G * D, W, 3.0)
            out[p + "mix.g"] = matrix(H * E, W, 2.0)
        out[p + "mix.o"] = matrix(W, H * E)
        mlp = layer.get("mlp")
        if mlp is None:
            continue
        out[p + "norm2"] = normal((W,), 0.1, 0.9)
        out[p + "norm2b"] = normal((W,), 0.1, 0.7)
        if mlp["kind"] == "dense":
            gated(p + "mlp.", mlp["ff"])
            continue
        n = mlp["router"]["experts"]
        out[p + "mlp.router"] = matrix(n, W, 4.0)
        out[p + "mlp.router.b"] = normal((n,), 0.5)
        for e in range(n):
            gated(p + f"mlp.e{e}.", mlp["expert"]["ff"])
        if mlp.get("shared"):
            gated(p + "mlp.shared.", mlp["shared"]["ff"])
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
    not, 1 to 6 query heads per key/value head, widths and vocabularies that are no multiple of 8, chunks around the
    sizes of pages and tiles, any order of the two kinds of layer, any loop."""
    import random
    r = random.Random(seed)
    width = r.choice([24, 40, 52, 64, 72, 100])
    layers = []
    for _ in range(r.randint(2, 5)):
        kv = r.choice([1, 2, 3])
        heads = kv * r.choice([1, 2, 3, 6])
        dim = r.choice([4, 8, 16, 20, 32, 48])
        chunk = r.choice([1, 3, 15, 16, 17, 31, 32, 33, 63, 64, 65, 100, 500])
        rot = r.choice([0, 2, dim // 2 // 2 * 2, dim])
        scale = r.choice([0.5, 1.0, 2.0]) * dim ** -0.5
        if r.random() < 0.5:
            vdim = 2 * dim if r.random() < 0.5 else r.choice([4, 12, 16, 24, dim])
            entry = two_maps(heads, kv, dim, vdim, chunk, rot, r.choice([10.0, 1000.0, 300000.0]), scale, r.choice([0.2, 0.4, 0.8]))
        else:
            entry = keys_as_values(heads, kv, dim, chunk, rot, r.choice([10.0, 1000.0, 20000.0]), r.choice([None, 2.0, 16.0]), scale)
        kind = r.choice(["none", "dense", "moe", "moe"])
        if kind == "dense":
            entry["mlp"] = dense(r.choice([16, 24, 50]))
        elif kind == "moe":
            n = r.choice([1, 2, 5, 9])
            entry["mlp"] = moe(n, r.randint(1, min(n, 4)), r.choice([6, 8, 16, 24]), r.choice([None, 8, 20]))
        else:
            entry["mlp"] = None
        layers.append(entry)
    loop = None
    if r.random() < 0.7:
        start = r.randint(0, len(layers) - 1)
        loop = (start, r.randint(start, len(layers)), r.randint(1, 3))
    return model(r.choice([33, 64, 90, 131]), width, r.choice([1e-6, 1e-5, 1e-3]), r.choice([1.0, 4.0, 10.0]),
                 r.choice([0.3, 1.0, 2.0]), layers, loop)
