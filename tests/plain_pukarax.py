"""The Pukarax decoder, plain and slow: whole sequences, no cache, no batch, one function per mechanism.

Written from the design's equations alone and sharing no code with the engine: its own reader of the model folder,
its own rotation, masks, routing. ``dtype`` is the float type everything is computed in (float64 by default).

The design in this file's notation (x the stream, h a sublayer's input, p a position counted from 0):

* x0 = E[token] * s_e.
* a layer: x += N1b(mixer(N1(x))); x += N2b(ff(N2(x))) with N(v) = v / sqrt(mean(v^2) + eps) * w; layers
  ``loop.start`` to ``loop.stop - 1`` are a group that is run ``loop.times`` times over, on one set of weights.
* mixer "attention" (two softmax maps per head, their difference): q and k hold per head [map 1 | map 2]; both
  maps are turned over their first ``rot.dims`` entries, pairs (2i, 2i + 1), angle p * base^(-2i / dims); the maps
  read the same values; lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + diff; o = a1 - lambda a2, divided by its root mean
  square over the value entries, times (1 - diff), times sigmoid(g_h . h) for head h; biases on q, k, v and o.
* mixer "attention_2": v = k as projected; q and k turned over their first ``rot.dims`` entries, pairs (i, i + dims/2),
  angle p * base^(-2i / dims) / factor, then divided by their root mean square per head; the concatenated heads are
  multiplied entry by entry with sigmoid(G h); no biases.
* both: scores q . k * scale; position i reads j <= i with floor(i / size) = floor(j / size); grouped key/value heads.
* feed-forward "dense": D(silu(G h) * (U h)). "moe": z = R h + b; the ``top`` largest z win (the lower number among
  equals), softmax(winners' z) weighs the winners' outputs, and a shared expert's output is added.
* logits = E N_f(x) * s_l.
"""
from __future__ import annotations

import json
import math
import os
import struct

import torch


def read_folder(folder: str) -> tuple[dict, dict]:
    """config.json and every tensor of model.safetensors (read by hand: 8 bytes of length, a JSON header, the data)."""
    with open(os.path.join(folder, "config.json")) as f:
        config = json.load(f)
    with open(os.path.join(folder, "model.safetensors"), "rb") as f:
        (n,) = struct.unpack("<Q", f.read(8))
        header = json.loads(f.read(n))
        data = f.read()
    kinds = {"BF16": torch.bfloat16, "F32": torch.float32, "I32": torch.int32, "F16": torch.float16}
    tensors = {}
    for name, entry in header.items():
        if name == "__metadata__":
            continue
        lo, hi = entry["data_offsets"]
        t = torch.frombuffer(bytearray(data[lo:hi]), dtype=kinds[entry["dtype"]]) if hi > lo else \
            torch.zeros(0, dtype=kinds[entry["dtype"]])
        tensors[name] = t.reshape(entry["shape"]).clone()
    return config, tensors


def rms_unit(v: torch.Tensor, eps: float) -> torch.Tensor:
    return v / torch.sqrt((v * v).mean(-1, keepdim=True) + eps)


def rms_norm(v: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    return rms_unit(v, eps) * w


def turn_interleaved(t: torch.Tensor, dims: int, base: float, positions: torch.Tensor) -> torch.Tensor:
    """t [n, heads, size]: pairs (2i, 2i + 1) of the first ``dims`` entries turn by position * base^(-2i / dims)."""
    if not dims:
        return t
    i = torch.arange(dims // 2, dtype=t.dtype)
    angle = positions.to(t.dtype)[:, None] * base ** (-2.0 * i / dims)[None, :]
    c, s = angle.cos()[:, None, :], angle.sin()[:, None, :]
    u, v = t[..., 0:dims:2], t[..., 1:dims:2]
    out = t.clone()
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


def turn_halves(t: torch.Tensor, dims: int, base: float, factor: float | None, positions: torch.Tensor) -> torch.Tensor:
    """t [n, heads, size]: pairs (i, i + dims / 2) of the first ``dims`` entries turn by position * f_i,
    f_i = base^(-2i / dims), divided by ``factor`` if there is one."""
    if not dims:
        return t
    half = dims // 2
    f = base ** (-2.0 * torch.arange(half, dtype=t.dtype) / dims)
    if factor is not None:
        f = f / factor
    angle = positions.to(t.dtype)[:, None] * f[None, :]
    c, s = angle.cos()[:, None, :], angle.sin()[:, None, :]
    u, v = t[..., :half], t[..., half:dims]
    out = t.clone()
    out[..., :half] = u * c - v * s
    out[..., half:dims] = v * c + u * s
    return out


def chunk_mask(n: int, size: int) -> torch.Tensor:
    """[n, n] True where query i reads key j: j <= i and both in the same block of ``size`` positions."""
    i = torch.arange(n)[:, None]
    j = torch.arange(n)[None, :]
    return (j <= i) & (i // size == j // size)


def softmax_read(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, mask: torch.Tensor) -> torch.Tensor:
    """q [n, H, d], k [n, G, d], v [n, G, e] -> [n, H, e]; query head h reads key/value head h // (H / G)."""
    H, G = q.shape[1], k.shape[1]
    out = []
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        s = s.masked_fill(~mask, -math.inf)
        out.append(torch.softmax(s, dim=-1) @ v[:, g])
    return torch.stack(out, dim=1)


def differential_attention(h: torch.Tensor, w: dict, m: dict, eps: float) -> torch.Tensor:
    n = h.shape[0]
    H, G, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    diff = m["diff"]
    q = (h @ w["q"].T + w["q.b"]).view(n, H, 2, d)
    k = (h @ w["k"].T + w["k.b"]).view(n, G, 2, d)
    v = (h @ w["v"].T + w["v.b"]).view(n, G, e)
    rot = m.get("rot") or {}
    pos = torch.arange(n)
    mask = chunk_mask(n, m["mask"]["size"]) if m.get("mask") else chunk_mask(n, n + 1)
    maps = []
    for c in range(2):
        qc = turn_interleaved(q[:, :, c], rot.get("dims", 0), rot.get("base", 1.0), pos)
        kc = turn_interleaved(k[:, :, c], rot.get("dims", 0), rot.get("base", 1.0), pos)
        maps.append(softmax_read(qc, kc, v, m["scale"], mask))
    lam = torch.exp((w["lq1"] * w["lk1"]).sum()) - torch.exp((w["lq2"] * w["lk2"]).sum()) + diff
    o = rms_unit(maps[0] - lam * maps[1], eps) * (1.0 - diff)
    gate = torch.sigmoid(h @ w["g"].T)                       # [n, H]
    o = o * gate[:, :, None]
    return o.reshape(n, H * e) @ w["o"].T + w["o.b"]


def keys_as_values_attention(h: torch.Tensor, w: dict, m: dict, eps: float) -> torch.Tensor:
    n = h.shape[0]
    H, G, d = m["heads"], m["kv_heads"], m["dim"]
    q = (h @ w["q"].T).view(n, H, d)
    k = (h @ w["k"].T).view(n, G, d)
    v = k
    rot = m.get("rot") or {}
    factor = (rot.get("scaling") or {}).get("factor")
    pos = torch.arange(n)
    q = rms_unit(turn_halves(q, rot.get("dims", 0), rot.get("base", 1.0), factor, pos), eps)
    k = rms_unit(turn_halves(k, rot.get("dims", 0), rot.get("base", 1.0), factor, pos), eps)
    mask = chunk_mask(n, m["mask"]["size"]) if m.get("mask") else chunk_mask(n, n + 1)
    o = softmax_read(q, k, v, m["scale"], mask).reshape(n, H * d)
    return (o * torch.sigmoid(h @ w["g"].T)) @ w["o"].T


def gated_ff(h: torch.Tensor, w: dict, prefix: str) -> torch.Tensor:
    g = h @ w[prefix + "gate"].T
    return ((g * torch.sigmoid(g)) * (h @ w[prefix + "up"].T)) @ w[prefix + "down"].T


def mixture(h: torch.Tensor, w: dict, mlp: dict) -> torch.Tensor:
    experts, top = mlp["router"]["experts"], mlp["router"]["top"]
    z = h @ w["router"].T + w["router.b"]
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        order = sorted(range(experts), key=lambda e: (-float(z[t, e]), e))[:top]
        weights = torch.softmax(z[t, order], dim=-1)
        for wt, e in zip(weights, order):
            out[t] += wt * gated_ff(h[t:t + 1], w, f"e{e}.")[0]
    if mlp.get("shared"):
        out = out + gated_ff(h, w, "shared.")
    return out


def run_order(config: dict) -> list[int]:
    n = len(config["layers"])
    loop = config.get("loop")
    if not loop:
        return list(range(n))
    start, stop, times = loop["start"], loop["stop"], loop["times"]
    return list(range(start)) + list(range(start, stop)) * times + list(range(stop, n))


def forward(config: dict, tensors: dict, tokens, dtype=torch.float64, streams: list | None = None) -> torch.Tensor:
    """Logits [len(tokens), vocab]. ``streams``, if a list, receives the stream after every layer run."""
    W = {k: v.to(dtype) for k, v in tensors.items()}
    eps = config["norm"]["eps"]
    x = W["embed"][torch.tensor(tokens)] * config["embedding"]["scale"]
    for i in run_order(config):
        layer = config["layers"][i]
        own = {k[len(f"l{i}."):]: v for k, v in W.items() if k.startswith(f"l{i}.")}
        mix = {k[len("mix."):]: v for k, v in own.items() if k.startswith("mix.")}
        h = rms_norm(x, own["norm1"], eps)
        if layer["type"] == "attention":
            y = differential_attention(h, mix, layer["mixer"], eps)
        elif layer["type"] == "attention_2":
            y = keys_as_values_attention(h, mix, layer["mixer"], eps)
        else:
            raise ValueError(layer["type"])
        x = x + rms_norm(y, own["norm1b"], eps)
        mlp = layer.get("mlp")
        if mlp is not None:
            ff = {k[len("mlp."):]: v for k, v in own.items() if k.startswith("mlp.")}
            h = rms_norm(x, own["norm2"], eps)
            y = gated_ff(h, ff, "") if mlp["kind"] == "dense" else mixture(h, ff, mlp)
            x = x + rms_norm(y, own["norm2b"], eps)
        if streams is not None:
            streams.append(x.clone())
    return (rms_norm(x, W["final.norm"], eps) @ W["embed"].T) * config["logit_scale"]


def greedy_generate(config: dict, tensors: dict, prompt, n: int, dtype=torch.float64) -> list[int]:
    """The ``n`` tokens that follow ``prompt`` when the most likely token is taken each time (the whole sequence is
    computed anew for every token)."""
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(forward(config, tensors, toks, dtype)[-1].argmax()))
    return toks[len(prompt):]
