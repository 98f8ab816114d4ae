"""Plain, slow, whole-sequence Vugelix decoder on the CPU: the oracle of the tests of this design.

No cache, no batching, no kernels and no code of the package: every function takes a whole sequence and writes
one mechanism out as loops and small tensor expressions. ``logits(config, tensors, tokens)`` runs a model
folder's contents (``read_model_folder``); ``dtype`` may be ``torch.float64`` for a sharper oracle.

Notation: T tokens, W the model's width, H query (or value) heads, G key heads, D the query/key head size, E the
value head size, n the number of streams, p a token's index in its sequence.
"""
from __future__ import annotations

import json
import math
import os

import torch


def read_model_folder(folder: str):
    """config.json as a dict and every tensor of model.safetensors (floats as float32)."""
    from safetensors import safe_open

    with open(os.path.join(folder, "config.json")) as f:
        config = json.load(f)
    tensors = {}
    with safe_open(os.path.join(folder, "model.safetensors"), framework="pt", device="cpu") as f:
        for name in f.keys():
            t = f.get_tensor(name)
            tensors[name] = t.to(torch.float32) if t.is_floating_point() else t
    return config, tensors


# ------------------------------------------------------------------ small pieces
def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """x over its root mean square along the last axis (eps under the root), times a weight per coordinate."""
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps) * weight


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 20, z, torch.log1p(torch.exp(torch.clamp(z, max=20.0))))


def squared_relu(z):
    return torch.relu(z) ** 2


def turn_first_dims(x: torch.Tensor, dims: int, base: float) -> torch.Tensor:
    """x[T, heads, size]: among the first ``dims`` coordinates of every head, coordinate i < dims / 2 and coordinate
    i + dims / 2 are one pair (a, b), which at position p becomes (a cos t - b sin t, b cos t + a sin t) with
    t = p base^(-2 i / dims). The other coordinates pass."""
    if not dims:
        return x
    T, r = x.shape[0], dims // 2
    f = float(base) ** (-2.0 * torch.arange(r, dtype=x.dtype) / dims)
    t = torch.arange(T, dtype=x.dtype)[:, None] * f[None, :]
    cos, sin = t.cos()[:, None, :], t.sin()[:, None, :]
    a, b = x[..., :r], x[..., r:dims]
    return torch.cat((a * cos - b * sin, b * cos + a * sin, x[..., dims:]), dim=-1)


def window_mask(T: int, size: int | None) -> torch.Tensor:
    """[T, T] bool: query i sees key j iff 0 <= i - j < size (``None``: every j <= i)."""
    d = torch.arange(T)[:, None] - torch.arange(T)[None, :]
    return (d >= 0) if size is None else (d >= 0) & (d < size)


def sink_attention(q, k, v, scale: float, cap: float | None, visible: torch.Tensor) -> torch.Tensor:
    """q[T, H, D], k[T, G, D], v[T, G, E] -> [T, H, E]. The score q . k times ``scale`` is squashed into (-cap, cap)
    by cap tanh(s / cap) where a cap is given; the weights are exp(s_j) / (1 + sum of exp(s_j) over the visible keys):
    one more term of score 0 stands in the denominator and brings no value."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[-1], dtype=q.dtype)
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        if cap is not None:
            s = cap * torch.tanh(s / cap)
        e = torch.exp(s).masked_fill(~visible, 0.0)
        out[:, h] = (e / (1.0 + e.sum(-1, keepdim=True))) @ v[:, g]
    return out


def causal_taps(x: torch.Tensor, taps: torch.Tensor) -> torch.Tensor:
    """x[T, C], taps[C, n]: y[t, c] = sum_j taps[c, j] x[t - (n - 1 - j), c], zeros before the start."""
    T, n = x.shape[0], taps.shape[1]
    y = torch.zeros_like(x)
    for t in range(T):
        for j in range(n):
            s = t - (n - 1 - j)
            if s >= 0:
                y[t] += taps[:, j] * x[s]
    return y


def delta_recurrence(q, k, v, decay, beta):
    """Per head, token by token, with a state S[D, E] that starts at zero:
        S <- decay_t S;  u = beta_t (v_t - S^T k_t);  S <- S + k_t u^T;  o_t = S^T q_t.
    q, k: [T, H, D]; v: [T, H, E]; decay, beta: [T, H] (one number per head and token). Returns o [T, H, E]."""
    T, H, D = q.shape
    E = v.shape[-1]
    out = torch.zeros(T, H, E, dtype=q.dtype)
    for h in range(H):
        S = torch.zeros(D, E, dtype=q.dtype)
        for t in range(T):
            S = decay[t, h] * S
            u = beta[t, h] * (v[t, h] - S.T @ k[t, h])
            S = S + torch.outer(k[t, h], u)
            out[t, h] = S.T @ q[t, h]
    return out


# ------------------------------------------------------------------ mixers
def left_mixer(x, w, prefix, m):
    """The attention half: grouped heads, rotation of the first coordinates, capped scores, a window, the extra term
    in the denominator, a gate per head from the mixer's input. ``m``: its entry of config.json."""
    T = x.shape[0]
    H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    rot = m.get("rot") or {"dims": 0, "base": 1.0}
    q = turn_first_dims((x @ w[prefix + "q"].T).view(T, H, D), rot["dims"], rot["base"])
    k = turn_first_dims((x @ w[prefix + "k"].T).view(T, G, D), rot["dims"], rot["base"])
    v = (x @ w[prefix + "v"].T).view(T, G, E)
    size = (m.get("mask") or {}).get("size")
    o = sink_attention(q, k, v, m["scale"], m.get("softcap"), window_mask(T, size))
    o = o * torch.sigmoid(x @ w[prefix + "g"].T)[:, :, None]
    return o.reshape(T, H * E) @ w[prefix + "o"].T


def right_mixer(x, w, prefix, m, eps):
    """The recurrent half. ``m``: its entry of config.json (heads, kv_heads, dim, vdim, conv)."""
    T = x.shape[0]
    H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]

    def short(name):
        return silu(causal_taps(x @ w[prefix + name].T, w[prefix + name + ".conv"]))

    def unit(z):
        return z / torch.sqrt(z.pow(2).sum(-1, keepdim=True) + 1e-6)

    rep = H // G
    q = unit(short("q").view(T, G, D)).repeat_interleave(rep, dim=1) * D ** -0.5
    k = unit(short("k").view(T, G, D)).repeat_interleave(rep, dim=1)
    v = short("v").view(T, H, E)
    beta = torch.sigmoid(x @ w[prefix + "b"].T)                                                   # [T, H]
    decay = torch.exp(-torch.exp(w[prefix + "A_log"]) * softplus(x @ w[prefix + "a"].T + w[prefix + "dt_bias"]))
    o = delta_recurrence(q, k, v, decay, beta)
    o = rms_norm(o, w[prefix + "norm"], eps) * silu(x @ w[prefix + "g"].T).view(T, H, E)
    return o.reshape(T, H * E) @ w[prefix + "o"].T


def parallel_mixer(x, w, prefix, m, eps):
    return m["left_scale"] * left_mixer(x, w, prefix + "left.", m["left"]) + \
        m["right_scale"] * right_mixer(x, w, prefix + "right.", m["right"], eps)


def dense_feed_forward(x, w, prefix):
    return squared_relu(x @ w[prefix + "up"].T) @ w[prefix + "down"].T


# ------------------------------------------------------------------ the streams
def sublayer_on_streams(X, w, prefix, norm_weight, eps, fn):
    """X[n, T, W]: the sublayer reads sum_s in[s] X_s through its norm; then, all at once from the old streams,
    X_t <- sum_s mix[s, t] X_s + out[t] y."""
    u = torch.einsum("s,stw->tw", w[prefix + "in"], X)
    y = fn(rms_norm(u, norm_weight, eps))
    return torch.einsum("sr,stw->rtw", w[prefix + "mix"], X) + w[prefix + "out"][:, None, None] * y[None]


# ------------------------------------------------------------------ the model
def hidden_states(config: dict, tensors: dict, tokens, dtype=torch.float32) -> list[torch.Tensor]:
    """[the embedding's output, the stream (the sum of the streams, where there are several) after every layer run],
    each [T, W]."""
    w = {k: (t.to(dtype) if t.is_floating_point() else t) for k, t in tensors.items()}
    eps = config["norm"]["eps"]
    x = w["embed"][torch.as_tensor(tokens, dtype=torch.long)] * (config.get("embedding") or {}).get("scale", 1.0)
    n = config.get("streams")
    X = x[None].repeat(n, 1, 1) if n else x
    out = [x]
    for i, layer in enumerate(config["layers"]):
        p = f"l{layer.get('weights_of', i)}."
        if layer["type"] != "parallel":
            raise ValueError(f"layer {i}: unknown type {layer['type']!r}")
        mix = lambda z: parallel_mixer(z, w, p + "mix.", layer["mixer"], eps)      # noqa: E731
        ff = None
        if layer.get("mlp") is not None:
            if layer["mlp"]["kind"] != "dense":
                raise ValueError(f"layer {i}: unknown feed-forward kind")
            ff = lambda z: dense_feed_forward(z, w, p + "mlp.")                   # noqa: E731
        if n:
            X = sublayer_on_streams(X, w, p + "hc1.", w[p + "norm1"], eps, mix)
            if ff is not None:
                X = sublayer_on_streams(X, w, p + "hc2.", w[p + "norm2"], eps, ff)
            out.append(X.sum(0))
        else:
            X = X + mix(rms_norm(X, w[p + "norm1"], eps))
            if ff is not None:
                X = X + ff(rms_norm(X, w[p + "norm2"], eps))
            out.append(X)
    return out


def logits(config: dict, tensors: dict, tokens, dtype=torch.float32) -> torch.Tensor:
    """[T, vocab]: the last norm, then the embedding table itself as the head, times ``logit_scale``."""
    x = hidden_states(config, tensors, tokens, dtype)[-1]
    x = rms_norm(x, tensors["final.norm"].to(dtype), config["norm"]["eps"])
    return x @ tensors["embed"].to(dtype).T * config.get("logit_scale", 1.0)


def greedy_generate(config, tensors, prompt, n: int) -> list[int]:
    ids = list(prompt)
    for _ in range(n):
        ids.append(int(logits(config, tensors, ids)[-1].argmax()))
    return ids[len(prompt):]
