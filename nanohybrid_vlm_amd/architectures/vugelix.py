"""The Vugelix decoder as a recipe of parts.

config.json: {"architecture": "Vugelix", "vocab", "width", "norm": {"eps"}, "embedding": {"scale"}, "logit_scale",
"streams", "layers": [...]}. Every entry of ``layers`` has ``type`` "parallel", the sizes of its mixer (``mixer``) and
its feed-forward (``mlp``: {"kind": "dense", "ff"} or null). An entry with ``weights_of: j`` has no tensors: it runs
layer j's weights (mixer, feed-forward, norms, stream coefficients) with a cache and a state of its own.

* the mixer is two mixers side by side on the same rows, ``left_scale`` times the left result plus ``right_scale``
  times the right one. ``left``: softmax attention with grouped key/value heads, rotation of the first ``rot.dims``
  coordinates of every query and key head (pairs (i, i + dims / 2), ``rot.base``), ``scale``, scores squashed by
  ``softcap``, a window of ``mask.size`` positions, one more term of score 0 in the softmax's denominator, and a
  sigmoid gate per head on the result. ``right``: a gated delta rule with short convolutions of ``conv`` taps, grouped
  query/key heads, one decay per head and a SiLU gate on its normed read-out.
* the feed-forward is down(relu(up(x))^2).
* the layer is pre-norm on ``streams`` residual streams with learned coefficients (``l<i>.hc1.*`` for the mixer,
  ``l<i>.hc2.*`` for the feed-forward); without the key ``streams`` it is the plain pre-norm layer on one stream.

The embedding's rows are multiplied by ``embedding.scale``; the head is the embedding table (unscaled) and the logits
are multiplied by ``logit_scale``.

Nothing here computes: ``parse_config`` checks and types the keys, ``build_spec`` turns them into a ``ModelSpec``,
``checkpoint_names`` places the stored tensors in the model's (packed) parameters.
"""
from __future__ import annotations

from dataclasses import dataclass, field

from ..config.model_config import ConfigError, require
from ..config.registry import Architecture, WeightSource, register_architecture
from ..parts.model import LayerSpec, ModelSpec, RunEntry

# positions are counted in float32 by the kernels that turn queries and keys: every integer up to here is exact
MAX_POSITION = 1 << 24
# the score of the softmax's extra term: exp(0) = 1 is added to every denominator
SINK_SCORE = 0.0


@dataclass(frozen=True)
class AttentionSizes:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int | None
    softcap: float | None
    rot_dims: int
    rot_base: float


@dataclass(frozen=True)
class DeltaSizes:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int


@dataclass(frozen=True)
class LayerSizes:
    attention: AttentionSizes
    delta: DeltaSizes
    left_scale: float
    right_scale: float
    ff: int | None = None                   # inner size of the feed-forward; None: the layer has none
    weights_of: int | None = None           # the layer (index in config.json) whose weights this one runs


@dataclass(frozen=True)
class VugelixConfig:
    vocab: int
    width: int
    eps: float
    layers: tuple
    streams: int | None = None              # None: one stream without coefficients
    embed_scale: float = 1.0
    logit_scale: float = 1.0
    max_position: int = MAX_POSITION
    raw: dict = field(default_factory=dict, compare=False, repr=False)

    def owners(self) -> list[int]:
        """Config indices of the layers that have tensors of their own, in order."""
        return [i for i, layer in enumerate(self.layers) if layer.weights_of is None]


def _where(i: int, key: str) -> str:
    return f"config.json: layers[{i}].{key}"


def _attention(i: int, m: dict) -> AttentionSizes:
    where = _where(i, "mixer.left")
    rot = m.get("rot") or {}
    mask = m.get("mask") or {}
    dims = require(rot, "dims") if rot else 0
    a = AttentionSizes(heads=require(m, "heads"), kv_heads=require(m, "kv_heads"), dim=require(m, "dim"),
                       vdim=require(m, "vdim"), scale=require(m, "scale", float),
                       window=require(mask, "size") if mask else None,
                       softcap=require(m, "softcap", float) if m.get("softcap") is not None else None,
                       rot_dims=dims, rot_base=require(rot, "base", float) if dims else 1.0)
    if min(a.heads, a.kv_heads, a.dim, a.vdim) <= 0 or a.heads % a.kv_heads:
        raise ConfigError(f"{where}: sizes must be positive and heads a multiple of kv_heads")
    if a.window is not None and a.window <= 0:
        raise ConfigError(f"{where}.mask.size must be positive")
    if a.softcap is not None and not a.softcap > 0:
        raise ConfigError(f"{where}.softcap must be positive")
    if a.rot_dims < 0 or a.rot_dims % 2 or a.rot_dims > a.dim:
        raise ConfigError(f"{where}: rot.dims {a.rot_dims} must be even and at most dim {a.dim}")
    if a.rot_dims and not a.rot_base > 0:
        raise ConfigError(f"{where}.rot.base must be positive")
    return a


def _delta(i: int, r: dict) -> DeltaSizes:
    d = DeltaSizes(heads=require(r, "heads"), kv_heads=require(r, "kv_heads"), dim=require(r, "dim"),
                   vdim=require(r, "vdim"), conv=require(r, "conv"))
    if min(d.heads, d.kv_heads, d.dim, d.vdim) <= 0 or d.heads % d.kv_heads:
        raise ConfigError(f"{_where(i, 'mixer.right')}: sizes must be positive and heads a multiple of kv_heads")
    if not 1 <= d.conv <= 16:
        raise ConfigError(f"{_where(i, 'mixer.right.conv')}: 1 to 16 taps are taken, got {d.conv}")
    return d


def parse_config(raw: dict) -> VugelixConfig:
    eps = require(raw.get("norm") or {}, "eps", float)
    if not eps > 0:
        raise ConfigError("config.json: norm.eps must be positive")
    entries = raw.get("layers")
    if not isinstance(entries, list) or not entries:
        raise ConfigError("config.json: 'layers' must be a list with at least one layer")
    layers = []
    for i, entry in enumerate(entries):
        kind, m = entry.get("type"), entry.get("mixer")
        if kind != "parallel":
            raise ConfigError(f"{_where(i, 'type')}: {kind!r} is not known ('parallel' is)")
        if not isinstance(m, dict) or not isinstance(m.get("left"), dict) or not isinstance(m.get("right"), dict):
            raise ConfigError(f"{_where(i, 'mixer')}: 'left' and 'right' are needed")
        mlp = entry.get("mlp")
        ff = None
        if mlp is not None:
            if mlp.get("kind") != "dense":
                raise ConfigError(f"{_where(i, 'mlp.kind')}: {mlp.get('kind')!r} is not known ('dense' is)")
            ff = require(mlp, "ff")
            if ff <= 0:
                raise ConfigError(f"{_where(i, 'mlp.ff')} must be positive")
        layer = LayerSizes(_attention(i, m["left"]), _delta(i, m["right"]),
                           left_scale=float(m["left_scale"]) if m.get("left_scale") is not None else 1.0,
                           right_scale=float(m["right_scale"]) if m.get("right_scale") is not None else 1.0,
                           ff=ff, weights_of=entry.get("weights_of"))
        j = layer.weights_of
        if j is not None:
            if not isinstance(j, int) or isinstance(j, bool) or not 0 <= j < i or layers[j].weights_of is not None:
                raise ConfigError(f"{_where(i, 'weights_of')}: {j!r} must name an earlier layer with tensors of its own")
            theirs = layers[j]
            if (layer.attention, layer.delta, layer.left_scale, layer.right_scale, layer.ff) != \
                    (theirs.attention, theirs.delta, theirs.left_scale, theirs.right_scale, theirs.ff):
                raise ConfigError(f"{_where(i, 'weights_of')}: the entry must equal layer {j}'s, whose weights it runs")
        layers.append(layer)
    streams = raw.get("streams")
    if streams is not None and (not isinstance(streams, int) or isinstance(streams, bool) or not 1 <= streams <= 16):
        raise ConfigError(f"config.json: 'streams' must be 1 to 16, got {streams!r}")
    embedding = raw.get("embedding") or {}
    cfg = VugelixConfig(vocab=require(raw, "vocab"), width=require(raw, "width"), eps=eps, layers=tuple(layers),
                        streams=streams,
                        embed_scale=float(embedding["scale"]) if embedding.get("scale") is not None else 1.0,
                        logit_scale=float(raw["logit_scale"]) if raw.get("logit_scale") is not None else 1.0,
                        max_position=min(int(raw.get("max_position") or MAX_POSITION), MAX_POSITION), raw=dict(raw))
    if cfg.vocab <= 0 or cfg.width <= 0:
        raise ConfigError("config.json: 'vocab' and 'width' must be positive")
    return cfg


def build_spec(cfg: VugelixConfig) -> ModelSpec:
    norm = {"kind": "stream_rmsnorm", "size": cfg.width, "eps": cfg.eps}
    block = {"kind": "stream_mix", "streams": cfg.streams or 1, "learned": cfg.streams is not None}
    layers, positions, index = [], {}, {}
    for i in cfg.owners():
        layer = cfg.layers[i]
        a, d = layer.attention, layer.delta
        positions[f"l{i}"] = {"kind": "rotary_frequencies", "rotary_dim": a.rot_dims, "base": a.rot_base}
        mixer = {"kind": "scaled_pair", "left_scale": layer.left_scale, "right_scale": layer.right_scale,
                 "left": {"kind": "rotary_attention", "hidden_size": cfg.width, "num_heads": a.heads,
                          "num_kv_heads": a.kv_heads, "head_dim": a.dim, "value_dim": a.vdim, "scale": a.scale,
                          "bias": False, "window": a.window, "softcap": a.softcap, "sink": SINK_SCORE, "head_gate": True},
                 "right": {"kind": "gated_delta_rule", "hidden_size": cfg.width, "num_heads": d.heads,
                           "num_kv_heads": d.kv_heads, "head_dim": d.dim, "value_dim": d.vdim, "conv_taps": d.conv,
                           "decay_rank": None, "gate_rank": None, "eps": cfg.eps, "decay_per_head": True,
                           "gate_activation": "silu"}}
        ff = None if layer.ff is None else {"kind": "plain_mlp", "hidden_size": cfg.width, "intermediate_size": layer.ff,
                                            "activation": "relu2"}
        index[i] = len(layers)
        layers.append(LayerSpec(mixer=mixer, feed_forward=ff, norm=norm, position=f"l{i}", block=block))
    order = [RunEntry(index[i if layer.weights_of is None else layer.weights_of]) for i, layer in enumerate(cfg.layers)]
    return ModelSpec(vocab_size=cfg.vocab, hidden_size=cfg.width, layers=layers, final_norm=norm, positions=positions,
                     max_position=cfg.max_position, tie_embeddings=True, run_order=order,
                     embedding={"kind": "scaled_float", "scale": cfg.embed_scale}, logit_scale=cfg.logit_scale)


def checkpoint_names(cfg: VugelixConfig) -> dict[str, WeightSource]:
    names = {"embed": WeightSource("embed.weight"), "final.norm": WeightSource("final_norm.weight")}
    for at, i in enumerate(cfg.owners()):
        layer = cfg.layers[i]
        src, dst = f"l{i}.", f"layers.{at}."
        names[src + "norm1"] = WeightSource(dst + "mixer_norm.weight")
        a, d = layer.attention, layer.delta
        ls, ld = src + "mix.left.", dst + "mixer.left."
        q, k, v = a.heads * a.dim, a.kv_heads * a.dim, a.kv_heads * a.vdim
        for name, start, rows in (("q", 0, q), ("k", q, k), ("v", q + k, v), ("g", q + k + v, a.heads)):
            names[ls + name] = WeightSource(ld + "qkv.weight", start, rows)
        names[ls + "o"] = WeightSource(ld + "o.weight")
        rs, rd = src + "mix.right.", dst + "mixer.right."
        qk, v = d.kv_heads * d.dim, d.heads * d.vdim
        for name, start, rows in (("q", 0, qk), ("k", qk, qk), ("v", 2 * qk, v)):
            names[rs + name] = WeightSource(rd + "in.weight", start, rows)
            names[rs + name + ".conv"] = WeightSource(rd + "conv.weight", start, rows)
        at_row = 2 * qk + v
        for name, rows in (("b", d.heads), ("a", d.heads), ("g", v)):
            names[rs + name] = WeightSource(rd + "in.weight", at_row, rows)
            at_row += rows
        names[rs + "o"] = WeightSource(rd + "o.weight")
        names[rs + "dt_bias"] = WeightSource(rd + "dt_bias")
        names[rs + "A_log"] = WeightSource(rd + "A_log")
        names[rs + "norm"] = WeightSource(rd + "norm.weight")
        sublayers = ("hc1",)
        if layer.ff is not None:
            names[src + "norm2"] = WeightSource(dst + "feed_forward_norm.weight")
            names[src + "mlp.up"] = WeightSource(dst + "feed_forward.up.weight")
            names[src + "mlp.down"] = WeightSource(dst + "feed_forward.down.weight")
            sublayers = ("hc1", "hc2")
        if cfg.streams is not None:
            for q_name in sublayers:
                for part in ("in", "mix", "out"):
                    names[f"{src}{q_name}.{part}"] = WeightSource(f"{dst}{q_name}.{part}")
    return names


def _shape(layers: int, width: int, ff: int, vocab: int, heads: int, kv_heads: int, dim: int, window: int,
           delta_heads: int, delta_kv_heads: int, delta_dim: int, streams: int | None = 4, repeat_from: int | None = None) -> dict:
    """A model of ``layers`` parallel layers at the sizes of a real model's layers; from layer ``repeat_from`` on the
    layers run the weights of the first ones again."""
    entries = []
    for i in range(layers):
        entry = {"type": "parallel",
                 "mixer": {"left": {"dim": dim, "heads": heads, "kv_heads": kv_heads, "mask": {"size": window},
                                    "rot": {"base": 10000.0, "dims": dim // 2}, "scale": dim ** -0.5, "softcap": 50.0,
                                    "vdim": dim},
                           "left_scale": 0.5,
                           "right": {"conv": 4, "dim": delta_dim, "heads": delta_heads, "kv_heads": delta_kv_heads,
                                     "vdim": delta_dim},
                           "right_scale": 0.5},
                 "mlp": {"kind": "dense", "ff": ff}}
        if repeat_from is not None and i >= repeat_from:
            entry["weights_of"] = i - repeat_from
        entries.append(entry)
    raw = {"architecture": "Vugelix", "embedding": {"scale": float(width) ** 0.5}, "layers": entries, "logit_scale": 1.0,
           "norm": {"eps": 1e-6}, "vocab": vocab, "width": width}
    if streams is not None:
        raw["streams"] = streams
    return raw


# config.json contents of sizes that measurements name; the engine itself takes every size from a config.json
SHAPES = {
    "vugelix-tiny": _shape(3, 64, 96, 211, 4, 2, 16, 24, 4, 2, 16, streams=2, repeat_from=2),
    "vugelix-1b": _shape(16, 2048, 6144, 32768, 16, 8, 128, 2048, 16, 8, 128),
    "vugelix-8b": _shape(36, 4096, 12288, 151936, 32, 8, 128, 4096, 32, 8, 128),
}


VUGELIX = Architecture(
    name="Vugelix",
    model_types=("vugelix",),
    parse_config=parse_config,
    build_spec=build_spec,
    checkpoint_names=checkpoint_names,
    named_shapes=SHAPES,
)
register_architecture(VUGELIX, replace=True)
