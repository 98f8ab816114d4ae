"""The Pukarax decoder as a recipe of parts.

config.json: {"architecture": "Pukarax", "vocab", "width", "norm": {"eps"}, "embedding": {"scale"}, "logit_scale",
"loop": {"start", "stop", "times"}, "layers": [...]}. Every entry of ``layers`` has ``type`` ("attention" or
"attention_2"), the sizes of its mixer (``mixer``) and its feed-forward (``mlp``, or null for none).

* a layer norms both sides of each sublayer on a float32 stream: x += norm1b(mixer(norm1(x))), then
  x += norm2b(mlp(norm2(x))); all norms are RMS norms with a weight vector and ``norm.eps``.
* "attention": two softmax maps per head over the same values (``differential_attention``): q and k hold
  [map 1 | map 2] per head, every map turned over its first ``rot.dims`` coordinates (pairs (2i, 2i + 1),
  ``rot.base``); the result a1 - lambda a2 with lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + ``diff`` is divided by its
  root mean square per head, multiplied by 1 - ``diff`` and by a sigmoid gate per head; biases on q, k, v and o.
* "attention_2": ``rotary_attention`` whose values are the keys as projected; q and k are turned (pairs
  (i, i + dims / 2), frequencies divided by ``rot.scaling.factor``) and then divided by their root mean square per
  head; a sigmoid gate per entry on the concatenated heads; no biases.
* both read, at position i, the keys j <= i of i's own block of ``mask.size`` positions, and group ``heads`` query
  heads over ``kv_heads`` key/value heads; ``scale`` multiplies the scores.
* ``mlp.kind`` "dense": down(silu(gate x) * (up x)) of inner size ``ff``. "moe": ``router.experts`` such feed-forwards
  of inner size ``expert.ff`` without biases, of which a token uses the ``router.top`` with the largest router logit
  (router weight and bias); the experts' outputs are summed with softmax(chosen logits) as their weights; ``shared``
  ({"ff"}) names one more such feed-forward that all tokens use, added to that sum.
* ``loop``: the group of layers start .. stop - 1 is run ``times`` times over before the layers after it, on one set
  of weights, every run with a cache of its own.

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
MIXER_TYPES = ("attention", "attention_2")


@dataclass(frozen=True)
class MixerSizes:
    kind: str                      # "attention": two maps per head; "attention_2": the values are the keys
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    chunk: int | None
    rot_dims: int
    rot_base: float
    rot_factor: float | None
    diff: float | None = None      # "attention" only


@dataclass(frozen=True)
class MlpSizes:
    kind: str                      # "dense" | "moe"
    ff: int                        # inner size of the dense feed-forward, or of one expert
    experts: int = 0
    top: int = 0
    shared_ff: int | None = None


@dataclass(frozen=True)
class LayerSizes:
    mixer: MixerSizes
    mlp: MlpSizes | None


@dataclass(frozen=True)
class PukaraxConfig:
    vocab: int
    width: int
    eps: float
    layers: tuple
    loop: tuple | None = None               # (start, stop, times)
    embed_scale: float = 1.0
    logit_scale: float = 1.0
    max_position: int = MAX_POSITION
    raw: dict = field(default_factory=dict, compare=False, repr=False)

    def order(self) -> list[int]:
        """The layers in the order in which they run."""
        n = len(self.layers)
        if self.loop is None:
            return list(range(n))
        start, stop, times = self.loop
        return list(range(start)) + list(range(start, stop)) * times + list(range(stop, n))


def _where(i: int, key: str) -> str:
    return f"config.json: layers[{i}].{key}"


def _mixer(i: int, kind: str, m: dict) -> MixerSizes:
    where = _where(i, "mixer")
    rot = m.get("rot") or {}
    mask = m.get("mask") or {}
    scaling = rot.get("scaling") or {}
    dims = require(rot, "dims") if rot else 0
    s = MixerSizes(kind=kind, heads=require(m, "heads"), kv_heads=require(m, "kv_heads"), dim=require(m, "dim"),
                   vdim=require(m, "vdim"), scale=require(m, "scale", float),
                   chunk=require(mask, "size") if mask else None, rot_dims=dims,
                   rot_base=require(rot, "base", float) if dims else 1.0,
                   rot_factor=require(scaling, "factor", float) if scaling else None,
                   diff=require(m, "diff", float) if kind == "attention" else None)
    if min(s.heads, s.kv_heads, s.dim, s.vdim) <= 0 or s.heads % s.kv_heads:
        raise ConfigError(f"{where}: sizes must be positive and heads a multiple of kv_heads")
    if s.chunk is not None and s.chunk <= 0:
        raise ConfigError(f"{where}.mask.size must be positive")
    if s.rot_dims < 0 or s.rot_dims % 2 or s.rot_dims > s.dim:
        raise ConfigError(f"{where}: rot.dims {s.rot_dims} must be even and at most dim {s.dim}")
    if s.rot_dims and not s.rot_base > 0:
        raise ConfigError(f"{where}.rot.base must be positive")
    if s.rot_factor is not None and not s.rot_factor > 0:
        raise ConfigError(f"{where}.rot.scaling.factor must be positive")
    if kind == "attention_2" and s.vdim != s.dim:
        raise ConfigError(f"{where}: the values are the keys, so vdim {s.vdim} must equal dim {s.dim}")
    return s


def _mlp(i: int, mlp: dict | None) -> MlpSizes | None:
    if mlp is None:
        return None
    where = _where(i, "mlp")
    kind = mlp.get("kind")
    if kind == "dense":
        out = MlpSizes("dense", require(mlp, "ff"))
    elif kind == "moe":
        router, shared = mlp.get("router") or {}, mlp.get("shared")
        out = MlpSizes("moe", require(mlp.get("expert") or {}, "ff"), experts=require(router, "experts"),
                       top=require(router, "top"), shared_ff=require(shared, "ff") if shared else None)
        if not 0 < out.top <= out.experts:
            raise ConfigError(f"{where}.router: {out.top} of {out.experts} experts")
        if out.shared_ff is not None and out.shared_ff <= 0:
            raise ConfigError(f"{where}.shared.ff must be positive")
    else:
        raise ConfigError(f"{where}.kind: {kind!r} is not known ('dense' and 'moe' are)")
    if out.ff <= 0:
        raise ConfigError(f"{where}: the inner size must be positive")
    return out


def parse_config(raw: dict) -> PukaraxConfig:
    eps = require(raw.get("norm") or {}, "eps", float)
    if not eps > 0:
        raise ConfigError("config.json: norm.eps must be positive")
    entries = raw.get("layers")
    if not isinstance(entries, list) or not entries:
        raise ConfigError("config.json: 'layers' must be a list with at least one layer")
    layers = []
    for i, entry in enumerate(entries):
        kind, m = entry.get("type"), entry.get("mixer")
        if kind not in MIXER_TYPES:
            raise ConfigError(f"{_where(i, 'type')}: {kind!r} is not known ({list(MIXER_TYPES)} are)")
        if not isinstance(m, dict):
            raise ConfigError(f"{_where(i, 'mixer')} is needed")
        layers.append(LayerSizes(_mixer(i, kind, m), _mlp(i, entry.get("mlp"))))
    loop = raw.get("loop")
    if loop is not None:
        loop = (require(loop, "start"), require(loop, "stop"), require(loop, "times"))
        if not (0 <= loop[0] <= loop[1] <= len(layers)) or loop[2] < 1:
            raise ConfigError(f"config.json: loop {loop} does not fit {len(layers)} layers")
    embedding = raw.get("embedding") or {}
    cfg = PukaraxConfig(vocab=require(raw, "vocab"), width=require(raw, "width"), eps=eps, layers=tuple(layers), loop=loop,
                        embed_scale=float(embedding["scale"]) if embedding.get("scale") is not None else 1.0,
                        logit_scale=float(raw["logit_scale"]) if raw.get("logit_scale") is not None else 1.0,
                        max_position=min(int(raw.get("max_position") or MAX_POSITION), MAX_POSITION), raw=dict(raw))
    if cfg.vocab <= 0 or cfg.width <= 0:
        raise ConfigError("config.json: 'vocab' and 'width' must be positive")
    return cfg


def _gated(width: int, ff: int) -> dict:
    return {"kind": "swiglu", "hidden_size": width, "intermediate_size": ff}


def build_spec(cfg: PukaraxConfig) -> ModelSpec:
    norm = {"kind": "stream_rmsnorm", "size": cfg.width, "eps": cfg.eps}
    layers, positions = [], {}
    for i, layer in enumerate(cfg.layers):
        m = layer.mixer
        positions[f"l{i}"] = {"kind": "rotary_frequencies", "rotary_dim": m.rot_dims, "base": m.rot_base,
                              "scaling_factor": m.rot_factor}
        common = {"hidden_size": cfg.width, "num_heads": m.heads, "num_kv_heads": m.kv_heads, "head_dim": m.dim,
                  "value_dim": m.vdim, "scale": m.scale, "chunk": m.chunk}
        if m.kind == "attention":
            mixer = dict(common, kind="differential_attention", diff=m.diff, eps=cfg.eps, bias=True,
                         rotation="interleaved", head_gate=True)
        else:
            mixer = dict(common, kind="rotary_attention", bias=False, rotation="halves", unit_norm_eps=cfg.eps,
                         values_are_keys=True, element_gate=True)
        ff = None
        if layer.mlp is not None and layer.mlp.kind == "dense":
            ff = _gated(cfg.width, layer.mlp.ff)
        elif layer.mlp is not None:
            p = layer.mlp
            ff = {"kind": "routed_experts", "hidden_size": cfg.width, "num_experts": p.experts, "top": p.top,
                  "expert_size": p.ff, "scoring": "softmax_of_chosen", "scores_on": "output", "router_bias": True,
                  "shared": _gated(cfg.width, p.shared_ff) if p.shared_ff is not None else None}
        layers.append(LayerSpec(mixer=mixer, feed_forward=ff, norm=norm, position=f"l{i}", block={"kind": "sandwich_norms"}))
    return ModelSpec(vocab_size=cfg.vocab, hidden_size=cfg.width, layers=layers, final_norm=norm, positions=positions,
                     max_position=cfg.max_position, tie_embeddings=True, run_order=[RunEntry(i) for i in cfg.order()],
                     embedding={"kind": "scaled_float", "scale": cfg.embed_scale}, logit_scale=cfg.logit_scale)


def checkpoint_names(cfg: PukaraxConfig) -> dict[str, WeightSource]:
    names = {"embed": WeightSource("embed.weight"), "final.norm": WeightSource("final_norm.weight")}
    for i, layer in enumerate(cfg.layers):
        src, dst = f"l{i}.", f"layers.{i}."
        names[src + "norm1"] = WeightSource(dst + "mixer_norm.weight")
        names[src + "norm1b"] = WeightSource(dst + "mixer_out_norm.weight")
        m = layer.mixer
        ms, md = src + "mix.", dst + "mixer."
        if m.kind == "attention":
            bands = (("q", 2 * m.heads * m.dim), ("k", 2 * m.kv_heads * m.dim), ("v", m.kv_heads * m.vdim), ("g", m.heads))
        else:
            bands = (("q", m.heads * m.dim), ("k", m.kv_heads * m.dim), ("g", m.heads * m.vdim))
        at = 0
        for name, rows in bands:
            names[ms + name] = WeightSource(md + "qkv.weight", at, rows)
            if m.kind == "attention" and name != "g":
                names[ms + name + ".b"] = WeightSource(md + "qkv.bias", at, rows)
            at += rows
        names[ms + "o"] = WeightSource(md + "o.weight")
        if m.kind == "attention":
            names[ms + "o.b"] = WeightSource(md + "o.bias")
            for name in ("lq1", "lk1", "lq2", "lk2"):
                names[ms + name] = WeightSource(md + name)
        p = layer.mlp
        if p is None:
            continue
        names[src + "norm2"] = WeightSource(dst + "feed_forward_norm.weight")
        names[src + "norm2b"] = WeightSource(dst + "feed_forward_out_norm.weight")
        fs, fd = src + "mlp.", dst + "feed_forward."

        def gated(s: str, d: str, ff: int) -> None:
            names[s + "gate"] = WeightSource(d + "gate_up.weight", 0, ff)
            names[s + "up"] = WeightSource(d + "gate_up.weight", ff, ff)
            names[s + "down"] = WeightSource(d + "down.weight")

        if p.kind == "dense":
            gated(fs, fd, p.ff)
            continue
        names[fs + "router"] = WeightSource(fd + "router.weight")
        names[fs + "router.b"] = WeightSource(fd + "router.bias")
        for e in range(p.experts):
            names[f"{fs}e{e}.gate"] = WeightSource(fd + "gate_up.weight", e * 2 * p.ff, p.ff)
            names[f"{fs}e{e}.up"] = WeightSource(fd + "gate_up.weight", e * 2 * p.ff + p.ff, p.ff)
            names[f"{fs}e{e}.down"] = WeightSource(fd + "down.weight", e * cfg.width, cfg.width)
        if p.shared_ff is not None:
            gated(fs + "shared.", fd + "shared.", p.shared_ff)
    return names


def _shape(layers: int, width: int, ff: int, vocab: int, heads: int, kv_heads: int, dim: int, chunk: int,
           experts: int = 0, top: int = 0, expert_ff: int = 0, shared_ff: int | None = None, differential_every: int = 4,
           loop: tuple | None = None) -> dict:
    """A model of ``layers`` layers at the sizes of a real model's layers: every ``differential_every``-th layer has two
    maps per head (of half the head size, so that its products have the other layers' sizes), the others use their
    keys as values; feed-forwards are dense and routed in turn where there are experts."""
    entries = []
    for i in range(layers):
        if differential_every and i % differential_every == differential_every - 1:
            half = dim // 2
            entry = {"type": "attention",
                     "mixer": {"diff": 0.4, "dim": half, "heads": heads, "kv_heads": kv_heads, "mask": {"size": chunk},
                               "rot": {"base": 100000.0, "dims": half}, "scale": half ** -0.5, "vdim": dim}}
        else:
            entry = {"type": "attention_2",
                     "mixer": {"dim": dim, "heads": heads, "kv_heads": kv_heads, "mask": {"size": chunk},
                               "rot": {"base": 10000.0, "dims": dim, "scaling": {"factor": 4.0}}, "scale": dim ** -0.5,
                               "vdim": dim}}
        if experts and i % 2:
            entry["mlp"] = {"kind": "moe", "expert": {"ff": expert_ff}, "router": {"experts": experts, "top": top},
                            "shared": {"ff": shared_ff} if shared_ff else None}
        else:
            entry["mlp"] = {"kind": "dense", "ff": ff}
        entries.append(entry)
    raw = {"architecture": "Pukarax", "embedding": {"scale": float(width) ** 0.5}, "layers": entries, "logit_scale": 1.0,
           "norm": {"eps": 1e-6}, "vocab": vocab, "width": width}
    if loop is not None:
        raw["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return raw


# config.json contents of sizes that measurements name; the engine itself takes every size from a config.json
SHAPES = {
    "pukarax-tiny": _shape(3, 64, 96, 211, 4, 2, 16, 24, experts=5, top=2, expert_ff=24, shared_ff=40,
                           differential_every=2, loop=(0, 2, 2)),
    "pukarax-1b": _shape(8, 2048, 6144, 32768, 16, 8, 128, 2048, experts=16, top=2, expert_ff=1536, shared_ff=1536),
    "pukarax-8b": _shape(4, 4096, 12288, 151936, 32, 8, 128, 4096, experts=32, top=4, expert_ff=1536, shared_ff=1536),
}


PUKARAX = Architecture(
    name="Pukarax",
    model_types=("pukarax",),
    parse_config=parse_config,
    build_spec=build_spec,
    checkpoint_names=checkpoint_names,
    named_shapes=SHAPES,
)
register_architecture(PUKARAX, replace=True)
