"""How a layer's norm, mixer and feed-forward are arranged."""
from __future__ import annotations

import torch

from ..native import ops
from .base import BLOCKS, ParamSpec, Part


@BLOCKS.register("prenorm")
class PreNormBlock(Part):
    """r += mixer(norm(r)); r += feed_forward(norm(r)), with each addition folded into
    the next norm (nanovllm/models/qwen3.py:152-159): the block takes and returns
    (hidden, residual), and ``residual`` is None before the first block."""

    # the norms this arrangement takes, by the names of its constructor's arguments: the model builds one per slot
    # from the layer's description (``LayerSpec.norms[slot]``, else ``LayerSpec.norm``)
    norm_slots = ("mixer_norm", "feed_forward_norm")

    def __init__(self, mixer, feed_forward, mixer_norm, feed_forward_norm):
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.mixer_norm = mixer_norm
        self.feed_forward_norm = feed_forward_norm

    def children(self):
        return {"mixer_norm": self.mixer_norm, "mixer": self.mixer,
                "feed_forward_norm": self.feed_forward_norm, "feed_forward": self.feed_forward}

    @property
    def takes_summed(self) -> bool:
        """Whether ``hidden`` may come as an ``ops.Summed`` (the block before has added it to the residual stream
        already): this block's first norm has to know what that is. A block that says so takes ``next_norm=``."""
        return getattr(self.mixer_norm, "takes_summed", False)

    def forward(self, hidden, residual, step, cache, next_norm=None, next_reader=None):
        """``next_norm``: the norm that takes this block's result next (the next block's first norm, or the model's
        last), if it takes an ``ops.Summed`` in place of ``hidden``; ``next_reader``: the part that reads that norm."""
        # A mixer or feed-forward that says ``adds_to_residual`` takes ``add_to=`` (the residual stream and the norm
        # that follows, ``ops.AddTo``) and may let its last product make the addition (it then returns an
        # ``ops.Summed``); one that says ``takes_deferred_norm`` may get an ``ops.Normed`` as its input, whose rows
        # its first product scales. Parts that say neither get tensors and return tensors.
        mixer, ff = self.mixer, self.feed_forward
        if residual is None:
            x, residual = self.mixer_norm.forward_start(hidden)
        else:
            x, residual = self.mixer_norm.forward_add(hidden, residual, **_deferred(self.mixer_norm, mixer))
        x = mixer.forward(x, step, cache, **_add_to(mixer, self.feed_forward_norm, residual, ff))
        x, residual = self.feed_forward_norm.forward_add(x, residual, **_deferred(self.feed_forward_norm, ff))
        x = ff.forward(x, step, **_add_to(ff, next_norm, residual, next_reader))
        return x, residual


def _deferred(norm, reader) -> dict:
    """The argument that lets ``norm`` hand its scaling on to ``reader``, if both are made for that."""
    both = getattr(norm, "defers_to_products", False) and getattr(reader, "takes_deferred_norm", False)
    return {"deferred": True} if both else {}


def _add_to(part, norm, residual, reader) -> dict:
    """The argument that lets ``part`` make the addition that ``norm`` would make, if both are made for that.
    ``reader``: the part that reads ``norm`` (it counts only if it takes the norm with its scaling left to do)."""
    if norm is not None and getattr(part, "adds_to_residual", False) and getattr(norm, "takes_summed", False):
        return {"add_to": norm.add_to(residual, reader if getattr(reader, "takes_deferred_norm", False) else None)}
    return {}


@BLOCKS.register("parallel_depth_mix")
class ParallelDepthMixBlock(Part):
    """One norm, mixer and feed-forward side by side on its output, and a weighted sum over depth:
        h = norm(x);  X_(i+1) = x + (mixer(h) + feed_forward(h));  x <- sum over j <= i + 1 of w[j] X_j,
    where X_0 is the stream that entered the first such block and i = ``depth_index`` counts the blocks before this
    one. The stream is float32 and is what the block takes and returns as ``hidden`` (there is no residual beside
    it); the results X_j of a step live in ``step.scratch`` ([``depth_total`` + 1, tokens, width] float32). The
    feed-forward may be absent."""

    norm_slots = ("norm",)
    # the sum over depth can norm what it hands on in its own kernel: the model names the next block's norm
    # (``next_norm=``), and that block finds its rows normed already in ``step.scratch``
    norms_ahead = True

    def __init__(self, mixer, feed_forward, norm, depth_index: int, depth_total: int):
        if not 0 <= depth_index < depth_total:
            raise ValueError(f"block {depth_index} of {depth_total}")
        self.mixer, self.feed_forward, self.norm = mixer, feed_forward, norm
        self.depth_index, self.depth_total = depth_index, depth_total
        self.row_dtype = None

    def children(self):
        out = {"norm": self.norm, "mixer": self.mixer}
        if self.feed_forward is not None:
            out["feed_forward"] = self.feed_forward
        return out

    def param_specs(self):
        n = self.depth_index + 2
        return {"depth.weight": ParamSpec((n,), always_float32=True, init_mean=1.0 / n, init_std=0.3 / n)}

    def forward(self, hidden, residual, step, cache, next_norm=None):
        if residual is not None:
            raise ValueError("this block carries its stream itself and takes no residual beside it")
        if hidden.dtype != torch.float32:
            hidden = hidden.float()
        T, W = hidden.shape
        results = step.scratch.get("depth_results")
        if results is None or self.depth_index == 0:
            results = step.scratch["depth_results"] = torch.empty((self.depth_total + 1, T, W), dtype=torch.float32,
                                                                   device=hidden.device)
        ahead = step.scratch.pop("normed_ahead", None)
        if ahead is not None and ahead[0] is self.norm and ahead[1] is hidden:
            h = ahead[2]                                   # the block before has normed this very stream for this norm
        else:
            h = self.norm.forward(hidden, out_dtype=self.row_dtype or torch.float32)
        # (a pair of mixers may leave its two norms and their mean to the sum over depth)
        mixed = self.mixer.forward(h, step, cache, **({"deferred": True} if getattr(self.mixer, "defers_pair_norm", False) else {}))
        fed = self.feed_forward.forward(h, step) if self.feed_forward is not None else None
        weight, eps = getattr(next_norm, "weight", None), getattr(next_norm, "eps", None)
        rows = mixed.a if isinstance(mixed, ops.NormedPairMean) else mixed
        if weight is not None and weight.numel() == 1 and eps is not None and rows.dtype == (self.row_dtype or torch.float32):
            out, normed = ops.depth_mix(hidden, mixed, fed, results, self.depth_index, self.depth_weight, gain=weight, eps=eps)
            step.scratch["normed_ahead"] = (next_norm, out, normed)
            return out, None
        return ops.depth_mix(hidden, mixed, fed, results, self.depth_index, self.depth_weight), None


@BLOCKS.register("parallel_two_norms")
class ParallelTwoNormsBlock(Part):
    """x <- x + (mixer(norm_a(x)) + feed_forward(norm_b(x))): both norms read the same x. The stream x is float32 and is
    what the block takes and returns as ``hidden`` (no residual beside it). The two norms share their mean and
    variance, so one kernel makes both; the additions of a block are left to the kernel that norms for the block after
    it (``pending`` in ``step.scratch``), or made by a kernel of their own after the last block. The feed-forward may
    be absent (then there is no second norm)."""

    norm_slots = ("mixer_norm", "feed_forward_norm")
    norms_ahead = True            # the model tells the block whether a block follows (``next_norm`` is that block's ``norm``)

    def __init__(self, mixer, feed_forward, mixer_norm, feed_forward_norm, keeps_unused_norm: bool = False):
        """``keeps_unused_norm``: a block without feed-forward holds its second norm's tensors all the same (a
        checkpoint that stores them), unused."""
        self.mixer, self.feed_forward = mixer, feed_forward
        self.mixer_norm, self.feed_forward_norm = mixer_norm, feed_forward_norm
        self.keeps_unused_norm = bool(keeps_unused_norm)
        if feed_forward is not None and feed_forward_norm.eps != mixer_norm.eps:
            raise ValueError("the two norms of this block share their statistics and so their eps")
        self.row_dtype = None

    @property
    def norm(self):
        """What the block before this one is shown as the norm that takes its result: this block adds what is
        pending itself, in its norms' kernel."""
        return self

    def children(self):
        out = {"mixer_norm": self.mixer_norm, "mixer": self.mixer}
        if self.feed_forward is not None or self.keeps_unused_norm:
            out["feed_forward_norm"] = self.feed_forward_norm
        if self.feed_forward is not None:
            out["feed_forward"] = self.feed_forward
        return out

    def forward(self, hidden, residual, step, cache, next_norm=None):
        if residual is not None:
            raise ValueError("this block carries its stream itself and takes no residual beside it")
        if hidden.dtype != torch.float32:
            hidden = hidden.float()
        pending = step.scratch.pop("pending_additions", None)
        add = pending[1] if pending is not None and pending[0] is hidden else ()
        dtype = self.row_dtype or torch.float32
        a, b = self.mixer_norm, self.feed_forward_norm
        second = (b.weight, b.bias) if self.feed_forward is not None else None
        h1, h2 = ops.layernorm_pair(hidden, (a.weight, a.bias), second, a.eps, dtype, add=add)
        mixed = self.mixer.forward(h1, step, cache)
        fed = self.feed_forward.forward(h2, step) if self.feed_forward is not None else None
        if isinstance(next_norm, ParallelTwoNormsBlock):
            step.scratch["pending_additions"] = (hidden, (mixed, fed))
        else:
            ops.add_streams_(hidden, mixed, fed)
        return hidden, None


@BLOCKS.register("stream_mix")
class StreamMixBlock(Part):
    """A pre-norm layer on ``streams`` residual streams X_1 .. X_n (hyper-connections). For each sublayer q (the
    mixer, then the feed-forward) with coefficients in_q [n], mix_q [n, n] (from, to) and out_q [n]:
        u = sum_s in_q[s] X_s;   y = sublayer(norm_q(u));   X_t <- sum_s mix_q[s, t] X_s + out_q[t] y,
    all streams at once from their old values. Before the first such block all streams equal the embedding's rows;
    after the last their sum goes on. ``learned`` False: one stream with coefficients of 1, which is the plain
    pre-norm layer x <- x + sublayer(norm(x)) on a float32 stream. The streams are float32 and are what the block
    takes and returns as ``hidden`` ([n, tokens, width]; the first block takes [tokens, width], the last returns
    that). One kernel stands between two sublayers: it takes the result of the one into the streams and reads the
    next one's input through its norm, also across the border to the next block. The feed-forward may be absent."""

    norm_slots = ("mixer_norm", "feed_forward_norm")
    norms_ahead = True            # the model tells the block which block follows (``next_norm`` is that block's ``norm``)

    def __init__(self, mixer, feed_forward, mixer_norm, feed_forward_norm, streams: int = 1, learned: bool = True):
        if not 1 <= streams <= 16:
            raise ValueError(f"1 to 16 streams are taken, got {streams}")
        if not learned and streams != 1:
            raise ValueError("several streams need coefficients")
        self.mixer, self.feed_forward = mixer, feed_forward
        self.mixer_norm, self.feed_forward_norm = mixer_norm, feed_forward_norm
        self.streams, self.learned = streams, bool(learned)
        self.row_dtype = None

    @property
    def norm(self):
        """What the block before this one is shown as the norm that takes its result: this block itself (its first
        sublayer's coefficients and norm are read in that block's last kernel)."""
        return self

    def children(self):
        out = {"mixer_norm": self.mixer_norm, "mixer": self.mixer}
        if self.feed_forward is not None:
            out["feed_forward_norm"] = self.feed_forward_norm
            out["feed_forward"] = self.feed_forward
        return out

    def param_specs(self):
        if not self.learned:
            return {}
        n = self.streams

        def three(q):
            return {f"{q}.in": ParamSpec((n,), always_float32=True, init_mean=1.0 / n, init_std=0.1),
                    f"{q}.mix": ParamSpec((n, n), always_float32=True, init_mean=1.0 / n, init_std=0.1),
                    f"{q}.out": ParamSpec((n,), always_float32=True, init_mean=1.0, init_std=0.1)}
        return dict(three("hc1"), **(three("hc2") if self.feed_forward is not None else {}))

    def bind(self, params):
        self.coefficients = {}
        for q in ("hc1", "hc2"):
            if f"{q}.in" in params:
                self.coefficients[q] = (params[f"{q}.in"], params[f"{q}.mix"], params[f"{q}.out"])
            else:
                self.coefficients[q] = (None, None, None)

    def _read(self, q: str, norm) -> tuple:
        return (self.coefficients[q][0], norm.weight, norm.eps)

    def first_read(self) -> tuple:
        """What the kernel before this block's mixer reads: (in, norm weight, eps)."""
        return self._read("hc1", self.mixer_norm)

    def forward(self, hidden, residual, step, cache, next_norm=None):
        if residual is not None:
            raise ValueError("this block carries its streams itself and takes no residual beside them")
        n, dtype = self.streams, self.row_dtype or torch.float32
        ahead = step.scratch.pop("stream_rows_ahead", None)
        if hidden.dim() == 2:                      # the first block: all streams start as the embedding's rows
            if hidden.dtype != torch.float32:
                hidden = hidden.float()
            T, W = hidden.shape
            X = torch.empty((n, T, W), dtype=torch.float32, device=hidden.device)
            h, _ = ops.streams_step(X, T, W, n, dtype, start=hidden, read=self.first_read())
        else:
            X = hidden
            _, T, W = X.shape
            if ahead is not None and ahead[0] is self and ahead[1] is X:
                h = ahead[2]                       # the block before has read this block's first input already
            else:
                h, _ = ops.streams_step(X, T, W, n, dtype, read=self.first_read())
        defer = {"deferred": True} if getattr(self.mixer, "defers_pair_sum", False) else {}
        y = self.mixer.forward(h, step, cache, **defer)
        _, mix, out = self.coefficients["hc1"]
        if self.feed_forward is not None:
            h, _ = ops.streams_step(X, T, W, n, dtype, update=(mix, out, y), read=self._read("hc2", self.feed_forward_norm))
            y = self.feed_forward.forward(h, step)
            _, mix, out = self.coefficients["hc2"]
        if isinstance(next_norm, StreamMixBlock) and next_norm.streams == n:
            h, _ = ops.streams_step(X, T, W, n, dtype, update=(mix, out, y), read=next_norm.first_read())
            step.scratch["stream_rows_ahead"] = (next_norm, X, h)
            return X, None
        if next_norm is not None:
            raise ValueError("a block of several streams is followed by a block of its kind and its number of streams")
        _, total = ops.streams_step(X, T, W, n, dtype, update=(mix, out, y), collapse=True)
        return total, None


@BLOCKS.register("sandwich_norms")
class SandwichNormsBlock(Part):
    """A layer whose sublayers are normed on both sides, on a float32 stream x:
        x <- x + mixer_out_norm(mixer(mixer_norm(x)));   x <- x + feed_forward_out_norm(feed_forward(feed_forward_norm(x))).
    The four norms are RMS norms with a weight vector (``stream_rmsnorm``: the block reads their weight and eps). The
    stream is what the block takes and returns as ``hidden`` (no residual beside it). One kernel stands between two
    sublayers: it norms the result of the one, adds it to the stream and norms the new stream for the next, also across
    the border to the next block of this kind. The feed-forward may be absent (then the block has two norms)."""

    norm_slots = ("mixer_norm", "mixer_out_norm", "feed_forward_norm", "feed_forward_out_norm")
    norms_ahead = True            # the model tells the block which block follows (``next_norm`` is that block's ``norm``)

    def __init__(self, mixer, feed_forward, mixer_norm, mixer_out_norm, feed_forward_norm, feed_forward_out_norm):
        self.mixer, self.feed_forward = mixer, feed_forward
        self.mixer_norm, self.mixer_out_norm = mixer_norm, mixer_out_norm
        self.feed_forward_norm, self.feed_forward_out_norm = feed_forward_norm, feed_forward_out_norm
        self.row_dtype = None

    @property
    def norm(self):
        """What the block before this one is shown as the norm that takes its result: this block itself (its first
        norm is read in that block's last kernel)."""
        return self

    def children(self):
        out = {"mixer_norm": self.mixer_norm, "mixer": self.mixer, "mixer_out_norm": self.mixer_out_norm}
        if self.feed_forward is not None:
            out.update({"feed_forward_norm": self.feed_forward_norm, "feed_forward": self.feed_forward,
                        "feed_forward_out_norm": self.feed_forward_out_norm})
        return out

    def first_read(self) -> tuple:
        """What the kernel before this block's mixer reads through: (norm weight, eps)."""
        return (self.mixer_norm.weight, self.mixer_norm.eps)

    def forward(self, hidden, residual, step, cache, next_norm=None):
        if residual is not None:
            raise ValueError("this block carries its stream itself and takes no residual beside it")
        if hidden.dtype != torch.float32:
            hidden = hidden.float()
        dtype = self.row_dtype or torch.float32
        ahead = step.scratch.pop("sandwich_rows_ahead", None)
        if ahead is not None and ahead[0] is self and ahead[1] is hidden:
            h = ahead[2]                           # the block before has read this block's first input already
        else:
            h = ops.sandwich_step(hidden, read=self.first_read(), rows_dtype=dtype)
        y = self.mixer.forward(h, step, cache)
        pending = (y, self.mixer_out_norm.weight, self.mixer_out_norm.eps)
        if self.feed_forward is not None:
            h = ops.sandwich_step(hidden, add=pending, read=(self.feed_forward_norm.weight, self.feed_forward_norm.eps),
                                  rows_dtype=dtype)
            y = self.feed_forward.forward(h, step)
            pending = (y, self.feed_forward_out_norm.weight, self.feed_forward_out_norm.eps)
        if isinstance(next_norm, SandwichNormsBlock):
            h = ops.sandwich_step(hidden, add=pending, read=next_norm.first_read(), rows_dtype=dtype)
            step.scratch["sandwich_rows_ahead"] = (next_norm, hidden, h)
        else:
            ops.sandwich_step(hidden, add=pending)
        return hidden, None
