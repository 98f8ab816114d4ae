"""Token mixers. ``GQAAttention`` follows nanovllm/models/qwen3.py:14-88 and
nanovllm/layers/attention.py:43-75. ``RotaryAttention`` is softmax attention in a more general make (value heads of
their own size, biases, a chunk mask, turned values, keys and values lent by another layer), ``GatedDeltaRule`` a
recurrent mixer with a matrix of state per head, ``NormedPair`` two mixers side by side, ``DifferentialAttention`` the
difference of two softmax maps per head over the same values."""
from __future__ import annotations

import torch

from ..native import ops
from .base import MIXERS, CacheView, CombinedNeed, PagedKVNeed, ParamSpec, Part, StateNeed


@MIXERS.register("gqa_attention")
class GQAAttention(Part):
    """Causal attention with grouped key/value heads over the paged cache.

    qkv = x W^T (+ b), rows of W ordered q | k | v (nanovllm/layers/linear.py:150-167);
    optional RMSNorm over each q and k head (qwen3.py:82-84); rotation; keys (normed
    and turned) and values are stored at the step's slots; every query reads its
    request's keys up to its own position (attention.py:64-74); output projection
    without bias (qwen3.py:49-53).
    """

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int, scale: float,
                 qk_norm_eps: float | None, qkv_bias: bool, position, window: int | None = None):
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} heads are not a multiple of {num_kv_heads} key/value heads")
        self.hidden_size = hidden_size
        self.num_heads = num_heads
        self.num_kv_heads = num_kv_heads
        self.head_dim = head_dim
        self.scale = scale
        self.qk_norm_eps = qk_norm_eps
        self.qkv_bias = qkv_bias
        self.position = position
        self.window = window
        self.qkv_weight = self.qkv_bias_t = self.o_weight = None
        self.q_norm_weight = self.k_norm_weight = None

    def param_specs(self):
        width = (self.num_heads + 2 * self.num_kv_heads) * self.head_dim
        specs = {
            "qkv.weight": ParamSpec((width, self.hidden_size)),
            "o.weight": ParamSpec((self.hidden_size, self.num_heads * self.head_dim)),
        }
        if self.qkv_bias:
            specs["qkv.bias"] = ParamSpec((width,), init="zeros")
        if self.qk_norm_eps is not None:
            specs["q_norm.weight"] = ParamSpec((self.head_dim,), init="norm", keeps_float32=True)
            specs["k_norm.weight"] = ParamSpec((self.head_dim,), init="norm", keeps_float32=True)
        return specs

    def bind(self, params):
        self.qkv_weight = params["qkv.weight"]
        self.o_weight = params["o.weight"]
        self.qkv_bias_t = params.get("qkv.bias")
        self.q_norm_weight = params.get("q_norm.weight")
        self.k_norm_weight = params.get("k_norm.weight")

    def cache_need(self):
        return PagedKVNeed(self.num_kv_heads, self.head_dim, self.window)

    takes_deferred_norm = True    # x goes straight into a product, which can norm it
    adds_to_residual = True       # the output projection can make the addition to the residual stream

    def first_product(self):
        """(weight, gated) of the product that x goes into."""
        return self.qkv_weight, False

    def forward(self, x, step, cache: CacheView, add_to=None):
        tables = step.groups[cache.group]
        qkv = ops.linear(x, self.qkv_weight)
        # an encoding over several position axes says which axis turns each pair; others turn by the first axis
        pair_axes = self.position.pair_axes() if hasattr(self.position, "pair_axes") else None
        q = ops.qk_rope_write(
            qkv, self.qkv_bias_t, self.q_norm_weight, self.k_norm_weight,
            self.qk_norm_eps if self.qk_norm_eps is not None else 0.0,
            self.position.rotation_table(), step.token_positions if pair_axes is None else step.positions,
            tables.slot_mapping, cache.k, cache.v, self.num_heads, self.num_kv_heads, self.head_dim,
            write_kv=cache.writes, pair_axes=pair_axes)
        o = ops.paged_attention(q, cache.k, cache.v, step.attention, tables.block_tables, self.scale, self.window)
        return ops.linear(o.view(o.shape[0], self.num_heads * self.head_dim), self.o_weight, add_to=add_to)


@MIXERS.register("rotary_attention")
class RotaryAttention(Part):
    """Softmax attention with grouped key/value heads over the paged cache, in a more general make than
    ``GQAAttention``: value heads of a size of their own (``value_dim``), optional biases on q, k and v, the rotation
    given by frequencies (``position``: a ``rotary_frequencies`` encoding; angles are taken from the position, no
    table), and which keys a query at position i reads: all j <= i, the last ``window`` of them, or (``chunk`` = n)
    those with floor(j / n) = floor(i / n), blocks counted from the start of the request. ``rotate_values``: the
    value at position j is stored turned by j over all its coordinates (pairs (m, m + value_dim / 2), frequencies of
    the encoding's base over value_dim, unscaled), and each head's result at position i is turned back by i.
    ``own_kv`` False: the layer has no key and value projections and reads the cache of the run-order entry it
    borrows from (keys as stored, after rotation) with queries, mask and output projection of its own.
    ``softcap`` c: a score s (after the scale) becomes c tanh(s / c). ``sink`` z: the softmax's denominator holds one
    more term exp(z), a key of that score that has no value. ``head_gate``: head h's result is multiplied by
    sigmoid(w_h . x), x the mixer's input; the rows w_h are the last ``num_heads`` rows of the packed projection.
    ``element_gate``: the concatenated heads are multiplied entry by entry with sigmoid(G x); the rows of G are the
    last ``num_heads * value_dim`` rows of the packed projection. ``rotation``: which coordinates make a pair,
    "halves" (i, i + r / 2) or "interleaved" (2i, 2i + 1). ``unit_norm_eps``: after the rotation every query and key head
    is divided by its root mean square (this eps under the root). ``values_are_keys``: there is no value projection; a
    token's values are its keys as projected, before rotation and norm (``value_dim`` equals ``head_dim``)."""

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int, value_dim: int, scale: float,
                 bias: bool, position, chunk: int | None = None, window: int | None = None, rotate_values: bool = False,
                 own_kv: bool = True, softcap: float | None = None, sink: float | None = None, head_gate: bool = False,
                 element_gate: bool = False, rotation: str = "halves", unit_norm_eps: float | None = None,
                 values_are_keys: bool = False):
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} heads are not a multiple of {num_kv_heads} key/value heads")
        if window and chunk:
            raise ValueError("a window or a chunk, not both")
        if rotate_values and value_dim % 2:
            raise ValueError(f"values of odd size {value_dim} cannot be turned")
        self.hidden_size, self.num_heads, self.num_kv_heads = hidden_size, num_heads, num_kv_heads
        self.head_dim, self.value_dim, self.scale, self.bias = head_dim, value_dim, scale, bias
        self.position, self.chunk, self.window = position, chunk or None, window or None
        self.rotate_values, self.own_kv = rotate_values, own_kv
        if softcap is not None and not softcap > 0:
            raise ValueError(f"a cap on the scores must be positive, got {softcap}")
        if head_gate and bias:
            raise ValueError("a gate per head and biases are not taken together")
        if element_gate and (head_gate or bias):
            raise ValueError("a gate per entry is not taken together with a gate per head or with biases")
        if rotation not in ("halves", "interleaved"):
            raise ValueError(f"rotation {rotation!r} is not known ('halves' and 'interleaved' are)")
        if unit_norm_eps is not None and not unit_norm_eps >= 0:
            raise ValueError(f"the eps of the unit norm must not be negative, got {unit_norm_eps}")
        if values_are_keys and (value_dim != head_dim or rotate_values or not own_kv):
            raise ValueError("values that are the keys as projected have the keys' size, are not turned and are the layer's own")
        self.softcap, self.sink, self.head_gate = softcap, sink, bool(head_gate)
        self.element_gate, self.rotation, self.unit_norm_eps = bool(element_gate), rotation, unit_norm_eps
        self.values_are_keys = bool(values_are_keys)
        self.qkv_weight = self.qkv_bias = self.o_weight = None

    def _packed_width(self) -> int:
        width = self.num_heads * self.head_dim
        if self.own_kv:
            width += self.num_kv_heads * (self.head_dim + (0 if self.values_are_keys else self.value_dim))
        return width

    def _gate_columns(self) -> int:
        return self.num_heads if self.head_gate else (self.num_heads * self.value_dim if self.element_gate else 0)

    def param_specs(self):
        gates = self._gate_columns()
        specs = {"qkv.weight": ParamSpec((self._packed_width() + gates, self.hidden_size)),
                 "o.weight": ParamSpec((self.hidden_size, self.num_heads * self.value_dim))}
        if self.bias:
            specs["qkv.bias"] = ParamSpec((self._packed_width(),), init="zeros")
        return specs

    def bind(self, params):
        self.qkv_weight, self.o_weight = params["qkv.weight"], params["o.weight"]
        self.qkv_bias = params.get("qkv.bias")

    def cache_need(self):
        return PagedKVNeed(self.num_kv_heads, self.head_dim, self.window,
                           None if self.value_dim == self.head_dim else self.value_dim, self.chunk)

    def forward(self, x, step, cache: CacheView):
        tables = step.groups[cache.group]
        writes = self.own_kv and cache.writes
        if not self.own_kv and cache.writes:
            raise ValueError("an attention layer without key and value projections must borrow another entry's cache")
        qkv = ops.linear(x, self.qkv_weight)
        gates = self._gate_columns()
        if self.own_kv and not writes:               # a layer with projections of its own that reads a lent cache
            if gates:
                raise ValueError("a layer with gates and projections of its own cannot read a lent cache")
            qkv = qkv[:, :self.num_heads * self.head_dim].contiguous()
        bias = self.qkv_bias if (self.qkv_bias is None or writes or not self.own_kv) else \
            self.qkv_bias[:self.num_heads * self.head_dim].contiguous()
        freqs = self.position.frequencies() if self.position is not None and self.position.rotary_dim else None
        v_freqs = self.position.frequencies_for(self.value_dim) if self.rotate_values else None
        q = ops.rotary_split_write(qkv, bias, freqs, v_freqs, step.token_positions, tables.slot_mapping, cache.k, cache.v,
                                   self.num_heads, self.num_kv_heads, self.head_dim, self.value_dim, with_kv=writes,
                                   more_columns=gates, interleaved=self.rotation == "interleaved",
                                   unit_eps=self.unit_norm_eps, values_from_keys=self.values_are_keys)
        # (the gates stay where the projection left them: the attention kernels read them from the packed rows)
        o = ops.paged_attention(q, cache.k, cache.v, step.attention, tables.block_tables, self.scale, self.window, self.chunk,
                                softcap=self.softcap, sink=self.sink,
                                gate=(qkv, qkv.shape[1] - gates) if self.head_gate else None)
        if self.rotate_values:
            ops.turn_back_(o, v_freqs, step.token_positions)
        o = o.view(o.shape[0], self.num_heads * self.value_dim)
        if self.element_gate:
            ops.gate_rows_(o, (qkv, qkv.shape[1] - gates))
        return ops.linear(o, self.o_weight)


@MIXERS.register("differential_attention")
class DifferentialAttention(Part):
    """Softmax attention whose heads each hold two maps: queries and keys have two parts per head ([map 1 | map 2], each
    of ``head_dim`` entries, each turned by the position on its own), both maps read the same values
    (``num_kv_heads`` heads of ``value_dim``), and head h's result is
        o = a1 - lam a2,   lam = exp(lq1 . lk1) - exp(lq2 . lk2) + diff   (one number for the layer),
    divided by its root mean square over the head's entries (``eps`` under the root, no weight), times (1 - diff) and,
    with ``head_gate``, times sigmoid(w_h . x), x the mixer's input. Mask (``chunk`` or ``window``), grouping of heads,
    scale and rotation (``position``: a ``rotary_frequencies`` encoding; ``rotation`` "halves" or "interleaved") are
    those of ``RotaryAttention``; ``bias``: q, k, v and the output projection have biases.
    To the cache and the attention kernels a key head's two maps are one key of 2 ``head_dim`` entries, stored side by
    side as projected, and a query map is a head of its own, 2 ``num_heads`` in all, of 2 ``head_dim`` entries with zeros
    in the other map's place: its product with the stored key is the product with its own map. So keys and values
    are stored once, in the sizes the projections give them, and the ordinary grouping of heads holds."""

    MAPS = 2

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int, value_dim: int, scale: float,
                 diff: float, eps: float, bias: bool, position, chunk: int | None = None, window: int | None = None,
                 rotation: str = "interleaved", head_gate: bool = False):
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} heads are not a multiple of {num_kv_heads} key/value heads")
        if window and chunk:
            raise ValueError("a window or a chunk, not both")
        if rotation not in ("halves", "interleaved"):
            raise ValueError(f"rotation {rotation!r} is not known ('halves' and 'interleaved' are)")
        if not eps >= 0:
            raise ValueError(f"eps must not be negative, got {eps}")
        self.hidden_size, self.num_heads, self.num_kv_heads = hidden_size, num_heads, num_kv_heads
        self.head_dim, self.value_dim, self.scale, self.diff, self.eps = head_dim, value_dim, scale, float(diff), eps
        self.bias, self.position, self.chunk, self.window = bool(bias), position, chunk or None, window or None
        self.rotation, self.head_gate = rotation, bool(head_gate)
        self.lam = None

    def _packed_width(self) -> int:
        n = self.MAPS
        return n * (self.num_heads + self.num_kv_heads) * self.head_dim + self.num_kv_heads * self.value_dim

    def param_specs(self):
        gates = self.num_heads if self.head_gate else 0
        specs = {"qkv.weight": ParamSpec((self._packed_width() + gates, self.hidden_size)),
                 "o.weight": ParamSpec((self.hidden_size, self.num_heads * self.value_dim))}
        if self.bias:
            specs["qkv.bias"] = ParamSpec((self._packed_width(),), init="zeros")
            specs["o.bias"] = ParamSpec((self.hidden_size,), init="zeros")
        for name in ("lq1", "lk1", "lq2", "lk2"):
            specs[name] = ParamSpec((self.head_dim,), always_float32=True, init_mean=0.0, init_std=0.3)
        return specs

    def bind(self, params):
        self.qkv_weight, self.o_weight = params["qkv.weight"], params["o.weight"]
        self.qkv_bias, self.o_bias = params.get("qkv.bias"), params.get("o.bias")
        # the layer's one number, from float32 parameters in float32, once
        lam = torch.exp((params["lq1"] * params["lk1"]).sum()) - torch.exp((params["lq2"] * params["lk2"]).sum()) + self.diff
        self.lam = lam.to(torch.float32).reshape(1).contiguous()

    def cache_need(self):
        key_dim = self.MAPS * self.head_dim
        return PagedKVNeed(self.num_kv_heads, key_dim, self.window, None if self.value_dim == key_dim else self.value_dim,
                           self.chunk)

    def forward(self, x, step, cache: CacheView):
        if not cache.writes:
            raise ValueError("a layer of two maps per head keeps its own keys and values")
        tables = step.groups[cache.group]
        n, H, G = self.MAPS, self.num_heads, self.num_kv_heads
        qkv = ops.linear(x, self.qkv_weight)
        gates = H if self.head_gate else 0
        freqs = self.position.frequencies() if self.position is not None and self.position.rotary_dim else None
        q = ops.rotary_split_write(qkv, self.qkv_bias, freqs, None, step.token_positions, tables.slot_mapping, cache.k, cache.v,
                                   n * H, n * G, self.head_dim, self.value_dim, more_columns=gates,
                                   interleaved=self.rotation == "interleaved", maps=n)
        a = ops.paged_attention(q, cache.k, cache.v, step.attention, tables.block_tables, self.scale, self.window, self.chunk)
        o = ops.differential_combine(a, self.lam, self.eps, 1.0 - self.diff,
                                     gate=(qkv, qkv.shape[1] - gates) if gates else None)
        return ops.linear(o.view(o.shape[0], H * self.value_dim), self.o_weight, self.o_bias)


@MIXERS.register("gated_delta_rule")
class GatedDeltaRule(Part):
    """A recurrent mixer: per head a matrix S[head_dim, value_dim] of float32 state per request,
        S <- diag(g_t) S;  u = beta_t (v_t - S^T k_t);  S <- S + k_t u^T;  o_t = S^T q_t
    (the read-out sees the token's own write). q, k (``num_kv_heads`` heads of ``head_dim``; head h of the
    ``num_heads`` value heads uses q/k head h // (num_heads / num_kv_heads)) and v pass a causal convolution over
    time of ``conv_taps`` taps per channel and SiLU; q and k are made unit vectors per head (1e-6 under the root),
    q also times head_dim^(-1/2); beta = sigmoid(W_b x); g = exp(-exp(A_log_h) softplus(W_a2 W_a1 x + dt_bias)) per
    head and key channel; the read-out is divided by its root mean square per head (``eps``), multiplied by a weight
    over value_dim and by sigmoid(W_g2 W_g1 x), and projected. The state and the last taps - 1 inputs of the
    convolutions live in the request's state slot; a request that starts at position 0 starts from zeros.
    ``decay_rank``, ``gate_rank``: the inner sizes of the two low-rank projections; both None: the decays' and the
    gates' linear parts are plain projections of x, rows of the one packed input projection (q | k | v | beta | a | g).
    ``decay_per_head``: one decay per head (a projection row and a ``dt_bias`` entry per head) in place of one per head
    and key channel. ``gate_activation``: "sigmoid", or "silu" (the read-out times g sigmoid(g))."""

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int, value_dim: int, conv_taps: int,
                 decay_rank: int | None, gate_rank: int | None, eps: float, position=None, decay_per_head: bool = False,
                 gate_activation: str = "sigmoid"):
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} heads are not a multiple of {num_kv_heads} key heads")
        if not 1 <= conv_taps <= 16:
            raise ValueError(f"1 to 16 taps are taken, got {conv_taps}")
        self.hidden_size, self.num_heads, self.num_kv_heads = hidden_size, num_heads, num_kv_heads
        self.head_dim, self.value_dim, self.conv_taps = head_dim, value_dim, conv_taps
        if (decay_rank is None) != (gate_rank is None):
            raise ValueError("the decays' and the gates' projections are both low-rank or both plain")
        if gate_activation not in ("sigmoid", "silu"):
            raise ValueError(f"gate activation {gate_activation!r} is not known ('sigmoid' and 'silu' are)")
        self.decay_rank, self.gate_rank, self.eps = decay_rank, gate_rank, eps
        self.decay_per_head, self.gate_activation = bool(decay_per_head), gate_activation
        self.decay_dim = 1 if decay_per_head else head_dim
        self.channels = 2 * num_kv_heads * head_dim + num_heads * value_dim

    def param_specs(self):
        H, D, E, W = self.num_heads, self.head_dim, self.value_dim, self.hidden_size
        if self.decay_rank is None:
            return {
                "in.weight": ParamSpec((self.channels + H + H * self.decay_dim + H * E, W)),     # q | k | v | beta | a | g
                "conv.weight": ParamSpec((self.channels, self.conv_taps), always_float32=True, init_mean=0.0, init_std=0.5),
                "dt_bias": ParamSpec((H * self.decay_dim,), always_float32=True, init_mean=-1.0, init_std=1.0),
                "A_log": ParamSpec((H,), always_float32=True, init_mean=-1.0, init_std=0.5),
                "norm.weight": ParamSpec((E,), init="norm", always_float32=True),
                "o.weight": ParamSpec((W, H * E)),
            }
        return {
            "in.weight": ParamSpec((self.channels + H, W)),                  # q | k | v | beta
            "conv.weight": ParamSpec((self.channels, self.conv_taps), always_float32=True, init_mean=0.0, init_std=0.5),
            "a1.weight": ParamSpec((self.decay_rank, W)),
            "a2.weight": ParamSpec((H * self.decay_dim, self.decay_rank)),
            "dt_bias": ParamSpec((H * self.decay_dim,), always_float32=True, init_mean=-1.0, init_std=1.0),
            "A_log": ParamSpec((H,), always_float32=True, init_mean=-1.0, init_std=0.5),
            "g1.weight": ParamSpec((self.gate_rank, W)),
            "g2.weight": ParamSpec((H * E, self.gate_rank)),
            "norm.weight": ParamSpec((E,), init="norm", always_float32=True),
            "o.weight": ParamSpec((W, H * E)),
        }

    def cache_need(self):
        return StateNeed({"S": ((self.num_heads, self.value_dim, self.head_dim), torch.float32),
                          "kept": ((self.channels, self.conv_taps - 1), torch.float32)})

    def forward(self, x, step, cache: CacheView):
        proj = ops.linear(x, self.in_weight, out_dtype=torch.float32)
        a_lin = g_lin = None                     # (plain projections: further columns of ``proj``)
        if self.decay_rank is not None:
            a_lin = ops.linear(ops.linear(x, self.a1_weight), self.a2_weight, out_dtype=torch.float32)
            g_lin = ops.linear(ops.linear(x, self.g1_weight), self.g2_weight, out_dtype=torch.float32)
        y = ops.gated_delta_rule(proj, a_lin, g_lin, self.conv_weight, self.dt_bias, self.A_log, self.norm_weight, self.eps,
                                 cache.state["kept"], cache.state["S"], step.attention, step.state_slots, self.num_heads,
                                 self.num_kv_heads, self.head_dim, self.value_dim, x.dtype,
                                 decay_per_head=self.decay_per_head, gate_activation=self.gate_activation)
        return ops.linear(y, self.o_weight)


@MIXERS.register("normed_pair")
class NormedPair(Part):
    """Two mixers side by side that read the same rows: half the sum of their results, each first RMS-normed over
    the width (``eps``) with a plain weight vector of its own. One of them may keep pages and the other state."""

    def __init__(self, hidden_size: int, left: dict, right: dict, eps: float, position=None, **offered):
        self.hidden_size, self.eps = hidden_size, eps
        self.left = MIXERS.build(left, offered=offered, position=position)
        self.right = MIXERS.build(right, offered=offered, position=position)
        self.recordable = self.left.recordable and self.right.recordable

    def children(self):
        return {"left": self.left, "right": self.right}

    def param_specs(self):
        return {"left_out.weight": ParamSpec((self.hidden_size,), init="norm", always_float32=True),
                "right_out.weight": ParamSpec((self.hidden_size,), init="norm", always_float32=True)}

    def cache_need(self):
        return _side_by_side_need(self.left, self.right)

    defers_pair_norm = True       # ``forward(..., deferred=True)`` may return an ``ops.NormedPairMean``

    def forward(self, x, step, cache: CacheView, deferred: bool = False):
        """``deferred``: the caller's next step is a kernel that takes the two results with their norms still to do
        (``ops.depth_mix``); it then gets an ``ops.NormedPairMean`` in place of a tensor."""
        a = self.left.forward(x, step, cache)
        b = self.right.forward(x, step, cache)
        pair = ops.NormedPairMean(a, self.left_out_weight, b, self.right_out_weight, self.eps)
        return pair if deferred else pair.tensor()


def _side_by_side_need(left, right):
    """What two mixers side by side need together: at most one of them keeps pages and at most one keeps state."""
    paged = state = None
    for need in (left.cache_need(), right.cache_need()):
        if isinstance(need, PagedKVNeed):
            if paged is not None:
                raise ValueError("two mixers side by side cannot both keep pages")
            paged = need
        elif isinstance(need, StateNeed):
            if state is not None:
                raise ValueError("two mixers side by side cannot both keep state")
            state = need
    return CombinedNeed(paged, state)


@MIXERS.register("scaled_pair")
class ScaledPair(Part):
    """Two mixers side by side that read the same rows: ``left_scale`` times the left one's result plus
    ``right_scale`` times the right one's. One of them may keep pages and the other state."""

    def __init__(self, left: dict, right: dict, left_scale: float, right_scale: float, position=None, **offered):
        self.left_scale, self.right_scale = float(left_scale), float(right_scale)
        self.left = MIXERS.build(left, offered=offered, position=position)
        self.right = MIXERS.build(right, offered=offered, position=position)
        self.recordable = self.left.recordable and self.right.recordable

    def children(self):
        return {"left": self.left, "right": self.right}

    def cache_need(self):
        return _side_by_side_need(self.left, self.right)

    defers_pair_sum = True        # ``forward(..., deferred=True)`` may return an ``ops.ScaledPairSum``

    def forward(self, x, step, cache: CacheView, deferred: bool = False):
        """``deferred``: the caller's next step is a kernel that takes the two results with their sum still to do
        (``ops.streams_step``); it then gets an ``ops.ScaledPairSum`` in place of a tensor."""
        a = self.left.forward(x, step, cache)
        b = self.right.forward(x, step, cache)
        pair = ops.ScaledPairSum(a, self.left_scale, b, self.right_scale)
        return pair if deferred else pair.tensor()
