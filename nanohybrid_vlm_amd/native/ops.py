"""The kernels as Python functions over torch tensors on the GPU.

Every function checks on the host that shapes, element types and devices are what
the kernel and its grid assume, before anything is launched; a size that a kernel
does not take is refused with an error that names it. Tensors are only memory
here: the work is done by the HIP library loaded through ``ctypes`` on the
current torch stream. If the library cannot be built or loaded this raises; there
is no other implementation behind these functions.
"""
from __future__ import annotations

import ctypes
import os
import sys
from dataclasses import dataclass

import torch

from . import library

CORE_SOURCES = ["error.hip", "elementwise.hip", "gemm_generic.hip", "gemm_skinny_bf16.hip", "gemm_fewrows_bf16.hip", "attention_generic.hip",
                "sampling.hip", "measure.hip", "stream_mixing.hip", "delta_rule.hip", "parallel_block.hip", "latent_attention.hip",
                "routed_experts.hip", "hyper_streams.hip", "head_outputs.hip", "sandwich_norms.hip"]
BLAS_SOURCES = ["error.hip", "gemm_library.hip"]                                                   # the vendor's matrix library, algorithm by number
BLAS_LINK = ["-lhipblaslt"]
ATTENTION_SOURCES = ["error.hip", "attention_decode_bf16.hip", "attention_prefill_bf16.hip"]      # compiled once per head size
ATTENTION_HEAD_DIMS_BUILT_AHEAD = [16, 32, 48, 64, 80, 96, 112, 128, 256]

F32, BF16 = 0, 1
# a measured choice for a matrix product: the own kernel, or what the rule gives (0, 1, ...: that algorithm of the library's list)
OWN, RULE = -1, -2
_DTYPE_CODE = {torch.float32: F32, torch.bfloat16: BF16}


class KernelError(RuntimeError):
    """A kernel refused its arguments or failed to launch."""


def dtype_code(t: torch.Tensor) -> int:
    try:
        return _DTYPE_CODE[t.dtype]
    except KeyError:
        raise KernelError(f"element type {t.dtype} is not supported (float32 and bfloat16 are)") from None


def _ptr(t: torch.Tensor | None):
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
# torch.mm takes out_dtype (a float32 result from bfloat16 operands) from version 2.8 on
_MM_GIVES_FLOAT32 = tuple(int(p) for p in torch.__version__.split("+")[0].split(".")[:2]) >= (2, 8)


def _stream():
    """torch's current stream of the current device, as the kernels' launch argument (asked for before every
    kernel: the direct call takes a tenth of the time of building a ``torch.cuda.Stream`` object)."""
    if _raw_stream is not None:
        return ctypes.c_void_p(_raw_stream(torch.cuda.current_device()))
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _need(cond: bool, msg) -> None:
    """``msg``: the message, or a function that makes it (the checks run before every kernel: a message that
    has to be formatted is only formatted when the check fails)."""
    if not cond:
        raise KernelError(msg() if callable(msg) else msg)


def _dense(t: torch.Tensor, name: str, shape: tuple | None = None, dtype=None) -> None:
    want = backend().device_type
    if t.device.type != want:
        raise KernelError(f"{name}: must live on a '{want}' device, is on {t.device}")
    if not t.is_contiguous():
        raise KernelError(f"{name}: must be contiguous")
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise KernelError(f"{name}: shape {tuple(t.shape)} but {tuple(shape)} is needed")
    if dtype is not None and t.dtype != dtype:
        raise KernelError(f"{name}: element type {t.dtype} but {dtype} is needed")


@dataclass
class AttentionBatch:
    """What attention has to know about the step's batch (device tensors are int32)."""

    num_tokens: int
    num_requests: int
    token_req: torch.Tensor        # [T] request index of every token
    positions: torch.Tensor        # [T] absolute position of every token
    cu_seqlens_q: torch.Tensor     # [B+1] first token of every request in the batch
    context_lens: torch.Tensor     # [B] keys of the request after this step
    max_q_len: int
    max_context_len: int


def _gate_args(gate):
    """(pointer to the first gate of the first row, entries between rows) of a gate given as (tensor, first column)."""
    if gate is None:
        return ctypes.c_void_p(0), ctypes.c_longlong(0)
    t, col = gate
    return ctypes.c_void_p(t.data_ptr() + col * t.element_size()), ctypes.c_longlong(t.shape[1])


class NativeBackend:
    """ctypes calls into the HIP library."""

    name = "hip"
    device_type = "cuda"
    few_rows = 16                 # up to this many rows the own matrix kernels are the rule
    library_rows = 64             # up to this many rows the way a product is done may be chosen by measurement (see _choose)
    library_algorithms = 48       # so many of the library's algorithms are asked for and tried
    library_workspace = 32 << 20  # bytes of scratch memory the library's algorithms may use
    own_kernels_only = False      # True: no library call (matrix products of up to 64 rows take the own kernels)
    planned_context = 0           # > 0 while a HIP graph is recorded: the lengths to plan for (the batch's own are bounds)
    covered_context = 0           # and the longest context that the recorder will let the graph meet
    measure_linears = False       # True: a product of few rows and a shape not seen before is timed in every way there is (see _choose)
    measure_many_rows = True      # a product of more than library_rows rows is timed in the third step that meets its shape
    measuring_allowed = True      # False: nothing is ever timed; a shape follows the table that was loaded, or the rule
    fuse_norms = True             # products of up to few_rows rows may take over the residual addition and the norm around them (see Summed, Normed)
    step_number = 0               # counted by the engine, one per eager step

    def __init__(self):
        if not torch.cuda.is_available():
            raise KernelError("no GPU is visible to torch; the HIP kernels are the only implementation")
        self.lib = library.load_library("nhv_core", CORE_SOURCES)
        self.lib.nhv_last_error.restype = ctypes.c_char_p
        self._attention_libs: dict[int, ctypes.CDLL] = {}
        # (M, N, K, float result, gated) of a product -> OWN, RULE or a library algorithm, measured. ``chosen`` is the
        # table in force: the process-wide one that engines share by default (a shape is timed once per process), or
        # the table of the engine that runs now (see ``use_choices``)
        self.shared_chosen: dict[tuple, int] = {}
        self.chosen: dict[tuple, int] = self.shared_chosen
        self._blas = None
        self._plans: dict[tuple, tuple[int, int]] = {}
        self.times: dict[tuple, tuple[float, float]] = {}   # measured shape -> (ms of the own kernel, ms of the library's best), cold
        self._met: dict[tuple, tuple[int, int]] = {}        # shape of many rows -> (steps that met it, the last of them)
        self._workspace = None
        self._sweep = None                                  # scratch memory whose reading empties the caches before a measurement

    def _call(self, fn_name: str, *args, lib=None) -> None:
        lib = lib or self.lib
        rc = getattr(lib, fn_name)(*args)
        if rc != 0:
            raise KernelError(lib.nhv_last_error().decode())

    def attention_lib(self, head_dim: int) -> ctypes.CDLL:
        """The bfloat16 attention kernels are compiled per head size, when a model first needs them."""
        lib = self._attention_libs.get(head_dim)
        if lib is None:
            lib = library.load_library(f"nhv_attention_d{head_dim}", ATTENTION_SOURCES, [f"-DNHV_HEAD_DIM={head_dim}"])
            lib.nhv_last_error.restype = ctypes.c_char_p
            self._attention_libs[head_dim] = lib
        return lib

    # -- each method launches one kernel; arguments were checked by the caller --
    def embed(self, ids, table, out, scale=1.0):
        T, H = out.shape
        self._call("nhv_embed", _ptr(ids), _ptr(table), _ptr(out), T, H, table.shape[0], dtype_code(table),
                   ctypes.c_float(scale), _stream())

    def soft_cap(self, x, cap):
        self._call("nhv_soft_cap", _ptr(x), ctypes.c_size_t(x.numel()), ctypes.c_float(cap), _stream())

    def rmsnorm(self, x, residual, residual_mode, w, y, eps):
        T, H = x.shape
        self._call("nhv_rmsnorm", _ptr(x), _ptr(residual), residual_mode,
                   F32 if residual is None else dtype_code(residual), _ptr(w), _ptr(y), T, H, ctypes.c_float(eps),
                   dtype_code(x), dtype_code(w), _stream())

    def silu_mul(self, gu, out):
        T, I = out.shape
        self._call("nhv_silu_mul", _ptr(gu), _ptr(out), T, I, dtype_code(gu), _stream())

    def gather_rows(self, x, rows, out):
        self._call("nhv_gather_rows", _ptr(x), _ptr(rows), _ptr(out), out.shape[0], x.shape[1], x.shape[0],
                   dtype_code(x), _stream())

    def qk_rope_write(self, qkv, bias, q_norm_w, k_norm_w, eps, cos_sin, rot, positions, slot_mapping,
                      q_out, k_cache, v_cache, Hq, Hkv, D, write_kv, pair_axes=None):
        wd = dtype_code(q_norm_w) if q_norm_w is not None else dtype_code(qkv)
        self._call("nhv_qk_rope_write", _ptr(qkv), _ptr(bias), _ptr(q_norm_w), _ptr(k_norm_w), ctypes.c_float(eps),
                   _ptr(cos_sin), rot, 0 if cos_sin is None else cos_sin.shape[0], _ptr(positions), _ptr(pair_axes),
                   _ptr(slot_mapping),
                   _ptr(q_out), _ptr(k_cache), _ptr(v_cache), qkv.shape[0], Hq, Hkv, D, int(write_kv),
                   dtype_code(qkv), wd, _stream())

    def paged_attention(self, q, k_cache, v_cache, out, batch: AttentionBatch, block_tables, scale, window, chunk=0,
                        cap=0.0, sink=None, gate=None):
        """``cap``: scores become cap tanh(score / cap); ``sink``: the score of one more term in the denominator;
        ``gate`` = (tensor [tokens, columns] of q's element type, first column): the sigmoid of column + head
        multiplies the head's result."""
        T, Hq, D = q.shape
        _, page_size, Hkv, _ = k_cache.shape
        E = v_cache.shape[3]
        plain = not cap and sink is None and gate is None
        more = () if plain else (ctypes.c_float(cap or 0.0), int(sink is not None), ctypes.c_float(sink or 0.0), *_gate_args(gate))
        # the kernels on the matrix cores take value heads of the key heads' size; a chunk goes to them as a negative window
        fast = q.dtype == torch.bfloat16 and E == D and D % 16 == 0 and D <= 256
        if chunk:
            window = -chunk
        if fast and batch.max_q_len == 1 and Hq // Hkv <= 16 and T <= 65535:
            return self._decode_attention(q, k_cache, v_cache, out, batch, block_tables, scale, window, more)
        if fast and plain and batch.max_q_len == 1 and Hkv == 1 and T <= 65535:
            # more than 16 query heads on one key/value head (a cached latent): sixteen heads at a time
            for h0 in range(0, Hq, 16):
                part = torch.empty((T, min(16, Hq - h0), E), dtype=out.dtype, device=out.device)
                self._decode_attention(q[:, h0:h0 + 16].contiguous(), k_cache, v_cache, part, batch, block_tables, scale, window)
                out[:, h0:h0 + 16] = part
            return None
        if fast and batch.num_requests <= 65535 and Hkv <= 65535:
            # prompt portions (and whatever single tokens share their batch) on the matrix cores
            return self._call("nhv_prefill_attention_bf16" + ("_more" if more else ""), _ptr(q), _ptr(k_cache), _ptr(v_cache),
                              _ptr(out), _ptr(batch.cu_seqlens_q), _ptr(batch.context_lens), _ptr(block_tables),
                              block_tables.shape[1], batch.num_requests, batch.max_q_len, Hq, Hkv, page_size,
                              ctypes.c_float(scale), window, *more, _stream(), lib=self.attention_lib(D))
        self._call("nhv_paged_attention_generic", _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(out),
                   _ptr(batch.token_req), _ptr(batch.positions), _ptr(block_tables), block_tables.shape[1], T, Hq, Hkv,
                   D, E, page_size, ctypes.c_float(scale), 0 if chunk else window, chunk, ctypes.c_float(cap or 0.0),
                   int(sink is not None), ctypes.c_float(sink or 0.0), *_gate_args(gate), dtype_code(q), _stream())

    # -- layers that are not the pre-norm kind: norms with one number, sums over depth, rotation without a table --
    def scalar_rmsnorm(self, x, gain, y, eps):
        T, W = x.shape
        self._call("nhv_scalar_rmsnorm", _ptr(x), dtype_code(x), _ptr(gain), _ptr(y), dtype_code(y), T, W,
                   ctypes.c_float(eps), _stream())

    def pair_norm_mean(self, a, wa, b, wb, y, eps):
        T, W = a.shape
        self._call("nhv_pair_norm_mean", _ptr(a), _ptr(wa), _ptr(b), _ptr(wb), _ptr(y), T, W, ctypes.c_float(eps),
                   dtype_code(a), _stream())

    def depth_mix(self, x, a, b, results, index, weights, out, gain, normed, eps, pair=None):
        T, W = x.shape
        a2, wa, wb, pair_eps = pair if pair is not None else (None, None, None, 0.0)
        self._call("nhv_depth_mix", _ptr(x), _ptr(a), _ptr(b), _ptr(results), ctypes.c_longlong(results.stride(0)), index,
                   _ptr(weights), _ptr(out), _ptr(gain), _ptr(normed), T, W, ctypes.c_float(eps), _ptr(a2), _ptr(wa),
                   _ptr(wb), ctypes.c_float(pair_eps), dtype_code(a), _stream())

    def rotary_split_write(self, qkv, bias, qk_freqs, rot, v_freqs, positions, slot_mapping, q_out, k_cache, v_cache,
                           Hq, Hkv, D, E, with_kv, more_columns=0, interleaved=False, unit_eps=None, values_from_keys=False,
                           maps=1):
        self._call("nhv_rotary_split_write", _ptr(qkv), _ptr(bias), _ptr(qk_freqs), rot, _ptr(v_freqs), _ptr(positions),
                   _ptr(slot_mapping), _ptr(q_out), _ptr(k_cache), _ptr(v_cache), qkv.shape[0], Hq, Hkv, D, E,
                   int(with_kv), more_columns, int(interleaved), int(unit_eps is not None), ctypes.c_float(unit_eps or 0.0),
                   int(values_from_keys), maps, dtype_code(qkv), _stream())

    # -- what heads' results pass before the output projection; a layer normed on both sides of its sublayers --
    def differential_combine(self, a, lam, out, eps, post, gate=None):
        T, H, E = out.shape
        self._call("nhv_differential_combine", _ptr(a), _ptr(lam), _ptr(out), T, H, E, ctypes.c_float(eps),
                   ctypes.c_float(post), *_gate_args(gate), dtype_code(a), _stream())

    def gate_rows(self, x, gate):
        T, N = x.shape
        self._call("nhv_gate_rows", _ptr(x), *_gate_args(gate), T, N, dtype_code(x), _stream())

    def sandwich_step(self, x, y, wb, eps_b, wa, eps_a, h):
        T, W = x.shape
        self._call("nhv_sandwich_step", _ptr(x), _ptr(y), dtype_code(y) if y is not None else 0, _ptr(wb),
                   ctypes.c_float(eps_b), _ptr(wa), ctypes.c_float(eps_a), _ptr(h), dtype_code(h) if h is not None else 0,
                   T, W, _stream())

    def turn_back(self, x, freqs, positions):
        T, H, E = x.shape
        self._call("nhv_turn_back", _ptr(x), _ptr(freqs), _ptr(positions), T, H, E, dtype_code(x), _stream())

    # -- the gated delta rule --
    def delta_prepare(self, proj, taps, kept, a_lin, dt_bias, a_log, batch, state_slots, q, k, v, beta, H, G, D, E,
                      decay=None, a_col=0):
        """``a_lin`` [tokens, columns] float32: the decays' linear part from column ``a_col`` on; ``decay``
        [tokens, heads, 1 or D]: where the decays go (None: into ``a_lin`` itself, which then holds nothing else)."""
        decay_dim = D if decay is None else decay.shape[2]
        self._call("nhv_delta_prepare", _ptr(proj), dtype_code(proj), proj.shape[1], _ptr(taps), taps.shape[1], _ptr(kept),
                   ctypes.c_void_p(a_lin.data_ptr() + 4 * a_col), ctypes.c_longlong(a_lin.shape[1]),
                   _ptr(a_lin if decay is None else decay), _ptr(dt_bias), _ptr(a_log), _ptr(batch.token_req),
                   _ptr(batch.positions), _ptr(batch.cu_seqlens_q), _ptr(state_slots), _ptr(q), _ptr(k), _ptr(v), _ptr(beta),
                   proj.shape[0], H, G, D, E, decay_dim, _stream())

    def conv_state_update(self, proj, kept, n_taps, batch, state_slots, channels):
        self._call("nhv_conv_state_update", _ptr(proj), dtype_code(proj), proj.shape[1], _ptr(kept), n_taps,
                   _ptr(batch.positions), _ptr(batch.cu_seqlens_q), _ptr(state_slots), batch.num_requests, channels,
                   _stream())

    def delta_rule(self, q, k, v, decay, beta, state, out, batch, state_slots):
        T, G, D = q.shape
        _, H, E = v.shape
        self._call("nhv_delta_rule", _ptr(q), _ptr(k), _ptr(v), _ptr(decay), _ptr(beta), _ptr(state), _ptr(out),
                   _ptr(batch.positions), _ptr(batch.cu_seqlens_q), _ptr(state_slots), batch.num_requests, H, G, D, E,
                   max(1, batch.max_q_len), decay.shape[2], _stream())

    def gated_head_norm(self, o, gate, w, y, eps, gate_col=0, gate_act=0):
        """``gate`` [tokens, columns] float32: the gates of (t, h, e) from column ``gate_col`` on; ``gate_act`` 0: the
        sigmoid, 1: SiLU."""
        T, H, E = o.shape
        self._call("nhv_gated_head_norm", _ptr(o), ctypes.c_void_p(gate.data_ptr() + 4 * gate_col),
                   ctypes.c_longlong(gate.shape[1]), _ptr(w), _ptr(y), T, H, E, ctypes.c_float(eps), dtype_code(y),
                   gate_act, _stream())

    # -- several residual streams side by side, and what models on them need --
    def streams_step(self, X, x0, mix, out_w, a, b, sa, sb, in_w, norm_w, eps, h, total, n, T, W, rows_dtype):
        self._call("nhv_streams_step", _ptr(X), ctypes.c_longlong(0 if X is None else X.stride(0)), _ptr(x0), _ptr(mix),
                   _ptr(out_w), _ptr(a), _ptr(b), ctypes.c_float(sa), ctypes.c_float(sb), _ptr(in_w), _ptr(norm_w),
                   ctypes.c_float(eps), _ptr(h), _ptr(total), n, T, W, _DTYPE_CODE[rows_dtype], _stream())

    def embed_float(self, ids, table, out, scale):
        T, W = out.shape
        self._call("nhv_embed_float", _ptr(ids), _ptr(table), _ptr(out), T, W, table.shape[0], dtype_code(table),
                   ctypes.c_float(scale), _stream())

    def activation(self, x, act):
        self._call("nhv_activation", _ptr(x), ctypes.c_size_t(x.numel()), act, dtype_code(x), _stream())

    def scaled_sum(self, a, b, y, sa, sb):
        self._call("nhv_scaled_sum", _ptr(a), _ptr(b), _ptr(y), ctypes.c_size_t(y.numel()), ctypes.c_float(sa),
                   ctypes.c_float(sb), dtype_code(a), _stream())

    def scale(self, x, factor):
        self._call("nhv_scale", _ptr(x), ctypes.c_size_t(x.numel()), ctypes.c_float(factor), _stream())

    # -- layers of two norms side by side, an embedding with a hashed pair row --
    def embed_pair_hash(self, ids, table, pair_table, out, batch, state_slots, prev_state, buckets, mul_prev, mul_cur):
        T, W = out.shape
        self._call("nhv_embed_pair_hash", _ptr(ids), _ptr(table), _ptr(pair_table), _ptr(out), _ptr(batch.positions),
                   _ptr(batch.cu_seqlens_q), _ptr(batch.token_req), _ptr(state_slots), _ptr(prev_state), T, W,
                   table.shape[0], buckets, mul_prev, mul_cur, dtype_code(table), _stream())

    def layernorm_pair(self, x, a, b, w1, b1, y1, w2, b2, y2, eps, rows_dtype):
        T, W = x.shape
        self._call("nhv_layernorm_pair", _ptr(x), _ptr(a), _ptr(b), _ptr(w1), _ptr(b1), _ptr(y1), _ptr(w2), _ptr(b2),
                   _ptr(y2), T, W, ctypes.c_float(eps), _DTYPE_CODE[rows_dtype], _stream())

    def add_streams(self, x, a, b):
        self._call("nhv_add_streams", _ptr(x), _ptr(a), _ptr(b), ctypes.c_size_t(x.numel()), dtype_code(a), _stream())

    def act_mul(self, gu, out, act):
        T, I = out.shape
        self._call("nhv_gelu_tanh_mul" if act == 1 else "nhv_silu_mul", _ptr(gu), _ptr(out), T, I, dtype_code(gu), _stream())

    # -- attention over a cached latent --
    def latent_prepare(self, a, q_off, q_rank, c_off, kv_rank, rot, wq, wc, eps, freqs, gain, positions, slot_mapping,
                       cache, cq):
        self._call("nhv_latent_prepare", _ptr(a), a.shape[1], q_off, q_rank, c_off, kv_rank, rot, _ptr(wq), _ptr(wc),
                   ctypes.c_float(eps), _ptr(freqs), ctypes.c_float(gain), _ptr(positions), _ptr(slot_mapping), _ptr(cache),
                   0 if cache is None else cache.shape[-1], _ptr(cq), a.shape[0], dtype_code(cq), _stream())

    def head_gemm(self, x, x_off, x_row, w, w_head, w_n, w_k, y, y_off, y_row, gate, gate_off, N, K, turn=None):
        """y[t, h, y_off : y_off + N] = M_h x[t, h, x_off : x_off + K]; x and y are [rows, heads, x_row / y_row].
        ``turn`` = (rot, x_rot_off, y_rot_off, freqs, gain, positions): also y[t, h, y_rot_off ...] = the ``rot`` entries
        of x from x_rot_off on, turned. Returns whether the turning was done (up to 16 rows: in the same launch)."""
        T, H = x.shape[0], x.shape[1]
        item = x.element_size()
        LL = ctypes.c_longlong
        gate_p = None if gate is None else ctypes.c_void_p(gate.data_ptr() + 4 * gate_off)
        x_p, y_p = ctypes.c_void_p(x.data_ptr() + item * x_off), ctypes.c_void_p(y.data_ptr() + item * y_off)
        gs_t = LL(0 if gate is None else gate.shape[1])
        if T <= 16 and 16 * K * 4 + (64 * item + 16) * K <= 96 * 1024:      # (the kernel keeps the rows and a piece of the matrix in LDS)
            rot, xr, yr, freqs, gain, positions = turn if turn is not None else (0, 0, 0, None, 1.0, None)
            self._call("nhv_head_gemm_fewrows", x_p, LL(H * x_row), LL(x_row), _ptr(w), LL(w_head), LL(w_n), LL(w_k), y_p,
                       LL(H * y_row), LL(y_row), gate_p, gs_t, T, H, N, K, rot, xr - x_off, yr - y_off, _ptr(freqs),
                       ctypes.c_float(gain), _ptr(positions), dtype_code(x), _stream())
            return True
        if x.dtype == torch.bfloat16 and not self.own_kernels_only and (gate is None or (y_off == 0 and y_row == N)):
            # many rows: the library's batched product, one matrix per head, on strided views
            xv = x[:, :, x_off:x_off + K].transpose(0, 1)                         # [H, T, K]
            wv = torch.as_strided(w, (H, K, N), (w_head, w_k, w_n))
            yv = y[:, :, y_off:y_off + N].transpose(0, 1)
            yv.copy_(torch.bmm(xv, wv))
            if gate is not None:
                self._call("nhv_head_gate", _ptr(y), gate_p, gs_t, T, H, N, dtype_code(y), _stream())
            return False
        self._call("nhv_head_gemm", x_p, LL(H * x_row), LL(x_row), _ptr(w), LL(w_head), LL(w_n), LL(w_k), y_p, LL(H * y_row),
                   LL(y_row), gate_p, gs_t, T, H, N, K, dtype_code(x), _stream())
        return False

    def rotate_interleaved(self, src, s_off, dst, d_off, rot, freqs, gain, positions):
        T, H, s_row = src.shape
        self._call("nhv_rotate_interleaved", _ptr(src), s_row, s_off, _ptr(dst), dst.shape[2], d_off, rot, _ptr(freqs),
                   ctypes.c_float(gain), _ptr(positions), T, H, dtype_code(src), _stream())

    # -- a feed-forward of many small experts --
    def route_topk(self, logits, ids, scores, bias=None, mode=0):
        T, E = logits.shape
        self._call("nhv_route_topk", _ptr(logits), _ptr(bias), _ptr(ids), _ptr(scores), T, E, ids.shape[1], mode, _stream())

    def experts_gate_up(self, h, ids, scores, gate_up, u, act):
        T, W = h.shape
        E, F2, _ = gate_up.shape
        self._call("nhv_experts_gate_up", _ptr(h), _ptr(ids), _ptr(scores), _ptr(gate_up), _ptr(u), T, W, F2 // 2,
                   ids.shape[1], E, act, dtype_code(h), _stream())

    def experts_grouped(self, h, ids, scores, gate_up, down, out, act, weights=None, add=None):
        """Many rows in bfloat16: the pairs sorted by expert, then both products on the matrix cores, then the sum over
        a token's experts."""
        T, W = h.shape
        E, F2, _ = gate_up.shape
        F, top = F2 // 2, ids.shape[1]
        P = T * top
        # places a tile (runs of an expert's pairs are filled up to whole tiles): 128 or 64 where an expert has pairs
        # enough (block tiles of 128 x 128 and 64 x 128 matrix rows). Tiles of 128 pairs x 256 matrix rows, which the
        # kernel can be built for as well, took the time of 64 x 128 at 4,096 pairs of 16 experts: half the bytes from
        # L2, but one block a compute unit, which then waits for every piece; 128 x 128 takes a tenth less.
        TM = 128 if P >= 192 * E else (64 if P >= 32 * E else 16)
        tiles = -(-P // TM) + E
        index = torch.empty(tiles * TM + tiles, dtype=torch.int32, device=h.device)
        sorted_pairs, tile_expert = index[:tiles * TM], index[tiles * TM:]
        self._call("nhv_experts_sort", _ptr(ids), P, E, TM, _ptr(sorted_pairs), tiles * TM, _ptr(tile_expert), tiles, _stream())
        u = torch.empty((P, F), dtype=h.dtype, device=h.device)
        self._call("nhv_experts_grouped_gate_up", _ptr(h), _ptr(gate_up), _ptr(u), _ptr(sorted_pairs), _ptr(tile_expert),
                   _ptr(scores), top, W, F, act, TM, tiles, _stream())
        y = torch.empty((P, W), dtype=torch.float32, device=h.device)
        self._call("nhv_experts_grouped_down", _ptr(u), _ptr(down), _ptr(y), _ptr(sorted_pairs), _ptr(tile_expert), W, F, TM,
                   tiles, _stream())
        self._call("nhv_experts_combine", _ptr(y), _ptr(out), T, W, top, _ptr(weights), _ptr(add), _stream())

    def experts_down(self, u, ids, down, out, weights=None, add=None):
        T, W = out.shape
        E, _, F = down.shape
        self._call("nhv_experts_down", _ptr(u), _ptr(ids), _ptr(down), _ptr(out), T, W, F, ids.shape[1], E,
                   _ptr(weights), _ptr(add), dtype_code(u), _stream())

    def _decode_attention(self, q, k_cache, v_cache, out, batch, block_tables, scale, window, more=()):
        """Single tokens in bfloat16: keys split over waves, then merged. ``more``: the arguments of a cap on the
        scores, a further term in the denominator and a gate per head, for the entry point that takes them."""
        T, Hq, D = q.shape
        _, page_size, Hkv, _ = k_cache.shape
        # inside a graph the lengths are only bounded (by max_model_len): the recorder says what to plan for
        span = min(self.planned_context, batch.max_context_len) if self.planned_context else batch.max_context_len
        if window:                                   # (a chunk comes as a negative window)
            span = min(span, abs(window) + 64)
        # One wave per SIMD of the chip (about a thousand) is the fastest while that leaves splits of up to 256
        # keys, half as many waves again from there on (a wave takes its keys one round after the other), and no
        # split is longer than 1,024 keys. Measured at 2,176 and 8,192 keys, 1 to 64 requests, 8 key/value heads: the
        # best split length is 64 to 128 keys for 8 x 2,176 keys in all, 256 for 32 x 2,176 (62 against 64 us with
        # 512), 512 for 48 and 64 x 2,176 (110 against 118 us with 1,024) and for 16 x 8,192, 1,024 for 32 x 8,192.
        want = max(1, T * Hkv * span // 1024)
        want = min(want, max(256, want * 2 // 3))
        # (splits of one round of 32 keys for one request of 2,100 keys, 525 waves: 3.64 against 3.66 ms a step; for two
        # requests 3.77 against 3.75: not taken)
        split_len = 64
        while split_len * 2 <= want and split_len < 1024:
            split_len *= 2
        # the splits cover the longest context this launch can meet: outside a graph the batch's own; inside one, what
        # the recorder says it will let the graph meet (``covered_context``: it replaces a graph before its contexts
        # outgrow that), not the bound of the block tables (max_model_len), whose splits would nearly all be empty blocks
        covered = batch.max_context_len
        if self.planned_context and self.covered_context:
            covered = min(covered, self.covered_context)
        n_splits = -(-covered // split_len)
        part_o = torch.empty((T, Hq, n_splits, D), dtype=torch.float32, device=q.device)
        part_ml = torch.empty((T, Hq, n_splits, 2), dtype=torch.float32, device=q.device)
        self._call("nhv_decode_attention_bf16" + ("_more" if more else ""), _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(out),
                   _ptr(part_o), _ptr(part_ml), _ptr(batch.token_req), _ptr(batch.positions), _ptr(block_tables),
                   block_tables.shape[1], T, Hq, Hkv, page_size, ctypes.c_float(scale), window, split_len, n_splits,
                   *more, _stream(), lib=self.attention_lib(D))

    # -- matrix products of few rows: own kernel or one of the library's algorithms, by measurement --
    def blas_lib(self) -> ctypes.CDLL:
        """The wrapper of the vendor's matrix library, loaded when a product is first given to it."""
        if self._blas is None:
            self._blas = library.load_library("nhv_blas", BLAS_SOURCES, link=BLAS_LINK)
            self._blas.nhv_last_error.restype = ctypes.c_char_p
        return self._blas

    def _library_plan(self, M: int, N: int, K: int, float_result: bool) -> tuple[int, int]:
        """(plan, number of algorithms) of the library for this shape."""
        key = (M, N, K, float_result)
        got = self._plans.get(key)
        if got is None:
            plan, count = ctypes.c_int(), ctypes.c_int()
            self._call("nhv_library_gemm_plan", M, N, K, F32 if float_result else BF16, self.library_algorithms,
                       ctypes.c_size_t(self.library_workspace), ctypes.byref(plan), ctypes.byref(count), lib=self.blas_lib())
            got = self._plans[key] = (plan.value, count.value)
        return got

    def _library_product(self, x, w, out, algorithm: int) -> None:
        plan, _ = self._library_plan(x.shape[0], w.shape[0], x.shape[1], out.dtype == torch.float32)
        if self._workspace is None:
            self._workspace = torch.empty(self.library_workspace, dtype=torch.uint8, device=x.device)
        self._call("nhv_library_gemm", plan, algorithm, _ptr(x), _ptr(w), _ptr(out), _ptr(self._workspace),
                   ctypes.c_size_t(self.library_workspace), _stream(), lib=self.blas_lib())

    def _time_cold(self, run, repeats: int) -> float:
        """The shortest of ``repeats`` runs in milliseconds, each alone and after a read of 512 MB has swept the
        caches (the memory-side one holds 256 MB): in a decoding step a weight comes from memory, and a weight
        left in a cache by the run before would be measured 15 to 20 % too fast, by an amount that differs from
        kernel to kernel. The sweep reads, as the step before a product does: after a sweep that writes, the
        caches are full of lines that have to go back to memory while the product runs, which adds 10 to 35 us."""
        times = []
        for _ in range(repeats):
            self._sweep.sum()
            start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record()
            run()
            end.record()
            end.synchronize()
            times.append(start.elapsed_time(end))
        return min(times)

    def _choose(self, x, w, out, gated: bool = False) -> int | None:
        """How this product is done: ``OWN`` (the own kernel; with ``gated`` the one that also does the
        SiLU-and-multiply), the number of one of the library's algorithms (``gated``: followed by the
        SiLU-and-multiply kernel), ``RULE`` (measured, and nothing beat what the rule gives), or ``None`` if the
        shape was never measured (then the rule holds too: own kernel up to ``few_rows`` rows, ``torch.mm`` above).
        Which is fastest depends on the shape in ways no rule here captures, and the library's own first guess is
        often far from its best (a 5120 x 17408 weight against 8 rows: 112 us by its first guess, 37 us by another
        of its algorithms, 50 us by the own kernel; a 4096 x 12288 weight: 22, 22 and 25 us; the same weight
        against 128 rows: 67 us by ``torch.mm``, 43 us by the library's sixth guess; against 2,048 rows the first
        guess is as good as any). So a shape is timed in
        every way there is, once, and the answer is kept for the life of the process: a shape of up to
        ``library_rows`` rows while ``measure_linears`` is set (the run before a graph is recorded), a shape of
        more rows (a portion of a prompt) in the third step that meets it, since only the sizes that come again
        and again (portions that fill the token budget) are worth the 50 ms. An algorithm whose result differs
        from the trusted way's (own kernel, ``torch.mm``) by more than rounding, or from its own on a second run,
        is left out. The trusted way stays unless a library algorithm takes less than 0.95 of its time (0.90 for the
        gated projection)."""
        M, K = x.shape
        N = w.shape[0]
        float_result = out.dtype == torch.float32
        key = (M, N, K, float_result, gated)
        known = self.chosen.get(key)
        if known is not None or not self.measuring_allowed or torch.cuda.is_current_stream_capturing():
            return known
        many = M > self.library_rows
        if many:
            met, step = self._met.get(key, (0, -1))
            if step != self.step_number:                     # (a model's layers meet the same shape in one step)
                met += 1
                self._met[key] = (met, self.step_number)
            if not self.measure_many_rows or (met < 3 and not self.measure_linears):
                return None                                  # (before a graph is recorded every new shape is measured at once)
        elif not self.measure_linears:
            return None
        try:
            how = self._measure(x, w, out, gated, many)
        except torch.OutOfMemoryError:
            how = RULE if many else None                     # no room to measure: the rule
        finally:
            if many:
                self._sweep = None                           # (a step of prompt portions is followed by no end_measurements)
        if how is not None:
            self.chosen[key] = how
            if gated and how >= 0:
                self.chosen[(M, N, K, False, False)] = how   # the packed product that follows a refusal of gated_linear
        return how

    def _measure(self, x, w, out, gated: bool, many: bool) -> int:
        M, K = x.shape
        N = w.shape[0]
        float_result = out.dtype == torch.float32
        if self._sweep is None:
            self._sweep = torch.zeros(128 << 20, dtype=torch.float32, device="cuda")      # (a sum of floats is one kernel and no copy)
        packed = torch.empty((M, N), dtype=x.dtype, device=x.device) if gated else out

        def trusted():
            if many:
                torch.mm(x, w.t(), out=out)
            elif gated:
                self._call("nhv_gemm_skinny_glu_bf16", _ptr(x), _ptr(w), _ptr(out), M, N // 2, K, dtype_code(out), _stream())
            else:
                self._call("nhv_gemm_skinny_bf16", _ptr(x), _ptr(w), None, _ptr(out), M, N, K, dtype_code(out), _stream())

        def by_library(algorithm):
            def run():
                self._library_product(x, w, packed, algorithm)
                if gated:
                    self.silu_mul(packed, out)
            return run

        trusted()
        reference = out.clone()
        bound = (1e-3 if float_result else 2e-2) * max(float(reference.abs().max()), 1e-30)
        incumbent = RULE if many else OWN
        runs = {incumbent: trusted} if many or M <= self.few_rows else {}
        _, count = self._library_plan(M, N, K, float_result and not gated)
        for algorithm in range(min(count, 16) if many else count):
            run = by_library(algorithm)
            try:
                out.zero_()
                run()
                first = out.clone()
                out.zero_()
                run()
            except KernelError:
                continue
            if torch.equal(first, out) and float((out - reference).abs().max()) <= bound:
                runs[algorithm] = run
            del first
        if not runs:
            return RULE                                      # the library has no algorithm for this shape that holds
        # every way once; then the four fastest, and the trusted way whatever its place, eight times more each (the
        # shortest run counts: a single run is off by up to a tenth, and a choice made on it changes from one start of
        # the engine to the next, by up to 5 % of a decoding step)
        once = sorted((self._time_cold(run, 1), how) for how, run in runs.items())
        finalists = once[:4] + [(t, h) for t, h in once[4:] if h == incumbent]
        best = sorted((min(t, self._time_cold(runs[how], 8)), how) for t, how in finalists)
        how = best[0][1]
        incumbent_time = next((t for t, h in best + once if h == incumbent), None)
        # (the fused gated kernel gives way only to a clear win: the library's way is two kernels, and the second one's
        # cost inside a step is the harder one to measure alone)
        if incumbent_time is not None and how != incumbent and best[0][0] >= (0.90 if gated else 0.95) * incumbent_time:
            how = incumbent
        library_times = [t for t, h in best + once if h >= 0]
        if incumbent_time is not None and library_times:
            self.times[(M, N, K, float_result, gated)] = (incumbent_time, min(library_times))
        if os.environ.get("NHV_SHOW_MEASUREMENTS"):
            name = {OWN: "own", RULE: "torch.mm"}
            first_guess = next((t for t, h in once if h == 0), float("nan"))
            print(f"[nanohybrid_vlm_amd] {'gated ' if gated else ''}product {M} x {K} . {N} x {K}: {name[incumbent]} "
                  f"{'-' if incumbent_time is None else format(1e3 * incumbent_time, '.1f')} us, library's first guess "
                  f"{1e3 * first_guess:.1f} us, fastest {1e3 * best[0][0]:.1f} us ({name.get(best[0][1], best[0][1])} "
                  f"of {len(runs)} ways); taken: {name.get(how, how)}", file=sys.stderr, flush=True)
        return how

    # -- the table of choices, so that a process can run by what another one measured --
    def choices_table(self, chosen: dict | None = None) -> dict[str, int]:
        """A table of choices (default: the one in force), by shape: "M,N,K,float result,gated" -> -1 (own kernel),
        -2 (the rule: ``torch.mm``) or the number of a library algorithm."""
        chosen = self.chosen if chosen is None else chosen
        return {",".join(str(int(v)) for v in key): how for key, how in sorted(chosen.items())}

    def parse_choices(self, table: dict[str, int]) -> dict[tuple, int]:
        """A table as ``choices_table`` gives it, as a table of this backend's own kind. Every entry is checked
        now: its shape's form, and a library algorithm's number against the library's list for that shape."""
        out = {}
        for text, how in table.items():
            parts = text.split(",")
            if len(parts) != 5:
                raise KernelError(f"a product's shape is 'M,N,K,float result,gated', got '{text}'")
            M, N, K, f, g = (int(v) for v in parts)
            if not isinstance(how, int) or how < RULE:
                raise KernelError(f"choice {how!r} for the product '{text}' is neither -1, -2 nor an algorithm's number")
            if how >= 0:
                _, count = self._library_plan(M, N, K, bool(f) and not bool(g))
                if how >= count:
                    raise KernelError(f"choice {how} for the product '{text}': the library names {count} algorithms for this shape")
            out[(M, N, K, bool(f), bool(g))] = how
        return out

    def use_choices(self, table: dict | None, measuring: bool) -> None:
        """Puts an engine's table in force (None: the process-wide one) and says whether shapes that it lacks may be timed."""
        self.chosen = self.shared_chosen if table is None else table
        self.measuring_allowed = bool(measuring)

    def end_measurements(self) -> None:
        """Gives the scratch memory of the measurements back (what was measured stays known)."""
        self._sweep = None

    def linear(self, x, w, bias, out):
        M, K = x.shape
        N = w.shape[0]
        if x.dtype == torch.bfloat16 and K % 8 == 0 and x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0:
            if bias is None and not self.own_kernels_only and (M <= self.library_rows or out.dtype == torch.bfloat16):
                how = self._choose(x, w, out)
                if how is not None and how >= 0:
                    return self._library_product(x, w, out, how)
            if M <= self.few_rows or (M <= 64 and self.own_kernels_only):
                return self._call("nhv_gemm_skinny_bf16", _ptr(x), _ptr(w), _ptr(bias), _ptr(out), M, N, K,
                                  dtype_code(out), _stream())
            if out.dtype == torch.bfloat16 and not self.own_kernels_only:
                # many rows: the library's matrix product (the reference's linears are library calls too,
                # nanovllm/layers/linear.py:88,192); a bias joins the rounded rows in a kernel of its own
                torch.mm(x, w.t(), out=out)
                if bias is not None:
                    self._call("nhv_add_bias_rows", _ptr(out), _ptr(bias), M, N, dtype_code(out), _stream())
                return None
            if out.dtype == torch.float32 and bias is None and not self.own_kernels_only and _MM_GIVES_FLOAT32:
                # the logits of many rows: the library's product with float sums and a float result (270 us for 64
                # rows of the 8B head against 400 us of the own kernel for 17 to 64 rows, which takes 64 rows a call)
                torch.mm(x, w.t(), out_dtype=torch.float32, out=out)
                return None
            if out.dtype == torch.float32:
                for m0 in range(0, M, 64):          # float32 output (logits), or more rows than a graph may hold in one call
                    m1 = min(M, m0 + 64)
                    self._call("nhv_gemm_skinny_bf16", _ptr(x[m0:m1]), _ptr(w), _ptr(bias), _ptr(out[m0:m1]),
                               m1 - m0, N, K, dtype_code(out), _stream())
                return None
        self._call("nhv_gemm_generic", _ptr(x), _ptr(w), _ptr(bias), _ptr(out), M, N, K, dtype_code(x),
                   dtype_code(out), _stream())

    norm_kernel_ms = 0.003        # what a norm's own kernel costs in a decoding step, about

    def _measured(self, x, w, gated: bool):
        """(the choice for this shape, (ms of the own kernel, ms of the library's best) or None); the shape is
        measured here if it is due, as ``linear`` would have it measured."""
        M, K = x.shape
        key = (M, w.shape[0], K, False, gated)
        how = self.chosen.get(key)
        if how is None and self.measure_linears and self.measuring_allowed and not torch.cuda.is_current_stream_capturing():
            scratch = torch.empty((M, w.shape[0] // 2 if gated else w.shape[0]), dtype=x.dtype, device=x.device)
            how = self._choose(x, w, scratch, gated=gated)
        return how, self.times.get(key)

    def fusion_pays(self, x, w, gated: bool = False) -> bool:
        """For a product whose rows come as a sum that still lacks its norm's scales: whether the own kernel, which
        scales its sums itself, beats what this shape is otherwise done by. Where a measurement chose a library
        algorithm for the shape, that algorithm and a kernel that scales the rows first have to be slower together
        than the own kernel alone."""
        if self.own_kernels_only:
            return True
        how, times = self._measured(x, w, gated)
        if how is None or how < 0:
            return True
        if times is None:
            return False                                     # (a choice from a table: followed as it stands)
        own, library = times
        return own <= library + self.norm_kernel_ms

    def addition_pays(self, x, w, reader_w=None, reader_gated: bool = False) -> bool:
        """For a product whose result is about to be added to the residual stream and normed: whether the own
        kernel, which makes the addition itself, is the one to take. That saves the norm's kernel only if the product
        that reads the norm (``reader_w``, of the same rows) scales its rows itself, so the two are priced together:
        own kernels for both, against each one's best way and the norm's kernel between them. Without times for both
        shapes the own kernel is taken where it is this shape's choice anyway."""
        if self.own_kernels_only:
            return True
        how, times = self._measured(x, w, False)
        if how is None or how < 0:
            return True
        if times is None or reader_w is None:
            return False
        reader_how = self.chosen.get((x.shape[0], reader_w.shape[0], reader_w.shape[1], False, reader_gated))
        reader_times = self.times.get((x.shape[0], reader_w.shape[0], reader_w.shape[1], False, reader_gated))
        if reader_how is None:
            return False                                     # (the reader's shape is not measured yet: next time)
        if reader_times is None:
            if reader_how >= 0:
                return False
            reader_times = (0.0, 0.0)                        # the own kernel is the reader's way whatever is fused
        own, library = times
        reader_own, reader_library = reader_times
        return own + reader_own <= min(own, library) + self.norm_kernel_ms + min(reader_own, reader_library)

    def fused_linear(self, x, w, bias, out, gated=False, row_scales=None, residual=None, sum_out=None, ss_out=None, next_w=None):
        """The own few-rows product with what it may take over. ``row_scales`` = (squares [M, tiles], eps): x is a
        sum whose rows still lack their norm's scales, which are applied to the finished sums. ``residual``: the
        result is added to it (in place); ``sum_out`` gets the sum times ``next_w`` (the next norm's weight), rounded,
        and ``ss_out`` the tiles' shares of the rows' sums of squares (``out`` is then not written)."""
        M, K = x.shape
        N = w.shape[0] // 2 if gated else w.shape[0]
        ss, eps = row_scales if row_scales is not None else (None, 0.0)
        self._call("nhv_gemm_fewrows_fused_bf16", _ptr(x), _ptr(ss), 0 if ss is None else ss.shape[1], ctypes.c_float(eps),
                   _ptr(w), _ptr(bias), _ptr(out), M, N, K, BF16 if out is None else dtype_code(out), int(gated),
                   _ptr(residual), F32 if residual is None else dtype_code(residual), _ptr(sum_out), _ptr(ss_out),
                   _ptr(next_w), F32 if next_w is None else dtype_code(next_w), _stream())

    def scale_rows(self, x, squares, eps, out):
        self._call("nhv_scale_rows", _ptr(x), _ptr(squares), squares.shape[1], ctypes.c_float(eps), _ptr(out), x.shape[0],
                   x.shape[1], _stream())

    def gated_linear(self, x, w, out, act: int = 0) -> bool:
        """act(x Wg^T) * (x Wu^T) in one kernel, if this batch is one for the few-rows kernel; else False.
        ``act``: 0 SiLU, 1 the tanh form of GELU (up to 16 rows)."""
        M, K = x.shape
        if act != 0:
            if x.dtype == torch.bfloat16 and K % 8 == 0 and x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0 and M <= self.few_rows:
                self._call("nhv_gemm_fewrows_glu_act_bf16", _ptr(x), _ptr(w), _ptr(out), M, out.shape[1], K, dtype_code(out),
                           act, _stream())
                return True
            return False
        if (x.dtype == torch.bfloat16 and K % 8 == 0 and x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0
                and (M <= self.few_rows or (M <= 64 and self.own_kernels_only))):
            if M <= self.few_rows and not self.own_kernels_only:
                how = self._choose(x, w, out, gated=True)
                if how is not None and how >= 0:
                    return False                             # the library's product, then silu_mul
            self._call("nhv_gemm_skinny_glu_bf16", _ptr(x), _ptr(w), _ptr(out), M, out.shape[1], K, dtype_code(out),
                       _stream())
            return True
        return False

    def activated_linear(self, x, w, out, act: int) -> bool:
        """act(x W^T) in one kernel, if this batch is one for the few-rows kernel and no library algorithm was found
        faster for the shape; else False. ``act``: a value of ``PLAIN_ACTIVATIONS``."""
        M, K = x.shape
        if not (x.dtype == torch.bfloat16 and K % 8 == 0 and x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0 and M <= self.few_rows):
            return False
        if not self.own_kernels_only:
            how = self._choose(x, w, out)
            if how is not None and how >= 0:
                return False                                 # the library's product, then the activation's kernel
        self._call("nhv_gemm_fewrows_act_bf16", _ptr(x), _ptr(w), _ptr(out), M, out.shape[1], K, dtype_code(out), act + 1,
                   _stream())
        return True

    def sample(self, logits, temperatures, keys, tokens):
        n, V = logits.shape
        pieces = self.lib.nhv_sample_pieces(V)
        piece_value = torch.empty((n, pieces), dtype=torch.float32, device=logits.device)
        piece_index = torch.empty((n, pieces), dtype=torch.int32, device=logits.device)
        self._call("nhv_sample", _ptr(logits), _ptr(temperatures), _ptr(keys), _ptr(tokens), n, V, _ptr(piece_value),
                   _ptr(piece_index), _stream())


def measured_peaks(device="cuda:0", read_bytes: int = 4 << 30, gemm_size: int = 8192) -> dict:
    """What this very GPU gives, for fractions beside those of the published peaks: the rate of a kernel that only
    reads ``read_bytes`` from memory (each byte once, far more than the caches hold), and the rate of a bfloat16
    matrix product of ``gemm_size``^3 by the vendor's library. The shortest of five runs each."""
    b = backend()
    data = torch.empty(read_bytes // 1024 * 1024, dtype=torch.uint8, device=device).zero_()
    sink = torch.zeros(1, dtype=torch.float32, device=device)

    def shortest(run, n=5):
        best = float("inf")
        for _ in range(n + 1):                      # (the first run is a warm-up)
            start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record()
            run()
            end.record()
            end.synchronize()
            best = min(best, start.elapsed_time(end) * 1e-3)
        return best

    read_s = shortest(lambda: b._call("nhv_measure_read", _ptr(data), _ptr(sink), ctypes.c_size_t(data.numel()), _stream()))
    del data
    a = torch.randn(gemm_size, gemm_size, dtype=torch.bfloat16, device=device)
    c = torch.empty_like(a)
    gemm_s = shortest(lambda: torch.mm(a, a.t(), out=c))
    return {"hbm_read_GBs": read_bytes // 1024 * 1024 / read_s / 1e9, "gemm_bf16_TFLOPs": 2.0 * gemm_size ** 3 / gemm_s / 1e12}


class KernelTimes:
    """Per-kernel device time of everything launched inside ``with kernel_times() as t`` (events around every
    call into the library; not for use while a graph is recorded). ``t.table()`` after the block."""

    def __init__(self):
        self.records: list[tuple[str, torch.cuda.Event, torch.cuda.Event]] = []

    def summary(self) -> dict[str, tuple[int, float]]:
        torch.cuda.synchronize()
        out: dict[str, tuple[int, float]] = {}
        for name, start, end in self.records:
            n, ms = out.get(name, (0, 0.0))
            out[name] = (n + 1, ms + start.elapsed_time(end))
        return out

    def table(self) -> str:
        rows = sorted(self.summary().items(), key=lambda kv: -kv[1][1])
        total = sum(ms for _, (_, ms) in rows) or 1.0
        lines = [f"{'kernel':40s} {'calls':>7s} {'total ms':>10s} {'mean us':>9s} {'share':>6s}"]
        for name, (n, ms) in rows:
            lines.append(f"{name:40s} {n:7d} {ms:10.3f} {ms / n * 1e3:9.1f} {100 * ms / total:5.1f}%")
        return "\n".join(lines)


class kernel_times:
    def __enter__(self) -> KernelTimes:
        self.times = KernelTimes()
        b = backend()
        self._old = b._call
        times = self.times

        def timed_call(fn_name, *args, lib=None):
            start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record()
            self._old(fn_name, *args, lib=lib)
            end.record()
            times.records.append((fn_name, start, end))

        b._call = timed_call
        return self.times

    def __exit__(self, *exc):
        backend()._call = self._old
        return False


_backend = None


def backend():
    global _backend
    if _backend is None:
        _backend = NativeBackend()
    return _backend


def set_backend(obj) -> None:
    """Replace the kernel library (tests of the engine's logic on a machine
    without a GPU put a stand-in here; the engine itself never does)."""
    global _backend
    _backend = obj


# ------------------------------------------------------------------ work that a product takes over from its neighbours
@dataclass
class AddTo:
    """What a part is handed in place of nothing when its result is about to be added to the residual stream and
    normed: the stream, the weight and eps of the norm that follows, and (if known) the first product of the part
    that reads that norm, as (weight, gated): whether making the addition in the product's kernel pays depends on
    whether that reader scales its rows itself."""

    residual: torch.Tensor
    norm_weight: torch.Tensor
    eps: float
    reader: tuple | None = None


@dataclass
class Summed:
    """What ``linear(..., add_to=AddTo(...))`` returns where the product's own kernel has made the addition: the
    residual stream holds the sum already. ``weighted`` is the sum times the weight of the norm that follows, in
    the rows' element type; ``squares`` [rows, tiles] holds every tile's share of each row's sum of squares. What the
    norm still has to do is scale the rows: a product that reads ``Normed(summed)`` does that itself."""

    weighted: torch.Tensor
    squares: torch.Tensor
    residual: torch.Tensor
    norm_weight: torch.Tensor
    eps: float

    @property
    def shape(self):
        return self.weighted.shape


@dataclass
class Normed:
    """The norm of a ``Summed`` with the scaling of its rows left to the product that reads it (``linear``,
    ``gated_linear``: a product is linear in its rows, so it scales its own sums). ``tensor()`` is the norm as a
    tensor, for any other reader (one small kernel)."""

    summed: Summed

    @property
    def shape(self):
        return self.summed.weighted.shape

    def tensor(self) -> torch.Tensor:
        s = self.summed
        out = torch.empty_like(s.weighted)
        backend().scale_rows(s.weighted, s.squares, float(s.eps), out)
        return out


def dense(x):
    """``x`` as a tensor, whatever work was left undone in it."""
    if isinstance(x, Normed):
        return x.tensor()
    if isinstance(x, Summed):
        raise KernelError("a sum that was made for a norm (ops.Summed) goes through that norm, not anywhere else")
    if isinstance(x, (NormedPairMean, ScaledPairSum)):
        return x.tensor()
    return x


def _may_fuse(x: torch.Tensor, w: torch.Tensor) -> bool:
    b = backend()
    return (getattr(b, "fuse_norms", False) and hasattr(b, "fused_linear") and x.dtype == torch.bfloat16
            and x.shape[0] <= getattr(b, "few_rows", 0) and x.shape[1] % 8 == 0 and x.data_ptr() % 16 == 0
            and w.data_ptr() % 16 == 0)


def _fusion_pays(x: torch.Tensor, w: torch.Tensor, gated: bool) -> bool:
    pays = getattr(backend(), "fusion_pays", None)
    return True if pays is None else pays(x, w, gated=gated)


def _addition_pays(x: torch.Tensor, w: torch.Tensor, add_to: AddTo) -> bool:
    pays = getattr(backend(), "addition_pays", None)
    if pays is None:
        return True
    reader_w, reader_gated = add_to.reader if add_to.reader is not None else (None, False)
    return pays(x, w, reader_w, reader_gated)


# ------------------------------------------------------------------ checked entry points
def embed(ids: torch.Tensor, table: torch.Tensor, scale: float | None = None) -> torch.Tensor:
    """Rows of ``table``; with ``scale`` each row times it (multiplied in float, rounded once)."""
    _need(table.dim() == 2, "embed: the table must be [vocab, width]")
    _dense(table, "embed: table")
    _dense(ids, "embed: ids", (ids.shape[0],), torch.int32)
    dtype_code(table)
    out = torch.empty((ids.shape[0], table.shape[1]), dtype=table.dtype, device=table.device)
    if scale is None:
        backend().embed(ids, table, out)
    else:
        backend().embed(ids, table, out, float(scale))
    return out


def soft_cap_(logits: torch.Tensor, cap: float) -> torch.Tensor:
    """logits <- cap * tanh(logits / cap), in place (float32)."""
    _dense(logits, "soft_cap: logits", dtype=torch.float32)
    _need(cap > 0, lambda: f"soft_cap: the cap must be positive, got {cap}")
    if logits.numel():
        backend().soft_cap(logits, float(cap))
    return logits


def rmsnorm(x: torch.Tensor, w: torch.Tensor, eps: float, residual: torch.Tensor | None = None,
            start_residual: bool = False, residual_float32: bool = True):
    """``rmsnorm(x, w, eps)``: the norm of x.
    ``residual=r``: r += x in place (the sum is taken in float and normed unrounded; r keeps it in its own element
    type) and the norm of the sum is returned.
    ``start_residual=True``: returns (norm of x, the residual that later norms add to): a new float32 tensor holding
    x, or, with ``residual_float32=False``, x itself (which later calls then add to in place)."""
    _need(x.dim() == 2, "rmsnorm: x must be [tokens, width]")
    _dense(x, "rmsnorm: x")
    _dense(w, "rmsnorm: weight", (x.shape[1],))
    _need(w.dtype == x.dtype or w.dtype == torch.float32,
          lambda: f"rmsnorm: weight of {w.dtype} with activations of {x.dtype}")
    dtype_code(x)
    y = torch.empty_like(x)
    if start_residual:
        _need(residual is None, "rmsnorm: a residual is either started or added to")
        if not residual_float32 and x.dtype != torch.float32:
            backend().rmsnorm(x, None, 0, w, y, float(eps))
            return y, x
        residual = torch.empty(x.shape, dtype=torch.float32, device=x.device)
        backend().rmsnorm(x, residual, 2, w, y, float(eps))
        return y, residual
    if residual is not None:
        _dense(residual, "rmsnorm: residual", tuple(x.shape))
        _need(residual.dtype == x.dtype or residual.dtype == torch.float32,
              lambda: f"rmsnorm: residual of {residual.dtype} with rows of {x.dtype}")
        backend().rmsnorm(x, residual, 1, w, y, float(eps))
        return y
    backend().rmsnorm(x, None, 0, w, y, float(eps))
    return y


def silu_mul(gate_up: torch.Tensor) -> torch.Tensor:
    _need(gate_up.dim() == 2 and gate_up.shape[1] % 2 == 0, "silu_mul: input must be [tokens, 2 * width]")
    _dense(gate_up, "silu_mul: input")
    dtype_code(gate_up)
    out = torch.empty((gate_up.shape[0], gate_up.shape[1] // 2), dtype=gate_up.dtype, device=gate_up.device)
    backend().silu_mul(gate_up, out)
    return out


def gather_rows(x: torch.Tensor, rows: torch.Tensor) -> torch.Tensor:
    _need(x.dim() == 2, "gather_rows: x must be [tokens, width]")
    _dense(x, "gather_rows: x")
    _dense(rows, "gather_rows: rows", (rows.shape[0],), torch.int32)
    dtype_code(x)
    out = torch.empty((rows.shape[0], x.shape[1]), dtype=x.dtype, device=x.device)
    backend().gather_rows(x, rows, out)
    return out


def qk_rope_write(qkv, bias, q_norm_w, k_norm_w, eps, cos_sin, positions, slot_mapping, k_cache, v_cache,
                  num_heads: int, num_kv_heads: int, head_dim: int, write_kv: bool = True,
                  pair_axes: torch.Tensor | None = None) -> torch.Tensor:
    """Splits the packed projection, norms and turns q and k, stores k and v in the
    paged cache and returns q as [tokens, heads, head_dim].
    ``positions``: [tokens], or [axes, tokens] with ``pair_axes`` [rotary size / 2] (int32): the axis whose
    coordinate turns each pair (without ``pair_axes`` every pair turns by the first axis)."""
    T = qkv.shape[0]
    width = (num_heads + 2 * num_kv_heads) * head_dim
    _dense(qkv, "qk_rope_write: qkv", (T, width))
    dtype_code(qkv)
    if bias is not None:
        _dense(bias, "qk_rope_write: bias", (width,), qkv.dtype)
    for name, w in (("q_norm", q_norm_w), ("k_norm", k_norm_w)):
        if w is not None:
            _dense(w, f"qk_rope_write: {name} weight", (head_dim,))
            _need(w.dtype == qkv.dtype or w.dtype == torch.float32, lambda: f"qk_rope_write: {name} weight of {w.dtype}")
    _need((q_norm_w is None) == (k_norm_w is None), "qk_rope_write: q and k norm weights come together")
    if q_norm_w is not None:
        _need(q_norm_w.dtype == k_norm_w.dtype, "qk_rope_write: q and k norm weights differ in element type")
    rot = 0
    if cos_sin is not None:
        _need(cos_sin.dim() == 2, "qk_rope_write: rotation table must be [positions, rotary size]")
        _dense(cos_sin, "qk_rope_write: rotation table", dtype=torch.float32)
        rot = cos_sin.shape[1]
        _need(rot % 2 == 0 and rot <= head_dim, lambda: f"qk_rope_write: rotary size {rot} with head size {head_dim}")
    if positions.dim() == 1:
        _dense(positions, "qk_rope_write: positions", (T,), torch.int32)
    else:
        _need(positions.dim() == 2 and positions.shape[1] == T and positions.shape[0] >= 1,
              lambda: f"qk_rope_write: positions {tuple(positions.shape)} for {T} tokens (want [axes, tokens])")
        _dense(positions, "qk_rope_write: positions", dtype=torch.int32)
    if pair_axes is not None:
        _need(cos_sin is not None, "qk_rope_write: axes of pairs without a rotation table")
        _dense(pair_axes, "qk_rope_write: pair_axes", (rot // 2,), torch.int32)
        _need(positions.dim() == 2, "qk_rope_write: pair_axes go with positions [axes, tokens]")
    if write_kv:
        _dense(slot_mapping, "qk_rope_write: slot_mapping", (T,), torch.int32)
        _need(k_cache.dim() == 4 and tuple(k_cache.shape[2:]) == (num_kv_heads, head_dim),
              lambda: f"qk_rope_write: cache shape {tuple(k_cache.shape)} does not fit {num_kv_heads} heads of {head_dim}")
        _dense(k_cache, "qk_rope_write: k_cache", dtype=qkv.dtype)
        _dense(v_cache, "qk_rope_write: v_cache", tuple(k_cache.shape), qkv.dtype)
    q_out = torch.empty((T, num_heads, head_dim), dtype=qkv.dtype, device=qkv.device)
    backend().qk_rope_write(qkv, bias, q_norm_w, k_norm_w, float(eps), cos_sin, rot, positions,
                            slot_mapping if write_kv else None, q_out, k_cache if write_kv else None,
                            v_cache if write_kv else None, num_heads, num_kv_heads, head_dim, write_kv,
                            **({} if pair_axes is None else {"pair_axes": pair_axes}))
    return q_out


def paged_attention(q, k_cache, v_cache, batch: AttentionBatch, block_tables, scale: float,
                    window: int | None = None, chunk: int | None = None, softcap: float | None = None,
                    sink: float | None = None, gate: tuple | None = None) -> torch.Tensor:
    """Every query reads its request's keys up to its own position: all of them, the last ``window``, or (``chunk``)
    those of its own block of ``chunk`` positions counted from the request's start. The value heads may have another
    size than the key heads: the result is [tokens, heads, value size].
    ``softcap``: a score s (after the scale) becomes softcap tanh(s / softcap). ``sink``: the softmax's denominator
    holds one more term exp(sink), a key of that score without a value. ``gate`` = (rows [tokens, columns] of q's
    element type, first column): head h's result at token t is multiplied by sigmoid(rows[t, first column + h])."""
    _need(q.dim() == 3, "attention: q must be [tokens, heads, head_dim]")
    T, Hq, D = q.shape
    _dense(q, "attention: q")
    dtype_code(q)
    _need(k_cache.dim() == 4 and k_cache.shape[3] == D, lambda: f"attention: cache shape {tuple(k_cache.shape)} with head size {D}")
    _dense(k_cache, "attention: k_cache", dtype=q.dtype)
    _need(v_cache.dim() == 4 and tuple(v_cache.shape[:3]) == tuple(k_cache.shape[:3]),
          lambda: f"attention: value cache {tuple(v_cache.shape)} beside key cache {tuple(k_cache.shape)}")
    _dense(v_cache, "attention: v_cache", dtype=q.dtype)
    _need(not (window and chunk), "attention: a window or a chunk, not both")
    _need(chunk is None or chunk > 0, lambda: f"attention: chunk {chunk}")
    Hkv = k_cache.shape[2]
    _need(Hq % Hkv == 0, lambda: f"attention: {Hq} query heads are not a multiple of {Hkv} key heads")
    _need(T == batch.num_tokens, lambda: f"attention: {T} tokens but the batch has {batch.num_tokens}")
    _dense(batch.token_req, "attention: token_req", (T,), torch.int32)
    _dense(batch.positions, "attention: positions", (T,), torch.int32)
    _need(block_tables.dim() == 2 and block_tables.shape[0] == batch.num_requests,
          lambda: f"attention: block tables {tuple(block_tables.shape)} for {batch.num_requests} requests")
    _dense(block_tables, "attention: block_tables", dtype=torch.int32)
    page_size = k_cache.shape[1]
    _need(block_tables.shape[1] * page_size >= batch.max_context_len,
          lambda: f"attention: block tables of {block_tables.shape[1]} pages of {page_size} are too short for "
          f"{batch.max_context_len} keys")
    out = torch.empty((T, Hq, v_cache.shape[3]), dtype=q.dtype, device=q.device)
    more = {}
    if softcap is not None:
        _need(softcap > 0, lambda: f"attention: the cap on scores must be positive, got {softcap}")
        more["cap"] = float(softcap)
    if sink is not None:
        more["sink"] = float(sink)
    if gate is not None:
        rows, col = gate
        _need(rows.dim() == 2 and rows.shape[0] == T and 0 <= col and col + Hq <= rows.shape[1],
              lambda: f"attention: gates {tuple(rows.shape)} for {Hq} heads from column {col}")
        _dense(rows, "attention: gates", dtype=q.dtype)
        more["gate"] = (rows, int(col))
    if chunk:
        backend().paged_attention(q, k_cache, v_cache, out, batch, block_tables, float(scale), 0, int(chunk), **more)
    else:
        backend().paged_attention(q, k_cache, v_cache, out, batch, block_tables, float(scale), int(window or 0), **more)
    return out


def linear(x, w: torch.Tensor, bias: torch.Tensor | None = None, out_dtype=None, add_to: AddTo | None = None):
    """x[M, K] . w[N, K]^T (+ bias), accumulated in float. ``out_dtype`` may be
    float32 for bfloat16 inputs (the logits).
    ``x`` may be a ``Normed``: where the product's kernel can, it scales the rows itself.
    ``add_to``: the residual stream [M, N] that the caller is about to add the result to, and the norm that follows.
    Where the product's kernel can, it makes the addition itself (in float; the stream is rewritten) and a ``Summed``
    is returned, which that norm takes; otherwise the plain result is returned and the stream is left alone."""
    normed = x if isinstance(x, Normed) else None
    if normed is not None:
        x = normed.summed.weighted
        _dense(w, "linear: w", dtype=x.dtype)
        if not (_may_fuse(x, w) and _fusion_pays(x, w, False)):
            x, normed = normed.tensor(), None
    _need(x.dim() == 2 and w.dim() == 2, "linear: x must be [rows, in] and w [out, in]")
    _need(x.shape[1] == w.shape[1], lambda: f"linear: x has {x.shape[1]} columns but w has {w.shape[1]}")
    _dense(x, "linear: x")
    _dense(w, "linear: w", dtype=x.dtype)
    dtype_code(x)
    if bias is not None:
        _dense(bias, "linear: bias", (w.shape[0],), x.dtype)
    out_dtype = out_dtype or x.dtype
    _need(out_dtype == x.dtype or out_dtype == torch.float32, lambda: f"linear: output of {out_dtype} from {x.dtype}")
    M, N = x.shape[0], w.shape[0]
    scales = None if normed is None else (normed.summed.squares, float(normed.summed.eps))
    if add_to is not None and out_dtype == x.dtype and _may_fuse(x, w) and (normed is not None or _addition_pays(x, w, add_to)):
        residual = add_to.residual
        _dense(residual, "linear: residual", (M, N))
        _need(residual.dtype == x.dtype or residual.dtype == torch.float32, lambda: f"linear: residual of {residual.dtype} with rows of {x.dtype}")
        _dense(add_to.norm_weight, "linear: the next norm's weight", (N,))
        dtype_code(add_to.norm_weight)
        weighted = torch.empty((M, N), dtype=x.dtype, device=x.device)
        squares = torch.empty((M, (N + 15) // 16), dtype=torch.float32, device=x.device)
        backend().fused_linear(x, w, bias, None, row_scales=scales, residual=residual, sum_out=weighted, ss_out=squares,
                               next_w=add_to.norm_weight)
        return Summed(weighted, squares, residual, add_to.norm_weight, add_to.eps)
    out = torch.empty((M, N), dtype=out_dtype, device=x.device)
    if normed is not None:
        backend().fused_linear(x, w, bias, out, row_scales=scales)
    else:
        backend().linear(x, w, bias, out)
    return out


def gated_linear(x, w: torch.Tensor, activation: str = "silu") -> torch.Tensor:
    """act(x . w[:I]^T) * (x . w[I:]^T) for a packed gate | up matrix w[2 I, K]: fused into one kernel for
    few rows, else the matrix product followed by ``act_mul``. ``x`` may be a ``Normed`` (see ``linear``; with SiLU)."""
    _need(activation in ACTIVATIONS, lambda: f"gated_linear: activation {activation!r} is not known ({sorted(ACTIVATIONS)} are)")
    if activation != "silu":
        x = dense(x)
        _need(x.dim() == 2 and w.dim() == 2 and w.shape[0] % 2 == 0, "gated_linear: x must be [rows, in] and w [2 * out, in]")
        _need(x.shape[1] == w.shape[1], lambda: f"gated_linear: x has {x.shape[1]} columns but w has {w.shape[1]}")
        _dense(x, "gated_linear: x")
        _dense(w, "gated_linear: w", dtype=x.dtype)
        dtype_code(x)
        fused = getattr(backend(), "gated_linear", None)
        if fused is not None:
            out = torch.empty((x.shape[0], w.shape[0] // 2), dtype=x.dtype, device=x.device)
            if fused(x, w, out, ACTIVATIONS[activation]):
                return out
        return act_mul(linear(x, w), activation)
    if isinstance(x, Normed):
        normed, x = x, x.summed.weighted
        _need(w.dim() == 2 and w.shape[0] % 2 == 0 and x.shape[1] == w.shape[1], "gated_linear: w must be [2 * out, in]")
        _dense(w, "gated_linear: w", dtype=x.dtype)
        if _may_fuse(x, w) and _fusion_pays(x, w, True):
            out = torch.empty((x.shape[0], w.shape[0] // 2), dtype=x.dtype, device=x.device)
            backend().fused_linear(x, w, None, out, gated=True, row_scales=(normed.summed.squares, float(normed.summed.eps)))
            return out
        x = normed.tensor()
    _need(x.dim() == 2 and w.dim() == 2 and w.shape[0] % 2 == 0, "gated_linear: x must be [rows, in] and w [2 * out, in]")
    _need(x.shape[1] == w.shape[1], lambda: f"gated_linear: x has {x.shape[1]} columns but w has {w.shape[1]}")
    _dense(x, "gated_linear: x")
    _dense(w, "gated_linear: w", dtype=x.dtype)
    dtype_code(x)
    fused = getattr(backend(), "gated_linear", None)
    if fused is not None:
        out = torch.empty((x.shape[0], w.shape[0] // 2), dtype=x.dtype, device=x.device)
        if fused(x, w, out):
            return out
    return silu_mul(linear(x, w))



# ------------------------------------------------------------------ two norms side by side, a hashed pair embedding
ACTIVATIONS = {"silu": 0, "gelu_tanh": 1}            # what a gate may pass (``gated_linear``, ``act_mul``)
PLAIN_ACTIVATIONS = {"silu": 0, "gelu_tanh": 1, "relu2": 2}    # what rows may pass on their own (``activation_``); relu2: max(z, 0)^2


def embed_pair_hash(ids: torch.Tensor, table: torch.Tensor, pair_table: torch.Tensor, batch: AttentionBatch,
                    state_slots: torch.Tensor, prev_state: torch.Tensor, buckets: int, mul_prev: int, mul_cur: int) -> torch.Tensor:
    """float32 [tokens, width]: table[id] + pair_table[(previous id * mul_prev + id * mul_cur) mod buckets], and for a
    token at position 0 the row ``buckets``. The id before a portion's first token is ``prev_state`` at the request's
    slot ([slots] int32), which then takes the portion's last id."""
    T = ids.shape[0]
    _need(table.dim() == 2 and pair_table.dim() == 2 and pair_table.shape[1] == table.shape[1],
          "embed_pair_hash: tables must be [rows, width] of one width")
    _dense(table, "embed_pair_hash: table")
    _dense(pair_table, "embed_pair_hash: pair table", dtype=table.dtype)
    _need(buckets > 0 and pair_table.shape[0] == buckets + 1,
          lambda: f"embed_pair_hash: a pair table of {pair_table.shape[0]} rows for {buckets} buckets and one row more")
    _dense(ids, "embed_pair_hash: ids", (T,), torch.int32)
    _need(T == batch.num_tokens, lambda: f"embed_pair_hash: {T} tokens but the batch has {batch.num_tokens}")
    _dense(batch.positions, "embed_pair_hash: positions", (T,), torch.int32)
    _dense(batch.token_req, "embed_pair_hash: token_req", (T,), torch.int32)
    _dense(batch.cu_seqlens_q, "embed_pair_hash: cu_seqlens_q", (batch.num_requests + 1,), torch.int32)
    _dense(state_slots, "embed_pair_hash: state_slots", (batch.num_requests,), torch.int32)
    _need(prev_state.dim() == 1, "embed_pair_hash: the kept tokens are one number a slot")
    _dense(prev_state, "embed_pair_hash: prev_state", dtype=torch.int32)
    dtype_code(table)
    out = torch.empty((T, table.shape[1]), dtype=torch.float32, device=table.device)
    backend().embed_pair_hash(ids, table, pair_table, out, batch, state_slots, prev_state, int(buckets), int(mul_prev), int(mul_cur))
    return out


def layernorm_pair(x: torch.Tensor, first, second, eps: float, out_dtype, add=()):
    """Layer norms (weight and bias, float32) of the float32 stream ``x``, one per (weight, bias) given: ``first`` and
    ``second`` (either may be None). ``add``: up to two tensors of rows that are added to ``x`` first, in float, in
    place. Mean and variance are taken once. Returns (y1 or None, y2 or None) in ``out_dtype``."""
    _need(x.dim() == 2, "layernorm_pair: x must be [tokens, width]")
    _dense(x, "layernorm_pair: x", dtype=torch.float32)
    W = x.shape[1]
    add = [t for t in add if t is not None]
    _need(len(add) <= 2, "layernorm_pair: at most two tensors are added")
    for t in add:
        _dense(t, "layernorm_pair: an added tensor", tuple(x.shape), out_dtype)
    _need(out_dtype in _DTYPE_CODE, lambda: f"layernorm_pair: rows of {out_dtype}")
    outs, args = [], []
    for wb in (first, second):
        if wb is None:
            outs.append(None)
            args += [None, None, None]
            continue
        w, b = wb
        _float32(w, "layernorm_pair: weight", (W,))
        _float32(b, "layernorm_pair: bias", (W,))
        y = torch.empty(x.shape, dtype=out_dtype, device=x.device)
        outs.append(y)
        args += [w, b, y]
    _need(outs[0] is not None or outs[1] is not None or add, "layernorm_pair: nothing to do")
    a = add[0] if add else None
    b = add[1] if len(add) > 1 else None
    backend().layernorm_pair(x, a, b, *args, float(eps), out_dtype)
    return outs[0], outs[1]


def add_streams_(x: torch.Tensor, a: torch.Tensor, b: torch.Tensor | None = None) -> torch.Tensor:
    """x += a (+ b) in float, in place; x is the float32 stream."""
    _dense(x, "add_streams: x", dtype=torch.float32)
    _dense(a, "add_streams: a", tuple(x.shape))
    dtype_code(a)
    if b is not None:
        _dense(b, "add_streams: b", tuple(x.shape), a.dtype)
    backend().add_streams(x, a, b)
    return x


def act_mul(gate_up: torch.Tensor, activation: str) -> torch.Tensor:
    """act(gate) * up for rows [gate | up]; ``activation``: "silu" or "gelu_tanh"."""
    _need(activation in ACTIVATIONS, lambda: f"act_mul: activation {activation!r} is not known ({sorted(ACTIVATIONS)} are)")
    if activation == "silu":
        return silu_mul(gate_up)
    _need(gate_up.dim() == 2 and gate_up.shape[1] % 2 == 0, "act_mul: input must be [tokens, 2 * width]")
    _dense(gate_up, "act_mul: input")
    dtype_code(gate_up)
    out = torch.empty((gate_up.shape[0], gate_up.shape[1] // 2), dtype=gate_up.dtype, device=gate_up.device)
    backend().act_mul(gate_up, out, ACTIVATIONS[activation])
    return out


# ------------------------------------------------------------------ attention over a cached latent
def latent_prepare(a: torch.Tensor, q_off: int, q_rank: int, c_off: int, kv_rank: int, rot: int, wq: torch.Tensor,
                   wc: torch.Tensor | None, eps: float, freqs: torch.Tensor | None, gain: float, positions: torch.Tensor,
                   slot_mapping: torch.Tensor | None, cache: torch.Tensor | None, out_dtype) -> torch.Tensor:
    """``a`` [tokens, columns] float32 holds the packed down projections of the step's rows. Returns the query latent
    (columns q_off ..., RMS-normed with ``wq``) as [tokens, q_rank] in ``out_dtype``; where ``kv_rank`` > 0 and a
    ``slot_mapping`` is given, stores [RMS-normed columns c_off ... | the ``rot`` columns after them, turned pairwise
    (2i, 2i + 1) by position * freqs[i], cosine and sine times ``gain``] at the tokens' slots of ``cache``."""
    T = a.shape[0]
    _need(a.dim() == 2, "latent_prepare: a must be [tokens, columns]")
    _dense(a, "latent_prepare: a", dtype=torch.float32)
    _float32(wq, "latent_prepare: query norm weight", (q_rank,))
    _dense(positions, "latent_prepare: positions", (T,), torch.int32)
    _need(out_dtype in _DTYPE_CODE, lambda: f"latent_prepare: rows of {out_dtype}")
    store = kv_rank > 0 and slot_mapping is not None
    if store:
        _float32(wc, "latent_prepare: latent norm weight", (kv_rank,))
        _dense(slot_mapping, "latent_prepare: slot_mapping", (T,), torch.int32)
        _need(cache is not None and cache.dim() == 4 and cache.shape[2] == 1 and cache.shape[3] >= kv_rank + rot,
              lambda: f"latent_prepare: cache of shape {None if cache is None else tuple(cache.shape)} for rows of {kv_rank} + {rot}")
        _dense(cache, "latent_prepare: cache", dtype=out_dtype)
        if rot:
            _dense(freqs, "latent_prepare: frequencies", (rot // 2,), torch.float64)
    cq = torch.empty((T, q_rank), dtype=out_dtype, device=a.device)
    backend().latent_prepare(a, q_off, q_rank, c_off, kv_rank if store else 0, rot if store else 0, wq, wc if store else None,
                             float(eps), freqs if store and rot else None, float(gain), positions,
                             slot_mapping if store else None, cache if store else None, cq)
    return cq


def head_gemm(x: torch.Tensor, w: torch.Tensor, transposed: bool, N: int, K: int, x_off: int = 0, out: torch.Tensor | None = None,
              out_off: int = 0, gate: torch.Tensor | None = None, gate_off: int = 0, turn: tuple | None = None) -> torch.Tensor:
    """One small matrix per head: out[t, h, out_off : out_off + N] = M_h x[t, h, x_off : x_off + K], sums in float.
    ``w`` is [heads * K, N] with M_h = w[h K : (h + 1) K]^T (``transposed``: x is multiplied from the left by the
    block's transpose) or [heads * N, K] with M_h = w[h N : (h + 1) N]. ``gate`` [tokens, columns] float32: the result
    of (t, h) is multiplied by sigmoid(gate[t, gate_off + h]). ``out``: [tokens, heads, row] to write into.
    ``turn`` = (rot, x_rot_off, out_rot_off, freqs, gain, positions): also out[t, h, out_rot_off + j] = x[t, h,
    x_rot_off + j] turned, j < rot, as ``rotate_interleaved`` does (for few rows in the same launch)."""
    _need(x.dim() == 3, "head_gemm: x must be [tokens, heads, row]")
    T, H, x_row = x.shape
    _dense(x, "head_gemm: x")
    dtype_code(x)
    _need(0 <= x_off and x_off + K <= x_row, lambda: f"head_gemm: columns {x_off}+{K} of {x_row}")
    _dense(w, "head_gemm: w", (H * K, N) if transposed else (H * N, K), x.dtype)
    if out is None:
        out = torch.empty((T, H, N), dtype=x.dtype, device=x.device)
    _need(out.dim() == 3 and tuple(out.shape[:2]) == (T, H) and 0 <= out_off and out_off + N <= out.shape[2],
          lambda: f"head_gemm: out {tuple(out.shape)} for {N} columns at {out_off}")
    _dense(out, "head_gemm: out", dtype=x.dtype)
    if gate is not None:
        _need(gate.dim() == 2 and gate.shape[0] == T and 0 <= gate_off and gate_off + H <= gate.shape[1],
              lambda: f"head_gemm: gate {tuple(gate.shape)} for {H} heads at {gate_off}")
        _dense(gate, "head_gemm: gate", dtype=torch.float32)
    if transposed:
        w_head, w_n, w_k = K * N, 1, N
    else:
        w_head, w_n, w_k = N * K, K, 1
    if turn is None:
        backend().head_gemm(x, x_off, x_row, w, w_head, w_n, w_k, out, out_off, out.shape[2], gate, gate_off, N, K)
        return out
    rot, x_rot, out_rot, freqs, gain, positions = turn
    _need(rot > 0 and rot % 2 == 0 and 0 <= x_rot and x_rot + rot <= x_row and 0 <= out_rot and out_rot + rot <= out.shape[2],
          lambda: f"head_gemm: {rot} turned entries at {x_rot} of {x_row} into {out_rot} of {out.shape[2]}")
    _dense(freqs, "head_gemm: frequencies", (rot // 2,), torch.float64)
    _dense(positions, "head_gemm: positions", (T,), torch.int32)
    done = backend().head_gemm(x, x_off, x_row, w, w_head, w_n, w_k, out, out_off, out.shape[2], gate, gate_off, N, K,
                               turn=(rot, x_rot, out_rot, freqs, float(gain), positions))
    if not done:
        backend().rotate_interleaved(x, x_rot, out, out_rot, rot, freqs, float(gain), positions)
    return out


def rotate_interleaved(src: torch.Tensor, s_off: int, dst: torch.Tensor, d_off: int, rot: int, freqs: torch.Tensor,
                       gain: float, positions: torch.Tensor) -> torch.Tensor:
    """dst[t, h, d_off + j] = src[t, h, s_off + j] turned, j < rot: pairs (2i, 2i + 1) by position * freqs[i]."""
    _need(src.dim() == 3 and dst.dim() == 3 and tuple(src.shape[:2]) == tuple(dst.shape[:2]),
          "rotate_interleaved: src and dst must be [tokens, heads, row]")
    _dense(src, "rotate_interleaved: src")
    _dense(dst, "rotate_interleaved: dst", dtype=src.dtype)
    dtype_code(src)
    _need(rot > 0 and rot % 2 == 0 and 0 <= s_off and s_off + rot <= src.shape[2] and 0 <= d_off and d_off + rot <= dst.shape[2],
          lambda: f"rotate_interleaved: {rot} entries at {s_off} of {src.shape[2]} into {d_off} of {dst.shape[2]}")
    _dense(freqs, "rotate_interleaved: frequencies", (rot // 2,), torch.float64)
    _dense(positions, "rotate_interleaved: positions", (src.shape[0],), torch.int32)
    backend().rotate_interleaved(src, s_off, dst, d_off, rot, freqs, float(gain), positions)
    return dst


# ------------------------------------------------------------------ a feed-forward of many small experts
ROUTER_SCORES = {"sigmoid": 0, "softmax_of_chosen": 1}


def route_topk(logits: torch.Tensor, top: int, bias: torch.Tensor | None = None, scoring: str = "sigmoid"):
    """(numbers [tokens, top] int32, scores [tokens, top] float32) of the ``top`` experts with the largest logits
    (``bias`` [experts] float32 is added to them first), the largest first, the lower number among equals. ``scoring``
    "sigmoid": a score is the sigmoid of its logit; "softmax_of_chosen": the scores are the softmax over the chosen
    logits alone."""
    _need(logits.dim() == 2, "route_topk: logits must be [tokens, experts]")
    _dense(logits, "route_topk: logits", dtype=torch.float32)
    _need(0 < top <= logits.shape[1], lambda: f"route_topk: {top} of {logits.shape[1]} experts")
    _need(scoring in ROUTER_SCORES, lambda: f"route_topk: scoring {scoring!r} is not known ({sorted(ROUTER_SCORES)} are)")
    ids = torch.empty((logits.shape[0], top), dtype=torch.int32, device=logits.device)
    scores = torch.empty((logits.shape[0], top), dtype=torch.float32, device=logits.device)
    more = {}
    if bias is not None:
        _float32(bias, "route_topk: bias", (logits.shape[1],))
        more["bias"] = bias
    if scoring != "sigmoid":
        more["mode"] = ROUTER_SCORES[scoring]
    if logits.shape[0]:
        backend().route_topk(logits, ids, scores, **more)
    return ids, scores


def routed_experts(h: torch.Tensor, ids: torch.Tensor, scores: torch.Tensor, gate_up: torch.Tensor, down: torch.Tensor,
                   activation: str = "silu", scores_on: str = "input", add: torch.Tensor | None = None) -> torch.Tensor:
    """sum over a token's experts e (``ids``) of D_e (act(G_e x) * (U_e x)), x = score * h: the score multiplies the
    expert's input (``scores_on`` "input"); or of score * D_e (act(G_e h) * (U_e h)): the score weighs the expert's
    output ("output"). ``add`` [tokens, width]: one more row added to every token's sum before it is rounded (an expert
    that all tokens use). ``gate_up`` [experts, 2 ff, width] (gate rows, then up rows), ``down`` [experts, width, ff]."""
    _need(scores_on in ("input", "output"), lambda: f"routed_experts: scores on {scores_on!r}")
    _need(h.dim() == 2, "routed_experts: h must be [tokens, width]")
    T, W = h.shape
    _dense(h, "routed_experts: h")
    dtype_code(h)
    _need(activation in ACTIVATIONS, lambda: f"routed_experts: activation {activation!r}")
    _need(gate_up.dim() == 3 and gate_up.shape[2] == W and gate_up.shape[1] % 2 == 0, "routed_experts: gate_up must be [experts, 2 ff, width]")
    E, F = gate_up.shape[0], gate_up.shape[1] // 2
    _dense(gate_up, "routed_experts: gate_up", dtype=h.dtype)
    _dense(down, "routed_experts: down", (E, W, F), h.dtype)
    _need(ids.dim() == 2 and ids.shape[0] == T, "routed_experts: ids must be [tokens, top]")
    _dense(ids, "routed_experts: ids", dtype=torch.int32)
    _dense(scores, "routed_experts: scores", tuple(ids.shape), torch.float32)
    out = torch.empty((T, W), dtype=h.dtype, device=h.device)
    b = backend()
    first, more = scores, {}
    if scores_on == "output":
        first, more = None, {"weights": scores}
    if add is not None:
        _dense(add, "routed_experts: add", (T, W), h.dtype)
        more["add"] = add
    if not T:
        return out
    if (h.dtype == torch.bfloat16 and T > getattr(b, "few_rows", 0) and W % 8 == 0 and F % 8 == 0 and E <= 4096
            and hasattr(b, "experts_grouped")):
        b.experts_grouped(h, ids, first, gate_up, down, out, ACTIVATIONS[activation], **more)
        return out
    u = torch.empty((T * ids.shape[1], F), dtype=h.dtype, device=h.device)
    b.experts_gate_up(h, ids, first, gate_up, u, ACTIVATIONS[activation])
    b.experts_down(u, ids, down, out, **more)
    return out

# ------------------------------------------------------------------ layers that are not the pre-norm kind
def _float32(t: torch.Tensor, name: str, shape: tuple) -> None:
    """A dense float32 tensor of this shape (weights and statistics that stay in 32-bit whatever the rows are)."""
    _dense(t, name, shape, torch.float32)


def scalar_rmsnorm(x: torch.Tensor, gain: torch.Tensor, eps: float, out_dtype=None) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) * gain, ``gain`` one float32 number on the device. ``x`` and the result may differ
    in element type (a float32 stream normed into bfloat16 rows, bfloat16 rows normed into a float32 stream)."""
    _need(x.dim() == 2, "scalar_rmsnorm: x must be [tokens, width]")
    _dense(x, "scalar_rmsnorm: x")
    _need(gain.numel() == 1, lambda: f"scalar_rmsnorm: the weight is one number, got {tuple(gain.shape)}")
    _dense(gain, "scalar_rmsnorm: weight", dtype=torch.float32)
    dtype_code(x)
    y = torch.empty(x.shape, dtype=out_dtype or x.dtype, device=x.device)
    dtype_code(y)
    if x.shape[0]:
        backend().scalar_rmsnorm(x, gain, y, float(eps))
    return y


def pair_norm_mean(a: torch.Tensor, wa: torch.Tensor, b: torch.Tensor, wb: torch.Tensor, eps: float) -> torch.Tensor:
    """(norm(a) * wa + norm(b) * wb) / 2 row by row, norm = x / sqrt(mean(x^2) + eps); float32 weights."""
    _need(a.dim() == 2, "pair_norm_mean: rows must be [tokens, width]")
    _dense(a, "pair_norm_mean: a")
    _dense(b, "pair_norm_mean: b", tuple(a.shape), a.dtype)
    _float32(wa, "pair_norm_mean: first weight", (a.shape[1],))
    _float32(wb, "pair_norm_mean: second weight", (a.shape[1],))
    dtype_code(a)
    y = torch.empty_like(a)
    backend().pair_norm_mean(a, wa, b, wb, y, float(eps))
    return y


@dataclass
class NormedPairMean:
    """Half the sum of two rows' norms (each over its root mean square, times a weight vector of its own) that is
    still to be taken: ``depth_mix`` takes it as its first addend and does the work in its own kernel; ``tensor()``
    is the same as a tensor (``pair_norm_mean``), for any other reader."""

    a: torch.Tensor
    wa: torch.Tensor
    b: torch.Tensor
    wb: torch.Tensor
    eps: float

    def tensor(self) -> torch.Tensor:
        return pair_norm_mean(self.a, self.wa, self.b, self.wb, self.eps)


def depth_mix(x: torch.Tensor, a, b: torch.Tensor | None, results: torch.Tensor, index: int,
              weights: torch.Tensor, gain: torch.Tensor | None = None, eps: float = 0.0):
    """results[index + 1] = x + (a + b) (and results[0] = x when ``index`` is 0); returns the float32 stream
    sum over j <= index + 1 of weights[j] * results[j], and with ``gain`` also its RMS norm (one number as weight)
    in the element type of ``a``. ``x``: [tokens, width] float32; ``results``: [depth, tokens, width] float32.
    ``a`` may be a ``NormedPairMean``."""
    _need(x.dim() == 2, "depth_mix: x must be [tokens, width]")
    T, W = x.shape
    _dense(x, "depth_mix: x", dtype=torch.float32)
    pair = None
    if isinstance(a, NormedPairMean):
        _dense(a.b, "depth_mix: the pair's second rows", (T, W), a.a.dtype)
        _float32(a.wa, "depth_mix: the pair's first weight", (W,))
        _float32(a.wb, "depth_mix: the pair's second weight", (W,))
        pair, a = (a.b, a.wa, a.wb, float(a.eps)), a.a
    _dense(a, "depth_mix: a", (T, W))
    dtype_code(a)
    if b is not None:
        _dense(b, "depth_mix: b", (T, W), a.dtype)
    _need(results.dim() == 3 and tuple(results.shape[1:]) == (T, W) and 0 <= index and index + 2 <= results.shape[0],
          lambda: f"depth_mix: results {tuple(results.shape)} for index {index} and rows {(T, W)}")
    _dense(results, "depth_mix: results", dtype=torch.float32)
    _float32(weights, "depth_mix: weights", (index + 2,))
    out = torch.empty_like(x)
    normed = None
    if gain is not None:
        _need(gain.numel() == 1, "depth_mix: the norm's weight is one number")
        _dense(gain, "depth_mix: norm weight", dtype=torch.float32)
        normed = torch.empty((T, W), dtype=a.dtype, device=a.device)
    backend().depth_mix(x, a, b, results, int(index), weights, out, gain, normed, float(eps), **({"pair": pair} if pair else {}))
    return (out, normed) if gain is not None else out


def rotary_split_write(qkv: torch.Tensor, bias: torch.Tensor | None, qk_freqs: torch.Tensor | None,
                       v_freqs: torch.Tensor | None, positions: torch.Tensor, slot_mapping, k_cache, v_cache,
                       num_heads: int, num_kv_heads: int, head_dim: int, value_dim: int, with_kv: bool = True,
                       more_columns: int = 0, interleaved: bool = False, unit_eps: float | None = None,
                       values_from_keys: bool = False, maps: int = 1) -> torch.Tensor:
    """Splits the packed projection q | k | v (``with_kv``) or q alone (followed by ``more_columns`` columns that
    another reader takes), adds the bias, turns pair (i, i + r) of every
    query and key head by position * qk_freqs[i] (r = len(qk_freqs); the coordinates from 2 r on pass), turns the
    value heads the same way over all their coordinates if ``v_freqs`` is given, stores keys and values at the
    step's slots and returns q as [tokens, heads, head_dim]. Angles are taken in float from the position: no table.
    ``interleaved``: the pairs are (2i, 2i + 1). ``unit_eps``: after the rotation every query and key head is divided
    by its root mean square (this eps under the root), in float. ``values_from_keys``: the projection holds no value
    columns; value head g is key head g as projected (not turned, not normed). ``maps`` n > 1: every query and key head
    holds n maps of ``head_dim`` entries, each turned (and normed) on its own; ``num_heads`` and ``num_kv_heads`` count
    maps. A key head's n maps are stored side by side as one key of n ``head_dim`` entries (the caches have
    num_kv_heads / n heads, and the projection as many value heads); every query map is returned as a head of its own,
    [tokens, num_heads, n head_dim], with zeros in the other maps' places, so that its product with a stored key is the
    product with its own map."""
    T = qkv.shape[0]
    _need(maps >= 1 and num_heads % maps == 0 and num_kv_heads % maps == 0,
          lambda: f"rotary_split_write: {maps} maps with {num_heads} and {num_kv_heads} heads")
    _need(not values_from_keys or (value_dim == head_dim and maps == 1),
          "rotary_split_write: values that are the keys as projected have the keys' size (and one map)")
    value_columns = 0 if values_from_keys else (num_kv_heads // maps) * value_dim
    width = num_heads * head_dim + (num_kv_heads * head_dim + value_columns if with_kv else 0)
    more = {}
    if interleaved:
        more["interleaved"] = True
    if unit_eps is not None:
        more["unit_eps"] = float(unit_eps)
    if values_from_keys:
        more["values_from_keys"] = True
    if maps != 1:
        more["maps"] = int(maps)
    _need(more_columns >= 0, "rotary_split_write: a negative number of further columns")
    _dense(qkv, "rotary_split_write: qkv", (T, width + more_columns))
    dtype_code(qkv)
    if bias is not None:
        _dense(bias, "rotary_split_write: bias", (width,), qkv.dtype)
    rot = 0
    if qk_freqs is not None:
        rot = 2 * qk_freqs.shape[0]
        _need(rot <= head_dim, lambda: f"rotary_split_write: rotary size {rot} with head size {head_dim}")
        _float32(qk_freqs, "rotary_split_write: frequencies", (rot // 2,))
    _dense(positions, "rotary_split_write: positions", (T,), torch.int32)
    if with_kv:
        _dense(slot_mapping, "rotary_split_write: slot_mapping", (T,), torch.int32)
        _need(k_cache.dim() == 4 and tuple(k_cache.shape[2:]) == (num_kv_heads // maps, maps * head_dim),
              lambda: f"rotary_split_write: key cache {tuple(k_cache.shape)} does not fit {num_kv_heads // maps} heads of {maps * head_dim}")
        _need(v_cache.dim() == 4 and tuple(v_cache.shape[2:]) == (num_kv_heads // maps, value_dim),
              lambda: f"rotary_split_write: value cache {tuple(v_cache.shape)} does not fit {num_kv_heads // maps} heads of {value_dim}")
        _dense(k_cache, "rotary_split_write: k_cache", dtype=qkv.dtype)
        _dense(v_cache, "rotary_split_write: v_cache", dtype=qkv.dtype)
        if v_freqs is not None:
            _need(value_dim % 2 == 0, "rotary_split_write: value heads of odd size cannot be turned")
            _float32(v_freqs, "rotary_split_write: value frequencies", (value_dim // 2,))
    q_out = torch.empty((T, num_heads, maps * head_dim), dtype=qkv.dtype, device=qkv.device)
    if T:
        backend().rotary_split_write(qkv, bias, qk_freqs, rot, v_freqs if with_kv else None, positions,
                                     slot_mapping if with_kv else None, q_out, k_cache if with_kv else None,
                                     v_cache if with_kv else None, num_heads, num_kv_heads, head_dim, value_dim, with_kv,
                                     **({"more_columns": int(more_columns)} if more_columns else {}), **more)
    return q_out


def differential_combine(a: torch.Tensor, lam: torch.Tensor, eps: float, post: float, gate: tuple | None = None) -> torch.Tensor:
    """a [tokens, 2 heads, size] holds two softmax maps per head over the same values, per head its map 1, then its map
    2. Returns
    [tokens, heads, size]: o = a1 - lam a2, divided by sqrt(mean(o^2) + eps) over the head's entries, times ``post``
    and, with ``gate`` = (rows [tokens, columns] of a's element type, first column), times sigmoid(rows[t, column + h]).
    ``lam``: one float32 number on the device."""
    _need(a.dim() == 3 and a.shape[1] % 2 == 0, "differential_combine: a must be [tokens, 2 heads, size]")
    _dense(a, "differential_combine: a")
    dtype_code(a)
    _float32(lam, "differential_combine: lambda", (1,))
    T, H, E = a.shape[0], a.shape[1] // 2, a.shape[2]
    out = torch.empty((T, H, E), dtype=a.dtype, device=a.device)
    more = {}
    if gate is not None:
        rows, col = gate
        _need(rows.dim() == 2 and rows.shape[0] == T and 0 <= col and col + H <= rows.shape[1],
              lambda: f"differential_combine: gates {tuple(rows.shape)} for {H} heads from column {col}")
        _dense(rows, "differential_combine: gates", dtype=a.dtype)
        more["gate"] = (rows, int(col))
    if T:
        backend().differential_combine(a, lam, out, float(eps), float(post), **more)
    return out


def gate_rows_(x: torch.Tensor, gate: tuple) -> torch.Tensor:
    """x [tokens, n] in place: x[t, i] *= sigmoid(rows[t, first column + i]) with ``gate`` = (rows [tokens, columns] of
    x's element type, first column)."""
    _need(x.dim() == 2, "gate_rows: x must be [tokens, n]")
    _dense(x, "gate_rows: x")
    dtype_code(x)
    rows, col = gate
    _need(rows.dim() == 2 and rows.shape[0] == x.shape[0] and 0 <= col and col + x.shape[1] <= rows.shape[1],
          lambda: f"gate_rows: gates {tuple(rows.shape)} for rows {tuple(x.shape)} from column {col}")
    _dense(rows, "gate_rows: gates", dtype=x.dtype)
    if x.shape[0]:
        backend().gate_rows(x, (rows, int(col)))
    return x


def sandwich_step(x: torch.Tensor, add: tuple | None = None, read: tuple | None = None, rows_dtype=None):
    """One launch between two sublayers of a layer that norms on both sides. x [tokens, width] float32, the stream.
    ``add`` = (y [tokens, width], weight [width] float32, eps): x += y / sqrt(mean(y^2) + eps) * weight, in place.
    ``read`` = (weight [width] float32, eps): returns x / sqrt(mean(x^2) + eps) * weight (of the new x) as rows of
    ``rows_dtype``; without it None is returned."""
    _need(x.dim() == 2, "sandwich_step: x must be [tokens, width]")
    T, W = x.shape
    _float32(x, "sandwich_step: x", (T, W))
    _need(add is not None or read is not None, "sandwich_step: nothing to add and nothing to read")
    y = wb = wa = h = None
    eps_a = eps_b = 0.0
    if add is not None:
        y, wb, eps_b = add
        _dense(y, "sandwich_step: y", (T, W))
        dtype_code(y)
        _float32(wb, "sandwich_step: the weight of the result's norm", (W,))
    if read is not None:
        wa, eps_a = read
        _float32(wa, "sandwich_step: the weight of the norm that is read through", (W,))
        h = torch.empty((T, W), dtype=rows_dtype or torch.float32, device=x.device)
        dtype_code(h)
    if T:
        backend().sandwich_step(x, y, wb, float(eps_b), wa, float(eps_a), h)
    return h


def turn_back_(x: torch.Tensor, freqs: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
    """x[tokens, heads, size] in place: pair (m, m + size / 2) of every head turns by -position * freqs[m]."""
    _need(x.dim() == 3 and x.shape[2] % 2 == 0, "turn_back: x must be [tokens, heads, even size]")
    _dense(x, "turn_back: x")
    dtype_code(x)
    _float32(freqs, "turn_back: frequencies", (x.shape[2] // 2,))
    _dense(positions, "turn_back: positions", (x.shape[0],), torch.int32)
    if x.shape[0]:
        backend().turn_back(x, freqs, positions)
    return x


def gated_delta_rule(proj: torch.Tensor, a_lin: torch.Tensor | None, gate_lin: torch.Tensor | None, taps: torch.Tensor,
                     dt_bias: torch.Tensor, a_log: torch.Tensor, norm_weight: torch.Tensor, eps: float,
                     kept: torch.Tensor, state: torch.Tensor, batch: AttentionBatch, state_slots: torch.Tensor,
                     num_heads: int, num_kv_heads: int, head_dim: int, value_dim: int, out_dtype,
                     decay_per_head: bool = False, gate_activation: str = "sigmoid") -> torch.Tensor:
    """The recurrent mixer between its projections: short causal convolutions and SiLU on q, k, v (``proj``:
    [tokens, q | k | v | beta ...] as projected; ``taps`` [channels, n]; ``kept`` [slots, channels, n - 1], a request's
    last inputs, updated here), unit length for q and k per head, beta = sigmoid, the decays
    exp(-exp(a_log) softplus(a_lin + dt_bias)) per head and key channel (``decay_per_head``: one per head, and then
    ``a_lin`` has a column and ``dt_bias`` an entry per head), the recurrence over every request's tokens in
    order from and into ``state`` [slots, heads, value_dim, head_dim] (a request whose first token is at position 0
    starts from zero), then per head the read-out over its root mean square times ``norm_weight`` times
    f(gate_lin), f = ``gate_activation`` ("sigmoid", or "silu": z sigmoid(z)). Returns [tokens, heads * value_dim]
    in ``out_dtype``. ``a_lin`` is overwritten with the decays. ``a_lin`` and ``gate_lin`` None: ``proj`` is float32
    and holds them as further columns, q | k | v | beta | a | gate (one product made them all)."""
    T = proj.shape[0]
    H, G, D, E = num_heads, num_kv_heads, head_dim, value_dim
    C = 2 * G * D + H * E
    Dd = 1 if decay_per_head else D
    _need(H % G == 0, lambda: f"gated_delta_rule: {H} heads are not a multiple of {G} key heads")
    _need(gate_activation in ("sigmoid", "silu"), lambda: f"gated_delta_rule: gate activation {gate_activation!r}")
    _need((a_lin is None) == (gate_lin is None), "gated_delta_rule: decays and gates come both packed or both apart")
    packed = a_lin is None
    if packed:
        _dense(proj, "gated_delta_rule: proj", (T, C + H + H * Dd + H * E), torch.float32)
    else:
        _dense(proj, "gated_delta_rule: proj", (T, C + H))
        dtype_code(proj)
        _float32(a_lin, "gated_delta_rule: decays' linear part", (T, H * Dd))
        _float32(gate_lin, "gated_delta_rule: gates' linear part", (T, H * E))
    _need(taps.dim() == 2 and taps.shape[0] == C and 1 <= taps.shape[1] <= 16,
          lambda: f"gated_delta_rule: taps {tuple(taps.shape)} for {C} channels (1 to 16 taps)")
    _dense(taps, "gated_delta_rule: taps", dtype=torch.float32)
    n = taps.shape[1]
    _float32(dt_bias, "gated_delta_rule: dt_bias", (H * Dd,))
    _float32(a_log, "gated_delta_rule: a_log", (H,))
    _float32(norm_weight, "gated_delta_rule: norm weight", (E,))
    _need(kept.dim() == 3 and tuple(kept.shape[1:]) == (C, n - 1), lambda: f"gated_delta_rule: kept inputs {tuple(kept.shape)}")
    _dense(kept, "gated_delta_rule: kept inputs", dtype=torch.float32)
    _need(state.dim() == 4 and tuple(state.shape[1:]) == (H, E, D) and state.shape[0] == kept.shape[0],
          lambda: f"gated_delta_rule: state {tuple(state.shape)}")
    _dense(state, "gated_delta_rule: state", dtype=torch.float32)
    B = batch.num_requests
    _need(T == batch.num_tokens, lambda: f"gated_delta_rule: {T} tokens but the batch has {batch.num_tokens}")
    _dense(batch.token_req, "gated_delta_rule: token_req", (T,), torch.int32)
    _dense(batch.positions, "gated_delta_rule: positions", (T,), torch.int32)
    _dense(batch.cu_seqlens_q, "gated_delta_rule: cu_seqlens_q", (B + 1,), torch.int32)
    _dense(state_slots, "gated_delta_rule: state_slots", (B,), torch.int32)
    dev = proj.device
    q = torch.empty((T, G, D), dtype=torch.float32, device=dev)
    k = torch.empty((T, G, D), dtype=torch.float32, device=dev)
    v = torch.empty((T, H, E), dtype=torch.float32, device=dev)
    beta = torch.empty((T, H), dtype=torch.float32, device=dev)
    o = torch.empty((T, H, E), dtype=torch.float32, device=dev)
    y = torch.empty((T, H * E), dtype=out_dtype, device=dev)
    dtype_code(y)
    if T == 0:
        return y
    b = backend()
    act = {"gate_act": 1} if gate_activation == "silu" else {}
    if packed:
        decay = torch.empty((T, H, Dd), dtype=torch.float32, device=dev)
        b.delta_prepare(proj, taps, kept, proj, dt_bias, a_log, batch, state_slots, q, k, v, beta, H, G, D, E, decay=decay,
                        a_col=C + H)
    elif decay_per_head:
        decay = a_lin.view(T, H, 1)
        b.delta_prepare(proj, taps, kept, a_lin, dt_bias, a_log, batch, state_slots, q, k, v, beta, H, G, D, E, decay=decay)
    else:
        decay = a_lin.view(T, H, D)
        b.delta_prepare(proj, taps, kept, a_lin, dt_bias, a_log, batch, state_slots, q, k, v, beta, H, G, D, E)
    b.conv_state_update(proj, kept, n, batch, state_slots, C)
    b.delta_rule(q, k, v, decay, beta, state, o, batch, state_slots)
    if packed:
        b.gated_head_norm(o, proj, norm_weight, y.view(T, H, E), float(eps), gate_col=C + H + H * Dd, **act)
    else:
        b.gated_head_norm(o, gate_lin, norm_weight, y.view(T, H, E), float(eps), **act)
    return y


# ------------------------------------------------------------------ several residual streams side by side
@dataclass
class ScaledPairSum:
    """sa a + sb b of two mixers' results that is still to be taken: ``streams_step`` takes it as the sublayer's
    result and does the sum in its own kernel; ``tensor()`` is the same as a tensor, for any other reader."""

    a: torch.Tensor
    sa: float
    b: torch.Tensor
    sb: float

    def tensor(self) -> torch.Tensor:
        _dense(self.a, "scaled sum: a")
        _dense(self.b, "scaled sum: b", tuple(self.a.shape), self.a.dtype)
        dtype_code(self.a)
        y = torch.empty_like(self.a)
        if y.numel():
            backend().scaled_sum(self.a, self.b, y, float(self.sa), float(self.sb))
        return y


def streams_step(streams: torch.Tensor | None, rows: int, width: int, n: int, rows_dtype, start: torch.Tensor | None = None,
                 update: tuple | None = None, read: tuple | None = None, collapse: bool = False):
    """One step of ``n`` residual streams [n, rows, width] (float32) between two sublayers.
    ``start`` [rows, width] float32: all streams equal it (``streams`` is then only written, or None with ``collapse``).
    ``update`` = (mix [n, n] (from, to), out [n], y): X_t <- sum_s mix[s, t] X_s + out[t] y, all at once from the old
    values; y: rows of ``rows_dtype`` or a ``ScaledPairSum`` of two such. (mix and out None: ones, for n = 1.)
    ``read`` = (in [n] or None for ones, norm weight [width], eps): returns the RMS norm of sum_s in[s] X_s (new values)
    times the weight, in ``rows_dtype``.
    ``collapse``: the sum of the (new) streams is returned as [rows, width] float32 and ``streams`` is not written.
    Returns (normed rows or None, sum or None)."""
    _need(1 <= n <= 16, lambda: f"streams_step: {n} streams (1 to 16 are taken)")
    _need(rows_dtype in _DTYPE_CODE, lambda: f"streams_step: rows of {rows_dtype}")
    if streams is not None:
        _dense(streams, "streams_step: streams", (n, rows, width), torch.float32)
    else:
        _need(start is not None and collapse, "streams_step: without streams there is a start and only a sum is wanted")
    if start is not None:
        _dense(start, "streams_step: start", (rows, width), torch.float32)
    dev = start.device if start is not None else streams.device
    mix = out_w = a = b = None
    sa = sb = 1.0
    if update is not None:
        mix, out_w, y = update
        if mix is None:
            _need(n == 1, "streams_step: several streams need their coefficients")
            mix, out_w = _ones(dev, 1).view(1, 1), _ones(dev, 1)
        _float32(mix, "streams_step: mix", (n, n))
        _float32(out_w, "streams_step: out", (n,))
        if isinstance(y, ScaledPairSum):
            a, sa, b, sb = y.a, float(y.sa), y.b, float(y.sb)
            _dense(b, "streams_step: the second result", (rows, width), rows_dtype)
        else:
            a = y
        _dense(a, "streams_step: the sublayer's result", (rows, width), rows_dtype)
    in_w = norm_w = h = None
    eps = 0.0
    if read is not None:
        in_w, norm_w, eps = read
        if in_w is not None:
            _float32(in_w, "streams_step: in", (n,))
        _float32(norm_w, "streams_step: norm weight", (width,))
        h = torch.empty((rows, width), dtype=rows_dtype, device=dev)
    total = torch.empty((rows, width), dtype=torch.float32, device=dev) if collapse else None
    _need(update is not None or read is not None or collapse or start is not None, "streams_step: nothing to do")
    if rows:
        backend().streams_step(streams, start, mix, out_w, a, b, sa, sb, in_w, norm_w, float(eps), h, total, n, rows, width,
                               rows_dtype)
    return h, total


_ONES: dict = {}


def _ones(device, n: int) -> torch.Tensor:
    key = (str(device), n)
    if key not in _ONES:
        _ONES[key] = torch.ones(n, dtype=torch.float32, device=device)
    return _ONES[key]


def embed_float(ids: torch.Tensor, table: torch.Tensor, scale: float | None = None) -> torch.Tensor:
    """Rows of ``table`` times ``scale`` as float32 [tokens, width] (the start of a float32 stream: nothing is rounded)."""
    _need(table.dim() == 2, "embed_float: the table must be [vocab, width]")
    _dense(table, "embed_float: table")
    _dense(ids, "embed_float: ids", (ids.shape[0],), torch.int32)
    dtype_code(table)
    out = torch.empty((ids.shape[0], table.shape[1]), dtype=torch.float32, device=table.device)
    if ids.shape[0]:
        backend().embed_float(ids, table, out, 1.0 if scale is None else float(scale))
    return out


def activation_(x: torch.Tensor, activation: str) -> torch.Tensor:
    """x <- act(x) in place, taken in float and rounded once; ``activation``: one of ``PLAIN_ACTIVATIONS``."""
    _need(activation in PLAIN_ACTIVATIONS, lambda: f"activation: {activation!r} is not known ({sorted(PLAIN_ACTIVATIONS)} are)")
    _dense(x, "activation: x")
    dtype_code(x)
    if x.numel():
        backend().activation(x, PLAIN_ACTIVATIONS[activation])
    return x


def activated_linear(x: torch.Tensor, w: torch.Tensor, activation: str) -> torch.Tensor:
    """act(x . w^T) without a gate and without bias: one kernel for few rows in bfloat16, else the matrix product
    followed by ``activation_``. Either way the activation is taken in float and the result rounded once more than the
    product alone (the fused kernel rounds once in all)."""
    _need(activation in PLAIN_ACTIVATIONS, lambda: f"activated_linear: {activation!r} is not known ({sorted(PLAIN_ACTIVATIONS)} are)")
    _need(x.dim() == 2 and w.dim() == 2 and x.shape[1] == w.shape[1],
          lambda: f"activated_linear: x {tuple(x.shape)} and w {tuple(w.shape)} do not fit")
    _dense(x, "activated_linear: x")
    _dense(w, "activated_linear: w", dtype=x.dtype)
    dtype_code(x)
    fused = getattr(backend(), "activated_linear", None)
    if fused is not None and x.shape[0]:
        out = torch.empty((x.shape[0], w.shape[0]), dtype=x.dtype, device=x.device)
        if fused(x, w, out, PLAIN_ACTIVATIONS[activation]):
            return out
    return activation_(linear(x, w), activation)


def scale_(x: torch.Tensor, factor: float) -> torch.Tensor:
    """x <- x * factor in place (float32)."""
    _dense(x, "scale: x", dtype=torch.float32)
    if x.numel():
        backend().scale(x, float(factor))
    return x


def sample(logits: torch.Tensor, temperatures: torch.Tensor, keys: torch.Tensor) -> torch.Tensor:
    _need(logits.dim() == 2, "sample: logits must be [rows, vocab]")
    n = logits.shape[0]
    _dense(logits, "sample: logits", dtype=torch.float32)
    _dense(temperatures, "sample: temperatures", (n,), torch.float32)
    _dense(keys, "sample: keys", (n,), torch.int64)
    tokens = torch.empty((n,), dtype=torch.int32, device=logits.device)
    backend().sample(logits, temperatures, keys, tokens)
    return tokens
