"""The Vugelix design in the engine against its plain whole-sequence implementation (``plain_vugelix.py``):
every mechanism alone through the kernels' entry points, then whole models through the step function (whole
prompts, decoding token by token, portions down to two tokens, unequal requests side by side on few pages and
slots that are used again), and greedy generation through the entry point and its scheduler. Every test runs on
the CPU stand-in for the kernels (the engine's logic) and, marked ``gpu``, on the HIP kernels in both element types.
"""
import json

import pytest
import torch

import plain_vugelix as plain
import vugelix_cases as vc
from helpers import first_difference, max_abs_diff, tolerance_for
from nanohybrid_vlm_amd.config.model_config import ConfigError
from nanohybrid_vlm_amd.config.registry import resolve_architecture
from nanohybrid_vlm_amd.engine.replay import replay
from nanohybrid_vlm_amd.engine.runner import ModelRunner
from nanohybrid_vlm_amd.native import ops
from nanohybrid_vlm_amd.native.ops import AttentionBatch

CPU = ("cpu", "float32")
ON_GPU = [pytest.param(("cuda:0", "float32"), marks=pytest.mark.gpu, id="gpu-float32"),
          pytest.param(("cuda:0", "bfloat16"), marks=pytest.mark.gpu, id="gpu-bfloat16")]
WHERE = [pytest.param(CPU, id="cpu-stand-in")] + ON_GPU


@pytest.fixture()
def kernels(request):
    """The kernel library for the test's device: the CPU stand-in, or the HIP library (then a GPU is needed)."""
    device, _ = request.getfixturevalue("where")
    if device == "cpu":
        from emulated_kernels import EmulatedBackend
        old = ops._backend
        ops.set_backend(EmulatedBackend())
        yield
        ops.set_backend(old)
    else:
        if not torch.cuda.is_available():
            pytest.skip("no GPU here")
        old = ops._backend
        ops.set_backend(None)
        yield
        ops.set_backend(old)


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    return {name: vc.write_model(str(tmp_path_factory.mktemp(f"vugelix_{name}")), cfg, seed)
            for name, (cfg, seed) in vc.CASES.items()}


def _dt(name):
    return {"float32": torch.float32, "bfloat16": torch.bfloat16}[name]


def _tol(dtype, plain_values, fine=2e-5, coarse=4e-2):
    """Largest allowed difference, as a share of the spread of the plain values."""
    return (fine if dtype == "float32" else coarse) * float(plain_values.float().std())


# ------------------------------------------------------------------ mechanisms alone
@pytest.mark.parametrize("where", WHERE)
@pytest.mark.parametrize("n", [1, 2, 3, 4, 7])
def test_streams_between_sublayers(where, kernels, n):
    """The one kernel between two sublayers: the start from the embedding's rows, an update with one result and with
    two scaled ones, the read through the next norm, and the sum at the end, against the plain update of all streams
    at once from their old values (so a kernel that updates stream by stream in place shows)."""
    device, dtype = where
    g = torch.Generator().manual_seed(n)
    T, W, eps = 6, 70, 1e-4
    x0 = torch.randn(T, W, generator=g) * 2
    w = {"in": torch.randn(n, generator=g), "mix": torch.randn(n, n, generator=g), "out": torch.randn(n, generator=g)}
    norm_w = torch.rand(W, generator=g) + 0.5
    dt = _dt(dtype)
    X = torch.full((n, T, W), float("nan")).to(device)
    h, _ = ops.streams_step(X, T, W, n, dt, start=x0.to(device), read=(w["in"].to(device), norm_w.to(device), eps))
    want_X = x0[None].repeat(n, 1, 1)
    want_h = plain.rms_norm(torch.einsum("s,stw->tw", w["in"], want_X), norm_w, eps)
    assert torch.equal(X.cpu(), want_X) and max_abs_diff(h.cpu(), want_h) <= _tol(dtype, want_h)
    a, b = (torch.randn(T, W, generator=g).to(dt) for _ in range(2))
    for y, y_plain in ((a.to(device), a.float()),
                       (ops.ScaledPairSum(a.to(device), 0.6, b.to(device), -1.5), 0.6 * a.float() - 1.5 * b.float())):
        h, _ = ops.streams_step(X, T, W, n, dt, update=(w["mix"].to(device), w["out"].to(device), y),
                                read=(w["in"].to(device), norm_w.to(device), eps))
        want_X = torch.einsum("sr,stw->rtw", w["mix"], want_X) + w["out"][:, None, None] * y_plain[None]
        want_h = plain.rms_norm(torch.einsum("s,stw->tw", w["in"], want_X), norm_w, eps)
        assert max_abs_diff(X.cpu(), want_X) <= 1e-5 * float(want_X.abs().max())
        assert max_abs_diff(h.cpu(), want_h) <= _tol(dtype, want_h)
        want_X = X.cpu().clone()
    before = X.clone()
    _, total = ops.streams_step(X, T, W, n, dt, update=(w["mix"].to(device), w["out"].to(device), b.to(device)), collapse=True)
    want = (torch.einsum("sr,stw->rtw", w["mix"], want_X) + w["out"][:, None, None] * b.float()[None]).sum(0)
    assert max_abs_diff(total.cpu(), want) <= 1e-5 * float(want.abs().max()) and torch.equal(X, before)
    pair = ops.ScaledPairSum(a.to(device), 0.6, b.to(device), -1.5).tensor()
    assert max_abs_diff(pair.float().cpu(), 0.6 * a.float() - 1.5 * b.float()) <= _tol(dtype, a.float())
    if n == 1:                                                  # one stream without coefficients: x + y, then the norm
        X1 = x0.clone().to(device).view(1, T, W)
        h, _ = ops.streams_step(X1, T, W, 1, dt, update=(None, None, a.to(device)), read=(None, norm_w.to(device), eps))
        assert max_abs_diff(X1[0].cpu(), x0 + a.float()) <= 1e-6 * float(x0.abs().max())
        assert max_abs_diff(h.cpu(), plain.rms_norm(x0 + a.float(), norm_w, eps)) <= _tol(dtype, want_h)
    else:
        with pytest.raises(ops.KernelError):
            ops.streams_step(X, T, W, n, dt, update=(None, None, a.to(device)))


@pytest.mark.parametrize("where", WHERE)
def test_small_kernels(where, kernels):
    device, dtype = where
    g = torch.Generator().manual_seed(3)
    dt = _dt(dtype)
    table = torch.randn(30, 20, generator=g).to(dt)
    ids = torch.tensor([4, 29, 0, 4], dtype=torch.int32)
    got = ops.embed_float(ids.to(device), table.to(device), 2.5)
    assert got.dtype == torch.float32 and torch.equal(got.cpu(), table.float()[ids.long()] * 2.5)
    z = (torch.randn(5, 33, generator=g) * 3).to(dt)
    for name, fn in (("relu2", plain.squared_relu), ("silu", plain.silu)):
        got = ops.activation_(z.clone().to(device), name)
        want = fn(z.float())                                   # (taken in float and rounded once: one part in 2^8 in bfloat16)
        assert bool(((got.float().cpu() - want).abs() <= (2e-6 if dtype == "float32" else 2.0 ** -8) * want.abs() + 1e-6).all())
    with pytest.raises(ops.KernelError):
        ops.activation_(z.clone().to(device), "cube")
    x = torch.randn(4, 9, generator=g)
    assert torch.equal(ops.scale_(x.clone().to(device), 0.25).cpu(), x * 0.25)
    # a product with its activation: few rows (one kernel in bfloat16 on the GPU) and many
    wm = (torch.randn(72, 40, generator=g) / 40 ** 0.5 * 2).to(dt)
    for rows in (1, 5, 16, 33, 200):
        xm = torch.randn(rows, 40, generator=g).to(dt)
        for name, fn in (("relu2", plain.squared_relu), ("silu", plain.silu), ("gelu_tanh", None)):
            got = ops.activated_linear(xm.to(device), wm.to(device), name)
            z = xm.float() @ wm.float().T
            want = fn(z) if fn is not None else torch.nn.functional.gelu(z, approximate="tanh")
            # (many rows in bfloat16: the product's rows are rounded before the activation, which may double their
            # relative error, and once after it)
            bound = _tol(dtype, want, coarse=1e-2) + (2.0 ** -6 * want.abs() if dtype == "bfloat16" else 0.0)
            assert got.dtype == dt and bool(((got.float().cpu() - want).abs() <= bound).all()), (rows, name)


def _single_request_batch(T, start, device, page_size, pages):
    pos = torch.arange(start, start + T, dtype=torch.int32)
    slots = torch.tensor([pages[p // page_size] * page_size + p % page_size for p in pos.tolist()], dtype=torch.int32)
    batch = AttentionBatch(num_tokens=T, num_requests=1, token_req=torch.zeros(T, dtype=torch.int32).to(device),
                           positions=pos.to(device), cu_seqlens_q=torch.tensor([0, T], dtype=torch.int32).to(device),
                           context_lens=torch.tensor([start + T], dtype=torch.int32).to(device), max_q_len=T,
                           max_context_len=start + T)
    return batch, slots.to(device), torch.tensor([pages], dtype=torch.int32).to(device)


def _attention_through_kernels(device, dtype, m, q_in, k_in, v_in, g_in, portions, page_size, sink=0.0):
    """q_in [T, H D], k_in [T, G D], v_in [T, G E], g_in [T, H] (or None) as projected: split, turned, stored and read
    back by the kernels in the given portions of one request, on pages handed out in a scrambled order."""
    T = q_in.shape[0]
    H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    n_pages = -(-T // page_size)
    pages = torch.randperm(n_pages + 2, generator=torch.Generator().manual_seed(T)).tolist()[:n_pages]
    dt = _dt(dtype)
    k_cache = torch.full((n_pages + 2, page_size, G, D), float("nan"), dtype=dt).to(device)
    v_cache = torch.full((n_pages + 2, page_size, G, E), float("nan"), dtype=dt).to(device)
    dims = m["rot"]["dims"]
    f = (m["rot"]["base"] ** (-2.0 * torch.arange(dims // 2, dtype=torch.float64) / dims)).float() if dims else None
    gates = 0 if g_in is None else H
    packed = torch.cat((q_in, k_in, v_in) + (() if g_in is None else (g_in,)), dim=1).to(dt).to(device)
    outs, at = [], 0
    for n in portions:
        batch, slots, table = _single_request_batch(n, at, device, page_size, pages)
        rows = packed[at:at + n].contiguous()
        q = ops.rotary_split_write(rows, None, None if f is None else f.to(device), None, batch.positions, slots, k_cache,
                                   v_cache, H, G, D, E, more_columns=gates)
        o = ops.paged_attention(q, k_cache, v_cache, batch, table, m["scale"], m["mask"]["size"], None,
                                softcap=m.get("softcap"), sink=sink, gate=(rows, rows.shape[1] - gates) if gates else None)
        outs.append(o.float().cpu())
        at += n
    assert at == T
    return torch.cat(outs)


def _plain_attention(m, q_in, k_in, v_in, g_in):
    T = q_in.shape[0]
    H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = plain.turn_first_dims(q_in.double().view(T, H, D), m["rot"]["dims"], m["rot"]["base"])
    k = plain.turn_first_dims(k_in.double().view(T, G, D), m["rot"]["dims"], m["rot"]["base"])
    o = plain.sink_attention(q, k, v_in.double().view(T, G, E), m["scale"], m.get("softcap"), plain.window_mask(T, m["mask"]["size"]))
    if g_in is not None:
        o = o * torch.sigmoid(g_in.double())[:, :, None]
    return o.float()


@pytest.mark.parametrize("where", WHERE)
@pytest.mark.parametrize("sizes", [(12, 20, 3), (32, 32, 2), (16, 16, 6), (64, 64, 1)], ids=lambda s: "D%d-E%d-group%d" % s)
@pytest.mark.parametrize("window", [7, 40, 1000])
def test_windowed_attention_alone(where, kernels, sizes, window):
    """Random queries, keys and values under a window, with a partial rotation, scores large enough that the cap bends
    them, the further term in the denominator and a gate per head; value heads of another size than the key heads, and
    of the same size in steps of 16 (which the kernels on the matrix cores take in bfloat16); portions that end inside
    pages and inside windows."""
    device, dtype = where
    D, E, group = sizes
    m = vc._left(2 * group, 2, D, E, window, 8, 300.0, 1.5 * D ** -0.5, 2.5)
    g = torch.Generator().manual_seed(5)
    T = 90
    q_in, k_in, v_in, g_in = (torch.randn(T, n, generator=g) for n in (2 * group * D, 2 * D, 2 * E, 2 * group))
    if dtype == "bfloat16":
        q_in, k_in, v_in, g_in = (t.bfloat16().float() for t in (q_in, k_in, v_in, g_in))
    want = _plain_attention(m, q_in, k_in, v_in, g_in)
    uncapped = _plain_attention(dict(m, softcap=None), q_in, k_in, v_in, g_in)
    assert max_abs_diff(want, uncapped) > 0.05                # the cap matters in this test
    for portions in ([T], [1] * T, [2, 5, 3, 11, 1, 2, 21, 45]):
        got = _attention_through_kernels(device, dtype, m, q_in, k_in, v_in, g_in, portions, 4)
        assert max_abs_diff(got, want) <= _tol(dtype, want), (portions, first_difference(got.flatten(1), want.flatten(1), _tol(dtype, want)))
    # without gate and without cap, with a sink of another score
    m2 = dict(m, softcap=None)
    want = _plain_attention(m2, q_in, k_in, v_in, None)
    got = _attention_through_kernels(device, dtype, m2, q_in, k_in, v_in, None, [37, 1, 1, 51], 4)
    assert max_abs_diff(got, want) <= _tol(dtype, want)


@pytest.mark.parametrize("where", WHERE)
@pytest.mark.parametrize("E", [6, 16], ids=["values of their own size", "values of the keys' size"])
def test_one_key_that_stands_out_under_a_window(where, kernels, E):
    """Among 300 keys one is made to carry nearly all the weight of every query that sees it; its value is a vector no
    other key has. A query then returns that value exactly when the key lies among the last ``window`` positions up to
    its own: for the marked key at the first place, at a page's border and far back, and for queries just inside and
    just outside, in a prompt and decoded one by one. All other scores are far below the further term of the
    denominator, so a query that does not see the key returns nearly nothing: a kernel that leaves that term out returns
    a mean of the values instead. No rotation, so the scores are known."""
    device, dtype = where
    window, page, T, D = 48, 16, 300, 16
    m = vc._left(2, 1, D, E, window, 0, 10.0, 1.0, 40.0)
    for marked in (0, 15, 16, 47, 48, 100, 191, 240, 251):
        g = torch.Generator().manual_seed(marked)
        q_in = 0.1 * torch.randn(T, 2 * D, generator=g)
        k_in = 0.1 * torch.randn(T, D, generator=g)
        v_in = 1.0 + 0.1 * torch.randn(T, E, generator=g)
        q_in[:, 0] = q_in[:, D] = 4.0                 # every query asks for coordinate 0 ...
        k_in[:, 0] = -2.0                             # ... which every key answers with a score of -8, far below the sink's 0,
        k_in[marked, 0] = 8.0                         # but for the marked key: its score is 32 (the cap leaves it at 26.6)
        v_in[marked] = torch.tensor([5.0, -5.0] * (E // 2))
        for portions in ([T], [marked + 1] + [1] * (T - marked - 1) if marked < 200 else [T - 60] + [1] * 60):
            got = _attention_through_kernels(device, dtype, m, q_in, k_in, v_in, None, portions, page)
            sees = torch.tensor([0 <= i - marked < window for i in range(T)])
            hit = (got[:, 0, 0] > 4.5) & (got[:, 1, 1] < -4.5)
            assert torch.equal(hit, sees), (marked, len(portions), (hit != sees).nonzero().flatten().tolist())
            assert got[~sees].abs().max() < 0.1, (marked, float(got[~sees].abs().max()))


def _delta_inputs(T, H, G, D, E, n, seed):
    g = torch.Generator().manual_seed(seed)
    C = 2 * G * D + H * E
    return {"proj": torch.randn(T, C + 2 * H + H * E, generator=g), "taps": 0.6 * torch.randn(C, n, generator=g),
            "dt_bias": torch.randn(H, generator=g) - 0.5, "a_log": 0.5 * torch.randn(H, generator=g) - 0.5,
            "norm": 1.0 + 0.2 * torch.randn(E, generator=g)}


def _plain_delta(x, H, G, D, E, eps):
    """The recurrent mixer between its projections, from the plain functions, in float64: one decay a head, q and k
    heads shared by groups of value heads, SiLU gates. ``proj``: q | k | v | beta | a | gate."""
    x = {k: v.double() for k, v in x.items()}
    T = x["proj"].shape[0]
    C = 2 * G * D + H * E
    act = plain.silu(plain.causal_taps(x["proj"][:, :C], x["taps"]))
    unit = lambda t: t / torch.sqrt(t.pow(2).sum(-1, keepdim=True) + 1e-6)      # noqa: E731
    rep = H // G
    q = unit(act[:, :G * D].view(T, G, D)).repeat_interleave(rep, dim=1) * D ** -0.5
    k = unit(act[:, G * D:2 * G * D].view(T, G, D)).repeat_interleave(rep, dim=1)
    v = act[:, 2 * G * D:].view(T, H, E)
    beta = torch.sigmoid(x["proj"][:, C:C + H])
    decay = torch.exp(-torch.exp(x["a_log"]) * plain.softplus(x["proj"][:, C + H:C + 2 * H] + x["dt_bias"]))
    o = plain.delta_recurrence(q, k, v, decay, beta)
    gate = plain.silu(x["proj"][:, C + 2 * H:]).view(T, H, E)
    return (plain.rms_norm(o, x["norm"], eps) * gate).reshape(T, H * E).float()


@pytest.mark.parametrize("where", WHERE)
@pytest.mark.parametrize("sizes", [(4, 2, 8, 6, 4), (1, 1, 3, 3, 1), (6, 3, 20, 5, 2), (2, 1, 64, 64, 3), (4, 1, 96, 40, 5)],
                         ids=lambda s: "H%d-G%d-D%d-E%d-taps%d" % s)
def test_delta_rule_with_one_decay_a_head(where, kernels, sizes):
    """Two requests of unequal length side by side, in portions (the state and the convolutions' last inputs go
    through the slots), against the recurrence written out token by token; then the slots are used again by new
    requests, which must start from zero. Decays, betas and gates are columns of the one packed projection."""
    device, dtype = where
    H, G, D, E, n = sizes
    eps, slots = 1e-5, 3
    C = 2 * G * D + H * E
    lengths = {"a": 23, "b": 9}
    x = {r: _delta_inputs(T, H, G, D, E, n, 7 + T) for r, T in lengths.items()}
    for r in x:           # both requests are the same layer: they share its weights
        for name in ("taps", "dt_bias", "a_log", "norm"):
            x[r][name] = x["a"][name]
    want = {r: _plain_delta(x[r], H, G, D, E, eps) for r in x}
    shared = {name: x["a"][name].to(device) for name in ("taps", "dt_bias", "a_log", "norm")}
    kept = torch.full((slots + 1, C, n - 1), float("nan")).to(device)           # (what a slot held before must not matter)
    state = torch.full((slots + 1, H, E, D), float("nan")).to(device)
    for round_, slot_of in enumerate(({"a": 2, "b": 0}, {"a": 0, "b": 2})):     # the second round uses the slots again
        at = {r: 0 for r in lengths}
        plan = [{"a": 5, "b": 1}, {"a": 1}, {"b": 2, "a": 2}, {"a": 3, "b": 1}, {"a": 1, "b": 5}, {"a": 11}]
        got = {r: [] for r in lengths}
        for step in plan:
            reqs = list(step)
            rows = torch.cat([torch.arange(at[r], at[r] + step[r]) for r in reqs])
            cu = torch.tensor([0] + list(torch.tensor([step[r] for r in reqs]).cumsum(0)), dtype=torch.int32)
            T = int(cu[-1])
            batch = AttentionBatch(num_tokens=T, num_requests=len(reqs),
                                   token_req=torch.repeat_interleave(torch.arange(len(reqs), dtype=torch.int32),
                                                                     torch.tensor([step[r] for r in reqs])).to(device),
                                   positions=rows.to(torch.int32).to(device), cu_seqlens_q=cu.to(device),
                                   context_lens=torch.tensor([at[r] + step[r] for r in reqs], dtype=torch.int32).to(device),
                                   max_q_len=max(step.values()), max_context_len=32)
            proj = torch.cat([x[r]["proj"][at[r]:at[r] + step[r]] for r in reqs]).to(device)
            y = ops.gated_delta_rule(proj, None, None, shared["taps"], shared["dt_bias"], shared["a_log"], shared["norm"], eps,
                                     kept, state, batch, torch.tensor([slot_of[r] for r in reqs], dtype=torch.int32).to(device),
                                     H, G, D, E, _dt(dtype), decay_per_head=True, gate_activation="silu")
            y = y.float().cpu()
            for i, r in enumerate(reqs):
                got[r].append(y[int(cu[i]):int(cu[i + 1])])
                at[r] += step[r]
        for r in lengths:
            assert at[r] == lengths[r]
            out = torch.cat(got[r])
            # (the result is rounded once to its element type: one part in 2^8 of every entry in bfloat16)
            bound = _tol(dtype, want[r], fine=1e-4, coarse=2e-2) + (2.0 ** -8 * want[r].abs() if dtype == "bfloat16" else 0.0)
            assert bool(((out - want[r]).abs() <= bound).all()), (round_, r, first_difference(out, want[r], 1e-3))


@pytest.mark.parametrize("where", WHERE)
def test_a_value_written_far_back_is_read_from_the_state(where, kernels):
    """One token writes a value under a key that no other token uses (its key is the unit vector of channel 0; all other
    keys have nothing there), with decays of nearly 1. Every later query that asks for channel 0 then reads that value
    back from the state, hundreds of tokens later, whatever the portions were (the slot held no numbers before); a
    query before the marked token reads nothing of it. One tap, so the inputs are known."""
    device, dtype = where
    H, G, D, E, eps = 2, 1, 8, 6, 1e-6
    C = 2 * G * D + H * E
    T, marked = 400, 37
    g = torch.Generator().manual_seed(4)
    proj = torch.zeros(T, C + 2 * H + H * E)
    q_in, k_in = torch.full((T, D), -30.0), 0.5 * torch.randn(T, D, generator=g).abs() + 0.5
    q_in[:, 0] = 6.0                                         # every query: the unit vector of channel 0
    k_in[:, 0] = -30.0                                       # no key has anything in channel 0 (SiLU of -30 is nothing) ...
    k_in[marked] = -30.0
    k_in[marked, 0] = 6.0                                    # ... but the marked one, which has nothing else
    v_in = 0.3 * torch.randn(T, H * E, generator=g)
    v_in[marked] = torch.tensor([3.0, -3.0, 3.0, 3.0, -3.0, -3.0] * H)
    proj[:, :D], proj[:, D:2 * D], proj[:, 2 * D:C] = q_in, k_in, v_in
    proj[:, C:C + H] = 8.0                                   # beta: nearly 1
    proj[:, C + H:C + 2 * H] = -12.0                         # decays: exp(-rate * softplus(-12 + bias)), nearly 1
    proj[:, C + 2 * H:] = 2.0                                # gates: SiLU(2), the same for every entry
    taps = torch.ones(C, 1)
    dt_bias, a_log, norm = torch.zeros(H), torch.zeros(H), torch.ones(E)
    want = torch.nn.functional.silu(v_in[marked]).view(H, E)         # what the marked token wrote, as the read-out's norm and gate leave it
    want = want / torch.sqrt(want.pow(2).mean(-1, keepdim=True) + eps) * float(torch.nn.functional.silu(torch.tensor(2.0)))
    kept = torch.zeros((3, C, 0)).to(device)
    for portions in ([T], [marked] + [1] * 20 + [T - marked - 20], [2, 33, 5, 1, 1, 200, 1, 1, 156]):
        state = torch.full((3, H, E, D), float("nan")).to(device)
        at, outs = 0, []
        for n in portions:
            batch = AttentionBatch(num_tokens=n, num_requests=1, token_req=torch.zeros(n, dtype=torch.int32).to(device),
                                   positions=torch.arange(at, at + n, dtype=torch.int32).to(device),
                                   cu_seqlens_q=torch.tensor([0, n], dtype=torch.int32).to(device),
                                   context_lens=torch.tensor([at + n], dtype=torch.int32).to(device), max_q_len=n,
                                   max_context_len=at + n)
            y = ops.gated_delta_rule(proj[at:at + n].contiguous().to(device), None, None, taps.to(device), dt_bias.to(device),
                                     a_log.to(device), norm.to(device), eps, kept, state, batch,
                                     torch.tensor([1], dtype=torch.int32).to(device), H, G, D, E, _dt(dtype),
                                     decay_per_head=True, gate_activation="silu")
            outs.append(y.float().cpu().view(n, H, E))
            at += n
        got = torch.cat(outs)
        # from the marked token on the read-out is the marked value alone; before it nothing is read: zeros
        close = ((got[marked:] - want).abs() < 0.05).all(-1).all(-1)
        assert bool(close.all()), (portions, marked + int((~close).nonzero()[0]))
        assert float(got[:marked].abs().max()) < 1e-2


# ------------------------------------------------------------------ configuration and weights
def test_configuration_and_names(folders):
    from nanohybrid_vlm_amd.parts.base import CombinedNeed
    from nanohybrid_vlm_amd.parts.model import DecoderModel
    arch = resolve_architecture(vc.CONFIG_A)
    assert arch.name == "Vugelix"
    cfg = arch.parse_config(vc.CONFIG_A)
    assert cfg.layers[2].weights_of == 0 and cfg.layers[1].ff is None and cfg.owners() == [0, 1, 3]
    spec = arch.build_spec(cfg)
    assert [e.layer for e in spec.order()] == [0, 1, 0, 2, 1] and all(e.cache is None for e in spec.order())
    model = DecoderModel(spec)
    # every stored tensor has its place, and every parameter is filled by stored tensors
    names = arch.checkpoint_names(cfg)
    assert set(names) == set(vc.random_tensors(vc.CONFIG_A, 0))
    assert {s.param for s in names.values()} == set(model.all_param_specs())
    # every run of a layer has pages and a state of its own, also where two runs share their weights
    needs = model.cache_needs()
    assert len(needs) == 5 and all(isinstance(n, CombinedNeed) for n in needs)
    assert needs[0] == needs[2] and needs[0].paged.window == 6 and needs[1].paged.value_size == 4
    # a model without stream coefficients has none among its tensors
    cfg_c = arch.parse_config(vc.CONFIG_C)
    assert cfg_c.streams is None and set(arch.checkpoint_names(cfg_c)) == set(vc.random_tensors(vc.CONFIG_C, 0))
    for change, match in ((lambda c: c["layers"][2].update(weights_of=2), "weights_of"),
                          (lambda c: c["layers"][4].update(weights_of=2), "weights_of"),
                          (lambda c: c["layers"][2]["mixer"].update(left_scale=0.1), "must equal"),
                          (lambda c: c["layers"][1].update(type="other"), "not known"),
                          (lambda c: c["layers"][0]["mixer"]["left"]["rot"].update(dims=3), "rot.dims"),
                          (lambda c: c["layers"][0]["mixer"]["right"].update(kv_heads=3), "multiple"),
                          (lambda c: c.update(streams=0), "streams")):
        bad = json.loads(json.dumps(vc.CONFIG_A))
        change(bad)
        with pytest.raises(ConfigError, match=match):
            arch.parse_config(bad)


# ------------------------------------------------------------------ whole models through the step function
def _requests(name, lengths):
    vocab = vc.CASES[name][0]["vocab"]
    return {f"r{i}": vc.tokens(vocab, n, 100 * i + n) for i, n in enumerate(lengths)}


def _plain_logits(folder, requests, dtype=torch.float64):
    """(in float64: what the comparison then shows is the engine's own rounding, not the oracle's)"""
    cfg, w = plain.read_model_folder(folder)
    return {rid: plain.logits(cfg, w, toks, dtype).float() for rid, toks in requests.items()}


def _replay(folder, where, steps, page_size, max_live, **options):
    device, dtype = where
    pages = max(1, vc.peak_tokens(steps, page_size) // page_size)
    runner = ModelRunner(folder, dtype=dtype, device=device, page_size=page_size, num_pages=pages, num_state_slots=max_live,
                         max_model_len=pages * page_size, poison_freed_pages=True, **options)
    got = replay(runner, steps)
    assert not runner.cache.requests and all(runner.cache.num_free_pages(g) == pages for g in range(len(runner.cache.groups)))
    return got


def _compare(got, want, dtype, what):
    """float32: every logit within 1e-4 of the logits' spread. bfloat16: the recurrent mixer's read-out is divided by
    its own root mean square, which at a request's first tokens is |q . k| times the size of one value vector, so where
    q . k is near zero a rounding of the mixer's input to eight bits moves the result by its own size (the same shows
    with the CPU stand-in's roundings): single positions are far off by rounding alone, and the bound is on the
    positions' errors taken together. What it cannot see (one key more or less in a window, a state or a page of
    another request) shows in the float32 run of the same steps and in the tests of the mechanisms alone, which hold
    the bfloat16 kernels to a close bound."""
    if dtype == "float32":
        tol = tolerance_for(dtype, want)
        for rid in want:
            assert max_abs_diff(got[rid], want[rid]) <= tol, (what, rid, first_difference(got[rid], want[rid], tol))
        return
    spread = float(torch.cat([t.reshape(-1) for t in want.values()]).float().std())
    errors = torch.cat([(got[rid].float() - want[rid].float()).abs().max(dim=-1).values for rid in want]) / spread
    assert bool(torch.isfinite(errors).all()), what
    assert float(errors.median()) <= 0.06 and float((errors > 0.15).float().mean()) <= 0.2 and float(errors.max()) <= 1.5, \
        (what, float(errors.median()), float((errors > 0.15).float().mean()), float(errors.max()))


@pytest.mark.parametrize("where", WHERE)
def test_layers_one_by_one(folders, where, kernels):
    """The stream after the last layer run is what the plain model has there (the engine's rows before its last norm
    are not handed out, so the comparison is of the last norm's input through a model whose last norm and head are
    the identity on a few coordinates: here simply the logits of models cut off after 1, 2, ... layer runs)."""
    device, dtype = where
    cfg, w = plain.read_model_folder(folders["A"])
    toks = vc.tokens(cfg["vocab"], 21, 9)
    import os
    for runs in range(1, len(cfg["layers"]) + 1):
        cut = dict(cfg, layers=cfg["layers"][:runs])
        keep = {f"l{i}." for i, layer in enumerate(cut["layers"]) if "weights_of" not in layer}
        tensors = {k: v.bfloat16() for k, v in w.items() if not k.startswith("l") or k[:k.index(".") + 1] in keep}
        folder = vc.write_model(os.path.join(folders["A"], f"cut{runs}"), cut, 0, tensors)
        want = {"a": plain.logits(cut, w, toks, torch.float64).float()}
        got = _replay(folder, where, vc.in_portions({"a": toks}, [8, 1, 5, 7]), page_size=4, max_live=1)
        _compare(got, want, dtype, f"{runs} layer runs")


@pytest.mark.parametrize("where", WHERE)
@pytest.mark.parametrize("name", ["A", "B", "C", "R"])
def test_ways_of_cutting_agree_with_the_plain_model(folders, where, kernels, name):
    """Whole prompts, a prompt followed by its last tokens one by one, portions of several sizes down to two tokens
    (and single tokens between them), and unequal requests side by side on pages and slots that are used again: all
    give the plain model's logits at every position. In float32 on the GPU the ways agree bit for bit."""
    device, dtype = where
    lengths = [1, 2, 26, 19, 37, 5, 30] if device == "cpu" else [1, 2, 26, 19, 61, 5, 150, 43]
    requests = _requests(name, lengths)
    want = _plain_logits(folders[name], requests)
    ways = {
        "whole": (vc.whole(requests), 3),
        "tail": ([s for rid, toks in requests.items()
                  for s in vc.in_portions({rid: toks}, [max(1, len(toks) - 12)] + [1] * 12)], 3),
        "portions": (vc.in_portions(requests, [2, 3, 5, 2, 1, 7, 4, 2, 11]), 3),
        "side by side": (vc.interleaved(requests, [3, 1, 2, 6, 1, 1, 4], 3), 3),
    }
    results = {}
    for what, (steps, live) in ways.items():
        for i, s in enumerate(steps):
            s["step"] = i
        results[what] = _replay(folders[name], where, steps, page_size=4, max_live=live)
        _compare(results[what], want, dtype, what)
    if device != "cpu" and dtype == "float32":
        for what in ("tail", "portions", "side by side"):
            for rid in want:
                assert torch.equal(results[what][rid], results["whole"][rid]), (what, rid)


@pytest.mark.parametrize("where", WHERE)
@pytest.mark.parametrize("seed", range(8))
def test_configurations_drawn_at_random(where, kernels, seed, tmp_path):
    """Models of sizes drawn at random (see ``vugelix_cases.random_config``) in portions, side by side and with a decoded
    tail, on pages of 16 tokens that are used again, against the plain model; float32 bit-equal across the ways on the GPU."""
    device, dtype = where
    cfg = vc.random_config(seed)
    folder = vc.write_model(str(tmp_path / "m"), cfg, 500 + seed)
    lengths = [1, 21, 40, 7] if device == "cpu" else [1, 70, 210, 33, 131]
    requests = {f"r{i}": vc.tokens(cfg["vocab"], n, 7 * i + n) for i, n in enumerate(lengths)}
    want = _plain_logits(folder, requests)
    ways = {"portions": vc.in_portions(requests, [17, 2, 3, 64, 1, 33]),
            "side by side": vc.interleaved(requests, [5, 1, 2, 31, 1, 1, 16], 3),
            "tail": [s for rid, toks in requests.items() for s in vc.in_portions({rid: toks}, [max(1, len(toks) - 20)] + [1] * 20)]}
    results = {}
    for what, steps in ways.items():
        for i, s in enumerate(steps):
            s["step"] = i
        results[what] = _replay(folder, where, steps, page_size=16, max_live=3)
        _compare(results[what], want, dtype, (seed, what))
    if device != "cpu" and dtype == "float32":
        for rid in want:
            assert torch.equal(results["portions"][rid], results["side by side"][rid]) and \
                torch.equal(results["portions"][rid], results["tail"][rid]), (seed, rid)


@pytest.mark.parametrize("where", ON_GPU)
def test_pages_of_64_and_windows_longer_than_a_page(folders, where, kernels):
    """Pages of 64 tokens (whole tiles of the prompt kernel lie in one page) under windows of 96 and 160 positions,
    requests of up to 400 tokens in portions that end anywhere, beside decoded tokens, on few pages."""
    device, dtype = where
    requests = _requests("S", [400, 130, 70, 257])
    want = _plain_logits(folders["S"], requests)
    for what, steps in (("portions", vc.in_portions(requests, [37, 2, 64, 5, 1, 129, 1, 1, 96])),
                        ("side by side", vc.interleaved(requests, [33, 1, 1, 64, 1, 7, 1, 100], 3))):
        got = _replay(folders["S"], where, steps, page_size=64, max_live=3)
        _compare(got, want, dtype, what)


@pytest.mark.parametrize("where", ON_GPU)
def test_sizes_of_a_real_models_layers(where, kernels, tmp_path):
    """Heads and states of 128 and 64 entries, a width of 1,024: the kernels' makes that real sizes take (the streams'
    kernel with 256 threads a block and more, the products of few rows with their activation, the recurrence with
    columns of 128), in portions and side by side on pages of 64, with decoded tokens between."""
    device, dtype = where
    folder = vc.write_model(str(tmp_path / "w"), vc.CONFIG_W, 26)
    requests = {f"r{i}": vc.tokens(vc.CONFIG_W["vocab"], n, 11 * i + n) for i, n in enumerate([300, 40, 129])}
    want = _plain_logits(folder, requests)
    for what, steps in (("portions", vc.in_portions(requests, [150, 1, 1, 16, 3, 64, 1, 1, 1])),
                        ("side by side", vc.interleaved(requests, [40, 1, 1, 1, 17, 1, 64, 1], 3))):
        got = _replay(folder, where, steps, page_size=64, max_live=3)
        _compare(got, want, dtype, what)


@pytest.mark.parametrize("where", WHERE)
def test_long_decoding(folders, where, kernels):
    """Two tokens of prompt, then many tokens one by one: the windows of every layer pass many times, pages go back
    to the pool on the way, and the recurrent state is carried through every step."""
    device, dtype = where
    n = 60 if device == "cpu" else 142
    requests = _requests("A", [n])
    want = _plain_logits(folders["A"], requests)
    steps = vc.in_portions(requests, [2] + [1] * n)
    got = _replay(folders["A"], where, steps, page_size=4, max_live=1)
    _compare(got, want, dtype, "decoding")


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_recorded_steps_equal_eager_steps(folders, dtype):
    """Steps replayed from HIP graphs (single tokens, and short mixed steps) give what eager steps give."""
    if not torch.cuda.is_available():
        pytest.skip("no GPU here")
    old = ops._backend
    ops.set_backend(None)
    try:
        requests = _requests("R", [40, 3, 17, 9])
        steps = vc.interleaved(requests, [3, 1, 1, 1, 2, 1, 1], 3)
        for s in steps:                                      # a recorded short step gives one place a request
            for e in s["entries"]:
                e["want"] = e["want"][-1:]
        where = ("cuda:0", dtype)
        eager = _replay(folders["R"], where, steps, page_size=8, max_live=3, use_graphs=False)
        recorded = _replay(folders["R"], where, steps, page_size=8, max_live=3, use_graphs=True)
        for rid in eager:
            if dtype == "float32":
                assert torch.equal(eager[rid], recorded[rid]), rid
            else:
                assert max_abs_diff(eager[rid], recorded[rid]) <= 0.05 * float(eager[rid].std()), rid
    finally:
        ops.set_backend(old)


# ------------------------------------------------------------------ generation through the entry point
@pytest.mark.parametrize("where", [pytest.param(CPU, id="cpu-stand-in"), ON_GPU[0]])
@pytest.mark.parametrize("options", [dict(kvcache_block_size=4, num_kvcache_blocks=64),
                                     dict(kvcache_block_size=8, num_kvcache_blocks=40, max_num_batched_tokens=7, max_num_seqs=2)],
                         ids=["whole prompts", "portions of 7, two at a time"])
def test_greedy_generation_through_the_entry_point(folders, where, kernels, options):
    from nanohybrid_vlm_amd import LLM, SamplingParams
    device, dtype = where
    cfg, w = plain.read_model_folder(folders["A"])
    prompts = [vc.tokens(cfg["vocab"], n, 300 + n) for n in (1, 13, 22)]
    llm = LLM(folders["A"], device=device, dtype=dtype, **options)
    outs = llm.generate(prompts, SamplingParams(temperature=0.0, max_tokens=9, ignore_eos=True), use_tqdm=False)
    for prompt, out in zip(prompts, outs):
        assert out["token_ids"] == plain.greedy_generate(cfg, w, prompt, 9)
    stats = llm.get_memory_stats()
    assert stats["live_requests"] == 0 and all(g["free_pages"] == g["pages"] for g in stats["groups"])
    assert stats["state_pool_bytes"] > 0


# ------------------------------------------------------------------ the command line
def _command(*args):
    import os
    import subprocess
    import sys
    repo = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    proc = subprocess.run([sys.executable, "-m", "nanohybrid_vlm_amd", *args], cwd=repo, capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-3000:]
    return proc.stdout


def test_random_model_of_a_named_shape(tmp_path, emulated_kernels):
    """``random-model --shape vugelix-tiny`` writes a folder that the plain implementation and the engine both read."""
    out = str(tmp_path / "m")
    _command("random-model", "--out", out, "--shape", "vugelix-tiny", "--seed", "5")
    cfg, w = plain.read_model_folder(out)
    assert cfg["architecture"] == "Vugelix" and "l2.norm1" not in w and w["l0.hc1.mix"].shape == (cfg["streams"],) * 2
    requests = {"a": vc.tokens(cfg["vocab"], 31, 1)}
    want = {"a": plain.logits(cfg, w, requests["a"])}
    got = _replay(out, CPU, vc.in_portions(requests, [4, 1, 9]), page_size=8, max_live=1)
    _compare(got, want, "float32", "portions")


@pytest.mark.gpu
def test_generate_command_with_random_weights():
    if not torch.cuda.is_available():
        pytest.skip("no GPU here")
    out = json.loads(_command("generate", "--random-weights", "4", "--shape", "vugelix-tiny", "--prompt-ids", "5 17 3",
                              "--prompt-ids", "9 8 7 6 5 4 3 2 1", "--output-tokens", "6", "--temperature", "0", "--ignore-eos",
                              "--block-size", "8", "--num-blocks", "32", "--max-model-len", "64", "--quiet"))
    assert [len(o["token_ids"]) for o in out] == [6, 6]


# ------------------------------------------------------------------ the replay program
@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_replay_program_on_a_model_of_this_design(folders, dtype, tmp_path):
    """``bin/trace_run`` as a user starts it: steps on standard input, ``<step>.f32`` files, pages of 64 and four
    state slots that several traces in one run use again, steps of single tokens and short mixed steps from graphs."""
    if not torch.cuda.is_available():
        pytest.skip("no GPU here")
    from test_replay import _logits_from_files, _renamed, _trace_run
    requests = _requests("S", [150, 9, 71, 2, 40])
    want = _plain_logits(folders["S"], requests)
    ways = {"portions": vc.in_portions(requests, [37, 2, 64, 5, 1, 1]),
            "side by side": vc.interleaved(requests, [33, 1, 1, 16, 1, 7, 1], 4)}
    steps, first = [], 0
    for k, (what, t) in enumerate(ways.items()):
        steps += _renamed(t, f"#{k}", first)
        first += len(t)
    out_dir = str(tmp_path / "out")
    _trace_run(folders["S"], dtype, steps, out_dir, max(vc.peak_tokens(t, 64) for t in ways.values()))
    got = _logits_from_files(out_dir, steps, vc.CONFIG_S["vocab"])
    for k, what in enumerate(ways):
        _compare({rid: got[f"{rid}#{k}"] for rid in want}, want, dtype, what)
