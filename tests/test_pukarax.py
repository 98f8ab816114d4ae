"""The Pukarax design in the engine against its plain whole-sequence implementation (``plain_pukarax.py``):
every mechanism alone through the kernels' entry points, then whole models through the step function (whole
prompts, decoding token by token, portions down to two tokens, unequal requests side by side on few pages and
slots that are used again), and greedy generation through the entry point and its scheduler. Every test runs on
the CPU stand-in for the kernels (the engine's logic) and, marked ``gpu``, on the HIP kernels in both element types.
"""
import json
import os

import pytest
import torch

import plain_pukarax as plain
import pukarax_cases as pc
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
    old = ops._backend
    if device == "cpu":
        from emulated_kernels import EmulatedBackend
        ops.set_backend(EmulatedBackend())
    else:
        if not torch.cuda.is_available():
            pytest.skip("no GPU here")
        ops.set_backend(None)
    yield
    ops.set_backend(old)


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    return {name: pc.write_model(str(tmp_path_factory.mktemp(f"pukarax_{name}")), cfg, seed)
            for name, (cfg, seed) in pc.CASES.items()}


def _dt(name):
    return {"float32": torch.float32, "bfloat16": torch.bfloat16}[name]


def _tol(dtype, plain_values, fine=2e-5, coarse=4e-2):
    """Largest allowed difference, as a share of the spread of the plain values."""
    return (fine if dtype == "float32" else coarse) * float(plain_values.float().std())


# ------------------------------------------------------------------ mechanisms alone
@pytest.mark.parametrize("where", WHERE)
@pytest.mark.parametrize("width", [5, 70, 1024, 1100, 4104])
def test_the_kernel_between_two_sublayers(where, kernels, width):
    """A read through a norm, a normed result added and the new stream read through the next norm, and a last addition
    alone, each against the plain norms; the stream stays float32 whatever the rows' type."""
    device, dtype = where
    g = torch.Generator().manual_seed(width)
    T, eps_a, eps_b, dt = 5, 1e-4, 1e-2, _dt(dtype)
    x = (torch.randn(T, width, generator=g) * 3)
    wa, wb = (torch.rand(width, generator=g) + 0.5 for _ in range(2))
    y = (torch.randn(T, width, generator=g) * 0.1).to(dt)           # (small: the eps under the root matters)
    stream = x.clone().to(device)
    h = ops.sandwich_step(stream, read=(wa.to(device), eps_a), rows_dtype=dt)
    want = plain.rms_norm(x, wa, eps_a)
    assert h.dtype == dt and torch.equal(stream.cpu(), x) and max_abs_diff(h.cpu(), want) <= _tol(dtype, want)
    h = ops.sandwich_step(stream, add=(y.to(device), wb.to(device), eps_b), read=(wa.to(device), eps_a), rows_dtype=dt)
    x1 = x + plain.rms_norm(y.float(), wb, eps_b)
    want = plain.rms_norm(x1, wa, eps_a)
    assert stream.dtype == torch.float32 and max_abs_diff(stream.cpu(), x1) <= 2e-6 * float(x1.abs().max())
    assert max_abs_diff(h.cpu(), want) <= _tol(dtype, want)
    assert ops.sandwich_step(stream, add=(y.to(device), wa.to(device), eps_a)) is None
    x2 = x1 + plain.rms_norm(y.float(), wa, eps_a)
    assert max_abs_diff(stream.cpu(), x2) <= 2e-6 * float(x2.abs().max())
    with pytest.raises(ops.KernelError):
        ops.sandwich_step(stream)


def _single_request_batch(T, start, device, page_size, pages):
    pos = torch.arange(start, start + T, dtype=torch.int32)
    slots = torch.tensor([pages[p // page_size] * page_size + p % page_size for p in pos.tolist()], dtype=torch.int32)
    batch = AttentionBatch(num_tokens=T, num_requests=1, token_req=torch.zeros(T, dtype=torch.int32).to(device),
                           positions=pos.to(device), cu_seqlens_q=torch.tensor([0, T], dtype=torch.int32).to(device),
                           context_lens=torch.tensor([start + T], dtype=torch.int32).to(device), max_q_len=T,
                           max_context_len=start + T)
    return batch, slots.to(device), torch.tensor([pages], dtype=torch.int32).to(device)


def _frequencies(rot):
    if not rot or not rot.get("dims"):
        return None
    f = rot["base"] ** (-2.0 * torch.arange(rot["dims"] // 2, dtype=torch.float64) / rot["dims"])
    factor = (rot.get("scaling") or {}).get("factor")
    return (f / factor if factor else f).float()


def _attention_through_kernels(device, dtype, kind, m, eps, rows, portions, page_size, lam=None):
    """``rows`` [T, columns]: the packed projection of one request as the layer's product leaves it (q | k | [v] |
    gates). Split, turned, stored and read back by the kernels in the given portions, on pages handed out in a
    scrambled order over stale contents; what comes back is what goes into the output projection."""
    T = rows.shape[0]
    H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    maps = 2 if kind == "attention" else 1
    n_pages = -(-T // page_size)
    pages = torch.randperm(n_pages + 2, generator=torch.Generator().manual_seed(T)).tolist()[:n_pages]
    dt = _dt(dtype)
    k_cache = torch.full((n_pages + 2, page_size, G, maps * D), float("nan"), dtype=dt).to(device)
    v_cache = torch.full((n_pages + 2, page_size, G, E), float("nan"), dtype=dt).to(device)
    f = _frequencies(m.get("rot"))
    f = None if f is None else f.to(device)
    packed = rows.to(dt).to(device)
    outs, at = [], 0
    for n in portions:
        batch, slots, table = _single_request_batch(n, at, device, page_size, pages)
        part = packed[at:at + n].contiguous()
        if kind == "attention":
            q = ops.rotary_split_write(part, None, f, None, batch.positions, slots, k_cache, v_cache, 2 * H, 2 * G, D, E,
                                       more_columns=H, interleaved=True, maps=2)
            a = ops.paged_attention(q, k_cache, v_cache, batch, table, m["scale"], None, m["mask"]["size"])
            o = ops.differential_combine(a, lam.to(device), eps, 1.0 - m["diff"], gate=(part, part.shape[1] - H))
            o = o.view(n, H * E)
        else:
            q = ops.rotary_split_write(part, None, f, None, batch.positions, slots, k_cache, v_cache, H, G, D, E,
                                       more_columns=H * E, unit_eps=eps, values_from_keys=True)
            o = ops.paged_attention(q, k_cache, v_cache, batch, table, m["scale"], None, m["mask"]["size"]).view(n, H * E)
            ops.gate_rows_(o, (part, part.shape[1] - H * E))
        outs.append(o.float().cpu())
        at += n
    assert at == T
    return torch.cat(outs)


def _plain_heads(kind, m, eps, rows, lam=None):
    """The same from the plain functions in float64: the mixers of ``plain_pukarax`` with the identity as their
    projections (the packed rows are cut into the 'projected' q, k, v and gates by hand)."""
    T = rows.shape[0]
    H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    x = rows.double()
    pos = torch.arange(T)
    rot = m.get("rot") or {}
    mask = plain.chunk_mask(T, m["mask"]["size"])
    if kind == "attention":
        q = x[:, :2 * H * D].view(T, H, 2, D)
        k = x[:, 2 * H * D:2 * (H + G) * D].view(T, G, 2, D)
        v = x[:, 2 * (H + G) * D:2 * (H + G) * D + G * E].view(T, G, E)
        a = [plain.softmax_read(plain.turn_interleaved(q[:, :, c], rot.get("dims", 0), rot.get("base", 1.0), pos),
                                plain.turn_interleaved(k[:, :, c], rot.get("dims", 0), rot.get("base", 1.0), pos),
                                v, m["scale"], mask) for c in range(2)]
        o = plain.rms_unit(a[0] - float(lam) * a[1], eps) * (1.0 - m["diff"])
        return (o * torch.sigmoid(x[:, -H:])[:, :, None]).reshape(T, H * E).float()
    factor = (rot.get("scaling") or {}).get("factor")
    q = x[:, :H * D].view(T, H, D)
    k = x[:, H * D:(H + G) * D].view(T, G, D)
    qn = plain.rms_unit(plain.turn_halves(q, rot.get("dims", 0), rot.get("base", 1.0), factor, pos), eps)
    kn = plain.rms_unit(plain.turn_halves(k, rot.get("dims", 0), rot.get("base", 1.0), factor, pos), eps)
    o = plain.softmax_read(qn, kn, k, m["scale"], mask).reshape(T, H * D)
    return (o * torch.sigmoid(x[:, -H * D:])).float()


def _columns(kind, m):
    H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    return 2 * (H + G) * D + G * E + H if kind == "attention" else (H + G) * D + H * E


@pytest.mark.parametrize("where", WHERE)
@pytest.mark.parametrize("sizes", [(12, 20, 3, 8), (32, 64, 2, 32), (16, 32, 6, 4), (64, 128, 1, 64), (8, 4, 1, 0), (16, 16, 2, 16)],
                         ids=lambda s: "D%d-E%d-group%d-rot%d" % s)
@pytest.mark.parametrize("chunk", [7, 40, 1000])
def test_two_maps_per_head_alone(where, kernels, sizes, chunk):
    """Random queries, keys, values and gates of a layer with two maps per head under a chunk mask: value heads of
    any size, among them twice the size of a map in steps of 16 (then a stored key, two maps side by side, has the
    values' size, which the kernels on the matrix cores take in bfloat16); partial, whole and no rotation of adjacent pairs; portions that end inside pages and inside chunks. The
    two maps differ (a kernel that reads one map's keys for both returns nearly nothing after the subtraction)."""
    device, dtype = where
    D, E, group, rot = sizes
    m = pc.two_maps(2 * group, 2, D, E, chunk, rot, 300.0, 1.5 * D ** -0.5, 0.4)["mixer"]
    g = torch.Generator().manual_seed(5)
    T, eps = 90, 1e-5
    rows = torch.randn(T, _columns("attention", m), generator=g)
    if dtype == "bfloat16":
        rows = rows.bfloat16().float()
    lam = torch.tensor([0.37])
    want = _plain_heads("attention", m, eps, rows, lam)
    for portions in ([T], [1] * T, [2, 5, 3, 11, 1, 2, 21, 45]):
        got = _attention_through_kernels(device, dtype, "attention", m, eps, rows, portions, 4, lam)
        # (the difference of two rounded maps is divided by its own size: twice the rounding of one map in bfloat16)
        assert max_abs_diff(got, want) <= _tol(dtype, want, coarse=8e-2), (portions, first_difference(got, want, _tol(dtype, want, coarse=8e-2)))


@pytest.mark.parametrize("where", WHERE)
@pytest.mark.parametrize("sizes", [(12, 3, 8, 4.0), (32, 2, 32, None), (16, 6, 4, 8.0), (64, 1, 64, 2.0), (6, 1, 0, None)],
                         ids=lambda s: "D%d-group%d-rot%d-factor%s" % s)
@pytest.mark.parametrize("chunk", [7, 40, 1000])
def test_keys_as_values_alone(where, kernels, sizes, chunk):
    """A layer whose values are its keys as projected, with queries and keys turned (halves paired, scaled
    frequencies) and then made unit vectors, and a gate per entry. The keys are drawn far from unit length, so a kernel
    that stores the normed keys as values, or norms before it turns with an eps that matters, shows."""
    device, dtype = where
    D, group, rot, factor = sizes
    m = pc.keys_as_values(2 * group, 2, D, chunk, rot, 300.0, factor, 8.0 / D)["mixer"]      # (unit vectors: scores up to 8)
    g = torch.Generator().manual_seed(6)
    T, eps = 90, 1e-2
    rows = torch.randn(T, _columns("attention_2", m), generator=g)
    rows[:, 2 * group * D:2 * (group + 1) * D] *= 0.05 + 3.0 * torch.rand(T, 1, generator=g)       # keys of many lengths
    if dtype == "bfloat16":
        rows = rows.bfloat16().float()
    want = _plain_heads("attention_2", m, eps, rows)
    for portions in ([T], [1] * T, [2, 5, 3, 11, 1, 2, 21, 45]):
        got = _attention_through_kernels(device, dtype, "attention_2", m, eps, rows, portions, 4)
        # (bfloat16: values, weights and the result are each rounded to eight bits: parts in 2^7 of every entry)
        bound = _tol(dtype, want) + (2.0 ** -7 * want.abs() if dtype == "bfloat16" else 0.0)
        assert bool(((got - want).abs() <= bound).all()), (portions, first_difference(got, want, _tol(dtype, want)))


@pytest.mark.parametrize("where", WHERE)
@pytest.mark.parametrize("kind", ["attention", "attention_2"])
def test_one_key_that_stands_out_under_a_chunk(where, kernels, kind):
    """Among 300 keys one is made to carry nearly all the weight of every query that sees it (for two maps per head: in
    the first map only; the second map stays nearly uniform); its value is a vector no other key has. A query then
    returns that value exactly when the key lies in its own block of ``chunk`` positions and not after it: for the
    marked key at a block's first and last place, at a page's border and far back, for queries just inside and just
    outside, in a prompt and decoded one by one. No rotation, so the scores are known."""
    device, dtype = where
    chunk, page, T, D = 48, 16, 300, 16
    for marked in (0, 15, 16, 47, 48, 95, 96, 100, 191, 240, 251):
        g = torch.Generator().manual_seed(marked)
        if kind == "attention":
            m = pc.two_maps(1, 1, D, D, chunk, 0, 1.0, 1.0, 0.5)["mixer"]
            rows = 0.1 * torch.randn(T, _columns(kind, m), generator=g)
            rows[:, 0] = 4.0                       # map 1 of every query asks for coordinate 0 ...
            rows[:, 2 * D] = -2.0                  # ... which map 1 of every key answers with -8,
            rows[marked, 2 * D] = 8.0              # but for the marked key: 32
            v0 = 4 * D
            rows[:, v0:v0 + D] = 1.0 + 0.1 * torch.randn(T, D, generator=g)
            rows[marked, v0:v0 + D] = torch.tensor([9.0, -9.0] * (D // 2))
            rows[:, -1] = 20.0                     # the gate is open
            lam = torch.tensor([0.5])
        else:
            m = pc.keys_as_values(1, 1, D, chunk, 0, 1.0, None, 30.0)["mixer"]
            rows = 0.02 * torch.randn(T, _columns(kind, m), generator=g)
            rows[:, 0] = 4.0                       # every query points along coordinate 0; as unit vectors: (4, 0, ...)
            rows[:, D + 1] = 1.0                   # every key points along coordinate 1: a score near 0,
            rows[marked, D:2 * D] = 0.02 * torch.randn(D, generator=g)
            rows[marked, D] = 7.0                  # but for the marked key, along coordinate 0: 30 * 4 * 4 = 480 as unit vectors,
            rows[:, 2 * D:] = 20.0                 # and its value is itself: 7 at coordinate 0 where all others have 0
            lam = None
        for portions in ([T], [marked + 1] + [1] * (T - marked - 1) if marked < 200 else [T - 60] + [1] * 60):
            got = _attention_through_kernels(device, dtype, kind, m, 1e-6, rows, portions, page, lam)
            sees = torch.tensor([i >= marked and i // chunk == marked // chunk for i in range(T)])
            if kind == "attention":
                # a1 is the marked value, a2 nearly the mean (1): o = (9 - 0.5, -9 - 0.5, ...) made a unit vector, times 0.5
                hit = (got[:, 0] > 0.35) & (got[:, 1] < -0.35)
            else:
                hit = got[:, 0] > 6.0
            assert torch.equal(hit, sees), (marked, len(portions), (hit != sees).nonzero().flatten().tolist())


@pytest.mark.parametrize("where", WHERE)
def test_small_kernels_after_the_heads(where, kernels):
    device, dtype = where
    g = torch.Generator().manual_seed(2)
    dt = _dt(dtype)
    T, H, E = 7, 3, 10
    a = torch.randn(T, 2 * H, E, generator=g).to(dt)
    gates = torch.randn(T, 4 + H, generator=g).to(dt)
    lam, eps, post = torch.tensor([-0.8]), 1e-3, 0.7
    got = ops.differential_combine(a.to(device), lam.to(device), eps, post, gate=(gates.to(device), 4))
    both = a.float().view(T, H, 2, E)
    o = plain.rms_unit(both[:, :, 0] + 0.8 * both[:, :, 1], eps) * post * torch.sigmoid(gates.float()[:, 4:])[:, :, None]
    assert got.shape == (T, H, E) and max_abs_diff(got.cpu(), o) <= _tol(dtype, o, coarse=1e-2)
    got = ops.differential_combine(a.to(device), lam.to(device), eps, post)
    assert max_abs_diff(got.cpu(), plain.rms_unit(both[:, :, 0] + 0.8 * both[:, :, 1], eps) * post) <= _tol(dtype, o, coarse=1e-2)
    x = torch.randn(T, 12, generator=g).to(dt)
    rows = torch.randn(T, 20, generator=g).to(dt)
    got = ops.gate_rows_(x.clone().to(device), (rows.to(device), 8))
    want = x.float() * torch.sigmoid(rows.float()[:, 8:])
    assert max_abs_diff(got.cpu(), want) <= _tol(dtype, want, coarse=1e-2)
    with pytest.raises(ops.KernelError):
        ops.gate_rows_(x.clone().to(device), (rows.to(device), 9))
    # a product with a bias, of few rows and of many
    w, b = (torch.randn(24, 16, generator=g) / 4).to(dt), torch.randn(24, generator=g).to(dt)
    for n in (1, 9, 40, 300):
        xm = torch.randn(n, 16, generator=g).to(dt)
        got = ops.linear(xm.to(device), w.to(device), b.to(device))
        want = xm.float() @ w.float().T + b.float()
        assert max_abs_diff(got.cpu(), want) <= _tol(dtype, want, coarse=2e-2), n


@pytest.mark.parametrize("where", WHERE)
@pytest.mark.parametrize("sizes", [(5, 2, 12, 40, 16), (1, 1, 10, 36, 0), (4, 4, 6, 36, 0), (12, 4, 64, 192, 128), (9, 3, 8, 64, 24), (40, 1, 16, 72, 8)],
                         ids=lambda s: "experts%d-top%d-ff%d-width%d-shared%d" % s)
def test_experts_weighed_by_the_softmax_over_the_chosen(where, kernels, sizes, tmp_path):
    """The routed feed-forward as a part, few rows and many (in bfloat16 on the GPU the two take different kernels),
    against the plain mixture: router logits with a bias that changes who is chosen, weights that sum to one over the
    chosen alone and weigh the outputs, a shared expert added; one expert, all experts chosen, widths that are no
    multiple of 8. A row alone gives what it gives in a batch."""
    from nanohybrid_vlm_amd.parts.base import FEED_FORWARDS
    device, dtype = where
    E, top, F, W, shared = sizes
    dt = _dt(dtype)
    cfg = pc.model(10, W, 1e-5, 1.0, 1.0, [dict(pc.keys_as_values(1, 1, 4, 4, 0, 1.0, None, 1.0), mlp=pc.moe(E, top, F, shared or None))])
    w = {k[len("l0.mlp."):]: v for k, v in pc.random_tensors(cfg, 3).items() if k.startswith("l0.mlp.")}
    w["router.b"] = (3.0 * torch.randn(E, generator=torch.Generator().manual_seed(1))).bfloat16()   # the bias decides some choices
    part = FEED_FORWARDS.build({"kind": "routed_experts", "hidden_size": W, "num_experts": E, "top": top, "expert_size": F,
                                "scoring": "softmax_of_chosen", "scores_on": "output", "router_bias": True,
                                "shared": {"kind": "swiglu", "hidden_size": W, "intermediate_size": shared} if shared else None})
    params = {"router.weight": w["router"].to(dt), "router.bias": w["router.b"].float(),
              "gate_up.weight": torch.cat([torch.cat((w[f"e{e}.gate"], w[f"e{e}.up"])) for e in range(E)]).to(dt),
              "down.weight": torch.cat([w[f"e{e}.down"] for e in range(E)]).to(dt)}
    if shared:
        params["shared.gate_up.weight"] = torch.cat((w["shared.gate"], w["shared.up"])).to(dt)
        params["shared.down.weight"] = w["shared.down"].to(dt)
    assert set(params) == set(part.all_param_specs())
    part.bind_all({k: v.to(device) for k, v in params.items()})
    g = torch.Generator().manual_seed(4)
    for n in (1, 3, 16, 17, 70):
        h = torch.randn(n, W, generator=g).to(dt)
        want = plain.mixture(h.double(), {k: v.double() for k, v in w.items()}, cfg["layers"][0]["mlp"]).float()
        got = part.forward(h.to(device), None).float().cpu()
        if dtype == "float32":
            assert max_abs_diff(got, want) <= _tol(dtype, want), (n, first_difference(got, want, _tol(dtype, want)))
            alone = part.forward(h[-1:].contiguous().to(device), None).float().cpu()
            assert max_abs_diff(alone, got[-1:]) <= 1e-6 * float(want.abs().max())
        else:
            # a close call of the router may turn the other way on rounded sums: all rows but a few agree
            bad = ((got - want).abs().max(dim=-1).values > _tol(dtype, want, coarse=6e-2)).sum()
            assert int(bad) <= max(1, n // 10), (n, int(bad))
    # the sigmoid scores on the experts' inputs are what they were
    ids, scores = ops.route_topk(torch.tensor([[0.5, 2.0, -1.0, 2.0]]).to(device), 2)
    assert ids.tolist() == [[1, 3]] and max_abs_diff(scores.cpu(), torch.sigmoid(torch.tensor([[2.0, 2.0]]))) < 1e-6
    ids, scores = ops.route_topk(torch.tensor([[0.5, 2.0, -1.0, 2.0]]).to(device), 3, bias=torch.tensor([2.0, 0.0, 0.0, -3.0]).to(device),
                                 scoring="softmax_of_chosen")
    assert ids.tolist() == [[0, 1, 2]] and max_abs_diff(scores.cpu(), torch.softmax(torch.tensor([[2.5, 2.0, -1.0]]), -1)) < 1e-6


# ------------------------------------------------------------------ configuration and weights
def test_configuration_and_checkpoint_names():
    from nanohybrid_vlm_amd.parts.base import PagedKVNeed
    from nanohybrid_vlm_amd.parts.model import DecoderModel
    arch = resolve_architecture(pc.CONFIG_A)
    assert arch.name == "Pukarax"
    cfg = arch.parse_config(pc.CONFIG_A)
    assert cfg.order() == [0, 1, 2, 1, 2, 1, 2, 3] and cfg.layers[2].mlp is None and cfg.layers[3].mlp.shared_ff is None
    spec = arch.build_spec(cfg)
    assert [e.layer for e in spec.order()] == cfg.order() and all(e.cache is None for e in spec.order())
    model = DecoderModel(spec)
    names = arch.checkpoint_names(cfg)
    assert set(names) == set(pc.random_tensors(pc.CONFIG_A, 0))
    assert {s.param for s in names.values()} == set(model.all_param_specs())
    # every run of a layer has pages of its own, also where runs share their weights; two maps per head keep two keys
    # per key/value head
    needs = model.cache_needs()
    assert len(needs) == 8 and all(isinstance(n, PagedKVNeed) for n in needs)
    assert needs[1] == needs[3] and needs[1].num_kv_heads == 1 and needs[1].head_dim == 12 and needs[1].value_size == 10 and needs[1].chunk == 5
    assert needs[0].num_kv_heads == 2 and needs[0].value_size == 8 and needs[0].chunk == 6
    assert arch.parse_config(pc.CONFIG_B).order() == [0, 1, 2, 3]
    for change, match in ((lambda c: c["layers"][1].update(type="other"), "not known"),
                          (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=3), "rot.dims"),
                          (lambda c: c["layers"][0]["mixer"].update(kv_heads=3), "multiple"),
                          (lambda c: c["layers"][0]["mixer"].update(vdim=5), "values are the keys"),
                          (lambda c: c["layers"][1]["mixer"].pop("diff"), "diff"),
                          (lambda c: c["layers"][1]["mlp"]["router"].update(top=6), "experts"),
                          (lambda c: c["layers"][0]["mlp"].update(kind="other"), "not known"),
                          (lambda c: c["loop"].update(stop=5), "loop"),
                          (lambda c: c["loop"].update(times=0), "loop")):
        bad = json.loads(json.dumps(pc.CONFIG_A))
        change(bad)
        with pytest.raises(ConfigError, match=match):
            arch.parse_config(bad)


# ------------------------------------------------------------------ whole models through the step function
def _requests(name, lengths):
    vocab = pc.CASES[name][0]["vocab"]
    return {f"r{i}": pc.tokens(vocab, n, 100 * i + n) for i, n in enumerate(lengths)}


class _Logits(dict):
    """The plain model's logits by request, and by how much each position moves when the plain model itself is
    evaluated in float32 (``moved``): the difference of two maps is divided by its own root mean square, and norms
    follow sublayers' results of any size, so single positions of a model with random weights are ill-conditioned."""
    moved: dict


def _plain_logits(folder, requests, dtype=torch.float64):
    """(in float64: what the comparison then shows is the engine's own rounding, not the oracle's)"""
    cfg, w = plain.read_folder(folder)
    out = _Logits({rid: plain.forward(cfg, w, toks, dtype).float() for rid, toks in requests.items()})
    out.moved = {}
    if dtype == torch.float64:
        out.moved = {rid: (plain.forward(cfg, w, toks, torch.float32) - out[rid]).abs().max(dim=-1).values
                     for rid, toks in requests.items()}
    return out


def _replay(folder, where, steps, page_size, max_live, **options):
    device, dtype = where
    pages = max(1, pc.peak_tokens(steps, page_size) // page_size)
    runner = ModelRunner(folder, dtype=dtype, device=device, page_size=page_size, num_pages=pages, num_state_slots=max_live,
                         max_model_len=pages * page_size, poison_freed_pages=True, **options)
    got = replay(runner, steps)
    assert not runner.cache.requests and all(runner.cache.num_free_pages(g) == pages for g in range(len(runner.cache.groups)))
    return got


def _compare(got, want, dtype, what):
    """float32: every logit within 1e-4 of the logits' spread, plus ten times what the position moves when the plain
    model itself is evaluated in float32 (see ``_Logits``). bfloat16: a router's close call may turn the other way on
    rounded rows, and a difference of two maps that nearly cancels is divided by its own size: either moves single
    tokens' logits by much, so one position in ten may be beyond the tolerance of a tenth of the logits' spread, none
    beyond twice the spread (the float32 run of the same steps is the sharp one, and the tests of the mechanisms alone
    hold the bfloat16 kernels to close bounds)."""
    tol = tolerance_for(dtype, want)
    if dtype == "float32":
        for rid in want:
            errors = (got[rid].float() - want[rid].float()).abs().max(dim=-1).values
            allowed = tol + 10.0 * getattr(want, "moved", {}).get(rid, torch.zeros_like(errors))
            assert bool((errors <= allowed).all()), (what, rid, (errors > allowed).nonzero().flatten().tolist()[:4], float(errors.max()))
        return
    errors = torch.cat([(got[rid].float() - want[rid].float()).pow(2).mean(dim=-1).sqrt() for rid in want])    # (over the vocabulary)
    assert bool(torch.isfinite(errors).all()), what
    assert float((errors > tol).float().mean()) <= 0.1 and float(errors.max()) <= 20 * tol, \
        (what, float((errors > tol).float().mean()), float(errors.max()) / tol)


@pytest.mark.parametrize("where", WHERE)
def test_layers_one_by_one(folders, where, kernels):
    """Models cut off after 1, 2, ... layers (with the loop over what is left of its layers) give the plain model's
    logits: the stream after every layer is right."""
    cfg, w = plain.read_folder(folders["A"])
    toks = pc.tokens(cfg["vocab"], 21, 9)
    for n in range(1, len(cfg["layers"]) + 1):
        cut = dict(cfg, layers=cfg["layers"][:n])
        loop = cfg["loop"]
        cut["loop"] = dict(loop, start=min(loop["start"], n), stop=min(loop["stop"], n))
        keep = tuple(f"l{i}." for i in range(n))
        tensors = {k: v for k, v in w.items() if not k.startswith("l") or k.startswith(keep)}
        folder = pc.write_model(os.path.join(folders["A"], f"cut{n}"), cut, 0, tensors)
        want = _plain_logits(folder, {"a": toks})
        got = _replay(folder, where, pc.in_portions({"a": toks}, [8, 1, 5, 7]), page_size=4, max_live=1)
        _compare(got, want, where[1], f"{n} layers")


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
        "whole": (pc.whole(requests), 3),
        "tail": ([s for rid, toks in requests.items()
                  for s in pc.in_portions({rid: toks}, [max(1, len(toks) - 12)] + [1] * 12)], 3),
        "portions": (pc.in_portions(requests, [2, 3, 5, 2, 1, 7, 4, 2, 11]), 3),
        "side by side": (pc.interleaved(requests, [3, 1, 2, 6, 1, 1, 4], 3), 3),
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
    """Models of sizes drawn at random (see ``pukarax_cases.random_config``) in portions, side by side and with a decoded
    tail, on pages of 16 tokens that are used again, against the plain model; float32 bit-equal across the ways on the GPU."""
    device, dtype = where
    cfg = pc.random_config(seed)
    folder = pc.write_model(str(tmp_path / "m"), cfg, 500 + seed)
    lengths = [1, 21, 40, 7] if device == "cpu" else [1, 70, 210, 33, 131]
    requests = {f"r{i}": pc.tokens(cfg["vocab"], n, 7 * i + n) for i, n in enumerate(lengths)}
    want = _plain_logits(folder, requests)
    ways = {"portions": pc.in_portions(requests, [17, 2, 3, 64, 1, 33]),
            "side by side": pc.interleaved(requests, [5, 1, 2, 31, 1, 1, 16], 3),
            "tail": [s for rid, toks in requests.items() for s in pc.in_portions({rid: toks}, [max(1, len(toks) - 20)] + [1] * 20)]}
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
def test_pages_of_64_and_chunks_longer_than_a_page(folders, where, kernels):
    """Pages of 64 tokens (whole tiles of the prompt kernel lie in one page) under chunks of 80, 128 and 150 positions,
    requests of up to 400 tokens in portions that end anywhere, beside decoded tokens, on few pages."""
    device, dtype = where
    requests = _requests("S", [400, 130, 70, 257])
    want = _plain_logits(folders["S"], requests)
    for what, steps in (("portions", pc.in_portions(requests, [37, 2, 64, 5, 1, 129, 1, 1, 96])),
                        ("side by side", pc.interleaved(requests, [33, 1, 1, 64, 1, 7, 1, 100], 3))):
        got = _replay(folders["S"], where, steps, page_size=64, max_live=3)
        _compare(got, want, dtype, what)


@pytest.mark.parametrize("where", ON_GPU)
def test_sizes_of_a_real_models_layers(where, kernels, tmp_path):
    """Heads of 128 and 64 entries, a width of 1,024, experts of 256: the kernels' makes that real sizes take, in
    portions and side by side on pages of 64, with decoded tokens between."""
    device, dtype = where
    folder = pc.write_model(str(tmp_path / "w"), pc.CONFIG_W, 26)
    requests = {f"r{i}": pc.tokens(pc.CONFIG_W["vocab"], n, 11 * i + n) for i, n in enumerate([300, 40, 129])}
    want = _plain_logits(folder, requests, torch.float32)
    for what, steps in (("portions", pc.in_portions(requests, [150, 1, 1, 16, 3, 64, 1, 1, 1])),
                        ("side by side", pc.interleaved(requests, [40, 1, 1, 1, 17, 1, 64, 1], 3))):
        got = _replay(folder, where, steps, page_size=64, max_live=3)
        _compare(got, want, dtype, what)


@pytest.mark.parametrize("where", WHERE)
def test_long_decoding(folders, where, kernels):
    """Two tokens of prompt, then many tokens one by one: the chunks of every layer pass many times and pages go back
    to the pool on the way."""
    device, dtype = where
    n = 60 if device == "cpu" else 142
    requests = _requests("A", [n])
    want = _plain_logits(folders["A"], requests)
    steps = pc.in_portions(requests, [2] + [1] * n)
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
        steps = pc.interleaved(requests, [3, 1, 1, 1, 2, 1, 1], 3)
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
    cfg, w = plain.read_folder(folders["A"])
    prompts = [pc.tokens(cfg["vocab"], n, 300 + n) for n in (1, 13, 22)]
    llm = LLM(folders["A"], device=device, dtype=dtype, **options)
    outs = llm.generate(prompts, SamplingParams(temperature=0.0, max_tokens=9, ignore_eos=True), use_tqdm=False)
    for prompt, out in zip(prompts, outs):
        assert out["token_ids"] == plain.greedy_generate(cfg, w, prompt, 9)
    stats = llm.get_memory_stats()
    assert stats["live_requests"] == 0 and all(g["free_pages"] == g["pages"] for g in stats["groups"])


# ------------------------------------------------------------------ the command line
def _command(*args):
    import subprocess
    import sys
    repo = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    proc = subprocess.run([sys.executable, "-m", "nanohybrid_vlm_amd", *args], cwd=repo, capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-3000:]
    return proc.stdout


def test_random_model_of_a_named_shape(tmp_path, emulated_kernels):
    """``random-model --shape pukarax-tiny`` writes a folder that the plain implementation and the engine both read."""
    out = str(tmp_path / "m")
    _command("random-model", "--out", out, "--shape", "pukarax-tiny", "--seed", "5")
    cfg, w = plain.read_folder(out)
    assert cfg["architecture"] == "Pukarax" and w["l1.mix.lq1"].shape == (cfg["layers"][1]["mixer"]["dim"],)
    requests = {"a": pc.tokens(cfg["vocab"], 31, 1)}
    want = _plain_logits(out, requests)
    got = _replay(out, CPU, pc.in_portions(requests, [4, 1, 9]), page_size=8, max_live=1)
    _compare(got, want, "float32", "portions")


@pytest.mark.gpu
def test_generate_command_with_random_weights():
    if not torch.cuda.is_available():
        pytest.skip("no GPU here")
    out = json.loads(_command("generate", "--random-weights", "4", "--shape", "pukarax-tiny", "--prompt-ids", "5 17 3",
                              "--prompt-ids", "9 8 7 6 5 4 3 2 1", "--output-tokens", "6", "--temperature", "0", "--ignore-eos",
                              "--block-size", "8", "--num-blocks", "32", "--max-model-len", "64", "--quiet"))
    assert [len(o["token_ids"]) for o in out] == [6, 6]


# ------------------------------------------------------------------ the replay program
@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_replay_program_on_a_model_of_this_design(folders, dtype, tmp_path):
    """``bin/trace_run`` as a user starts it: steps on standard input, ``<step>.f32`` files, pages of 64 and four
    slots that several traces in one run use again, steps of single tokens and short mixed steps from graphs."""
    if not torch.cuda.is_available():
        pytest.skip("no GPU here")
    from test_replay import _logits_from_files, _renamed, _trace_run
    requests = _requests("S", [150, 9, 71, 2, 40])
    want = _plain_logits(folders["S"], requests)
    ways = {"portions": pc.in_portions(requests, [37, 2, 64, 5, 1, 1]),
            "side by side": pc.interleaved(requests, [33, 1, 1, 16, 1, 7, 1], 4)}
    steps, first = [], 0
    for k, (what, t) in enumerate(ways.items()):
        steps += _renamed(t, f"#{k}", first)
        first += len(t)
    out_dir = str(tmp_path / "out")
    _trace_run(folders["S"], dtype, steps, out_dir, max(pc.peak_tokens(t, 64) for t in ways.values()))
    got = _logits_from_files(out_dir, steps, pc.CONFIG_S["vocab"])
    for k, what in enumerate(ways):
        _compare({rid: got[f"{rid}#{k}"] for rid in want}, want, dtype, what)
