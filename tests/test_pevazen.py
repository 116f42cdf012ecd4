"""The Pevazen design in the engine against its plain whole-sequence implementation (``plain_pevazen.py``):
every mechanism alone through the kernels' entry points, then whole models through the step function (whole
prompts, decoding token by token, portions down to two tokens, unequal requests side by side on few pages and
slots that are used again), and greedy generation through the entry point and its scheduler. Every test runs on
the CPU stand-in for the kernels (the engine's logic) and, marked ``gpu``, on the HIP kernels in both element types.
"""
import json

import pytest
import torch

import pevazen_cases as pc
import plain_pevazen as plain
from helpers import first_difference, max_abs_diff, tolerance_for
from nanohybrid_vlm_amd.cache.manager import CacheManager, PagedGroupSpec
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
    return {name: pc.write_model(str(tmp_path_factory.mktemp(f"pevazen_{name}")), cfg, ranks, seed)
            for name, (cfg, ranks, seed) in pc.CASES.items()}


def _dt(name):
    return {"float32": torch.float32, "bfloat16": torch.bfloat16}[name]


def _tol(dtype, plain_values, fine=2e-5, coarse=4e-2):
    """Largest allowed difference, as a share of the spread of the plain values."""
    return (fine if dtype == "float32" else coarse) * float(plain_values.float().std())


# ------------------------------------------------------------------ one request's batch, by hand
def _single_request_batch(T, start, device, page_size, pages):
    """A batch of one request that brings T tokens from position ``start`` on; its pages are ``pages``."""
    pos = torch.arange(start, start + T, dtype=torch.int32)
    slots = torch.tensor([pages[p // page_size] * page_size + p % page_size for p in pos.tolist()], dtype=torch.int32)
    batch = AttentionBatch(num_tokens=T, num_requests=1, token_req=torch.zeros(T, dtype=torch.int32).to(device),
                           positions=pos.to(device), cu_seqlens_q=torch.tensor([0, T], dtype=torch.int32).to(device),
                           context_lens=torch.tensor([start + T], dtype=torch.int32).to(device), max_q_len=T,
                           max_context_len=start + T)
    return batch, slots.to(device), torch.tensor([pages], dtype=torch.int32).to(device)


# ------------------------------------------------------------------ mechanisms alone
@pytest.mark.parametrize("where", WHERE)
def test_norms_and_depth_sum(where, kernels):
    device, dtype = where
    g = torch.Generator().manual_seed(1)
    T, W, eps = 7, 50, 1e-3
    x = torch.randn(T, W, generator=g) * 3
    gain = torch.tensor(0.7)
    for out in (torch.float32, _dt(dtype)):
        got = ops.scalar_rmsnorm(x.to(device), gain.to(device), eps, out_dtype=out)
        want = plain.scalar_norm(x, gain, eps)
        assert got.dtype == out and max_abs_diff(got.cpu(), want) <= _tol("float32" if out == torch.float32 else dtype, want)
    a, b = (torch.randn(T, W, generator=g).to(_dt(dtype)) for _ in range(2))
    wa, wb = torch.rand(W, generator=g) + 0.5, torch.rand(W, generator=g) + 0.5
    got = ops.pair_norm_mean(a.to(device), wa.to(device), b.to(device), wb.to(device), eps)
    want = 0.5 * (plain.vector_norm(a.float(), wa, eps) + plain.vector_norm(b.float(), wb, eps))
    assert max_abs_diff(got.cpu(), want) <= _tol(dtype, want)
    # three layers' sums over depth; the second has no feed-forward
    depth = 3
    results = torch.zeros(depth + 1, T, W).to(device)
    stream, outputs = x.clone(), [x.clone()]
    for i in range(depth):
        m, f = (torch.randn(T, W, generator=g).to(_dt(dtype)) for _ in range(2))
        f = None if i == 1 else f
        w = torch.randn(i + 2, generator=g)
        got = ops.depth_mix(stream.to(device), m.to(device), None if f is None else f.to(device), results, i, w.to(device))
        outputs.append(stream + (m.float() if f is None else m.float() + f.float()))
        stream = sum(w[j] * outputs[j] for j in range(i + 2))
        assert max_abs_diff(got.cpu(), stream) <= 1e-5 * float(stream.abs().max())
        stream = got.cpu()
    with pytest.raises(ops.KernelError):
        ops.depth_mix(x.to(device), a.to(device), None, results, depth, torch.ones(depth + 2).to(device))
    # a pair of rows whose norms and mean are left to the sum over depth, with the next norm taken in the same kernel
    pair = ops.NormedPairMean(a.to(device), wa.to(device), b.to(device), wb.to(device), eps)
    w = torch.tensor([0.3, 0.9])
    got, normed = ops.depth_mix(x.to(device), pair, b.to(device), results, 0, w.to(device), gain=gain.to(device), eps=eps)
    mean = 0.5 * (plain.vector_norm(a.float(), wa, eps) + plain.vector_norm(b.float(), wb, eps))
    want = w[0] * x + w[1] * (x + (mean + b.float()))
    assert max_abs_diff(got.cpu(), want) <= 1e-5 * float(want.abs().max())
    assert max_abs_diff(normed.float().cpu(), plain.scalar_norm(want, gain, eps)) <= _tol(dtype, want)
    assert max_abs_diff(pair.tensor().float().cpu(), mean) <= _tol(dtype, mean)


def _attention_through_kernels(device, dtype, m, q_in, k_in, v_in, portions, page_size, rotate_values, bias=None):
    """q_in [T, H D], k_in [T, G D], v_in [T, G E] as projected: split, turned, stored and read back by the kernels
    in the given portions of one request, on pages handed out in a scrambled order."""
    T = q_in.shape[0]
    H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    n_pages = -(-T // page_size)
    pages = torch.randperm(n_pages + 2, generator=torch.Generator().manual_seed(T)).tolist()[:n_pages]
    dt = _dt(dtype)
    k_cache = torch.full((n_pages + 2, page_size, G, D), float("nan"), dtype=dt).to(device)
    v_cache = torch.full((n_pages + 2, page_size, G, E), float("nan"), dtype=dt).to(device)
    f = plain.pair_frequencies(m["rot"]["dims"], m["rot"]["base"], torch.float32)
    if m["rot"].get("scaling"):
        f = f / m["rot"]["scaling"]["factor"]
    vf = plain.pair_frequencies(E, m["rot"]["base"], torch.float32).to(device) if rotate_values else None
    packed = torch.cat((q_in, k_in, v_in), dim=1).to(dt).to(device)
    outs, at = [], 0
    for n in portions:
        batch, slots, table = _single_request_batch(n, at, device, page_size, pages)
        q = ops.rotary_split_write(packed[at:at + n].contiguous(), bias, f.to(device) if len(f) else None, vf, batch.positions,
                                   slots, k_cache, v_cache, H, G, D, E)
        o = ops.paged_attention(q, k_cache, v_cache, batch, table, m["scale"], None, m["mask"]["size"])
        if rotate_values:
            ops.turn_back_(o, vf, batch.positions)
        outs.append(o.float().cpu())
        at += n
    assert at == T
    return torch.cat(outs)


def _plain_attention(m, q_in, k_in, v_in, rotate_values):
    T = q_in.shape[0]
    H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pos = torch.arange(T)
    f = plain.pair_frequencies(m["rot"]["dims"], m["rot"]["base"], torch.float64)
    if m["rot"].get("scaling"):
        f = f / m["rot"]["scaling"]["factor"]
    q = plain.turn_halves(q_in.double().view(T, H, D), pos, f)
    k = plain.turn_halves(k_in.double().view(T, G, D), pos, f)
    v = v_in.double().view(T, G, E)
    if rotate_values:
        v = plain.turn_halves(v, pos, plain.pair_frequencies(E, m["rot"]["base"], torch.float64))
    o = plain.masked_attention(q, k, v, m["scale"], plain.chunk_mask(T, m["mask"]["size"]))
    if rotate_values:
        o = plain.turn_halves(o, pos, plain.pair_frequencies(E, m["rot"]["base"], torch.float64), sign=-1.0)
    return o.float()


@pytest.mark.parametrize("where", WHERE)
@pytest.mark.parametrize("rotate_values", [False, True])
@pytest.mark.parametrize("sizes", [(12, 20), (32, 32)], ids=["D12-E20", "D32-E32"])
def test_chunked_attention_alone(where, kernels, rotate_values, sizes):
    """Random queries, keys and values; a partial rotation with scaled frequencies; value heads of another size than
    the key heads, and of the same size in steps of 16 (which the kernels on the matrix cores take in bfloat16);
    portions that end inside pages and inside chunks."""
    device, dtype = where
    D, E = sizes
    m = pc._attention(6, 2, D, E, 7, 8, 300.0, 0.35, factor=2.5)
    g = torch.Generator().manual_seed(5)
    T = 45
    q_in, k_in, v_in = torch.randn(T, 6 * D, generator=g), torch.randn(T, 2 * D, generator=g), torch.randn(T, 2 * E, generator=g)
    if dtype == "bfloat16":
        q_in, k_in, v_in = (t.bfloat16().float() for t in (q_in, k_in, v_in))
    want = _plain_attention(m, q_in, k_in, v_in, rotate_values)
    for portions in ([T], [1] * T, [2, 5, 3, 11, 1, 2, 21]):
        got = _attention_through_kernels(device, dtype, m, q_in, k_in, v_in, portions, 4, rotate_values)
        assert max_abs_diff(got, want) <= _tol(dtype, want), (portions, first_difference(got.flatten(1), want.flatten(1), _tol(dtype, want)))


@pytest.mark.parametrize("where", WHERE)
@pytest.mark.parametrize("E", [6, 16], ids=["values of their own size", "values of the keys' size"])
def test_one_key_that_stands_out(where, kernels, E):
    """Among 300 keys one is made to carry nearly all the weight of every query that sees it; its value is a
    vector no other key has. A query then returns that value exactly when the key lies in its own chunk at or
    before it: for the marked key at the first and the last place of a chunk, at a page's border, far back, and for
    queries just inside and just outside, in a prompt and decoded one by one. No rotation, so the scores are known.
    (With value heads of the key heads' size the bfloat16 run takes the kernels on the matrix cores.)"""
    device, dtype = where
    chunk, page, T, D = 48, 16, 300, 16
    m = pc._attention(2, 1, D, E, chunk, 0, 10.0, 1.0)
    for marked in (0, 47, 48, 95, 96, 143, 144, 191, 240, 287):
        g = torch.Generator().manual_seed(marked)
        q_in = 0.1 * torch.randn(T, 2 * D, generator=g)
        k_in = 0.1 * torch.randn(T, D, generator=g)
        v_in = 0.1 * torch.randn(T, E, generator=g)
        q_in[:, 0] = q_in[:, D] = 4.0                 # every query asks for coordinate 0 ...
        k_in[marked, 0] = 8.0                         # ... which only the marked key has: its score is 32 above the rest
        v_in[marked] = torch.tensor([5.0, -5.0] * (E // 2))
        for portions in ([T], [marked + 1] + [1] * (T - marked - 1) if marked < 200 else [T - 40] + [1] * 40):
            got = _attention_through_kernels(device, dtype, m, q_in, k_in, v_in, portions, page, False)
            sees = torch.tensor([marked <= i and i // chunk == marked // chunk for i in range(T)])
            hit = (got[:, 0, 0] > 4.5) & (got[:, 1, 1] < -4.5)
            assert torch.equal(hit, sees), (marked, len(portions), (hit != sees).nonzero().flatten().tolist())
            assert got[~sees].abs().max() < 1.0


def _delta_inputs(T, H, G, D, E, n, seed):
    g = torch.Generator().manual_seed(seed)
    C = 2 * G * D + H * E
    return {"proj": torch.randn(T, C + H, generator=g), "a_lin": torch.randn(T, H * D, generator=g),
            "g_lin": torch.randn(T, H * E, generator=g), "taps": 0.6 * torch.randn(C, n, generator=g),
            "dt_bias": torch.randn(H * D, generator=g) - 0.5, "a_log": 0.5 * torch.randn(H, generator=g) - 0.5,
            "norm": 1.0 + 0.2 * torch.randn(E, generator=g)}


def _plain_delta(x, H, G, D, E, eps):
    """The recurrent mixer between its projections, from the plain functions, in float64."""
    x = {k: v.double() for k, v in x.items()}
    T = x["proj"].shape[0]
    C = 2 * G * D + H * E
    act = plain.silu(plain.causal_taps(x["proj"][:, :C], x["taps"]))
    unit = lambda t: t / torch.sqrt(t.pow(2).sum(-1, keepdim=True) + 1e-6)
    rep = H // G
    q = unit(act[:, :G * D].view(T, G, D)).repeat_interleave(rep, dim=1) * D ** -0.5
    k = unit(act[:, G * D:2 * G * D].view(T, G, D)).repeat_interleave(rep, dim=1)
    v = act[:, 2 * G * D:].view(T, H, E)
    beta = torch.sigmoid(x["proj"][:, C:])
    decay = torch.exp(-torch.exp(x["a_log"])[None, :, None] * plain.softplus(x["a_lin"] + x["dt_bias"]).view(T, H, D))
    o = plain.gated_delta_rule(q, k, v, decay, beta)
    return (plain.unit_rms(o, eps) * x["norm"] * torch.sigmoid(x["g_lin"]).view(T, H, E)).reshape(T, H * E).float()


@pytest.mark.parametrize("where", WHERE)
@pytest.mark.parametrize("sizes", [(4, 2, 8, 6, 4), (1, 1, 3, 3, 1), (3, 3, 20, 5, 2), (2, 1, 64, 64, 3), (2, 2, 96, 40, 5)],
                         ids=lambda s: "H%d-G%d-D%d-E%d-taps%d" % s)
def test_gated_delta_rule_alone(where, kernels, sizes):
    """Two requests of unequal length side by side, in portions (the state and the convolutions' last inputs go
    through the slots), against the recurrence written out token by token; then the slots are used again by new
    requests, which must start from zero."""
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

            def rows_of(name):
                return torch.cat([x[r][name][at[r]:at[r] + step[r]] for r in reqs]).to(device)
            y = ops.gated_delta_rule(rows_of("proj"), rows_of("a_lin"), rows_of("g_lin"), shared["taps"], shared["dt_bias"],
                                     shared["a_log"], shared["norm"], eps, kept, state, batch,
                                     torch.tensor([slot_of[r] for r in reqs], dtype=torch.int32).to(device), H, G, D, E,
                                     _dt(dtype))
            y = y.float().cpu()
            for i, r in enumerate(reqs):
                got[r].append(y[int(cu[i]):int(cu[i + 1])])
                at[r] += step[r]
        for r in lengths:
            assert at[r] == lengths[r]
            out = torch.cat(got[r])
            assert max_abs_diff(out, want[r]) <= _tol(dtype, want[r], fine=1e-4, coarse=2e-2), (round_, r, first_difference(out, want[r], 1e-3))


def test_chunked_group_gives_pages_back():
    """Pages of a chunked group go back as soon as the next query's chunk begins after them."""
    cache = CacheManager([PagedGroupSpec("chunk 6", page_size=4, num_pages=8, chunk=6), PagedGroupSpec("all", page_size=4, num_pages=8)], 2)
    cache.admit("r")
    freed = []
    for new_len in range(1, 26):
        cache.reserve("r", new_len)
        freed += cache.commit("r", new_len)[0]
        cache.check()
        table = cache.block_table("r", 0)
        start = new_len - new_len % 6                      # the first key that the query at position new_len reads
        assert all((p == -1) == ((lp + 1) * 4 <= start) for lp, p in enumerate(table)), (new_len, table)
        assert all(p != -1 for p in cache.block_table("r", 1))
    assert len(freed) == 6 and cache.num_free_pages(0) == 8 - 1
    with pytest.raises(ValueError):
        PagedGroupSpec("both", page_size=4, num_pages=2, window=3, chunk=3)


# ------------------------------------------------------------------ configuration and weights
def test_configuration_and_names(folders, tmp_path):
    from nanohybrid_vlm_amd.parts.model import DecoderModel
    from nanohybrid_vlm_amd.weights.loader import checkpoint_shapes
    arch = resolve_architecture(pc.CONFIG_P)
    assert arch.name == "Pevazen"
    cfg = arch.parse_config(pc.CONFIG_P, checkpoint_shapes(folders["P"]))
    assert (cfg.layers[0].delta.decay_rank, cfg.layers[0].delta.gate_rank) == pc.RANKS_P[0]
    assert cfg.layers[3].attention.kv_from == 1 and cfg.layers[1].ff is None
    model = DecoderModel(arch.build_spec(cfg))
    # every stored tensor has its place, and every parameter is filled by stored tensors
    names = arch.checkpoint_names(cfg)
    assert set(names) == set(pc.random_tensors(pc.CONFIG_P, pc.RANKS_P, 0))
    assert {s.param for s in names.values()} == set(model.all_param_specs())
    # layer 3 reads layer 1's pages under a chunk of another size: the pages are then kept for all keys
    needs = model.cache_needs()
    assert needs[3] is None and needs[1].chunk is None and needs[1].value_size == 4 and needs[0].paged.chunk == 6
    with pytest.raises(ConfigError, match="neither"):
        arch.parse_config(pc.CONFIG_P)                     # no stored tensors and no ranks in the configuration
    bad = json.loads(json.dumps(pc.CONFIG_P))
    bad["layers"][3]["mixer"]["kv_from"] = 0               # a pair of mixers lends nothing
    with pytest.raises(ConfigError, match="kv_from"):
        arch.parse_config(bad, checkpoint_shapes(folders["P"]))
    bad = json.loads(json.dumps(pc.CONFIG_P))
    bad["layers"][3]["mixer"]["rot"]["base"] = 7.0         # another rotation than the lender's
    with pytest.raises(ConfigError, match="rotation"):
        arch.parse_config(bad, checkpoint_shapes(folders["P"]))
    bad = json.loads(json.dumps(pc.CONFIG_P))
    bad["layers"][1]["type"] = "other"
    with pytest.raises(ConfigError, match="not known"):
        arch.parse_config(bad, checkpoint_shapes(folders["P"]))


# ------------------------------------------------------------------ whole models through the step function
def _requests(name, lengths):
    vocab = pc.CASES[name][0]["vocab"]
    return {f"r{i}": pc.tokens(vocab, n, 100 * i + n) for i, n in enumerate(lengths)}


def _plain_logits(folder, requests, dtype=torch.float32):
    cfg, w = plain.read_model_folder(folder)
    return {rid: plain.logits(cfg, w, toks, dtype).float() for rid, toks in requests.items()}


def _replay(folder, where, steps, page_size, max_live, **options):
    device, dtype = where
    pages = max(1, pc.peak_tokens(steps, page_size) // page_size)
    runner = ModelRunner(folder, dtype=dtype, device=device, page_size=page_size, num_pages=pages, num_state_slots=max_live,
                         max_model_len=pages * page_size, poison_freed_pages=True, **options)
    got = replay(runner, steps)
    assert not runner.cache.requests and all(runner.cache.num_free_pages(g) == pages for g in range(len(runner.cache.groups)))
    return got


def _compare(got, want, dtype, what):
    tol = tolerance_for(dtype, want)
    for rid in want:
        assert max_abs_diff(got[rid], want[rid]) <= tol, (what, rid, first_difference(got[rid], want[rid], tol))


@pytest.mark.parametrize("where", WHERE)
@pytest.mark.parametrize("name", ["P", "Q", "R"])
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


@pytest.mark.parametrize("where", ON_GPU)
def test_pages_of_64_and_chunks_longer_than_a_page(folders, where, kernels):
    """Pages of 64 tokens (whole tiles of the prompt kernel lie in one page) under chunks of 96, 128 and 160
    positions, requests of up to 400 tokens in portions that end anywhere, beside decoded tokens, on few pages."""
    device, dtype = where
    requests = _requests("S", [400, 130, 70, 257])
    want = _plain_logits(folders["S"], requests)
    for what, steps in (("portions", pc.in_portions(requests, [37, 2, 64, 5, 1, 129, 1, 1, 96])),
                        ("side by side", pc.interleaved(requests, [33, 1, 1, 64, 1, 7, 1, 100], 3))):
        got = _replay(folders["S"], where, steps, page_size=64, max_live=3)
        _compare(got, want, dtype, what)


@pytest.mark.parametrize("where", WHERE)
def test_long_decoding(folders, where, kernels):
    """Two tokens of prompt, then 140 tokens one by one: the chunks of every layer pass many times, pages go back
    to the pool on the way, and the recurrent state is carried through every step."""
    device, dtype = where
    n = 60 if device == "cpu" else 142
    requests = _requests("P", [n])
    want = _plain_logits(folders["P"], requests)
    steps = pc.in_portions(requests, [2] + [1] * n)
    got = _replay(folders["P"], where, steps, page_size=4, max_live=1)
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
    cfg, w = plain.read_model_folder(folders["P"])
    prompts = [pc.tokens(cfg["vocab"], n, 300 + n) for n in (1, 13, 22)]
    llm = LLM(folders["P"], device=device, dtype=dtype, **options)
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
    """``random-model --shape pevazen-tiny`` writes a folder that the plain implementation and the engine both read
    (its config.json names the two inner sizes that a checkpoint would show by its tensors' shapes)."""
    out = str(tmp_path / "m")
    _command("random-model", "--out", out, "--shape", "pevazen-tiny", "--seed", "5")
    cfg, w = plain.read_model_folder(out)
    assert cfg["architecture"] == "Pevazen" and w["l0.mix.right.a1"].shape[0] == cfg["layers"][0]["mixer"]["right"]["decay_rank"]
    requests = {"a": pc.tokens(cfg["vocab"], 31, 1)}
    want = {"a": plain.logits(cfg, w, requests["a"])}
    got = _replay(out, CPU, pc.in_portions(requests, [4, 1, 9]), page_size=8, max_live=1)
    _compare(got, want, "float32", "portions")


@pytest.mark.gpu
def test_generate_command_with_random_weights():
    if not torch.cuda.is_available():
        pytest.skip("no GPU here")
    out = json.loads(_command("generate", "--random-weights", "4", "--shape", "pevazen-tiny", "--prompt-ids", "5 17 3",
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
