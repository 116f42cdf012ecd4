"""The Fazovik design in the engine against its plain whole-sequence implementation (``plain_fazovik.py``): every
mechanism alone through the kernels' entry points, then whole models through the step function (whole prompts,
decoding token by token, portions down to two tokens, unequal requests side by side on few pages and slots that are
used again), and greedy generation through the entry point and its scheduler. Every test runs on the CPU stand-in
for the kernels (the engine's logic) and, marked ``gpu``, on the HIP kernels in both element types.
"""
import json

import pytest
import torch

import fazovik_cases as fc
import pevazen_cases as pc          # the ways of cutting requests into steps
import plain_fazovik as plain
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
    return {name: fc.write_model(str(tmp_path_factory.mktemp(f"fazovik_{name}")), cfg, seed)
            for name, (cfg, seed) in fc.CASES.items()}


def _dt(name):
    return {"float32": torch.float32, "bfloat16": torch.bfloat16}[name]


def _tol(dtype, plain_values, fine=2e-5, coarse=4e-2):
    """Largest allowed difference, as a share of the spread of the plain values."""
    return (fine if dtype == "float32" else coarse) * float(plain_values.float().std())


def _batch(lengths, starts, device):
    """A batch of requests that bring ``lengths`` tokens from positions ``starts`` on."""
    T = sum(lengths)
    req = torch.tensor([r for r, n in enumerate(lengths) for _ in range(n)], dtype=torch.int32)
    pos = torch.tensor([s + j for s, n in zip(starts, lengths) for j in range(n)], dtype=torch.int32)
    cu = torch.tensor([0] + list(torch.tensor(lengths).cumsum(0)), dtype=torch.int32)
    ctx = torch.tensor([s + n for s, n in zip(starts, lengths)], dtype=torch.int32)
    return AttentionBatch(num_tokens=T, num_requests=len(lengths), token_req=req.to(device), positions=pos.to(device),
                          cu_seqlens_q=cu.to(device), context_lens=ctx.to(device), max_q_len=max(lengths),
                          max_context_len=int(ctx.max()))


# ------------------------------------------------------------------ mechanisms alone
@pytest.mark.parametrize("where", WHERE)
def test_hashed_pair_embedding_in_portions_and_on_slots_used_again(where, kernels):
    device, dtype = where
    g = torch.Generator().manual_seed(3)
    V, W, buckets, mp, mc = 23, 10, 7, 31, 5
    table = torch.randn(V, W, generator=g).to(_dt(dtype))
    pair = torch.randn(buckets + 1, W, generator=g).to(_dt(dtype))
    seqs = [pc.tokens(V, n, 40 + n) for n in (9, 1, 6, 4)]
    want = [table[torch.tensor(s)].float() + pair[torch.tensor(plain.bigram_rows(s, buckets, mp, mc))].float() for s in seqs]
    prev = torch.full((3,), 5, dtype=torch.int32).to(device)           # stale numbers in every slot
    # requests 0 and 1 side by side in portions; then request 2 takes request 1's slot, request 3 that of request 0
    plan = [([(0, 0, 4), (1, 0, 1)], {0: 0, 1: 2}), ([(0, 4, 2)], {0: 0}), ([(0, 6, 3), (2, 0, 2)], {0: 0, 2: 2}),
            ([(2, 2, 4), (3, 0, 1)], {2: 2, 3: 0}), ([(3, 1, 3)], {3: 0})]
    got = [[] for _ in seqs]
    for entries, slot_of in plan:
        ids = torch.tensor([t for r, lo, n in entries for t in seqs[r][lo:lo + n]], dtype=torch.int32).to(device)
        batch = _batch([n for _, _, n in entries], [lo for _, lo, _ in entries], device)
        slots = torch.tensor([slot_of[r] for r, _, _ in entries], dtype=torch.int32).to(device)
        out = ops.embed_pair_hash(ids, table.to(device), pair.to(device), batch, slots, prev, buckets, mp, mc)
        assert out.dtype == torch.float32
        at = 0
        for r, lo, n in entries:
            got[r].append(out[at:at + n].cpu())
            at += n
    for r in range(len(seqs)):
        assert torch.equal(torch.cat(got[r]), want[r]), r


@pytest.mark.parametrize("where", WHERE)
def test_two_layer_norms_of_one_stream_with_pending_additions(where, kernels):
    device, dtype = where
    g = torch.Generator().manual_seed(4)
    T, W, eps = 5, 37, 1e-3
    x = torch.randn(T, W, generator=g) * 3 + 1
    a, b = (torch.randn(T, W, generator=g).to(_dt(dtype)) for _ in range(2))
    w1, b1, w2, b2 = (torch.randn(W, generator=g) for _ in range(4))
    stream = x.clone().to(device)
    y1, y2 = ops.layernorm_pair(stream, (w1.to(device), b1.to(device)), (w2.to(device), b2.to(device)), eps, _dt(dtype),
                                add=(a.to(device), b.to(device)))
    s = x + a.float() + b.float()
    assert max_abs_diff(stream.cpu(), s) <= 1e-6 * float(s.abs().max())
    for y, w, c in ((y1, w1, b1), (y2, w2, b2)):
        want = plain.layer_norm(s.double(), w.double(), c.double(), eps).float()
        assert y.dtype == _dt(dtype) and max_abs_diff(y.cpu(), want) <= _tol(dtype, want)
    only, none = ops.layernorm_pair(stream, None, (w2.to(device), b2.to(device)), eps, _dt(dtype))
    assert only is None and max_abs_diff(none.cpu(), y2.cpu()) == 0
    ops.add_streams_(stream, a.to(device))
    assert max_abs_diff(stream.cpu(), s + a.float()) <= 1e-6 * float(s.abs().max())
    gu = torch.randn(T, 2 * 9, generator=g).to(_dt(dtype))
    got = ops.act_mul(gu.to(device), "gelu_tanh")
    want = plain.gelu_tanh(gu[:, :9].double()) * gu[:, 9:].double()
    assert max_abs_diff(got.cpu(), want.float()) <= _tol(dtype, want)
    # the gate-and-up product with this activation: few rows (one kernel where the rows are bfloat16) and many
    for rows in (3, 40):
        x = torch.randn(rows, 24, generator=g).to(_dt(dtype))
        w = (torch.randn(2 * 16, 24, generator=g) / 24 ** 0.5).to(_dt(dtype))
        got = ops.gated_linear(x.to(device), w.to(device), "gelu_tanh")
        both = x.double() @ w.double().T
        want = plain.gelu_tanh(both[:, :16]) * both[:, 16:]
        assert max_abs_diff(got.cpu(), want.float()) <= _tol(dtype, want), rows


def test_scaled_frequencies_of_the_position_encoding():
    from nanohybrid_vlm_amd.parts.positions import YarnFrequencies
    for rot in ({"dims": 12, "base": 30000.0, "scaling": {"factor": 3.0, "fast": 16.0, "original": 256, "slow": 0.5}},
                {"dims": 8, "base": 100.0, "scaling": {"factor": 8.0, "fast": 4.0, "original": 64, "slow": 2.0}},
                {"dims": 6, "base": 10000.0}):
        s = rot.get("scaling") or {}
        enc = YarnFrequencies(rot["dims"], rot["base"], 1 << 20, s.get("factor"), s.get("original"), s.get("fast"), s.get("slow"))
        f, gain = plain.scaled_frequencies(rot)
        assert torch.allclose(enc.frequencies(), f, rtol=1e-14, atol=0) and abs(enc.gain() - gain) < 1e-15
    # the second case has pairs that keep their frequency, pairs that are divided by the factor, and pairs between
    rot = {"dims": 8, "base": 100.0, "scaling": {"factor": 8.0, "fast": 4.0, "original": 64, "slow": 2.0}}
    ratio = plain.scaled_frequencies(rot)[0] / plain.scaled_frequencies({"dims": 8, "base": 100.0})[0]
    assert float(ratio.max()) == 1.0 and abs(float(ratio.min()) - 1 / 8) < 1e-12 and ((ratio > 0.2) & (ratio < 0.9)).any()


def _latent_layer(device, dtype, m, W, portions, page_size, seed, lender_rot=0):
    """One latent attention mixer through its part, in portions of one request on scrambled pages, against the plain
    function. Returns (got, want)."""
    from nanohybrid_vlm_amd.parts.base import CacheView
    from nanohybrid_vlm_amd.parts.context import GroupTables, StepContext
    from nanohybrid_vlm_amd.parts.latent import LatentAttention
    from nanohybrid_vlm_amd.parts.positions import YarnFrequencies
    g = torch.Generator().manual_seed(seed)
    T = sum(portions)
    rot = m.get("rot_dim", 0)
    cfg = {"width": W, "vocab": 4, "layers": [{"type": "latent_attention" if rot else "latent_attention_2", "mixer": m, "mlp": None}]}
    w = {k[len("l0.mix."):]: v.double() for k, v in fc.random_tensors(cfg, seed).items() if k.startswith("l0.mix.")}
    h = torch.randn(T, W, generator=g).to(torch.bfloat16)
    fn = plain.latent_attention if rot else plain.latent_attention_2
    want, _ = fn(h.double(), w, "", m, 1e-5, {})
    position = None
    if rot:
        s = m["rot"].get("scaling") or {}
        position = YarnFrequencies(rot, m["rot"]["base"], 1 << 20, s.get("factor"), s.get("original"), s.get("fast"),
                                   s.get("slow")).to(device)
    part = LatentAttention(W, m["heads"], m["dim"], rot, m["vdim"], m["q_rank"], m["kv_rank"], m["scale"], 1e-5, gated=bool(rot),
                           position=position)
    dt = _dt(dtype)
    down = torch.cat([w["dq"], w["dkv"]] + ([w["g"]] if rot else []))
    part.bind({"down.weight": down.to(dt).to(device), "q_norm.weight": w["dq.norm"].float().to(device),
               "kv_norm.weight": w["dkv.norm"].float().to(device), "uq.weight": w["uq"].to(dt).to(device),
               "uk.weight": w["uk"].to(dt).to(device), "uv.weight": w["uv"].to(dt).to(device), "o.weight": w["o"].to(dt).to(device)})
    n_pages = -(-T // page_size)
    pages = torch.randperm(n_pages + 2, generator=g).tolist()[:n_pages]
    cache = torch.full((n_pages + 2, page_size, 1, part.row), float("nan"), dtype=dt).to(device)
    view = CacheView(kind="paged", group=0, k=cache, v=cache, writes=True)
    outs, at = [], 0
    for n in portions:
        batch = _batch([n], [at], device)
        slots = torch.tensor([pages[p // page_size] * page_size + p % page_size for p in range(at, at + n)], dtype=torch.int32)
        step = StepContext(num_tokens=n, num_requests=1, input_ids=None, positions=batch.positions.view(1, -1),
                           token_positions=batch.positions, attention=batch,
                           groups=[GroupTables(slots.to(device), torch.tensor([pages], dtype=torch.int32).to(device))],
                           state_slots=None, logit_rows=None)
        outs.append(part.forward(h[at:at + n].to(dt).to(device), step, view).float().cpu())
        at += n
    return torch.cat(outs), want.float()


@pytest.mark.parametrize("where", WHERE)
@pytest.mark.parametrize("case", ["rotary, scaled", "rotary, rows of 64", "no positions", "one head"])
def test_latent_attention_alone_in_portions(where, kernels, case):
    device, dtype = where
    m, W = {
        "rotary, scaled": (fc.CONFIG_F["layers"][0]["mixer"], 20),
        "rotary, rows of 64": (fc.CONFIG_G["layers"][1]["mixer"], 32),
        "no positions": (fc.CONFIG_F["layers"][1]["mixer"], 24),
        "one head": (dict(fc.CONFIG_G["layers"][2]["mixer"], kv_from=None), 16),
    }[case]
    m = {k: v for k, v in m.items() if v is not None}
    got, want = _latent_layer(device, dtype, m, W, [7, 2, 1, 1, 30, 1, 5, 2, 1], page_size=4, seed=5)
    tol = _tol(dtype, want)
    assert max_abs_diff(got, want) <= tol, first_difference(got, want, tol)


@pytest.mark.parametrize("where", WHERE)
@pytest.mark.parametrize("row", [64, 24])
def test_one_far_key_outweighs_hundreds(where, kernels, row):
    """Stored rows serve as keys and as values. One row, far back, at the last place of a page, at the first of the
    next, or just before the query, is made to stand out for one head; the result of that head must be that row, as
    a prompt's portion and as a single decoded token, on scrambled pages."""
    device, dtype = where
    dt = _dt(dtype)
    g = torch.Generator().manual_seed(row)
    n_keys, page_size, H = (330, 64, 3) if device != "cpu" else (140, 16, 2)
    n_pages = -(-n_keys // page_size)
    pages = torch.randperm(n_pages + 1, generator=g).tolist()[:n_pages]
    for place in (0, page_size - 1, page_size, 2 * page_size - 1, n_keys - 2, n_keys - 1):
        rows = 0.1 * torch.randn(n_keys, row, generator=g)
        rows[place, 0] = 6.0
        cache = torch.full((n_pages + 1, page_size, 1, row), float("nan"), dtype=dt)
        for p in range(n_keys):
            cache[pages[p // page_size], p % page_size, 0] = rows[p].to(dt)
        cache = cache.to(device)
        table = torch.tensor([pages], dtype=torch.int32).to(device)
        for n_q in (1, 5):                                  # decoded alone, and the end of a portion
            first = n_keys - n_q
            q = torch.zeros(n_q, H, row)
            q[:, 1, 0] = 8.0                                # head 1 looks for the planted row; the others see noise
            q[:, 0] = torch.randn(n_q, row, generator=g)
            batch = _batch([n_q], [first], device)
            got = ops.paged_attention(q.to(dt).to(device), cache, cache, batch, table, 1.0).float().cpu()
            for j in range(n_q):
                p = first + j
                if place > p:
                    continue
                keys = rows[:p + 1].to(dt).double()
                want = torch.softmax(keys @ q[j].to(dt).double().T, dim=0).T @ keys           # [H, row]
                assert max_abs_diff(got[j], want.float()) <= (1e-4 if dtype == "float32" else 3e-2), (place, n_q, j)
                assert abs(float(got[j, 1, 0]) - 6.0) < 0.1                                     # it is the planted row


@pytest.mark.parametrize("where", WHERE)
def test_routed_experts_alone(where, kernels):
    device, dtype = where
    dt = _dt(dtype)
    g = torch.Generator().manual_seed(8)
    for E, top, F, W, T in ((5, 2, 12, 20, 9), (1, 1, 8, 16, 3), (7, 7, 4, 12, 4), (70, 3, 8, 24, 21), (2, 1, 16, 32, 70),
                            (3, 2, 24, 40, 130), (2, 2, 136, 72, 300)):
        w = {"router": (torch.randn(E, W, generator=g) * 0.6).to(torch.bfloat16).double()}
        for e in range(E):
            w[f"e{e}.gate"] = (torch.randn(F, W, generator=g) / W ** 0.5).to(torch.bfloat16).double()
            w[f"e{e}.up"] = (torch.randn(F, W, generator=g) / W ** 0.5).to(torch.bfloat16).double()
            w[f"e{e}.down"] = (torch.randn(W, F, generator=g) / F ** 0.5).to(torch.bfloat16).double()
        h = torch.randn(T, W, generator=g).to(torch.bfloat16)
        want = plain.routed_ff(h.double(), w, "", {"router": {"experts": E, "top": top}}).float()
        logits = ops.linear(h.to(dt).to(device), w["router"].to(dt).to(device), out_dtype=torch.float32)
        ids, scores = ops.route_topk(logits, top)
        s = torch.sigmoid(h.double() @ w["router"].T)
        assert torch.equal(ids.cpu().long().sort(dim=-1).values, torch.topk(s, top, dim=-1).indices.sort(dim=-1).values)
        assert max_abs_diff(scores.cpu(), torch.gather(s, 1, ids.cpu().long()).float()) < 1e-5
        gate_up = torch.stack([torch.cat((w[f"e{e}.gate"], w[f"e{e}.up"])) for e in range(E)]).to(dt).to(device)
        down = torch.stack([w[f"e{e}.down"] for e in range(E)]).to(dt).to(device)
        got = ops.routed_experts(h.to(dt).to(device), ids, scores, gate_up, down, "silu")
        assert max_abs_diff(got.float().cpu(), want) <= _tol(dtype, want), (E, top)
        # a token's result does not depend on its batch mates
        alone = ops.routed_experts(h[2:3].to(dt).to(device), ids[2:3].contiguous(), scores[2:3].contiguous(), gate_up, down, "silu")
        assert max_abs_diff(alone.float().cpu(), got[2:3].float().cpu()) <= (0 if dtype == "float32" else _tol(dtype, want))


# ------------------------------------------------------------------ configuration and weights
def test_configuration_and_names(folders):
    from nanohybrid_vlm_amd.parts.model import DecoderModel
    arch = resolve_architecture(fc.CONFIG_F)
    assert arch.name == "Fazovik"
    cfg = arch.parse_config(fc.CONFIG_F)
    assert cfg.layers[3].mixer.kv_from == 1 and cfg.layers[2].mlp is None and cfg.layers[1].mlp.top == 2
    model = DecoderModel(arch.build_spec(cfg))
    names = arch.checkpoint_names(cfg)
    assert set(names) == set(fc.random_tensors(fc.CONFIG_F, 0))
    assert {s.param for s in names.values()} == set(model.all_param_specs())
    needs = model.cache_needs()
    # a token stores its latent (and rotated key part) once; borrowers store nothing
    assert needs[3] is None and needs[4] is None and needs[0].head_dim == 13 + 4 and needs[1].head_dim == 18
    assert all(n is None or (n.values_in_keys and n.num_kv_heads == 1) for n in needs)
    assert model.layers[4].mixer.pad_dim == 4 and model.embedding_state_need() is not None
    for change, match in ((lambda c: c["layers"][3]["mixer"].update(kv_from=3), "kv_from"),
                          (lambda c: c["layers"][3]["mixer"].update(kv_from=4), "kv_from"),
                          (lambda c: c["layers"][3]["mixer"].update(kv_rank=17), "kv_rank"),
                          (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=6), "rot.dims"),
                          (lambda c: c["layers"][1].update(type="other"), "not known"),
                          (lambda c: c["layers"][1]["mlp"].update(kind="sparse"), "not known"),
                          (lambda c: c["layers"][1]["mlp"]["router"].update(top=6), "top"),
                          (lambda c: c["norm"].update(eps=0), "eps")):
        bad = json.loads(json.dumps(fc.CONFIG_F))
        change(bad)
        with pytest.raises(ConfigError, match=match):
            arch.parse_config(bad)


def test_a_layer_without_feed_forward_may_store_its_second_norm(tmp_path, emulated_kernels):
    """Such a layer's second norm has nothing to norm for; a checkpoint that stores it all the same is read."""
    import os
    from safetensors.torch import save_file
    folder = str(tmp_path / "m")
    fc.write_model(folder, fc.CONFIG_F, 3)
    tensors = fc.random_tensors(fc.CONFIG_F, 3)
    tensors["l2.norm2"] = torch.ones(fc.CONFIG_F["width"], dtype=torch.bfloat16)
    tensors["l2.norm2.b"] = torch.zeros(fc.CONFIG_F["width"], dtype=torch.bfloat16)
    save_file({k: v.contiguous() for k, v in tensors.items()}, os.path.join(folder, "model.safetensors"))
    requests = {"a": pc.tokens(fc.CONFIG_F["vocab"], 17, 2)}
    got = _replay(folder, CPU, pc.in_portions(requests, [5, 1, 11]), page_size=4, max_live=1)
    _compare(got, _plain_logits(folder, requests), "float32", "portions")


def test_a_model_without_the_pair_table(tmp_path, emulated_kernels):
    """Without ``embedding.bigram`` the embedding is the table's rows alone (and no request keeps a previous token)."""
    config = json.loads(json.dumps(fc.CONFIG_G))
    del config["embedding"]
    folder = fc.write_model(str(tmp_path / "m"), config, 5)
    requests = {"a": pc.tokens(config["vocab"], 14, 3), "b": pc.tokens(config["vocab"], 6, 4)}
    got = _replay(folder, CPU, pc.interleaved(requests, [3, 1, 4], 2), page_size=4, max_live=2)
    _compare(got, _plain_logits(folder, requests), "float32", "side by side")


# ------------------------------------------------------------------ whole models through the step function
def _requests(name, lengths):
    vocab = fc.CASES[name][0]["vocab"]
    return {f"r{i}": pc.tokens(vocab, n, 100 * i + n) for i, n in enumerate(lengths)}


def _plain_logits(folder, requests):
    cfg, w = plain.read_folder(folder)
    return {rid: plain.forward(cfg, w, toks).float() for rid, toks in requests.items()}


def _replay(folder, where, steps, page_size, max_live, **options):
    device, dtype = where
    pages = max(1, pc.peak_tokens(steps, page_size) // page_size)
    runner = ModelRunner(folder, dtype=dtype, device=device, page_size=page_size, num_pages=pages, num_state_slots=max_live,
                         max_model_len=pages * page_size, poison_freed_pages=True, **options)
    got = replay(runner, steps)
    assert not runner.cache.requests and all(runner.cache.num_free_pages(g) == pages for g in range(len(runner.cache.groups)))
    return got


def _compare(got, want, dtype, what):
    """float32: every position within the tolerance. bfloat16: rounding can turn a router's close call the other way,
    which changes that token's logits by much and those of later tokens by a little; so a few positions (one in
    twenty-five) may lie beyond the tolerance there. (The float32 run is what pins the engine's logic; the bfloat16
    run is about its other kernels, whose faults would show at most positions.)"""
    tol = tolerance_for(dtype, want)
    rows = over = 0
    for rid in want:
        if dtype == "float32":
            assert max_abs_diff(got[rid], want[rid]) <= tol, (what, rid, first_difference(got[rid], want[rid], tol))
        d = (got[rid].float() - want[rid].float()).abs().amax(dim=-1)
        rows += d.numel()
        over += int((d > tol).sum())
    assert over <= max(1, rows // 25), (what, f"{over} of {rows} positions beyond the tolerance")


@pytest.mark.parametrize("where", WHERE)
def test_residual_stream_after_every_layer(folders, where, kernels):
    """The stream after each layer of a short request, against the plain model's (the additions of a layer are made
    by the next layer's norm kernel, those of the last by a kernel of their own)."""
    device, dtype = where
    cfg, w = plain.read_folder(folders["F"])
    toks = pc.tokens(cfg["vocab"], 19, 7)
    _, want = plain.forward(cfg, w, toks, return_layers=True)
    runner = ModelRunner(folders["F"], dtype=dtype, device=device, page_size=8, num_pages=4, num_state_slots=1)
    seen = []
    for i, layer in enumerate(runner.model.layers):
        inner = layer.forward

        def spy(hidden, residual, step, cache, _inner=inner, **more):
            out = _inner(hidden, residual, step, cache, **more)
            pending = step.scratch.get("pending_additions")
            x = out[0].clone()
            if pending is not None:
                x = x + sum(t.float() for t in pending[1] if t is not None)
            seen.append(x.cpu())
            return out
        layer.forward = spy
    from nanohybrid_vlm_amd.engine.runner import StepEntry
    runner.step([StepEntry("a", toks, [len(toks) - 1])])
    for i, x in enumerate(seen):
        ref = want[i].float()
        assert max_abs_diff(x, ref) <= (3e-5 if dtype == "float32" else 6e-2) * float(ref.std()), i


@pytest.mark.parametrize("where", WHERE)
@pytest.mark.parametrize("name", ["F", "G"])
def test_ways_of_cutting_agree_with_the_plain_model(folders, where, kernels, name):
    """Whole prompts, a prompt followed by its last tokens one by one, portions of several sizes down to two tokens
    (and single tokens between them), and unequal requests side by side on pages and slots that are used again: all
    give the plain model's logits at every position. In float32 on the GPU the ways agree bit for bit."""
    device, dtype = where
    lengths = [1, 2, 26, 19, 37, 5] if device == "cpu" else [1, 2, 26, 19, 61, 5, 150, 43]
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
def test_pages_of_64_and_longer_requests(folders, where, kernels):
    """Pages of 64 tokens (whole tiles of the prompt kernel lie in one page), requests of up to 400 tokens in portions
    that end anywhere, beside decoded tokens, on few pages."""
    requests = _requests("G", [400, 130, 70, 257])
    want = _plain_logits(folders["G"], requests)
    for what, steps in (("portions", pc.in_portions(requests, [37, 2, 64, 5, 1, 129, 1, 1, 96])),
                        ("side by side", pc.interleaved(requests, [33, 1, 1, 64, 1, 7, 1, 100], 3))):
        got = _replay(folders["G"], where, steps, page_size=64, max_live=3)
        _compare(got, want, where[1], what)


@pytest.mark.parametrize("where", WHERE)
def test_long_decoding(folders, where, kernels):
    """Two tokens of prompt, then many tokens one by one through the cache and the kept previous token."""
    device, dtype = where
    n = 50 if device == "cpu" else 142
    requests = _requests("F", [n])
    want = _plain_logits(folders["F"], requests)
    got = _replay(folders["F"], where, pc.in_portions(requests, [2] + [1] * n), page_size=4, max_live=1)
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
        requests = _requests("G", [40, 3, 17, 9])
        steps = pc.interleaved(requests, [3, 1, 1, 1, 2, 1, 1], 3)
        for s in steps:                                      # a recorded short step gives one place a request
            for e in s["entries"]:
                e["want"] = e["want"][-1:]
        where = ("cuda:0", dtype)
        eager = _replay(folders["G"], where, steps, page_size=8, max_live=3, use_graphs=False)
        recorded = _replay(folders["G"], where, steps, page_size=8, max_live=3, use_graphs=True)
        for rid in eager:
            if dtype == "float32":
                assert torch.equal(eager[rid], recorded[rid]), rid
            else:
                assert max_abs_diff(eager[rid], recorded[rid]) <= 0.05 * float(eager[rid].std()), rid
    finally:
        ops.set_backend(old)


# ------------------------------------------------------------------ generation through the entry point
def _greedy(cfg, w, prompt, n):
    ids = list(prompt)
    for _ in range(n):
        ids.append(int(plain.forward(cfg, w, ids)[-1].argmax()))
    return ids[len(prompt):]


@pytest.mark.parametrize("where", [pytest.param(CPU, id="cpu-stand-in"), ON_GPU[0]])
@pytest.mark.parametrize("options", [dict(kvcache_block_size=4, num_kvcache_blocks=64),
                                     dict(kvcache_block_size=8, num_kvcache_blocks=40, max_num_batched_tokens=7, max_num_seqs=2)],
                         ids=["whole prompts", "portions of 7, two at a time"])
def test_greedy_generation_through_the_entry_point(folders, where, kernels, options):
    from nanohybrid_vlm_amd import LLM, SamplingParams
    device, dtype = where
    cfg, w = plain.read_folder(folders["F"])
    prompts = [pc.tokens(cfg["vocab"], n, 300 + n) for n in (1, 13, 22)]
    llm = LLM(folders["F"], device=device, dtype=dtype, **options)
    outs = llm.generate(prompts, SamplingParams(temperature=0.0, max_tokens=7, ignore_eos=True), use_tqdm=False)
    for prompt, out in zip(prompts, outs):
        assert out["token_ids"] == _greedy(cfg, w, prompt, 7)
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
    """``random-model --shape fazovik-tiny`` writes a folder that the plain implementation and the engine both read."""
    out = str(tmp_path / "m")
    _command("random-model", "--out", out, "--shape", "fazovik-tiny", "--seed", "5")
    cfg, w = plain.read_folder(out)
    assert cfg["architecture"] == "Fazovik" and w["bigram"].shape[0] == cfg["embedding"]["bigram"]["buckets"] + 1
    requests = {"a": pc.tokens(cfg["vocab"], 31, 1)}
    want = {"a": plain.forward(cfg, w, requests["a"]).float()}
    got = _replay(out, CPU, pc.in_portions(requests, [4, 1, 9]), page_size=8, max_live=1)
    _compare(got, want, "float32", "portions")


@pytest.mark.gpu
def test_generate_command_with_random_weights():
    if not torch.cuda.is_available():
        pytest.skip("no GPU here")
    out = json.loads(_command("generate", "--random-weights", "4", "--shape", "fazovik-tiny", "--prompt-ids", "5 17 3",
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
    requests = _requests("G", [150, 9, 71, 2, 40])
    want = _plain_logits(folders["G"], requests)
    ways = {"portions": pc.in_portions(requests, [37, 2, 64, 5, 1, 1]),
            "side by side": pc.interleaved(requests, [33, 1, 1, 16, 1, 7, 1], 4)}
    steps, first = [], 0
    for k, (what, t) in enumerate(ways.items()):
        steps += _renamed(t, f"#{k}", first)
        first += len(t)
    out_dir = str(tmp_path / "out")
    _trace_run(folders["G"], dtype, steps, out_dir, max(pc.peak_tokens(t, 64) for t in ways.values()))
    got = _logits_from_files(out_dir, steps, fc.CONFIG_G["vocab"])
    for k, what in enumerate(ways):
        _compare({rid: got[f"{rid}#{k}"] for rid in want}, want, dtype, what)
