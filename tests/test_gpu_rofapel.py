"""The Rofapel decoder on the GPU against the plain implementation in ``plain_rofapel.py``: each mechanism
alone, whole prompts, decoding, portions, mixed batches, pages and slots used again, peaked attention at the
edges of windows and far back, the first tokens of a sequence, sizes that are 1, equal or odd, and greedy
generation through ``LLM``."""

import copy
from types import SimpleNamespace

import pytest
import torch

import plain_rofapel as plain
import rofapel_util as ru
from replay_util import mixed_trace, portion_trace, random_tokens, round64, run_steps, tail_trace, whole_trace

pytestmark = pytest.mark.gpu

F64 = torch.float64
LENGTHS = {"a": 83, "b": 40, "c": 7, "d": 1, "e": 118, "f": 29, "g": 2}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    out = {}
    for name, cfg, seed in (("mixed", ru.MIXED, 41), ("sharp", ru.SHARP, 42), ("ones", ru.ONES, 43), ("odd", ru.ODD, 44),
                            ("tail_loop", ru.TAIL_LOOP, 45), ("crossed", ru.CROSSED, 46), ("no_rotation", ru.NO_ROTATION, 47)):
        out[name] = ru.write_model(str(tmp_path_factory.mktemp(name)), cfg, seed)
    return out


def _oracle(folder, tokens, store=None, cfg_edit=None, tensors_edit=None):
    cfg, tensors = plain.rofapel_read(folder, F64)
    if cfg_edit is not None:
        cfg_edit(cfg)
    if tensors_edit is not None:
        tensors_edit(tensors)
    return plain.rofapel_forward(cfg, tensors, tokens, store or plain._keep).to(torch.float32)


def _rel_rows(got, want):
    """Per row: RMS of the difference (mean taken off) over the RMS of the wanted row."""
    d = (got - want).double()
    d = d - d.mean(dim=1, keepdim=True)
    return d.pow(2).mean(dim=1).sqrt() / want.double().pow(2).mean(dim=1).sqrt()


def _rel(got, want):
    return _rel_rows(got, want).max().item()


def _like_rounding(errors, rounding, slack=1e-3):
    """``errors``: per-row distances of the engine's bfloat16 logits from exact arithmetic; ``rounding``:
    the same for the plain model with its stored activations rounded to bfloat16.  Rounding moves single
    rows far (a router's choice between two experts whose logits all but tie falls the other way), in the
    plain model as in the engine, so the two are compared as distributions."""
    return (errors.median() < 2 * rounding.median() + slack
            and errors.quantile(0.9) < 3 * rounding.quantile(0.9) + slack)


def _replayer(folder, dtype, max_tokens, max_live=4):
    from qwen25vl_lite_amd.engine.replay import Replayer
    return Replayer(folder, dtype, max_tokens, 16, max_live)


def _rows(got, rid, n):
    return torch.stack([got[(rid, p)] for p in range(n)])


def _requests(vocab, seed=0):
    return {rid: random_tokens(n, vocab, seed + i) for i, (rid, n) in enumerate(LENGTHS.items())}


# ---------------------------------------------------------------------------------------------
# each mechanism alone
# ---------------------------------------------------------------------------------------------
def _one_layer(tmp_path, lay, dtype=torch.float32, seed=0, width=56, tensors_edit=None, name="one", loop=None):
    from qwen25vl_lite_amd.config import EngineConfig, load_config
    from qwen25vl_lite_amd.engine import ModelRunner
    from qwen25vl_lite_amd.models import build_model
    from qwen25vl_lite_amd.weights import load_weights
    cfg = ru.config(width, 50, lay if isinstance(lay, list) else [lay], eps=1e-4, scale=1.3, loop=loop)
    tensors = ru.random_tensors(cfg, seed)
    if tensors_edit is not None:
        tensors_edit(tensors)
    d = ru.write_model(str(tmp_path / name), cfg, seed, tensors)
    model = build_model(load_config(d), dtype, "cuda:0")
    load_weights(d, model)
    ecfg = EngineConfig(num_blocks=32, block_size=16, max_num_seqs=3, max_num_batched_tokens=512, max_model_len=512,
                        enable_prefix_cache=False, dtype=dtype)
    _, t64 = plain.rofapel_read(d, F64)
    return ModelRunner(model, ecfg), model, t64


def _step_for(runner, runs):
    """A step context for ``runs``: (request id, tokens, start); a request is admitted at start 0 and its
    state rows cleared as the runner does."""
    from qwen25vl_lite_amd.engine import StepEntry
    from qwen25vl_lite_amd.engine.batch import build_step
    entries = []
    for rid, n, start in runs:
        if start == 0:
            runner.admit(rid)
        entries.append(StepEntry(rid, [0] * n, start))
        runner.cache.reserve(rid, start + n)
    runner._clear_state(entries)
    return build_step(entries, runner.cache, 1, runner.dtype, runner.device)


def _commit(runner, runs):
    for rid, n, start in runs:
        runner.cache.commit(rid, start + n)


def _run_mixer(runner, mixer, runs, x, dtype):
    step = _step_for(runner, runs)
    out = mixer.forward(x.to(dtype).cuda(), step, runner.slots[0])
    _commit(runner, runs)
    return (out.sum(0) if out.dim() == 3 else out).double().cpu()


MIXER_CASES = {
    "attention": (ru.attention(6, 2, 24, 16, base=80.0, dims=16, scale=0.7), plain.attention),
    "attention_full_rotation": (ru.attention(2, 2, 16, 16, base=30.0, scale=0.5), plain.attention),
    "attention_one_group": (ru.attention(5, 1, 10, 7, base=80.0, dims=6, scale=0.7), plain.attention),
    "attention_2": (ru.attention_2(4, 2, 16, mask=9, conv=3, base=500.0, dims=8, scale=0.9, factor=3.0), plain.attention_2),
    "attention_2_wide_window": (ru.attention_2(3, 3, 24, mask=70, conv=4, base=200.0, scale=0.6, factor=None), plain.attention_2),
    "attention_2_one_token": (ru.attention_2(2, 1, 8, mask=1, conv=1, base=20.0, scale=0.6, factor=1.0), plain.attention_2),
    "attention_2_odd": (ru.attention_2(3, 1, 10, mask=5, conv=5, base=77.0, dims=6, scale=0.5, factor=1.5), plain.attention_2),
    "latent": (ru.latent(3, 16, 8, 24, 40, base=300.0, scale=0.6, ramp=(4.0, 48, 8.0, 1.5)), plain.latent_attention),
    "latent_no_ramp": (ru.latent(2, 8, 16, 8, 24, base=50.0, scale=0.8, ramp=None), plain.latent_attention),
    "latent_odd": (ru.latent(3, 10, 6, 7, 13, base=77.0, scale=0.7, ramp=(2.5, 40, 6.0, 1.2)), plain.latent_attention),
}


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("case", sorted(MIXER_CASES))
def test_a_mixer_alone_whole_in_two_steps_and_token_by_token(case, dtype, tmp_path):
    """The mixer's own forward against the plain function: one run of 90 tokens, the same cut inside a page,
    and (in float32) the same token by token through the cache beside another request's tokens."""
    spec, fn = MIXER_CASES[case]
    runner, model, t = _one_layer(tmp_path, ru.layer(spec), dtype=dtype)
    mixer = model.blocks[0].mixer
    torch.manual_seed(5)
    n = 90
    x = torch.randn(n, 56, dtype=F64)
    other = torch.randn(21, 56, dtype=F64)
    store = plain._keep if dtype == torch.float32 else plain.to_bfloat16_and_back
    want = fn(store(x), torch.arange(n), t, "l0.mix.", spec["mixer"], 1e-4, store)
    want_other = fn(store(other), torch.arange(21), t, "l0.mix.", spec["mixer"], 1e-4, store)
    tol = (2e-5 if dtype == torch.float32 else 3e-2) * want.abs().max().item()
    got = _run_mixer(runner, mixer, [("a", n, 0)], x, dtype)
    assert torch.allclose(got, want, atol=tol), (got - want).abs().max()
    first = _run_mixer(runner, mixer, [("b", 23, 0)], x[:23], dtype)
    second = _run_mixer(runner, mixer, [("b", n - 23, 23)], x[23:], dtype)
    assert torch.allclose(torch.cat([first, second]), want, atol=tol)
    if dtype == torch.float32:
        runner.release("a")
        runner.release("b")
        rows = []
        for p in range(n):
            if p == 30:      # another request's whole prompt beside the decoded token
                out = _run_mixer(runner, mixer, [("o", 21, 0), ("d", 1, p)], torch.cat([other, x[p:p + 1]]), dtype)
                assert torch.allclose(out[:21], want_other, atol=tol)
                rows.append(out[21:])
            else:
                rows.append(_run_mixer(runner, mixer, [("d", 1, p)], x[p:p + 1], dtype))
        assert torch.allclose(torch.cat(rows), want, atol=tol)


@pytest.mark.parametrize("c, stride", [(70, 70), (72, 96), (1100, 1100), (96, 100)])
@pytest.mark.parametrize("taps", [1, 2, 4, 7])
def test_convolution_without_its_input_on_columns_of_a_wider_tensor(taps, c, stride):
    """Runs of several requests in portions shorter and longer than the taps; a slot used again by another
    request; the input's rows further apart than the convolved channels."""
    from qwen25vl_lite_amd.ops.short_conv import short_conv
    torch.manual_seed(taps + c)
    w = torch.randn(c, taps)
    xs = {rid: torch.randn(n, c) for rid, n in (("p", 40), ("q", 11), ("r", 9))}
    want = {rid: plain.causal_conv(x.double(), w.double()) for rid, x in xs.items()}
    state = torch.zeros(3, taps - 1, c, device="cuda") if taps > 1 else None
    got = {rid: [] for rid in xs}
    slots = {"p": 0, "q": 1, "r": 1}
    sizes = {"p": [1, 2, 1, 5, 1, 1, 9, 3, 17], "q": [4, 1, 1, 5], "r": [9]}
    at = {rid: 0 for rid in xs}
    plan = [["p", "q"], ["q", "p"], ["p"], ["p", "q"], ["p", "q"], ["p"], ["p"], ["r", "p"], ["p"]]
    for live in plan:
        if "r" in live and state is not None:
            state[1].zero_()         # the runner clears a slot when a new request takes it
        runs = [(rid, sizes[rid].pop(0)) for rid in live]
        rows = torch.cat([xs[rid][at[rid]:at[rid] + n] for rid, n in runs])
        wide = torch.full((rows.shape[0], stride), 5.0)
        wide[:, :c] = rows
        cu = torch.tensor([0] + list(torch.tensor([n for _, n in runs]).cumsum(0)), dtype=torch.int32).cuda()
        req = torch.cat([torch.full((n,), i, dtype=torch.int32) for i, (_, n) in enumerate(runs)]).cuda()
        sl = torch.tensor([slots[rid] for rid, _ in runs], dtype=torch.int32).cuda()
        out = short_conv(wide.cuda()[:, :c], w.t().contiguous().cuda(), state, cu, sl, req, torch.float32).cpu()
        k = 0
        for rid, n in runs:
            got[rid].append(out[k:k + n])
            at[rid] += n
            k += n
    for rid in xs:
        assert torch.allclose(torch.cat(got[rid]).double(), want[rid], atol=1e-5), rid


@pytest.mark.parametrize("nq, nkv, hd", [(6, 2, 24), (3, 3, 10), (1, 1, 64), (40, 8, 128)])
def test_a_norm_over_the_whole_projection_then_rotation(nq, nkv, hd):
    """Queries of one token are normed together, its keys together, each with weights over all its channels;
    one head is made ten times larger than the rest, so a norm per head would give other values."""
    from qwen25vl_lite_amd.ops import gated
    torch.manual_seed(nq)
    n, ps, rot = 37, 16, (hd // 2) // 2 * 2
    x = torch.randn(n, (nq + 2 * nkv) * hd + 5)
    x[:, :hd] *= 10.0
    x[:, nq * hd:(nq + 1) * hd] *= 10.0
    qw, kw = 1 + 0.3 * torch.randn(nq * hd), 1 + 0.3 * torch.randn(nkv * hd)
    pos = torch.arange(100, 100 + n)
    f = plain.frequencies({"base": 50.0, "dims": rot})
    angle = pos.double()[:, None] * f[None, :]
    cs = torch.stack([angle.cos(), angle.sin()], dim=-1).float()
    slots = torch.randperm(4 * ps)[:n].to(torch.int32)
    k_cache = torch.zeros(4, nkv, ps, hd, device="cuda")
    v_cache = torch.zeros(4, nkv, hd, ps, device="cuda")
    q = gated.qk_norm_rope_write(x.cuda(), qw.cuda(), kw.cuda(), 1e-5, cs.cuda(), slots.cuda(), k_cache, v_cache, nq, nkv,
                                 hd, ps, torch.float32, interleaved=False, values_are_keys=False, norm="whole").cpu()
    xq, xk = x[:, :nq * hd].double(), x[:, nq * hd:(nq + nkv) * hd].double()
    want_q = plain.rotate((plain.unit_rms(xq, 1e-5) * qw.double()).view(n, nq, hd), pos, f, 1.0, "halves")
    want_k = plain.rotate((plain.unit_rms(xk, 1e-5) * kw.double()).view(n, nkv, hd), pos, f, 1.0, "halves")
    assert torch.allclose(q.double().view(n, nq, hd), want_q, atol=2e-5)
    got_k = k_cache.cpu()[slots.long() // ps, :, slots.long() % ps]
    got_v = v_cache.cpu()[slots.long() // ps, :, :, slots.long() % ps]
    assert torch.allclose(got_k.double(), want_k, atol=2e-5)
    assert torch.equal(got_v, x[:, (nq + nkv) * hd:(nq + 2 * nkv) * hd].view(n, nkv, hd))
    per_head = plain.unit_rms(xq.view(n, nq, hd), 1e-5)
    if nq > 1:
        assert not torch.allclose(plain.unit_rms(xq, 1e-5).view(n, nq, hd), per_head, atol=1e-2)


@pytest.mark.parametrize("width", [5, 72, 1000, 4100, 9000])
@pytest.mark.parametrize("pending", [None, "float32", "bfloat16", "slabs"])
def test_two_norms_of_one_sum_in_one_pass(width, pending):
    """What is pending and a vector for every row are folded into the sum, which is then normed once and written
    under two gains."""
    from qwen25vl_lite_amd.ops.gated import sandwich_norm
    torch.manual_seed(width)
    n = 11
    h = torch.randn(n, width) * 3 + 0.5
    vec = torch.randn(width)
    w1, w2 = 1 + 0.3 * torch.randn(width), 1 + 0.3 * torch.randn(width)
    y = None
    if pending == "slabs":
        y = torch.randn(3, n, width)
    elif pending is not None:
        y = torch.randn(n, width).to(getattr(torch, pending))
    total = h.double() + vec.double() + (0 if y is None else (y.double().sum(0) if y.dim() == 3 else y.double()))
    for out_dtype, tol in ((torch.float32, 1e-5), (torch.bfloat16, 2e-2)):
        hd = h.cuda()
        a, b = sandwich_norm(hd, None if y is None else y.cuda(), None, 0.0, 1.0, vec.cuda(), w1.cuda(), 1e-5, out_dtype,
                             weight2=w2.cuda())
        assert torch.allclose(hd.cpu().double(), total, atol=1e-5)
        unit = plain.unit_rms(total, 1e-5)
        assert torch.allclose(a.float().cpu().double(), unit * w1.double(), atol=tol, rtol=tol)
        assert torch.allclose(b.float().cpu().double(), unit * w2.double(), atol=tol, rtol=tol)


@pytest.mark.parametrize("dtype, width, ff", [(torch.float32, 56, 24), (torch.bfloat16, 64, 40), (torch.bfloat16, 56, 23),
                                             (torch.bfloat16, 128, 96)])
@pytest.mark.parametrize("rows", [3, 150, 700])
def test_routed_experts_with_a_router_bias_alone(dtype, width, ff, rows, tmp_path):
    """Few pairs an expert and many, with a shared expert; the bias decides some choices."""
    mlp = ru.moe(5, 2, ff, shared=ff + 8)
    lay = ru.layer(ru.attention(1, 1, 8, 8), mlp)
    runner, model, t = _one_layer(tmp_path, lay, dtype=dtype, width=width)
    torch.manual_seed(rows)
    x = torch.randn(rows, width, dtype=F64)
    store = plain._keep if dtype == torch.float32 else plain.to_bfloat16_and_back
    want = plain.moe_ff(store(x), t, "l0.mlp.", mlp, store)
    z = store(x) @ t["l0.mlp.router"].T
    with_bias, without = plain.route(z + t["l0.mlp.router.b"], 2)[0], plain.route(z, 2)[0]
    assert (with_bias.sort(-1).values != without.sort(-1).values).any()
    ffn = model.blocks[0].ffn
    got = ffn.forward(x.to(dtype).cuda(), SimpleNamespace(residual=None))
    got = (got.sum(0) if got.dim() == 3 else got).double().cpu()
    if dtype == torch.float32:
        ids, wts = ffn.route(x.float().cuda())
        idx, w = plain.route(z + t["l0.mlp.router.b"], 2)
        assert torch.equal(ids.cpu().long().sort(-1).values, idx.sort(-1).values)
        assert torch.allclose(wts.cpu().double().gather(1, ids.cpu().long().argsort(-1)), w.gather(1, idx.argsort(-1)), atol=1e-6)
        assert torch.allclose(got, want, atol=2e-5 * want.abs().max().item())
    else:
        err = (got - want).pow(2).mean(dim=1).sqrt() / want.pow(2).mean().sqrt()
        assert err.median() < 2e-2, err.median()     # single rows may choose another expert where logits all but tie


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("ff", [88, 27])
def test_dense_feed_forward_alone(dtype, ff, tmp_path):
    lay = ru.layer(ru.attention(1, 1, 8, 8), ru.dense(ff))
    runner, model, t = _one_layer(tmp_path, lay, dtype=dtype)
    torch.manual_seed(1)
    x = torch.randn(70, 56, dtype=F64)
    store = plain._keep if dtype == torch.float32 else plain.to_bfloat16_and_back
    want = plain.gated_ff(store(x), t, "l0.mlp.", store)
    got = model.blocks[0].ffn.forward(x.to(dtype).cuda(), SimpleNamespace(residual=None))
    got = (got.sum(0) if got.dim() == 3 else got).double().cpu()
    assert torch.allclose(got, want, atol=(2e-5 if dtype == torch.float32 else 3e-2) * want.abs().max().item())


def test_a_pass_starts_from_the_mixed_sum_and_its_vector(tmp_path):
    """One layer looped twice: after the model's step the residual sum equals the plain model's, whose passes
    start from ``Win [x; x0] + step_t``; with the embedding's half of ``Win`` zeroed the result changes."""
    lay = ru.layer(ru.attention(2, 1, 8, 12, base=50.0), ru.dense(24))
    runner, model, t = _one_layer(tmp_path, [lay], loop=(0, 1, 2))
    from qwen25vl_lite_amd.engine import StepEntry
    toks = random_tokens(19, 50, 2)
    captured = []
    block = model.blocks[0]
    inner = block.forward

    def spy(stream, step, slot):
        out = inner(stream, step, slot)
        h = out.h.clone()
        if out.pending is not None:
            p = out.pending.float()
            h += p.sum(0) if p.dim() == 3 else p
        captured.append(h.double().cpu())
        return out
    block.forward = spy
    runner.admit("a")
    runner.execute([StepEntry("a", toks, 0, want=[len(toks) - 1])])
    cfg, _ = plain.rofapel_read(str(tmp_path / "one"))
    trace = []
    plain.rofapel_forward(cfg, t, toks, trace=trace)
    assert len(captured) == len(trace) == 2
    for got, want in zip(captured, trace):
        assert torch.allclose(got, want, atol=2e-5 * want.abs().max().item())
    t2 = dict(t)
    t2["loop.in"] = t["loop.in"].clone()
    t2["loop.in"][:, 56:] = 0
    other = []
    plain.rofapel_forward(cfg, t2, toks, trace=other)
    assert not torch.allclose(other[1], trace[1], atol=1e-2)
    assert model.embedding.scale == 1.3
    first = model.embedding.forward(torch.tensor(toks, dtype=torch.int32).cuda(), None).double().cpu()
    assert torch.allclose(first, t["embed"][torch.tensor(toks)] * 1.3, atol=1e-6)


def test_one_key_just_inside_and_just_outside_a_window_and_the_sink(tmp_path):
    """Window 8.  Token 5's key is made to stand out through its input: queries 5 .. 12 see it and none after.
    Token by token through the cache the same.  A very large sink takes all the weight: the output vanishes."""
    spec = ru.attention_2(2, 1, 16, mask=8, conv=2, base=50.0, scale=0.25, factor=2.0)
    m = spec["mixer"]
    runner, model, t = _one_layer(tmp_path, ru.layer(spec))
    mixer = model.blocks[0].mixer
    torch.manual_seed(7)
    n = 40
    x = torch.randn(n, 56, dtype=F64) * 0.1
    x[5] *= 200.0
    want = plain.attention_2(x, torch.arange(n), t, "l0.mix.", m, 1e-4)
    m7 = copy.deepcopy(m)
    m7["mask"]["size"] = 7
    assert not torch.allclose(plain.attention_2(x, torch.arange(n), t, "l0.mix.", m7, 1e-4)[12], want[12],
                              atol=1e-2 * want.abs().max().item())          # a window one token short shows at query 12
    tol = 2e-5 * want.abs().max().item()
    assert torch.allclose(_run_mixer(runner, mixer, [("a", n, 0)], x, torch.float32), want, atol=tol)
    runner.release("a")
    rows = [_run_mixer(runner, mixer, [("d", 1, p)], x[p:p + 1], torch.float32) for p in range(n)]
    assert torch.allclose(torch.cat(rows), want, atol=tol)
    mixer.sink.fill_(60.0)
    runner.release("d")
    assert _run_mixer(runner, mixer, [("z", n, 0)], x, torch.float32).abs().max() < 1e-6 * want.abs().max()


# ---------------------------------------------------------------------------------------------
# whole models, every schedule
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("name", ["mixed", "ones", "odd", "tail_loop", "crossed", "no_rotation"])
def test_float32_every_schedule_against_the_plain_model(name, folders):
    """Whole prompts, decoded tails, portions down to two tokens, mixed batches with more requests
    than slots: all the same logits, and the plain model's."""
    folder = folders[name]
    cfg, _ = plain.rofapel_read(folder, F64)
    reqs = _requests(cfg["vocab"], seed=20)
    want = {rid: _oracle(folder, toks) for rid, toks in reqs.items()}
    mixed, peak = mixed_trace(reqs, seed=4, max_live=4)
    holders = {}
    for steps, size in ((whole_trace(reqs), 128), (tail_trace(reqs, 50), 128), (portion_trace(reqs), 128), (mixed, peak)):
        got = run_steps(_replayer(folder, "float32", size), steps, holders if steps is mixed else None)
        for rid, toks in reqs.items():
            assert _rel(_rows(got, rid, len(toks)), want[rid]) < 2e-5, (name, rid)
    assert any(len(who) > 1 for who in holders.values()), "no page was used by two requests"


@pytest.mark.parametrize("name", ["mixed", "ones", "odd"])
def test_bfloat16_within_rounding_of_the_plain_model(name, folders):
    """bfloat16 kernels: no further from exact arithmetic than rounding the stored activations to
    bfloat16 takes the plain model, whatever the schedule."""
    folder = folders[name]
    cfg, _ = plain.rofapel_read(folder, F64)
    reqs = _requests(cfg["vocab"], seed=30)
    exact = {rid: _oracle(folder, toks) for rid, toks in reqs.items()}
    rounding = torch.cat([_rel_rows(_oracle(folder, toks, plain.to_bfloat16_and_back), exact[rid])
                          for rid, toks in reqs.items()])
    mixed, peak = mixed_trace(reqs, seed=5, max_live=4)
    for steps, size in ((whole_trace(reqs), 128), (tail_trace(reqs, 50), 128), (portion_trace(reqs), 128), (mixed, peak)):
        got = run_steps(_replayer(folder, "bfloat16", size), steps)
        errors = torch.cat([_rel_rows(_rows(got, rid, len(toks)), exact[rid]) for rid, toks in reqs.items()])
        assert _like_rounding(errors, rounding), (name, errors.median(), rounding.median(), errors.quantile(0.9),
                                                  rounding.quantile(0.9))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_peaked_attention_at_window_edges_and_far_keys(dtype, folders):
    """Score scales so large that the softmax picks single keys: in the layers that see everything, hundreds
    of tokens back and across page borders; in the windowed ones, right at the window's edge.  The last 70
    tokens are decoded, so both windows (9, 37) pass over decoded tokens; then the same in portions."""
    folder = folders["sharp"]
    toks = random_tokens(330, ru.SHARP["vocab"], 40)
    want = _oracle(folder, toks)
    if dtype == "float32":
        # scores this large make float32 arithmetic itself visible: the measure is the plain model run in float32
        cfg, t32 = plain.rofapel_read(folder, torch.float32)
        rounding, slack = _rel_rows(plain.rofapel_forward(cfg, t32, toks), want), 1e-5
    else:
        rounding, slack = _rel_rows(_oracle(folder, toks, plain.to_bfloat16_and_back), want), 1e-3
    for steps in (tail_trace({"s": toks}, 70), portion_trace({"s": toks}, (64, 3, 41, 2, 17, 90))):
        got = _rows(run_steps(_replayer(folder, dtype, round64(len(toks))), steps), "s", len(toks))
        errors = _rel_rows(got, want)
        assert _like_rounding(errors, rounding, slack), (errors.median(), rounding.median(), errors.quantile(0.9),
                                                         rounding.quantile(0.9))
        assert errors.max() < 4 * rounding.max() + slack, (errors.max(), rounding.max())


def test_sharpening_matters(folders):
    """The test above would see a window that is one token off, a lost far key, a sink left out, a norm per
    head in place of the whole projection's or the other pairing of rotated channels: each changes the plain
    model's last logits."""
    toks = random_tokens(330, ru.SHARP["vocab"], 40)
    whole = _oracle(folders["sharp"], toks)[-30:]

    def one_off(cfg):
        for lay in cfg["layers"]:
            if lay["mixer"].get("mask"):
                lay["mixer"]["mask"]["size"] -= 1

    def no_sink(t):
        for name in t:
            if name.endswith(".sink"):
                t[name] = torch.full_like(t[name], -1e4)

    assert _rel(_oracle(folders["sharp"], toks, cfg_edit=one_off)[-30:], whole) > 0.02
    assert _rel(_oracle(folders["sharp"], toks, tensors_edit=no_sink)[-30:], whole) > 0.02
    # the far past: the same sequence with its first 200 tokens replaced
    other = random_tokens(200, ru.SHARP["vocab"], 41) + toks[200:]
    assert _rel(_oracle(folders["sharp"], other)[-30:], whole) > 0.02


def test_long_decoding(folders):
    """A short prompt and 200 tokens decoded one by one, through several pages, windows moving on."""
    folder = folders["mixed"]
    toks = random_tokens(205, ru.MIXED["vocab"], 50)
    want = _oracle(folder, toks)
    got = _rows(run_steps(_replayer(folder, "float32", 256), tail_trace({"l": toks}, 200)), "l", len(toks))
    assert _rel(got, want) < 2e-5


def test_windowed_groups_give_pages_back_while_decoding(folders):
    from qwen25vl_lite_amd.engine.replay import Replayer
    rp = Replayer(folders["mixed"], "float32", 256, 16, 2)
    toks = random_tokens(200, ru.MIXED["vocab"], 51)
    run_steps(rp, [{"step": 0, "entries": [{"id": "x", "tokens": toks, "want": []}], "end": []}])
    cache = rp.runner.cache
    held = {(g.need.window, g.need.head_dim): sum(p >= 0 for p in cache.table("x", i)) for i, g in enumerate(cache.groups)}
    # a window of 9 keys lies in one or two pages, one of 37 in three or four; the other groups keep all 13
    assert held[(9, 16)] <= 2 and held[(37, 24)] <= 4
    assert all(n == 13 for (window, _), n in held.items() if window is None)
    rp.step({"entries": [], "end": ["x"]})
    cache.check()


@pytest.mark.parametrize("graph", [False, True])
def test_greedy_generation_through_the_entry_point(graph, folders):
    """``LLM.generate`` with the scheduler (three prompts, two slots, portions of 16 tokens, decode
    steps from HIP graphs or not) picks the plain model's tokens."""
    from qwen25vl_lite_amd import LLM, SamplingParams
    folder = folders["mixed"]
    prompts = [random_tokens(n, ru.MIXED["vocab"], 70 + n) for n in (37, 5, 21)]
    steps = 12
    want = []
    for p in prompts:
        ids = list(p)
        for _ in range(steps):
            ids.append(int(torch.argmax(_oracle(folder, ids)[-1])))
        want.append(ids[len(p):])
    with LLM(folder, dtype="float32", num_blocks=32, block_size=16, max_num_seqs=2, max_num_batched_tokens=16,
             hip_graph=graph) as llm:
        outs = llm.generate(prompts, SamplingParams(temperature=0.0, max_tokens=steps, ignore_eos=True))
    assert [o.output_token_ids for o in outs] == want


@pytest.mark.parametrize("dtype, tol", [("float32", 2e-5), ("bfloat16", 5e-2)])
def test_the_replay_program_and_the_command_line(dtype, tol, folders, tmp_path):
    """``bin/trace_run`` as a user calls it on a Rofapel folder (steps on standard input, ``done`` lines, files of
    float32 logits), and ``generate`` of the command line, whose tokens are the plain model's."""
    import ast
    import json
    import os
    import subprocess
    import sys

    import numpy as np
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    folder = folders["mixed"]
    vocab = ru.MIXED["vocab"]
    toks = random_tokens(45, vocab, 4)
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": toks[:19], "want": [0, 18]}], "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": toks[19:44], "want": []}], "end": []},
        {"step": 2, "entries": [{"id": "a", "tokens": toks[44:], "want": [0]},
                                {"id": "b", "tokens": toks[:3], "want": [2]}], "end": ["a", "b"]},
    ]
    out = tmp_path / "out"
    proc = subprocess.run(
        [sys.executable, os.path.join(root, "bin", "trace_run"), "--model", folder, "--dtype", dtype, "--out", str(out),
         "--max-tokens", "128"],
        input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=110)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [w for w in proc.stdout.split() if w == "done" or w.isdigit()][-6:] == ["done", "0", "done", "1", "done", "2"]
    assert sorted(os.listdir(out)) == ["0.f32", "2.f32"]
    want = _oracle(folder, toks)
    s0 = torch.from_numpy(np.fromfile(out / "0.f32", dtype="<f4").reshape(2, vocab))
    s2 = torch.from_numpy(np.fromfile(out / "2.f32", dtype="<f4").reshape(2, vocab))
    assert _rel(torch.cat([s0, s2]), want[[0, 18, 44, 2]]) < tol
    if dtype == "float32":
        prompt = toks[:12]
        cli = [sys.executable, os.path.join(root, "bin", "qwen25vl-lite"), "generate", "--model", folder, "--dtype", "float32",
               "--num-blocks", "32", "--max-num-seqs", "2", "--max-model-len", "256", "--max-tokens", "6", "--ignore-eos",
               "--prompt-token-ids", ",".join(map(str, prompt))]
        proc = subprocess.run(cli, capture_output=True, text=True, timeout=110)
        assert proc.returncode == 0, proc.stderr[-2000:]
        ids = list(prompt)
        for _ in range(6):
            ids.append(int(torch.argmax(_oracle(folder, ids)[-1])))
        assert ast.literal_eval(proc.stdout.strip().splitlines()[-1]) == ids[len(prompt):]


def test_bfloat16_generation_from_graphs_matches_eager_steps(folders):
    from qwen25vl_lite_amd import LLM, SamplingParams
    prompts = [random_tokens(n, ru.MIXED["vocab"], 90 + n) for n in (18, 3, 40, 9)]
    outs = []
    for graph in (False, True):
        with LLM(folders["mixed"], dtype="bfloat16", num_blocks=48, block_size=16, max_num_seqs=4,
                 max_num_batched_tokens=64, hip_graph=graph) as llm:
            outs.append([o.output_token_ids for o in
                         llm.generate(prompts, SamplingParams(temperature=0.0, max_tokens=10, ignore_eos=True))])
    assert outs[0] == outs[1]
