"""The Rapisun decoder on the GPU against the plain implementation in ``plain_rapisun.py``: each
mechanism alone, whole prompts, decoding, portions, mixed batches, pages and slots used again, peaked
attention at the edges of windows and far back, a slow channel of the recurrence that remembers a far
token, sizes that are 1, equal or odd, and greedy generation through ``LLM``."""

import copy

import pytest
import torch

import plain_rapisun as plain
import rapisun_util as ru
from replay_util import mixed_trace, portion_trace, random_tokens, round64, run_steps, tail_trace, whole_trace

pytestmark = pytest.mark.gpu

F64 = torch.float64
LENGTHS = {"a": 83, "b": 40, "c": 7, "d": 1, "e": 118, "f": 29, "g": 2}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    out = {}
    for name, cfg, seed in (("mixed", ru.MIXED, 31), ("sharp", ru.SHARP, 32), ("ones", ru.ONES, 33), ("odd", ru.ODD, 34),
                            ("no_conv", ru.NO_CONV, 35)):
        out[name] = ru.write_model(str(tmp_path_factory.mktemp(name)), cfg, seed)
    return out


def _oracle(folder, tokens, store=None, cfg_edit=None, tensors_edit=None):
    cfg, tensors = plain.rapisun_read(folder, F64)
    if cfg_edit is not None:
        cfg_edit(cfg)
    if tensors_edit is not None:
        tensors_edit(tensors)
    return plain.rapisun_forward(cfg, tensors, tokens, store or plain._keep).to(torch.float32)


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
    rows far (a router's choice between two experts whose scores all but tie falls the other way), in the
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
def _one_layer(tmp_path, lay, dtype=torch.float32, seed=0, width=56, taps=3, tensors_edit=None, name="one"):
    from qwen25vl_lite_amd.config import EngineConfig, load_config
    from qwen25vl_lite_amd.engine import ModelRunner
    from qwen25vl_lite_amd.models import build_model
    from qwen25vl_lite_amd.weights import load_weights
    cfg = ru.config(width, 50, lay if isinstance(lay, list) else [lay], eps=1e-4, taps=taps)
    tensors = ru.random_tensors(cfg, seed)
    if tensors_edit is not None:
        tensors_edit(tensors)
    d = ru.write_model(str(tmp_path / name), cfg, seed, tensors)
    model = build_model(load_config(d), dtype, "cuda:0")
    load_weights(d, model)
    ecfg = EngineConfig(num_blocks=32, block_size=16, max_num_seqs=3, max_num_batched_tokens=512, max_model_len=512,
                        enable_prefix_cache=False, dtype=dtype)
    _, t64 = plain.rapisun_read(d, F64)
    return ModelRunner(model, ecfg), model.blocks, t64


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


@pytest.mark.parametrize("width", [5, 72, 1000, 9000, 20000, 33002])
@pytest.mark.parametrize("ydtype", [torch.float32, torch.bfloat16])
def test_layer_norm_adds_into_the_sum(width, ydtype):
    from qwen25vl_lite_amd.ops import rownorm
    torch.manual_seed(width)
    n = 13
    h = torch.randn(n, width, dtype=torch.float32) * 3 + 1.5
    y = (torch.randn(n, width) * 2 + 0.7).to(ydtype)
    w = 1 + 0.3 * torch.randn(width)
    want = h.double() + plain.layer_norm(y.double(), w.double(), 1e-5)
    hd = h.cuda()
    copy_ = rownorm.layer_norm_add_(hd, y.cuda(), w.cuda(), 1e-5, torch.bfloat16)
    assert torch.allclose(hd.cpu().double(), want, atol=1e-5, rtol=1e-5)
    assert torch.equal(copy_.cpu(), hd.cpu().to(torch.bfloat16))
    # float32 slabs are added in order before the norm
    slabs = torch.randn(3, n, width)
    want = h.double() + plain.layer_norm(slabs.double().sum(0), w.double(), 1e-5)
    hd = h.cuda()
    rownorm.layer_norm_add_(hd, slabs.cuda(), w.cuda(), 1e-5)
    assert torch.allclose(hd.cpu().double(), want, atol=2e-5, rtol=1e-5)
    # chosen rows of the sum, normed
    rows = torch.tensor([7, 0, 12], dtype=torch.int32)
    out = rownorm.layer_norm(h.cuda(), w.cuda(), 1e-5, torch.float32, rows=rows.cuda())
    assert torch.allclose(out.cpu().double(), plain.layer_norm(h.double()[rows.long()], w.double(), 1e-5), atol=1e-5)


@pytest.mark.parametrize("inter", [3, 88, 2048, 8200, 18960, 33000])
def test_normed_powers(inter):
    from qwen25vl_lite_amd.ops import rownorm
    torch.manual_seed(inter)
    z = torch.randn(9, inter) * 1.7
    coeff = torch.tensor([0.6, -0.4, 0.3, 0.2])
    want = plain.poly_norm(z.double(), coeff.double(), 1e-5)
    got = rownorm.normed_powers(z.cuda(), coeff.cuda(), 1e-5, torch.float32).cpu().double()
    assert torch.allclose(got, want, atol=1e-5, rtol=1e-5)
    zb = z.to(torch.bfloat16)
    got = rownorm.normed_powers(zb.cuda(), coeff.cuda(), 1e-5, torch.bfloat16).cpu().double()
    want = plain.poly_norm(zb.double(), coeff.double(), 1e-5)
    assert torch.allclose(got, want, atol=2e-2, rtol=1e-2)


@pytest.mark.parametrize("c", [70, 72, 1100])
@pytest.mark.parametrize("taps", [1, 2, 4, 7])
def test_short_convolution_across_steps_and_requests(taps, c, tmp_path):
    """One run of 40 tokens against the same tokens in portions (1, 2, 1, 5, ... tokens: shorter and longer than
    the taps) beside another request whose slot is then used again by a third."""
    from qwen25vl_lite_amd.ops.short_conv import short_conv_add
    torch.manual_seed(taps)
    w = torch.randn(c, taps)
    xs = {rid: torch.randn(n, c) for rid, n in (("p", 40), ("q", 11), ("r", 9))}
    want = {rid: (x.double() + plain.causal_conv(x.double(), w.double())) for rid, x in xs.items()}
    state = torch.zeros(3, max(taps - 1, 0), c, device="cuda") if taps > 1 else None
    if state is not None:
        state[1].fill_(9.0)      # the slot "q" gets was used before: the runner clears it at admission
        state[1].zero_()
    got = {rid: [] for rid in xs}
    slots = {"p": 0, "q": 1, "r": 1}
    sizes = {"p": [1, 2, 1, 5, 1, 1, 9, 3, 17], "q": [4, 1, 1, 5], "r": [9]}
    at = {rid: 0 for rid in xs}
    plan = [["p", "q"], ["q", "p"], ["p"], ["p", "q"], ["p", "q"], ["p"], ["p"], ["r", "p"], ["p"]]
    for live in plan:
        if "r" in live and state is not None:
            state[1].zero_()
        runs = [(rid, sizes[rid].pop(0)) for rid in live]
        x = torch.cat([xs[rid][at[rid]:at[rid] + n] for rid, n in runs]).cuda()
        cu = torch.tensor([0] + list(torch.tensor([n for _, n in runs]).cumsum(0)), dtype=torch.int32).cuda()
        req = torch.cat([torch.full((n,), i, dtype=torch.int32) for i, (_, n) in enumerate(runs)]).cuda()
        sl = torch.tensor([slots[rid] for rid, _ in runs], dtype=torch.int32).cuda()
        out = short_conv_add(x, w.t().contiguous().cuda(), state, cu, sl, req, torch.float32).cpu()
        k = 0
        for rid, n in runs:
            got[rid].append(out[k:k + n])
            at[rid] += n
            k += n
    for rid in xs:
        assert torch.allclose(torch.cat(got[rid]).double(), want[rid], atol=1e-5), rid


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads, dim, vdim", [(3, 12, 20), (1, 5, 7), (2, 64, 48)])
def test_hgrn2_alone_whole_in_steps_and_in_chunks(heads, dim, vdim, dtype, tmp_path):
    """A run long enough for the chunked scan, the same in steps of 1 to 150 tokens, beside a second request."""
    runner, blocks, t = _one_layer(tmp_path, ru.layer(ru.hgrn2(heads, dim, vdim)), dtype=dtype)
    mixer = blocks[0].mixer
    torch.manual_seed(3)
    n = 300
    x = torch.randn(n, 56, dtype=F64)
    other = torch.randn(33, 56, dtype=F64)
    store = plain._keep if dtype == torch.float32 else plain.to_bfloat16_and_back
    want = plain.hgrn2(store(x), t, "l0.mix.", ru.hgrn2(heads, dim, vdim)["mixer"], 1e-4, store)
    want_other = plain.hgrn2(store(other), t, "l0.mix.", ru.hgrn2(heads, dim, vdim)["mixer"], 1e-4, store)
    tol = (2e-5 if dtype == torch.float32 else 3e-2) * want.abs().max().item()

    def run(runs, xs):
        step = _step_for(runner, runs)
        out = mixer.forward(torch.cat(xs).to(dtype).cuda(), step, runner.slots[0].by_part["mix"])
        _commit(runner, runs)
        if out.dim() == 3:
            out = out.sum(0)
        return out.double().cpu()

    got = run([("w", n, 0)], [x])
    assert torch.allclose(got, want, atol=tol), (got - want).abs().max()
    runner.release("w")
    pieces, at = [], 0
    for k, size in enumerate((1, 1, 2, 150, 3, 1, 64, 70, 8)):
        if k == 3:     # the long portion runs beside the whole of another request
            out = run([("o", 33, 0), ("s", size, at)], [other, x[at:at + size]])
            assert torch.allclose(out[:33], want_other, atol=tol)
            out = out[33:]
        else:
            out = run([("s", size, at)], [x[at:at + size]])
        pieces.append(out)
        at += size
    assert at == n
    assert torch.allclose(torch.cat(pieces), want, atol=tol)


def test_a_slow_channel_remembers_a_far_token(tmp_path):
    """One key channel of the recurrence is made to forget almost nothing (a floor of 0.98) and is the only one
    the late queries read: what token 3 wrote is still there 250 tokens on, and a state lost on the way
    (a slot cleared, a chunk's carry dropped) would show."""
    heads, dim, vdim = 2, 8, 8

    def edit(t):
        low = torch.full((heads * dim,), 0.05)
        low[::dim] = 0.98                       # the first channel of every head
        t["l0.mix.lower"] = low.to(torch.bfloat16)
        gate, bias = t["l0.mix.f"].clone(), t["l0.mix.f.b"].clone()
        gate[::dim] = 0                         # its gate stands at the floor plus half the rest, whatever the token
        bias[::dim] = 0
        t["l0.mix.f"], t["l0.mix.f.b"] = gate, bias
        q = t["l0.mix.q"].clone()
        keep = torch.zeros(heads * dim, 1, dtype=q.dtype)
        keep[::dim] = 1
        t["l0.mix.q"] = q * keep                # queries read that channel only
    runner, blocks, t = _one_layer(tmp_path, ru.layer(ru.hgrn2(heads, dim, vdim)), tensors_edit=edit)
    mixer = blocks[0].mixer
    torch.manual_seed(9)
    n = 260
    x = torch.randn(n, 56, dtype=F64)
    x[3] *= 30.0                                # a token that writes much
    m = ru.hgrn2(heads, dim, vdim)["mixer"]
    want = plain.hgrn2(x, t, "l0.mix.", m, 1e-4)
    x2 = x.clone()
    x2[3] = -x[3]
    moved = plain.hgrn2(x2, t, "l0.mix.", m, 1e-4)
    assert (moved[-5:] - want[-5:]).abs().max() > 1e-2 * want.abs().max()    # the far token matters to the end
    pieces, at = [], 0
    for size in (5, 140, 1, 1, 100, 13):
        step = _step_for(runner, [("s", size, at)])
        out = mixer.forward(x[at:at + size].float().cuda(), step, runner.slots[0].by_part["mix"])
        _commit(runner, [("s", size, at)])
        pieces.append((out.sum(0) if out.dim() == 3 else out).double().cpu())
        at += size
    assert torch.allclose(torch.cat(pieces), want, atol=2e-5 * want.abs().max().item())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("mask", [None, 7, 70, 1])
def test_latent_attention_alone_whole_and_in_two_steps(mask, dtype, tmp_path):
    spec = ru.latent(3, 16, 8, 24, 40, 24, base=300.0, scale=0.9, mask=mask)
    m = spec["mixer"]
    runner, blocks, t = _one_layer(tmp_path, ru.layer(spec), dtype=dtype)
    mixer = blocks[0].mixer
    torch.manual_seed(5)
    n = 90
    x = torch.randn(n, 56, dtype=F64)
    store = plain._keep if dtype == torch.float32 else plain.to_bfloat16_and_back
    pos = torch.arange(n)
    want = plain.latent_attention(store(x), pos, t, "l0.mix.", m, 1e-4,
                                  plain.latent_cache(store(x), pos, t, "l0.mix.", m, 1e-4, store), store)
    tol = (2e-5 if dtype == torch.float32 else 3e-2) * want.abs().max().item()

    def run(runs, xs):
        step = _step_for(runner, runs)
        out = mixer.forward(xs.to(dtype).cuda(), step, runner.slots[0].by_part["mix"])
        _commit(runner, runs)
        return (out.sum(0) if out.dim() == 3 else out).double().cpu()

    got = run([("a", n, 0)], x)
    assert torch.allclose(got, want, atol=tol), (got - want).abs().max()
    # the same tokens in two steps, cut inside a page: the second step reads the pages of the first
    first = run([("b", 23, 0)], x[:23])
    second = run([("b", n - 23, 23)], x[23:])
    assert torch.allclose(torch.cat([first, second]), want, atol=tol)


def test_one_key_just_inside_and_just_outside_a_window_and_the_sink(tmp_path):
    """Window 8.  The latent of token 5 is made huge through its input: a query sees it while the token is
    within the window (queries 5 .. 12) and never after.  A very large sink takes all the weight: the
    output vanishes."""
    spec = ru.latent(2, 16, 8, 16, 24, 16, base=50.0, scale=0.25, mask=8)
    m = spec["mixer"]
    runner, blocks, t = _one_layer(tmp_path, ru.layer(spec))
    mixer = blocks[0].mixer
    torch.manual_seed(7)
    n = 40
    x = torch.randn(n, 56, dtype=F64) * 0.1
    x[5] *= 200.0
    pos = torch.arange(n)
    want = plain.latent_attention(x, pos, t, "l0.mix.", m, 1e-4, plain.latent_cache(x, pos, t, "l0.mix.", m, 1e-4))
    step = _step_for(runner, [("a", n, 0)])
    got = mixer.forward(x.float().cuda(), step, runner.slots[0].by_part["mix"]).double().cpu()
    assert torch.allclose(got, want, atol=2e-5 * want.abs().max().item())
    # token by token through the cache
    runner.release("a")
    rows = []
    for p in range(n):
        step = _step_for(runner, [("d", 1, p)])
        rows.append(mixer.forward(x[p:p + 1].float().cuda(), step, runner.slots[0].by_part["mix"]).double().cpu())
        _commit(runner, [("d", 1, p)])
    assert torch.allclose(torch.cat(rows), want, atol=2e-5 * want.abs().max().item())
    # the sink
    mixer.sink.fill_(60.0)
    runner.release("d")
    step = _step_for(runner, [("z", n, 0)])
    assert mixer.forward(x.float().cuda(), step, runner.slots[0].by_part["mix"]).abs().max() < 1e-6 * want.abs().max()


def test_a_layer_that_reads_another_layers_cache_with_a_longer_window(tmp_path):
    """Layer 0 sees 5 keys and owns the cache; layer 1 reads it and sees 40: the pages stay for the longer of
    the two, through decoding."""
    lays = [ru.layer(ru.latent(2, 8, 8, 8, 16, 16, base=30.0, scale=1.5, mask=5)),
            ru.layer(ru.latent(3, 16, 8, 8, 24, 16, base=30.0, scale=1.5, mask=40, kv_from=0))]
    cfg = ru.config(56, 50, lays, eps=1e-4, taps=2)
    d = ru.write_model(str(tmp_path / "two"), cfg, 11)
    toks = random_tokens(120, 50, 3)
    want = _oracle(d, toks)
    rp = _replayer(d, "float32", 128)
    got = _rows(run_steps(rp, tail_trace({"t": toks}, 60)), "t", len(toks))
    assert _rel(got, want) < 2e-5
    assert [g.need.window for g in rp.runner.cache.groups] == [40]


@pytest.mark.parametrize("e, top", [(8, 3), (6, 2), (1, 1), (9, 9), (64, 6), (5, 1)])
def test_softmax_router(e, top):
    from qwen25vl_lite_amd.ops import moe as moe_ops
    torch.manual_seed(e)
    z = torch.randn(50, e) * 2
    idx, w = plain.route(z.double(), torch.eye(e, dtype=F64), top)      # an identity router: the logits are z
    ids, wts = moe_ops.route(z.cuda(), top, 1, 1, 1.0, "softmax", True, 1e-20)
    assert torch.equal(ids.cpu().long().sort(dim=-1).values, idx.sort(dim=-1).values)
    order = ids.cpu().long().argsort(dim=-1)
    assert torch.allclose(wts.cpu().double().gather(1, order), w.gather(1, idx.argsort(dim=-1)), atol=1e-6)


@pytest.mark.parametrize("dtype, heads, k, r", [(torch.float32, 3, 12, 20), (torch.bfloat16, 5, 24, 40), (torch.bfloat16, 28, 128, 192),
                                               (torch.bfloat16, 2, 64, 96), (torch.bfloat16, 3, 20, 7)])
@pytest.mark.parametrize("rows", [1, 9, 70, 300])
def test_a_product_per_head_on_slices_of_rows(dtype, heads, k, r, rows):
    """``out[n, h, :r] = x[n, h, :k] @ w[h].T`` where a head's slice is part of a longer row, on both sides:
    what lies beside the slices stays as it was."""
    from qwen25vl_lite_amd.ops import moe as moe_ops
    torch.manual_seed(rows + heads)
    x = torch.randn(rows, heads, k + 8).to(dtype).cuda()
    w = (torch.randn(heads, r, k) / k ** 0.5).to(dtype).cuda()
    out = torch.full((rows, heads, r + 16), 7.0, dtype=dtype, device="cuda")
    order, offsets = moe_ops.pairs_by_column(rows, heads, "cuda")
    moe_ops.expert_products(x.view(rows * heads, k + 8)[:, :k], w, order, offsets, rows * heads, 1, dtype,
                            out=out.view(rows * heads, r + 16)[:, :r])
    want = torch.einsum("nhk,hrk->nhr", x[:, :, :k].double(), w.double())
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    assert (out[:, :, :r].double() - want).abs().max() < tol * max(1.0, want.abs().max().item())
    assert torch.all(out[:, :, r:] == 7.0)
    # and into a tensor of its own
    y = moe_ops.expert_products(x.view(rows * heads, k + 8)[:, :k], w, order, offsets, rows * heads, 1, dtype)
    assert y.is_contiguous() and torch.equal(y.view(rows, heads, r), out[:, :, :r])


@pytest.mark.parametrize("dtype, width, ff", [(torch.float32, 56, 24), (torch.bfloat16, 64, 40), (torch.bfloat16, 56, 24),
                                             (torch.bfloat16, 128, 96)])
@pytest.mark.parametrize("rows", [3, 150, 700])
def test_squared_relu_experts_alone(dtype, width, ff, rows, tmp_path):
    """Few pairs an expert and many (the matrix-core kernels with and without tiles through LDS), with a
    shared expert."""
    mlp = ru.moe(5, 2, ff, shared=ff + 8)
    lay = ru.layer(ru.hgrn2(1, 8, 8), mlp)
    runner, blocks, t = _one_layer(tmp_path, lay, dtype=dtype, width=width)
    torch.manual_seed(rows)
    x = torch.randn(rows, width, dtype=F64)
    store = plain._keep if dtype == torch.float32 else plain.to_bfloat16_and_back
    want = plain.moe_ff(store(x), t, "l0.mlp.", mlp, store)
    from types import SimpleNamespace
    got = blocks[0].ffn.forward(x.to(dtype).cuda(), SimpleNamespace(residual=None))
    got = (got.sum(0) if got.dim() == 3 else got).double().cpu()
    if dtype == torch.float32:
        assert torch.allclose(got, want, atol=2e-5 * want.abs().max().item())
    else:
        err = (got - want).pow(2).mean(dim=1).sqrt() / want.pow(2).mean().sqrt()
        assert err.median() < 2e-2, err.median()     # single rows may choose another expert where scores all but tie


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_dense_feed_forward_alone(dtype, tmp_path):
    lay = ru.layer(ru.hgrn2(1, 8, 8), ru.dense(88))
    runner, blocks, t = _one_layer(tmp_path, lay, dtype=dtype)
    torch.manual_seed(1)
    x = torch.randn(70, 56, dtype=F64)
    store = plain._keep if dtype == torch.float32 else plain.to_bfloat16_and_back
    want = plain.dense_ff(store(x), t, "l0.mlp.", 1e-4, store)
    step = _step_for(runner, [("a", 70, 0)])
    got = blocks[0].ffn.forward(x.to(dtype).cuda(), step)
    got = (got.sum(0) if got.dim() == 3 else got).double().cpu()
    assert torch.allclose(got, want, atol=(2e-5 if dtype == torch.float32 else 3e-2) * want.abs().max().item())


# ---------------------------------------------------------------------------------------------
# the attention kernels with a sink, against dense masked attention
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("hd, vd, nq, ps", [(32, 24, 3, 16), (128, 64, 7, 16), (64, 32, 20, 16), (40, 24, 5, 16)])
@pytest.mark.parametrize("window", [9, 37, 70, None])
def test_attention_with_a_sink_on_the_matrix_cores(hd, vd, nq, ps, window):
    """One key/value head whose values are the first channels of its keys, as the latent attention keeps them:
    prompt portions and decoded tokens, both forms of the kernel, and the float32-arithmetic kernel."""
    from types import SimpleNamespace
    from qwen25vl_lite_amd.ops import attention_window, kernels
    torch.manual_seed(hd + (window or 0))
    runs = [(70, 70), (1, 55), (23, 100), (1, 1), (2, 130)]         # (tokens of the step, context after it)
    pages_per = [(ctx + ps - 1) // ps for _, ctx in runs]
    table = torch.full((len(runs), max(pages_per)), -1, dtype=torch.int32)
    perm = torch.randperm(sum(pages_per) + 3)
    k_cache = torch.zeros(sum(pages_per) + 3, 1, ps, hd)
    v_cache = torch.zeros(sum(pages_per) + 3, 1, vd, ps)
    keys, at = [], 0
    for r, (_, ctx) in enumerate(runs):
        k = torch.randn(ctx, hd)
        keys.append(k)
        for i in range(pages_per[r]):
            page = int(perm[at]); at += 1
            table[r, i] = page
            chunk = k[i * ps:(i + 1) * ps]
            k_cache[page, 0, :chunk.shape[0]] = chunk
            v_cache[page, 0, :, :chunk.shape[0]] = chunk[:, :vd].T
    sinks = torch.randn(nq) * 2
    n = sum(q for q, _ in runs)
    q = torch.randn(n, nq * hd)
    cu = [0]
    for qn, _ in runs:
        cu.append(cu[-1] + qn)
    token_req = torch.cat([torch.full((qn,), r, dtype=torch.int32) for r, (qn, _) in enumerate(runs)])
    token_pos = torch.cat([torch.arange(ctx - qn, ctx, dtype=torch.int32) for qn, ctx in runs])
    scale = 0.3

    def dense(qq, kk, vv_dim, dt):
        out = torch.zeros(n, nq, vv_dim, dtype=F64)
        for r, (qn, ctx) in enumerate(runs):
            kr = kk[r].to(dt).double()
            for i in range(qn):
                p = ctx - qn + i
                lo = max(0, p - window + 1) if window else 0
                for h in range(nq):
                    s = (kr[lo:p + 1] @ qq[cu[r] + i].to(dt).double().view(nq, hd)[h]) * scale
                    top = max(s.max().item(), sinks[h].item())
                    e = torch.exp(s - top)
                    w = e / (e.sum() + torch.exp(sinks[h].double() - top))
                    out[cu[r] + i, h] = w @ kr[lo:p + 1, :vv_dim]
        return out.view(n, nq * vv_dim)

    want32 = dense(q, keys, vd, torch.float32)
    got = kernels.paged_attention_generic(q.cuda(), k_cache.cuda(), v_cache.cuda(), table.cuda(), token_req.cuda(),
                                          token_pos.cuda(), nq, window, scale, sinks=sinks.cuda())
    assert torch.allclose(got.cpu().double(), want32, atol=2e-5)
    want16 = dense(q, keys, vd, torch.bfloat16)
    step = SimpleNamespace(num_tokens=n, num_reqs=len(runs), cu_q=torch.tensor(cu, dtype=torch.int32).cuda(),
                           ctx_len=torch.tensor([c for _, c in runs], dtype=torch.int32).cuda(), cu_q_host=cu,
                           ctx_len_host=[c for _, c in runs], max_q_len=max(qn for qn, _ in runs),
                           max_ctx_len=max(c for _, c in runs), derived={}, token_req=token_req.cuda(),
                           token_seqpos=token_pos.cuda())
    for share in (False, True):
        got = attention_window.try_attention(q.bfloat16().cuda(), k_cache.bfloat16().cuda(), v_cache.bfloat16().cuda(),
                                             table.cuda(), step, nq, window, 0, scale, share=share, sinks=sinks.cuda())
        assert got is not None
        assert torch.allclose(got.float().cpu().double(), want16, atol=3e-2), (share, (got.float().cpu() - want16).abs().max())


# ---------------------------------------------------------------------------------------------
# whole models, every schedule
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("name", ["mixed", "ones", "odd", "no_conv"])
def test_float32_every_schedule_against_the_plain_model(name, folders):
    """Whole prompts, decoded tails, portions down to two tokens, mixed batches with more requests
    than slots: all the same logits, and the plain model's."""
    folder = folders[name]
    cfg, _ = plain.rapisun_read(folder, F64)
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
    cfg, _ = plain.rapisun_read(folder, F64)
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
    """Score scales so large that the softmax picks single keys: in the layer that sees everything,
    hundreds of tokens back and across page borders; in the windowed ones, right at the window's edge.  The
    last 70 tokens are decoded, so every window (9, 21, 37) passes over decoded tokens; then the same in
    portions."""
    folder = folders["sharp"]
    toks = random_tokens(330, ru.SHARP["vocab"], 40)
    want = _oracle(folder, toks)
    if dtype == "float32":
        # scores this large make float32 arithmetic itself visible: the measure is the plain model run in float32
        cfg, t32 = plain.rapisun_read(folder, torch.float32)
        rounding, slack = _rel_rows(plain.rapisun_forward(cfg, t32, toks), want), 1e-5
    else:
        rounding, slack = _rel_rows(_oracle(folder, toks, plain.to_bfloat16_and_back), want), 1e-3
    for steps in (tail_trace({"s": toks}, 70), portion_trace({"s": toks}, (64, 3, 41, 2, 17, 90))):
        got = _rows(run_steps(_replayer(folder, dtype, round64(len(toks))), steps), "s", len(toks))
        errors = _rel_rows(got, want)
        assert _like_rounding(errors, rounding, slack), (errors.median(), rounding.median(), errors.quantile(0.9),
                                                         rounding.quantile(0.9))
        assert errors.max() < 4 * rounding.max() + slack, (errors.max(), rounding.max())


def test_sharpening_matters(folders):
    """The test above would see a window that is one token off, a lost far key or a sink left out: each
    changes the plain model's last logits."""
    toks = random_tokens(330, ru.SHARP["vocab"], 40)
    whole = _oracle(folders["sharp"], toks)[-30:]

    def one_off(cfg):
        for lay in cfg["layers"]:
            if lay["mixer"].get("mask"):
                lay["mixer"]["mask"]["size"] -= 1

    def nothing_far(cfg):
        cfg["layers"][5]["mixer"]["mask"] = {"size": 200}

    def no_sink(t):
        for name in t:
            if name.endswith(".sink"):
                t[name] = torch.full_like(t[name], -1e4)

    for edit in (one_off, nothing_far):
        assert _rel(_oracle(folders["sharp"], toks, cfg_edit=edit)[-30:], whole) > 0.02, edit.__name__
    assert _rel(_oracle(folders["sharp"], toks, tensors_edit=no_sink)[-30:], whole) > 0.02


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
    held = {g.need.window: sum(p >= 0 for p in cache.table("x", i)) for i, g in enumerate(cache.groups)}
    # the first cache is kept for the longer window of its reader (21 keys: two pages), the second for a reader
    # that sees everything
    assert held == {21: 2, None: 13}
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
