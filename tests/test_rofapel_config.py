"""The Rofapel architecture without a GPU: its reader of config.json, its spec, tensor names, the run list of
looped passes, caches and state per request, the random-weights folder, and the plain implementation's own
pieces."""

import copy
import math

import pytest
import torch

import plain_rofapel as plain
import rofapel_util as ru


def _spec(cfg):
    from qwen25vl_lite_amd.config import load_config
    from qwen25vl_lite_amd.models import build_model
    return build_model(load_config(copy.deepcopy(cfg)), torch.float32, "meta")


@pytest.mark.parametrize("cfg", [ru.MIXED, ru.ONES, ru.ODD, ru.TAIL_LOOP])
def test_the_spec_expects_the_files_tensors(cfg):
    model = _spec(cfg)
    got = {model.spec.store_name(k): tuple(v.shape) for k, v in model.expected_tensors().items()}
    assert got == ru.tensor_shapes(cfg)
    for name in ru.tensor_shapes(cfg):
        assert model.spec.store_name(model.spec.map_name(name)) == name


def test_the_run_list_of_looped_passes():
    from qwen25vl_lite_amd.models.rofapel import rofapel_run_list
    run = rofapel_run_list(5, {"start": 1, "stop": 3, "times": 3})
    assert [e.layer for e in run] == [0, 1, 2, 1, 2, 1, 2, 3, 4]
    assert [e.add_vector for e in run] == [None, 0, None, 1, None, 2, None, None, None]
    assert [e.mix_input for e in run] == [False, True, False, True, False, True, False, False, False]
    assert [(e.layer, e.mix_input) for e in rofapel_run_list(3, None)] == [(0, False), (1, False), (2, False)]
    # the plain implementation's order is the same
    assert [(i, k) for i, k in plain.run_order(ru.MIXED)] == [(e.layer, e.add_vector) for e in run]
    once = rofapel_run_list(3, {"start": 0, "stop": 3, "times": 1})
    assert [(e.layer, e.add_vector, e.mix_input) for e in once] == [(0, 0, True), (1, None, False), (2, None, False)]


def test_every_pass_has_a_cache_and_a_state_of_its_own():
    model = _spec(ru.MIXED)
    groups = {(g.need.num_kv_heads, g.need.head_dim, g.need.v_dim, g.need.window): g.num_layers
              for g in model.cache_groups()}
    # layer 0 once, layers 1 and 2 three times each, layers 3 and 4 once: one cache layer per run
    # (a latent's cache has one key/value head: latent and rotated part wide, the value the latent alone)
    assert groups == {(2, 16, 16, 9): 1, (1, 48, 40, None): 3, (2, 24, 16, None): 3, (3, 24, 24, 37): 1,
                      (1, 40, 24, None): 1}
    shapes = [None if s is None else tuple(s.shape) for s in model.entry_state]
    # the convolution's last projected rows (taps - 1 of them) over the queries' and keys' channels
    assert shapes == [(1, 96), None, None, None, None, None, None, (3, 144), None]
    ones = _spec(ru.ONES)       # one tap: no state
    assert all(s is None for s in ones.entry_state)
    assert ones.blocks[0].mixer.conv_taps == 1 and ones.blocks[0].mixer.window == 1


def test_what_the_parts_are_told():
    model = _spec(ru.MIXED)
    a2, lat, att = model.blocks[0].mixer, model.blocks[1].mixer, model.blocks[2].mixer
    assert (a2.values_are_keys, a2.has_sinks, a2.head_gate, a2.qk_norm_scope, a2.window) == (True, True, True, "head", 9)
    assert (att.qk_norm_scope, att.head_gate, att.has_sinks, att.window, att.vd, att.hd) == ("whole", True, False, None, 16, 24)
    assert a2.position.divide == 3.0 and att.position.divide is None and not att.position.interleaved
    assert lat.q_rank == 0 and lat.interleaved and not lat.has_sinks and lat.window is None
    assert lat.position.amplitude == pytest.approx(0.1 * math.log(4.0) + 1.0)
    assert model.blocks[4].mixer.position.amplitude == 1.0 and model.blocks[4].mixer.position.ramp is None
    assert model.blocks[3].ffn is None and model.blocks[3].norm2 is None and model.blocks[0].norm2 is not None
    assert model.embedding.scale == 1.7 and not model.spec.tie_word_embeddings
    moe = model.blocks[1].ffn
    assert (moe.score, moe.normalize, moe.floor, moe.router_bias, moe.alpha, moe.limit, moe.shift) == \
        ("softmax", True, 0.0, True, 1.0, None, 0.0)


def test_scalings_and_masks_are_read_by_their_keys_in_every_mixer():
    model = _spec(ru.CROSSED)
    att, lat, a2 = (b.mixer for b in model.blocks)
    assert att.position.ramp is not None and att.position.amplitude > 1.0 and att.window == 13
    assert lat.position.divide == 2.5 and lat.position.amplitude == 1.0 and lat.window == 20
    assert a2.position.ramp is not None and a2.window == 11
    windows = sorted((g.need.window or 0) for g in model.cache_groups())
    assert windows == [11, 13, 20]


def test_frequency_tables():
    from qwen25vl_lite_amd.parts.base import PartSpec, build_part
    lin = build_part("position", PartSpec("rope", {"theta": 500.0, "rotary_dim": 8,
                                                   "scaling": {"kind": "linear", "factor": 3.0}}), torch.float32, "cpu")
    want, _ = plain.divided_frequencies({"base": 500.0, "dims": 8, "scaling": {"factor": 3.0}})
    assert torch.allclose(lin.rotary_tables(16)[0].double(), want, rtol=1e-6)
    rot = {"base": 300.0, "dims": 8, "scaling": {"factor": 4.0, "original": 48, "fast": 8.0, "slow": 1.5}}
    ramp = build_part("position", PartSpec("rope", {"theta": 300.0, "rotary_dim": 8, "scaling": dict(rot["scaling"], kind="ramp")}),
                      torch.float32, "cpu")
    want, amp = plain.ramp_frequencies(rot)
    assert torch.allclose(ramp.rotary_tables(8)[0].double(), want, rtol=1e-6) and ramp.amplitude == pytest.approx(amp)
    plain_f = plain.frequencies(rot)
    assert not torch.allclose(want, plain_f) and not torch.allclose(want, plain_f / 4.0)   # the ramp is in between


@pytest.mark.parametrize("bad, text", [
    (lambda c: c.pop("width"), "width"),
    (lambda c: c["norm"].pop("eps"), "eps"),
    (lambda c: c.pop("embedding"), "embedding"),
    (lambda c: c["embedding"].pop("scale"), "scale"),
    (lambda c: c["layers"][0].__setitem__("type", "conv"), "type"),
    (lambda c: c["layers"][1]["mixer"].pop("vdim"), "vdim"),
    (lambda c: c["layers"][1]["mixer"].pop("kv_rank"), "kv_rank"),
    (lambda c: c["layers"][2]["mixer"].pop("kv_heads"), "kv_heads"),
    (lambda c: c["layers"][2]["mixer"].__setitem__("kv_heads", 4), "multiple"),
    (lambda c: c["layers"][0]["mixer"]["rot"].__setitem__("dims", 7), "rot.dims"),
    (lambda c: c["layers"][1]["mixer"]["rot"].__setitem__("dims", 10), "rot.dims"),
    (lambda c: c["layers"][1]["mixer"]["rot"]["scaling"].pop("slow"), "slow"),
    (lambda c: c["layers"][0]["mixer"]["rot"]["scaling"].__setitem__("factor", 0), "factor"),
    (lambda c: c["layers"][0]["mixer"].pop("conv"), "conv"),
    (lambda c: c["layers"][0]["mixer"]["mask"].pop("size"), "size"),
    (lambda c: c["layers"][0]["mixer"].__setitem__("vdim", 8), "vdim"),
    (lambda c: c["layers"][1]["mlp"]["router"].__setitem__("top", 7), "cannot be chosen"),
    (lambda c: c["layers"][1]["mlp"].__setitem__("kind", "gated"), "kind"),
    (lambda c: c["layers"][0]["mlp"].pop("ff"), "ff"),
    (lambda c: c["loop"].__setitem__("stop", 6), "loop"),
    (lambda c: c["loop"].__setitem__("times", 0), "loop"),
    (lambda c: c["loop"].pop("start"), "start"),
])
def test_config_errors_name_the_key(bad, text):
    from qwen25vl_lite_amd.config import load_config
    from qwen25vl_lite_amd.config.model_config import ConfigError
    cfg = copy.deepcopy(ru.MIXED)
    bad(cfg)
    with pytest.raises(ConfigError, match=text):
        load_config(cfg)


def test_optional_blocks_may_be_absent():
    cfg = copy.deepcopy(ru.ODD)
    cfg["layers"][0]["mixer"]["rot"].pop("scaling")
    cfg["layers"][0]["mlp"]["shared"] = None
    cfg["layers"][1]["mixer"]["rot"]["scaling"] = None
    cfg["layers"][1]["mlp"] = None
    cfg["loop"] = None
    model = _spec(cfg)
    names = model.expected_tensors()
    assert "l0.mlp.shared.up.weight" not in names and "l1.norm2.weight" not in names and "loop.in.weight" not in names
    assert model.pass_mix is None and model.pass_vectors is None
    assert model.spec.map_name("l1.norm2") is None and model.spec.map_name("l0.norm2") == "l0.norm2.weight"
    # a loop over an empty range is no loop, and its tensors, if a file has them, are passed over
    cfg["loop"] = {"start": 2, "stop": 2, "times": 3}
    model = _spec(cfg)
    assert [e.layer for e in model.spec.run] == [0, 1, 2] and model.pass_mix is None
    assert model.spec.map_name("loop.in") is None and model.spec.map_name("loop.step") is None


def test_random_weights_folder_loads_back(tmp_path):
    from qwen25vl_lite_amd.config import load_config
    from qwen25vl_lite_amd.weights import write_random_model
    from qwen25vl_lite_amd.weights.safetensors_io import SafetensorsFile
    folder = write_random_model(load_config(copy.deepcopy(ru.TAIL_LOOP)), str(tmp_path / "m"), seed=3, std=0.3)
    with SafetensorsFile(folder + "/model.safetensors") as f:
        assert {n: tuple(f.shape(n)) for n in f.keys()} == ru.tensor_shapes(ru.TAIL_LOOP)
    cfg, tensors = plain.rofapel_read(folder)
    logits = plain.rofapel_forward(cfg, tensors, [1, 2, 3, 4, 5, 6, 7])
    assert logits.shape == (7, 77) and torch.isfinite(logits).all()


# ---------------------------------------------------------------------------------------------
# the plain implementation's pieces against what their definitions say
# ---------------------------------------------------------------------------------------------
def test_plain_convolution_is_causal_and_starts_from_zeros():
    u = torch.arange(1.0, 7.0, dtype=torch.float64)[:, None].repeat(1, 2)
    w = torch.tensor([[1.0, 10.0, 100.0], [0.0, 0.0, 1.0]], dtype=torch.float64)      # the last tap is the token itself
    out = plain.causal_conv(u, w)
    assert out[:, 0].tolist() == [100.0, 210.0, 321.0, 432.0, 543.0, 654.0]
    assert out[:, 1].tolist() == u[:, 1].tolist()


def test_plain_rotations_pair_the_right_channels():
    x = torch.zeros(1, 1, 6, dtype=torch.float64)
    x[0, 0, 0] = 1.0
    quarter = torch.tensor([math.pi / 2, 0.0], dtype=torch.float64)      # at position 1: a quarter turn of pair 0
    pos = torch.tensor([1])
    halves = plain.rotate(x, pos, quarter, 1.0, "halves")[0, 0]
    near = plain.rotate(x, pos, quarter, 2.0, "neighbours")[0, 0]
    assert torch.allclose(halves, torch.tensor([0.0, 0, 1.0, 0, 0, 0], dtype=torch.float64), atol=1e-12)   # partner 0 + 4/2
    assert torch.allclose(near, torch.tensor([0.0, 2.0, 0, 0, 0, 0], dtype=torch.float64), atol=1e-12)     # partner 1, doubled
    y = torch.randn(3, 2, 6, dtype=torch.float64)
    assert torch.equal(plain.rotate(y, torch.arange(3), quarter, 1.0, "halves")[..., 4:], y[..., 4:])      # beyond dims: as it was


def test_plain_sink_and_window():
    q = torch.zeros(3, 1, 2, dtype=torch.float64)
    k = torch.zeros(3, 1, 2, dtype=torch.float64)
    v = torch.tensor([[[3.0]], [[6.0]], [[12.0]]], dtype=torch.float64)
    # all scores are 0: the visible keys and the sink (exp(0) = 1) share the weight evenly
    out = plain.attend(q, k, v, 1.0, window=2, sink=torch.zeros(1, dtype=torch.float64))
    assert torch.allclose(out[:, 0, 0], torch.tensor([1.5, 3.0, 6.0], dtype=torch.float64))
    out = plain.attend(q, k, v, 1.0)
    assert torch.allclose(out[:, 0, 0], torch.tensor([3.0, 4.5, 7.0], dtype=torch.float64))


def test_plain_router():
    z = torch.tensor([[1.0, 3.0, 2.0, -1.0]], dtype=torch.float64)
    idx, w = plain.route(z, 2)
    assert idx[0].tolist() == [1, 2] and w.sum().item() == pytest.approx(1.0)
    assert w[0, 0].item() == pytest.approx(1.0 / (1.0 + math.exp(-1.0)))


def test_plain_whole_projection_norm_differs_from_a_norm_per_head():
    torch.manual_seed(0)
    x = torch.randn(4, 6, dtype=torch.float64)
    x[:, :3] *= 10.0                    # the first head is much larger
    whole = plain.unit_rms(x, 0.0)
    per_head = plain.unit_rms(x.view(4, 2, 3), 0.0).view(4, 6)
    assert (whole[:, 3:].abs().max() < 0.5 * per_head[:, 3:].abs().max())
