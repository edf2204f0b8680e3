"""The Rapisun architecture without a GPU: its reader of config.json, its spec, tensor names, which layer
reads whose cache and how far back pages are kept, state per request, the random-weights folder, and
the plain implementation's own pieces."""

import copy

import pytest
import torch

import plain_rapisun as plain
import rapisun_util as ru


def _spec(cfg):
    from qwen25vl_lite_amd.config import load_config
    from qwen25vl_lite_amd.models import build_model
    return build_model(load_config(copy.deepcopy(cfg)), torch.float32, "meta")


@pytest.mark.parametrize("cfg", [ru.MIXED, ru.ONES, ru.ODD, ru.NO_CONV])
def test_the_spec_expects_the_files_tensors(cfg):
    model = _spec(cfg)
    got = {model.spec.store_name(k): tuple(v.shape) for k, v in model.expected_tensors().items()}
    assert got == ru.tensor_shapes(cfg)
    for name in ru.tensor_shapes(cfg):
        assert model.spec.store_name(model.spec.map_name(name)) == name


def test_a_reader_shares_its_owners_cache_and_pages_stay_for_the_longest_window():
    from qwen25vl_lite_amd.models.rapisun import retained_keys
    assert retained_keys(ru.MIXED["layers"]) == {0: 21, 3: None}
    model = _spec(ru.MIXED)
    assert [e.cache_from for e in model.spec.run] == [None, None, 0, None, None, 3]
    groups = model.cache_groups()
    # two caches of one layer each: (latent + rotated part, latent) wide, one key/value head
    assert {(g.need.num_kv_heads, g.need.head_dim, g.need.v_dim, g.need.window, g.num_layers) for g in groups} == \
        {(1, 32, 24, 21, 1), (1, 56, 40, None, 1)}
    mixers = [b.mixer for b in model.blocks]
    assert (mixers[0].window, mixers[0].retain, mixers[2].window, mixers[2].retain) == (9, 21, 21, 21)
    assert mixers[2].kv_shared and not mixers[0].kv_shared and mixers[5].window is None


def test_state_per_request():
    model = _spec(ru.MIXED)
    shapes = sorted(tuple(s.shape) for s in model.entry_state if s is not None)
    # a convolution's last inputs in every layer (three taps: two rows), a matrix per head in the recurrent layers
    assert shapes == sorted([(2, 72)] * 6 + [(2, 12, 20), (3, 20, 8)])
    assert all(s is None or s.dtype == torch.float32 for s in model.entry_state)
    ones = _spec(ru.ONES)       # one tap: no state for the convolution
    assert sorted(tuple(s.shape) for s in ones.entry_state if s is not None) == [(1, 16, 16)]
    assert _spec(ru.NO_CONV).blocks[0].filter is None


@pytest.mark.parametrize("bad, text", [
    (lambda c: c.pop("width"), "width"),
    (lambda c: c["norm"].pop("eps"), "eps"),
    (lambda c: c["canon"].__setitem__("taps", 0), "taps"),
    (lambda c: c["layers"][0].__setitem__("type", "conv"), "type"),
    (lambda c: c["layers"][1]["mixer"].pop("vdim"), "vdim"),
    (lambda c: c["layers"][0]["mixer"].pop("kv_rank"), "kv_rank"),
    (lambda c: c["layers"][0]["mixer"]["rot"].__setitem__("dims", 7), "rot.dims"),
    (lambda c: c["layers"][3]["mixer"]["rot"].__setitem__("dims", 18), "rot.dims"),
    (lambda c: c["layers"][0]["mlp"]["router"].__setitem__("top", 7), "cannot be chosen"),
    (lambda c: c["layers"][0]["mlp"].__setitem__("kind", "gated"), "kind"),
    (lambda c: c["layers"][1]["mlp"].pop("ff"), "ff"),
    (lambda c: c["layers"][0]["mixer"]["mask"].pop("size"), "size"),
    (lambda c: c["layers"][2]["mixer"].__setitem__("kv_from", 1), "kv_from"),
    (lambda c: c["layers"][2]["mixer"].__setitem__("kv_from", 3), "kv_from"),
    (lambda c: c["layers"][5]["mixer"].__setitem__("kv_from", 2), "kv_from"),
    (lambda c: c["layers"][2]["mixer"].__setitem__("kv_rank", 16), "differs"),
    (lambda c: c["layers"][5]["mixer"]["rot"].__setitem__("base", 81.0), "differs"),
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
    cfg["layers"][0]["mixer"].pop("mask")
    cfg["layers"][0]["mlp"]["shared"] = None
    cfg["layers"][1]["mlp"] = None
    cfg["canon"] = None
    model = _spec(cfg)
    names = model.expected_tensors()
    assert "l0.mlp.shared.up.weight" not in names and "l1.norm2.weight" not in names and "l0.canon1.weight" not in names
    assert model.blocks[0].mixer.window is None and model.cache_groups()[0].need.window is None


def test_random_weights_folder_loads_back(tmp_path):
    from qwen25vl_lite_amd.config import load_config
    from qwen25vl_lite_amd.weights import write_random_model
    from qwen25vl_lite_amd.weights.safetensors_io import SafetensorsFile
    folder = write_random_model(load_config(copy.deepcopy(ru.ODD)), str(tmp_path / "m"), seed=3, std=0.3)
    with SafetensorsFile(folder + "/model.safetensors") as f:
        assert {n: tuple(f.shape(n)) for n in f.keys()} == ru.tensor_shapes(ru.ODD)
    cfg, tensors = plain.rapisun_read(folder)
    assert 0 <= tensors["l1.mix.lower"].min() and tensors["l1.mix.lower"].max() < 1     # a floor of a gate
    logits = plain.rapisun_forward(cfg, tensors, [1, 2, 3, 4, 5, 6, 7])
    assert logits.shape == (7, 101) and torch.isfinite(logits).all()


def test_silu_mask():
    from qwen25vl_lite_amd.ops.linear_attention import silu_mask
    assert [silu_mask(s) for s in (True, False, None, "", "q", "kv", "qkv")] == [7, 0, 0, 0, 1, 6, 7]


# ---------------------------------------------------------------------------------------------
# the plain implementation's pieces against what their definitions say
# ---------------------------------------------------------------------------------------------
def test_plain_convolution_is_causal_and_starts_from_zeros():
    h = torch.arange(1.0, 7.0, dtype=torch.float64)[:, None].repeat(1, 2)
    w = torch.tensor([[1.0, 10.0, 100.0], [0.0, 0.0, 1.0]], dtype=torch.float64)      # the last tap is the token itself
    out = plain.causal_conv(h, w)
    assert out[:, 0].tolist() == [100.0, 210.0, 321.0, 432.0, 543.0, 654.0]
    assert out[:, 1].tolist() == h[:, 1].tolist()


def test_plain_forget_gate_recurrence_by_hand():
    m = {"heads": 1, "dim": 1, "vdim": 1}
    t = {"q": torch.tensor([[1.0]]), "v": torch.tensor([[1.0]]), "f": torch.tensor([[0.0]]), "f.b": torch.tensor([0.0]),
         "lower": torch.tensor([0.5]), "norm": torch.tensor([1.0]), "o": torch.tensor([[1.0]])}
    t = {"m." + k: v.double() for k, v in t.items()}
    h = torch.tensor([[2.0], [0.0], [0.0]], dtype=torch.float64)
    # f = 0.5 + 0.5 * 0.5 = 0.75 everywhere: the state after the first token is 0.25 * 2, then decays by 0.75 a token;
    # the output is state * silu(h), normed to +-1 (or 0 where the query is 0)
    out = plain.hgrn2(h, t, "m.", m, 0.0)
    assert out[0].item() == pytest.approx(1.0) and out[1].isnan().all() | (out[1] == 0).all()


def test_plain_sink_takes_its_share():
    m = {"heads": 1, "dim": 2, "rot_dim": 2, "vdim": 2, "q_rank": 2, "kv_rank": 2, "scale": 1.0,
         "rot": {"base": 10.0, "dims": 2}}
    eye = torch.eye(2, dtype=torch.float64)
    t = {"m.dq": eye, "m.dq.norm": torch.ones(2).double(), "m.uq": torch.zeros(4, 2).double(), "m.uk": eye, "m.uv": eye,
         "m.o": eye, "m.sink": torch.tensor([0.0]).double()}
    h = torch.tensor([[1.0, 0.0]], dtype=torch.float64)
    kept = (torch.tensor([[3.0, 4.0]], dtype=torch.float64), torch.zeros(1, 2, dtype=torch.float64))
    # all scores are 0 (the query is 0): the one key and the sink share the weight evenly
    out = plain.latent_attention(h, torch.arange(1), t, "m.", m, 0.0, kept)
    assert torch.allclose(out, torch.tensor([[1.5, 2.0]], dtype=torch.float64))


def test_plain_router():
    z = torch.tensor([[1.0, 3.0, 2.0, -1.0]], dtype=torch.float64)
    idx, w = plain.route(z, torch.eye(4, dtype=torch.float64), 2)
    assert sorted(idx[0].tolist()) == [1, 2] and w.sum().item() == pytest.approx(1.0)
    s = torch.softmax(z, -1)[0]
    assert w[0, idx[0].tolist().index(1)].item() == pytest.approx((s[1] / (s[1] + s[2])).item())
