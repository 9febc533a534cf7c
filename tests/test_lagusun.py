"""Lagusun on the host: the configuration, the order of layer runs and what begins a pass, the cache every layer asks for
and when its pages go back, what is refused, and the plain implementation's own mechanisms (tests/plain_lagusun.py)."""
import copy
import math

import pytest
import torch

import lagusun_models
import plain_lagusun as plain
from bare_cuda_4gib_amd.config import LagusunConfig
from bare_cuda_4gib_amd.config.registry import architecture_for
from bare_cuda_4gib_amd.errors import ConfigError


def described(config):
    arch = architecture_for(config)
    assert arch.name == "Lagusun"
    cfg = arch.config_class.from_dict(config)
    from bare_cuda_4gib_amd.engine.model import Model
    return cfg, Model(arch.describe(cfg))


@pytest.mark.parametrize("name", sorted(lagusun_models.CONFIGS))
def test_the_model_wants_exactly_the_tensors_of_the_design(name):
    config = lagusun_models.CONFIGS[name]
    _, model = described(config)
    want = {k: tuple(v.shape) for k, v in lagusun_models.tensors_for(config, 1).items()}
    got = {k: tuple(v.shape) for k, v in model.expected_weights().items()}
    assert got == want


def test_the_order_of_layer_runs_and_the_passes_they_begin():
    cfg, model = described(lagusun_models.CONFIGS["A"])          # layers 1..2 twice
    assert cfg.runs() == [(0, 0, None), (1, 0, 0), (2, 0, None), (1, 1, 1), (2, 1, None), (3, 0, None)]
    assert [(e.layer, e.cache, e.reenter) for e in model.schedule] == [(0, (0, 0), None), (1, (1, 0), 0), (2, (2, 0), None),
                                                                       (1, (1, 1), 1), (2, (2, 1), None), (3, (3, 0), None)]
    assert model.reentry is not None and model.reentry.part.passes == 2
    cfg, model = described(lagusun_models.CONFIGS["B"])          # no loop: nothing replaces the stream
    assert [r[2] for r in cfg.runs()] == [None, None, None] and model.reentry is None
    cfg, model = described(lagusun_models.CONFIGS["F"])          # a loop of one pass still begins that pass
    assert cfg.runs() == [(0, 0, None), (1, 0, 0)] and model.reentry.part.passes == 1
    cfg, _ = described(lagusun_models.CONFIGS["C"])              # the first layer three times
    assert cfg.runs() == [(0, 0, 0), (0, 1, 1), (0, 2, 2), (1, 0, None), (2, 0, None)]
    empty = copy.deepcopy(lagusun_models.CONFIGS["B"])
    empty["loop"] = dict(start=2, stop=2, times=5)               # an empty range loops nothing
    cfg, model = described(empty)
    assert len(cfg.runs()) == 3 and model.reentry is None


def test_every_pass_has_a_cache_of_its_own_and_pages_go_back_by_the_mask():
    from bare_cuda_4gib_amd.cache.specs import PagedHeads
    _, model = described(lagusun_models.CONFIGS["A"])
    streams = model.cache_streams()
    assert set(streams) == {(0, 0), (1, 0), (2, 0), (1, 1), (2, 1), (3, 0)}
    assert streams[(0, 0)] == PagedHeads(2, 12, 2, 12, 0, 0, 9) and streams[(1, 1)] == PagedHeads(3, 10, 3, 6, 11, 0, 0)
    block, window = streams[(3, 0)], streams[(2, 0)]
    assert block.group_key() == ("block", 33) and window.group_key() == ("window", 20)
    # a query at position `length` and all later ones read nothing before the start of its block / its window
    assert [block.first_kept(n) for n in (0, 1, 32, 33, 34, 65, 66, 99)] == [0, 0, 0, 33, 33, 33, 66, 99]
    assert [window.first_kept(n) for n in (0, 19, 20, 21, 100)] == [0, 0, 1, 2, 81]
    _, model = described(lagusun_models.CONFIGS["D"])            # no mask: every key is kept
    assert model.cache_streams()[(0, 0)].group_key() == ("window", 0)


def test_the_cache_manager_gives_back_the_pages_before_the_current_block():
    from bare_cuda_4gib_amd.cache.manager import CacheManager
    from bare_cuda_4gib_amd.cache.specs import PagedHeads
    cache = CacheManager({"s": PagedHeads(1, 4, 1, 4, 0, 0, 10)}, page_tokens=4, num_pages=6, max_requests=2, max_tokens=64,
                         dtype=torch.float32, device="cpu")
    cache.admit("r")
    held = []
    for n in (3, 6, 1, 9, 2, 20):           # lengths 3, 9, 10, 19, 21, 41
        cache.reserve([("r", n)])
        cache.advance("r", n)
        held.append((cache.length("r"), [i for i, p in enumerate(cache.table(("block", 10), "r")) if p >= 0]))
    assert held == [(3, [0]), (9, [0, 1, 2]), (10, [2]), (19, [2, 3, 4]), (21, [5]), (41, [10])]
    cache.release("r")
    assert cache.pages_in_use() == 0


@pytest.mark.parametrize("change,message", [
    (lambda c: c["layers"][0].__setitem__("type", "attention_3"), "type"),
    (lambda c: c["layers"][0]["mixer"].pop("scale"), "lacks scale"),
    (lambda c: c["layers"][0]["mixer"].__setitem__("vdim", 5), "values are the keys"),
    (lambda c: c["norm"].__setitem__("groups", 5), "groups"),
    (lambda c: c["loop"].__setitem__("stop", 9), "loop"),
    (lambda c: c["layers"][0]["mlp"].__setitem__("kind", "dense"), "kind"),
    (lambda c: c["layers"][1]["mixer"]["rot"]["scaling"].pop("low"), "low"),
    (lambda c: c["layers"][1]["mixer"].__setitem__("softcap", -1.0), "softcap"),
    (lambda c: c["layers"][0]["mixer"].__setitem__("kv_heads", 3), "share"),
])
def test_what_is_refused(change, message):
    config = copy.deepcopy(lagusun_models.CONFIGS["A"])
    change(config)
    with pytest.raises(ConfigError, match=message):
        described(config)


def test_absent_keys_have_the_design_s_defaults():
    config = copy.deepcopy(lagusun_models.CONFIGS["B"])
    cfg = LagusunConfig.from_dict(config)
    assert cfg.embedding_scale == 1.0 and cfg.norm_groups == 1 and cfg.loop_range() == (0, 0, 1)
    _, model = described(config)
    mixer = model.layers[1].mixer
    assert mixer.block == 70 and mixer.window == 0 and mixer.unit_sink and not mixer.own_values and mixer.row_norm
    mixer = model.layers[0].mixer
    assert mixer.window == 50 and mixer.cap == 0.0 and mixer.squash and mixer.bias and mixer.value_unit_norm and mixer.unit_norm
    ffn = model.layers[0].ffn
    assert ffn.squash and ffn.normalize and ffn.route_scale == 1.0 and not ffn.gated and not ffn.shared_gate
    assert model.layers[2].ffn.route_scale == 2.5 and model.layers[1].ffn is None


@pytest.mark.parametrize("dims,base,scaling", [(10, 100.0, (4.0, 1.0, 3.0, 40)), (12, 1000.0, (6.0, 1.0, 3.0, 64)), (6, 20.0, (2.0, 0.5, 2.0, 16)),
                                               (8, 300.0, (16.0, 2.0, 8.0, 100)), (64, 250000.0, (6.0, 1.0, 3.0, 4096)), (6, 9.0, None)])
def test_the_rotary_part_scales_frequencies_by_wavelength(dims, base, scaling):
    from bare_cuda_4gib_amd.parts.position import Rotary
    as_dict = dict(zip(("factor", "low", "high", "original"), scaling)) if scaling else None
    freqs, amplitude = Rotary(base, dims, scaling=as_dict).frequencies()
    want = plain.scaled_frequencies(dims, base, as_dict)
    assert amplitude == 1.0 and torch.allclose(torch.tensor(freqs, dtype=torch.float64), want, rtol=1e-14, atol=0)
    if scaling:         # all three ranges occur: kept, divided by the factor, and between
        plain_f = plain.scaled_frequencies(dims, base, None)
        ratio = want / plain_f
        assert float(ratio.max()) == 1.0 and abs(float(ratio.min()) - 1.0 / scaling[0]) < 1e-12
        if dims != 6:
            assert bool(((ratio > 1.0 / scaling[0] + 1e-9) & (ratio < 1.0 - 1e-9)).any())


def test_the_plain_mechanisms():
    torch.manual_seed(0)
    v, g = torch.randn(5, 12, dtype=torch.float64), torch.rand(12, dtype=torch.float64) + 0.5
    normed = plain.grouped_norm(v, g, 0.0, 3) / g
    assert torch.allclose((normed.view(5, 3, 4) ** 2).mean(-1), torch.ones(5, 3, dtype=torch.float64))
    assert not torch.allclose(normed, plain.grouped_norm(v, g, 0.0, 1) / g)
    mask = plain.block_mask(7, 3)
    assert mask.int().tolist() == [[1, 0, 0, 0, 0, 0, 0], [1, 1, 0, 0, 0, 0, 0], [1, 1, 1, 0, 0, 0, 0], [0, 0, 0, 1, 0, 0, 0],
                                   [0, 0, 0, 1, 1, 0, 0], [0, 0, 0, 1, 1, 1, 0], [0, 0, 0, 0, 0, 0, 1]]
    assert plain.window_mask(4, 2).int().tolist() == [[1, 0, 0, 0], [1, 1, 0, 0], [0, 1, 1, 0], [0, 0, 1, 1]]
    s = torch.randn(2, 7, 7, dtype=torch.float64)
    p = plain.softmax_plus_one(s, mask)
    direct = torch.exp(s) * mask / (1.0 + (torch.exp(s) * mask).sum(-1, keepdim=True))
    assert torch.allclose(p, direct) and bool((p.sum(-1) < 1.0).all())
    big = plain.softmax_plus_one(s + 800.0, mask)               # (no overflow: the one is counted from the same maximum)
    assert bool(torch.isfinite(big).all()) and torch.allclose(big.sum(-1), torch.ones(2, 7, dtype=torch.float64))
    assert torch.allclose(plain.capped(torch.tensor([0.01, 100.0, -100.0]), 2.0), torch.tensor([0.01, 2.0, -2.0]), atol=1e-6)
    w = plain.sigmoid_weights(s, plain.window_mask(7, 2), torch.tensor([0.0, -1.0], dtype=torch.float64))
    assert float(w[0, 3, 1]) == 0.0 and abs(float(w[1, 3, 2]) - 1.0 / (1.0 + math.exp(1.0 - float(s[1, 3, 2])))) < 1e-12
    x = torch.randn(3, 2, 6, dtype=torch.float64)
    turned = plain.half_rotation(x, torch.tensor([0, 1, 5]), torch.tensor([1.0, 0.1], dtype=torch.float64))
    assert torch.equal(turned[0], x[0]) and torch.equal(turned[..., 4:], x[..., 4:])         # position 0, and beyond the rotated part
    assert abs(float(turned[1, 0, 0]) - (float(x[1, 0, 0]) * math.cos(1.0) - float(x[1, 0, 2]) * math.sin(1.0))) < 1e-12
    assert abs(float(turned[2, 1, 3]) - (float(x[2, 1, 3]) * math.cos(0.5) + float(x[2, 1, 1]) * math.sin(0.5))) < 1e-12
    z = torch.tensor([[0.0, 2.0, -1.0, 1.0]], dtype=torch.float64)
    chosen, weights, margin = plain.route(z, torch.tensor([1.0, 0.0, 0.0, 0.0], dtype=torch.float64), 2, 3.0)
    s_ = torch.sigmoid(z[0])
    assert chosen.tolist() == [[0, 1]]                           # (0.5 + 1 beats sigmoid(1) = 0.73: the correction chooses)
    assert torch.allclose(weights[0], 3.0 * s_[[0, 1]] / (s_[0] + s_[1])) and abs(float(margin) - float(s_[1] - s_[3])) < 1e-12
    assert abs(float(plain.exact_gelu(torch.tensor(1.0, dtype=torch.float64))) - 0.8413447460685429) < 1e-12


@pytest.mark.parametrize("name", sorted(lagusun_models.CONFIGS))
def test_the_plain_model_does_not_look_ahead_and_every_piece_counts(name, tmp_path):
    folder = lagusun_models.write_folder(tmp_path, name, "float32")
    model = plain.PlainLagusun(folder)
    ids = [(7 * i + 3) % model.cfg["vocab"] for i in range(40)]
    whole, after = model.forward(ids, return_layers=True)
    assert len(after) == len(model.runs()) and bool(torch.isfinite(whole).all())
    assert torch.allclose(model.forward(ids[:23]), whole[:23], atol=1e-5, rtol=1e-5)
    # the factor on the embedding, the sublayers' scales and the pass vectors are seen in the logits
    for key in ["l0.ls1", "final.norm"] + (["loop.step", "loop.in"] if "loop.in" in model.w else []):
        kept = model.w[key].clone()
        model.w[key] = kept * 1.1
        assert float((model.forward(ids) - whole).abs().max()) > 1e-3, key
        model.w[key] = kept


def test_the_random_weights_mode_writes_a_folder_that_loads(tmp_path):
    """The framework's own random-weights mode over a Lagusun configuration: every tensor the design names, norm weights
    and the sublayers' scales at one, a folder whose configuration reads back."""
    from bare_cuda_4gib_amd.config.registry import load_config
    from bare_cuda_4gib_amd.weights import write_random_model
    from safetensors.torch import load_file
    folder = write_random_model(lagusun_models.CONFIGS["A"], 5, str(tmp_path / "random"), "bfloat16")
    arch, cfg = load_config(folder)
    assert arch.name == "Lagusun" and cfg.embedding_scale == 2.5 and cfg.norm_groups == 3
    tensors = load_file(folder + "/model.safetensors")
    assert set(tensors) == set(lagusun_models.tensors_for(lagusun_models.CONFIGS["A"], 1))
    assert bool((tensors["l1.ls1"] == 1.0).all()) and bool((tensors["l0.norm2"] == 1.0).all())
    assert tuple(tensors["loop.step"].shape) == (2, 48) and float(tensors["loop.in"].float().std()) > 0
