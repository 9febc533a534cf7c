"""Milenex on the host: its configuration, the model and the schedule it describes (layers that run several times, each
pass with a cache of its own), what its layers ask of the cache manager, what is refused, and the plain implementation's
mechanisms against hand-made cases."""
import copy
import math

import pytest
import torch

import milenex_models
import plain_milenex as plain


def _describe(config):
    from bare_cuda_4gib_amd.config.registry import architecture_for
    arch = architecture_for(config)
    return arch, arch.config_class.from_dict(config)


def test_the_architecture_is_chosen_by_its_name():
    arch, cfg = _describe(milenex_models.CONFIGS["A"])
    assert arch.name == "Milenex" and cfg.vocab_size == 96 and cfg.hidden_size == 48 and cfg.norm_eps == 1e-5
    spec = arch.describe(cfg)
    assert [l.block for l in spec.layers] == ["prenorm"] * 4 and [l.mixer.kind for l in spec.layers] == ["sink_attention"] * 4
    first, second = spec.layers[0].mixer.params, spec.layers[1].mixer.params
    assert first["window"] == 9 and first["conv_taps"] == 3 and first["unit_norm"] and first["scale"] == 0.5
    assert first["position"].params == dict(theta=500.0, dim=8, pairing="neighbours")
    assert not first.get("talking") and not first.get("distance") and not first.get("head_gate")
    assert second["talking"] and second["distance"] and second["head_gate"] and not second.get("unit_norm") and second.get("position") is None
    assert [None if l.ffn is None else l.ffn.kind for l in spec.layers] == ["dense_gelu", "routed_experts", None, "routed_experts"]
    routed = spec.layers[1].ffn.params
    assert (routed["experts"], routed["top"], routed["groups"], routed["keep"], routed["shared_size"], routed["shared_limit"]) == (6, 2, 3, 2, 16, 0.7)
    assert spec.layers[3].ffn.params["groups"] == 1 and spec.layers[3].ffn.params["shared_size"] == 0
    assert all("mixer_shift" in l.extras for l in spec.layers)


@pytest.mark.parametrize("name,runs", [
    ("A", [(0, 0, False), (1, 0, False), (0, 1, True), (1, 1, False), (2, 0, False), (3, 0, False)]),
    ("B", [(0, 0, False), (1, 0, False), (2, 0, False)]),
    ("C", [(0, 0, False), (1, 0, False), (1, 1, True), (1, 2, True), (2, 0, False)]),
    ("D", [(0, 0, False), (1, 0, False), (2, 0, False), (1, 1, True), (2, 1, False)])])
def test_the_schedule_runs_looped_layers_again_with_caches_of_their_own(name, runs):
    from bare_cuda_4gib_amd.engine import Model
    arch, cfg = _describe(milenex_models.CONFIGS[name])
    assert cfg.runs() == runs
    spec = arch.describe(cfg)
    assert [(e.layer, e.cache, e.add_embedding) for e in spec.schedule] == [(i, (i, turn), add) for i, turn, add in runs]
    streams = Model(spec).cache_streams()
    assert len(streams) == len(runs)                       # every run keeps its own keys, values, tails
    assert plain.PlainMilenex.order(type("M", (), {"cfg": milenex_models.CONFIGS[name]})()) == [(i, add) for i, _, add in runs]


@pytest.mark.parametrize("name", sorted(milenex_models.CONFIGS))
def test_the_model_asks_for_exactly_the_tensors_of_the_design(name):
    from bare_cuda_4gib_amd.engine import Model
    config = milenex_models.CONFIGS[name]
    arch, cfg = _describe(config)
    expected = Model(arch.describe(cfg)).expected_weights()
    drawn = milenex_models.tensors_for(config, 1)
    assert set(expected) == set(drawn)
    for n, spec in expected.items():
        assert tuple(spec.shape) == tuple(drawn[n].shape), n


def test_what_a_layer_keeps():
    from bare_cuda_4gib_amd.cache.specs import Bundle, PagedHeads, States
    from bare_cuda_4gib_amd.engine import Model
    arch, cfg = _describe(milenex_models.CONFIGS["B"])
    streams = Model(arch.describe(cfg)).cache_streams()
    shift = States((("tail", (1, 64), None),))
    assert streams[(0, 0)] == Bundle((("mixer", PagedHeads(1, 24, 1, 130, 50, 0)), ("shift", shift)))
    channels = 2 * 40 + 2 * 40 + 2 * 24
    assert streams[(1, 0)] == Bundle((("mixer", Bundle((("kv", PagedHeads(2, 40, 2, 24, 70, 0)),
                                                        ("conv", States((("tail", (4, channels), None),)))))), ("shift", shift)))
    assert streams[(2, 0)] == Bundle((("mixer", PagedHeads(1, 72, 1, 200, 17, 0)), ("shift", shift)))    # one tap: no tail
    # pages that the window has passed go back: a request far longer than its pool fits
    spec = streams[(0, 0)].members[0][1]
    assert spec.first_kept(200) == 151 and spec.first_kept(10) == 0


def test_what_is_refused():
    from bare_cuda_4gib_amd.engine import Model
    from bare_cuda_4gib_amd.errors import ConfigError
    base = milenex_models.CONFIGS["A"]

    def changed(edit):
        c = copy.deepcopy(base)
        edit(c)
        return c
    bad = [
        lambda c: c["layers"][0].__setitem__("type", "attention_3"),
        lambda c: c["layers"][0]["mixer"].pop("scale"),
        lambda c: c["layers"][0]["mixer"].__setitem__("heads", 2.5),
        lambda c: c["layers"][0]["mixer"]["rot"].pop("base"),
        lambda c: c["layers"][0]["mlp"].__setitem__("kind", "sparse"),
        lambda c: c["layers"][1]["mlp"]["router"].pop("top"),
        lambda c: c["layers"][1]["mlp"]["expert"].pop("limit"),
        lambda c: c["loop"].__setitem__("stop", 9),
        lambda c: c["loop"].__setitem__("times", 0),
        lambda c: c.pop("norm"),
    ]
    for edit in bad:
        with pytest.raises(ConfigError):
            _describe(changed(edit))
    built_bad = [
        lambda c: c["layers"][0]["mixer"].__setitem__("kv_heads", 3),                    # 4 heads cannot share 3
        lambda c: c["layers"][0]["mixer"]["rot"].__setitem__("dims", 14),                # more than a head has
        lambda c: c["layers"][0]["mixer"]["rot"].__setitem__("dims", 5),                 # pairs
        lambda c: c["layers"][1]["mlp"]["router"].__setitem__("top", 5),                 # 2 groups of 2 hold 4
        lambda c: c["layers"][1]["mlp"]["router"]["groups"].__setitem__("count", 4),     # 6 experts in 4 groups
        lambda c: c["layers"][1]["mlp"]["router"]["groups"].__setitem__("keep", 4),
    ]
    for edit in built_bad:
        arch, cfg = _describe(changed(edit))
        with pytest.raises(ConfigError):
            Model(arch.describe(cfg))


def test_plain_token_shift_and_convolution():
    h = torch.tensor([[1.0, 10.0], [2.0, 20.0], [4.0, 40.0]], dtype=torch.float64)
    m = torch.tensor([0.25, 1.0], dtype=torch.float64)
    assert torch.equal(plain.token_shift(h, m), torch.tensor([[0.75, 0.0], [1.75, 10.0], [3.5, 20.0]], dtype=torch.float64))
    w = torch.tensor([[100.0, 10.0, 1.0]], dtype=torch.float64)                        # the last tap is the current token's
    u = torch.tensor([[1.0], [2.0], [3.0], [4.0]], dtype=torch.float64)
    assert plain.short_convolution(u, w).view(-1).tolist() == [1.0, 12.0, 123.0, 234.0]


def test_plain_rotation_turns_neighbouring_pairs():
    v = torch.zeros(2, 1, 6, dtype=torch.float64)
    v[:, 0] = torch.tensor([1.0, 0.0, 0.0, 2.0, 5.0, 7.0])
    out = plain.neighbour_rotation(v, torch.tensor([0, 3]), 4, 100.0)
    assert torch.equal(out[0], v[0])
    a0, a1 = 3.0, 3.0 * 100.0 ** -0.5
    want = torch.tensor([math.cos(a0), math.sin(a0), -2 * math.sin(a1), 2 * math.cos(a1), 5.0, 7.0], dtype=torch.float64)
    assert torch.allclose(out[1, 0], want, atol=1e-12)


def test_plain_weights_have_a_window_a_sink_and_a_penalty_on_distance():
    q, k = torch.zeros(5, 2, dtype=torch.float64), torch.zeros(5, 2, dtype=torch.float64)
    w = plain.window_weights(q, k, 1.0, 3, sink=0.0)
    assert torch.allclose(w[0], torch.tensor([0.5, 0, 0, 0, 0], dtype=torch.float64))                # one key and the sink
    assert torch.allclose(w[4], torch.tensor([0, 0, 0.25, 0.25, 0.25], dtype=torch.float64))         # three keys and the sink
    w = plain.window_weights(q, k, 1.0, 5, sink=-50.0, r1=1.0, r2=1.0)                               # exp(-ln(1 + n)) = 1 / (1 + n)
    assert torch.allclose(w[2], torch.tensor([1 / 3, 1 / 2, 1.0, 0, 0], dtype=torch.float64) / (1 + 1 / 2 + 1 / 3))


def test_plain_router_keeps_groups_and_weighs_by_the_plain_scores():
    z = torch.log(torch.tensor([[0.30, 0.05, 0.25, 0.05, 0.20, 0.15]], dtype=torch.float64))
    none = torch.zeros(6, dtype=torch.float64)
    chosen, weights = plain.route(z, none, 2, 1, 1)
    assert chosen.tolist() == [[0, 2]] and torch.allclose(weights, torch.tensor([[0.30, 0.25]], dtype=torch.float64))
    # three groups of two, the best two kept: experts 0, 1 (0.30) and 2, 3 (0.25); the third's 0.20 cannot be chosen
    chosen, _ = plain.route(z, none, 3, 3, 2)
    assert sorted(chosen[0].tolist()) == [0, 1, 2] or sorted(chosen[0].tolist()) == [0, 2, 3]
    # the correction moves the choice, not the weights; choices below zero still beat experts of groups left out
    correction = torch.tensor([-1.0, -1.0, -1.0, -1.0, -2.0, 0.5], dtype=torch.float64)
    chosen, weights = plain.route(z, correction, 3, 3, 2)
    # groups count 0.65 and -0.70 (against -0.75): expert 1 at -0.95 is chosen before expert 2 at -0.75, whose group is out
    assert sorted(chosen[0].tolist()) == [0, 1, 5]
    assert torch.allclose(weights.sum(), torch.tensor(0.15 + 0.30 + 0.05, dtype=torch.float64))
    assert float(plain.route_margin(z, correction, 3, 3, 2)) == pytest.approx(0.05)


def test_plain_experts_are_clamped_from_above_only_in_the_gate():
    g, u = torch.tensor([-9.0, 0.3, 5.0]), torch.tensor([-7.0, 0.2, 7.0])
    out = plain.clamped_glu(g.double(), u.double(), 2.0)
    sig = lambda v: 1.0 / (1.0 + math.exp(-1.702 * v))       # noqa: E731
    assert out.tolist() == pytest.approx([-9.0 * sig(-9.0) * (-2.0 + 1.0), 0.3 * sig(0.3) * 1.2, 2.0 * sig(2.0) * 3.0])


@pytest.mark.parametrize("name", sorted(milenex_models.CONFIGS))
def test_plain_prefix_of_a_sequence_is_the_sequence_of_the_prefix(tmp_path, name):
    """Nothing in the plain model looks ahead: the logits of the first tokens do not change when tokens follow."""
    import helpers
    folder = milenex_models.write_folder(tmp_path, name, "float32")
    model = plain.PlainMilenex(folder)
    ids = helpers.random_ids(40, model.cfg["vocab"], 3)
    whole, part = model.forward(ids), model.forward(ids[:13])
    assert torch.allclose(whole[:13], part, atol=1e-9, rtol=1e-9)
