"""The plain Ledudra implementation pinned to cases worked out by hand and to closed forms, and the design's
configuration. No GPU."""
import math

import pytest
import torch

import plain_ledudra as P
from ledudra_models import CONFIGS


def test_layer_norm_by_hand():
    x = torch.tensor([[1.0, 2.0, 3.0, 6.0]], dtype=P.F)                  # mean 3, squared deviations 4 1 0 9: variance 3.5
    got = P.layer_norm(x, torch.tensor([1.0, 2.0, 1.0, 1.0], dtype=P.F), torch.tensor([0.0, 0.0, 5.0, 0.0], dtype=P.F), 0.5)
    assert torch.allclose(got, torch.tensor([[-1.0, -1.0, 5.0, 1.5]], dtype=P.F))      # the eps stands inside the root: sqrt(4) = 2


def test_the_shift_reads_the_row_before_as_it_was():
    h = torch.tensor([[2.0, 4.0], [6.0, 8.0], [10.0, 0.0]], dtype=P.F)
    got = P.towards_the_token_before(h, torch.tensor([0.5, 1.0], dtype=P.F))
    assert torch.equal(got, torch.tensor([[1.0, 0.0], [4.0, 4.0], [8.0, 8.0]], dtype=P.F))


def test_rotation_turns_neighbours_and_leaves_the_rest():
    u = torch.zeros(2, 1, 6, dtype=P.F)
    u[:, 0] = torch.tensor([1.0, 0.0, 0.0, 2.0, 7.0, 9.0])
    freqs = torch.tensor([math.pi / 2, math.pi], dtype=P.F)
    got = P.rotate_neighbours(u, [0, 1], freqs, 2.0)
    assert torch.allclose(got[0, 0], torch.tensor([2.0, 0.0, 0.0, 4.0, 7.0, 9.0], dtype=P.F))            # angle 0: only the magnitude
    assert torch.allclose(got[1, 0], torch.tensor([0.0, 2.0, 0.0, -4.0, 7.0, 9.0], dtype=P.F), atol=1e-12)
    # the product of a rotated query and key depends on their distance alone
    q, k = torch.randn(1, 1, 6, dtype=P.F), torch.randn(1, 1, 6, dtype=P.F)
    freqs, _ = P.rotary_frequencies(4, 100.0)
    dots = [float((P.rotate_neighbours(q, [a + 5], freqs, 1.0) * P.rotate_neighbours(k, [a], freqs, 1.0)).sum()) for a in (0, 3, 40)]
    assert max(dots) - min(dots) < 1e-12


def test_stretched_frequencies():
    plain, one = P.rotary_frequencies(8, 10000.0)
    assert one == 1.0 and torch.allclose(plain, torch.tensor([1.0, 0.1, 0.01, 0.001], dtype=P.F))
    # c(t) = 8 ln(64 / (2 pi t)) / (2 ln 10000): c(16) < 0 so lo = 0, c(2) = 0.707 so hi = 1: pair 0 stays, the others are slowed
    got, magnitude = P.rotary_frequencies(8, 10000.0, {"factor": 8.0, "original": 64, "fast": 16.0, "slow": 2.0})
    assert torch.allclose(got, torch.tensor([1.0, 0.1 / 8, 0.01 / 8, 0.001 / 8], dtype=P.F))
    assert abs(magnitude - (0.1 * math.log(8.0) + 1.0)) < 1e-15
    # lo = hi: the ramp's width is held at 0.001, a step from 0 to 1 between two pairs
    got, _ = P.rotary_frequencies(8, 10000.0, {"factor": 2.0, "original": 64, "fast": 2.0, "slow": 2.0})
    assert float(got[0]) == 1.0 and abs(float(got[1]) - 0.05) < 1e-15


def test_buckets_of_distance():
    rows, far = 12, 90
    assert [P.distance_bucket(n, rows, far) for n in range(6)] == list(range(6))       # below half the rows: the distance itself
    assert P.distance_bucket(6, rows, far) == 6 and P.distance_bucket(89, rows, far) == 11 and P.distance_bucket(10 ** 6, rows, far) == 11
    buckets = [P.distance_bucket(n, rows, far) for n in range(200)]
    assert buckets == sorted(buckets) and set(buckets) == set(range(12))
    # a step of the logarithm: 6 * 15^(k / 6) is where bucket 6 + k begins
    for k in range(1, 6):
        edge = 6 * 15 ** (k / 6)
        assert P.distance_bucket(math.ceil(edge), rows, far) == 6 + k and P.distance_bucket(math.ceil(edge) - 1, rows, far) == 6 + k - 1
    assert [P.distance_bucket(n, 7, 20) for n in (2, 3, 4, 19, 20)] == [2, 3, 3, 6, 6]   # an odd number of rows: half is 3, four rows beyond


def test_sigmoid_weights_are_not_shared_between_keys():
    """With scores of zero every visible key weighs 1/2 whatever their number: the output grows with the window."""
    T, W = 6, 4
    m = {"heads": 1, "kv_heads": 1, "dim": 4, "vdim": 4, "scale": 1.0, "mask": {"size": 3}}
    t = {"q": torch.zeros(4, W), "q.b": torch.zeros(4), "k": torch.zeros(4, W), "k.b": torch.zeros(4), "v": torch.zeros(4, W),
         "v.b": torch.ones(4), "talk": torch.ones(1, 1), "pb": torch.zeros(1), "g": torch.zeros(1, W), "o": torch.eye(4), "o.b": torch.zeros(4)}
    t = {"p." + k: v.to(P.F) for k, v in t.items()}
    out, _ = P.gated_sigmoid_attention(torch.randn(T, W, dtype=P.F), list(range(T)), m, t, "p.", None)
    # keys seen: 1, 2, 3, 3, 3, 3; each weighs 1/2, values are ones, the gate is sigmoid(0) = 1/2
    assert torch.allclose(out[:, 0], torch.tensor([0.25, 0.5, 0.75, 0.75, 0.75, 0.75], dtype=P.F))


def test_the_first_layer_that_shares_values_gives_them_unblended():
    raw = {"architecture": "Ledudra", "vocab": 11, "width": 8, "norm": {"eps": 1e-5}, "residual_mult": 1.0, "layers": [
        {"type": "attention_2", "mlp": None, "mixer": {"heads": 2, "kv_heads": 1, "dim": 4, "vdim": 4, "scale": 0.5, "v_mix": True, "bias_max": 5}},
        {"type": "attention_2", "mlp": None, "mixer": {"heads": 2, "kv_heads": 1, "dim": 4, "vdim": 4, "scale": 0.5, "v_mix": True, "bias_max": 5}}]}
    generator = torch.Generator().manual_seed(0)
    rand = lambda *shape: torch.randn(*shape, generator=generator, dtype=P.F)
    t = {"embed": rand(11, 8), "final.norm": torch.ones(8, dtype=P.F), "final.norm.b": torch.zeros(8, dtype=P.F), "head": rand(11, 8)}
    for i in range(2):
        p = f"l{i}."
        for n in ("norm1", "norm1b"):
            t[p + n], t[p + n + ".b"] = torch.ones(8, dtype=P.F), torch.zeros(8, dtype=P.F)
        t[p + "shift"] = torch.zeros(8, dtype=P.F)
        t.update({p + "mix.q": rand(8, 8), p + "mix.k": rand(4, 8), p + "mix.v": rand(4, 8), p + "mix.o": rand(8, 8),
                  p + "mix.q.norm": torch.ones(4, dtype=P.F), p + "mix.k.norm": torch.ones(4, dtype=P.F), p + "mix.rel": rand(4, 2),
                  p + "mix.vmix": torch.tensor(0.0, dtype=P.F)})
    tokens = [3, 1, 4, 1, 5]
    base = P.forward(raw, t, tokens)
    t["l0.mix.vmix"] = torch.tensor(0.9, dtype=P.F)                      # the first such layer's own share is not used
    assert torch.equal(P.forward(raw, t, tokens), base)
    t["l1.mix.vmix"] = torch.tensor(0.9, dtype=P.F)                      # the second layer's is
    assert not torch.allclose(P.forward(raw, t, tokens), base)


# ---- the configuration ------------------------------------------------------------------------------------------

def test_configurations_parse_and_come_back():
    from xeno_rt_amd.config import parse_config
    for raw in CONFIGS.values():
        config = parse_config(raw)
        assert config.architecture == "Ledudra" and config.vocab_size == raw["vocab"] and config.num_hidden_layers == len(raw["layers"])
        assert parse_config(config.to_dict()) == config


def test_a_configuration_that_cannot_be_is_refused():
    import copy
    from xeno_rt_amd.config import ConfigError, parse_config
    good = CONFIGS["mixed"]

    def broken(change):
        raw = copy.deepcopy(good)
        change(raw)
        return raw

    cases = [lambda r: r["layers"][0].update(type="retention"),
             lambda r: r["layers"][0]["mixer"].update(heads=5),                         # 5 heads on 3 key/value heads
             lambda r: r["layers"][0]["mixer"]["rot"].update(dims=7),
             lambda r: r["layers"][0]["mixer"]["rot"].update(dims=22),                  # more than the head has
             lambda r: r["layers"][1]["mixer"].pop("bias_max"),
             lambda r: r["layers"][2]["mixer"].update(vdim=20),                         # 40 shared numbers where the first layer has 36
             lambda r: r["layers"][0]["mlp"].update(kind="experts"),
             lambda r: r.pop("norm"),
             lambda r: r["layers"][0]["mixer"].pop("scale")]
    for change in cases:
        with pytest.raises(ConfigError):
            parse_config(broken(change))


def test_the_model_declares_the_designs_tensors():
    from xeno_rt_amd.config import architecture, parse_config
    config = parse_config(CONFIGS["mixed"])
    spec = architecture("Ledudra").build(config)
    names = spec.weight_specs()
    assert names["l0.mix.talk"].shape == (6, 6) and names["l0.mix.g"].shape == (6, 40) and names["l0.mix.o.b"].shape == (40,)
    assert names["l1.mix.rel"].shape == (10, 4) and names["l1.mix.q.norm"].shape == (24,) and "l1.mix.q.b" not in names
    assert names["l0.mix.vmix"].shape == () and "l1.norm2" not in names and names["l2.norm2b.b"].shape == (40,)
    needs = spec.cache_needs()
    assert [need.kv.window for need in needs] == [17, 70, None] and [need.kv.value_width for need in needs] == [12, 36, 18]
    assert all(dict(need.states)["shift"].shape == (1, 40) for need in needs)
    assert spec.capturable()


def test_a_layer_that_shares_no_values_may_still_carry_its_share():
    """A checkpoint may hold the share of a blend for a layer that blends nothing in: the model lists it as not read."""
    import copy
    from xeno_rt_amd.config import architecture, parse_config
    from xeno_rt_amd.weights.loader import check_names
    raw = copy.deepcopy(CONFIGS["wide"])
    raw["layers"][3]["mixer"].pop("v_mix")                              # (absent means no)
    spec = architecture("Ledudra").build(parse_config(raw))
    assert sorted(spec.ignored_names()) == ["l2.mix.vmix", "l3.mix.vmix"]
    names = spec.weight_specs()
    assert "l0.mix.vmix" in names and "l1.mix.vmix" in names and "l2.mix.vmix" not in names
    found = {name: ("BF16", tuple(s.shape)) for name, s in names.items()}
    found["l3.mix.vmix"] = ("BF16", ())
    check_names("a folder", names, found, spec.ignored_names())
