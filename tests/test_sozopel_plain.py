"""The plain Sozopel implementation against closed forms and hand-made cases, and the design's configuration; no GPU."""
import json
import math

import pytest
import torch

import plain_sozopel as P
from sozopel_models import CONFIGS, make_sozopel_folder


def test_convolution_looks_back_and_never_ahead():
    u = torch.zeros(6, 2, dtype=torch.float64)
    u[2] = 1.0
    w = torch.tensor([[1.0, 10.0, 100.0], [2.0, 20.0, 200.0]], dtype=torch.float64)
    y = P.causal_conv(u, w)
    assert y[:, 0].tolist() == [0, 0, 100, 10, 1, 0] and y[:, 1].tolist() == [0, 0, 200, 20, 2, 0]


def test_recurrence_without_decay_is_a_running_sum():
    generator = torch.Generator().manual_seed(0)
    T, H, dim, vdim = 7, 2, 3, 4
    q, k, v = (torch.randn(T, H, d, generator=generator, dtype=torch.float64) for d in (dim, dim, vdim))
    ones = torch.ones(T, H, dim, dtype=torch.float64)
    got = P.recurrence(q, k, v, ones)
    for t in range(T):
        for h in range(H):
            want = sum((q[t, h] @ k[s, h]) * v[s, h] for s in range(t + 1))
            assert torch.allclose(got[t, h], want)
    # with a bonus the current token counts u-fold and the tokens before it as they are
    u = torch.full((H, dim), 3.0, dtype=torch.float64)
    got = P.recurrence(q, k, v, ones, bonus=u)
    for t in range(T):
        want = sum((q[t, 0] @ k[s, 0]) * v[s, 0] for s in range(t)) + 3.0 * (q[t, 0] @ k[t, 0]) * v[t, 0]
        assert torch.allclose(got[t, 0], want)


def test_a_decay_acts_on_the_rows_of_the_key_channels():
    q = torch.tensor([[[0.0, 0.0]], [[1.0, 1.0]]], dtype=torch.float64)
    k = torch.tensor([[[1.0, 1.0]], [[0.0, 0.0]]], dtype=torch.float64)
    v = torch.tensor([[[5.0]], [[0.0]]], dtype=torch.float64)
    decay = torch.tensor([[[1.0, 1.0]], [[0.5, 0.25]]], dtype=torch.float64)
    assert float(P.recurrence(q, k, v, decay)[1, 0, 0]) == 5.0 * 0.5 + 5.0 * 0.25


def test_xielu_is_continuous_with_slope_one_half_at_zero_and_quadratic_above():
    p, q = torch.tensor(0.4, dtype=torch.float64), torch.tensor(-0.2, dtype=torch.float64)
    z = torch.tensor([-1e-6, 0.0, 1e-6, 2.0], dtype=torch.float64)
    y = P.xielu(z, p, q)
    assert abs(float(y[1])) == 0.0 and abs(float(y[2] - y[0]) / 2e-6 - 0.5) < 1e-5
    assert abs(float(y[3]) - (math.log1p(math.exp(0.4)) * 4.0 + 1.0)) < 1e-12
    assert abs(float(P.xielu(torch.tensor(-50.0, dtype=torch.float64), p, q)) - ((0.5 + math.log1p(math.exp(-0.2))) * 49.0 - 25.0)) < 1e-9


def test_the_norm_has_eps_inside_the_root():
    x = torch.tensor([[3.0, 4.0]], dtype=torch.float64)
    assert torch.allclose(P.rms_divide(x, 0.5), x / math.sqrt(12.5 + 0.5))


@pytest.fixture(scope="module")
def mixed(tmp_path_factory):
    folder = make_sozopel_folder(CONFIGS["mixed"], tmp_path_factory.mktemp("mixed"), seed=3)
    return folder, P.PlainModel(folder)


def test_the_plain_model_is_causal_and_windowed(mixed):
    _, plain = mixed
    ids = [5, 9, 2, 77, 31, 8, 8, 40, 3, 60, 11, 12]
    whole = plain.logits(ids)
    assert torch.allclose(plain.logits(ids[:7]), whole[:7], atol=1e-6)


def test_configuration_round_trip_and_registry(mixed):
    from xeno_rt_amd.config import ConfigError, architecture, load_config, parse_config
    folder, _ = mixed
    config = load_config(folder)
    assert config.architecture == "Sozopel" and config.vocab_size == 101 and config.max_position_embeddings == 320
    assert parse_config(config.to_dict()) == config
    spec = architecture("Sozopel").build(config)
    assert [call.layer for call in spec.schedule] == [0, 1, 2]
    names = set(spec.weight_specs())
    assert {"embed", "pos", "head", "final.norm", "l0.canon1", "l0.canon2", "l0.mix.left.q.conv", "l0.mix.right.a2.b",
            "l1.mix.g", "l2.mix.mu.w", "l2.mix.u", "l2.canon1"} <= names and "l2.canon2" not in names and "l2.norm2" not in names
    needs = spec.cache_needs()
    assert needs[0].kv.window == 17 and needs[0].kv.value_width == 40 and needs[1].kv is None
    assert dict(needs[2].states)["mix.state"].shape == (2, 24, 24)
    for broken, message in (({"layers": []}, "layers"), ({"canon": {"taps": 0}}, "taps"), ({"width": -1}, "width")):
        with pytest.raises(ConfigError, match=message):
            parse_config({**CONFIGS["mixed"], **broken})
    raw = json.loads(json.dumps(CONFIGS["mixed"]))
    raw["layers"][1]["mixer"]["decay"] = [0.5]
    with pytest.raises(ConfigError, match="decay"):
        parse_config(raw)
    raw = json.loads(json.dumps(CONFIGS["mixed"]))
    raw["layers"][0]["type"] = "convolution"
    with pytest.raises(ConfigError, match="type"):
        parse_config(raw)


def test_inner_widths_are_read_from_the_shapes(tmp_path):
    from xeno_rt_amd.config import ConfigError, architecture, load_config
    from xeno_rt_amd.weights import tensor_shapes
    folder = make_sozopel_folder(CONFIGS["wide"], tmp_path, seed=4, keep_rank=False)
    config = load_config(folder)
    with pytest.raises(ConfigError, match="rank"):
        architecture("Sozopel").build(config)
    complete = config.completed_from(tensor_shapes(folder))
    assert complete.layers[0]["mixer"]["rank"] == 8 and complete.layers[3]["mixer"]["right"]["rank"] == 16
    assert set(architecture("Sozopel").build(complete).weight_specs()) == set(tensor_shapes(folder))
