"""The plain Depunex implementation against closed forms and hand-made cases, and the design's configuration; no GPU."""
import json
import math

import pytest
import torch

import plain_depunex as P
from depunex_models import CONFIGS, make_depunex_folder

F = torch.float64


def test_the_hashed_row_of_a_pair_and_of_a_first_token():
    assert P.bigram_rows([5, 9, 9, 0], 7, 3, 2) == [7, (5 * 3 + 9 * 2) % 7, (9 * 3 + 9 * 2) % 7, (9 * 3) % 7]


def test_the_convolution_looks_back_and_never_ahead_and_adds_its_bias_before_silu():
    u = torch.zeros(6, 2, dtype=F)
    u[2] = 1.0
    w = torch.tensor([[1.0, 10.0, 100.0], [2.0, 20.0, 200.0]], dtype=F)
    b = torch.tensor([0.5, -0.5], dtype=F)
    y = P.causal_conv_silu(u, w, b)
    want = torch.tensor([[0, 0, 100, 10, 1, 0], [0, 0, 200, 20, 2, 0]], dtype=F).T + b
    assert torch.allclose(y, want * torch.sigmoid(want))


def test_a_state_without_decay_is_a_running_sum_of_stepped_inputs():
    """Mamba-2 with A_log = -inf (no decay), one head, no convolution effect beyond a tap of one: y_t = sum_s dt_s (B_s . C_t) x_s + D x_t."""
    torch.manual_seed(0)
    tokens, vdim, n, width = 5, 3, 4, 6
    m = {"heads": 1, "vdim": vdim, "state": n, "groups": 1, "norm_groups": 1, "conv": 1}
    p = {"in": torch.randn(2 * vdim + 2 * n + 1, width, dtype=F), "conv": torch.ones(vdim + 2 * n, 1, dtype=F),
         "conv.b": torch.zeros(vdim + 2 * n, dtype=F), "dt_bias": torch.tensor([0.3], dtype=F), "A_log": torch.tensor([-800.0], dtype=F),
         "D": torch.tensor([0.7], dtype=F), "norm": torch.ones(vdim, dtype=F), "o": torch.eye(vdim, dtype=F)}
    h = torch.randn(tokens, width, dtype=F)
    proj = h @ p["in"].T
    z, xbc, dt = proj[:, :vdim], P.silu(proj[:, vdim:2 * vdim + 2 * n]), P.softplus(proj[:, -1] + 0.3)
    x, b, c = xbc[:, :vdim], xbc[:, vdim:vdim + n], xbc[:, vdim + n:]
    y = torch.stack([sum(dt[s] * (b[s] @ c[t]) * x[s] for s in range(t + 1)) + 0.7 * x[t] for t in range(tokens)])
    want = P.rms_divided(y * P.silu(z), 1e-5)
    assert torch.allclose(P.mamba2(h, p, m, 1e-5), want)


def test_a_channel_of_the_selective_scan_decays_by_its_own_step():
    """One channel with one entry of state, every projection a single number, worked out with Python floats."""
    silu = lambda z: z / (1 + math.exp(-z))
    softplus = lambda z: math.log1p(math.exp(z))
    p = {"in": torch.eye(2, dtype=F), "conv": torch.ones(1, 1, dtype=F), "conv.b": torch.tensor([0.2], dtype=F),
         "x": torch.tensor([[0.5], [-1.5], [2.0]], dtype=F), "dt": torch.tensor([[3.0]], dtype=F), "dt.b": torch.tensor([-0.4], dtype=F),
         "A_log": torch.tensor([[0.3]], dtype=F), "D": torch.tensor([0.1], dtype=F), "o": torch.tensor([[2.0]], dtype=F)}
    h = torch.tensor([[1.0, 0.5], [-0.7, 1.5], [0.3, -2.0], [2.0, 0.1]], dtype=F)
    state, want = 0.0, []
    for x_in, z in h.tolist():
        x = silu(x_in + 0.2)
        dt = softplus(3.0 * 0.5 * x - 0.4)
        state = math.exp(-math.exp(0.3) * dt) * state + dt * x * (-1.5 * x)
        want.append((state * 2.0 * x + 0.1 * x) * silu(z) * 2.0)
    got = P.mamba(h, p, {"inner": 1, "state": 1, "dt_rank": 1})
    assert got[:, 0].tolist() == pytest.approx(want)


def test_frequencies_stay_are_divided_or_blended_by_their_wavelength():
    scaling = {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 64}
    plain = P.rotary_frequencies(12, 1000.0, None)
    got = P.rotary_frequencies(12, 1000.0, scaling)
    assert got[0] == plain[0] and got[5] == plain[5] / 8.0                 # wavelengths 6.3 (< 16) and 1987 (> 64)
    wavelength = 2 * math.pi / plain[1]                                       # 19.9: between
    share = (64 / wavelength - 1.0) / 3.0
    assert got[1] == pytest.approx((1 - share) * plain[1] / 8.0 + share * plain[1]) and plain[1] / 8.0 < got[1] < plain[1]


def test_the_rotation_pairs_the_halves_of_the_first_dims_and_passes_the_rest():
    x = torch.zeros(2, 1, 6, dtype=F)
    x[1, 0] = torch.tensor([1.0, 2.0, 3.0, 4.0, 5.0, 6.0])
    f = [0.5, 0.25]
    y = P.rotate(x, 4, f)[1, 0]
    assert y[4:].tolist() == [5.0, 6.0]
    assert float(y[0]) == pytest.approx(1.0 * math.cos(0.5) - 3.0 * math.sin(0.5)) and float(y[2]) == pytest.approx(3.0 * math.cos(0.5) + 1.0 * math.sin(0.5))
    assert float(y[1]) == pytest.approx(2.0 * math.cos(0.25) - 4.0 * math.sin(0.25))


def test_a_query_sees_its_own_chunk_only():
    """All keys alike but for their values: the output is the mean of the values from the chunk's first position to the query."""
    tokens, size = 11, 4
    m = {"heads": 1, "kv_heads": 1, "dim": 2, "vdim": 1, "scale": 1.0, "mask": {"size": size}}
    p = {"q": torch.zeros(2, 3, dtype=F), "k": torch.zeros(2, 3, dtype=F), "v": torch.tensor([[1.0, 0.0, 0.0]], dtype=F), "o": torch.eye(1, dtype=F)}
    h = torch.zeros(tokens, 3, dtype=F)
    h[:, 0] = torch.arange(tokens, dtype=F)
    got = P.chunked_attention(h, p, m)[:, 0]
    for i in range(tokens):
        first = i - i % size
        assert float(got[i]) == pytest.approx(sum(range(first, i + 1)) / (i + 1 - first))


def test_experts_are_chosen_inside_the_best_groups_and_their_weights_sum_to_one():
    # scores per expert (through the router): groups {0,1}, {2,3}, {4,5}; group scores .9+.1, .6+.5, .8+.05 -> groups 1 and 0 stay
    scores = torch.tensor([[0.9, 0.1, 0.6, 0.5, 0.8, 0.05]], dtype=F)
    logits = torch.log(scores / (1 - scores))
    chosen, weights = P.route(torch.eye(1, dtype=F), logits.T, 6, 2, 3, 2)
    assert chosen.tolist() == [[0, 2]] and weights[0].tolist() == pytest.approx([0.9 / 1.5, 0.6 / 1.5])
    chosen, _ = P.route(torch.eye(1, dtype=F), logits.T, 6, 3, 3, 2)
    assert chosen.tolist() == [[0, 2, 3]]                                    # expert 4 (0.8) is outside the kept groups
    chosen, _ = P.route(torch.eye(1, dtype=F), logits.T, 6, 3)
    assert chosen.tolist() == [[0, 4, 2]]                                    # without groups it is taken


def test_the_dense_feed_forward_clamps_before_it_multiplies():
    p = {"gate": torch.tensor([[1.0]], dtype=F), "up": torch.tensor([[1.0]], dtype=F), "down": torch.tensor([[1.0]], dtype=F)}
    y = P.dense_ff(torch.tensor([[5.0], [-5.0], [0.5]], dtype=F), p, {"limit": 2.0})[:, 0]
    sig = lambda g: 1 / (1 + math.exp(-1.702 * g))
    assert y.tolist() == pytest.approx([2.0 * sig(2.0) * 3.0, -5.0 * sig(-5.0) * (-2.0 + 1.0), 0.5 * sig(0.5) * 1.5])


@pytest.fixture(scope="module")
def mixed(tmp_path_factory):
    folder = make_depunex_folder(CONFIGS["mixed"], tmp_path_factory.mktemp("mixed"), seed=3)
    return folder, P.PlainModel(folder)


def test_the_plain_model_is_causal_and_its_logits_are_capped(mixed):
    _, plain = mixed
    ids = [5, 9, 2, 77, 31, 8, 8, 40, 3, 60, 11, 12] * 3
    whole = plain.logits(ids)
    assert torch.allclose(plain.logits(ids[:7]), whole[:7], atol=1e-6)
    assert float(whole.abs().max()) < CONFIGS["mixed"]["logit_softcap"]


def test_configuration_round_trip_registry_and_what_the_layers_keep(mixed):
    from xeno_rt_amd.config import ConfigError, architecture, load_config, parse_config
    folder, _ = mixed
    config = load_config(folder)
    assert config.architecture == "Depunex" and config.vocab_size == 97 and config.hidden_size == 48 and config.bigram == (53, 7, 13)
    assert parse_config(config.to_dict()) == config
    spec = architecture("Depunex").build(config)
    names = set(spec.weight_specs())
    assert {"embed", "bigram", "side.embed", "final.norm", "l0.norm1", "l0.ls1", "l0.ls2", "l0.mix.left.q", "l0.mix.right.conv.b", "l0.mix.right.dt.b",
            "l0.mlp.router", "l0.mlp.e7.down", "l1.mix.dt_bias", "l1.mix.conv.b", "l1.mlp.gate", "l2.side.gate", "l2.ls1"} <= names
    assert "l2.ls2" not in names and "head" not in names and not any(name.startswith("l2.mlp") for name in names)
    assert spec.weight_specs()["bigram"].shape == (54, 48) and spec.weight_specs()["side.embed"].shape == (97, 18)
    needs = spec.cache_needs()
    assert len(needs) == 4 and needs[0].kv.head_dim == 24 and needs[0].kv.value_width == 16 and needs[1].kv is None
    assert dict(needs[0].states)["mix.right.state"].shape == (40, 10) and dict(needs[1].states)["mix.state"].shape == (4, 20, 12)
    assert dict(needs[1].states)["mix.state.conv"].shape == (3, 12 * 4 + 2 * 2 * 20)
    assert dict(needs[3].states)["token_before"].dtype == torch.int32 and spec.cache_sources() == [0, 1, 2, 3]
    wide = architecture("Depunex").build(parse_config(CONFIGS["wide"]))
    assert "bigram" not in wide.weight_specs() and "side.embed" not in wide.weight_specs() and wide.head.softcap is None
    for path, value, message in ((("layers",), [], "layers"), (("width",), -1, "width"), (("layers", 0, "type"), "attention", "type"),
                                 (("layers", 1, "mixer", "groups"), 3, "groups"), (("layers", 1, "mixer", "norm_groups"), 5, "norm groups"),
                                 (("layers", 0, "mlp", "router", "top"), 5, "chosen"), (("layers", 0, "mixer", "left", "kv_heads"), 3, "key/value"),
                                 (("layers", 0, "mixer", "left", "rot", "dims"), 26, "rotated"), (("layers", 1, "mlp", "limit"), 0, "limit")):
        raw = json.loads(json.dumps(CONFIGS["mixed"]))
        at = raw
        for key in path[:-1]:
            at = at[key]
        at[path[-1]] = value
        with pytest.raises(ConfigError, match=message):
            parse_config(raw)
