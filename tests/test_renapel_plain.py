"""The plain Renapel implementation (tests/plain_renapel.py) against closed forms and cases worked out by hand, and the
configuration class. No GPU."""
import copy
import math

import pytest
import torch

import plain_renapel as P
from renapel_models import CONFIGS, make_renapel_folder

F = torch.float64


def rand(*shape, seed=0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=F)


# ---- the copies of the residual stream ---------------------------------------------------------------------------------------

def test_copies_with_an_identity_mix_are_a_plain_residual_stream():
    X = rand(3, 5, 7)
    y = rand(5, 7, seed=1)
    new = P.copies_write(X, y, torch.eye(3, dtype=F), torch.tensor([1.0, 0.0, 2.0], dtype=F))
    assert torch.allclose(new[0], X[0] + y) and torch.allclose(new[1], X[1]) and torch.allclose(new[2], X[2] + 2 * y)
    assert torch.allclose(P.copies_read(X, torch.tensor([0.0, 1.0, 0.0])), X[1])


def test_the_mix_is_indexed_from_to():
    X = rand(2, 4, 3)
    mix = torch.tensor([[0.0, 1.0], [0.0, 0.0]], dtype=F)           # copy 0 goes to copy 1, nothing else moves
    new = P.copies_write(X, torch.zeros(4, 3, dtype=F), mix, torch.zeros(2, dtype=F))
    assert torch.allclose(new[1], X[0]) and torch.allclose(new[0], torch.zeros(4, 3, dtype=F))


# ---- lightning attention ---------------------------------------------------------------------------------------------------------

def test_lightning_is_a_decayed_sum_of_outer_products():
    tokens, width, heads, d, e = 9, 6, 2, 3, 4
    p = {"q": rand(heads * d, width, seed=1), "k": rand(heads * d, width, seed=2), "v": rand(heads * e, width, seed=3),
         "g": rand(heads * e, width, seed=4), "o": torch.eye(heads * e, dtype=F), "norm": torch.ones(heads * e, dtype=F)}
    m = {"heads": heads, "dim": d, "vdim": e, "decay": [0.5, 1.0]}
    h = rand(tokens, width, seed=5)
    got = P.lightning(h, p, m, 1e-6)
    q, k, v = (P.silu(h @ p[n].T) for n in "qkv")
    raw = torch.zeros(tokens, heads * e, dtype=F)
    for t in range(tokens):
        for head in range(heads):
            for j in range(t + 1):
                weight = m["decay"][head] ** (t - j) * (q[t, head * d:(head + 1) * d] @ k[j, head * d:(head + 1) * d])
                raw[t, head * e:(head + 1) * e] += weight * v[j, head * e:(head + 1) * e]
    want = raw / torch.sqrt((raw * raw).mean(dim=-1, keepdim=True) + 1e-6) * torch.sigmoid(h @ p["g"].T)
    assert torch.allclose(got, want, atol=1e-12)


# ---- the softmax with a sink -------------------------------------------------------------------------------------------------------

def test_the_sink_counts_once_in_the_denominator():
    scores = torch.zeros(1, 1, 5, dtype=F)
    weights = P.softmax_with_sink(scores, torch.tensor([math.log(3.0)], dtype=F))
    assert torch.allclose(weights, torch.full((1, 1, 5), 1.0 / 8.0, dtype=F))
    plain = P.softmax_with_sink(rand(2, 3, 4), torch.tensor([-math.inf, -math.inf], dtype=F))
    assert torch.allclose(plain.sum(dim=-1), torch.ones(2, 3, dtype=F))


def test_buckets_of_distance_by_hand():
    # 8 rows that end at distance 64: the distances below 4 have a row each, then rows 4 .. 7 begin at 4, 8, 16 and 32
    want = {0: 0, 1: 1, 3: 3, 4: 4, 7: 4, 8: 5, 15: 5, 16: 6, 31: 6, 32: 7, 63: 7, 64: 7, 5000: 7}
    for n, row in want.items():
        assert P.distance_bucket(n, 8, 64) == row, n
    assert [P.distance_bucket(n, 4, 9) for n in range(10)] == [0, 1, 2, 2, 2, 3, 3, 3, 3, 3]


def test_the_query_temperature_grows_in_steps():
    temps = P.query_temperature(10, 0.5, 4)
    assert torch.allclose(temps[:3], torch.ones(3, dtype=F))                         # positions 0, 1, 2: (p + 1) // 4 = 0
    assert abs(float(temps[3]) - (1 + 0.5 * math.log(2))) < 1e-15 and abs(float(temps[7]) - (1 + 0.5 * math.log(3))) < 1e-15


def attention_tensors(width, heads, kv_heads, d, e, rows, seed=0):
    return {"q": rand(heads * d, width, seed=seed), "q.b": rand(heads * d, seed=seed + 1), "k": rand(kv_heads * d, width, seed=seed + 2),
            "k.b": rand(kv_heads * d, seed=seed + 3), "v": rand(kv_heads * e, width, seed=seed + 4), "v.b": rand(kv_heads * e, seed=seed + 5),
            "rel": rand(rows, heads, seed=seed + 6), "sink": rand(heads, seed=seed + 7), "o": rand(width, heads * e, seed=seed + 8)}


def test_attention_token_by_token_by_hand():
    width, heads, kv_heads, d, e, tokens = 8, 4, 2, 6, 5, 12
    m = {"heads": heads, "kv_heads": kv_heads, "dim": d, "vdim": e, "scale": 0.4, "bias_max": 9, "q_temp": {"coef": 0.3, "every": 3}}
    p = attention_tensors(width, heads, kv_heads, d, e, rows=4)
    h = rand(tokens, width, seed=20)
    got = P.attention(h, p, m, 1e-5)
    rms = lambda x: x / math.sqrt(float((x * x).mean()) + 1e-5)
    out = torch.zeros(tokens, heads * e, dtype=F)
    for i in range(tokens):
        for head in range(heads):
            g = head // (heads // kv_heads)
            q = rms(h[i] @ p["q"][head * d:(head + 1) * d].T + p["q.b"][head * d:(head + 1) * d]) * (1 + 0.3 * math.log((i + 1) // 3 + 1))
            terms, values = [], []
            for j in range(i + 1):
                k = rms(h[j] @ p["k"][g * d:(g + 1) * d].T + p["k.b"][g * d:(g + 1) * d])
                terms.append(float(q @ k) * 0.4 + float(p["rel"][P.distance_bucket(i - j, 4, 9), head]))
                values.append(h[j] @ p["v"][g * e:(g + 1) * e].T + p["v.b"][g * e:(g + 1) * e])
            denominator = sum(math.exp(s) for s in terms) + math.exp(float(p["sink"][head]))
            out[i, head * e:(head + 1) * e] = sum(math.exp(s) / denominator * v for s, v in zip(terms, values))
    assert torch.allclose(got, out @ p["o"].T, atol=1e-10)


# ---- attention through a latent --------------------------------------------------------------------------------------------------

def test_rotation_of_neighbours_keeps_lengths_and_sees_distances_only():
    x, y = rand(1, 8, seed=1), rand(1, 8, seed=2)
    a = P.rotate_neighbours(torch.cat([torch.zeros(5, 8, dtype=F), x]), 6, 100.0)[5]
    b = P.rotate_neighbours(torch.cat([torch.zeros(2, 8, dtype=F), y]), 6, 100.0)[2]
    c = P.rotate_neighbours(torch.cat([torch.zeros(9, 8, dtype=F), x]), 6, 100.0)[9]
    e = P.rotate_neighbours(torch.cat([torch.zeros(6, 8, dtype=F), y]), 6, 100.0)[6]
    assert abs(float(a @ b) - float(c @ e)) < 1e-12                  # both pairs are three positions apart
    assert torch.allclose(a[6:], x[0, 6:]) and abs(float(a[:2].norm()) - float(x[0, :2].norm())) < 1e-12
    first = P.rotate_neighbours(torch.cat([torch.zeros(1, 2, dtype=F), torch.tensor([[1.0, 0.0]], dtype=F)]), 2, 10.0)[1]
    assert torch.allclose(first, torch.tensor([math.cos(1.0), math.sin(1.0)], dtype=F))   # (u, v) -> (u cos - v sin, v cos + u sin)


def test_latent_attention_through_the_cached_row_alone():
    """The same scores and outputs from what a cache keeps (the latent and the turned key part): the plain part of a query
    through its head's key matrix transposed, the weighted latents through the head's value matrix."""
    width, heads, d, r, e, rank, q_rank, tokens = 10, 3, 4, 6, 5, 7, 9, 11
    m = {"heads": heads, "dim": d, "rot_dim": r, "vdim": e, "kv_rank": rank, "q_rank": q_rank, "scale": 0.3, "rot": {"dims": 4, "base": 50.0}}
    p = {"dq": rand(q_rank, width, seed=1), "dq.norm": rand(q_rank, seed=2), "uq": rand(heads * (d + r), q_rank, seed=3),
         "dkv": rand(rank + r, width, seed=4), "dkv.norm": rand(rank, seed=5), "uk": rand(heads * d, rank, seed=6),
         "uv": rand(heads * e, rank, seed=7), "sink": rand(heads, seed=8), "o": rand(width, heads * e, seed=9)}
    h = rand(tokens, width, seed=10)
    got = P.latent_attention(h, p, m, 1e-6)
    q = (P.rms_norm(h @ p["dq"].T, p["dq.norm"], 1e-6) @ p["uq"].T).reshape(tokens, heads, d + r)
    down = h @ p["dkv"].T
    latent = P.rms_norm(down[:, :rank], p["dkv.norm"], 1e-6)
    row = torch.cat([latent, P.rotate_neighbours(down[:, rank:], 4, 50.0)], dim=1)                      # what the cache keeps
    absorbed = torch.einsum("thd,hdr->thr", q[..., :d], p["uk"].reshape(heads, d, rank))
    full = torch.cat([absorbed, P.rotate_neighbours(q[..., d:], 4, 50.0)], dim=-1)
    scores = torch.einsum("ihc,jc->hij", full, row) * 0.3
    scores = scores.masked_fill(~P.causal_mask(tokens), -math.inf)
    summed = torch.einsum("hij,jr->ihr", P.softmax_with_sink(scores, p["sink"]), latent)
    out = torch.einsum("ihr,her->ihe", summed, p["uv"].reshape(heads, e, rank)).reshape(tokens, heads * e)
    assert torch.allclose(got, out @ p["o"].T, atol=1e-10)


# ---- experts --------------------------------------------------------------------------------------------------------------------------

def test_an_expert_outside_the_kept_groups_is_never_chosen():
    router = {"experts": 6, "top": 2, "scale": 2.5, "groups": {"count": 3, "keep": 2}}
    # one token whose logits are the router matrix's first column: groups (0, 1), (2, 3), (4, 5) score 5, 4, 3 by their best
    logits = torch.tensor([[5.0, 0.0, 4.0, 3.9, 3.0, 2.9]], dtype=F)
    weights = P.route(torch.ones(1, 1, dtype=F), logits.T.contiguous(), router)
    scores = torch.softmax(logits, dim=-1)
    assert (weights[0] > 0).tolist() == [True, False, True, False, False, False]
    assert abs(float(weights.sum()) - 2.5) < 1e-12
    assert abs(float(weights[0, 0]) - 2.5 * float(scores[0, 0] / (scores[0, 0] + scores[0, 2]))) < 1e-12
    # the third group's best (3.0) does not beat the second's (4.0): with all groups kept, expert 3 (3.9) is still the third choice
    router = {"experts": 6, "top": 3, "groups": {"count": 3, "keep": 3}}
    assert (P.route(torch.ones(1, 1, dtype=F), logits.T.contiguous(), router)[0] > 0).tolist() == [True, False, True, True, False, False]


def test_an_expert_clamps_gate_and_up():
    gate = torch.tensor([[10.0], [-10.0], [0.5]], dtype=F)
    up = torch.tensor([[10.0], [-10.0], [0.5]], dtype=F)
    down = torch.eye(3, dtype=F)
    y = P.expert(torch.ones(1, 1, dtype=F), gate, up, down, 2.0)[0]
    swish = lambda g: g / (1 + math.exp(-1.702 * g))
    assert abs(float(y[0]) - swish(2.0) * 3.0) < 1e-12               # both clamped from above
    assert abs(float(y[1]) - swish(-10.0) * (-2.0 + 1.0)) < 1e-12     # the gate is not clamped from below, up is
    assert abs(float(y[2]) - swish(0.5) * 1.5) < 1e-12


# ---- the whole model, and the configuration ------------------------------------------------------------------------------------

@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_configurations_round_trip_and_the_plain_model_runs(name, tmp_path):
    from xeno_rt_amd.config import parse_config
    from xeno_rt_amd.weights.loader import tensor_shapes
    raw = CONFIGS[name]
    config = parse_config(raw)
    assert parse_config(config.to_dict()) == config and config.streams == raw.get("streams")
    folder = make_renapel_folder(raw, tmp_path, seed=3, name_the_rows=False)
    from xeno_rt_amd.config import load_config
    loaded = load_config(folder)
    assert all("bias_rows" not in layer["mixer"] for layer in loaded.layers)
    assert loaded.completed_from(tensor_shapes(folder)) == config
    model = P.PlainModel(folder)
    streams = []
    with torch.no_grad():
        logits = P.forward(list(range(20)), model.tensors, model.raw, streams)
    assert logits.shape == (20, raw["vocab"]) and len(streams) == len(raw["layers"]) and torch.isfinite(logits).all()
    # causality: the first tokens' logits do not know of the later ones
    assert torch.allclose(model.logits(list(range(12))), logits[:12].float(), atol=1e-5)


def test_the_configuration_refuses_what_cannot_be_built():
    from xeno_rt_amd.config import ConfigError, parse_config

    def broken(change):
        raw = copy.deepcopy(CONFIGS["wide"])
        change(raw)
        with pytest.raises(ConfigError):
            parse_config(raw)

    broken(lambda raw: raw["layers"][2]["mixer"].update(kv_from=3))             # a later layer
    broken(lambda raw: raw["layers"][2]["mixer"].update(kv_from=0))             # a layer that is no softmax attention
    broken(lambda raw: raw["layers"][4]["mixer"].update(kv_from=2))             # a layer that has no keys of its own either
    broken(lambda raw: raw["layers"][2]["mixer"].update(dim=16))                # other sizes than the keys it would read
    broken(lambda raw: raw["layers"][0]["mixer"]["rot"].update(dims=7))         # pairs need an even number
    broken(lambda raw: raw["layers"][0]["mixer"]["rot"].update(dims=18))        # more than the part that turns
    broken(lambda raw: raw["layers"][3]["mixer"].update(decay=[0.5]))           # a decay per head
    broken(lambda raw: raw["layers"][3]["mlp"]["router"].update(top=7))         # more than the kept groups hold
    broken(lambda raw: raw["layers"][0]["mlp"]["expert"].update(limit=0))
    broken(lambda raw: raw["layers"][1].update(type="mamba"))
    broken(lambda raw: raw.update(streams=0))
