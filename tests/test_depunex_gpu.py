"""The Depunex decoder on the GPU against the plain implementation (tests/plain_depunex.py), for three small
configurations that differ in every size and option: whole prompts, token-by-token decoding from the first token,
portions of several sizes, unequal batches through reused slots, long decoding across chunk and block borders, greedy
generation through the library's loop and programs; and every new mechanism alone against plain arithmetic, with inputs
made so that a chunk's edge, a far state or a closed group of experts shows."""
import math

import pytest
import torch

from helpers import errors, run_batched, run_whole, token_ids
from depunex_models import CONFIGS, make_depunex_folder
import plain_depunex as P

pytestmark = pytest.mark.gpu
DTYPES = ["float32", "bfloat16"]
NAMES = sorted(CONFIGS)
LENGTH = {"mixed": 150, "wide": 160, "edges": 140}
F = torch.float64

# Largest difference from the plain implementation (float64), relative to the largest logit. Both recurrences multiply
# what they read by exponentials of sums of rounded step sizes, and the experts' weights divide by a sum of a few scores,
# so float32 sums in another order show up a little above their own rounding; in bfloat16 the projections' outputs that
# feed a state (x, B, C) are rounded to 8 bits and stay in the state for good.
# In bfloat16 the router reads the rounded rows, and with random weights a token now and then has two experts (or two groups)
# whose scores lie closer than that rounding: the engine then takes the other expert than the float64 model, and that one row
# is off by what the two experts differ in (seen: up to 0.4 of the largest logit, and gone when the experts are replaced by a
# dense feed-forward). So in bfloat16 up to OUTLIER_ROWS of a request's rows (two of a short request's, one of a few rows) may exceed the limit on single logits, while the
# root mean square over all rows must hold; 32-bit has no such allowance, and it runs the same kernels.
LIMITS = {"float32": dict(max=1e-4, rms=2e-5), "bfloat16": dict(max=1e-1, rms=2.5e-2)}
OUTLIER_ROWS = 0.03
WORST = {}


def assert_logits(got, want, dtype, what):
    assert torch.isfinite(got).all(), f"{what}: logits are not finite"
    worst, rms = errors(got, want)
    if dtype == "bfloat16" and worst > LIMITS[dtype]["max"]:
        per_row = (got.double().cpu() - want.double()).abs().max(dim=1).values / float(want.abs().max())
        over = int((per_row > LIMITS[dtype]["max"]).sum())
        assert over <= (1 if want.shape[0] < 20 else max(2, int(OUTLIER_ROWS * want.shape[0]))), f"{what} [{dtype}]: {over} of {want.shape[0]} rows exceed {LIMITS[dtype]['max']:.1e}"
        worst = float(per_row[per_row <= LIMITS[dtype]["max"]].max()) if over < want.shape[0] else worst
    seen = WORST.setdefault(dtype, [0.0, 0.0])
    seen[0], seen[1] = max(seen[0], worst), max(seen[1], rms)
    assert worst <= LIMITS[dtype]["max"] and rms <= LIMITS[dtype]["rms"], \
        f"{what} [{dtype}]: max error {worst:.3e} (limit {LIMITS[dtype]['max']:.1e}), rms {rms:.3e} (limit {LIMITS[dtype]['rms']:.1e})"


def first_bad_position(got, want, dtype):
    scale = float(want.abs().max())
    for t in range(want.shape[0]):
        if float((got[t].double().cpu() - want[t].double()).abs().max()) / scale > LIMITS[dtype]["max"]:
            return t
    return None


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    """name -> (folder, plain model, ids, plain logits)"""
    out = {}
    for index, name in enumerate(NAMES):
        folder = make_depunex_folder(CONFIGS[name], tmp_path_factory.mktemp(name), seed=15 + index)
        plain = P.PlainModel(folder)
        ids = token_ids(CONFIGS[name]["vocab"], LENGTH[name], seed=400 + index)
        out[name] = (folder, plain, ids, plain.logits(ids))
    return out


@pytest.fixture(scope="module")
def engines(models):
    from xeno_rt_amd.engine import Engine
    cache = {}

    def get(name, dtype):
        if (name, dtype) not in cache:
            cache[(name, dtype)] = Engine.load(models[name][0], dtype=dtype, max_tokens=64 * 9, max_slots=3)
        return cache[(name, dtype)]
    return get


def same_but_for_rounding(got, want):
    return float((got - want).abs().max()) <= 3e-5 * float(want.abs().max())


def in_portions(engine, ids, sizes):
    """The request alone, cut into steps of the given sizes (the last size repeats); logits of every token."""
    slot = engine.alloc_slot()
    rows, at, index = [], 0, 0
    try:
        while at < len(ids):
            size = min(sizes[min(index, len(sizes) - 1)], len(ids) - at)
            rows.append(engine.step([(slot, ids[at:at + size], list(range(size)))]))
            at, index = at + size, index + 1
        return torch.cat(rows)
    finally:
        engine.free_slot(slot)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_whole_prompts(name, dtype, models, engines):
    engine = engines(name, dtype)
    _, plain, ids, want = models[name]
    got = run_whole(engine, ids)
    assert_logits(got, want, dtype, f"depunex {name} whole, first bad row {first_bad_position(got, want, dtype)}")
    for length in (1, 2, 3, 66):                                    # the first tokens of a sequence, and just past a block
        got = run_whole(engine, ids[:length])
        assert_logits(got, want[:length], dtype, f"depunex {name} whole, {length} tokens")
    engine.cache.check()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_token_by_token_from_the_first(name, dtype, models, engines):
    """Every token in a step of its own: long decoding through recorded steps, across chunks and cache blocks."""
    engine = engines(name, dtype)
    _, plain, ids, want = models[name]
    got = in_portions(engine, ids, [1])
    assert_logits(got, want, dtype, f"depunex {name} token by token, first bad row {first_bad_position(got, want, dtype)}")
    if dtype == "float32":
        assert same_but_for_rounding(got, run_whole(engine, ids)), "a decoded token differs from the same token in a prompt"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("sizes", [[2], [3, 7], [64, 1], [65, 2, 2, 1, 30], [33], [1, 1, 2, 61, 5]])
@pytest.mark.parametrize("name", NAMES)
def test_portions(name, sizes, dtype, models, engines):
    engine = engines(name, dtype)
    _, plain, ids, want = models[name]
    got = in_portions(engine, ids, sizes)
    assert_logits(got, want, dtype, f"depunex {name} portions {sizes}, first bad row {first_bad_position(got, want, dtype)}")
    if dtype == "float32":
        assert same_but_for_rounding(got, run_whole(engine, ids)), f"portions {sizes} change more than the rounding"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_unequal_batches_through_reused_slots(name, dtype, models, engines):
    """Three requests of different lengths start together and end one after the other, twice over, so that the second
    round runs in slots, blocks and states (the token before included) that the first has used."""
    engine = engines(name, dtype)
    _, plain, ids, want = models[name]
    vocab = CONFIGS[name]["vocab"]
    requests = [ids, token_ids(vocab, 37, seed=900), token_ids(vocab, 71, seed=901)]
    wants = [want, plain.logits(requests[1]), plain.logits(requests[2])]
    for prompts in ([len(ids) - 40, 5, 66], [3, 36, 1]):
        got = run_batched(engine, requests, prompts)
        for index, (g, w) in enumerate(zip(got, wants)):
            assert_logits(g, w, dtype, f"depunex {name} batch {prompts} request {index}, first bad row {first_bad_position(g, w, dtype)}")
            if dtype == "float32":
                assert same_but_for_rounding(g, run_whole(engine, requests[index])), "a request depends on its batch"
    engine.cache.check()


MANY_EXPERTS = {
    "architecture": "Depunex", "vocab": 80, "width": 64, "norm": {"eps": 1e-5}, "logit_softcap": 12.0,
    "embedding": {"scale": 2.0, "bigram": {"buckets": 31, "mul_prev": 3, "mul_cur": 5}},
    "layers": [
        {"type": "mamba2", "mixer": {"heads": 2, "vdim": 32, "state": 16, "groups": 1, "norm_groups": 2, "conv": 3},
         "mlp": {"kind": "moe", "expert": {"ff": 64}, "router": {"experts": 16, "top": 2, "groups": {"count": 4, "keep": 2}}}},
        {"type": "parallel",
         "mixer": {"left": {"heads": 2, "kv_heads": 1, "dim": 64, "vdim": 64, "scale": 0.125, "mask": {"size": 128},
                            "rot": {"dims": 32, "base": 1000.0}},
                   "right": {"inner": 32, "state": 4, "dt_rank": 2, "conv": 2}, "left_scale": 1.0, "right_scale": 1.0},
         "mlp": {"kind": "moe", "expert": {"ff": 128}, "router": {"experts": 12, "top": 2}}},
    ],
}


def test_prompts_long_enough_for_sorted_experts_and_chunks_on_the_matrix_cores(tmp_path):
    """A model whose experts' widths and whose attention suit the kernels that only steps of many tokens take: prompts of some
    hundred tokens whole (picks sorted by expert, chunks on the matrix cores), in halves, two in one step and with their ends
    decoded, against the same engine with every token meeting every expert: the router reads the same rows and chooses the
    same experts either way, so what differs is rounding alone. (Against the plain model a token whose best scores lie
    closer than bfloat16 rounds the rows takes another expert, with sixteen experts every thirtieth token or so: there the
    root mean square is held, and the other tests hold single rows on models with fewer experts.)"""
    from xeno_rt_amd.engine import Engine
    folder = make_depunex_folder(MANY_EXPERTS, tmp_path, seed=77)
    plain = P.PlainModel(folder)
    requests = [token_ids(MANY_EXPERTS["vocab"], length, seed=length) for length in (300, 281)]
    engine = Engine.load(folder, dtype="bfloat16", max_tokens=64 * 12, max_slots=2)
    ops = engine.runtime.ops
    h = torch.zeros(300, 64, dtype=torch.bfloat16, device="cuda")
    for layer in engine.model.spec.layers:                       # (the test is about these paths: it says so if they are not taken)
        mlp = layer.feed_forward
        assert ops.experts_sorted_takes(h, mlp.w_gate_up, mlp.w_down, mlp.experts, mlp.intermediate, mlp.top)
    takes = ops.experts_sorted_takes
    ops.experts_sorted_takes = lambda *operands: False
    wants = [run_whole(engine, ids) for ids in requests]
    ops.experts_sorted_takes = takes
    for ids, want in zip(requests, wants):
        assert errors(want, plain.logits(ids))[1] <= 5e-2

    def close(got, want, what):
        # (the second layer's router reads what the first layer's experts made: a rare row may change its experts there too)
        per_row = (got.double() - want.double()).abs().max(dim=1).values / float(want.abs().max())
        rms = errors(got, want)[1]
        assert int((per_row > 4e-2).sum()) <= 3 and rms <= 1e-2, \
            f"{what}: sorted picks differ from every token with every expert in rows {(per_row > 4e-2).nonzero().flatten().tolist()}, rms {rms:.2e}"

    for ids, want in zip(requests, wants):
        close(run_whole(engine, ids), want, f"{len(ids)} tokens whole")
        close(in_portions(engine, ids, [len(ids) // 2 + 1]), want, f"{len(ids)} tokens in halves")
    for prompts in ([300, 281], [270, 281]):
        for index, (got, want) in enumerate(zip(run_batched(engine, requests, prompts), wants)):
            close(got, want, f"batch {prompts} request {index}")
    engine.cache.check()


@pytest.mark.parametrize("dtype", DTYPES)
def test_greedy_generation_through_the_loop(dtype, models, engines):
    from xeno_rt_amd.engine import GenerateRequest, generate
    name = "mixed"
    engine = engines(name, dtype)
    _, plain, ids, _ = models[name]
    prompts = [ids[:9], ids[20:21], ids[40:75]]
    requests = [GenerateRequest(p, max_tokens=8, temperature=0.0, repetition_penalty=1.0, stop_ids=[]) for p in prompts]
    got = [r.tokens for r in generate(engine, requests)]
    for prompt, tokens in zip(prompts, got):
        assert len(tokens) == 8
        history = list(prompt)
        for index, token in enumerate(tokens):
            row = plain.logits(history)[-1]
            if dtype == "float32":
                assert token == int(row.argmax()), f"token {index} is {token}, the plain loop chooses {int(row.argmax())}"
            else:
                assert float(row.max() - row[token]) <= 0.1 * float(row.abs().max()), f"token {index} ({token}) is not among the best"
            history.append(token)


# ---- every mechanism alone -------------------------------------------------------------------------------------

class Step:
    """A step's sequences as the kernels want them described: `counts[i]` new tokens of the sequence in `slots[i]`."""

    def __init__(self, slots, counts, starts, ids=None, device="cuda"):
        ints = lambda values: torch.tensor(values, dtype=torch.int32, device=device)
        offsets = [0]
        for count in counts:
            offsets.append(offsets[-1] + count)
        self.n_tokens, self.n_sequences, self.max_count = offsets[-1], len(slots), max(counts)
        self.sequence_offsets, self.sequence_slots, self.sequence_starts = ints(offsets), ints(slots), ints(starts)
        self.positions = ints([start + t for start, count in zip(starts, counts) for t in range(count)])
        self.slots = ints([slot for slot, count in zip(slots, counts) for _ in range(count)])
        self.max_context = max(start + count for start, count in zip(starts, counts))
        self.token_ids = None if ids is None else ints(ids)


def schedules(length):
    """Ways to cut a sequence of `length` tokens into steps."""
    return [[length], [1] * length, [2] * (length // 2) + [length % 2] * (length % 2), [length - 3, 1, 2], [70, length - 70]]


@pytest.fixture(scope="module")
def ops():
    from xeno_rt_amd.ops import load_ops
    return load_ops()


def test_the_hashed_table_reads_the_token_before_across_steps_and_slots(ops):
    """Two sequences and padding between them, cut differently; a slot that another sequence has used starts afresh at
    position 0 whatever token it kept."""
    width, buckets, mul_prev, mul_cur, scale = 24, 11, 5, 3, 2.5
    generator = torch.Generator().manual_seed(1)
    table = torch.randn(buckets + 1, width, generator=generator)
    a, b = token_ids(50, 40, seed=1), token_ids(50, 9, seed=2)
    want = {name: torch.stack([table[row] for row in P.bigram_rows(ids, buckets, mul_prev, mul_cur)]) for name, ids in (("a", a), ("b", b))}
    before = torch.full((4,), 33, dtype=torch.int32, device="cuda")          # what other sequences left in the slots
    got = {"a": [], "b": []}
    at_a = at_b = 0
    for count_a, count_b in ((5, 1), (1, 1), (30, 3), (4, 4)):
        ids = a[at_a:at_a + count_a] + [7, 7] + b[at_b:at_b + count_b]
        step = Step([2, -1, 0], [count_a, 2, count_b], [at_a, 0, at_b], ids)
        x = torch.ones(len(ids), width, device="cuda")
        ops.bigram_add(x, scale, step, table.cuda(), before, buckets, mul_prev, mul_cur)
        got["a"].append(x[:count_a]); got["b"].append(x[count_a + 2:])
        at_a, at_b = at_a + count_a, at_b + count_b
    for name in "ab":
        assert torch.allclose(torch.cat(got[name]).cpu(), want[name] + scale, atol=1e-6), name
    assert before.tolist() == [b[-1], 33, a[-1], 33]
    x = torch.zeros(3, width, device="cuda")
    ops.bigram_add(x, 4.0, Step([1], [3], [0], [1, 2, 3]))                   # no table: the scale alone
    assert float(x.abs().max()) == 0.0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("taps", [1, 2, 4, 5])
def test_short_convolution_with_bias_and_silu_of_float32_inputs(taps, dtype, ops):
    length, channels = 150, 72
    generator = torch.Generator().manual_seed(taps)
    u = torch.randn(length, channels + 8, generator=generator)                # (the inputs are columns of a wider float32 matrix)
    w, b = torch.randn(channels, taps, generator=generator).to(dtype), torch.randn(channels, generator=generator).to(dtype)
    want = P.causal_conv_silu(u[:, 3:3 + channels].double(), w.double(), b.double())
    for cuts in schedules(length):
        state = torch.full((3, taps - 1, channels), 7.0, device="cuda")
        state[1].zero_()
        rows, at = [], 0
        for count in cuts:
            out = torch.empty(2 + count, channels, dtype=dtype, device="cuda")
            step = Step([-1, 1], [2, count], [0, at])
            x = torch.cat([torch.ones(2, channels + 8), u[at:at + count]]).cuda()
            ops.short_conv(x[:, 3:3 + channels], w.cuda(), state, step, out, bias=b.cuda(), activation="silu")
            rows.append(out[2:])
            at += count
        got = torch.cat(rows).double().cpu()
        limit = 1e-5 if dtype == torch.float32 else 1e-2
        assert float((got - want).abs().max()) <= limit * float(want.abs().max()), f"taps {taps}, cuts {cuts[:4]}"
        if taps > 1:
            assert float(state[0].min()) == 7.0 and float(state[2].max()) == 7.0, "another sequence's state was touched"
            assert torch.equal(state[1].cpu(), u[length - taps + 1:, 3:3 + channels]), "the state keeps the inputs unrounded"


def plain_stepped_recurrence(x, b, c, z, dt, heads, vdim, n, groups, rate, skip):
    """Mamba-2's recurrence with its gate, before the norm: [tokens, heads * vdim]."""
    tokens = x.shape[0]
    x, b, c = x.reshape(tokens, heads, vdim), b.reshape(tokens, groups, n), c.reshape(tokens, groups, n)
    y = torch.zeros(tokens, heads, vdim, dtype=F)
    for head in range(heads):
        group = head // (heads // groups)
        state = torch.zeros(n, vdim, dtype=F)
        for t in range(tokens):
            state = torch.exp(-rate[head] * dt[t, head]) * state + dt[t, head] * torch.outer(b[t, group], x[t, head])
            y[t, head] = state.T @ c[t, group] + skip[head] * x[t, head]
    return y.reshape(tokens, heads * vdim) * P.silu(z)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,vdim,n,groups,norm_groups", [(4, 12, 20, 2, 3), (1, 136, 16, 1, 2), (2, 40, 72, 1, 1), (3, 16, 8, 3, 6),
                                                            (6, 64, 128, 2, 1), (2, 24, 200, 2, 4)])
def test_the_recurrence_with_step_sizes_shared_keys_a_skip_and_a_norm_in_parts(heads, vdim, n, groups, norm_groups, dtype, ops):
    length, inner = 100, heads * vdim
    generator = torch.Generator().manual_seed(n)
    rand = lambda *shape: torch.randn(*shape, generator=generator)
    x, b, c = rand(length, inner).to(dtype), (0.3 * rand(length, groups * n)).to(dtype), rand(length, groups * n).to(dtype)
    wide = rand(length, inner + heads + 5)                                     # gate and raw step sizes: float32 columns of one matrix
    z, raw = wide[:, :inner], wide[:, inner + 5:]
    bias, a_log, skip, weight = rand(heads) - 1.0, rand(heads) - 1.0, rand(heads), 1 + 0.3 * rand(inner)
    eps = 1e-4
    dt = P.softplus((raw + bias).double())
    y = plain_stepped_recurrence(x.double(), b.double(), c.double(), z.double(), dt, heads, vdim, n, groups, torch.exp(a_log.double()), skip.double())
    want = P.rms_divided(y.reshape(length, norm_groups, inner // norm_groups), eps).reshape(length, inner) * weight.double()
    for cuts in schedules(length):
        state = torch.zeros(2, heads, n, vdim, device="cuda")
        rows, at = [], 0
        for count in cuts:
            cut = lambda t: t[at:at + count].cuda()
            both = cut(wide)
            out = torch.empty(count, inner, dtype=dtype, device="cuda")
            ops.linear_recurrence(cut(c), cut(b), cut(x), state, Step([1], [count], [at]), out, heads, n, vdim, both[:, inner + 5:], "step",
                                  decay_bias=bias.cuda(), decay_rate=a_log.cuda(), qk_heads=groups, skip=skip.cuda(), norm_eps=eps,
                                  norm_weight=weight.cuda(), norm_groups=norm_groups, gate=both[:, :inner], gate_activation="silu")
            rows.append(out)
            at += count
        got = torch.cat(rows).double().cpu()
        limit = 3e-5 if dtype == torch.float32 else 2e-2
        assert float((got - want).abs().max()) <= limit * float(want.abs().max()), f"cuts {cuts[:4]}"
        assert float(state[0].abs().max()) == 0.0, "another sequence's state was touched"


def plain_scan(x, step, b, c, a_log, skip, gate):
    tokens, channels = x.shape
    a = -torch.exp(a_log)
    state, y = torch.zeros(channels, a.shape[1], dtype=F), torch.zeros(tokens, channels, dtype=F)
    for t in range(tokens):
        state = torch.exp(step[t][:, None] * a) * state + (step[t] * x[t])[:, None] * b[t][None, :]
        y[t] = state @ c[t] + skip * x[t]
    return y * P.silu(gate)


def run_scan(ops, x, raw, bc, gate, cuts, dtype, a_log, bias, skip, n, slots=2, slot=1, state=None):
    channels = x.shape[1]
    state = torch.zeros(slots, channels, n, device="cuda") if state is None else state
    rows, at = [], 0
    for count in cuts:
        cut = lambda t: t[at:at + count].cuda()
        both = cut(bc)
        out = torch.empty(count, channels, dtype=dtype, device="cuda")
        ops.selective_scan(cut(x), cut(raw), both[:, :n], both[:, n:], state, Step([slot], [count], [at]), out, a_log.cuda(),
                           step_bias=bias.cuda(), skip=skip.cuda(), gate=cut(gate))
        rows.append(out)
        at += count
    return torch.cat(rows).double().cpu(), state


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("channels,n", [(40, 10), (100, 16), (64, 33), (16, 1), (72, 24), (8, 5), (320, 64)])
def test_the_selective_scan(channels, n, dtype, ops):
    length = 150
    generator = torch.Generator().manual_seed(channels + n)
    rand = lambda *shape: torch.randn(*shape, generator=generator)
    x, raw, bc, gate = rand(length, channels).to(dtype), rand(length, channels), rand(length, 2 * n), rand(length, channels)
    a_log, bias, skip = rand(channels, n) - 1.0, rand(channels) - 1.0, rand(channels)
    want = plain_scan(x.double(), P.softplus((raw + bias).double()), bc[:, :n].double(), bc[:, n:].double(), a_log.double(), skip.double(), gate.double())
    for cuts in schedules(length):
        got, state = run_scan(ops, x, raw, bc, gate, cuts, dtype, a_log, bias, skip, n)
        limit = 2e-5 if dtype == torch.float32 else 1e-2
        assert float((got - want).abs().max()) <= limit * float(want.abs().max()), f"cuts {cuts[:4]}"
        assert float(state[0].abs().max()) == 0.0, "another sequence's state was touched"


def test_scans_of_unequal_sequences_in_one_step_and_a_long_prompt_in_segments(ops):
    """Sequences of 700, 65 and 3 tokens and one that is padding in one step (the long one in segments side by side), then one
    more token each: every sequence as it is alone, and the padding's rows zeros."""
    channels, n, lengths = 48, 12, [700, 65, 3]
    generator = torch.Generator().manual_seed(5)
    rand = lambda *shape: torch.randn(*shape, generator=generator)
    a_log, bias, skip = rand(channels, n) - 2.0, rand(channels) - 2.0, rand(channels)
    data = [(rand(length + 1, channels), rand(length + 1, channels), rand(length + 1, 2 * n), rand(length + 1, channels)) for length in lengths]
    wants = [plain_scan(x.double(), P.softplus((raw + bias).double()), bc[:, :n].double(), bc[:, n:].double(), a_log.double(), skip.double(), gate.double())
             for x, raw, bc, gate in data]
    pad = [torch.ones(2, width) for width in (channels, channels, 2 * n, channels)]
    packed = [torch.cat([data[0][i][:-1], pad[i], data[1][i][:-1], data[2][i][:-1]]).cuda() for i in range(4)]
    state = torch.zeros(5, channels, n, device="cuda")
    out = torch.empty(sum(lengths) + 2, channels, device="cuda")
    step = Step([3, -1, 1, 4], [lengths[0], 2, lengths[1], lengths[2]], [0, 0, 0, 0])
    ops.selective_scan(packed[0], packed[1], packed[2][:, :n], packed[2][:, n:], state, step, out, a_log.cuda(), step_bias=bias.cuda(),
                       skip=skip.cuda(), gate=packed[3])
    more = torch.empty(3, channels, device="cuda")
    last = [torch.stack([d[i][-1] for d in data]).cuda() for i in range(4)]
    ops.selective_scan(last[0], last[1], last[2][:, :n], last[2][:, n:], state, Step([3, 1, 4], [1, 1, 1], lengths), more, a_log.cuda(),
                       step_bias=bias.cuda(), skip=skip.cuda(), gate=last[3])
    at = 0
    for index, length in enumerate(lengths):
        if index == 1:
            assert float(out[at:at + 2].abs().max()) == 0.0
            at += 2
        got = torch.cat([out[at:at + length], more[index:index + 1]]).double().cpu()
        assert float((got - wants[index]).abs().max()) <= 3e-5 * float(wants[index].abs().max()), f"sequence {index}"
        at += length
    assert float(state[0].abs().max()) == 0.0 and float(state[2].abs().max()) == 0.0


def test_a_state_keeps_a_token_from_far_back(ops):
    """With steps that hardly decay, what the first token fed is read a thousand tokens on, in a prompt and decoded; with steps
    that decay at once it is gone."""
    length, channels, n = 1000, 8, 4
    x, bc, gate = torch.zeros(length, channels), torch.zeros(length, 2 * n), torch.full((length, channels), 1.0)
    x[0], x[-1] = 1.0, 0.0
    bc[0, 2], bc[-1, n + 2] = 1.0, 1.0                                         # fed at the first token, read at the last
    skip, bias = torch.zeros(channels), torch.zeros(channels)
    for a_value, raw_value, kept in ((-30.0, 1.0, True), (3.0, 1.0, False)):
        a_log, raw = torch.full((channels, n), a_value), torch.full((length, channels), raw_value)
        step = math.log1p(math.exp(raw_value))
        want = step * math.exp(-math.exp(a_value) * step * (length - 1)) / (1 + math.exp(-1.0)) if kept else 0.0
        for cuts in ([length], [length - 40] + [1] * 40):
            got, _ = run_scan(ops, x, raw, bc, gate, cuts, torch.float32, a_log, bias, skip, n)
            assert abs(float(got[-1, 0]) - want) <= 1e-5 and (kept is False or want > 0.9), (a_value, cuts[:2])


def attend(ops, q, k, v, cuts, dtype, n_heads, n_kv_heads, dim, vdim, **options):
    """Keys and values through `kv_store` into a paged cache whose blocks lie in another order than the sequence's, then
    the general attention kernel on the queries alone, step by step."""
    from xeno_rt_amd.cache import BLOCK_TOKENS
    from xeno_rt_amd.cache.sequence_cache import KVView
    from xeno_rt_amd.parts.base import KVSpec
    length = q.shape[0]
    blocks = (length + BLOCK_TOKENS - 1) // BLOCK_TOKENS
    table = torch.full((2, blocks), -1, dtype=torch.int32)
    table[1] = torch.arange(blocks - 1, -1, -1, dtype=torch.int32) + 1
    kv = KVView(KVSpec(n_kv_heads, dim, None, vdim),
                torch.zeros(blocks + 1, n_kv_heads, BLOCK_TOKENS, dim, dtype=dtype, device="cuda"),
                torch.zeros(blocks + 1, n_kv_heads, vdim, BLOCK_TOKENS, dtype=dtype, device="cuda"), table.cuda())
    rows, at = [], 0
    for count in cuts:
        if count == 0:
            continue
        step = Step([1], [count], [at])
        cut = lambda t: t[at:at + count].to(dtype).cuda().contiguous()
        ops.kv_store(cut(k), cut(v), n_kv_heads, dim, vdim, kv, step)
        out = torch.empty(count, n_heads * vdim, dtype=dtype, device="cuda")
        ops.attention(cut(q), n_heads, n_kv_heads, dim, kv, step, out, value_dim=vdim, queries_alone=True, **options)
        rows.append(out)
        at += count
    return torch.cat(rows).double().cpu()


def plain_chunked(q, k, v, n_heads, n_kv_heads, dim, vdim, scale, chunk):
    length = q.shape[0]
    q, k, v = q.double().reshape(length, n_heads, dim), k.double().reshape(length, n_kv_heads, dim), v.double().reshape(length, n_kv_heads, vdim)
    out = torch.zeros(length, n_heads, vdim, dtype=F)
    for head in range(n_heads):
        group = head // (n_heads // n_kv_heads)
        for i in range(length):
            lo = i - i % chunk if chunk else 0
            out[i, head] = torch.softmax((k[lo:i + 1, group] @ q[i, head]) * scale, dim=0) @ v[lo:i + 1, group]
    return out.reshape(length, n_heads * vdim)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n_heads,n_kv_heads,dim,vdim,chunk", [(4, 2, 24, 16, 20), (2, 2, 32, 48, 70), (3, 1, 16, 8, None), (1, 1, 64, 64, 64),
                                                              (4, 4, 8, 4, 1), (2, 1, 16, 24, 128), (8, 2, 96, 96, 100)])
def test_attention_inside_chunks_of_positions(n_heads, n_kv_heads, dim, vdim, chunk, dtype, ops):
    length = 150
    generator = torch.Generator().manual_seed(dim + vdim)
    q, k = torch.randn(length, n_heads * dim, generator=generator), torch.randn(length, n_kv_heads * dim, generator=generator)
    v = torch.randn(length, n_kv_heads * vdim, generator=generator)
    q, k, v = (t.to(dtype).float() for t in (q, k, v))
    scale = 0.4 / math.sqrt(dim)
    want = plain_chunked(q, k, v, n_heads, n_kv_heads, dim, vdim, scale, chunk)
    first = None
    for cuts in schedules(length):
        got = attend(ops, q, k, v, cuts, dtype, n_heads, n_kv_heads, dim, vdim, scale=scale, chunk=chunk)
        limit = 1e-5 if dtype == torch.float32 else 2e-2
        assert float((got - want).abs().max()) <= limit * float(want.abs().max()), f"chunk {chunk}, cuts {cuts[:4]}"
        # (bfloat16 heads of 64 or 128 dims in chunks of whole cache blocks: steps of several tokens go to the matrix cores,
        # steps of one token do not, and the two agree but for rounding)
        if first is None:
            first = got
        elif not (dtype == torch.bfloat16 and dim == vdim and dim in (64, 128) and (chunk or 0) % 64 == 0):
            assert torch.equal(got, first), f"cuts {cuts[:4]} change the bits"


@pytest.mark.parametrize("n_heads,n_kv_heads,dim,chunk", [(4, 2, 64, 64), (2, 1, 128, 128), (4, 4, 128, 192), (6, 2, 64, 320), (2, 2, 128, None),
                                                          (8, 2, 128, 512)])
def test_attention_inside_chunks_on_the_matrix_cores(n_heads, n_kv_heads, dim, chunk, ops):
    """Prompts long enough for several tiles of queries in one chunk, whole and in portions that begin and end inside chunks,
    on chunk borders and on cache block borders, against the plain sum; the probabilities keep sixteen bits, so the error
    is that of the rounded operands and result."""
    length = 700
    generator = torch.Generator().manual_seed(dim + n_heads)
    q, k = torch.randn(length, n_heads * dim, generator=generator), torch.randn(length, n_kv_heads * dim, generator=generator)
    v = torch.randn(length, n_kv_heads * dim, generator=generator)
    q, k, v = (t.to(torch.bfloat16).float() for t in (q, k, v))
    scale = 1.5 / math.sqrt(dim)
    want = plain_chunked(q, k, v, n_heads, n_kv_heads, dim, dim, scale, chunk)
    for cuts in ([length], [length - 3, 1, 2], [70, length - 70], [64, 64, 300, 272], [129, 257, 2, 312], [5] * 140, [191, 193, 316]):
        got = attend(ops, q, k, v, cuts, torch.bfloat16, n_heads, n_kv_heads, dim, dim, scale=scale, chunk=chunk)
        error = (got - want).abs()
        assert float(error.max()) <= 6e-3 * float(want.abs().max()), f"chunk {chunk}, cuts {cuts[:4]}: row {int(error.max(dim=1).values.argmax())}"


@pytest.mark.parametrize("chunk", [64, 128, 192])
def test_the_matrix_cores_see_a_chunks_first_key_and_not_the_one_before(chunk, ops):
    n_heads, dim, length = 2, 64, 450
    for query in sorted({chunk, 2 * chunk - 1, chunk + chunk // 2, (449 // chunk) * chunk, 449}):
        first = query - query % chunk
        for key, seen in ((first, True), (first - 1, False)):
            q, k, v = (torch.zeros(length, n_heads * dim) for _ in range(3))
            q[query], k[key], v[key] = 3.0, 3.0, 1.0
            for cuts in ([length], [query - 1, 2, length - query - 1], [first, length - first], [first + 1, length - first - 1]):
                got = attend(ops, q, k, v, cuts, torch.bfloat16, n_heads, n_heads, dim, dim, scale=0.05, chunk=chunk)
                assert abs(float(got[query, 0]) - (1.0 if seen else 0.0)) < 1e-2, f"chunk {chunk}, query {query}, key {key}, cuts {cuts}"


@pytest.mark.parametrize("chunk", [1, 3, 20, 64, 70, 128])
def test_a_key_at_the_chunks_first_place_is_seen_and_the_one_before_it_is_not(chunk, ops):
    """One key whose score towers over the rest, at the first place of the query's chunk and at the last of the chunk before,
    for queries at a chunk's first and last place and in its middle, in a prompt and decoded, on either side of a cache
    block's border."""
    n_heads, dim, vdim, length = 2, 16, 8, 270
    for query in sorted({chunk, 2 * chunk - 1, 128 + chunk // 2, (269 // chunk) * chunk, 269} & set(range(1, length))):
        first = query - query % chunk
        for key, seen in ((first, True), (first - 1, False)):
            if key < 0:
                continue
            q, k = torch.zeros(length, n_heads * dim), torch.zeros(length, n_heads * dim)
            v = torch.zeros(length, n_heads * vdim)
            q[query], k[key], v[key] = 6.0, 6.0, 1.0
            visible = query - first + 1
            # (a key that is the query's own place is always seen; the others share what the towering key leaves)
            want_value = 1.0 if seen else 0.0
            for cuts in ([length], [query, 1, length - query - 1], [query - 1, 2, length - query - 1]):
                got = attend(ops, q, k, v, cuts, torch.float32, n_heads, n_heads, dim, vdim, scale=0.05, chunk=chunk)
                assert abs(float(got[query, 0]) - want_value) < 1e-3, f"chunk {chunk}, query {query}, key {key}, {visible} visible, cuts {cuts}"


def test_a_far_key_is_found_among_hundreds(ops):
    n_heads, dim, vdim, length, chunk = 1, 32, 16, 900, 1024
    generator = torch.Generator().manual_seed(2)
    q, k, v = (0.1 * torch.randn(length, width, generator=generator) for width in (dim, dim, vdim))
    q[-1], k[5] = 3.0, 3.0
    v[5] = 7.0
    for cuts in ([length], [length - 33] + [1] * 33):
        got = attend(ops, q, k, v, cuts, torch.float32, n_heads, n_heads, dim, vdim, scale=0.1, chunk=chunk)
        assert abs(float(got[-1, 0]) - 7.0) < 1e-2


def test_rotation_of_halves_over_a_part_of_the_head_with_stretched_frequencies(ops):
    """What completes q, k and v after their projection, against the plain rotation: the first dims of every head in pairs of
    halves, the rest untouched, values untouched, at positions of a prompt and of decoded tokens."""
    from xeno_rt_amd.parts import PairRotation
    from xeno_rt_amd.parts.base import Runtime
    n_heads, n_kv_heads, dim, vdim, dims = 3, 1, 20, 12, 12
    scaling = {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 64}
    rotation = PairRotation(dims, 1000.0, neighbours=False, scaling=scaling)
    rotation.bind({}, Runtime(ops, torch.float32, "cuda"))
    frequencies = P.rotary_frequencies(dims, 1000.0, scaling)
    assert rotation.frequencies.cpu().tolist() == pytest.approx(frequencies, rel=1e-6)
    length = 90
    proj = torch.randn(length, (n_heads + n_kv_heads) * dim + n_kv_heads * vdim, generator=torch.Generator().manual_seed(3))
    want_q = P.rotate(proj[:, :n_heads * dim].double().reshape(length, n_heads, dim), dims, frequencies).reshape(length, -1)
    for cuts in ([length], [50] + [1] * 40):
        rows, at = [], 0
        for count in cuts:
            q = torch.empty(count, n_heads * dim, device="cuda")
            f, d, neighbours, magnitude = rotation.pair_rotation()
            ops.qkv_complete(proj[at:at + count].cuda(), n_heads, n_kv_heads, dim, vdim, Step([0], [count], [at]), q, frequencies=f, rot_dims=d,
                             neighbours=neighbours, magnitude=magnitude)
            rows.append(q)
            at += count
        assert torch.allclose(torch.cat(rows).double().cpu(), want_q, atol=2e-5)


@pytest.mark.parametrize("experts,top,groups,keep", [(8, 2, 4, 2), (6, 3, 1, 1), (12, 1, 3, 1), (4, 4, 2, 2), (9, 2, 3, 2), (256, 8, 1, 1),
                                                     (64, 6, 8, 3), (16, 5, 16, 5)])
def test_experts_are_chosen_inside_the_best_groups(experts, top, groups, keep, ops):
    tokens = 300
    logits = 2.0 * torch.randn(tokens, experts, generator=torch.Generator().manual_seed(experts))
    chosen, weights = P.route(logits.double(), torch.eye(experts, dtype=F), experts, top, groups, keep)     # (a router that passes its input on)
    want = torch.zeros(tokens, experts, dtype=F)
    want.scatter_(1, chosen, weights)
    got, picked = torch.empty(tokens, experts, device="cuda"), torch.empty(tokens, top, dtype=torch.int32, device="cuda")
    ops.route_experts(logits.cuda(), got, top, groups, keep, chosen=picked)
    assert torch.equal(picked.cpu().long().sort(dim=1).values, chosen.sort(dim=1).values)
    assert torch.allclose(got.double().cpu(), want, atol=1e-6) and torch.allclose(got.sum(dim=1).cpu(), torch.ones(tokens), atol=1e-5)


def test_an_expert_outside_the_kept_groups_is_never_chosen_however_large_its_score(ops):
    # groups {0,1} {2,3} {4,5}: expert 4 has the largest score of all, but its group's two best sum to less than the others'
    scores = torch.tensor([[0.7, 0.6, 0.65, 0.6, 0.9, 0.01]])
    logits = torch.log(scores / (1 - scores)).cuda()
    weights = torch.empty(1, 6, device="cuda")
    ops.route_experts(logits, weights, 2, 3, 2)
    assert weights[0, 4].item() == 0.0 and weights[0].nonzero().flatten().tolist() == [0, 2]
    assert weights[0, 0].item() == pytest.approx(0.7 / 1.35, rel=1e-5)


def expert_operands(ops, tokens, hidden, width, experts, seed, packed_down):
    generator = torch.Generator().manual_seed(seed)
    h = torch.randn(tokens, hidden, generator=generator).bfloat16()
    gates, ups = (0.3 * torch.randn(experts, width, hidden, generator=generator).bfloat16() for _ in range(2))
    downs = 0.3 * torch.randn(experts, hidden, width, generator=generator).bfloat16()
    logits = torch.randn(tokens, experts, generator=generator)
    w_gate_up = ops.pack(torch.cat([gates.reshape(-1, hidden), ups.reshape(-1, hidden)]).cuda(), "gated", gated_n=experts * width)
    w_down = torch.cat(list(downs), dim=1).contiguous().cuda()
    return h, gates, ups, downs, logits, w_gate_up, ops.pack(w_down, "tiles") if packed_down else w_down


@pytest.mark.parametrize("tokens,hidden,width,experts,top,groups,keep,packed_down", [
    (300, 64, 64, 8, 2, 4, 2, False), (1000, 128, 192, 16, 4, 1, 1, True), (257, 192, 64, 3, 1, 1, 1, False), (640, 64, 128, 32, 2, 8, 3, True),
    (129, 320, 64, 5, 5, 1, 1, True), (1700, 64, 128, 4, 2, 2, 1, True)])           # (the last: experts with picks enough for the larger tile)
def test_experts_multiply_only_the_tokens_that_chose_them(tokens, hidden, width, experts, top, groups, keep, packed_down, ops):
    """The picks sorted by expert against the plain sum over every token's experts, against the way in which every token
    meets every expert, and a token's bits with other tokens around it. (One expert may be chosen by no one, another by all.)"""
    h, gates, ups, downs, logits, w_gate_up, w_down = expert_operands(ops, tokens, hidden, width, experts, tokens + experts, packed_down)
    logits[:, 1] -= 30.0                                       # nobody's choice, unless all are chosen
    weights = torch.empty(tokens, experts, device="cuda")
    chosen = torch.empty(tokens, top, dtype=torch.int32, device="cuda")
    ops.route_experts(logits.cuda(), weights, top, groups, keep, chosen=chosen)
    out = torch.full((tokens, hidden), float("nan"), device="cuda")
    ops.experts_sorted(h.cuda(), w_gate_up, w_down, weights, chosen, width, out)
    want = torch.zeros(tokens, hidden, dtype=F)
    for e in range(experts):
        takers = (chosen.cpu() == e).any(dim=1)
        x = h[takers].double()
        gate, up = x @ gates[e].double().T, x @ ups[e].double().T
        want[takers] += weights.cpu()[takers, e].double()[:, None] * ((gate * torch.sigmoid(gate) * up) @ downs[e].double().T)
    assert float((out.double().cpu() - want).abs().max()) <= 1e-2 * float(want.abs().max())
    # every token with every expert: the same but for the rounding of the weighted activations
    act = torch.empty(tokens, experts * width, dtype=torch.bfloat16, device="cuda")
    ops.linear_glu(h.cuda(), w_gate_up, act)
    ops.scale_blocks(act, weights, width)
    dense = torch.empty(tokens, hidden, device="cuda")
    ops.linear(act, w_down, dense)
    assert float((out - dense).abs().max()) <= 1e-2 * float(want.abs().max())
    # other company, other rows in the sort: the same bits
    some = torch.arange(tokens - 1, -1, -3)
    fewer = torch.empty(len(some), hidden, device="cuda")
    ops.experts_sorted(h[some].cuda(), w_gate_up, w_down, weights[some.cuda()].contiguous(), chosen[some.cuda()].contiguous(), width, fewer)
    assert torch.equal(fewer, out[some.cuda()])


def test_sorted_experts_are_taken_for_steps_of_many_tokens_only(ops):
    h, _, _, _, _, w_gate_up, w_down = expert_operands(ops, 512, 64, 64, 8, 1, True)
    assert ops.experts_sorted_takes(h.cuda(), w_gate_up, w_down, 8, 64, 2)
    assert not ops.experts_sorted_takes(h[:8].cuda(), w_gate_up, w_down, 8, 64, 2)          # a decode step reads every expert once either way
    assert not ops.experts_sorted_takes(h.cuda(), w_gate_up, w_down, 8, 64, 8)              # every token uses every expert: nothing to save
    assert not ops.experts_sorted_takes(h.float().cuda(), w_gate_up, w_down, 8, 64, 2)


def test_small_operations(ops):
    generator = torch.Generator().manual_seed(9)
    rows, width = 7, 40
    residual, a, b, c = (torch.randn(rows, width, generator=generator) for _ in range(4))
    ga, gc = torch.randn(width, generator=generator), torch.randn(width, generator=generator)
    got = residual.clone().cuda()
    ops.add_weighted(got, [(a.cuda(), ga.cuda(), 0.7), (b.cuda(), None, 1.3), (c.cuda(), gc.cuda(), 1.0)])
    assert torch.allclose(got.cpu(), residual + 0.7 * a * ga + 1.3 * b + c * gc, atol=1e-5)
    sums, limit = 3.0 * torch.randn(rows, 2 * width, generator=generator), 1.25
    g, u = sums[:, :width].clamp(max=limit), sums[:, width:].clamp(-limit, limit)
    out = torch.empty(rows, width, device="cuda")
    ops.glu_clamped(sums.cuda(), out, limit, 1.702)
    assert torch.allclose(out.cpu(), g * torch.sigmoid(1.702 * g) * (u + 1), atol=1e-5)
    x = 20.0 * torch.randn(rows, width, generator=generator)
    capped = x.clone().cuda()
    ops.softcap(capped, 15.0)
    assert torch.allclose(capped.cpu(), 15.0 * torch.tanh(x / 15.0), atol=1e-5)
    table, s = torch.randn(11, 3 * width, generator=generator), torch.randn(rows, width + 4, generator=generator)
    ids = torch.tensor([3, 0, 10, 3, 1, 1, 9], dtype=torch.int32)
    out = torch.empty(rows, width, device="cuda")
    ops.gated_rows(s.cuda()[:, :width], table.cuda(), ids.cuda(), width, out)
    assert torch.allclose(out.cpu().double(), P.gelu_tanh(s[:, :width].double()) * table[ids.long(), width:2 * width].double(), atol=1e-5)
    act, weights = torch.randn(rows, 5 * 8, generator=generator), torch.rand(rows, 5, generator=generator)
    scaled = act.clone().cuda()
    ops.scale_blocks(scaled, weights.cuda(), 8)
    assert torch.allclose(scaled.cpu(), (act.reshape(rows, 5, 8) * weights[:, :, None]).reshape(rows, 40), atol=1e-6)


# ---- through the programs a user runs ----------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", DTYPES)
def test_trace_replay_of_whole_requests_decoded_tails_and_batches(dtype, models, tmp_path):
    from test_trace_run_gpu import collect, replay, trace_batches, trace_tail, trace_whole
    folder, plain, _, _ = models["edges"]
    vocab = CONFIGS["edges"]["vocab"]
    lengths = {"a": 40, "b": 7, "c": 140, "d": 65, "e": 1, "f": 90}
    requests = {n: token_ids(vocab, length, seed=length) for n, length in lengths.items()}
    want = {n: plain.logits(ids) for n, ids in requests.items()}
    whole = trace_whole(requests)
    got_whole = collect(whole, replay(folder, dtype, tmp_path / "whole", whole, 256))
    tail = trace_tail(requests)
    got_tail = collect(tail, replay(folder, dtype, tmp_path / "tail", tail, 256))
    names = list(requests)
    batches = [{n: requests[n] for n in names[:3]}, {n: requests[n] for n in names[3:]}]
    batched = trace_batches(batches, lambda n, ids: max(1, len(ids) - 5 - ord(n) % 3))
    got_batched = collect(batched, replay(folder, dtype, tmp_path / "batched", batched, 384))
    for n in names:
        assert_logits(got_whole[n], want[n], dtype, f"trace whole {n}")
        assert_logits(got_tail[n], want[n], dtype, f"trace tail {n}")
        assert_logits(got_batched[n], want[n], dtype, f"trace batched {n}")


def test_the_command_line_generates_what_the_plain_loop_does(models):
    import os
    import subprocess
    import sys
    folder, plain, ids, _ = models["mixed"]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    prompts = [ids[:5], ids[30:31]]
    done = subprocess.run([sys.executable, os.path.join(root, "bin", "xrt"), "generate", "--model", folder, "--dtype", "float32",
                           "--prompt-ids", ";".join(",".join(map(str, p)) for p in prompts), "--max-tokens", "6",
                           "--temperature", "0", "--repetition-penalty", "1.0", "--stop-ids", ""],
                          capture_output=True, text=True, timeout=600)
    assert done.returncode == 0, done.stderr
    lines = [line for line in done.stdout.splitlines() if line.strip()]
    assert [[int(t) for t in line.split()] for line in lines] == [P.generate_greedy(plain, p, 6) for p in prompts]


# ---- configurations drawn at random: other sizes, orders and constants than any above -----------------------------------

def random_configuration(seed):
    import random
    r = random.Random(seed)
    width = r.choice([24, 40, 72, 96, 136])
    layers = []
    for _ in range(r.randint(2, 5)):
        kind = r.choice(["mamba2", "parallel"])
        if kind == "mamba2":
            groups = r.randint(1, 3)
            heads, vdim = groups * r.randint(1, 3), r.choice([8, 12, 20, 32, 64, 72])
            parts = r.choice([d for d in (1, 2, 3, 4, heads) if (heads * vdim) % d == 0])
            mixer = {"heads": heads, "vdim": vdim, "state": r.choice([4, 16, 24, 48, 64, 80, 128]), "groups": groups, "norm_groups": parts,
                     "conv": r.randint(1, 5)}
        else:
            kv_heads, dim = r.randint(1, 3), r.choice([6, 16, 20, 32, 64, 96])
            left = {"heads": kv_heads * r.randint(1, 3), "kv_heads": kv_heads, "dim": dim, "vdim": r.choice([4, 16, 24, 32, 96]),
                    "scale": r.choice([0.1, 0.25, 0.5])}
            if r.random() < 0.85:
                left["mask"] = {"size": r.choice([1, 2, 9, 40, 64, 65, 100, 300])}
            if r.random() < 0.85:
                left["rot"] = {"dims": r.choice([d for d in (2, 4, 6, 16, 20, 32, 48, 64, 96) if d <= dim]), "base": r.choice([100.0, 10000.0, 500000.0])}
                if r.random() < 0.7:
                    low = r.choice([1.0, 2.0])
                    left["rot"]["scaling"] = {"factor": r.choice([2.0, 8.0, 32.0]), "low": low, "high": low * r.choice([2.0, 4.0]),
                                              "original": r.choice([16, 64, 256])}
            mixer = {"left": left, "right": {"inner": r.choice([8, 40, 64, 100, 136]), "state": r.choice([1, 4, 8, 16, 24, 40]),
                                             "dt_rank": r.randint(1, 9), "conv": r.randint(1, 5)},
                     "left_scale": r.choice([0.5, 1.0, 1.25]), "right_scale": r.choice([0.5, 1.0, 1.25])}
        choice = r.random()
        if choice < 0.2:
            mlp = None
        elif choice < 0.6:
            mlp = {"kind": "dense", "ff": r.choice([16, 56, 104]), "limit": r.choice([0.5, 1.0, 7.0])}
        else:
            count = r.randint(1, 4)
            per = r.randint(1, 4)
            keep = r.randint(1, count)
            router = {"experts": count * per, "top": r.randint(1, keep * per)}
            if count > 1 or r.random() < 0.5:
                router["groups"] = {"count": count, "keep": keep}
            mlp = {"kind": "moe", "expert": {"ff": r.choice([8, 20, 48])}, "router": router}
        layers.append({"type": kind, "mixer": mixer, "mlp": mlp})
    raw = {"architecture": "Depunex", "vocab": r.choice([50, 97, 160]), "width": width, "norm": {"eps": r.choice([1e-6, 1e-5, 1e-3])},
           "embedding": {"scale": r.choice([1.0, 4.0, 9.5])}, "layers": layers}
    if r.random() < 0.8:
        raw["embedding"]["bigram"] = {"buckets": r.choice([1, 13, 211]), "mul_prev": r.randint(0, 40), "mul_cur": r.randint(1, 40)}
    if r.random() < 0.8:
        raw["token_side"] = {"dim": r.choice([1, 4, 16, 24])}
    if r.random() < 0.8:
        raw["logit_softcap"] = r.choice([5.0, 30.0])
    return raw


@pytest.mark.parametrize("seed", [1, 2, 3, 4, 5, 6, 7, 8, 9, 10])
def test_configurations_drawn_at_random(seed, tmp_path):
    from xeno_rt_amd.engine import Engine
    raw = random_configuration(seed)
    folder = make_depunex_folder(raw, tmp_path / "model", seed=seed, std=0.1)
    plain = P.PlainModel(folder)
    ids, other = token_ids(raw["vocab"], 150, seed=seed), token_ids(raw["vocab"], 45, seed=seed + 50)
    want, want_other = plain.logits(ids), plain.logits(other)
    for dtype in DTYPES:
        engine = Engine.load(folder, dtype=dtype, max_tokens=64 * 8, max_slots=2)
        what = f"drawn {seed}: {[layer['type'] for layer in raw['layers']]}"
        assert_logits(run_whole(engine, ids), want, dtype, what + " whole")
        assert_logits(in_portions(engine, ids, [70, 2, 1]), want, dtype, what + " in portions and decoded")
        got = run_batched(engine, [ids, other], [100, 3])
        assert_logits(got[0], want, dtype, what + " batched")
        assert_logits(got[1], want_other, dtype, what + " batched, the other")
        engine.cache.check()


def random_configuration_for_long_steps(seed):
    """Sizes that the kernels for steps of many tokens serve (heads of 64 or 128 whose values are as wide, chunks of whole cache
    blocks, experts' widths and a model width in multiples of 64, many experts of which few are chosen), mixed with some that
    they do not serve."""
    import random
    r = random.Random(1000 + seed)
    width = r.choice([64, 128, 192])
    layers = []
    for index in range(r.randint(2, 3)):
        if index % 2 == seed % 2:
            heads = r.randint(1, 3)
            mixer = {"heads": heads, "vdim": r.choice([16, 32]), "state": r.choice([8, 32]), "groups": 1, "norm_groups": r.choice([1, heads]),
                     "conv": r.randint(2, 4)}
            kind = "mamba2"
        else:
            kv_heads, dim = r.randint(1, 2), r.choice([64, 128])
            left = {"heads": kv_heads * r.randint(1, 2), "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": dim ** -0.5}
            if r.random() < 0.8:
                left["mask"] = {"size": r.choice([64, 128, 192, 100])}
            left["rot"] = {"dims": r.choice([16, dim // 2, dim]), "base": 10000.0}
            mixer = {"left": left, "right": {"inner": 32, "state": 4, "dt_rank": 2, "conv": 3}, "left_scale": 1.0, "right_scale": 0.5}
            kind = "parallel"
        count = r.choice([1, 2, 4])
        per = r.choice([3, 4, 6])
        router = {"experts": count * per, "top": r.randint(1, 2)}
        if count > 1:
            router["groups"] = {"count": count, "keep": r.randint(1, count)}
        layers.append({"type": kind, "mixer": mixer, "mlp": {"kind": "moe", "expert": {"ff": r.choice([64, 128, 48])}, "router": router}})
    return {"architecture": "Depunex", "vocab": 90, "width": width, "norm": {"eps": 1e-5}, "embedding": {"scale": 2.0}, "logit_softcap": 20.0,
            "layers": layers}


@pytest.mark.parametrize("seed", [1, 2, 3, 4, 5, 6])
def test_configurations_drawn_at_random_for_steps_of_many_tokens(seed, tmp_path):
    """In float32 against the plain model; in bfloat16 the kernels that only steps of many tokens take (sorted experts, chunks
    on the matrix cores) against the same engine without them, which chooses the same experts from the same rows."""
    from xeno_rt_amd.engine import Engine
    raw = random_configuration_for_long_steps(seed)
    folder = make_depunex_folder(raw, tmp_path / "model", seed=seed, std=0.1, router_std=0.08)
    plain = P.PlainModel(folder)
    requests = [token_ids(raw["vocab"], length, seed=seed + length) for length in (330, 290)]
    engine = Engine.load(folder, dtype="float32", max_tokens=64 * 12, max_slots=2)
    for ids in requests:
        assert_logits(run_whole(engine, ids), plain.logits(ids), "float32", f"drawn for long steps {seed}, {len(ids)} tokens")
    del engine
    engine = Engine.load(folder, dtype="bfloat16", max_tokens=64 * 12, max_slots=2)
    ops = engine.runtime.ops
    fast = (ops.experts_sorted_takes, ops._attention_stretches)
    ops.experts_sorted_takes, ops._attention_stretches = (lambda *operands: False), (lambda *operands: False)
    wants = [run_whole(engine, ids) for ids in requests]
    ops.experts_sorted_takes, ops._attention_stretches = fast

    def close(got, want, what):
        per_row = (got.double() - want.double()).abs().max(dim=1).values / float(want.abs().max())
        rms = errors(got, want)[1]
        assert int((per_row > 5e-2).sum()) <= max(3, len(per_row) // 50) and rms <= 1.5e-2, \
            f"drawn for long steps {seed}, {what}: rows {(per_row > 5e-2).nonzero().flatten().tolist()} differ, rms {rms:.2e}"

    for ids, want in zip(requests, wants):
        close(run_whole(engine, ids), want, f"{len(ids)} tokens whole")
        close(in_portions(engine, ids, [200, 100, 1]), want, f"{len(ids)} tokens in portions")
    for index, (got, want) in enumerate(zip(run_batched(engine, requests, [330, 280]), wants)):
        close(got, want, f"batched, request {index}")
    engine.cache.check()


def test_zz_the_largest_errors_seen_are_reported():
    for dtype, (worst, rms) in WORST.items():
        print(f"depunex {dtype}: largest max error {worst:.3e}, largest rms error {rms:.3e}")
