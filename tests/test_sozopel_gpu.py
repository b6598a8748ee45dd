"""The Sozopel decoder on the GPU against the plain implementation (tests/plain_sozopel.py), for three small
configurations that differ in every size and option: whole prompts, token-by-token decoding from the first token,
portions of several sizes, unequal batches through reused slots, long decoding across window and block borders, greedy
generation through the library's loop; and every new mechanism alone against plain arithmetic, with inputs made so
that a window's edge, a far state or a sink shows.

In 32-bit the kernels work a sequence off in its own order whatever the step looks like, so logits are also compared
bit for bit between schedules, as long as no step brings a sequence more than 32 tokens: a longer portion is cut into
segments whose recurrent states are worked out side by side and joined afterwards, the same sums in another order,
and is compared within the sums' rounding instead."""
import math

import pytest
import torch

from helpers import errors, run_batched, run_whole, token_ids
from sozopel_models import CONFIGS, make_sozopel_folder
import plain_sozopel as P

pytestmark = pytest.mark.gpu
DTYPES = ["float32", "bfloat16"]
NAMES = sorted(CONFIGS)
LENGTH = {"mixed": 150, "wide": 140, "one_tap": 90}

# Largest difference from the plain implementation (float64), relative to the largest logit. This design divides the
# output of every head of a recurrence by its own root mean square: where a head's output is small because q . k nearly
# cancels (the first tokens of a sequence, whose state holds one or two keys), the rounding of that sum is scaled up
# with it, so single logits, and the root mean square over a sequence of one or two tokens, differ by more than the
# sums' own rounding (largest seen: 2.8e-5 and 8.8e-6, on a one-token sequence).
# In bfloat16 the same happens to the rounding of q and k themselves, so single logits stand out from a root mean square of 1e-2.
LIMITS = {"float32": dict(max=1e-4, rms=2e-5), "bfloat16": dict(max=1e-1, rms=2.5e-2)}
WORST = {}


def assert_logits(got, want, dtype, what):
    assert torch.isfinite(got).all(), f"{what}: logits are not finite"
    worst, rms = errors(got, want)
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
        folder = make_sozopel_folder(CONFIGS[name], tmp_path_factory.mktemp(name), seed=5 + index, keep_rank=(name != "wide"))
        plain = P.PlainModel(folder)
        ids = token_ids(CONFIGS[name]["vocab"], LENGTH[name], seed=300 + index)
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
    return float((got - want).abs().max()) <= 2e-5 * float(want.abs().max())


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
    assert_logits(got, want, dtype, f"sozopel {name} whole, first bad row {first_bad_position(got, want, dtype)}")
    for length in (1, 2, 3, 66):                                    # the first tokens of a sequence, and just past a block
        got = run_whole(engine, ids[:length])
        assert_logits(got, want[:length], dtype, f"sozopel {name} whole, {length} tokens")
    engine.cache.check()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_token_by_token_from_the_first(name, dtype, models, engines):
    """Every token in a step of its own: long decoding through recorded steps, across windows and cache blocks."""
    engine = engines(name, dtype)
    _, plain, ids, want = models[name]
    got = in_portions(engine, ids, [1])
    assert_logits(got, want, dtype, f"sozopel {name} token by token, first bad row {first_bad_position(got, want, dtype)}")
    if dtype == "float32":
        assert same_but_for_rounding(got, run_whole(engine, ids)), "a decoded token differs from the same token in a prompt"
        assert torch.equal(got[:30], run_whole(engine, ids[:30])), "a decoded token's bits differ from the same token's in a short prompt"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("sizes", [[2], [3, 7], [64, 1], [65, 2, 2, 1, 30], [33], [1, 1, 2, 61, 5]])
@pytest.mark.parametrize("name", NAMES)
def test_portions(name, sizes, dtype, models, engines):
    engine = engines(name, dtype)
    _, plain, ids, want = models[name]
    got = in_portions(engine, ids, sizes)
    assert_logits(got, want, dtype, f"sozopel {name} portions {sizes}, first bad row {first_bad_position(got, want, dtype)}")
    if dtype == "float32":
        assert same_but_for_rounding(got, run_whole(engine, ids)), f"portions {sizes} change more than the rounding"
        if max(sizes) <= 32:
            assert torch.equal(got, in_portions(engine, ids, [1])), f"portions {sizes} change the bits"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_unequal_batches_through_reused_slots(name, dtype, models, engines):
    """Three requests of different lengths start together and end one after the other, twice over, so that the second
    round runs in slots, blocks and states that the first has used."""
    engine = engines(name, dtype)
    _, plain, ids, want = models[name]
    vocab = CONFIGS[name]["vocab"]
    requests = [ids, token_ids(vocab, 37, seed=900), token_ids(vocab, 71, seed=901)]
    wants = [want, plain.logits(requests[1]), plain.logits(requests[2])]
    for prompts in ([len(ids) - 40, 5, 66], [3, 36, 1]):
        got = run_batched(engine, requests, prompts)
        for index, (g, w) in enumerate(zip(got, wants)):
            assert_logits(g, w, dtype, f"sozopel {name} batch {prompts} request {index}, first bad row {first_bad_position(g, w, dtype)}")
            if dtype == "float32":
                assert same_but_for_rounding(g, run_whole(engine, requests[index])), "a request depends on its batch"
                if max(prompts) <= 32:
                    assert torch.equal(g, in_portions(engine, requests[index], [1])), "a request's bits depend on its batch"
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


def test_inner_widths_come_from_the_tensors_when_the_configuration_leaves_them_out(models, engines):
    engine = engines("wide", "float32")                              # its config.json has no 'rank'
    assert [layer["mixer"].get("rank") or layer["mixer"].get("right", {}).get("rank") for layer in engine.config.layers] == [8, 4, None, 16]


# ---- every mechanism alone -------------------------------------------------------------------------------------

class Step:
    """A step's sequences as the kernels want them described: `counts[i]` new tokens of the sequence in `slots[i]`."""

    def __init__(self, slots, counts, starts, device="cuda"):
        ints = lambda values: torch.tensor(values, dtype=torch.int32, device=device)
        offsets = [0]
        for count in counts:
            offsets.append(offsets[-1] + count)
        self.n_tokens, self.n_sequences, self.max_count = offsets[-1], len(slots), max(counts)
        self.sequence_offsets, self.sequence_slots, self.sequence_starts = ints(offsets), ints(slots), ints(starts)
        self.positions = ints([start + t for start, count in zip(starts, counts) for t in range(count)])
        self.slots = ints([slot for slot, count in zip(slots, counts) for _ in range(count)])
        self.max_context = max(start + count for start, count in zip(starts, counts))


def schedules(length):
    """Ways to cut a sequence of `length` tokens into steps."""
    return [[length], [1] * length, [2] * (length // 2) + [length % 2] * (length % 2), [length - 3, 1, 2], [70, length - 70]]


@pytest.fixture(scope="module")
def ops():
    from xeno_rt_amd.ops import load_ops
    return load_ops()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("taps,plus_input", [(1, True), (2, False), (4, True), (5, False)])
def test_short_convolution(taps, plus_input, dtype, ops):
    length, channels = 150, 72
    generator = torch.Generator().manual_seed(taps)
    u = torch.randn(length, channels, generator=generator).to(dtype)
    w = torch.randn(channels, taps, generator=generator).to(dtype)
    want = P.causal_conv(u.double(), w.double()) + (u.double() if plus_input else 0)
    for cuts in schedules(length):
        state = torch.full((3, taps - 1, channels), 7.0, device="cuda")     # slots 0 and 2 hold what another sequence left
        state[1].zero_()
        rows, at = [], 0
        for count in cuts:
            out = torch.empty(2 + count, channels, dtype=dtype, device="cuda")
            # the sequence under test between a padding sequence and nothing: its rows are 1 .. count
            step = Step([-1, 1], [2, count], [0, at])
            x = torch.cat([torch.ones(2, channels, dtype=dtype), u[at:at + count]]).cuda()
            ops.short_conv(x, w.cuda(), state, step, out, mode="plus_input" if plus_input else "plain")
            assert float(out[:2].abs().max()) == 0.0
            rows.append(out[2:])
            at += count
        got = torch.cat(rows).double().cpu()
        limit = 1e-5 if dtype == torch.float32 else 3e-2
        assert float((got - want).abs().max()) <= limit * float(want.abs().max()), f"taps {taps}, cuts {cuts[:4]}"
        if taps > 1:
            assert float(state[0].min()) == 7.0 and float(state[2].max()) == 7.0, "another sequence's state was touched"


def test_token_shift_gives_every_reader_its_own_mix(ops):
    length, channels = 9, 40
    generator = torch.Generator().manual_seed(3)
    u, mu = torch.randn(length, channels, generator=generator), torch.rand(3, channels, generator=generator)
    before = torch.cat([torch.zeros(1, channels), u[:-1]])
    want = torch.stack([u + (before - u) * m for m in mu])
    for cuts in ([length], [1] * length, [4, 5]):
        state, rows, at = torch.zeros(2, 1, channels, device="cuda"), [], 0
        for count in cuts:
            out = torch.empty(3, count, channels, device="cuda")
            ops.short_conv(u[at:at + count].cuda(), mu.cuda(), state, Step([1], [count], [at]), out, mode="towards_last")
            rows.append(out)
            at += count
        assert torch.allclose(torch.cat(rows, dim=1).cpu(), want, atol=1e-6)


def run_recurrence(ops, q, k, v, cuts, dtype, heads, dim, vdim, **options):
    state = torch.zeros(2, heads, dim, vdim, device="cuda")
    rows, at = [], 0
    for count in cuts:
        cut = lambda t: None if t is None else t[at:at + count].to("cuda")
        out = torch.empty(count, heads * vdim, dtype=dtype, device="cuda")
        step_options = dict(options)
        if step_options.get("decay_mode", "per_head") != "per_head":
            step_options["decay"] = cut(options["decay"])
        if "gate" in options:
            step_options["gate"] = cut(options["gate"])
        ops.linear_recurrence(cut(q), cut(k), cut(v), state, Step([1], [count], [at]), out, heads, dim, vdim, **step_options)
        rows.append(out)
        at += count
    return torch.cat(rows).double().cpu(), state


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,dim,vdim", [(3, 20, 36), (1, 8, 136), (2, 64, 64), (2, 136, 16), (1, 256, 40)])
def test_linear_recurrence_in_its_three_forms(heads, dim, vdim, dtype, ops):
    length = 90
    generator = torch.Generator().manual_seed(dim)
    rand = lambda *shape: torch.randn(*shape, generator=generator)
    q, k, v = rand(length, heads * dim).to(dtype), rand(length, heads * dim).to(dtype), rand(length, heads * vdim).to(dtype)
    gate = rand(length, heads * vdim).to(dtype)
    z, bias, bonus = rand(length, heads * dim), rand(heads * dim), rand(heads, dim)
    weight_head, weight_all = 1 + 0.3 * rand(vdim), 1 + 0.3 * rand(heads * vdim)
    qd, kd, vd = (t.double().reshape(length, heads, -1) for t in (q, k, v))
    per_head = torch.tensor([0.5 + 0.49 * h / heads for h in range(heads)])
    eps = 1e-3
    cases = {
        "fixed decay, k scaled, unit norm, silu gate": (
            dict(decay=per_head.cuda(), decay_mode="per_head", k_scale=dim ** -0.5, norm_eps=eps, gate=gate),
            lambda: P.rms_divide(P.recurrence(qd, kd * dim ** -0.5, vd, per_head.double()[None, :, None].expand(length, heads, dim)), eps)
            .reshape(length, -1) * P.silu(gate.double())),
        "sigmoid decay with power, q scaled, weight per head": (
            dict(decay=z, decay_mode="sigmoid_power", decay_bias=bias.cuda(), decay_power=1 / 7.0, q_scale=dim ** -0.5, norm_eps=eps,
                 norm_weight=weight_head.cuda(), gate=gate),
            lambda: (P.rms_divide(P.recurrence(qd * dim ** -0.5, kd, vd, torch.sigmoid((z + bias).double()).pow(1 / 7.0).reshape(length, heads, dim)), eps)
                     * weight_head.double()).reshape(length, -1) * P.silu(gate.double())),
        "double exponential decay, bonus, weight over all heads": (
            dict(decay=z, decay_mode="exp_neg_exp", decay_bias=bias.cuda(), bonus=bonus.cuda(), norm_eps=eps, norm_weight=weight_all.cuda(), gate=gate),
            lambda: P.rms_divide(P.recurrence(qd, kd, vd, torch.exp(-torch.exp((z + bias).double())).reshape(length, heads, dim), bonus=bonus.double()), eps)
            .reshape(length, -1) * weight_all.double() * P.silu(gate.double())),
        "decay given, nothing after": (
            dict(decay=torch.sigmoid(z), decay_mode="given"),
            lambda: P.recurrence(qd, kd, vd, torch.sigmoid(z).double().reshape(length, heads, dim)).reshape(length, -1)),
    }
    for what, (options, plain) in cases.items():
        want = plain()
        first = None
        for cuts in schedules(length):
            got, state = run_recurrence(ops, q, k, v, cuts, dtype, heads, dim, vdim, **options)
            limit = 2e-5 if dtype == torch.float32 else 2e-2
            assert float((got - want).abs().max()) <= limit * float(want.abs().max()), f"{what}, cuts {cuts[:4]}"
            assert float(state[0].abs().max()) == 0.0, "another sequence's state was touched"
            if max(cuts) > 32:                       # (segments side by side: the same sums in another order)
                continue
            if first is None:
                first = (got, state.clone())
            else:
                assert torch.equal(got, first[0]) and torch.equal(state, first[1]), f"{what}: cuts {cuts[:4]} change the bits"


def test_recurrence_of_unequal_sequences_in_one_step(ops):
    """Sequences of 200, 65 and 3 tokens and one that is padding, in one step (the long ones in several segments) and then one
    more token each: every sequence as it is alone, and the padding's rows zeros."""
    heads, dim, vdim, lengths = 2, 24, 40, [200, 65, 3]
    generator = torch.Generator().manual_seed(8)
    total = sum(lengths) + 2
    q, k = torch.randn(total + 3, heads * dim, generator=generator), torch.randn(total + 3, heads * dim, generator=generator)
    v, z = torch.randn(total + 3, heads * vdim, generator=generator), torch.randn(total + 3, heads * dim, generator=generator)
    options = dict(decay_mode="sigmoid_power", decay_power=0.25, norm_eps=1e-5)
    state = torch.zeros(5, heads, dim, vdim, device="cuda")
    out = torch.empty(total, heads * vdim, device="cuda")
    step = Step([3, -1, 1, 4], [lengths[0], 2, lengths[1], lengths[2]], [0, 0, 0, 0])
    ops.linear_recurrence(q[:total].cuda(), k[:total].cuda(), v[:total].cuda(), state, step, out, heads, dim, vdim, z[:total].cuda(), **options)
    more = torch.empty(3, heads * vdim, device="cuda")
    ops.linear_recurrence(q[total:].cuda(), k[total:].cuda(), v[total:].cuda(), state, Step([3, 1, 4], [1, 1, 1], lengths), more,
                          heads, dim, vdim, z[total:].cuda(), **options)
    assert float(out[200:202].abs().max()) == 0.0 and float(state[0].abs().max()) == 0.0 and float(state[2].abs().max()) == 0.0
    begins = [0, 202, 267]
    for index, (begin, length) in enumerate(zip(begins, lengths)):
        rows = list(range(begin, begin + length)) + [total + index]
        qd, kd, vd = (t[rows].double().reshape(length + 1, heads, -1) for t in (q, k, v))
        decay = torch.sigmoid(z[rows].double()).pow(0.25).reshape(length + 1, heads, dim)
        want = P.rms_divide(P.recurrence(qd, kd, vd, decay), 1e-5).reshape(length + 1, -1)
        got = torch.cat([out[begin:begin + length], more[index:index + 1]]).double().cpu()
        assert float((got - want).abs().max()) <= 2e-5 * float(want.abs().max()), f"sequence {index}"


def test_a_state_keeps_a_token_from_far_back(ops):
    """With a decay of one, what the first token wrote is read unchanged three hundred tokens on, in a prompt and decoded."""
    length, heads, dim, vdim = 300, 1, 16, 32
    q, k, v = torch.zeros(length, dim), torch.zeros(length, dim), torch.randn(length, vdim, generator=torch.Generator().manual_seed(1))
    k[0, 3], q[-1, 3] = 1.0, 2.0
    decay = torch.ones(1, device="cuda")
    for cuts in ([length], [length - 40] + [1] * 40):
        got, _ = run_recurrence(ops, q, k, v, cuts, torch.float32, heads, dim, vdim, decay=decay)
        assert torch.allclose(got[-1].float(), 2.0 * v[0]) and float(got[1:-1].abs().max()) == 0.0


def attend(ops, q, k, v, cuts, dtype, n_heads, n_kv_heads, dim, vdim, **options):
    """Keys and values through `kv_store` into a paged cache whose blocks lie in another order than the sequence's, then
    the general attention kernel, step by step."""
    from xeno_rt_amd.cache import BLOCK_TOKENS
    from xeno_rt_amd.cache.sequence_cache import KVView
    from xeno_rt_amd.parts.base import KVSpec
    length = q.shape[0]
    blocks = (length + BLOCK_TOKENS - 1) // BLOCK_TOKENS
    table = torch.full((2, blocks), -1, dtype=torch.int32)
    table[1] = torch.arange(blocks - 1, -1, -1, dtype=torch.int32) + 1
    kv = KVView(KVSpec(n_kv_heads, dim, options.get("window"), vdim),
                torch.zeros(blocks + 1, n_kv_heads, BLOCK_TOKENS, dim, dtype=dtype, device="cuda"),
                torch.zeros(blocks + 1, n_kv_heads, vdim, BLOCK_TOKENS, dtype=dtype, device="cuda"), table.cuda())
    rows, at = [], 0
    for count in cuts:
        if count == 0:
            continue
        step = Step([1], [count], [at])
        qkv = torch.cat([q[at:at + count], k[at:at + count], v[at:at + count]], dim=1).to(dtype).cuda().contiguous()
        ops.kv_store(qkv[:, n_heads * dim:(n_heads + n_kv_heads) * dim], qkv[:, (n_heads + n_kv_heads) * dim:], n_kv_heads, dim, vdim, kv, step)
        out = torch.empty(count, n_heads * vdim, dtype=dtype, device="cuda")
        ops.attention(qkv, n_heads, n_kv_heads, dim, kv, step, out, value_dim=vdim, **options)
        rows.append(out)
        at += count
    return torch.cat(rows).double().cpu()


def plain_attention(q, k, v, n_heads, n_kv_heads, dim, vdim, scale, window, slopes, sink):
    length = q.shape[0]
    q, k, v = q.double().reshape(length, n_heads, dim), k.double().reshape(length, n_kv_heads, dim), v.double().reshape(length, n_kv_heads, vdim)
    out = torch.zeros(length, n_heads, vdim, dtype=torch.float64)
    for head in range(n_heads):
        group = head // (n_heads // n_kv_heads)
        for i in range(length):
            lo = max(0, i - window + 1) if window else 0
            s = (k[lo:i + 1, group] @ q[i, head]) * scale
            if slopes is not None:
                s = s - float(slopes[head]) * (i - torch.arange(lo, i + 1, dtype=torch.float64))
            e = torch.exp(s - (max(float(s.max()), 0.0) if sink else s.max()))
            total = e.sum() + (math.exp(-max(float(s.max()), 0.0)) if sink else 0.0)
            out[i, head] = (e / total) @ v[lo:i + 1, group]
    return out.reshape(length, n_heads * vdim)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n_heads,n_kv_heads,dim,vdim,window", [(6, 3, 24, 40, 17), (2, 2, 32, 32, 70), (4, 1, 16, 8, 3),
                                                               (1, 1, 64, 96, None), (8, 2, 48, 20, 64)])
def test_attention_with_a_sink_a_window_a_bias_and_values_of_their_own_width(n_heads, n_kv_heads, dim, vdim, window, dtype, ops):
    length = 150
    generator = torch.Generator().manual_seed(dim + vdim)
    q, k = torch.randn(length, n_heads * dim, generator=generator), torch.randn(length, n_kv_heads * dim, generator=generator)
    v = torch.randn(length, n_kv_heads * vdim, generator=generator)
    q, k, v = (t.to(dtype).float() for t in (q, k, v))
    slopes = torch.tensor([2.0 ** (-8.0 * (h + 1) / n_heads) for h in range(n_heads)])
    scale = 0.4 / math.sqrt(dim)
    for sink, biased in ((True, True), (True, False), (False, True)):
        want = plain_attention(q, k, v, n_heads, n_kv_heads, dim, vdim, scale, window, slopes if biased else None, sink)
        options = dict(scale=scale, window=window, sink=sink, **({"distance_slopes": slopes.cuda()} if biased else {}))
        first = None
        for cuts in schedules(length):
            got = attend(ops, q, k, v, cuts, dtype, n_heads, n_kv_heads, dim, vdim, **options)
            limit = 1e-5 if dtype == torch.float32 else 2e-2
            assert float((got - want).abs().max()) <= limit * float(want.abs().max()), f"sink {sink}, biased {biased}, cuts {cuts[:4]}"
            if first is None:
                first = got
            else:
                assert torch.equal(got, first), f"cuts {cuts[:4]} change the bits"


@pytest.mark.parametrize("window", [3, 17, 64, 70, 129])
def test_a_key_just_inside_the_window_is_seen_and_one_just_outside_is_not(window, ops):
    """One key whose score towers over the rest, at the last place the window keeps and at the first it drops, for queries
    in a prompt and decoded, with the key on either side of a cache block's border."""
    n_heads, dim, vdim, length = 2, 16, 8, 200
    for query in (window + 1, 130, 199):
        for distance, seen in ((window - 1, True), (window, False)):
            key = query - distance
            if key < 0:
                continue
            q, k = torch.zeros(length, n_heads * dim), torch.zeros(length, n_heads * dim)
            v = torch.zeros(length, n_heads * vdim)
            q[query], k[key], v[key] = 6.0, 6.0, 1.0                       # score 6 * 6 * 16 * scale
            want_value = 1.0 if seen else 0.0
            for cuts in ([length], [query, 1, length - query - 1], [query - 1, 2, length - query - 1]):
                got = attend(ops, q, k, v, cuts, torch.float32, n_heads, n_heads, dim, vdim, scale=0.05, window=window, sink=True)
                assert abs(float(got[query, 0]) - want_value) < 1e-3, f"window {window}, query {query}, key {key}, cuts {cuts}"


def test_the_sink_takes_its_share(ops):
    """With all scores zero, n keys and the sink share the weight evenly: the output is the values' sum over n + 1."""
    n, dim, vdim = 5, 16, 16
    q, k, v = torch.zeros(n, dim), torch.randn(n, dim), torch.ones(n, vdim)
    got = attend(ops, q, k, v, [n], torch.float32, 1, 1, dim, vdim, scale=1.0, window=None, sink=True)
    for i in range(n):
        assert abs(float(got[i, 0]) - (i + 1) / (i + 2)) < 1e-6


def test_small_operations(ops):
    generator = torch.Generator().manual_seed(9)
    rows, width = 7, 40
    residual, a, b = (torch.randn(rows, width, generator=generator) for _ in range(3))
    ga, gb = torch.randn(width, generator=generator), torch.randn(width, generator=generator)
    want = residual.double() + 0.5 * (P.rms_divide(a.double(), 1e-5) * ga.double() + P.rms_divide(b.double(), 1e-5) * gb.double())
    got = residual.clone().cuda()
    ops.add_normed(got, [(a.cuda(), ga.cuda()), (b.cuda(), gb.cuda())], 1e-5, 0.5)
    assert torch.allclose(got.cpu().double(), want, atol=1e-5)
    z = torch.linspace(-6, 6, 301)
    params = torch.tensor([0.3, -0.7])
    for kind, plain in (("tanh", torch.tanh(z.double())), ("silu", P.silu(z.double())),
                        ("xielu", P.xielu(z.double(), params[0].double(), params[1].double()))):
        out = torch.empty(301, device="cuda")
        ops.activation(z.cuda(), out, kind, params.cuda() if kind == "xielu" else None)
        assert torch.allclose(out.cpu().double(), plain, atol=1e-5), kind
    table, x = torch.randn(11, width, generator=generator), torch.randn(4, width, generator=generator)
    ids = torch.tensor([3, 0, 10, 3], dtype=torch.int32)
    got = x.clone().cuda()
    ops.rows_add(table.cuda(), ids.cuda(), got)
    assert torch.equal(got.cpu(), x + table[ids.long()])


# ---- through the programs a user runs ----------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", DTYPES)
def test_trace_replay_of_whole_requests_decoded_tails_and_batches(dtype, models, tmp_path):
    """`bin/trace_run` as a program of its own on a folder whose config.json leaves the inner widths to the tensors: each
    request whole, with its last tokens one by one, and in batches of unequal requests that are decoded together."""
    from test_trace_run_gpu import collect, replay, trace_batches, trace_tail, trace_whole
    folder, plain, _, _ = models["wide"]
    vocab = CONFIGS["wide"]["vocab"]
    lengths = {"a": 40, "b": 7, "c": 100, "d": 65, "e": 1, "f": 90}
    requests = {n: token_ids(vocab, length, seed=length) for n, length in lengths.items()}
    want = {n: plain.logits(ids) for n, ids in requests.items()}
    whole = trace_whole(requests)
    got_whole = collect(whole, replay(folder, dtype, tmp_path / "whole", whole, 128))
    tail = trace_tail(requests)
    got_tail = collect(tail, replay(folder, dtype, tmp_path / "tail", tail, 128))
    names = list(requests)
    batches = [{n: requests[n] for n in names[:3]}, {n: requests[n] for n in names[3:]}]
    batched = trace_batches(batches, lambda n, ids: max(1, len(ids) - 5 - ord(n) % 3))
    got_batched = collect(batched, replay(folder, dtype, tmp_path / "batched", batched, 256))
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
        kind = r.choice(["retention", "wkv", "parallel"])
        if kind == "retention":
            heads = r.randint(1, 4)
            mixer = {"heads": heads, "dim": r.choice([4, 12, 20, 32, 48]), "vdim": r.choice([8, 20, 40, 72]),
                     "decay": [round(1.0 - 2.0 ** -r.randint(1, 9), 6) for _ in range(heads)]}
        elif kind == "wkv":
            mixer = {"heads": r.randint(1, 5), "dim": r.choice([8, 16, 24, 40, 64]), "rank": r.choice([3, 8, 12])}
        else:
            kv_heads = r.randint(1, 3)
            mixer = {"left": {"heads": kv_heads * r.randint(1, 3), "kv_heads": kv_heads, "dim": r.choice([6, 16, 20, 32, 64]),
                              "vdim": r.choice([4, 16, 24, 32, 96]), "conv": r.randint(1, 6), "mask": {"size": r.choice([1, 2, 9, 40, 64, 65, 300])},
                              "scale": r.choice([0.1, 0.25, 0.5])},
                     "right": {"heads": r.randint(1, 3), "dim": r.choice([8, 24, 32, 72]), "vdim": r.choice([8, 24, 64, 80]),
                               "tau": r.choice([1.0, 4.0, 16.0, 64.0]), "rank": r.choice([2, 8, 16])}}
        layers.append({"type": kind, "mixer": mixer, "mlp": r.choice([None, {"kind": "dense", "ff": r.choice([16, 56, 104])}])})
    return {"architecture": "Sozopel", "vocab": r.choice([50, 97, 160]), "width": width, "max_positions": 200,
            "norm": {"eps": r.choice([1e-6, 1e-5, 1e-3])}, "canon": {"taps": r.randint(1, 6)}, "layers": layers}


@pytest.mark.parametrize("seed", [1, 2, 3, 4, 5, 6, 7, 8])
def test_configurations_drawn_at_random(seed, tmp_path):
    from xeno_rt_amd.engine import Engine
    raw = random_configuration(seed)
    # (matrices of deviation 0.1: with 0.2, as in the fixed configurations, the widest of these models round single logits by 16 % in bfloat16)
    folder = make_sozopel_folder(raw, tmp_path / "model", seed=seed, std=0.1, keep_rank=seed % 2 == 0)
    plain = P.PlainModel(folder)
    ids, other = token_ids(raw["vocab"], 110, seed=seed), token_ids(raw["vocab"], 45, seed=seed + 50)
    want, want_other = plain.logits(ids), plain.logits(other)
    for dtype in DTYPES:
        engine = Engine.load(folder, dtype=dtype, max_tokens=64 * 6, max_slots=2)
        what = f"drawn {seed}: {[layer['type'] for layer in raw['layers']]}"
        assert_logits(run_whole(engine, ids), want, dtype, what + " whole")
        assert_logits(in_portions(engine, ids, [70, 2, 1]), want, dtype, what + " in portions and decoded")
        got = run_batched(engine, [ids, other], [80, 3])
        assert_logits(got[0], want, dtype, what + " batched")
        assert_logits(got[1], want_other, dtype, what + " batched, the other")
        engine.cache.check()


def test_the_largest_errors_seen_are_reported():
    print("largest errors against the plain model (max, rms):", {k: [f"{x:.2e}" for x in v] for k, v in WORST.items()})
