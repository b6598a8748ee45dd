"""The Ledudra decoder on the GPU against the plain implementation (tests/plain_ledudra.py), for three small
configurations that differ in every size and option: whole prompts, token-by-token decoding from the first token,
portions of several sizes, unequal batches through reused slots, long decoding across window and block borders, greedy
generation through the library's loop; and every new mechanism alone against plain arithmetic, with inputs made so
that a window's edge, a far key, a bucket of distances or a share of another layer's values shows.

In 32-bit every kernel of this design works a token off in an order that depends on the token alone, so logits are also
compared bit for bit between schedules."""
import math

import pytest
import torch

from helpers import errors, run_batched, run_whole, token_ids
from ledudra_models import CONFIGS, make_ledudra_folder
import plain_ledudra as P

pytestmark = pytest.mark.gpu
DTYPES = ["float32", "bfloat16"]
NAMES = sorted(CONFIGS)
LENGTH = {"mixed": 150, "wide": 200, "narrow": 90}

# Largest difference from the plain implementation (float64), relative to the largest logit. A layer norm stands behind
# every sublayer, so what a sublayer's rounding does to the stream does not depend on how large its output is; weights
# that are not normalised over the keys add up roundings of up to a window's worth of values. Largest seen over all tests
# below: float32 6.4e-7 (rms 1.4e-7), bfloat16 1.3e-2 (rms 2.2e-3).
LIMITS = {"float32": dict(max=5e-6, rms=1e-6), "bfloat16": dict(max=5e-2, rms=1e-2)}
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
        folder = make_ledudra_folder(CONFIGS[name], tmp_path_factory.mktemp(name), seed=11 + index, keep_rows=(name != "wide"))
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
            cache[(name, dtype)] = Engine.load(models[name][0], dtype=dtype, max_tokens=64 * 10, max_slots=3)
        return cache[(name, dtype)]
    return get


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
    assert_logits(got, want, dtype, f"ledudra {name} whole, first bad row {first_bad_position(got, want, dtype)}")
    for length in (1, 2, 3, 66):                                    # the first tokens of a sequence, and just past a block
        got = run_whole(engine, ids[:length])
        assert_logits(got, want[:length], dtype, f"ledudra {name} whole, {length} tokens")
    engine.cache.check()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_token_by_token_from_the_first(name, dtype, models, engines):
    """Every token in a step of its own: long decoding through recorded steps, across windows and cache blocks."""
    engine = engines(name, dtype)
    assert engine.graphs is not None, "a decode step of this design is recorded"
    _, plain, ids, want = models[name]
    got = in_portions(engine, ids, [1])
    assert_logits(got, want, dtype, f"ledudra {name} token by token, first bad row {first_bad_position(got, want, dtype)}")
    if dtype == "float32":
        assert torch.equal(got, run_whole(engine, ids)), "a decoded token's bits differ from the same token's in a prompt"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("sizes", [[2], [3, 7], [64, 1], [65, 2, 2, 1, 30], [33], [1, 1, 2, 61, 5]])
@pytest.mark.parametrize("name", NAMES)
def test_portions(name, sizes, dtype, models, engines):
    engine = engines(name, dtype)
    _, plain, ids, want = models[name]
    got = in_portions(engine, ids, sizes)
    assert_logits(got, want, dtype, f"ledudra {name} portions {sizes}, first bad row {first_bad_position(got, want, dtype)}")
    if dtype == "float32":
        assert torch.equal(got, run_whole(engine, ids)), f"portions {sizes} change the bits"


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
            assert_logits(g, w, dtype, f"ledudra {name} batch {prompts} request {index}, first bad row {first_bad_position(g, w, dtype)}")
            if dtype == "float32":
                assert torch.equal(g, run_whole(engine, requests[index])), "a request's bits depend on its batch"
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


def test_the_rows_of_a_bias_table_come_from_the_tensors_when_the_configuration_leaves_them_out(models, engines):
    engine = engines("wide", "float32")                              # its config.json has no 'bias_rows'
    assert [layer["mixer"].get("bias_rows") for layer in engine.config.layers] == [7, None, 32, None]


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


@pytest.mark.parametrize("small", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width", [40, 64, 257, 1000])
def test_layer_norms(width, small, ops):
    """The norm alone, gathered rows, and the norm behind a sublayer with a bias on its way in and the next norm on its way out."""
    generator = torch.Generator().manual_seed(width)
    rand = lambda *shape: torch.randn(*shape, generator=generator)
    rows = 9
    x, y = 3.0 + 2.0 * rand(rows, width), rand(rows, width)
    w, b, pre = (1 + 0.3 * rand(width)).to(small), (0.3 * rand(width)).to(small), rand(width).to(small)
    w2, b2 = (1 + 0.3 * rand(width)).to(small), (0.3 * rand(width)).to(small)
    eps = 1e-2
    want = P.layer_norm(x.double(), w.double(), b.double(), eps)
    out = torch.empty(rows, width, device="cuda")
    ops.layernorm(x.cuda(), w.cuda(), b.cuda(), eps, out)
    assert torch.allclose(out.cpu().double(), want, atol=2e-5)
    picked = torch.tensor([8, 0, 3], dtype=torch.int32)
    out = torch.empty(3, width, dtype=torch.bfloat16, device="cuda")
    ops.layernorm(x.cuda(), w.cuda(), b.cuda(), eps, out, rows=picked.cuda())
    assert torch.allclose(out.cpu().double(), want[picked.long()], atol=3e-2)
    # behind a sublayer: x += 0.7 * norm(y + pre), and the next norm of the new x
    new_x = x.double() + 0.7 * P.layer_norm(y.double() + pre.double(), w.double(), b.double(), eps)
    got_x, then = x.clone().cuda(), torch.empty(rows, width, device="cuda")
    ops.add_layernormed(got_x, y.cuda(), w.cuda(), b.cuda(), eps, 0.7, pre_bias=pre.cuda(), then=(w2.cuda(), b2.cuda(), 1e-6), then_out=then)
    assert torch.allclose(got_x.cpu().double(), new_x, atol=2e-5)
    assert torch.allclose(then.cpu().double(), P.layer_norm(new_x, w2.double(), b2.double(), 1e-6), atol=5e-5)
    alone = x.clone().cuda()
    ops.add_layernormed(alone, y.cuda(), w.cuda(), b.cuda(), eps, 0.7, pre_bias=pre.cuda())
    assert torch.equal(alone, got_x), "the norm that follows changes what is added"
    # an eps that decides the result: rows of equal numbers have no deviation at all
    flat = torch.full((2, width), 5.0)
    out = torch.empty(2, width, device="cuda")
    ops.layernorm(flat.cuda(), w.cuda(), b.cuda(), eps, out)
    assert torch.allclose(out.cpu(), b.float().expand(2, width), atol=1e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_the_norm_that_moves_towards_the_token_before(dtype, ops):
    """Cut every way, between a padding sequence and foreign states that must stay untouched; the state is the normed row."""
    length, width, eps = 150, 72, 1e-5
    generator = torch.Generator().manual_seed(5)
    x = torch.randn(length, width, generator=generator) * 2 + 1
    w, b, mu = 1 + 0.3 * torch.randn(width, generator=generator), 0.3 * torch.randn(width, generator=generator), torch.rand(width, generator=generator)
    h = P.layer_norm(x.double(), w.double(), b.double(), eps)
    want = P.towards_the_token_before(h, mu.double())
    first = None
    for cuts in schedules(length):
        state = torch.full((3, width), 7.0, device="cuda")
        state[1].zero_()
        rows, at = [], 0
        for count in cuts:
            pad = min(2, count)                                    # (a step of one token a sequence keeps its state in the same launch)
            out = torch.empty(pad + count, width, dtype=dtype, device="cuda")
            step = Step([-1, 1], [pad, count], [0, at])
            rows_in = torch.cat([torch.ones(pad, width), x[at:at + count]]).cuda()
            ops.layernorm_shift(rows_in, w.cuda(), b.cuda(), eps, mu.cuda(), state, step, out)
            assert float(out[:pad].abs().max()) == 0.0
            rows.append(out[pad:])
            at += count
        got = torch.cat(rows).double().cpu()
        limit = 1e-5 if dtype == torch.float32 else 2e-2
        assert float((got - want).abs().max()) <= limit * float(want.abs().max()), f"cuts {cuts[:4]}"
        assert float(state[0].min()) == 7.0 and float(state[2].max()) == 7.0, "another sequence's state was touched"
        assert torch.allclose(state[1].cpu().double(), h[-1], atol=1e-5), "the state is the last normed row"
        first = got if first is None else first
        assert torch.equal(got, first), f"cuts {cuts[:4]} change the bits"


def paged_cache(length, n_kv_heads, dim, vdim, dtype, window=None):
    """A cache whose blocks lie in another order than the sequence's, for the sequence in slot 1."""
    from xeno_rt_amd.cache import BLOCK_TOKENS
    from xeno_rt_amd.cache.sequence_cache import KVView
    from xeno_rt_amd.parts.base import KVSpec
    blocks = (length + BLOCK_TOKENS - 1) // BLOCK_TOKENS
    table = torch.full((2, blocks), -1, dtype=torch.int32)
    table[1] = torch.arange(blocks - 1, -1, -1, dtype=torch.int32) + 1
    return KVView(KVSpec(n_kv_heads, dim, window, vdim),
                  torch.zeros(blocks + 1, n_kv_heads, BLOCK_TOKENS, dim, dtype=dtype, device="cuda"),
                  torch.zeros(blocks + 1, n_kv_heads, vdim, BLOCK_TOKENS, dtype=dtype, device="cuda"), table.cuda())


def attend(ops, q, k, v, cuts, dtype, n_heads, n_kv_heads, dim, vdim, scale, window=None, sigmoid=None, table=None, complete=None):
    """q, k and v (float32 sums of a projection, as rows [tokens, heads * size]) through the kernel that completes them
    into a paged cache, then the attention kernel, step by step. sigmoid: dict(head_mix, head_bias, gate) for the
    weights that are no softmax; table: biases by distance for the softmax; complete: options of the completion."""
    length = q.shape[0]
    kv = paged_cache(length, n_kv_heads, dim, vdim, dtype, window)
    complete = dict(complete or {})
    values_in, gate = complete.pop("values_in", None), (sigmoid or {}).get("gate")
    rows, at = [], 0
    for count in cuts:
        if count == 0:
            continue
        step = Step([1], [count], [at])
        proj = torch.cat([q[at:at + count], k[at:at + count], v[at:at + count]], dim=1).float().cuda().contiguous()
        q_out = torch.empty(count, n_heads * dim, dtype=dtype, device="cuda")
        ops.qkv_complete(proj, n_heads, n_kv_heads, dim, vdim, step, q_out, kv=kv,
                         values_in=None if values_in is None else values_in[at:at + count].cuda().contiguous(), **complete)
        out = torch.empty(count, n_heads * vdim, dtype=dtype, device="cuda")
        if sigmoid is not None:
            ops.attention_sigmoid(q_out, n_heads, n_kv_heads, dim, vdim, kv, step, out, scale, window=window,
                                  head_mix=None if sigmoid.get("head_mix") is None else sigmoid["head_mix"].cuda(),
                                  head_bias=None if sigmoid.get("head_bias") is None else sigmoid["head_bias"].cuda(),
                                  gate=None if gate is None else gate[at:at + count].cuda().contiguous())
        else:
            ops.attention(q_out, n_heads, n_kv_heads, dim, kv, step, out, scale=scale, window=window, value_dim=vdim,
                          distance_bias=None if table is None else table.cuda(), queries_alone=True)
        rows.append(out)
        at += count
    return torch.cat(rows).double().cpu()


def plain_weights_summed(q, k, v, n_heads, n_kv_heads, dim, vdim, scale, window, head_mix, head_bias, gate):
    """Sigmoid weights: for query i and key j inside the window, w_h = sigmoid(sum_g M[h, g] s_g + b_h); o_h = sum_j w_h v_j."""
    length = q.shape[0]
    q, k, v = q.double().reshape(length, n_heads, dim), k.double().reshape(length, n_kv_heads, dim), v.double().reshape(length, n_kv_heads, vdim)
    share = n_heads // n_kv_heads
    out = torch.zeros(length, n_heads, vdim, dtype=torch.float64)
    for i in range(length):
        lo = max(0, i - window + 1) if window else 0
        s = torch.stack([k[lo:i + 1, head // share] @ q[i, head] for head in range(n_heads)]) * scale
        if head_mix is not None:
            s = head_mix.double() @ s
        if head_bias is not None:
            s = s + head_bias.double()[:, None]
        w = P.sigmoid(s)
        for head in range(n_heads):
            out[i, head] = w[head] @ v[lo:i + 1, head // share]
        if gate is not None:
            out[i] *= P.sigmoid(gate[i].double())[:, None]
    return out.reshape(length, n_heads * vdim)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n_heads,n_kv_heads,dim,vdim,window", [(6, 3, 20, 12, 17), (2, 2, 32, 32, 70), (8, 1, 16, 8, 3), (1, 1, 64, 96, None),
                                                               (12, 2, 48, 20, 64), (3, 1, 7, 130, 129), (5, 5, 136, 9, 65),
                                                               (32, 8, 128, 128, 100)])         # (the last: more LDS than a launch has by default)
def test_attention_with_sigmoid_weights_mixed_heads_and_a_gate(n_heads, n_kv_heads, dim, vdim, window, dtype, ops):
    length = 150
    generator = torch.Generator().manual_seed(dim + vdim)
    rand = lambda *shape: torch.randn(*shape, generator=generator)
    q, k, v = (rand(length, n * size).to(dtype).float() for n, size in ((n_heads, dim), (n_kv_heads, dim), (n_kv_heads, vdim)))
    mix, bias, gate = torch.eye(n_heads) + 0.4 * rand(n_heads, n_heads), rand(n_heads) - 1.0, rand(length, n_heads)
    scale = 0.6 / math.sqrt(dim)
    for options in (dict(head_mix=mix, head_bias=bias, gate=gate), dict(head_bias=bias), dict(head_mix=mix), dict()):
        want = plain_weights_summed(q, k, v, n_heads, n_kv_heads, dim, vdim, scale, window, options.get("head_mix"), options.get("head_bias"), options.get("gate"))
        first = None
        for cuts in schedules(length):
            got = attend(ops, q, k, v, cuts, dtype, n_heads, n_kv_heads, dim, vdim, scale, window=window, sigmoid=options)
            limit = 1e-5 if dtype == torch.float32 else 2e-2
            assert float((got - want).abs().max()) <= limit * float(want.abs().max()), f"{sorted(options)}, cuts {cuts[:4]}"
            first = got if first is None else first
            assert torch.equal(got, first), f"cuts {cuts[:4]} change the bits"


@pytest.mark.parametrize("window", [None, 100])
def test_a_step_of_many_tokens_and_steps_of_few_give_the_same_bits(window, ops):
    """A step of few tokens is shared out among more workgroups than one of many: the blocks' parts are added in the same order."""
    n_heads, n_kv_heads, dim, vdim, length = 6, 2, 16, 24, 330
    generator = torch.Generator().manual_seed(11)
    q, k, v = (torch.randn(length, n * size, generator=generator) for n, size in ((n_heads, dim), (n_kv_heads, dim), (n_kv_heads, vdim)))
    options = dict(head_mix=torch.eye(n_heads) + 0.2 * torch.randn(n_heads, n_heads, generator=generator), head_bias=torch.full((n_heads,), -2.0))
    want = plain_weights_summed(q, k, v, n_heads, n_kv_heads, dim, vdim, 0.2, window, options["head_mix"], options["head_bias"], None)
    whole = attend(ops, q, k, v, [length], torch.float32, n_heads, n_kv_heads, dim, vdim, 0.2, window=window, sigmoid=options)
    assert float((whole - want).abs().max()) <= 1e-5 * float(want.abs().max())
    for cuts in ([300, 30], [64] * 5 + [10], [290] + [1] * 40):
        assert torch.equal(attend(ops, q, k, v, cuts, torch.float32, n_heads, n_kv_heads, dim, vdim, 0.2, window=window, sigmoid=options), whole), cuts


@pytest.mark.parametrize("window", [1, 3, 17, 64, 70, 129])
def test_a_key_just_inside_the_window_is_seen_and_one_just_outside_is_not(window, ops):
    """One key whose weight is one where all others' are nothing, at the last place the window keeps and at the first it
    drops, for queries in a prompt and decoded, with the key on either side of a cache block's border; with sigmoid
    weights and with a softmax under a table of biases."""
    n_heads, dim, vdim, length = 2, 16, 8, 200
    for query in (window + 1, 130, 199):
        for distance, seen in ((window - 1, True), (window, False)):
            key = query - distance
            if key < 0:
                continue
            q, k = torch.zeros(length, n_heads * dim), torch.zeros(length, n_heads * dim)
            v = torch.zeros(length, n_heads * vdim)
            q[query], k[key], v[key] = 6.0, 6.0, 1.0                       # score 6 * 6 * 16 * scale = 28.8
            for cuts in ([length], [query, 1, length - query - 1], [query - 1, 2, length - query - 1]):
                # every other key's weight is sigmoid(-20); the marked key's is sigmoid(8.8)
                got = attend(ops, q, k, v, cuts, torch.float32, n_heads, n_heads, dim, vdim, 0.05, window=window,
                             sigmoid=dict(head_bias=torch.full((n_heads,), -20.0)))
                assert abs(float(got[query, 0]) - (1.0 if seen else 0.0)) < 1e-3, f"sigmoid: window {window}, query {query}, key {key}, cuts {cuts}"
                # softmax: if the marked key is not seen the weights are shared evenly by keys whose values are nothing
                got = attend(ops, q, k, v, cuts, torch.float32, n_heads, n_heads, dim, vdim, 0.05, window=window,
                             table=torch.zeros(n_heads, 4))
                assert abs(float(got[query, 0]) - (1.0 if seen else 0.0)) < 1e-3, f"softmax: window {window}, query {query}, key {key}, cuts {cuts}"


def test_a_far_key_is_found_among_hundreds(ops):
    """No window: the first key of 700 is the one that counts, for the last query, in a prompt and decoded."""
    n_heads, dim, vdim, length = 4, 32, 16, 700
    generator = torch.Generator().manual_seed(2)
    q, k, v = (0.1 * torch.randn(length, n * size, generator=generator) for n, size in ((n_heads, dim), (2, dim), (2, vdim)))
    q[-1], k[0] = 3.0, 3.0                                                # score 3 * 3 * 32 * 0.1 = 28.8 against sigmoid(-15) elsewhere
    for cuts in ([length], [length - 33] + [1] * 33):
        got = attend(ops, q, k, v, cuts, torch.float32, n_heads, 2, dim, vdim, 0.1, sigmoid=dict(head_bias=torch.full((n_heads,), -15.0)))
        assert torch.allclose(got[-1].reshape(n_heads, vdim)[3].float(), v[0, vdim:], atol=2e-3)
        got = attend(ops, q, k, v, cuts, torch.float32, n_heads, 2, dim, vdim, 0.1, table=torch.zeros(n_heads, 1))
        assert torch.allclose(got[-1].reshape(n_heads, vdim)[0].float(), v[0, :vdim], atol=2e-3)


@pytest.mark.parametrize("rows,far", [(16, 100), (7, 20), (4, 9), (32, 300), (2, 2)])
def test_biases_by_bucket_of_distance(rows, far, ops):
    """The table by distance that the part makes of the learnt rows against the plain bucket rule, and the attention that
    adds it: with keys that are all alike, the weights are the softmax of the biases alone."""
    from xeno_rt_amd.parts import DistanceBuckets
    from xeno_rt_amd.parts.base import Runtime
    n_heads, dim, vdim, length, window = 3, 8, 6, 140, 90
    generator = torch.Generator().manual_seed(rows)
    learnt = torch.randn(rows, n_heads, generator=generator)
    part = DistanceBuckets("rel", n_heads, rows, far)
    part.bind({"rel": learnt}, Runtime(ops, torch.float32, "cuda:0"))
    table = part.score_bias_table().cpu()
    assert table.shape[0] == n_heads and table.shape[1] <= far + 1
    for n in range(0, 400):
        want = learnt[P.distance_bucket(n, rows, far)]
        assert torch.equal(table[:, min(n, table.shape[1] - 1)], want), f"distance {n}"
    q, k = torch.zeros(length, n_heads * dim), torch.zeros(length, n_heads * dim)
    v = torch.randn(length, n_heads * vdim, generator=generator)
    for cuts in ([length], [length - 20] + [1] * 20):
        got = attend(ops, q, k, v, cuts, torch.float32, n_heads, n_heads, dim, vdim, 1.0, window=window, table=table).reshape(length, n_heads, vdim)
        for i in (0, 5, 89, 90, 139):
            lo = max(0, i - window + 1)
            for head in range(n_heads):
                bias = torch.stack([learnt[P.distance_bucket(i - j, rows, far), head] for j in range(lo, i + 1)]).double()
                want = torch.softmax(bias, 0) @ v[lo:i + 1, head * vdim:(head + 1) * vdim].double()
                assert torch.allclose(got[i, head], want, atol=1e-5), f"query {i}, head {head}"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("neighbours", [True, False])
def test_what_completes_q_k_and_v(neighbours, dtype, ops):
    """Biases, head norms, the rotation of a part of a head with stretched frequencies, and the blend with other values: q
    directly, k and v through the attention that reads them from the cache."""
    from xeno_rt_amd.parts import PairRotation
    from xeno_rt_amd.parts.base import Runtime
    n_heads, n_kv_heads, dim, vdim, length, rot = 4, 2, 24, 10, 100, 12
    generator = torch.Generator().manual_seed(7)
    rand = lambda *shape: torch.randn(*shape, generator=generator)
    q, k, v, other = rand(length, n_heads * dim), rand(length, n_kv_heads * dim), rand(length, n_kv_heads * vdim), rand(length, n_kv_heads * vdim)
    b_q, b_k, b_v = rand(n_heads * dim), rand(n_kv_heads * dim), rand(n_kv_heads * vdim)
    g_q, g_k, lam, eps = 1 + 0.3 * rand(dim), 1 + 0.3 * rand(dim), torch.tensor(0.3), 1e-3
    scaling = {"factor": 4.0, "original": 32, "fast": 8.0, "slow": 1.0}
    part = PairRotation(rot, 1000.0, neighbours=neighbours, scaling=scaling)
    part.bind({}, Runtime(ops, torch.float32, "cuda:0"))
    freqs, magnitude = P.rotary_frequencies(rot, 1000.0, scaling)
    assert torch.allclose(part.pair_rotation()[0].cpu().double(), freqs, rtol=1e-7) and abs(part.pair_rotation()[3] - magnitude) < 1e-12
    assert magnitude > 1.1 and float(freqs[-1]) < 1000.0 ** (-(rot - 2) / rot) / 3.9, "the slowest wave is stretched by the factor"

    def plain_side(x, bias, gain, heads):
        x = P.rms_norm((x.double() + bias.double()).reshape(length, heads, dim), gain.double(), eps)
        if not neighbours:                                             # pairs (n, n + rot / 2): bring them side by side, turn, and back
            order = [i for n in range(rot // 2) for i in (n, n + rot // 2)] + list(range(rot, dim))
            turned = P.rotate_neighbours(x[:, :, order], list(range(length)), freqs, magnitude)
            back = torch.empty_like(turned)
            back[:, :, order] = turned
            return back
        return P.rotate_neighbours(x, list(range(length)), freqs, magnitude)

    want_q, want_k = plain_side(q, b_q, g_q, n_heads), plain_side(k, b_k, g_k, n_kv_heads)
    want_v = (1 - lam.double()) * (v.double() + b_v.double()) + lam.double() * other.double()
    # q as the kernel writes it
    step = Step([1], [length], [0])
    proj = torch.cat([q, k, v, rand(length, 3)], dim=1).cuda()              # (columns beyond q, k and v are another reader's)
    q_out = torch.empty(length, n_heads * dim, dtype=dtype, device="cuda")
    kept = torch.empty(length, n_kv_heads * vdim, device="cuda")
    options = dict(biases=(b_q.cuda(), b_k.cuda(), b_v.cuda()), norms=(g_q.cuda(), g_k.cuda()), norm_eps=eps,
                   frequencies=part.pair_rotation()[0], rot_dims=rot, neighbours=neighbours, magnitude=part.pair_rotation()[3])
    ops.qkv_complete(proj, n_heads, n_kv_heads, dim, vdim, step, q_out, values_out=kept, **options)
    limit = 1e-5 if dtype == torch.float32 else 1e-2
    assert float((q_out.cpu().double().reshape(want_q.shape) - want_q).abs().max()) <= limit * float(want_q.abs().max())
    assert torch.allclose(kept.cpu().double(), v.double() + b_v.double(), atol=1e-6), "the values as projected, before the blend"
    # k and v through the cache: softmax attention of the completed rows against the plain one on the plain rows
    want = plain_softmax(want_q.reshape(length, -1), want_k.reshape(length, -1), want_v, n_heads, n_kv_heads, dim, vdim, 0.2, 33)
    for cuts in ([length], [1] * length, [67, 2, 31]):
        got = attend(ops, q, k, v, cuts, dtype, n_heads, n_kv_heads, dim, vdim, 0.2, window=33,
                     complete=dict(options, values_in=other, blend=lam.reshape(1).cuda()))
        limit = 2e-5 if dtype == torch.float32 else 3e-2
        assert float((got - want).abs().max()) <= limit * float(want.abs().max()), f"cuts {cuts[:3]}"


def plain_softmax(q, k, v, n_heads, n_kv_heads, dim, vdim, scale, window):
    length = q.shape[0]
    q, k, v = q.double().reshape(length, n_heads, dim), k.double().reshape(length, n_kv_heads, dim), v.double().reshape(length, n_kv_heads, vdim)
    out = torch.zeros(length, n_heads, vdim, dtype=torch.float64)
    for head in range(n_heads):
        group = head // (n_heads // n_kv_heads)
        for i in range(length):
            lo = max(0, i - window + 1) if window else 0
            out[i, head] = torch.softmax((k[lo:i + 1, group] @ q[i, head]) * scale, 0) @ v[lo:i + 1, group]
    return out.reshape(length, n_heads * vdim)


def test_a_share_of_one_takes_the_other_layers_values_whole(ops):
    """With lambda = 1 the attention reads nothing but the other layer's values; with lambda = 0 nothing of them."""
    n_heads, dim, vdim, length = 2, 16, 8, 70
    generator = torch.Generator().manual_seed(4)
    q, k, v, other = (torch.randn(length, n_heads * size, generator=generator) for size in (dim, dim, vdim, vdim))
    for lam, values in ((1.0, other), (0.0, v)):
        want = plain_softmax(q, k, values, n_heads, n_heads, dim, vdim, 0.3, None)
        got = attend(ops, q, k, v, [length - 5] + [1] * 5, torch.float32, n_heads, n_heads, dim, vdim, 0.3,
                     complete=dict(values_in=other, blend=torch.tensor([lam]).cuda()))
        assert torch.allclose(got, want, atol=1e-5)


# ---- through the programs a user runs ----------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", DTYPES)
def test_trace_replay_of_whole_requests_decoded_tails_and_batches(dtype, models, tmp_path):
    """`bin/trace_run` as a program of its own on a folder whose config.json leaves the rows of the bias tables to the
    tensors: each request whole, with its last tokens one by one, and in batches of unequal requests decoded together."""
    from test_trace_run_gpu import collect, replay, trace_batches, trace_tail, trace_whole
    folder, plain, _, _ = models["wide"]
    vocab = CONFIGS["wide"]["vocab"]
    lengths = {"a": 40, "b": 7, "c": 100, "d": 65, "e": 1, "f": 190}
    requests = {n: token_ids(vocab, length, seed=length) for n, length in lengths.items()}
    want = {n: plain.logits(ids) for n, ids in requests.items()}
    whole = trace_whole(requests)
    got_whole = collect(whole, replay(folder, dtype, tmp_path / "whole", whole, 256))
    tail = trace_tail(requests)
    got_tail = collect(tail, replay(folder, dtype, tmp_path / "tail", tail, 256))
    names = list(requests)
    batches = [{n: requests[n] for n in names[:3]}, {n: requests[n] for n in names[3:]}]
    batched = trace_batches(batches, lambda n, ids: max(1, len(ids) - 5 - ord(n) % 3))
    got_batched = collect(batched, replay(folder, dtype, tmp_path / "batched", batched, 512))
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
    want = []
    for prompt in prompts:
        history = list(prompt)
        for _ in range(6):
            history.append(int(plain.logits(history)[-1].argmax()))
        want.append(history[len(prompt):])
    assert [[int(t) for t in line.split()] for line in lines] == want


# ---- configurations drawn at random: other sizes, orders and constants than any above -----------------------------------

def random_configuration(seed):
    import random
    r = random.Random(seed)
    width = r.choice([24, 40, 72, 96, 136])
    shared = r.choice([12, 24, 48, 60])                                  # numbers a token's values have in the layers that share them
    layers = []
    for _ in range(r.randint(2, 5)):
        kind = r.choice(["attention", "attention_2"])
        v_mix = r.random() < 0.7
        if v_mix:
            kv_heads = r.choice([n for n in (1, 2, 3, 4, 6) if shared % n == 0])
            vdim = shared // kv_heads
        else:
            kv_heads, vdim = r.randint(1, 3), r.choice([4, 16, 24, 33, 96])
        mixer = {"heads": kv_heads * r.choice([1, 1, 2, 3, 5]), "kv_heads": kv_heads, "dim": r.choice([6, 16, 20, 32, 64, 72]), "vdim": vdim,
                 "scale": r.choice([0.1, 0.25, 0.5]), "v_mix": v_mix}
        if r.random() < 0.85:
            mixer["mask"] = {"size": r.choice([1, 2, 9, 40, 64, 65, 300])}
        if kind == "attention":
            if r.random() < 0.8:
                dims = r.choice([d for d in (2, 4, 6, 16, 20, 32, 64) if d <= mixer["dim"]])
                mixer["rot"] = {"dims": dims, "base": r.choice([100.0, 10000.0, 1000000.0])}
                if r.random() < 0.6:
                    mixer["rot"]["scaling"] = {"factor": r.choice([2.0, 4.0, 16.0]), "original": r.choice([16, 64, 256]),
                                               "fast": r.choice([8.0, 32.0]), "slow": r.choice([0.5, 1.0, 2.0])}
        else:
            mixer["bias_rows"] = r.choice([2, 5, 8, 16, 33])
            mixer["bias_max"] = r.choice([n for n in (3, 20, 64, 150, 500) if n > mixer["bias_rows"] // 2])
        layers.append({"type": kind, "mixer": mixer, "mlp": r.choice([None, {"kind": "dense", "ff": r.choice([16, 56, 104])}])})
    return {"architecture": "Ledudra", "vocab": r.choice([50, 97, 160]), "width": width, "norm": {"eps": r.choice([1e-6, 1e-5, 1e-3])},
            "residual_mult": r.choice([0.3, 1.0, 2.0]), "layers": layers}


@pytest.mark.parametrize("seed", [1, 2, 3, 4, 5, 6, 7, 8])
def test_configurations_drawn_at_random(seed, tmp_path):
    from xeno_rt_amd.engine import Engine
    raw = random_configuration(seed)
    folder = make_ledudra_folder(raw, tmp_path / "model", seed=seed, std=0.1, keep_rows=seed % 2 == 0)
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


def test_zz_the_largest_errors_seen_are_reported():
    print("largest errors against the plain model (max, rms):", {k: [f"{x:.2e}" for x in v] for k, v in WORST.items()})
