"""The Larozen design on the GPU against the plain implementation: every mechanism alone,
then whole models replayed whole, with a decoded tail, in portions down to two tokens, mixed
in a pool so small that pages and state slots are used again, decoded from the first token
on, with the attention sharpened onto far keys and keys at page borders, with sinks that
carry most of the weight, and generated greedily through the engine's entry point."""

from __future__ import annotations

import pytest
import torch

from tests import helpers
from tests.larozen_cases import CASES, SMALL, folder_for, write_folder
from tests.plain import larozen_plain as plain

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

# float32 results are held to float32 tolerances.  The bfloat16 bound is derived: the plain
# implementation run with bfloat16 roundings between its products says what the format costs
# on that input; the engine may be off by BF16_SLACK times that.
F32 = dict(atol=2e-5, rtol=2e-5)
BF16_SLACK = 1.5


def rnd(*shape, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g) * scale


def settle(acc, pending):
    if pending is not None:
        acc += pending.sum(0)
    return acc


def bind_random(part, dtype, scale=0.1, seed=0, around_one=()):
    """Random tensors for a part (norm weights around one), bound on the GPU; returns them on
    the host, as float32 values the dtype holds, under the part's local names."""
    params = {}
    for i, (name, spec) in enumerate(part.param_specs().items()):
        t = rnd(*spec.shape, seed=seed + i, scale=scale)
        if spec.init == "one_plus_normal" or name in around_one:
            t = 1 + t
        params[name] = t.to(dtype)
    part.bind({n: t.to(DEV) for n, t in params.items()}, dtype, DEV)
    return {n: t.float() for n, t in params.items()}


def plain_names(params):
    """The part's local names ('q.norm.weight', 'q.bias') as the plain implementation calls
    them ('p.q.norm', 'p.q.b')."""
    out = {}
    for n, t in params.items():
        if n.endswith(".weight"):
            n = n[:-len(".weight")]
        elif n.endswith(".bias"):
            n = n[:-len(".bias")] + ".b"
        out["p." + n] = t
    return out


def close(got, want, dtype, rounded=None):
    if dtype == torch.float32:
        # absolute differences relative to the size of the outputs: a sum of many products of
        # size 20 is not known to 2e-5 in float32, whatever the size of the one entry
        size = max(1.0, float(want.abs().max()))
        torch.testing.assert_close(got, want, atol=F32["atol"] * size, rtol=F32["rtol"])
        return
    cost = float((rounded - want).abs().max())
    worst = float((got - want).abs().max())
    assert worst <= BF16_SLACK * cost + 1e-3, f"off by {worst:.3e}; bfloat16 costs the plain run {cost:.3e}"


NAMES = {"q": "q", "k": "k", "v": "v", "o": "o", "q_norm": "q.norm", "k_norm": "k.norm", "sink": "sink"}
PORTIONS_ALONE = ((0, 21), (21, 2), (23, 9), (32, 1), (33, 1), (34, 6))


def run_mixer_in_portions(part, x, dtype, hidden, pages=8, page=16, portions=PORTIONS_ALONE):
    """The mixer over one sequence cut into PORTIONS_ALONE (pages of 16: portions end inside
    pages, two of them are single tokens), from a cache and a state slot of its own."""
    from mercury_amd.cache import CacheManager
    from mercury_amd.engine.batch import SeqChunk, build_step
    from mercury_amd.parts import LayerCache

    spec, state_spec = part.cache_spec(), part.state_spec()
    part.prepare(pages * page, DEV)
    from mercury_amd.parts import CacheSpec

    # a manager always has a cache group; a mixer without a cache leaves it unused
    manager = CacheManager({0: spec or CacheSpec(1, 8)}, pages, page, 2, state_spec is not None)
    cache = state = None
    if spec:
        cache = LayerCache(torch.zeros(pages, spec.kv_heads, page, spec.head_dim, dtype=dtype, device=DEV),
                           torch.zeros(pages, spec.kv_heads, spec.v_dim, page, dtype=dtype, device=DEV),
                           0, page, True)
    if state_spec:
        # a slot that held something else before: the step that starts a sequence clears it
        state = torch.full((2, *state_spec.shape), 3.0, dtype=state_spec.dtype, device=DEV)
    out = []
    for start, count in portions:
        if not manager.holds("s"):
            manager.admit("s", [], count)
        manager.grow("s", start, start + count)
        step = build_step([SeqChunk("s", [0] * count, start, [])], manager, 10, 4096, DEV)
        if state is not None and step.fresh_slots:
            state[step.fresh_slots] = 0
        acc = torch.zeros(count, hidden, device=DEV)
        settle(acc, part.forward(x[start:start + count].to(DEV).contiguous(), step, cache, state, acc))
        out.append(acc.cpu())
    return torch.cat(out)


# ------------------------------------------------------------------- mechanisms, one by one


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("sizes", [(64, 4, 2, 32, 16, 20.0), (100, 3, 1, 12, 12, 0.0),
                                   (64, 6, 6, 16, 0, 5.0), (128, 8, 2, 64, 32, 30.0),
                                   (64, 20, 1, 32, 16, 8.0)],
                         ids=["partly-turned", "odd-whole-turn-no-cap", "no-turn-own-kv-heads", "sized",
                              "twenty-heads-a-group"])
def test_rotated_attention_whose_values_are_its_keys(dtype, sizes):
    from mercury_amd.parts import Attention, NoPosition, RotaryPosition

    hidden, heads, kv_heads, dim, turned, cap = sizes
    position = RotaryPosition(dim, 700.0, rotary_dim=turned, interleaved=True) if turned else NoPosition()
    part = Attention(hidden, heads, kv_heads, dim, position, qkv_bias=True, scale=0.3, names=NAMES,
                     score_cap=cap or None, values="keys")
    assert "v.weight" not in part.param_specs()
    params = bind_random(part, dtype, scale=0.25, seed=3)
    x = rnd(40, hidden, seed=30).to(dtype)
    got = run_mixer_in_portions(part, x, dtype, hidden)
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "scale": 0.3, "softcap": cap,
         "rot": {"base": 700.0, "dims": turned}}
    at = torch.arange(40)
    want = plain.attention_mixer(x.float(), plain_names(params), "p.", m, at)
    rounded = plain.attention_mixer(x.float(), plain_names(params), "p.", m, at, plain.to_bf16)
    close(got, want, dtype, rounded)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("sizes", [(64, 4, 4, 16, 24, (0.7, 8)), (100, 2, 1, 10, 10, None),
                                   (128, 8, 2, 64, 64, (0.3, 1)), (64, 6, 3, 48, 8, (2.0, 30)),
                                   (64, 36, 2, 32, 32, (0.4, 16))],
                         ids=["wide-values", "odd-no-temperature", "sized-every-1", "narrow-values",
                              "eighteen-heads-a-group"])
def test_sink_attention(dtype, sizes):
    """Norms over the whole q and k, a temperature whose step falls inside the sequence (and
    inside a portion), sinks that take a good part of the weight, biases on all four."""
    from mercury_amd.parts import Attention, NoPosition

    hidden, heads, kv_heads, dim, vdim, temp = sizes
    part = Attention(hidden, heads, kv_heads, dim, NoPosition(), qkv_bias=True, o_bias=True, scale=0.4,
                     names=NAMES, value_dim=vdim, qk_norm="whole", norm_eps=1e-5, q_temp=temp,
                     sinks=True)
    params = bind_random(part, dtype, scale=0.25, seed=5)
    params["sink.weight"] = torch.linspace(-1.0, 3.0, heads).to(dtype).float()
    part.bind({n: t.to(dtype).to(DEV) for n, t in params.items()}, dtype, DEV)
    x = rnd(40, hidden, seed=31).to(dtype)
    got = run_mixer_in_portions(part, x, dtype, hidden)
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": 0.4}
    if temp:
        m["q_temp"] = {"coef": temp[0], "every": temp[1]}
    at = torch.arange(40)
    want = plain.sink_attention(x.float(), plain_names(params), "p.", m, at, 1e-5)
    rounded = plain.sink_attention(x.float(), plain_names(params), "p.", m, at, 1e-5, plain.to_bf16)
    close(got, want, dtype, rounded)
    # the sinks matter: without them the result is another
    m_none = dict(m)
    free = plain.sink_attention(x.float(), {**plain_names(params), "p.sink": torch.full((heads,), -80.0)},
                                "p.", m_none, at, 1e-5)
    assert (free - want).abs().max() > 20 * F32["atol"]


SS_NAMES = {"in": "in", "conv": "conv", "dt_bias": "dt_bias", "a_log": "A_log", "d": "D",
            "norm": "norm", "out": "o"}


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("sizes", [(64, 4, 16, 24, 1, 4, 1), (100, 3, 10, 9, 3, 2, 3),
                                   (128, 4, 64, 128, 2, 4, 4), (64, 2, 40, 130, 1, 3, 2),
                                   (64, 2, 8, 16, 2, 1, 1)],
                         ids=["small", "odd", "sized-two-workgroups-a-head", "wide-state-odd-columns",
                              "no-carried-inputs"])
def test_state_space_mixer_carries_its_state(dtype, sizes):
    """Convolution inputs and recurrent state carried over portions of 21, 2, 9, 1, 1 and 6
    tokens, from a slot that held another request's state."""
    from mercury_amd.parts import StateSpaceMixer

    hidden, heads, vdim, state, groups, conv, parts = sizes
    part = StateSpaceMixer(hidden, heads, vdim, state, groups, conv, norm_groups=parts, eps=1e-5,
                           names=SS_NAMES)
    params = bind_random(part, dtype, scale=0.3, seed=7)
    x = rnd(40, hidden, seed=32).to(dtype)
    got = run_mixer_in_portions(part, x, dtype, hidden)
    m = {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv, "norm_groups": parts}
    want = plain.state_space_mixer(x.float(), plain_names(params), "p.", m, 1e-5)
    rounded = plain.state_space_mixer(x.float(), plain_names(params), "p.", m, 1e-5, plain.to_bf16)
    close(got, want, dtype, rounded)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("sizes", [(64, 4, 16, 24, 2, 4, 1), (128, 2, 64, 128, 1, 3, 2)], ids=["small", "sized"])
def test_long_portions_run_the_recurrence_in_chunks(dtype, sizes):
    """Portions of 300, 1, 129, 128 and 2 tokens: sequences longer than a chunk of the
    recurrence run as chunks side by side, from the state the step before left (a chunk that
    is full to its last token, one of a single token, then direct steps again)."""
    from mercury_amd.parts import StateSpaceMixer

    hidden, heads, vdim, state, groups, conv, parts = sizes
    part = StateSpaceMixer(hidden, heads, vdim, state, groups, conv, norm_groups=parts, eps=1e-5,
                           names=SS_NAMES)
    params = bind_random(part, dtype, scale=0.3, seed=19)
    x = rnd(560, hidden, seed=34).to(dtype)
    portions = ((0, 300), (300, 1), (301, 129), (430, 128), (558, 2))
    got = run_mixer_in_portions(part, x, dtype, hidden, pages=40, portions=portions)
    m = {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv, "norm_groups": parts}
    want = plain.state_space_mixer(x.double(), {k: v.double() for k, v in plain_names(params).items()},
                                   "p.", m, 1e-5).float()
    rounded = plain.state_space_mixer(x.float(), plain_names(params), "p.", m, 1e-5, plain.to_bf16)
    close(got, want, dtype, rounded)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_state_decays_and_is_forgotten_as_the_equations_say(dtype):
    """A long run of one mixer token by token (300 steps): the state neither drifts from the
    plain recurrence nor leaks between two sequences that share the tensor."""
    from mercury_amd.cache import CacheManager
    from mercury_amd.engine.batch import SeqChunk, build_step
    from mercury_amd.parts import StateSpaceMixer

    hidden = 64
    part = StateSpaceMixer(hidden, 4, 16, 24, 2, 3, norm_groups=2, eps=1e-5, names=SS_NAMES)
    params = bind_random(part, dtype, scale=0.3, seed=11)
    xs = {"a": rnd(300, hidden, seed=1).to(dtype), "b": rnd(120, hidden, seed=2).to(dtype)}
    from mercury_amd.parts import CacheSpec

    manager = CacheManager({0: CacheSpec(1, 8)}, 40, 16, 2, True)
    state = torch.zeros((2, *part.state_spec().shape), device=DEV)
    out = {"a": [], "b": []}
    done = {"a": 0, "b": 0}
    while done["a"] < 300:
        chunks = []
        for key in ("a", "b"):
            if done[key] >= len(xs[key]):
                continue
            if not manager.holds(key):
                manager.admit(key, [], 1)
            manager.grow(key, done[key], done[key] + 1)
            chunks.append(SeqChunk(key, [0], done[key], []))
        step = build_step(chunks, manager, 10, 4096, DEV)
        x = torch.stack([xs[c.key][done[c.key]] for c in chunks]).to(DEV)
        acc = torch.zeros(len(chunks), hidden, device=DEV)
        settle(acc, part.forward(x, step, None, state, acc))
        for row, c in enumerate(chunks):
            out[c.key].append(acc[row].cpu())
            done[c.key] += 1
    m = {"heads": 4, "vdim": 16, "state": 24, "groups": 2, "conv": 3, "norm_groups": 2}
    for key in ("a", "b"):
        want = plain.state_space_mixer(xs[key].float(), plain_names(params), "p.", m, 1e-5)
        rounded = plain.state_space_mixer(xs[key].float(), plain_names(params), "p.", m, 1e-5, plain.to_bf16)
        close(torch.stack(out[key]), want, dtype, rounded)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_two_mixers_side_by_side(dtype):
    from mercury_amd.parts import Attention, NoPosition, NormedMixerSum, StateSpaceMixer

    hidden = 64
    left = Attention(hidden, 4, 2, 16, NoPosition(), qkv_bias=True, o_bias=True, scale=0.4,
                     names=NAMES, value_dim=24, qk_norm="whole", norm_eps=1e-5, q_temp=(0.5, 8), sinks=True)
    right = StateSpaceMixer(hidden, 4, 16, 24, 1, 4, norm_groups=1, eps=1e-5, names=SS_NAMES)
    part = NormedMixerSum(hidden, left, right, {"a": "left.", "b": "right.", "norm_a": "left.out",
                                                "norm_b": "right.out"}, eps=1e-5, mult=0.5)
    params = bind_random(part, dtype, scale=0.25, seed=13)
    x = rnd(40, hidden, seed=33).to(dtype)
    got = run_mixer_in_portions(part, x, dtype, hidden)
    m = {"left": {"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 24, "scale": 0.4,
                  "q_temp": {"coef": 0.5, "every": 8}},
         "right": {"heads": 4, "vdim": 16, "state": 24, "groups": 1, "conv": 4, "norm_groups": 1}}
    at = torch.arange(40)
    want = plain.parallel_mixer(x.float(), plain_names(params), "p.", m, at, 1e-5)
    rounded = plain.parallel_mixer(x.float(), plain_names(params), "p.", m, at, 1e-5, plain.to_bf16)
    close(got, want, dtype, rounded)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows", [3, 37, 300])
def test_squared_relu_feed_forward_and_the_one_plus_norm(dtype, rows):
    from mercury_amd.parts import RMSNorm, UnaryMLP

    part = UnaryMLP(72, 136, "relu2", names={"up": "up", "down": "down"})
    params = bind_random(part, dtype, scale=0.2, seed=17)
    x = rnd(rows, 72, seed=9).to(dtype)
    acc = rnd(rows, 72, seed=8)
    acc_d = acc.clone().to(DEV)
    settle(acc_d, part.forward(x.to(DEV), None, acc_d))
    want = acc + plain.squared_relu_ff(x.float(), plain_names(params), "p.")
    rounded = acc + plain.squared_relu_ff(x.float(), plain_names(params), "p.", plain.to_bf16)
    close(acc_d.cpu(), want, dtype, rounded)

    norm = RMSNorm(72, 1e-5, one_plus=True, round_once=True)
    g = (rnd(72, seed=4, scale=0.1)).to(dtype)
    norm.bind({"weight": g.to(DEV)}, dtype, DEV)
    h = rnd(rows, 72, seed=5, scale=3.0)
    got = norm.forward(h.to(DEV), dtype).float().cpu()
    want = plain.norm_one_plus(h, g.float(), 1e-5)
    if dtype == torch.float32:
        torch.testing.assert_close(got, want, atol=1e-5, rtol=1e-5)
    else:       # rounded once: never further than half a step of bfloat16
        assert ((got - want).abs() <= want.abs() * 2.0 ** -8 + 1e-6).all()


# --------------------------------------------------------------------------- whole models

LENGTHS = {"a": 150, "b": 97, "c": 64, "d": 41, "e": 33, "f": 5}
PORTIONS = [16, 7, 2, 5, 3, 2, 33, 2, 64, 9, 2, 17]


class Case:
    def __init__(self, name, page):
        self.name, self.page = name, page
        self.folder = folder_for(name)
        self.cfg = plain.read_config(self.folder)
        self.weights = plain.read_weights(self.folder)
        self.reqs = {k: helpers.random_tokens(self.cfg["vocab"], n, seed=ord(k))
                     for k, n in LENGTHS.items()}
        exact = plain.read_weights(self.folder, torch.float64)
        self.want = {k: plain.forward(self.cfg, exact, v).float() for k, v in self.reqs.items()}
        self.cost = {k: float((plain.forward(self.cfg, self.weights, v, plain.to_bf16)
                               - self.want[k]).abs().max()) for k, v in self.reqs.items()}

    def session(self, dtype, max_tokens, max_live=4):
        from mercury_amd.engine.replay import ReplaySession

        return ReplaySession(self.folder, dtype, max_tokens, page_size=self.page, max_live=max_live)

    def check(self, got, key, dtype, what, rows=None):
        want = self.want[key] if rows is None else self.want[key][rows]
        check(got, want, dtype, f"{self.name} {what} {key}", self.cost[key])


def check(got, want, dtype, what, bf16_cost):
    assert got.shape == want.shape, f"{what}: {tuple(got.shape)} vs {tuple(want.shape)}"
    assert torch.isfinite(got).all(), f"{what}: non-finite logits"
    diff = (got - want).abs()
    if dtype == "bfloat16":
        bound = torch.full_like(want, BF16_SLACK * bf16_cost)
    else:
        # relative to the size of the logits: sums of hundreds of products of that size
        bound = F32["atol"] * max(1.0, float(want.abs().max())) + F32["rtol"] * want.abs()
    bad = (diff > bound).any(-1)
    if bad.any():
        first = int(bad.nonzero()[0])
        raise AssertionError(
            f"{what}: worst difference {diff.max().item():.3e} (bound {bound.max().item():.3e}), "
            f"first wrong token {first} of {got.shape[0]}, {int(bad.sum())} wrong")


MODELS = [("small", 16), ("odd", 16), ("sized", 32)]


@pytest.fixture(scope="module", params=MODELS, ids=[f"{n}-page{p}" for n, p in MODELS])
def model(request):
    return Case(*request.param)


def entry(key, tokens):
    return {"id": key, "tokens": tokens, "want": list(range(len(tokens)))}


def test_model_cut_after_every_layer_run():
    """The model cut after its first 1, 2, ... layers (float32), so that a wrong layer names
    itself; the loop is kept as far as the cut allows."""
    import copy

    from mercury_amd.engine.replay import ReplaySession

    tokens = helpers.random_tokens(SMALL["vocab"], 23, seed=4)
    for depth in range(1, len(SMALL["layers"]) + 1):
        cut = copy.deepcopy(SMALL)
        cut["layers"] = cut["layers"][:depth]
        if depth <= cut["loop"]["start"]:
            del cut["loop"]
        else:
            cut["loop"]["stop"] = min(cut["loop"]["stop"], depth)
        folder = write_folder(cut, seed=21 + depth)
        want = plain.forward(cut, plain.read_weights(folder), tokens)
        got = ReplaySession(folder, "float32", 64).step([entry("r", tokens)], ["r"])
        torch.testing.assert_close(got, want, msg=f"cut after layer {depth - 1}", **F32)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_each_request_alone_and_whole(model, dtype):
    s = model.session(dtype, 192)
    for key, tokens in model.reqs.items():
        got = s.step([entry(key, tokens)], [key])
        model.check(got, key, dtype, "whole")
    assert s.manager.leaked_pages() == 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_prompt_then_the_last_tokens_one_by_one(model, dtype):
    s = model.session(dtype, 192)
    for key in ("a", "d", "e"):
        tokens = model.reqs[key]
        head = len(tokens) - 32
        rows = [s.step([entry(key, tokens[:head])], [])]
        for i in range(head, len(tokens)):
            rows.append(s.step([entry(key, tokens[i:i + 1])], [key] if i == len(tokens) - 1 else []))
        model.check(torch.cat(rows), key, dtype, "tail-decode")
    assert s.manager.leaked_pages() == 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_portions_of_changing_size_down_to_two_tokens(model, dtype):
    s = model.session(dtype, 192)
    for shift, key in enumerate(("a", "b", "c")):
        tokens, done, rows, n = model.reqs[key], 0, [], shift
        while done < len(tokens):
            count = min(PORTIONS[n % len(PORTIONS)], len(tokens) - done)
            n += 1
            last = done + count == len(tokens)
            rows.append(s.step([entry(key, tokens[done:done + count])], [key] if last else []))
            done += count
        model.check(torch.cat(rows), key, dtype, "portions")
    assert s.manager.leaked_pages() == 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decoding_from_the_first_token(model, dtype):
    """Every token a step of its own, from position 0 (the first tokens of a sequence, the
    convolution's zeros before the start, then a long decode across page borders through the
    captured graphs, whose warm-up run must not advance the state)."""
    s = model.session(dtype, 192)
    tokens = model.reqs["a"]
    rows = [s.step([entry("a", tokens[i:i + 1])], ["a"] if i == len(tokens) - 1 else [])
            for i in range(len(tokens))]
    model.check(torch.cat(rows), "a", dtype, "decode-from-0")
    assert s.manager.leaked_pages() == 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_unequal_requests_mixed_in_a_pool_that_is_used_again(model, dtype):
    """Up to four live requests over four state slots, portions of some beside single tokens of
    others; the pool holds one long and a few short requests, so that pages and slots are given
    back and taken again (a slot's old state must not reach the request that takes it)."""
    unit = max(64, model.page)
    live_cap = 5 * unit
    s = model.session(dtype, live_cap, max_live=4)
    order = ["a", "d", "e", "b", "f", "c", "d", "a", "f", "e"]      # some requests run twice
    got = {i: [] for i in range(len(order))}
    done = {i: 0 for i in range(len(order))}
    waiting, live, n = list(range(len(order))), [], 0
    rounded = lambda i: -(-len(model.reqs[order[i]]) // unit) * unit
    while waiting or live:
        while waiting and len(live) < 4 and sum(map(rounded, live)) + rounded(waiting[0]) <= live_cap:
            live.append(waiting.pop(0))
        entries, ends = [], []
        for slot, i in enumerate(list(live)):
            tokens = model.reqs[order[i]]
            left = len(tokens) - done[i]
            # the oldest request decodes token by token once it is past its first half; the
            # newest sits out every third step
            if slot == len(live) - 1 and len(live) > 1 and n % 3 == 2:
                n += 1
                continue
            count = 1 if (slot == 0 and done[i] > len(tokens) // 2) else PORTIONS[n % len(PORTIONS)]
            n += 1
            count = min(count, left)
            entries.append((i, {"id": f"r{i}", "tokens": tokens[done[i]:done[i] + count],
                                "want": list(range(count))}))
            done[i] += count
            if done[i] == len(tokens):
                ends.append(f"r{i}")
                live.remove(i)
        out = s.step([e for _, e in entries], ends)
        at = 0
        for i, e in entries:
            got[i].append(out[at:at + len(e["tokens"])])
            at += len(e["tokens"])
    for i, key in enumerate(order):
        model.check(torch.cat(got[i]), key, dtype, f"mixed (request {i})")
    assert s.manager.leaked_pages() == 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_sharpened_attention_on_far_keys_and_page_borders(dtype):
    """Queries scaled so that a row's attention sits on a handful of keys, many of them
    hundreds of tokens back: a prompt of 700 whole, then decoded on past page borders, against
    the plain implementation in float64."""
    from mercury_amd.engine.replay import ReplaySession

    folder = folder_for("small", sharpen=6.0, sink=-2.0)
    cfg = plain.read_config(folder)
    w64, w32 = plain.read_weights(folder, torch.float64), plain.read_weights(folder)
    tokens = helpers.random_tokens(cfg["vocab"], 740, seed=77)
    want = plain.forward(cfg, w64, tokens).float()
    f32 = plain.forward(cfg, w32, tokens)
    # the model does look far back: moving the first 300 tokens changes late logits
    moved = tokens[:]
    moved[:300] = helpers.random_tokens(cfg["vocab"], 300, seed=78)
    assert (plain.forward(cfg, w32, moved)[-40:] - f32[-40:]).abs().max() > 0.02
    cost = float((plain.forward(cfg, w32, tokens, plain.to_bf16) - want).abs().max())
    s = ReplaySession(folder, dtype, 768, page_size=16)
    rows = [s.step([entry("r", tokens[:700])], [])]
    for i in range(700, 740):
        rows.append(s.step([entry("r", tokens[i:i + 1])], ["r"] if i == 739 else []))
    got = torch.cat(rows)
    if dtype == "float32":
        slack = float((f32 - want).abs().max())      # what float32 costs the plain implementation
        bound = F32["atol"] + F32["rtol"] * want.abs() + 1.5 * slack
        assert ((got - want).abs() <= bound).all(), f"worst {(got - want).abs().max():.3e}, plain's own {slack:.3e}"
    else:
        check(got, want, dtype, "sharpened", cost)
    assert s.manager.leaked_pages() == 0


@pytest.mark.parametrize("sink", [6.0, -30.0])
def test_sinks_that_take_most_of_the_weight_or_none(sink):
    from mercury_amd.engine.replay import ReplaySession

    folder = folder_for("small", sink=sink)
    cfg, w = plain.read_config(folder), plain.read_weights(folder)
    tokens = helpers.random_tokens(cfg["vocab"], 70, seed=5)
    want = plain.forward(cfg, w, tokens)
    s = ReplaySession(folder, "float32", 128)
    got = torch.cat([s.step([entry("r", tokens[:50])], []), s.step([entry("r", tokens[50:])], ["r"])])
    torch.testing.assert_close(got, want, **F32)


# ------------------------------------------------ generation through the engine's entry point


@pytest.mark.parametrize("name", ["small", "odd"])
def test_greedy_generation_through_the_engine(name):
    from mercury_amd import Engine, EngineConfig, SamplingParams

    folder = folder_for(name)
    cfg, weights = plain.read_config(folder), plain.read_weights(folder)
    prompts = [helpers.random_tokens(cfg["vocab"], n, seed=40 + n) for n in (3, 19, 41, 7, 26)]

    def greedy(prompt, count):
        tokens = list(prompt)
        for _ in range(count):
            tokens.append(int(plain.forward(cfg, weights, tokens)[-1].argmax()))
        return tokens[len(prompt):]

    want = [greedy(p, 12) for p in prompts]
    # three requests at a time over three state slots, prompts admitted in portions of 16
    engine = Engine(EngineConfig(model=str(folder), device=DEV, dtype="float32", num_blocks=24,
                                 block_size=16, max_model_len=128, prefill_budget=16, max_running=3))
    got = engine.generate(prompts, SamplingParams(ignore_eos=True), max_tokens=12)
    assert got == want
    assert engine.leaked_blocks() == 0
    engine = Engine(EngineConfig(model=str(folder), device=DEV, dtype="bfloat16", num_blocks=24,
                                 block_size=16, max_model_len=128, max_running=3))
    out = engine.generate(prompts, SamplingParams(ignore_eos=True), max_tokens=12)
    for prompt, tokens in zip(prompts, out):
        logits = plain.forward(cfg, weights, prompt + tokens)
        cost = float((plain.forward(cfg, weights, prompt + tokens, plain.to_bf16) - logits).abs().max())
        for i, token in enumerate(tokens):
            row = logits[len(prompt) - 1 + i]
            assert row.max() - row[token] <= 2 * BF16_SLACK * cost, f"token {i} of {tokens}"


def test_command_line_and_trace_replay(tmp_path):
    """`random-weights` and `generate` on the command line for this architecture, and the trace
    runner as a program of its own."""
    import json
    import subprocess
    import sys

    config = tmp_path / "config.json"
    config.write_text(json.dumps(SMALL))
    out = subprocess.run([sys.executable, "-m", "mercury_amd", "random-weights", "--config",
                          str(config), "--out", str(tmp_path / "m"), "--seed", "5", "--std", "0.08"],
                         capture_output=True, text=True, cwd=helpers.ROOT)
    assert out.returncode == 0, out.stderr
    prompt = [(i * 7) % 300 for i in range(20)]
    run = subprocess.run([sys.executable, "-m", "mercury_amd", "generate", "--model",
                          str(tmp_path / "m"), "--prompt-ids", ",".join(map(str, prompt)),
                          "--max-tokens", "5", "--dtype", "float32", "--num-blocks", "32",
                          "--max-model-len", "256", "--ignore-eos"],
                         capture_output=True, text=True, cwd=helpers.ROOT)
    assert run.returncode == 0, run.stderr
    cfg, weights = plain.read_config(tmp_path / "m"), plain.read_weights(tmp_path / "m")
    tokens = list(prompt)
    for _ in range(5):
        tokens.append(int(plain.forward(cfg, weights, tokens)[-1].argmax()))
    assert json.loads(run.stdout.strip().splitlines()[0])["tokens"] == tokens[20:]

    steps = [{"step": 0, "entries": [{"id": "x", "tokens": prompt[:13], "want": [12]}], "end": []},
             {"step": 1, "entries": [{"id": "x", "tokens": prompt[13:], "want": [0, 6]},
                                     {"id": "y", "tokens": prompt[:4], "want": []}], "end": ["x"]},
             {"step": 2, "entries": [{"id": "y", "tokens": prompt[4:5], "want": [0]}], "end": ["y"]}]
    replay = subprocess.run([sys.executable, str(helpers.ROOT / "bin" / "trace_run"), "--model",
                             str(tmp_path / "m"), "--dtype", "float32", "--out", str(tmp_path / "o"),
                             "--max-tokens", "128"], input="\n".join(map(json.dumps, steps)) + "\n",
                            capture_output=True, text=True, cwd=helpers.ROOT)
    assert replay.returncode == 0, replay.stderr
    assert [l for l in replay.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    import numpy as np

    want = plain.forward(cfg, weights, prompt)
    read = lambda n: torch.from_numpy(np.fromfile(tmp_path / "o" / f"{n}.f32", dtype="<f4").reshape(-1, 300).copy())
    torch.testing.assert_close(read(0), want[12:13], **F32)
    torch.testing.assert_close(read(1), want[[13, 19]], **F32)
    torch.testing.assert_close(read(2), want[4:5], **F32)


# ------------------------------------------------------------------- drawn configurations


def draw_config(seed: int) -> dict:
    """A configuration whose every size, count, constant and the order of its layers are drawn:
    widths that are and are not multiples of 8, one to many heads in one to as many groups,
    head sizes the matrix cores take and others, values narrower and wider than keys, states of
    few to many rows, convolutions over 1 to 5 tokens, loops anywhere or none."""
    import random

    from tests.larozen_cases import attention, layer, side_by_side, sink_attention, state_space

    r = random.Random(seed)
    width = r.choice([48, 50, 64, 72, 75, 100, 128, 136])
    count = r.randint(1, 4)
    layers = []
    for _ in range(count):
        kv = r.choice([1, 2, 3])
        heads = kv * r.choice([1, 2, 4])
        dim = r.choice([8, 12, 16, 32, 64])
        if r.random() < 0.5:
            turned = r.choice([0, 2, dim // 2, dim])
            turned -= turned % 2
            mixer = attention(heads, kv, dim, r.uniform(0.1, 0.5), rot=(r.uniform(50, 20000), turned) if turned else None,
                              softcap=r.choice([None, 2.0, 15.0, 50.0]))
            kind = "attention"
        else:
            vdim = r.choice([dim, 8, 24, 40])
            groups = r.choice([1, 2, 3])
            ss_heads = groups * r.choice([1, 2, 3])
            ss_vdim = r.choice([4, 8, 16, 24, 40])
            parts = r.choice([d for d in (1, 2, 3, 4, 6) if (ss_heads * ss_vdim) % d == 0])
            mixer = side_by_side(
                sink_attention(heads, kv, dim, vdim, r.uniform(0.1, 0.5),
                               q_temp=(r.uniform(0.1, 1.5), r.choice([1, 3, 16, 64])) if r.random() < 0.7 else None),
                state_space(ss_heads, ss_vdim, r.choice([4, 9, 16, 33, 64, 130]), groups, r.randint(1, 5), parts))
            kind = "parallel"
        layers.append(layer(kind, mixer, r.choice([0, 40, 64, 90])))
    cfg = {"architecture": "Larozen", "vocab": r.choice([97, 256, 301]), "width": width,
           "norm": {"eps": r.choice([1e-6, 1e-5, 1e-3])}, "layers": layers}
    if r.random() < 0.7:
        start = r.randint(0, count - 1)
        cfg["loop"] = {"start": start, "stop": r.randint(start + 1, count), "times": r.randint(1, 3)}
    return cfg


def check_positions(got, want, rounded, what):
    """bfloat16 on configurations that may be badly conditioned (one head, a norm over a few
    columns): position by position.  The error of a position is the root mean square over the
    vocabulary of the difference of the logits, their mean taken off; the engine's may be 3
    times what rounding costs the plain implementation at that position (or at the median
    position, where that is more); one position in fifty may be over, none by more than half."""
    assert got.shape == want.shape and torch.isfinite(got).all(), what

    def error(x):
        d = x - want
        return (d - d.mean(-1, keepdim=True)).pow(2).mean(-1).sqrt()

    plain_cost = error(rounded)
    allowed = 3.0 * torch.maximum(plain_cost, plain_cost.median())
    ratio = error(got) / allowed
    over = int((ratio > 1).sum())
    assert ratio.max() <= 1.5 and over <= max(1, got.shape[0] // 50), (
        f"{what}: {over} positions over, the worst {ratio.max():.2f} times its allowance "
        f"(position {int(ratio.argmax())})")
    assert error(got).median() <= 1.5 * plain_cost.median(), f"{what}: the median position"


@pytest.mark.parametrize("seed", range(60))
def test_drawn_configurations(seed):
    """Whole, then a portion that ends inside a page, a portion of two tokens and decoding, in
    both dtypes, for configurations nobody chose."""
    from mercury_amd.engine.replay import ReplaySession

    cfg = draw_config(seed)
    folder = write_folder(cfg, std=0.1, seed=100 + seed)
    tokens = helpers.random_tokens(cfg["vocab"], 171, seed=seed)
    want = plain.forward(cfg, plain.read_weights(folder, torch.float64), tokens).float()
    rounded = plain.forward(cfg, plain.read_weights(folder), tokens, plain.to_bf16)
    for dtype in ("float32", "bfloat16"):
        s = ReplaySession(folder, dtype, 256, max_live=2)
        whole = s.step([entry("w", tokens)], ["w"])
        rows = [s.step([entry("r", tokens[:137])], []), s.step([entry("r", tokens[137:139])], [])]
        for i in range(139, 171):
            rows.append(s.step([entry("r", tokens[i:i + 1])], ["r"] if i == 170 else []))
        for got, how in ((whole, "whole"), (torch.cat(rows), "cut")):
            if dtype == "float32":
                check(got, want, dtype, f"drawn {seed} {how} {cfg}", 0.0)
            else:
                check_positions(got, want, rounded, f"drawn {seed} {how} {cfg}")
        assert s.manager.leaked_pages() == 0


LONG = {
    "architecture": "Larozen", "vocab": 211, "width": 128, "norm": {"eps": 1e-5},
    "layers": [
        {"type": "attention", "mlp": {"kind": "dense", "ff": 128},
         "mixer": {"heads": 6, "kv_heads": 2, "dim": 64, "vdim": 64, "scale": 0.125, "softcap": 12.0,
                   "rot": {"base": 8000.0, "dims": 48}}},
        {"type": "parallel", "mlp": None,
         "mixer": {"left": {"heads": 4, "kv_heads": 4, "dim": 128, "vdim": 128, "scale": 0.09,
                            "q_temp": {"coef": 0.6, "every": 256}},
                   "right": {"heads": 2, "vdim": 32, "state": 16, "groups": 1, "conv": 3, "norm_groups": 1}}},
    ],
    "loop": {"start": 0, "stop": 2, "times": 2},
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_context_where_decoding_splits_the_keys(dtype):
    """Head sizes the matrix cores take, a bound on the score, sinks that matter and queries
    sharpened onto far keys, at 1,300 tokens and beyond: decoding splits every row's keys over
    wavefronts and workgroups (the sink belongs to the first part alone), prompt portions over
    a long prefix too, and the query temperature steps at 255, 511, 767, ... inside them."""
    from mercury_amd.engine.replay import ReplaySession

    folder = write_folder(LONG, std=0.09, seed=31, sharpen=3.0, sink=1.5)
    w64, w32 = plain.read_weights(folder, torch.float64), plain.read_weights(folder)
    tokens = helpers.random_tokens(LONG["vocab"], 1340, seed=9)
    want = plain.forward(LONG, w64, tokens).float()
    f32 = plain.forward(LONG, w32, tokens)
    moved = tokens[:]
    moved[:600] = helpers.random_tokens(LONG["vocab"], 600, seed=10)
    assert (plain.forward(LONG, w32, moved)[-40:] - f32[-40:]).abs().max() > 0.02
    cost = float((plain.forward(LONG, w32, tokens, plain.to_bf16) - want).abs().max())
    slack = float((f32 - want).abs().max())

    def compare(got, rows, what):
        if dtype == "float32":
            bound = F32["atol"] * max(1.0, float(want.abs().max())) + F32["rtol"] * want[rows].abs() + 1.5 * slack
            worst = (got - want[rows]).abs()
            assert (worst <= bound).all(), f"{what}: worst {worst.max():.3e}, plain's own {slack:.3e}"
        else:
            check(got, want[rows], dtype, what, cost)

    s = ReplaySession(folder, dtype, 2 * 1344, page_size=16, max_live=2)
    # whole, then decoded on
    rows = [s.step([entry("r", tokens[:1300])], [])]
    for i in range(1300, 1340):
        rows.append(s.step([entry("r", tokens[i:i + 1])], ["r"] if i == 1339 else []))
    compare(torch.cat(rows), slice(0, 1340), "whole then decoded")
    # portions over a growing prefix beside a decoding neighbour
    s.step([{"id": "n", "tokens": tokens[:1000], "want": []}], [])
    got_p, got_n, at, n_at = [], [], 0, 1000
    for count in (500, 12, 300, 2, 486):
        out = s.step([entry("p", tokens[at:at + count]), entry("n", tokens[n_at:n_at + 1])], [])
        got_p.append(out[:count])
        got_n.append(out[count:])
        at += count
        n_at += 1
    s.step([], ["p", "n"])
    compare(torch.cat(got_p), slice(0, 1300), "portions over a prefix")
    compare(torch.cat(got_n), slice(1000, 1005), "the neighbour's decoded tokens")
    assert s.manager.leaked_pages() == 0


@pytest.mark.parametrize("d", [64, 128])
@pytest.mark.parametrize("cap", [None, 6.0])
def test_bounded_score_and_sinks_in_every_kernel_that_has_them(d, cap):
    """Two prompts of 300 and 150 tokens, 8 heads in 2 groups: the float32-arithmetic kernel
    in both dtypes, the matrix-core kernel of 16-row tiles unsplit and with the keys split in
    3 and in 8 (parts that four wavefronts add up), and the kernel that stages keys through
    LDS with 1, 2 and (heads of 64) 4 key groups, against the formula in float32."""
    from mercury_amd.kernels import ops
    from tests.helpers import context_from_spans

    n_q, n_kv, page, lens = 8, 2, 16, [300, 150]
    sinks = torch.linspace(-2.0, 4.0, n_q)
    scale = d ** -0.5
    q = [rnd(n, n_q, d, seed=50 + i, scale=1.5) for i, n in enumerate(lens)]
    k = [rnd(n, n_kv, d, seed=60 + i, scale=1.5) for i, n in enumerate(lens)]
    v = [rnd(n, n_kv, d, seed=70 + i) for i, n in enumerate(lens)]
    as_bf16 = lambda t: t.to(torch.bfloat16).float()

    def formula(q, k, v):
        kk, vv = k.repeat_interleave(n_q // n_kv, 1), v.repeat_interleave(n_q // n_kv, 1)
        score = torch.einsum("ihd,jhd->hij", q, kk) * scale
        if cap:
            score = cap * torch.tanh(score / cap)
        score = score.masked_fill(~torch.ones(len(q), len(q), dtype=torch.bool).tril(), float("-inf"))
        top = torch.maximum(score.max(-1, keepdim=True).values, sinks[:, None, None])
        e = torch.exp(score - top)
        p = e / (e.sum(-1, keepdim=True) + torch.exp(sinks[:, None, None] - top))
        return torch.einsum("hij,jhd->ihd", p, vv)

    per = -(-max(lens) // page)
    table = torch.stack([torch.arange(s * per, (s + 1) * per, dtype=torch.int32) for s in range(len(lens))])
    step = context_from_spans([(n, 0) for n in lens], DEV)

    def run(dtype, **how):
        cast = (lambda t: t) if dtype == torch.float32 else as_bf16
        k_cache = torch.zeros(len(lens) * per, n_kv, page, d)
        v_cache = torch.zeros_like(k_cache)
        for s, n in enumerate(lens):
            for pos in range(n):
                k_cache[s * per + pos // page, :, pos % page] = k[s][pos]
                v_cache[s * per + pos // page, :, pos % page] = v[s][pos]
        q_flat = torch.cat([x.reshape(len(x), n_q * d) for x in q]).to(dtype).to(DEV)
        got = ops.attention(q_flat, n_q * d, k_cache.to(dtype).to(DEV),
                            v_cache.transpose(2, 3).contiguous().to(dtype).to(DEV), step, table.to(DEV),
                            n_q, n_kv, d, scale, None, score_cap=cap, sinks=sinks.to(DEV), **how)
        want = torch.cat([formula(cast(a), cast(b), cast(c)) for a, b, c in zip(q, k, v)])
        return got.float().cpu().view(-1, n_q, d), want

    got, want = run(torch.float32, kernel="generic")
    torch.testing.assert_close(got, want, atol=2e-5, rtol=2e-5)
    # without the sinks the result is another
    bare = torch.cat([formula(a, b, c) for a, b, c in zip(q, k, v)])
    variants = [dict(kernel="generic"), dict(kernel="mfma", tile_rows=16, staged=False),
                dict(kernel="mfma", tile_rows=16, staged=False, split_override=(3, 0)),
                dict(kernel="mfma", tile_rows=16, staged=False, split_override=(8, 0)),
                dict(kernel="mfma", staged=1), dict(kernel="mfma", staged=2)]
    if d == 64:
        variants.append(dict(kernel="mfma", staged=4))
    for how in variants:
        got, want = run(torch.bfloat16, **how)
        torch.testing.assert_close(got, want, atol=2e-2, rtol=2e-2, msg=lambda m: f"{how}: {m}")
    with pytest.raises(RuntimeError, match="16 rows a wavefront"):
        run(torch.bfloat16, kernel="mfma", tile_rows=32)


def test_preemption_and_sampling_with_per_request_state():
    """A pool so small that requests are preempted and start over (their state slot is given
    back, taken again and cleared): the greedy tokens stay the plain implementation's.  Sampled
    tokens (temperature, nucleus) do not depend on what else is in the batch."""
    from mercury_amd import Engine, EngineConfig, SamplingParams

    folder = folder_for("small")
    cfg, weights = plain.read_config(folder), plain.read_weights(folder)
    prompts = [helpers.random_tokens(cfg["vocab"], 60, seed=70 + i) for i in range(4)]

    def greedy(prompt, count):
        tokens = list(prompt)
        for _ in range(count):
            tokens.append(int(plain.forward(cfg, weights, tokens)[-1].argmax()))
        return tokens[len(prompt):]

    tight = Engine(EngineConfig(model=str(folder), device=DEV, dtype="float32", num_blocks=14,
                                block_size=16, max_model_len=128, max_running=4,
                                debug_invariants=True))
    got = tight.generate(prompts, SamplingParams(ignore_eos=True), max_tokens=24)
    assert tight.sched.stats["preemptions"] > 0
    assert got == [greedy(p, 24) for p in prompts]
    assert tight.leaked_blocks() == 0

    def fresh():
        return Engine(EngineConfig(model=str(folder), device=DEV, dtype="float32", num_blocks=48,
                                   block_size=16, max_model_len=128, seed=9))

    params = SamplingParams(temperature=0.9, top_p=0.8, ignore_eos=True)
    together = fresh().generate(prompts[:3], params, max_tokens=10)
    alone = fresh().generate(prompts[:1], params, max_tokens=10)
    assert together[0] == alone[0] and len(set(together[0])) > 1


def test_state_layout_formula_is_the_kernel_library_s():
    """The part sizes a request's state without the kernel library; the library says the same."""
    from mercury_amd.hostcore import core
    from mercury_amd.kernels import lib
    from mercury_amd.parts import StateSpaceMixer

    lib.load("core")
    for heads, vdim, state in ((4, 16, 24), (3, 10, 9), (16, 64, 128), (2, 40, 130), (1, 33, 256), (5, 8, 4)):
        part = StateSpaceMixer(64, heads, vdim, state, 1, 2)
        assert part.recurrent_floats() == core.ssm_state_floats(heads, vdim, state)


def test_the_benchmark_s_layer_sizes(tmp_path):
    """The model `bench.py --larozen` times at its smaller sizes (2,048 wide, 64 state-space
    heads of 64 columns and 128 rows, four layers, one re-entry; a smaller vocabulary), against
    the plain implementation: whole, and 290 tokens with 40 decoded behind them."""
    import sys

    from mercury_amd.engine.replay import ReplaySession
    from mercury_amd.weights import write_random_model

    sys.path.insert(0, str(helpers.ROOT))
    import bench

    sizes = dict(bench.LAROZEN_SIZES["small"], vocab=2000)
    cfg = bench.larozen_configs(sizes)["larozen"]
    folder = write_random_model(tmp_path / "m", cfg, seed=3, std=0.02, dtype=torch.bfloat16)
    tokens = helpers.random_tokens(cfg["vocab"], 330, seed=1)
    weights = plain.read_weights(folder)
    want = plain.forward(cfg, {k: v.double() for k, v in weights.items()}, tokens).float()
    rounded = plain.forward(cfg, weights, tokens, plain.to_bf16)
    for dtype in ("float32", "bfloat16"):
        s = ReplaySession(folder, dtype, 512, max_live=2)
        whole = s.step([entry("w", tokens)], ["w"])
        rows = [s.step([entry("r", tokens[:290])], [])]
        for i in range(290, 330):
            rows.append(s.step([entry("r", tokens[i:i + 1])], ["r"] if i == 329 else []))
        for got, how in ((whole, "whole"), (torch.cat(rows), "cut")):
            if dtype == "float32":
                check(got, want, dtype, f"benchmark sizes {how}", 0.0)
            else:
                check_positions(got, want, rounded, f"benchmark sizes {how}")
        assert s.manager.leaked_pages() == 0
