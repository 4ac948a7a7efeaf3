"""The Talolorn design on the GPU against the plain implementation: every mechanism alone,
then whole models replayed whole, with a decoded tail, in portions down to two tokens, mixed
in a pool so small that pages and slots are used again, decoded from the first token on, with
the attention sharpened onto far keys and keys at page borders, and generated greedily
through the engine's entry point and scheduler."""

from __future__ import annotations

import pytest
import torch

from tests import helpers
from tests.plain import talolorn_plain as plain
from tests.talolorn_cases import CASES, folder_for

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}

# float32 results are held to float32 tolerances.  The bfloat16 bound is derived: the plain
# implementation run with bfloat16 roundings between its products says what the format costs
# on that request; the engine, which rounds two more intermediates (the absorbed queries and
# the weighted sums of latents), may be off by BF16_SLACK times that.
F32 = dict(atol=2e-5, rtol=2e-5)
BF16_SLACK = 2.0
# A token whose routing is a close call (the last chosen expert's score within this fraction
# of the first one left out) may go to another expert once its input is rounded to bfloat16:
# such tokens are compared in float32 only.
CLOSE_CALL = 0.03


def rnd(*shape, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g) * scale


def settle(acc, pending):
    if pending is not None:
        acc += pending.sum(0)
    return acc


def bind_random(part, dtype, scale=0.1, seed=0):
    """Random tensors for a part (norm weights around one), bound on the GPU; returns them on
    the host, as float32 values the dtype holds, under the part's local names."""
    params = {}
    for i, (name, spec) in enumerate(part.param_specs().items()):
        t = rnd(*spec.shape, seed=seed + i, scale=scale)
        if spec.init == "one_plus_normal":
            t = 1 + t
        params[name] = t.to(dtype)
    part.bind({n: t.to(DEV) for n, t in params.items()}, dtype, DEV)
    return {n: t.float() for n, t in params.items()}


def plain_names(params):
    """The part's local names ('dq.norm.weight') as the plain implementation calls them."""
    return {"p." + n[:-len(".weight")]: t for n, t in params.items()}


def close(got, want, dtype, rounded=None):
    """float32: the tolerance F32.  bfloat16: `rounded` is the plain result with bfloat16
    roundings between the products; its distance from `want` times BF16_SLACK is the bound."""
    if dtype == torch.float32:
        torch.testing.assert_close(got, want, **F32)
        return
    cost = float((rounded - want).abs().max())
    worst = float((got - want).abs().max())
    assert worst <= BF16_SLACK * cost + 1e-3, f"off by {worst:.3e}; bfloat16 costs the plain run {cost:.3e}"


# ------------------------------------------------------------------- mechanisms, one by one


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("sizes", [(72, 6, 16, 8, 24, 40, 48, 8), (100, 1, 12, 6, 10, 20, 36, 4),
                                   (64, 16, 32, 32, 16, 64, 96, 32), (48, 2, 8, 0, 8, 16, 24, 0)],
                         ids=["six-heads", "odd-one-head", "sixteen-heads", "no-rotated-part"])
def test_latent_attention_alone_over_two_portions(dtype, sizes):
    """21 tokens, then 9 more of the same sequence (pages of 16: both portions end inside a
    page), equal the plain mixer over all 30."""
    from mercury_amd.cache import CacheManager
    from mercury_amd.engine.batch import SeqChunk, build_step
    from mercury_amd.parts import LatentAttention, LayerCache, NoPosition, RotaryPosition

    hidden, heads, dim, rot, vdim, q_rank, kv_rank, turned = sizes
    page = 16
    position = RotaryPosition(rot, 700.0, rotary_dim=turned, interleaved=True) if turned else NoPosition()
    part = LatentAttention(hidden, heads, dim, rot, vdim, q_rank, kv_rank, position, eps=1e-5,
                           scale=0.3)
    params = bind_random(part, dtype, scale=0.15, seed=3)
    part.prepare(64, DEV)
    spec = part.cache_spec()
    manager = CacheManager({0: spec}, 8, page, 2)
    cache = LayerCache(torch.zeros(8, 1, page, spec.head_dim, dtype=dtype, device=DEV),
                       torch.zeros(8, 1, spec.v_dim, page, dtype=dtype, device=DEV), 0, page, True)
    x = rnd(30, hidden, seed=30).to(dtype)
    out = []
    for start, count in ((0, 21), (21, 9)):
        if not manager.holds("s"):
            manager.admit("s", [], count)
        manager.grow("s", start, start + count)
        step = build_step([SeqChunk("s", [0] * count, start, [])], manager, 10, 4096, DEV)
        acc = torch.zeros(count, hidden, device=DEV)
        settle(acc, part.forward(x[start:start + count].to(DEV).contiguous(), step, cache, None, acc))
        out.append(acc.cpu())
    m = {"heads": heads, "dim": dim, "rot_dim": rot, "vdim": vdim, "kv_rank": kv_rank, "scale": 0.3,
         "rot": {"base": 700.0, "dims": turned}}
    want = plain.latent_attention(x.float(), plain_names(params), "p.", m, 1e-5)
    rounded = plain.latent_attention(x.float(), plain_names(params), "p.", m, 1e-5, plain.to_bf16)
    close(torch.cat(out), want, dtype, rounded)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("sizes", [(64, 6, 2, 40), (100, 4, 4, 50), (128, 5, 1, 24)],
                         ids=["two-of-six", "all-of-four-odd", "one-of-five"])
def test_routed_experts_alone(dtype, sizes):
    from mercury_amd.parts import RoutedExperts

    hidden, experts, top, ff = sizes
    part = RoutedExperts(hidden, experts, top, ff, scale=1.7, activation="swish_clamp", limit=0.9,
                         alpha=1.702, beta=1.0)
    params = bind_random(part, dtype, scale=0.2, seed=5)
    x = rnd(37, hidden, seed=9).to(dtype)
    acc = rnd(37, hidden, seed=8)
    acc_d = acc.clone().to(DEV)
    settle(acc_d, part.forward(x.to(DEV), None, acc_d))
    ff_cfg = {"router": {"experts": experts, "top": top, "scale": 1.7},
              "expert": {"ff": ff, "limit": 0.9}}
    want = acc + plain.routed_ff(x.float(), plain_names(params), "p.", ff_cfg)
    rounded = acc + plain.routed_ff(x.float(), plain_names(params), "p.", ff_cfg, plain.to_bf16)
    close(acc_d.cpu(), want, dtype, rounded)


def test_routing_kernel_picks_the_largest_scores_in_order():
    from mercury_amd.kernels import lib as _lib

    lib = _lib.load("core")
    experts, top, tokens = 70, 5, 33      # more experts than lanes of a wavefront
    logits = rnd(tokens, experts, seed=2, scale=2.0)
    logits[0, 3] = logits[0, 66] = 9.0    # equal scores: the lower index comes first
    ids = torch.zeros(tokens, top, dtype=torch.int32, device=DEV)
    weights = torch.zeros(tokens, top, device=DEV)
    _lib.check(lib, lib.mk_route_topk(logits.to(DEV).data_ptr(), experts, top, 2.5, 0, ids.data_ptr(),
                                      weights.data_ptr(), tokens,
                                      torch.cuda.current_stream().cuda_stream), "route")
    chosen, want = plain.route(torch.eye(tokens), logits.T.contiguous(), experts, top, 2.5)
    assert ids.cpu().tolist() == chosen.tolist()
    assert ids[0, :2].tolist() == [3, 66]
    torch.testing.assert_close(weights.cpu(), want, atol=1e-6, rtol=1e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows", [5, 70])
def test_clamped_gate_feed_forward_alone(dtype, rows):
    """Few rows (the skinny kernel's epilogue in bfloat16) and many (the tiled kernel's)."""
    from mercury_amd.parts import GatedMLP

    part = GatedMLP(96, 200, activation="swish_clamp", limit=0.8, alpha=1.702, beta=1.0,
                    names={"gate": "gate", "up": "up", "down": "down"})
    params = bind_random(part, dtype, scale=0.2, seed=21)
    x = rnd(rows, 96, seed=7).to(dtype)
    acc = rnd(rows, 96, seed=8)
    acc_d = acc.clone().to(DEV)
    settle(acc_d, part.forward(x.to(DEV), None, acc_d))
    want = acc + plain.dense_ff(x.float(), plain_names(params), "p.", {"limit": 0.8})
    rounded = acc + plain.dense_ff(x.float(), plain_names(params), "p.", {"limit": 0.8}, plain.to_bf16)
    close(acc_d.cpu(), want, dtype, rounded)
    with pytest.raises(ValueError, match="limit"):
        GatedMLP(8, 8, activation="swish_clamp")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("mult", [1.0, 0.6])
@pytest.mark.parametrize("lowered", [True, False], ids=["lowered", "from-python"])
def test_parallel_block_around_the_other_mixer_and_feed_forward(dtype, mult, lowered):
    """The arrangement alone, with the package's ordinary attention and SiLU-gated projection as
    its sublayers: x + m * (mixer(norm(x)) + ff(norm(x))), over two portions.  With a
    feed-forward whose `forward` is its own (so that it cannot hand its work over) the block
    runs from Python, on the same kernels."""
    from mercury_amd.cache import CacheManager
    from mercury_amd.engine.batch import SeqChunk, build_step
    from mercury_amd.parts import (Attention, GatedMLP, LayerCache, ParallelBlock, RMSNorm,
                                   RotaryPosition)
    from tests.plain import qwen2_plain

    class OwnForward(GatedMLP):
        def forward(self, x, step, accum):
            return super().forward(x, step, accum)

    hidden, n_q, n_kv, d, page = 64, 4, 2, 16, 16
    block = ParallelBlock(Attention(hidden, n_q, n_kv, d, RotaryPosition(d, 10000.0), qkv_bias=True),
                          (GatedMLP if lowered else OwnForward)(hidden, 96), RMSNorm(hidden, 1e-6),
                          {"mixer": "attn.", "ffn": "mlp.", "norm": "norm."}, residual_mult=mult)
    assert block.lowerable_with(None) == lowered
    params = bind_random(block, dtype, scale=0.1, seed=50)
    block.prepare(64, DEV)
    manager = CacheManager({0: block.mixer.cache_spec()}, 8, page, 2)
    cache = LayerCache(torch.zeros(8, n_kv, page, d, dtype=dtype, device=DEV),
                       torch.zeros(8, n_kv, d, page, dtype=dtype, device=DEV), 0, page, True)
    x = rnd(30, hidden, seed=31)
    out = []
    for start, count in ((0, 19), (19, 11)):
        if not manager.holds("s"):
            manager.admit("s", [], count)
        manager.grow("s", start, start + count)
        step = build_step([SeqChunk("s", [0] * count, start, [])], manager, 10, 4096, DEV)
        h = x[start:start + count].to(DEV).contiguous()
        settle(h, block.forward(h, step, cache, None, dtype))
        out.append(h.cpu())

    def plain_block(cast_dtype):
        w = {k: v.to(cast_dtype) for k, v in params.items()}
        normed, _ = qwen2_plain.rms_norm(x.to(cast_dtype), w["norm.weight"], 1e-6)
        cos, sin = qwen2_plain.rotary_table(d, range(30), 10000.0)
        cfg = {"num_attention_heads": n_q, "num_key_value_heads": n_kv, "head_dim": d}
        attn = {k[len("attn."):]: v for k, v in w.items() if k.startswith("attn.")}
        mixed = qwen2_plain.attention_layer(normed, attn, "", cfg, cos, sin, None)
        ff = qwen2_plain.gated_mlp(normed, w["mlp.gate_proj.weight"], w["mlp.up_proj.weight"],
                                   w["mlp.down_proj.weight"])
        return x + mult * (mixed.float() + ff.float())

    close(torch.cat(out), plain_block(torch.float32), dtype, plain_block(torch.bfloat16))


# ---------------------------------------------------------------------------- whole models


LENGTHS = {"a": 150, "b": 97, "c": 64, "d": 40, "e": 33, "f": 1}
PORTIONS = [16, 7, 2, 5, 3, 2, 33, 2, 64, 9, 2, 17]


class Case:
    def __init__(self, name, page):
        self.name, self.page = name, page
        self.folder = folder_for(name)
        self.cfg = plain.read_config(self.folder)
        self.weights = plain.read_weights(self.folder)
        self.reqs = {k: helpers.random_tokens(self.cfg["vocab"], n, seed=ord(k))
                     for k, n in LENGTHS.items()}
        self.want, self.clear = {}, {}
        for k, v in self.reqs.items():
            gaps = []
            self.want[k] = plain.forward_logits(self.weights, self.cfg, v, gaps=gaps)
            least = torch.stack(gaps).min(0).values if gaps else torch.full((len(v),), 1.0)
            self.clear[k] = least > CLOSE_CALL
        self.cost = {k: float((plain.forward_logits(self.weights, self.cfg, v, plain.to_bf16)
                               - self.want[k])[self.clear[k]].abs().max())
                     for k, v in self.reqs.items()}

    def session(self, dtype, max_tokens, max_live=4):
        from mercury_amd.engine.replay import ReplaySession

        return ReplaySession(self.folder, dtype, max_tokens, page_size=self.page, max_live=max_live)

    def check(self, got, key, dtype, what, rows=None):
        want = self.want[key] if rows is None else self.want[key][rows]
        if dtype == "bfloat16":
            clear = self.clear[key] if rows is None else self.clear[key][rows]
            assert clear.float().mean() > 0.8
            got, want = got[clear], want[clear]
        check(got, want, dtype, f"{self.name} {what} {key}", self.cost[key])


def check(got, want, dtype, what, bf16_cost):
    assert got.shape == want.shape, f"{what}: {tuple(got.shape)} vs {tuple(want.shape)}"
    assert torch.isfinite(got).all(), f"{what}: non-finite logits"
    diff = (got - want).abs()
    if dtype == "bfloat16":
        bound = torch.full_like(want, BF16_SLACK * bf16_cost)
    else:
        bound = F32["atol"] + F32["rtol"] * want.abs()
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


def test_residual_stream_layer_by_layer():
    """The stream after every layer run (float32), so that a wrong layer names itself: the
    model is cut after each layer by giving the engine a configuration of its first layers."""
    import copy
    import json
    import tempfile
    from pathlib import Path

    from mercury_amd.engine.replay import ReplaySession
    from mercury_amd.weights import save_file

    folder = folder_for("small")
    cfg = plain.read_config(folder)
    tokens = helpers.random_tokens(cfg["vocab"], 23, seed=4)
    stored = plain.read_weights(folder, torch.bfloat16)
    for depth in range(1, len(cfg["layers"]) + 1):
        cut = copy.deepcopy(cfg)
        cut["layers"] = cut["layers"][:depth]
        # with an identity head over a unit norm weight the logits are the normed stream
        cut["vocab"] = cfg["width"]
        part = {k: v for k, v in stored.items()
                if k == "embed" or any(k.startswith(f"l{i}.") for i in range(depth))}
        part["embed"] = stored["embed"][:cfg["width"]].contiguous()
        part["final.norm"] = torch.ones(cfg["width"], dtype=torch.bfloat16)
        part["head"] = torch.eye(cfg["width"], dtype=torch.bfloat16)
        where = Path(tempfile.mkdtemp(prefix="mercury_talolorn_cut_"))
        (where / "config.json").write_text(json.dumps(cut))
        save_file(part, where / "model.safetensors", metadata={"format": "pt"})
        small_tokens = [t % cfg["width"] for t in tokens]
        want = plain.forward_logits(plain.read_weights(where), cut, small_tokens)
        got = ReplaySession(where, "float32", 64).step([entry("r", small_tokens)], ["r"])
        torch.testing.assert_close(got, want, atol=2e-5, rtol=2e-5, msg=f"after layer {depth - 1}")


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
    """Every token a step of its own, from position 0 (the first tokens of a sequence, then a
    long decode across page borders through the captured graphs)."""
    s = model.session(dtype, 192)
    tokens = model.reqs["b"]
    rows = [s.step([entry("b", tokens[i:i + 1])], ["b"] if i == len(tokens) - 1 else [])
            for i in range(len(tokens))]
    model.check(torch.cat(rows), "b", dtype, "decode-from-0")
    assert s.manager.leaked_pages() == 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_unequal_requests_mixed_in_a_pool_that_is_used_again(model, dtype):
    """Up to four live requests, portions of some beside single tokens of others; the pool holds
    one long and a few short requests, so that pages and slots are given back and taken again."""
    unit = max(64, model.page)
    live_cap = 5 * unit
    s = model.session(dtype, live_cap, max_live=4)
    order = ["a", "d", "e", "b", "f", "c", "d", "a"]      # some requests run twice
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
            # the oldest request decodes token by token once it is past its first half
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
    """Queries and keys scaled so that a row's attention sits on a handful of keys, many of them
    hundreds of tokens back: a prompt of 700 whole, then decoded on past page borders, against
    the plain implementation in float64."""
    from mercury_amd.engine.replay import ReplaySession

    folder = folder_for("small", sharpen=4.0)
    cfg = plain.read_config(folder)
    w64, w32 = plain.read_weights(folder, torch.float64), plain.read_weights(folder)
    tokens = helpers.random_tokens(cfg["vocab"], 740, seed=77)
    want = plain.forward_logits(w64, cfg, tokens).float()
    f32 = plain.forward_logits(w32, cfg, tokens)
    # the attention does look far back: moving the first 300 tokens changes late logits
    moved = tokens[:]
    moved[:300] = helpers.random_tokens(cfg["vocab"], 300, seed=78)
    assert (plain.forward_logits(w32, cfg, moved)[-40:] - f32[-40:]).abs().max() > 0.05
    cost = float((plain.forward_logits(w32, cfg, tokens, plain.to_bf16) - want).abs().max())
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


# ------------------------------------------------ generation through the engine's entry point


@pytest.mark.parametrize("name", ["small", "odd"])
def test_greedy_generation_through_the_engine(name):
    from mercury_amd import Engine, EngineConfig, SamplingParams

    folder = folder_for(name)
    cfg, weights = plain.read_config(folder), plain.read_weights(folder)
    prompts = [helpers.random_tokens(cfg["vocab"], n, seed=40 + n) for n in (3, 19, 41)]
    want = [plain.greedy_generate(weights, cfg, p, 12) for p in prompts]
    engine = Engine(EngineConfig(model=str(folder), device=DEV, dtype="float32", num_blocks=24,
                                 block_size=16, max_model_len=128, prefill_budget=16))
    got = engine.generate(prompts, SamplingParams(ignore_eos=True), max_tokens=12)
    assert got == want
    assert engine.leaked_blocks() == 0
    # bfloat16: the tokens are the plain implementation's, or so close to its choice that the
    # format's own error can have swapped them
    engine = Engine(EngineConfig(model=str(folder), device=DEV, dtype="bfloat16", num_blocks=24,
                                 block_size=16, max_model_len=128))
    out = engine.generate(prompts, SamplingParams(ignore_eos=True), max_tokens=12)
    for prompt, tokens in zip(prompts, out):
        logits = plain.forward_logits(weights, cfg, prompt + tokens)
        cost = float((plain.forward_logits(weights, cfg, prompt + tokens, plain.to_bf16) - logits).abs().max())
        for i, token in enumerate(tokens):
            row = logits[len(prompt) - 1 + i]
            assert row.max() - row[token] <= 2 * BF16_SLACK * cost, f"token {i} of {tokens}"


def test_command_line_and_sampling(tmp_path):
    """`random-weights` and `generate` on the command line for this architecture, and sampled
    tokens (temperature, nucleus) that do not depend on what else is in the batch."""
    import json
    import subprocess
    import sys

    from mercury_amd import Engine, EngineConfig, SamplingParams
    from tests.talolorn_cases import SMALL

    config = tmp_path / "config.json"
    config.write_text(json.dumps(SMALL))
    out = subprocess.run([sys.executable, "-m", "mercury_amd", "random-weights", "--config",
                          str(config), "--out", str(tmp_path / "m"), "--seed", "5", "--std", "0.08"],
                         capture_output=True, text=True, cwd=helpers.ROOT)
    assert out.returncode == 0, out.stderr
    prompt = [(i * 7) % 300 for i in range(20)]
    run = subprocess.run([sys.executable, "-m", "mercury_amd", "generate", "--model",
                          str(tmp_path / "m"), "--prompt-ids", ",".join(map(str, prompt)),
                          "--prompt-ids", "1 2 3", "--max-tokens", "5", "--dtype", "float32",
                          "--num-blocks", "32", "--max-model-len", "256", "--ignore-eos"],
                         capture_output=True, text=True, cwd=helpers.ROOT)
    assert run.returncode == 0, run.stderr
    lines = [json.loads(line) for line in run.stdout.strip().splitlines()]
    cfg, weights = plain.read_config(tmp_path / "m"), plain.read_weights(tmp_path / "m")
    assert lines[0] == {"prompt_index": 0, "tokens": plain.greedy_generate(weights, cfg, prompt, 5)}
    assert lines[1]["tokens"] == plain.greedy_generate(weights, cfg, [1, 2, 3], 5)

    # a request's random numbers are keyed by the engine's seed, its id and the token's index:
    # the first request of two engines with one seed draws the same tokens alone and in a batch
    def fresh():
        return Engine(EngineConfig(model=str(tmp_path / "m"), device=DEV, dtype="float32",
                                   num_blocks=32, block_size=16, max_model_len=128, seed=9))

    params = SamplingParams(temperature=0.9, top_p=0.8, ignore_eos=True)
    others = [helpers.random_tokens(300, n, seed=n) for n in (7, 30)]
    engine = fresh()
    together = engine.generate([prompt] + others, params, max_tokens=10)
    alone = fresh().generate([prompt], params, max_tokens=10)
    assert together[0] == alone[0]
    assert len(set(together[0])) > 1 and engine.leaked_blocks() == 0


SHAPES = [(64, 32, 24, 16), (64, 64, 48, 16), (96, 64, 56, 16), (128, 64, 56, 48), (128, 128, 112, 16),
          (160, 128, 120, 16), (192, 128, 120, 48), (256, 256, 240, 16), (320, 256, 248, 16),
          (384, 256, 248, 96), (576, 512, 504, 16), (640, 512, 504, 96)]


@pytest.mark.parametrize("shape", SHAPES, ids=[f"{k}x{v}" for k, v, _, _ in SHAPES])
def test_every_compiled_cache_shape(shape, tmp_path):
    """Latent and rotated widths that fall into each of the shapes the matrix-core attention is
    compiled for, with 5, 20, 33 or 40 heads (tiles of 16 and of 64 rows straddle tokens, or a
    token's heads fill several tiles): a prompt, a portion, decoding."""
    from mercury_amd.engine.replay import ReplaySession
    from mercury_amd.hostcore import core
    from mercury_amd.weights import write_random_model

    key_width, value_width, kv_rank, rot = shape
    assert core.latent_cache_widths(kv_rank + rot, kv_rank) == (key_width, value_width)
    heads = (5, 20, 33, 40)[SHAPES.index(shape) % 4]
    mixer = {"heads": heads, "dim": 16, "rot_dim": rot, "vdim": 24, "q_rank": 40, "kv_rank": kv_rank,
             "scale": 0.2, "rot": {"base": 3000.0, "dims": rot}}
    layer = {"type": "latent_attention", "mixer": mixer, "mlp": {"kind": "dense", "ff": 64, "limit": 1.5}}
    cfg = {"architecture": "Talolorn", "vocab": 257, "width": 64, "embedding": {"scale": 3.0},
           "norm": {"eps": 1e-5}, "residual_mult": 1.3, "layers": [layer, dict(layer, weights_of=0)]}
    folder = write_random_model(tmp_path / "m", cfg, seed=key_width + value_width, std=0.1,
                                dtype=torch.bfloat16)
    weights = plain.read_weights(folder)
    tokens = helpers.random_tokens(257, 150, seed=kv_rank)
    want = plain.forward_logits(weights, cfg, tokens)
    cost = float((plain.forward_logits(weights, cfg, tokens, plain.to_bf16) - want).abs().max())
    for dtype in ("float32", "bfloat16"):
        s = ReplaySession(folder, dtype, 192)
        rows = [s.step([entry("r", tokens[:90])], []), s.step([entry("r", tokens[90:130])], [])]
        for i in range(130, 150):
            rows.append(s.step([entry("r", tokens[i:i + 1])], ["r"] if i == 149 else []))
        check(torch.cat(rows), want, dtype, f"shape {shape} {dtype}", cost)
