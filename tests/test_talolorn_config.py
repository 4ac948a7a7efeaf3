"""The Talolorn configuration and model description (no GPU): keys, refusals, tensor names,
the execution list of layers that share tensors, and pins of the plain implementation."""

from __future__ import annotations

import copy
import math

import pytest
import torch

from mercury_amd.config import ConfigError
from mercury_amd.config.model_config import TalolornConfig
from mercury_amd.config.registry import build_model, resolve
from tests.plain import talolorn_plain as plain
from tests.talolorn_cases import SMALL, ODD


def test_config_reads_every_size_and_constant():
    cfg, _ = resolve(SMALL)
    assert isinstance(cfg, TalolornConfig)
    assert (cfg.vocab, cfg.width, cfg.embedding_scale, cfg.residual_mult) == (300, 64, 4.0, 0.5)
    m = cfg.layers[0].mixer
    assert (m.heads, m.dim, m.rot_dim, m.vdim, m.q_rank, m.kv_rank) == (3, 16, 8, 24, 40, 48)
    assert (m.scale, m.rot_base, m.rot_dims) == (0.21, 5000.0, 8)
    assert cfg.layers[0].mlp.experts == 0 and cfg.layers[0].mlp.ff == 96
    moe = cfg.layers[1].mlp
    assert (moe.experts, moe.top, moe.router_scale, moe.ff, moe.limit) == (6, 2, 1.5, 40, 1.0)
    assert cfg.layers[2].weights_of == 1 and cfg.layers[3].mlp is None
    assert TalolornConfig.from_dict(cfg.to_dict()) == cfg


def test_config_refuses_what_is_not_implemented():
    bad = copy.deepcopy(SMALL)
    bad["layers"][0]["type"] = "convolution"
    with pytest.raises(ConfigError, match="type"):
        resolve(bad)
    bad = copy.deepcopy(SMALL)
    bad["layers"][0]["mlp"]["kind"] = "maxout"
    with pytest.raises(ConfigError, match="kind"):
        resolve(bad)
    bad = copy.deepcopy(SMALL)
    bad["layers"][2]["weights_of"] = 2          # a layer without tensors of its own
    with pytest.raises(ConfigError, match="weights_of"):
        resolve(bad)
    bad = copy.deepcopy(SMALL)
    bad["layers"][1]["mlp"]["router"]["top"] = 7
    with pytest.raises(ConfigError, match="top"):
        resolve(bad)
    bad = copy.deepcopy(SMALL)
    del bad["layers"][0]["mixer"]["kv_rank"]
    with pytest.raises(ConfigError, match="kv_rank"):
        resolve(bad)
    bad = copy.deepcopy(SMALL)
    bad["layers"][0]["mixer"]["rot"]["dims"] = 10   # more than the rotated part holds
    with pytest.raises(ConfigError, match="rotated"):
        resolve(bad)


def test_model_declares_the_stored_tensor_names():
    model = build_model(SMALL)
    specs = model.param_specs()
    assert specs["embed"].shape == (300, 64) and specs["head"].shape == (300, 64)
    assert specs["final.norm"].shape == (64,) and specs["l0.norm1"].shape == (64,)
    assert specs["l0.mix.dq"].shape == (40, 64) and specs["l0.mix.dq.norm"].shape == (40,)
    assert specs["l0.mix.dkv"].shape == (48 + 8, 64) and specs["l0.mix.dkv.norm"].shape == (48,)
    assert specs["l0.mix.uq"].shape == (3 * 24, 40)
    assert specs["l0.mix.uk"].shape == (3 * 16, 48) and specs["l0.mix.uv"].shape == (3 * 24, 48)
    assert specs["l0.mix.o"].shape == (64, 3 * 24)
    assert specs["l0.mlp.gate"].shape == (96, 64) and specs["l0.mlp.down"].shape == (64, 96)
    assert specs["l1.mlp.router"].shape == (6, 64) and specs["l1.mlp.e5.up"].shape == (40, 64)
    # layers 2 (shares layer 1's) and 3's absent feed-forward own nothing
    assert not any(n.startswith("l2.") for n in specs)
    assert not any(n.startswith("l3.mlp") for n in specs) and "l3.mix.o" in specs
    # the execution list runs layer 1's tensors twice, each time over a cache of its own
    assert [(c.layer, c.cache) for c in model.calls] == [(0, 0), (1, 1), (1, 2), (2, 3)]
    assert len(model.cache_slots) == 4
    spec = model.cache_slots[0]
    assert (spec.kv_heads, spec.head_dim, spec.v_dim) == (1, 64, 64)   # 56 and 48 padded to a compiled shape


def test_odd_sizes_build():
    model = build_model(ODD)
    spec = model.cache_slots[0]
    assert (spec.kv_heads, spec.head_dim, spec.v_dim) == (1, 64, 64)   # 36 + 6 and 36, padded
    assert model.layers[0].mixer.position.rotary_dim == 4


# ---- pins of the plain implementation


def test_plain_attention_without_rotation_is_the_library_attention():
    """With no rotated part turning (dims 0), the mixer is ordinary causal attention over keys
    [W_uk c | r] and values W_uv c: compared with the library's routine, head by head."""
    torch.manual_seed(0)
    T, width = 9, 20
    m = {"heads": 2, "dim": 6, "rot_dim": 4, "vdim": 5, "q_rank": 7, "kv_rank": 8, "scale": 0.3,
         "rot": {"base": 100.0, "dims": 0}}
    shapes = {"dq": (7, width), "dq.norm": (7,), "uq": (2 * 10, 7), "dkv": (12, width),
              "dkv.norm": (8,), "uk": (12, 8), "uv": (10, 8), "o": (width, 10)}
    w = {"p." + k: torch.randn(*s, dtype=torch.float64) for k, s in shapes.items()}
    h = torch.randn(T, width, dtype=torch.float64)
    got = plain.latent_attention(h, w, "p.", m, 1e-6)
    c_q = plain.rms_norm(h @ w["p.dq"].T, w["p.dq.norm"], 1e-6)
    q = (c_q @ w["p.uq"].T).view(T, 2, 10)
    down = h @ w["p.dkv"].T
    c = plain.rms_norm(down[:, :8], w["p.dkv.norm"], 1e-6)
    k = torch.cat([(c @ w["p.uk"].T).view(T, 2, 6), down[:, None, 8:].expand(T, 2, 4)], dim=-1)
    v = (c @ w["p.uv"].T).view(T, 2, 5)
    lib = torch.nn.functional.scaled_dot_product_attention(
        q.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1), is_causal=True, scale=0.3)
    want = lib.transpose(0, 1).reshape(T, 10) @ w["p.o"].T
    torch.testing.assert_close(got, want, atol=2e-5, rtol=2e-5)   # the plain softmax is float32


def test_plain_rotation_pairs_neighbours_and_keeps_scores_relative():
    x = torch.arange(6, dtype=torch.float64).view(1, 6)
    out = plain.rotate_interleaved(x, torch.tensor([3]), 10.0, 4)
    a0, a1 = 3.0, 3.0 * 10.0 ** -0.5
    want = [0 * math.cos(a0) - 1 * math.sin(a0), 1 * math.cos(a0) + 0 * math.sin(a0),
            2 * math.cos(a1) - 3 * math.sin(a1), 3 * math.cos(a1) + 2 * math.sin(a1), 4.0, 5.0]
    torch.testing.assert_close(out[0], torch.tensor(want, dtype=torch.float64), atol=1e-6, rtol=1e-6)
    # a dot product of two turned vectors depends on the distance of their positions only
    torch.manual_seed(1)
    q, k = torch.randn(1, 8, dtype=torch.float64), torch.randn(1, 8, dtype=torch.float64)
    dot = lambda pq, pk: float(plain.rotate_interleaved(q, torch.tensor([pq]), 50.0, 8)[0]
                               @ plain.rotate_interleaved(k, torch.tensor([pk]), 50.0, 8)[0])
    assert abs(dot(7, 3) - dot(104, 100)) < 1e-4


def test_plain_routing_and_activation():
    h = torch.eye(4)
    # token t's logits are column t
    router = torch.tensor([[0.0, 1.0, 3.0, 1.0], [2.0, 1.0, 0.0, 1.0], [1.0, 1.0, 1.0, 5.0]])
    chosen, weights = plain.route(h, router, 3, 2, 2.0)
    scores = torch.softmax(router.T, -1)
    assert chosen[0].tolist() == [1, 2] and chosen[2].tolist() == [0, 2]
    assert chosen[1].tolist() == [0, 1]            # equal scores: the lower index first
    torch.testing.assert_close(weights[0], 2.0 * scores[0, [1, 2]])
    assert float(weights[3].sum()) < 2.0           # not renormalised
    g, u = torch.tensor([-1.0, 0.5, 9.0]), torch.tensor([-7.0, 0.25, 7.0])
    want = [-1.0 / (1 + math.exp(1.702)) * (-2.0 + 1), 0.5 / (1 + math.exp(-0.851)) * 1.25,
            2.0 / (1 + math.exp(-3.404)) * 3.0]
    torch.testing.assert_close(plain.gate_activation(g, u, 2.0), torch.tensor(want))
