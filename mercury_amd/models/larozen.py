"""The Larozen decoder, put together from parts.

Pre-norm layers over the float32 stream, the norms' stored weights lying around zero
(1 + w multiplies).  A layer of type ``attention`` mixes with a grouped-query attention whose
queries and keys turn in interleaved pairs over the first dims of a head, whose scaled score
is bounded by a tanh, and whose values are its keys as projected; a layer of type ``parallel``
with two mixers side by side, a sink attention (norms over the whole q and k projections, a
query temperature that grows with the position, no rotation) and a state-space mixer, each
output RMS-normed over the width before half their sum enters the stream.  The feed-forward
is down(relu(up(x))^2), or absent.  A run of layers may loop: the same tensors several times,
every pass over a cache and state of its own, the stream re-entering each pass through
``loop.in`` applied to [stream ; embedding output].  The head is the embedding.
Tensors are stored without a ``.weight`` suffix and biases as ``.b``: ``embed``, ``loop.in``,
``l<i>.norm1``, ``l<i>.mix.q``, ``l<i>.mix.q.b``, ``l<i>.mix.left.q.norm``,
``l<i>.mix.right.conv.b``, ``l<i>.mlp.up``, ``final.norm``.
"""

from __future__ import annotations

from ..config.model_config import LarozenConfig
from ..config.registry import register_architecture
from ..parts import (Attention, DecoderModel, LayerCall, NoPosition, NormedMixerSum, PreNormBlock,
                     RMSNorm, RotaryPosition, StateSpaceMixer, StreamMix, UnaryMLP)

BLOCK_NAMES = {"mixer": "mix.", "ffn": "mlp.", "norm_mixer": "norm1.", "norm_ffn": "norm2."}
ATTENTION_NAMES = {"q": "q", "k": "k", "v": "v", "o": "o", "q_norm": "q.norm", "k_norm": "k.norm",
                   "sink": "sink"}
STATE_SPACE_NAMES = {"in": "in", "conv": "conv", "dt_bias": "dt_bias", "a_log": "A_log", "d": "D",
                     "norm": "norm", "out": "o"}
SIDE_NAMES = {"a": "left.", "b": "right.", "norm_a": "left.out", "norm_b": "right.out"}
FF_NAMES = {"up": "up", "down": "down"}
# the design's constant: the two mixers of a parallel layer enter with half their sum
SIDE_BY_SIDE_MULT = 0.5


def stored_name(name: str) -> str:
    if name.endswith(".weight"):
        return name[:-len(".weight")]
    if name.endswith(".bias"):
        return name[:-len(".bias")] + ".b"
    return name


def _norm(cfg: LarozenConfig) -> RMSNorm:
    return RMSNorm(cfg.width, cfg.norm_eps, one_plus=True, round_once=True)


@register_architecture("Larozen", LarozenConfig)
def build_larozen(cfg: LarozenConfig) -> DecoderModel:
    positions: dict = {}    # one angle table per (head size, base, turned dims)
    layers = []
    for entry in cfg.layers:
        a = entry.attention
        if entry.kind == "attention":
            key = (a.dim, a.rot_base, a.rot_dims)
            if key not in positions:
                positions[key] = (RotaryPosition(a.dim, a.rot_base, rotary_dim=a.rot_dims,
                                                 interleaved=True) if a.rot_dims else NoPosition())
            mixer = Attention(cfg.width, a.heads, a.kv_heads, a.dim, positions[key], qkv_bias=True,
                              o_bias=False, scale=a.scale, names=ATTENTION_NAMES,
                              score_cap=a.softcap or None, values="keys")
        else:
            s = entry.state_space
            left = Attention(cfg.width, a.heads, a.kv_heads, a.dim, NoPosition(), qkv_bias=True,
                             o_bias=True, scale=a.scale, names=ATTENTION_NAMES, value_dim=a.vdim,
                             qk_norm="whole", norm_eps=cfg.norm_eps,
                             q_temp=(a.q_temp_coef, a.q_temp_every) if a.q_temp_every else None,
                             sinks=True)
            right = StateSpaceMixer(cfg.width, s.heads, s.vdim, s.state, s.groups, s.conv,
                                    norm_groups=s.norm_groups, eps=cfg.norm_eps,
                                    names=STATE_SPACE_NAMES)
            mixer = NormedMixerSum(cfg.width, left, right, SIDE_NAMES, eps=cfg.norm_eps,
                                   mult=SIDE_BY_SIDE_MULT)
        ffn = UnaryMLP(cfg.width, entry.ff, "relu2", names=FF_NAMES) if entry.ff else None
        layers.append(PreNormBlock(mixer, ffn, _norm(cfg), _norm(cfg) if ffn else None, BLOCK_NAMES))
    # every run of a layer has a cache slot and a state of its own
    calls = [LayerCall(i, n, mix=first) for n, (i, first) in enumerate(cfg.order())]
    return DecoderModel(
        vocab_size=cfg.vocab, hidden_size=cfg.width, layers=layers, final_norm=_norm(cfg),
        tied_head=True, calls=calls, layer_prefix="l{}.", embed_name="embed.weight",
        norm_prefix="final.norm.", head_name="head.weight", max_positions=0,
        eos_token_ids=cfg.eos_token_ids, config=cfg,
        stream_mix=StreamMix(cfg.width) if cfg.loops else None, mix_prefix="loop.in.",
        stored_name=stored_name)
