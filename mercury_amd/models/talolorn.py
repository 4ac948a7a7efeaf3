"""The Talolorn decoder, put together from parts.

Every layer is a parallel block: one RMS norm, a latent-attention mixer (interleaved rotary
pairs on the rotated part of queries and on the one rotated key part the heads share) and a
feed-forward that both read the norm's output, their sum scaled into the residual stream.  The
feed-forward is a gated one with the clamped activation g' * sigmoid(1.702 g') * (u' + 1),
dense or as routed experts (softmax over all experts, the top scores times a scale, not
renormalised), or absent.  A layer may run another layer's tensors over a cache of its own.
Tensors are stored without a ``.weight`` suffix: ``embed``, ``l<i>.norm1``, ``l<i>.mix.dq``,
``l<i>.mix.dq.norm``, ``l<i>.mlp.gate``, ``l<i>.mlp.e<k>.up``, ``l<i>.mlp.router``,
``final.norm``, ``head``.
"""

from __future__ import annotations

from ..config.model_config import TalolornConfig
from ..config.registry import register_architecture
from ..parts import (DecoderModel, GatedMLP, LatentAttention, LayerCall, NoPosition, ParallelBlock,
                     RMSNorm, RotaryPosition, RoutedExperts, TokenEmbedding)

PART_NAMES = {"mixer": "mix.", "ffn": "mlp.", "norm": "norm1."}
FF_NAMES = {"gate": "gate", "up": "up", "down": "down"}
# constants of the design's gate activation
SWISH_ALPHA = 1.702
UP_SHIFT = 1.0


def stored_name(name: str) -> str:
    return name[:-len(".weight")] if name.endswith(".weight") else name


def _feed_forward(cfg: TalolornConfig, ff):
    if ff is None:
        return None
    act = dict(activation="swish_clamp", limit=ff.limit, alpha=SWISH_ALPHA, beta=UP_SHIFT)
    if not ff.experts:
        return GatedMLP(cfg.width, ff.ff, names=FF_NAMES, **act)
    return RoutedExperts(cfg.width, ff.experts, ff.top, ff.ff, scale=ff.router_scale,
                         renormalize=False, **act)


@register_architecture("Talolorn", TalolornConfig)
def build_talolorn(cfg: TalolornConfig) -> DecoderModel:
    layers, layer_ids, place = [], [], {}
    positions: dict = {}    # one angle table per (width, base, turned dims)
    for i, entry in enumerate(cfg.layers):
        if entry.weights_of is not None:
            continue
        m = entry.mixer
        key = (m.rot_dim, m.rot_base, m.rot_dims)
        if key not in positions:
            positions[key] = (RotaryPosition(m.rot_dim, m.rot_base, rotary_dim=m.rot_dims,
                                             interleaved=True) if m.rot_dims else NoPosition())
        position = positions[key]
        mixer = LatentAttention(cfg.width, m.heads, m.dim, m.rot_dim, m.vdim, m.q_rank, m.kv_rank,
                                position, eps=cfg.norm_eps, scale=m.scale)
        place[i] = len(layers)
        layer_ids.append(i)
        layers.append(ParallelBlock(mixer, _feed_forward(cfg, entry.mlp),
                                    RMSNorm(cfg.width, cfg.norm_eps), PART_NAMES,
                                    residual_mult=cfg.residual_mult))
    calls = [LayerCall(place[i if entry.weights_of is None else entry.weights_of], i)
             for i, entry in enumerate(cfg.layers)]
    return DecoderModel(
        vocab_size=cfg.vocab, hidden_size=cfg.width, layers=layers,
        final_norm=RMSNorm(cfg.width, cfg.norm_eps), tied_head=False, calls=calls,
        layer_prefix="l{}.", embed_name="embed.weight", norm_prefix="final.norm.",
        head_name="head.weight", max_positions=0, eos_token_ids=cfg.eos_token_ids, config=cfg,
        embedding=TokenEmbedding(cfg.vocab, cfg.width, scale=cfg.embedding_scale),
        layer_ids=layer_ids, stored_name=stored_name)
