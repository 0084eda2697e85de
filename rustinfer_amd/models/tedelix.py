"""Tedelix: a decoder whose layers are listed in config.json, each a parallel block (one norm;
mixer and feed-forward read its output) with one of three mixers: windowed softmax attention with
turned values, lightning attention, or a generalized delta rule.  The feed-forward is
``down(relu(up(x))^2)``; the head shares the embedding table and soft-caps the logits.

Checkpoint names: ``embed``, ``l<i>.norm1``, ``l<i>.mix.*``, ``l<i>.mlp.up|down``, ``final.norm``.
"""
from __future__ import annotations

from ..config.model_config import (GeneralDeltaSpec, LightningSpec, TedelixConfig, WindowAttentionSpec)
from ..config.registry import register_architecture
from ..parts import (DenseMLP, Embedding, GeneralDeltaRule, LMHead, LightningAttention, ParallelBlock, RMSNorm,
                     RotaryEmbedding, WindowAttention)
from .decoder import DecoderModel


DEFAULT_DECAY_RANK = 16     # where neither a checkpoint nor the caller says otherwise (random weights)


def build_tedelix(cfg: TedelixConfig) -> DecoderModel:
    width, eps = cfg.hidden_size, cfg.norm_eps
    rotations = {}

    def rotation(size, base, dims):
        key = (size, base, dims)
        if key not in rotations:
            rotations[key] = RotaryEmbedding(size, base, rot_dim=dims)
        return rotations[key]

    layers = []
    for i, layer in enumerate(cfg.layers):
        m = layer.mixer
        if isinstance(m, WindowAttentionSpec):
            mixer = WindowAttention(width, m.heads, m.kv_heads, m.dim, m.vdim, m.scale, window=m.window,
                                    pos_enc=rotation(m.dim, m.rot_base, m.rot_dims),
                                    value_pos_enc=rotation(m.vdim, m.rot_base, m.vdim))
        elif isinstance(m, LightningSpec):
            mixer = LightningAttention(width, m.heads, m.dim, m.vdim, m.decay, eps)
        elif isinstance(m, GeneralDeltaSpec):
            mixer = GeneralDeltaRule(width, m.heads, m.dim, m.decay_rank or DEFAULT_DECAY_RANK, eps)
        else:
            raise TypeError(f"layer {i}: unknown mixer {m!r}")
        ffn = DenseMLP(width, layer.ff, "relu2") if layer.ff is not None else None
        layers.append(ParallelBlock(width, RMSNorm(width, eps, weight_name=""), mixer, ffn,
                                    names={"norm": "norm1", "mixer": "mix", "ffn": "mlp"}))
    embed = Embedding(cfg.vocab_size, width, weight_name="")
    head = LMHead(cfg.vocab_size, width, tied_to=embed, logit_scale=cfg.logit_scale, softcap=cfg.logit_softcap)
    return DecoderModel(cfg, embed, layers, RMSNorm(width, eps, weight_name=""), head,
                        position_encodings=list(rotations.values()),
                        names={"embed": "embed", "layer": "l{i}", "final_norm": "final.norm", "lm_head": "head"})


register_architecture("Tedelix", TedelixConfig, build_tedelix)
