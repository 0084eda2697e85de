"""Belorax: a decoder whose layers are listed in config.json.  Each sub-layer reads the residual
stream itself, and what it returns is normed (``1 + w`` weights) and added times ``residual_mult``:
``x <- x + m norm1(mixer(x)); x <- x + m norm2(ff(x))``.  The mixer is softmax attention with normed
queries and keys and a query temperature (a layer may read the keys and values of an earlier one),
attention through a latent vector with a YaRN-stretched interleaved rotation, or retention; the
feed-forward is a gated one or a mixture of experts.  Embedded rows are scaled; the head has its own
matrix.

Checkpoint names: ``embed``, ``l<i>.norm1|norm2``, ``l<i>.mix.*``, ``l<i>.mlp.*``, ``final.norm``, ``head``.
"""
from __future__ import annotations

import torch

from ..config.model_config import BeloraxConfig, LatentAttentionSpec, NormedAttentionSpec, RetentionSpec
from ..config.registry import register_architecture
from ..parts import (Embedding, LMHead, LatentAttention, MoEFeedForward, OutputRMSNorm, PostNormBlock, RMSNorm,
                     Retention, RotaryEmbedding, SwiGLUMLP, WindowAttention)
from .decoder import DecoderModel, LayerCall


def build_belorax(cfg: BeloraxConfig) -> DecoderModel:
    width, eps, mult = cfg.hidden_size, cfg.norm_eps, cfg.residual_mult
    rotations = {}

    def rotation(size, base, dims, scaling=None):
        key = (size, base, dims, scaling)
        if key not in rotations:
            rotations[key] = RotaryEmbedding(size, base, scaling=scaling, rot_dim=dims)
        return rotations[key]

    layers, schedule = [], []
    for i, layer in enumerate(cfg.layers):
        m = layer.mixer
        reads = i                                     # the cache this layer's call uses
        if isinstance(m, NormedAttentionSpec):
            mixer = WindowAttention(width, m.heads, m.kv_heads, m.dim, m.vdim, m.scale, qk_norm_eps=eps,
                                    q_temperature=(m.temp_coef, m.temp_every) if m.temp_every > 0 else None,
                                    own_kv=m.kv_from is None)
            reads = i if m.kv_from is None else m.kv_from
        elif isinstance(m, LatentAttentionSpec):
            mixer = LatentAttention(width, m.heads, m.dim, m.rot_dim, m.vdim, m.kv_rank, m.scale, eps,
                                    pos_enc=rotation(m.rot_dim, m.rot_base, m.rot_dims, m.rot_scaling), interleaved=True)
        elif isinstance(m, RetentionSpec):
            mixer = Retention(width, m.heads, m.dim, m.vdim, m.decay, eps, pos_enc=rotation(m.dim, m.rot_base, m.rot_dims, m.rot_scaling))
        else:
            raise TypeError(f"layer {i}: unknown mixer {m!r}")
        ffn = ffn_norm = None
        if layer.mlp is not None:
            if layer.mlp.kind == "dense":
                ffn = SwiGLUMLP(width, layer.mlp.ff, names={"gate": "gate", "up": "up", "down": "down"}, delta_dtype=torch.float32)
            else:
                ffn = MoEFeedForward(width, layer.mlp.ff, layer.mlp.experts, layer.mlp.top)
            ffn_norm = OutputRMSNorm(width, eps, mult, weight_name="", one_plus=True)
        layers.append(PostNormBlock(width, mixer, OutputRMSNorm(width, eps, mult, weight_name="", one_plus=True), ffn, ffn_norm))
        schedule.append(LayerCall(i, cache=reads, write=reads == i))
    embed = Embedding(cfg.vocab_size, width, weight_name="", scale=cfg.embedding_scale)
    head = LMHead(cfg.vocab_size, width, weight_name="")
    return DecoderModel(cfg, embed, layers, RMSNorm(width, eps, weight_name="", one_plus=True), head,
                        position_encodings=list(rotations.values()), schedule=schedule,
                        names={"embed": "embed", "layer": "l{i}", "final_norm": "final.norm", "lm_head": "head"})


register_architecture("Belorax", BeloraxConfig, build_belorax)
