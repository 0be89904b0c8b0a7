"""The Modinex decoder assembled from parts.

    x = embed[token] + pos[position]
    every layer:  x += norm1b(mixer(norm1(x)));  x += norm2b(ff(norm2(x)))   (the second only if the layer has a feed-forward)
    logits = head(final.norm(x))

with every norm an RMS norm in groups. A layer's mixer is, by its ``type``,
  * ``attention``: grouped key/value heads, values of their own size, q and k normed per head and rotated over
    their first ``rot.dims`` channels, sigmoid weights with a bias per head and no normalization over the keys,
    each token seeing the keys of its own chunk of ``mask.size`` positions;
  * ``gla``: gated linear attention with a matrix of 32-bit state per request and head.
The feed-forward is dense with the tanh form of GELU and biases. Tensor names: ``embed``, ``pos``,
``l<i>.norm1`` ..., ``l<i>.mix.<name>``, ``l<i>.mlp.<name>`` (+ ``.b`` for a bias), ``final.norm``, ``head``.
"""
from __future__ import annotations

from tokenmill_amd.config.model_config import ModinexConfig, ModinexLayer
from tokenmill_amd.config.registry import register_architecture
from tokenmill_amd.models.decoder import DecoderModel
from tokenmill_amd.parts import (DenseFeedForward, GatedLinearAttention, GroupRMSNorm, LearnedPositions, OutputHead,
                                 RotaryEmbedding, SandwichBlock, SigmoidAttention, TokenEmbedding)

SUFFIXES = ("", ".b")       # a matrix is stored under the bare name, its bias under name + ".b"


def _mixer(cfg: ModinexConfig, layer: ModinexLayer, n_pos: int, tables: dict):
    m, hidden = layer.mixer, cfg.hidden_size
    if layer.type == "gla":
        return GatedLinearAttention(hidden, int(m["heads"]), int(m["dim"]), int(m["vdim"]), float(m["tau"]), cfg.norm_eps,
                                    gate_rank=m.get("rank"), suffixes=SUFFIXES)
    rot = m.get("rot") or {}
    dims = int(rot.get("dims", 0))
    rotary = None
    if dims:
        key = (int(m["dim"]), float(rot["base"]), dims)
        if key not in tables:           # layers with the same rotation share one table
            tables[key] = RotaryEmbedding(key[0], key[1], n_pos, rotary_dim=dims)
        rotary = tables[key]
    chunk = (m.get("mask") or {}).get("size")
    return SigmoidAttention(hidden, int(m["heads"]), int(m.get("kv_heads") or m["heads"]), int(m["dim"]), int(m["vdim"]),
                            float(m["scale"]), rotary=rotary, qk_norm_eps=cfg.norm_eps, head_bias=True,
                            chunk=int(chunk) if chunk else None, suffixes=SUFFIXES)


def build_modinex(cfg: ModinexConfig, max_positions: int | None = None) -> DecoderModel:
    n_pos = min(max_positions or cfg.max_position_embeddings, cfg.max_position_embeddings)
    hidden = cfg.hidden_size

    def norm():
        return GroupRMSNorm(hidden, cfg.norm_eps, cfg.norm_groups, name="")

    embedding = TokenEmbedding(cfg.vocab_size, hidden, name="embed",
                               places=LearnedPositions(cfg.max_position_embeddings, hidden, name="pos"))
    tables: dict = {}
    layers = []
    for layer in cfg.layers:
        mixer = _mixer(cfg, layer, n_pos, tables)
        if layer.ff is None:
            layers.append(SandwichBlock(norm(), mixer, norm()))
        else:
            ffn = DenseFeedForward(hidden, layer.ff, "gelu_tanh", bias=True, suffixes=SUFFIXES)
            layers.append(SandwichBlock(norm(), mixer, norm(), norm(), ffn, norm()))
    head = OutputHead(hidden, cfg.vocab_size, tied_to=None, name="head", suffixes=SUFFIXES)
    return DecoderModel(cfg, embedding, layers, norm(), head, names=("", "l{i}.", "final.norm", ""))


register_architecture(ModinexConfig.architecture, ModinexConfig.from_dict, build_modinex, replace=True)
