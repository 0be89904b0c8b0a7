"""The Lusolix decoder assembled from parts.

    x = embed[token] + pos[position]
    every layer:  n = norm1(x);  x += m * mixer(n + conv(n)) * sigmoid(rg1 n + b)
                  n = norm2(x);  x += m * ff(n) * sigmoid(rg2 n + b)                  (only if the layer has a feed-forward)
    logits = embed . final.norm(x)

with every norm a layer norm with weight and bias, m = ``residual_mult``, conv a causal convolution of ``canon.taps``
taps over time on each channel (none when config.json gives no taps). A layer's mixer is attention through a shared
latent inside a sliding window (``latent_attention``); its feed-forward is dense with the PolyNorm activation, or a set
of small SwiGLU experts of which a table row of the token id names the ones a token uses.
Tensor names: ``embed``, ``pos``, ``l<i>.norm1`` (+ ``.b``), ``l<i>.canon1``, ``l<i>.rg1`` (+ ``.b``), ``l<i>.mix.<name>``,
``l<i>.mlp.<name>``, ``final.norm`` (+ ``.b``).
"""
from __future__ import annotations

from tokenmill_amd.config.model_config import LusolixConfig, LusolixLayer
from tokenmill_amd.config.registry import register_architecture
from tokenmill_amd.models.decoder import DecoderModel
from tokenmill_amd.parts import (DenseFeedForward, GatedResidualBlock, LatentAttention, LayerNorm, LearnedPositions, Linear,
                                 OutputHead, RotaryEmbedding, ShortConvolution, TableRoutedExperts, TokenEmbedding)

SUFFIXES = ("", ".b")       # a matrix or a norm's weight is stored under the bare name, its bias under name + ".b"


def _mixer(cfg: LusolixConfig, layer: LusolixLayer, n_pos: int, tables: dict):
    m = layer.mixer
    rot = m.get("rot") or {}
    dims = int(rot.get("dims", 0))
    rotary = None
    if dims:
        key = (int(m["rot_dim"]), float(rot["base"]), dims)
        if key not in tables:           # layers with the same rotation share one table of angles
            tables[key] = RotaryEmbedding(key[0], key[1], n_pos, rotary_dim=dims, interleaved=True)
        rotary = tables[key]
    window = (m.get("mask") or {}).get("size")
    return LatentAttention(cfg.hidden_size, int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"]), int(m["q_rank"]),
                           int(m["kv_rank"]), float(m["scale"]), cfg.norm_eps, rotary=rotary,
                           window=int(window) if window else None, suffixes=SUFFIXES)


def _feed_forward(cfg: LusolixConfig, mlp: dict):
    if mlp["kind"] == "dense":
        return DenseFeedForward(cfg.hidden_size, mlp["ff"], "poly_norm", bias=False, suffixes=SUFFIXES, act_eps=cfg.norm_eps)
    return TableRoutedExperts(cfg.hidden_size, mlp["ff"], mlp["experts"], mlp["top"], cfg.vocab_size)


def build_lusolix(cfg: LusolixConfig, max_positions: int | None = None) -> DecoderModel:
    n_pos = min(max_positions or cfg.max_position_embeddings, cfg.max_position_embeddings)
    hidden = cfg.hidden_size

    def norm():
        return LayerNorm(hidden, cfg.norm_eps, names=SUFFIXES)

    def gate(name):
        return Linear(hidden, hidden, name, bias=True, suffixes=SUFFIXES)

    embedding = TokenEmbedding(cfg.vocab_size, hidden, name="embed",
                               places=LearnedPositions(cfg.max_position_embeddings, hidden, name="pos"))
    tables: dict = {}
    layers = []
    unused: list[str] = []              # what a checkpoint may hold for a sublayer that a layer does not have
    for i, layer in enumerate(cfg.layers):
        conv = ShortConvolution(hidden, cfg.conv_taps, name="canon1") if cfg.conv_taps else None
        mixer = _mixer(cfg, layer, n_pos, tables)
        if layer.mlp is None:
            unused += [f"l{i}.norm2", f"l{i}.norm2.b", f"l{i}.rg2", f"l{i}.rg2.b"]
            layers.append(GatedResidualBlock(norm(), mixer, gate_mixed=gate("rg1"), conv=conv, mult=cfg.residual_mult))
        else:
            layers.append(GatedResidualBlock(norm(), mixer, norm(), _feed_forward(cfg, layer.mlp), gate("rg1"), gate("rg2"), conv,
                                             cfg.residual_mult))
    head = OutputHead(hidden, cfg.vocab_size, tied_to=embedding, name="head", suffixes=SUFFIXES)
    return DecoderModel(cfg, embedding, layers, norm(), head, names=("", "l{i}.", "final.norm", ""), ignorable=tuple(unused))


register_architecture(LusolixConfig.architecture, LusolixConfig.from_dict, build_lusolix, replace=True)
