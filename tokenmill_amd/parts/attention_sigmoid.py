"""Attention whose weights are not normalized over the keys.

A visible key j weighs sigmoid(scale * q.k_j + b_h) for query head h (b: one learned number per head), and the
output is the plain sum of the weighted values: there is no softmax, so no key competes with another. Around
that the mixer has what its constructor is given: grouped key/value heads, values of another size than keys, an
RMS norm of every head of q and k (one weight vector shared by the heads) before the position encoding, a
rotation of the first channels of each head, and a mask that lets a token see the keys of its own chunk of
positions only (chunks counted from position 0 of the sequence) and / or of a window.

Keys and values live in the paged cache like any attention's; prompt portions and single tokens go through the
same kernels, which read them in place through the block tables.
"""
from __future__ import annotations

import torch

from tokenmill_amd import profiling
from tokenmill_amd.hip import ops
from tokenmill_amd.parts.base import KVCacheSpec, KVCacheView, Mixer, StepContext, as_tensor
from tokenmill_amd.parts.linear import Linear
from tokenmill_amd.parts.position import RotaryEmbedding
from tokenmill_amd.weights.loader import TensorSpec

MAX_HEAD_DIM = 256


class SigmoidAttention(Mixer):
    SPLIT_KEYS = 256        # keys of a single token that one wavefront sums; more are dealt to several

    def __init__(self, hidden: int, num_heads: int, num_kv_heads: int, head_dim: int, v_head_dim: int, scale: float,
                 rotary: RotaryEmbedding | None = None, qk_norm_eps: float | None = None, head_bias: bool = True,
                 chunk: int | None = None, window: int | None = None,
                 names: tuple[str, str, str, str] = ("q", "k", "v", "o"),
                 extra_names: tuple[str, str, str] = ("q.norm", "k.norm", "pb"),
                 suffixes: tuple[str, str] = ("", ".b")):
        """``qk_norm_eps``: None for no norm of q and k. ``rotary``: None for no rotation; its ``rotary_dim`` may be
        smaller than the head. ``chunk`` / ``window``: None for none. ``extra_names``: the checkpoint's names of the
        two norm weights and the per-head bias, under the mixer's prefix."""
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} query heads do not divide into {num_kv_heads} kv heads")
        if not 0 < head_dim <= MAX_HEAD_DIM or not 0 < v_head_dim <= MAX_HEAD_DIM:
            raise ValueError(f"head sizes {head_dim} / {v_head_dim}: the kernels take up to {MAX_HEAD_DIM}")
        if chunk is not None and chunk < 1 or window is not None and window < 1:
            raise ValueError("a chunk or a window holds at least one position")
        if rotary is not None and rotary.rotary_dim > head_dim:
            raise ValueError(f"{rotary.rotary_dim} rotated channels in a head of {head_dim}")
        self.hidden, self.num_heads, self.num_kv_heads = hidden, num_heads, num_kv_heads
        self.head_dim, self.v_head_dim = head_dim, v_head_dim
        self.scale, self.rotary, self.qk_norm_eps = float(scale), rotary, qk_norm_eps
        self.has_head_bias, self.chunk, self.window = head_bias, chunk, window
        self.q_size, self.k_size, self.v_size = num_heads * head_dim, num_kv_heads * head_dim, num_kv_heads * v_head_dim
        self.qkv = Linear(hidden, [self.q_size, self.k_size, self.v_size], list(names[:3]), bias=False, suffixes=suffixes)
        self.o = Linear(num_heads * v_head_dim, hidden, names[3], bias=False, suffixes=suffixes)
        self.extra_names = extra_names
        self.q_norm: torch.Tensor | None = None
        self.k_norm: torch.Tensor | None = None
        self.head_bias: torch.Tensor | None = None

    def tensor_specs(self, prefix: str):
        specs = {**self.qkv.tensor_specs(prefix), **self.o.tensor_specs(prefix)}
        qn, kn, pb = self.extra_names
        if self.qk_norm_eps is not None:
            specs[prefix + qn] = TensorSpec((self.head_dim,), init="ones")
            specs[prefix + kn] = TensorSpec((self.head_dim,), init="ones")
        if self.has_head_bias:
            specs[prefix + pb] = TensorSpec((self.num_heads,))
        return specs

    def load(self, tensors, prefix: str) -> None:
        self.qkv.load(tensors, prefix)
        self.o.load(tensors, prefix)
        qn, kn, pb = self.extra_names
        # the small vectors that meet 32-bit scores and statistics are kept in 32-bit
        if self.qk_norm_eps is not None:
            self.q_norm = tensors[prefix + qn].float().contiguous()
            self.k_norm = tensors[prefix + kn].float().contiguous()
        if self.has_head_bias:
            self.head_bias = tensors[prefix + pb].float().contiguous()
        if self.rotary is not None:
            self.rotary.load(tensors, prefix)

    def cache_spec(self):
        return KVCacheSpec(self.num_kv_heads, self.head_dim, self.window, v_head_dim=self.v_head_dim, chunk=self.chunk)

    def visible_pairs(self, step: StepContext) -> tuple[int, int]:
        """(keys read, (query, key) pairs) of a step, for a profile's floor."""
        keys = pairs = 0
        for start, n in zip(step.start_positions, step.q_lens):
            first = None
            for p in range(start, start + n):
                lo = p // self.chunk * self.chunk if self.chunk else 0
                if self.window:
                    lo = max(lo, p - self.window + 1)
                pairs += p - lo + 1
                first = lo if first is None else min(first, lo)
            keys += start + n - first
        return keys, pairs

    def cost(self, label: str, step: StepContext | None, rows: int) -> tuple[int, int]:
        if label == "qkv":
            return self.qkv.cost(rows)
        if label == "o_proj":
            return self.o.cost(rows)
        elem = self.qkv.weight.element_size()
        keys, pairs = self.visible_pairs(step)
        moved = keys * (self.k_size + self.v_size) * elem + step.num_tokens * (self.q_size + self.num_heads * self.v_head_dim) * elem
        return moved, 2 * pairs * self.num_heads * (self.head_dim + self.v_head_dim)

    def forward(self, x, step: StepContext, cache: KVCacheView, residual: torch.Tensor | None = None):
        x = as_tensor(x)
        T = x.shape[0]
        H, G, D, Dv = self.num_heads, self.num_kv_heads, self.head_dim, self.v_head_dim
        rot = self.rotary
        if rot is not None and step.max_context_len > rot.max_positions:
            raise ValueError(f"position {step.max_context_len - 1} is beyond the rotary table ({rot.max_positions} positions)")
        with profiling.label("qkv", lambda: self.qkv.cost(T)):
            qkv = self.qkv.forward(x)
            group = step.groups[cache.group]
            write = cache.write
            ops.qk_norm_rope_store(qkv, H, G, D, Dv, self.q_norm, self.k_norm, self.qk_norm_eps or 1.0,
                                   rot.cos if rot is not None else None, rot.sin if rot is not None else None,
                                   step.positions, group.slot_mapping if write else None,
                                   cache.k if write else None, cache.v if write else None)
        out = torch.empty((T, H * Dv), dtype=x.dtype, device=x.device)
        with profiling.label("attention", lambda: self.cost("attention", step, T)):
            self._attend(qkv, out, step, cache, group)
        with profiling.label("o_proj", lambda: self.o.cost(T)):
            return self.o.forward(out)

    def _attend(self, qkv, out, step: StepContext, cache: KVCacheView, group) -> None:
        """Prompt portions on the matrix unit where its kernel takes the sizes, single tokens (the step's last
        ``num_decode`` rows) and everything else through the kernel that takes a token and a head a wavefront."""
        H, G, D, Dv = self.num_heads, self.num_kv_heads, self.head_dim, self.v_head_dim
        T = qkv.shape[0]
        tiles = step.prefill_tiles
        first_single = T - step.num_decode
        if (tiles is not None and tiles.shape[0] and first_single > 0 and qkv.data_ptr() % 16 == 0
                and ops.attn_sigmoid_prefill_takes(qkv.dtype, D, Dv, cache.k.shape[1], qkv.stride(0))):
            ops.attn_sigmoid_prefill(qkv, out, cache.k, cache.v, group.block_tables, tiles, self.head_bias, H, G, D, Dv,
                                     self.scale, self.chunk or 0, self.window or 0)
            if step.num_decode == 0:
                return
            rows = slice(first_single, T)
        else:
            rows = slice(0, T)
        # Single tokens are few and may see many keys: where the model lets a token see more than SPLIT_KEYS of them, its
        # keys are dealt in runs of that many to wavefronts of their own (whether they are is the model's matter, not
        # the step's, so a token's sums have one order whatever it is batched with; a run beyond a token's keys adds zeros)
        split = most = 0
        if rows.start == first_single and step.num_decode > 0:
            bound = min(x for x in (self.chunk, self.window, self.rotary.max_positions if self.rotary is not None else None, 1 << 30)
                        if x is not None)
            if bound > self.SPLIT_KEYS:
                split, most = self.SPLIT_KEYS, max(1, min(bound, step.max_decode_context))
        ops.attn_sigmoid_paged(qkv[rows], out[rows], cache.k, cache.v, group.block_tables, step.seq_of_token[rows],
                               step.positions[rows], self.head_bias, H, G, D, Dv, self.scale, self.chunk or 0, self.window or 0,
                               split_keys=split, most_keys=most)
