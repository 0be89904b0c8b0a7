"""A short causal convolution over time, channel by channel, added to its input.

    out_t = h_t + sum_{j < taps} w[:, j] * h_(t - taps + 1 + j)        zeros before a sequence's first token

The last ``taps - 1`` inputs of a request are its state (a ``StateSpec`` slot in the model's storage type), so a
prompt cut anywhere, or a token decoded alone, sees the same rows as the whole prompt would.
"""
from __future__ import annotations

import torch

from tokenmill_amd import profiling
from tokenmill_amd.hip import ops
from tokenmill_amd.parts.base import Part, StateSpec, StepContext
from tokenmill_amd.weights.loader import TensorSpec

MAX_TAPS = 16


class ShortConvolution(Part):
    def __init__(self, width: int, taps: int, name: str = "conv"):
        if not 1 <= taps <= MAX_TAPS:
            raise ValueError(f"a convolution of {taps} taps: the kernel takes 1 to {MAX_TAPS}")
        self.width, self.taps, self.name = width, taps, name
        self.weight: torch.Tensor | None = None

    def tensor_specs(self, prefix: str):
        return {prefix + self.name: TensorSpec((self.width, self.taps))}

    def load(self, tensors, prefix: str) -> None:
        self.weight = tensors[prefix + self.name]

    def state_spec(self) -> StateSpec | None:
        return StateSpec((self.taps - 1, self.width), None) if self.taps > 1 else None

    def cost(self, label, step, rows):
        e = self.weight.element_size()
        return rows * self.width * 2 * e + (step.num_seqs if step is not None else 1) * 2 * (self.taps - 1) * self.width * e, \
            2 * rows * self.width * self.taps

    def forward(self, h: torch.Tensor, step: StepContext, state: torch.Tensor | None) -> torch.Tensor:
        """h [T, width] -> h + conv(h), request by request; ``state`` [slots, taps - 1, width] is read and advanced."""
        out = torch.empty_like(h)
        with profiling.label("conv", lambda: self.cost("conv", step, h.shape[0])):
            return ops.short_conv(h, self.weight, state, step.cu_q_lens, step.state_slots, step.seq_of_token, step.num_seqs, out,
                                  most_rows=step.max_q_len)
