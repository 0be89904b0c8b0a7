"""A feed-forward of many small experts, of which every token uses a few.

    y[t] = sum over the token's experts e of weight(t, e) * W_down[e] (silu(W_gate[e] x[t]) * (W_up[e] x[t]))

``TableRoutedExperts``: there is no router; a table with one row per token id names the token's experts (the entries of
a row differ) and every one of them weighs 1 / (entries of a row). Experts have no biases.

The step's (token, expert) pairs are sorted by expert on the device and every expert multiplies its own rows, in tiles,
from one launch per product; nothing about the routing crosses to the host, so a step of single tokens can be recorded
into a graph like any other.
"""
from __future__ import annotations

import torch

from tokenmill_amd import profiling
from tokenmill_amd.hip import ops
from tokenmill_amd.parts.base import FeedForward, StepContext, as_tensor
from tokenmill_amd.weights.loader import TensorSpec


class TableRoutedExperts(FeedForward):
    def __init__(self, hidden: int, intermediate: int, experts: int, top: int, vocab: int,
                 names: tuple[str, str, str] = ("gate", "up", "down"), expert_prefix: str = "e{e}.", table_name: str = "table",
                 suffix: str = ""):
        if not 0 < top <= experts <= ops.MOE_MAX_EXPERTS:
            raise ValueError(f"{top} of {experts} experts: a token uses at least one and at most all, of up to {ops.MOE_MAX_EXPERTS}")
        self.hidden, self.intermediate, self.experts, self.top, self.vocab = hidden, intermediate, experts, top, vocab
        self.names, self.expert_prefix, self.table_name, self.suffix = names, expert_prefix, table_name, suffix
        self.gate_up: torch.Tensor | None = None       # [E, 2 F, hidden]: an expert's gate rows, then its up rows
        self.down: torch.Tensor | None = None          # [E, hidden, F]
        self.table: torch.Tensor | None = None         # int32 [vocab, top]

    def _name(self, prefix: str, e: int, which: int) -> str:
        return prefix + self.expert_prefix.format(e=e) + self.names[which] + self.suffix

    def tensor_specs(self, prefix: str):
        F, W = self.intermediate, self.hidden
        specs = {prefix + self.table_name: TensorSpec((self.vocab, self.top), kind="int", init=f"distinct_below:{self.experts}")}
        for e in range(self.experts):
            specs[self._name(prefix, e, 0)] = TensorSpec((F, W))
            specs[self._name(prefix, e, 1)] = TensorSpec((F, W))
            specs[self._name(prefix, e, 2)] = TensorSpec((W, F))
        return specs

    def load(self, tensors, prefix: str) -> None:
        E = self.experts
        self.gate_up = torch.stack([torch.cat([tensors[self._name(prefix, e, 0)], tensors[self._name(prefix, e, 1)]]) for e in range(E)]).contiguous()
        self.down = torch.stack([tensors[self._name(prefix, e, 2)] for e in range(E)]).contiguous()
        table = tensors[prefix + self.table_name]
        # an entry outside the experts would send a kernel beyond the matrices: refused here, once
        if table.numel() and (int(table.min()) < 0 or int(table.max()) >= E):
            raise ValueError(f"{prefix}{self.table_name} names an expert outside 0..{E - 1}")
        if self.top > 1:
            rows = table.sort(dim=1).values
            if bool((rows[:, 1:] == rows[:, :-1]).any()):
                raise ValueError(f"{prefix}{self.table_name}: a row names an expert twice")
        self.table = table.to(torch.int32).contiguous()

    def other_matrices(self) -> list[torch.Tensor]:
        """The matrices kept outside ``Linear`` parts (for a count of parameters)."""
        return [self.gate_up, self.down]

    def cost(self, label: str, step: StepContext | None, rows: int) -> tuple[int, int]:
        e = self.gate_up.element_size()
        used = min(self.experts, rows * self.top)               # matrices read at least once each when every pair differs
        moved = used * 3 * self.intermediate * self.hidden * e + rows * self.hidden * 2 * e + rows * self.top * self.intermediate * 2 * e
        return moved, 6 * rows * self.top * self.intermediate * self.hidden

    def forward(self, x, step: StepContext, residual: torch.Tensor | None = None):
        x = as_tensor(x)
        T = x.shape[0]
        out = torch.empty((T, self.hidden), dtype=x.dtype, device=x.device)
        with profiling.label("experts", lambda: self.cost("experts", step, T)):
            mfma = x.dtype == torch.bfloat16 and self.hidden % 8 == 0 and self.intermediate % 8 == 0 and x.stride(0) % 8 == 0
            rows = ops.moe_tile_rows(T * self.top, self.experts, x.dtype) if mfma else ops.MOE_TILE_ROWS
            routed = ops.moe_route(step.token_ids, self.table, self.experts, rows)
            return ops.moe_experts(x, routed, self.gate_up, self.down, self.top, 1.0 / self.top, out)
