"""Feed-forward parts."""

from __future__ import annotations

import torch

from tokamak_amd.config.registry import register_part
from tokamak_amd.kernels.linear import gated_linear, linear
from tokamak_amd.kernels.ops import GATE_ACTIVATIONS
from tokamak_amd.parts.base import FeedForward, Fetch
from tokamak_amd.weights.spec import TensorSpec


class SwiGLU(FeedForward):
    """down(silu(gate(x)) * up(x)), no biases
    (reference: src/tokamak/model/layers.py:92-104).

    ``gate_proj`` and ``up_proj`` are held as one [2I, H] matrix so one product
    yields both halves.  ``activation``: what the gate passes through, ``"silu"`` or
    ``"gelu_tanh"`` (0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3)))).
    """

    capturable = True
    fuses_residual = True
    replayable = True

    def __init__(self, *, hidden_size: int, intermediate_size: int, dtype, device,
                 names: tuple[str, str, str] = ("gate_proj.weight", "up_proj.weight", "down_proj.weight"),
                 activation: str = "silu") -> None:
        super().__init__(dtype=dtype, device=device)
        if activation not in GATE_ACTIVATIONS:
            raise ValueError(f"activation is one of {sorted(GATE_ACTIVATIONS)}, got {activation!r}")
        self.activation = activation
        self.hidden_size = int(hidden_size)
        self.intermediate_size = int(intermediate_size)
        self.names = tuple(names)       # gate, up, down behind the part's prefix
        self.gate_up: torch.Tensor | None = None
        self.down: torch.Tensor | None = None

    def expected_tensors(self, prefix: str) -> dict[str, TensorSpec]:
        h, i = self.hidden_size, self.intermediate_size
        gate, up, down = self.names
        return {prefix + gate: TensorSpec((i, h)), prefix + up: TensorSpec((i, h)), prefix + down: TensorSpec((h, i))}

    def bind(self, prefix: str, fetch: Fetch) -> None:
        gate, up, down = self.names
        self.gate_up = torch.cat([fetch(prefix + gate), fetch(prefix + up)], dim=0).contiguous()
        self.down = fetch(prefix + down)

    def forward(self, h, batch, add_into=None):
        return linear(gated_linear(h, self.gate_up, self.activation), self.down, allow_partials=True, add_into=add_into)


register_part("feed_forward", "swiglu", SwiGLU)
