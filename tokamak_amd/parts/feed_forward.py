"""Feed-forward parts."""

from __future__ import annotations

import torch

from tokamak_amd.config.registry import register_part
from tokamak_amd.kernels import ops
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
    ``bias_suffix``: every projection has a bias, whose tensor is the projection's name plus this
    suffix: down(act(gate(x) + b_g) * (up(x) + b_u)) + b_d.  The biases are float32 and are added to
    the products' results in float32; the last one may be left to whoever adds the output to the
    residual stream (``output_bias``, ``forward(defer_bias=True)``).
    """

    capturable = True
    replayable = True

    def __init__(self, *, hidden_size: int, intermediate_size: int, dtype, device,
                 names: tuple[str, str, str] = ("gate_proj.weight", "up_proj.weight", "down_proj.weight"),
                 activation: str = "silu", bias_suffix: str | None = None) -> None:
        super().__init__(dtype=dtype, device=device)
        if activation not in GATE_ACTIVATIONS:
            raise ValueError(f"activation is one of {sorted(GATE_ACTIVATIONS)}, got {activation!r}")
        self.activation = activation
        self.hidden_size = int(hidden_size)
        self.intermediate_size = int(intermediate_size)
        self.names = tuple(names)       # gate, up, down behind the part's prefix
        self.bias_suffix = None if bias_suffix is None else str(bias_suffix)
        # (the products that add into the stream and finish a pending norm have no form with a bias)
        self.fuses_residual = self.bias_suffix is None
        self.gate_up: torch.Tensor | None = None
        self.down: torch.Tensor | None = None
        self.gate_up_bias: torch.Tensor | None = None
        self.output_bias: torch.Tensor | None = None

    def expected_tensors(self, prefix: str) -> dict[str, TensorSpec]:
        h, i = self.hidden_size, self.intermediate_size
        gate, up, down = self.names
        out = {prefix + gate: TensorSpec((i, h)), prefix + up: TensorSpec((i, h)), prefix + down: TensorSpec((h, i))}
        if self.bias_suffix is not None:
            b = self.bias_suffix
            out.update({prefix + gate + b: TensorSpec((i,), held="float32"),
                        prefix + up + b: TensorSpec((i,), held="float32"),
                        prefix + down + b: TensorSpec((h,), held="float32")})
        return out

    def bind(self, prefix: str, fetch: Fetch) -> None:
        gate, up, down = self.names
        self.gate_up = torch.cat([fetch(prefix + gate), fetch(prefix + up)], dim=0).contiguous()
        self.down = fetch(prefix + down)
        if self.bias_suffix is not None:
            b = self.bias_suffix
            self.gate_up_bias = torch.cat([fetch(prefix + gate + b), fetch(prefix + up + b)]).contiguous()
            self.output_bias = fetch(prefix + down + b)

    def forward(self, h, batch, add_into=None, defer_bias: bool = False):
        if self.bias_suffix is None:
            return linear(gated_linear(h, self.gate_up, self.activation), self.down, allow_partials=True, add_into=add_into)
        act = torch.empty((h.shape[0], self.intermediate_size), dtype=h.dtype, device=h.device)
        ops.silu_mul(linear(h, self.gate_up), act, self.activation, bias=self.gate_up_bias)
        if defer_bias:
            # (the caller adds ``output_bias`` where it adds the output to the stream)
            return linear(act, self.down, allow_partials=True)
        out = linear(act, self.down)
        ops.add_bias(out, self.output_bias)
        return out


register_part("feed_forward", "swiglu", SwiGLU)
