"""RMSNorm fused with the residual add."""

from __future__ import annotations

import torch

from tokamak_amd.config.registry import register_part
from tokamak_amd.kernels import ops
from tokamak_amd.kernels.linear import Added, DeferredNorm, StreamSink
from tokamak_amd.parts.base import BranchPair, Fetch, Norm
from tokamak_amd.weights.spec import TensorSpec


class RMSNorm(Norm):
    """x = resid + delta; out = x * rsqrt(mean(x^2) + eps) * weight.

    Statistics and the product with the weight are float32; one rounding to the
    compute dtype at the end (reference: src/tokamak/model/layers.py:28-33
    computes the statistics in float32, rounds, then multiplies by the weight).
    ``offset``: the checkpoint stores the weight less this number (a weight kept around
    zero has offset 1); it is added once, in float32, at binding.
    """

    capturable = True
    fuses_residual = True
    replayable = True

    def __init__(self, *, dim: int, eps: float, dtype, device, tensor: str = "weight", offset: float = 0.0) -> None:
        super().__init__(dtype=dtype, device=device)
        self.dim = int(dim)
        self.eps = float(eps)
        self.offset = float(offset)
        self.tensor = str(tensor)       # the weight's name behind the part's prefix
        self.weight: torch.Tensor | None = None

    def expected_tensors(self, prefix: str) -> dict[str, TensorSpec]:
        return {prefix + self.tensor: TensorSpec((self.dim,), role="vector")}

    def bind(self, prefix: str, fetch: Fetch) -> None:
        self.weight = fetch(prefix + self.tensor)
        if self.offset != 0.0:
            self.weight = (self.weight + self.offset).contiguous()

    def sink(self, resid: torch.Tensor) -> StreamSink:
        return StreamSink(resid, self.weight)

    def forward(self, resid, delta, *, rows=None, write_resid=True, defer=False):
        if isinstance(delta, Added):
            # the product before has added into the stream; if it has left the stream times
            # this norm's weight, the product after may finish the norm
            if defer and rows is None and delta.scaled is not None and delta.gamma is self.weight:
                return DeferredNorm(resid, self.weight, self.eps, self.dtype, delta.scaled, delta.sumsq)
            delta = None
        m = resid.shape[0] if rows is None else rows.numel()
        out = torch.empty((m, self.dim), dtype=self.dtype, device=resid.device)
        if isinstance(delta, BranchPair):
            # two branches that read the same normed input: their sum is formed first, then added
            ops.add_norm2(resid, delta.first, delta.second, self.weight, self.eps, out, center=False, rows=rows,
                          write_resid=write_resid)
            return out
        ops.add_rmsnorm(resid, delta, self.weight, self.eps, out, rows=rows, write_resid=write_resid)
        return out


class ScalarRMSNorm(RMSNorm):
    """RMSNorm whose gain is a single number for all coordinates:
    out = x * rsqrt(mean(x^2) + eps) * g.  The checkpoint holds g as a tensor without
    dimensions; it is spread over the row once, at binding, and the kernels of ``RMSNorm`` run."""

    def expected_tensors(self, prefix: str) -> dict[str, TensorSpec]:
        return {prefix + self.tensor: TensorSpec((), role="vector")}

    def bind(self, prefix: str, fetch: Fetch) -> None:
        self.weight = fetch(prefix + self.tensor).reshape(1).expand(self.dim).contiguous()


class LayerNorm(Norm):
    """x = resid + delta; out = (x - mean(x)) / sqrt(mean((x - mean(x))^2) + eps) * weight: a layer
    norm with a weight and no bias.  Mean, variance and the product with the weight are float32;
    one rounding to the compute dtype at the end.  ``delta`` may be a ``BranchPair``: the outputs
    of two sub-layers that read the same normed input, added to each other first and to the stream
    once."""

    capturable = True
    replayable = True

    def __init__(self, *, dim: int, eps: float, dtype, device, tensor: str = "weight") -> None:
        super().__init__(dtype=dtype, device=device)
        self.dim = int(dim)
        self.eps = float(eps)
        self.tensor = str(tensor)       # the weight's name behind the part's prefix
        self.weight: torch.Tensor | None = None

    def expected_tensors(self, prefix: str) -> dict[str, TensorSpec]:
        return {prefix + self.tensor: TensorSpec((self.dim,), role="vector")}

    def bind(self, prefix: str, fetch: Fetch) -> None:
        self.weight = fetch(prefix + self.tensor)

    def forward(self, resid, delta, *, rows=None, write_resid=True):
        first, second = (delta.first, delta.second) if isinstance(delta, BranchPair) else (delta, None)
        m = resid.shape[0] if rows is None else rows.numel()
        out = torch.empty((m, self.dim), dtype=self.dtype, device=resid.device)
        ops.add_norm2(resid, first, second, self.weight, self.eps, out, center=True, rows=rows, write_resid=write_resid)
        return out


register_part("norm", "rmsnorm", RMSNorm)
register_part("norm", "layernorm", LayerNorm)
register_part("norm", "scalar_rmsnorm", ScalarRMSNorm)
