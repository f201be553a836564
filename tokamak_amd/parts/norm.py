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
            # branches that belong to one residual add: their sum is formed first, then added
            ops.add_norm2(resid, delta.first, delta.second, self.weight, self.eps, out, center=False, rows=rows,
                          write_resid=write_resid, c=delta.third, bias=delta.bias, scale=delta.scale)
            return out
        ops.add_rmsnorm(resid, delta, self.weight, self.eps, out, rows=rows, write_resid=write_resid)
        return out

    def forward_pair(self, other: "RMSNorm", resid, delta):
        """(this norm's output, ``other``'s) of the same stream resid + delta, from one kernel: the row's root
        mean square is formed once and the row leaves twice, each time with one of the two weights.  None if
        the two norms do not agree on the size and eps (the caller then runs them one after the other)."""
        if type(other) is not type(self) or other.dim != self.dim or other.eps != self.eps or other.dtype != self.dtype:
            return None
        if isinstance(delta, Added):
            delta = None
        pair = delta if isinstance(delta, BranchPair) else BranchPair(delta) if delta is not None else None
        out = torch.empty((resid.shape[0], self.dim), dtype=self.dtype, device=resid.device)
        out2 = torch.empty_like(out)
        ops.add_norm2(resid, pair.first if pair else None, pair.second if pair else None, self.weight, self.eps, out,
                      center=False, c=pair.third if pair else None, bias=pair.bias if pair else None,
                      scale=pair.scale if pair else 1.0, weight2=other.weight, out2=out2)
        return out, out2


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
        pair = delta if isinstance(delta, BranchPair) else BranchPair(delta)
        m = resid.shape[0] if rows is None else rows.numel()
        out = torch.empty((m, self.dim), dtype=self.dtype, device=resid.device)
        ops.add_norm2(resid, pair.first, pair.second, self.weight, self.eps, out, center=True, rows=rows,
                      write_resid=write_resid, c=pair.third, bias=pair.bias, scale=pair.scale)
        return out


register_part("norm", "rmsnorm", RMSNorm)
register_part("norm", "layernorm", LayerNorm)
register_part("norm", "scalar_rmsnorm", ScalarRMSNorm)
