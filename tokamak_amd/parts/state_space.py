"""A selective state-space mixer with a scalar decay per head (the Mamba-2 form)."""

from __future__ import annotations

import torch

from tokamak_amd.config.registry import register_part
from tokamak_amd.kernels import ops
from tokamak_amd.kernels.linear import linear
from tokamak_amd.parts.base import Fetch, Mixer, PositionData, StateArray
from tokamak_amd.weights.spec import TensorSpec


class SelectiveStateSpace(Mixer):
    """State-space duality mixer.

    With inner = ``num_heads`` * ``value_dim``, N = ``state_size`` and G = ``groups``, the input
    projection W_in h is laid out [z: inner | x: inner | B: G N | C: G N | dt: heads].  x, B and C
    together pass a causal convolution per channel over ``conv_taps`` positions (weight
    [channels, taps] whose last column meets the token itself, a bias, zeros before the sequence's
    start) and SiLU.  Per head a (which reads group a // (heads / G)), with the state S [N, value_dim]
    (zeros at a sequence's start):

        dt  = softplus(dt + dt_bias_a)                       (no clamp)
        S  <- exp(-exp(A_log_a) dt) S + dt B_t x_t^T
        y_t = S^T C_t + D_a x_t

    y (heads side by side) is multiplied by silu(z), THEN divided by its root mean square over each
    of ``norm_groups`` equal parts of the row (``norm_eps``) and multiplied by a weight, and
    projected by W_o.  The request's state is S (float32, held as [heads, value_dim / 4, N, 4]) and the
    convolution's last taps - 1 inputs,
    both carried from step to step; step sizes, decays, the recurrence, the gate's product and the
    norm are float32.
    Tensors: in, conv, conv.b, dt_bias, A_log, D, norm, o behind the part's prefix.
    """

    capturable = True
    replayable = True

    def __init__(self, *, hidden_size: int, num_heads: int, value_dim: int, state_size: int, groups: int,
                 conv_taps: int, norm_groups: int, norm_eps: float, dtype, device,
                 names: tuple[str, ...] = ("in", "conv", "conv.b", "dt_bias", "A_log", "D", "norm", "o")) -> None:
        super().__init__(dtype=dtype, device=device)
        if min(hidden_size, num_heads, value_dim, state_size, groups, norm_groups) < 1:
            raise ValueError("every size of the state-space mixer must be >= 1")
        if num_heads % groups:
            raise ValueError(f"num_heads ({num_heads}) must be a multiple of groups ({groups})")
        if (num_heads * value_dim) % norm_groups:
            raise ValueError(f"norm_groups ({norm_groups}) must divide heads * value_dim ({num_heads * value_dim})")
        if not 1 <= conv_taps <= ops.SSM_MAX_TAPS:
            raise ValueError(f"the convolution has 1 to {ops.SSM_MAX_TAPS} taps, got {conv_taps}")
        if max(value_dim, state_size) > 1024:
            raise ValueError("value_dim and state_size are at most 1,024 for the scan kernel")
        self.hidden_size, self.num_heads, self.value_dim = int(hidden_size), int(num_heads), int(value_dim)
        self.state_size, self.groups, self.conv_taps = int(state_size), int(groups), int(conv_taps)
        self.norm_groups, self.norm_eps = int(norm_groups), float(norm_eps)
        self.inner = self.num_heads * self.value_dim
        self.conv_channels = self.inner + 2 * self.groups * self.state_size
        self.proj_width = 2 * self.inner + 2 * self.groups * self.state_size + self.num_heads
        self.names = tuple(names)
        self.w_in = self.conv = self.conv_bias = self.dt_bias = self.a_log = self.skip = self.gain = self.o = None

    def expected_tensors(self, prefix: str) -> dict[str, TensorSpec]:
        w_in, conv, conv_b, dt_bias, a_log, skip, norm, o = self.names
        heads, c = self.num_heads, self.conv_channels
        return {
            prefix + w_in: TensorSpec((self.proj_width, self.hidden_size)),
            prefix + conv: TensorSpec((c, self.conv_taps), held="float32"),
            prefix + conv_b: TensorSpec((c,), held="float32"),
            prefix + dt_bias: TensorSpec((heads,), held="float32"),
            prefix + a_log: TensorSpec((heads,), held="float32"),
            prefix + skip: TensorSpec((heads,), held="float32"),
            prefix + norm: TensorSpec((self.inner,), role="vector"),
            prefix + o: TensorSpec((self.hidden_size, self.inner)),
        }

    def bind(self, prefix: str, fetch: Fetch) -> None:
        w_in, conv, conv_b, dt_bias, a_log, skip, norm, o = self.names
        self.w_in, self.o = fetch(prefix + w_in), fetch(prefix + o)
        self.conv, self.conv_bias = fetch(prefix + conv), fetch(prefix + conv_b)
        self.dt_bias, self.a_log, self.skip = fetch(prefix + dt_bias), fetch(prefix + a_log), fetch(prefix + skip)
        self.gain = fetch(prefix + norm)

    def state_request(self) -> dict[str, StateArray]:
        # (a head's value columns in groups of four, as the scan's threads own them)
        out = {"S": StateArray((self.num_heads, -(-self.value_dim // 4), self.state_size, 4), torch.float32)}
        if self.conv_taps > 1:
            out["conv"] = StateArray((self.conv_taps - 1, self.conv_channels), torch.float32)
        return out

    def forward(self, h, batch, store, writes_cache: bool = True, position: PositionData | None = None):
        n = h.shape[0]
        inner = self.inner
        # (split products leave float32 partial sums, which the kernels below add as they load)
        proj = linear(h, self.w_in, allow_partials=True)
        u = torch.empty((n, self.conv_channels), dtype=self.dtype, device=h.device)
        ops.conv_silu(proj, inner, self.conv, self.conv_bias, store.state.get("conv"), u, batch)
        y = torch.empty((n, inner), dtype=torch.float32, device=h.device)
        ops.ssd_scan(u, proj, inner + self.conv_channels, self.dt_bias, self.a_log, self.skip, store.state["S"], y, batch,
                     heads=self.num_heads, groups=self.groups, state_size=self.state_size, vdim=self.value_dim)
        gated = torch.empty((n, inner), dtype=self.dtype, device=h.device)
        ops.gated_group_norm(y, proj, 0, self.gain, gated, groups=self.norm_groups, eps=self.norm_eps)
        return linear(gated, self.o, allow_partials=True)


register_part("mixer", "selective_state_space", SelectiveStateSpace)
