"""A routed feed-forward: a mixture of small gated experts."""

from __future__ import annotations

import torch

from tokamak_amd.config.registry import register_part
from tokamak_amd.kernels import ops
from tokamak_amd.kernels.linear import gated_linear, linear
from tokamak_amd.parts.base import FeedForward, Fetch
from tokamak_amd.weights.spec import TensorSpec


class RoutedExperts(FeedForward):
    """``num_experts`` feed-forwards down(silu(gate x) * up x) without biases, of which every token
    uses ``top``.

    The router's logits z = W_r h and the scores are float32: s = sigmoid(z), or with
    ``scoring="softmax"`` the softmax of z over all experts; the ``top`` experts
    with the largest scores are chosen (the lower index on a tie) and weighted by their scores
    as they are, not renormalised.  ``weight_on`` says where a weight w acts: ``"input"``, the
    expert sees w * h (out = sum expert(w h)), or ``"output"``, out = sum w * expert(h).  On the
    input the kernels use gate(w h) = w gate(h): the weight scales the two first products in
    float32; on the output they use w down(a) = down(w a): the weight scales the activations.  Tensors: router, e<i>.gate, e<i>.up, e<i>.down; an expert's gate and up are held as
    one matrix and the experts as one array each.

    ``correction``: a tensor of that name [experts] is added to the scores for the CHOICE only (the weights
    stay the scores without it); it may be absent from the checkpoint.  ``groups`` = (count, keep): the
    experts form ``count`` equal groups of neighbours, a group's score is the sum of its two largest choice
    scores, and only experts of the ``keep`` best groups can be chosen.  ``normalise``: the chosen weights
    are divided by their sum (+ 1e-20).  ``weight_scale``: all weights times this number.
    ``shared_size``: one more expert of that inner size (tensors ``shared.gate``, ``shared.up``,
    ``shared.down``) that every token uses with weight one; ``forward`` then returns two terms, the routed
    experts' partial sums and the shared expert's output.
    """

    capturable = True
    replayable = True

    def __init__(self, *, hidden_size: int, intermediate_size: int, num_experts: int, top: int,
                 weight_on: str = "input", scoring: str = "sigmoid", dtype, device,
                 names: tuple[str, str, str, str, str] = ("router", "e{}.", "gate", "up", "down"),
                 correction: str | None = None, groups: tuple[int, int] | None = None, normalise: bool = False,
                 weight_scale: float = 1.0, shared_size: int | None = None, shared_prefix: str = "shared.") -> None:
        super().__init__(dtype=dtype, device=device)
        self.hidden_size, self.intermediate_size = int(hidden_size), int(intermediate_size)
        self.num_experts, self.top = int(num_experts), int(top)
        if not 1 <= self.top <= self.num_experts:
            raise ValueError(f"top ({top}) must be between 1 and the number of experts ({num_experts})")
        if weight_on not in ("input", "output"):
            raise ValueError(f"weight_on is 'input' or 'output', got {weight_on!r}")
        if scoring not in ("sigmoid", "softmax"):
            raise ValueError(f"scoring is 'sigmoid' or 'softmax', got {scoring!r}")
        self.weight_on, self.scoring = weight_on, scoring
        self.names = tuple(names)
        self.correction_name = None if correction is None else str(correction)
        self.groups = None if groups is None else (int(groups[0]), int(groups[1]))
        if self.groups is not None:
            count, keep = self.groups
            if count < 1 or self.num_experts % count or not 1 <= keep <= count or keep * (self.num_experts // count) < self.top:
                raise ValueError(f"groups ({count}, keep {keep}) must divide the {num_experts} experts evenly and the kept "
                                 f"groups must hold at least top ({top}) experts")
        self.normalise, self.weight_scale = bool(normalise), float(weight_scale)
        self.shared_size = None if shared_size is None else int(shared_size)
        if self.shared_size is not None and self.shared_size < 1:
            raise ValueError(f"shared_size must be >= 1, got {shared_size}")
        self.shared_prefix = str(shared_prefix)
        self.router = self.gate_up = self.down = None
        self.correction = self.shared_gate_up = self.shared_down = None

    def expected_tensors(self, prefix: str) -> dict[str, TensorSpec]:
        h, f = self.hidden_size, self.intermediate_size
        router, expert, gate, up, down = self.names
        out = {prefix + router: TensorSpec((self.num_experts, h), held="float32")}
        for e in range(self.num_experts):
            base = prefix + expert.format(e)
            out.update({base + gate: TensorSpec((f, h)), base + up: TensorSpec((f, h)), base + down: TensorSpec((h, f))})
        if self.correction_name is not None:
            out[prefix + self.correction_name] = TensorSpec((self.num_experts,), held="float32", optional=True)
        if self.shared_size is not None:
            base, s = prefix + self.shared_prefix, self.shared_size
            out.update({base + gate: TensorSpec((s, h)), base + up: TensorSpec((s, h)), base + down: TensorSpec((h, s))})
        return out

    def bind(self, prefix: str, fetch: Fetch) -> None:
        router, expert, gate, up, down = self.names
        self.router = fetch(prefix + router)
        bases = [prefix + expert.format(e) for e in range(self.num_experts)]
        self.gate_up = torch.stack([torch.cat([fetch(b + gate), fetch(b + up)], dim=0) for b in bases]).contiguous()
        self.down = torch.stack([fetch(b + down) for b in bases]).contiguous()
        if self.correction_name is not None:
            self.correction = fetch(prefix + self.correction_name)      # (None if the checkpoint has none)
        if self.shared_size is not None:
            base = prefix + self.shared_prefix
            self.shared_gate_up = torch.cat([fetch(base + gate), fetch(base + up)], dim=0).contiguous()
            self.shared_down = fetch(base + down)

    def matrix_share(self, tokens: int) -> tuple[float, float]:
        e, top = self.num_experts, self.top
        router, expert = e * self.hidden_size, 3 * self.intermediate_size * self.hidden_size
        met = e * (1.0 - (1.0 - top / e) ** max(tokens, 0))     # experts that a step of so many tokens meets, on average
        shared = 0 if self.shared_size is None else 3 * self.shared_size * self.hidden_size
        total = router + e * expert + shared
        return (router + top * expert + shared) / total, (router + met * expert + shared) / total

    def forward(self, h, batch):
        """Float32 partial sums [top, N, width]: layer k holds every token's k-th chosen expert's output;
        whoever adds the sub-layer's output to the stream sums them in that order.  With a shared expert a
        tuple: those, and the shared expert's output."""
        routed = self._routed(h)
        if self.shared_size is None:
            return routed
        return routed, linear(gated_linear(h, self.shared_gate_up), self.shared_down, allow_partials=True)

    def _routed(self, h):
        n, top = h.shape[0], self.top
        chosen = torch.empty((n, top), dtype=torch.int32, device=h.device)
        weight = torch.empty((n, top), dtype=torch.float32, device=h.device)
        ops.moe_route(h, self.router, chosen, weight, top, self.scoring, correction=self.correction, groups=self.groups,
                      normalise=self.normalise, scale=self.weight_scale)
        on_output = self.weight_on == "output"
        act = torch.empty((n * top, self.intermediate_size), dtype=h.dtype, device=h.device)
        out = torch.empty((top, n, self.hidden_size), dtype=torch.float32, device=h.device)
        if ops.moe_grouped_fits(h, self.gate_up, self.down, n * top):
            # many tokens: the pairs listed expert by expert, tiles of one expert on the matrix cores
            lists = ops.moe_sort(chosen, self.num_experts)
            ops.moe_grouped(h, self.gate_up, lists, weight, act, tokens=n, top=top, gated=True, weight_on_output=on_output)
            ops.moe_grouped(act, self.down, lists, None, out, tokens=n, top=top, gated=False)
            return out
        ops.moe_gate_up(h, self.gate_up, chosen, weight, act, top, on_output)
        ops.moe_down(act, self.down, chosen, out, top)
        return out


register_part("feed_forward", "routed_experts", RoutedExperts)
