"""Grouped-query attention over a paged cache."""

from __future__ import annotations

import torch

from tokamak_amd.config.registry import register_part
from tokamak_amd.kernels import ops
from tokamak_amd.kernels.attention import (ATTENTION_WORK, check_page_size, decode_attention_fused, fused_decode_fits,
                                            paged_attention)
from tokamak_amd.kernels.linear import linear
from tokamak_amd.parts.base import CacheRequest, Fetch, Mixer, PositionData
from tokamak_amd.weights.spec import TensorSpec


class GQAAttention(Mixer):
    """q/k/v projections, optional per-head RMSNorm of q and k, rotation of q and k
    by the tables the layer's position encoding prepared (none: no rotation),
    causal softmax attention over the request's pages, o projection
    (reference: src/tokamak/model/transformer.py:22-86).

    Query head a reads kv head a // (num_heads / num_kv_heads).  Keys are cached
    after norm and rotation, values as projected (transformer.py:71-82).  The
    three projections are held as one [(nh + 2 nkv) hd, H] matrix.
    ``window``: None for full causal attention, W to see the last W positions.
    """

    capturable = True
    fuses_residual = True
    replayable = True

    def __init__(self, *, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 qk_norm_eps: float | None, softmax_scale: float, window: int | None,
                 dtype, device) -> None:
        super().__init__(dtype=dtype, device=device)
        if num_heads % num_kv_heads:
            raise ValueError(f"num_heads ({num_heads}) must be divisible by num_kv_heads ({num_kv_heads})")
        if head_dim % 16 or head_dim > 512:
            raise ValueError(f"head_dim must be a multiple of 16 and at most 512, got {head_dim}")
        self.hidden_size, self.num_heads, self.num_kv_heads = int(hidden_size), int(num_heads), int(num_kv_heads)
        self.head_dim = int(head_dim)
        self.qk_norm_eps = None if qk_norm_eps is None else float(qk_norm_eps)
        self.softmax_scale = float(softmax_scale)
        self.window = None if window is None else int(window)
        self.qkv: torch.Tensor | None = None
        self.o: torch.Tensor | None = None
        self.q_norm: torch.Tensor | None = None
        self.k_norm: torch.Tensor | None = None

    def expected_tensors(self, prefix: str) -> dict[str, TensorSpec]:
        h, nh, nkv, hd = self.hidden_size, self.num_heads, self.num_kv_heads, self.head_dim
        out = {
            prefix + "q_proj.weight": TensorSpec((nh * hd, h)),
            prefix + "k_proj.weight": TensorSpec((nkv * hd, h)),
            prefix + "v_proj.weight": TensorSpec((nkv * hd, h)),
            prefix + "o_proj.weight": TensorSpec((h, nh * hd)),
        }
        if self.qk_norm_eps is not None:
            out[prefix + "q_norm.weight"] = TensorSpec((hd,), role="vector")
            out[prefix + "k_norm.weight"] = TensorSpec((hd,), role="vector")
        return out

    def bind(self, prefix: str, fetch: Fetch) -> None:
        self.qkv = torch.cat([fetch(prefix + n + "_proj.weight") for n in "qkv"], dim=0).contiguous()
        self.o = fetch(prefix + "o_proj.weight")
        if self.qk_norm_eps is not None:
            self.q_norm = fetch(prefix + "q_norm.weight")
            self.k_norm = fetch(prefix + "k_norm.weight")

    def cache_request(self) -> CacheRequest:
        width = self.num_kv_heads * self.head_dim
        return CacheRequest.of(window=self.window, k=width, v=width)

    def step_planner(self):
        return ATTENTION_WORK

    def check_page_size(self, page_size: int) -> None:
        check_page_size(page_size)

    def pair_flops(self) -> float:
        # q.k and p.v: two multiply-adds per head and head element
        return 4.0 * self.num_heads * self.head_dim

    def forward(self, h, batch, store, writes_cache: bool = True,
                position: PositionData | None = None, add_into=None):
        nh, nkv, hd = self.num_heads, self.num_kv_heads, self.head_dim
        n = h.shape[0]
        weight = self.qkv if writes_cache else self.qkv[: nh * hd]
        qkv = linear(h, weight, allow_partials=True)
        cos = sin = None
        rotary_dim = 0
        if position is not None:
            if position.score_slopes is not None:
                raise ops.KernelError("this attention part has no kernel for a bias on the scores; "
                                      "it takes rotary tables or no position data")
            if position.interleaved:
                raise ops.KernelError("this attention part's kernels rotate half-split pairs only")
            cos, sin, rotary_dim = position.cos, position.sin, position.rotary_dim
        tables = batch.block_tables[store.group]
        attended = torch.empty((n, nh * hd), dtype=h.dtype, device=h.device)
        if fused_decode_fits(h.dtype, hd, store.page_size, nh // nkv, self.window, rotary_dim, batch):
            # a step of decode tokens only: norm, rotation, cache write and attention in one kernel
            if decode_attention_fused(
                    qkv, self.q_norm, self.k_norm, cos, sin, store.arrays["k"], store.arrays["v"], tables, batch,
                    attended, num_heads=nh, num_kv_heads=nkv, head_dim=hd, rotary_dim=rotary_dim,
                    page_size=store.page_size, eps=self.qk_norm_eps or 0.0, scale=self.softmax_scale,
                    store=writes_cache):
                return linear(attended, self.o, allow_partials=True, add_into=add_into)
        q = torch.empty((n, nh * hd), dtype=h.dtype, device=h.device)
        ops.qknorm_rope_store(
            qkv, self.q_norm, self.k_norm, cos, sin, batch.positions, batch.req_of_token, tables, q,
            store.arrays["k"], store.arrays["v"], num_heads=nh, num_kv_heads=nkv, head_dim=hd,
            rotary_dim=rotary_dim, page_size=store.page_size,
            eps=self.qk_norm_eps or 0.0, store=writes_cache)
        paged_attention(q, store.arrays["k"], store.arrays["v"], tables, batch, attended,
                        num_heads=nh, num_kv_heads=nkv, head_dim=hd, page_size=store.page_size,
                        scale=self.softmax_scale, window=self.window)
        return linear(attended, self.o, allow_partials=True, add_into=add_into)


class RotatedUnitAttention(Mixer):
    """Grouped-query attention whose queries and keys are rotated first and then each divided
    by its root mean square per head (a unit norm without a weight), with values of a size of
    their own and an optional chunked mask.

    q = W_q h, k = W_k h (``num_heads`` / ``num_kv_heads`` heads of ``head_dim``), v = W_v h
    (``num_kv_heads`` heads of ``value_dim``), no biases; the layer's position encoding rotates
    the first ``rotary_dim`` dims of q and k (half-split pairs), the rest pass; then
    q, k <- x / sqrt(mean(x^2) + ``norm_eps``) per head (``norm_eps`` None: no norm);
    score = q . k * ``softmax_scale``; with ``chunk`` = C position i sees j <= i only if
    i // C == j // C, chunks counted from position 0 of the sequence whatever the step's cut; with
    ``window`` = W only if i - j < W, or, with ``keep_first`` = F, if j < F (the first F positions of a
    sequence stay visible at their true positions); softmax; o projection over the concatenated heads.  Keys are
    cached after rotation and norm, values as projected.  Tensors: q, k, v, o behind the part's prefix.

    ``sink``: every head has a learned number s_a (tensor ``sink`` [heads], float32) whose exp(s_a)
    is one more term of its softmax's denominator: it has no key and no value and is not scaled.
    ``value_mix``: values shared across layers.  The layer that says ``"source"`` leaves its values,
    as projected, for the layers after it in the same step; a layer that says ``"mix"`` caches
    (1 - lambda) v + lambda v_source, with v_source the source's values of the same token and lambda
    its own tensor ``vmix`` (one number; the source has the tensor too and does not use it).  All
    layers of one model that mix have kv heads and value sizes alike.  The rotation pairs dimensions
    as the layer's position encoding says (half-split or interleaved).
    """

    capturable = True
    replayable = True

    def __init__(self, *, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int, value_dim: int,
                 softmax_scale: float, norm_eps: float | None, chunk: int | None, dtype, device,
                 names: tuple[str, str, str, str] = ("q", "k", "v", "o"), window: int | None = None,
                 sink: bool = False, value_mix: str | None = None,
                 extra_names: tuple[str, str] = ("sink", "vmix"), keep_first: int = 0) -> None:
        super().__init__(dtype=dtype, device=device)
        if num_heads < 1 or num_kv_heads < 1 or num_heads % num_kv_heads:
            raise ValueError(f"num_heads ({num_heads}) must be a multiple of num_kv_heads ({num_kv_heads})")
        if min(head_dim, value_dim) < 1 or max(ops.padded_sizes(head_dim, value_dim)) > 512:
            raise ValueError(f"head_dim and value_dim must be 1 to 512; got {head_dim}, {value_dim}")
        if chunk is not None and chunk < 1:
            raise ValueError(f"chunk must be >= 1, got {chunk}")
        self.hidden_size, self.num_heads, self.num_kv_heads = int(hidden_size), int(num_heads), int(num_kv_heads)
        self.head_dim, self.value_dim = int(head_dim), int(value_dim)
        # cache pages, queries and attention outputs are laid out for keys in pieces of 8 channels and
        # values in blocks of 16: sizes that do not fill them are padded with zeros, which add nothing
        self.key_size, self.value_size = ops.padded_sizes(self.head_dim, self.value_dim)
        self.softmax_scale = float(softmax_scale)
        self.norm_eps = None if norm_eps is None else float(norm_eps)
        self.chunk = None if chunk is None else int(chunk)
        if window is not None and (window < 1 or chunk is not None):
            raise ValueError("window must be >= 1 and does not go together with chunks")
        if value_mix not in (None, "source", "mix"):
            raise ValueError(f"value_mix is None, 'source' or 'mix', got {value_mix!r}")
        self.window = None if window is None else int(window)
        if keep_first < 0 or (keep_first and window is None):
            raise ValueError("keep_first must be >= 0 and goes with a window")
        self.keep_first = int(keep_first)
        self.has_sink, self.value_mix = bool(sink), value_mix
        self.extra_names = tuple(extra_names)
        self.sink: torch.Tensor | None = None
        self.vmix: torch.Tensor | None = None
        self.names = tuple(names)
        self.qkv: torch.Tensor | None = None
        self.o: torch.Tensor | None = None

    def expected_tensors(self, prefix: str) -> dict[str, TensorSpec]:
        h, nh, nkv, hd, vd = self.hidden_size, self.num_heads, self.num_kv_heads, self.head_dim, self.value_dim
        q, k, v, o = self.names
        out = {prefix + q: TensorSpec((nh * hd, h)), prefix + k: TensorSpec((nkv * hd, h)),
               prefix + v: TensorSpec((nkv * vd, h)), prefix + o: TensorSpec((h, nh * vd))}
        if self.has_sink:
            out[prefix + self.extra_names[0]] = TensorSpec((nh,), role="vector")
        if self.value_mix is not None:
            out[prefix + self.extra_names[1]] = TensorSpec((), role="vector")
        return out

    def bind(self, prefix: str, fetch: Fetch) -> None:
        q, k, v, o = self.names
        self.qkv = torch.cat([fetch(prefix + n) for n in (q, k, v)], dim=0).contiguous()
        self.o = fetch(prefix + o)
        if self.has_sink:
            self.sink = fetch(prefix + self.extra_names[0])
        if self.value_mix is not None:
            self.vmix = fetch(prefix + self.extra_names[1]).reshape(1).contiguous()
        if self.value_size != self.value_dim:
            # (the attention's output has the padded value size: columns of zeros in between)
            wide = torch.zeros((self.hidden_size, self.num_heads, self.value_size), dtype=self.o.dtype, device=self.o.device)
            wide[:, :, :self.value_dim] = self.o.view(self.hidden_size, self.num_heads, self.value_dim)
            self.o = wide.view(self.hidden_size, self.num_heads * self.value_size).contiguous()

    def cache_request(self) -> CacheRequest:
        return CacheRequest.of(window=self.window, keep_first=self.keep_first, k=self.num_kv_heads * self.key_size,
                               v=self.num_kv_heads * self.value_size)

    def step_planner(self):
        return ATTENTION_WORK

    def check_page_size(self, page_size: int) -> None:
        check_page_size(page_size)

    def pair_flops(self) -> float:
        return 2.0 * self.num_heads * (self.head_dim + self.value_dim)

    def visible_keys(self, position: int) -> int:
        if self.window is not None:
            behind = max(0, position + 1 - self.window)      # positions behind the window, of which the first stay
            return min(position + 1, self.window) + min(behind, self.keep_first)
        return position + 1 if self.chunk is None else position % self.chunk + 1

    def _shared_values(self, batch, n: int, device):
        """(the step's values of the source layer, float32 [N, kv heads * value_dim]; what this layer
        does with them: 0 nothing, 1 fills them, 2 mixes them in)."""
        if self.value_mix is None:
            return None, 0
        key = ("value_mix", self.num_kv_heads, self.value_dim)
        kept = batch.memo.get(key)
        if self.value_mix == "source":
            kept = batch.memo[key] = torch.empty((n, self.num_kv_heads * self.value_dim), dtype=torch.float32, device=device)
            return kept, 1
        if kept is None:
            raise ops.KernelError("a layer mixes in another layer's values, but no layer before it in this step "
                                  "is their source (or its kv heads and value size differ)")
        return kept, 2

    def forward(self, h, batch, store, writes_cache: bool = True, position: PositionData | None = None):
        nh, nkv, hd, vd = self.num_heads, self.num_kv_heads, self.head_dim, self.value_dim
        n = h.shape[0]
        weight = self.qkv if writes_cache else self.qkv[: nh * hd]
        qkv = linear(h, weight, allow_partials=True)
        cos = sin = None
        rotary_dim, interleaved = 0, False
        if position is not None:
            if position.score_slopes is not None:
                raise ops.KernelError("this attention part has no kernel for a bias on the scores")
            cos, sin, rotary_dim, interleaved = position.cos, position.sin, position.rotary_dim, position.interleaved
        tables = batch.block_tables[store.group]
        q = torch.empty((n, nh * self.key_size), dtype=h.dtype, device=h.device)
        kept, value_mode = self._shared_values(batch, n, h.device) if writes_cache else (None, 0)
        ops.rope_norm_store(
            qkv, None, None, cos, sin, batch.positions, batch.req_of_token, tables, q, store.arrays["k"],
            store.arrays["v"], num_heads=nh, num_kv_heads=nkv, head_dim=hd, value_dim=vd, rotary_dim=rotary_dim,
            page_size=store.page_size, unit_norm=self.norm_eps is not None, eps=self.norm_eps or 0.0, store=writes_cache,
            interleaved=interleaved, value_keep=kept, value_mode=value_mode, value_lambda=self.vmix)
        attended = torch.empty((n, nh * self.value_size), dtype=h.dtype, device=h.device)
        paged_attention(q, store.arrays["k"], store.arrays["v"], tables, batch, attended, num_heads=nh,
                        num_kv_heads=nkv, head_dim=self.key_size, value_dim=self.value_size, page_size=store.page_size,
                        scale=self.softmax_scale, chunk=self.chunk, window=self.window, sinks=self.sink,
                        keep_first=self.keep_first)
        return linear(attended, self.o, allow_partials=True)


register_part("mixer", "gqa_attention", GQAAttention)
register_part("mixer", "rotated_unit_attention", RotatedUnitAttention)
