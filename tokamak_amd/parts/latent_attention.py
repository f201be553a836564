"""Attention whose keys and values are made from a cached low-rank latent."""

from __future__ import annotations

import torch

from tokamak_amd.config.registry import register_part
from tokamak_amd.kernels import ops
from tokamak_amd.kernels.attention import ATTENTION_WORK, check_page_size, paged_attention
from tokamak_amd.kernels.linear import linear
from tokamak_amd.parts.base import CacheRequest, Fetch, Mixer, PositionData
from tokamak_amd.weights.spec import TensorSpec


class LatentAttention(Mixer):
    """Multi-head attention over a compressed cache.

    q = W_q h, head by head [``head_dim`` unrotated | ``rot_dim`` rotated].  W_dkv h has ``rank`` +
    ``rot_dim`` rows: the first ``rank``, divided by their root mean square (``norm_eps``) and
    multiplied by a weight, are the latent c; the last ``rot_dim`` are one rotated key part shared
    by all heads.  Head a's key is [W_uk,a c | rotated part], its value W_uv,a c (``value_dim``);
    score = (q_unrotated . k_unrotated + q_rotated . k_rotated) * ``softmax_scale``.  The layer's
    position encoding rotates the first ``rotary_dim`` dims of the rotated parts of q and of the
    key.  ``window`` = W: position i sees j with 0 <= i - j < W (None: every j <= i).  ``sink``:
    a learned number per head whose exponential is one more term of the softmax's denominator.

    Only c and the rotated key part are cached, as ONE key/value head: the key is [c | rotated
    part], the value is c.  Since (W_uk,a c) . q = c . (W_uk,a^T q), a token's query is carried into
    the latent's space once (a small product per head), the engine's paged attention runs over the
    latents with ``num_heads`` query heads on one kv head, and the head's result, a weighted sum of
    latents, goes through W_uv,a afterwards; the up-projections of cached tokens are never formed.
    Tensors: q, dkv, dkv.norm, uk, uv, o (and sink) behind the part's prefix.

    ``q_rank``: the queries go through a latent of their own, c_q = W_dq h divided by its root mean
    square (``norm_eps``) times a weight, q = W_uq c_q (tensors dq, dq.norm, uq in place of q; without
    a rotated part).
    ``own_latent`` False: the layer has no W_dkv and caches nothing; it attends over the latents that
    another layer of the same rank left in the cache slot its call names, with its own W_uk and W_uv.
    """

    capturable = True
    replayable = True

    def __init__(self, *, hidden_size: int, num_heads: int, head_dim: int, rot_dim: int, value_dim: int, rank: int,
                 softmax_scale: float, norm_eps: float, window: int | None, sink: bool, dtype, device,
                 names: tuple[str, ...] = ("q", "dkv", "dkv.norm", "uk", "uv", "o", "sink"),
                 q_rank: int | None = None, own_latent: bool = True,
                 q_names: tuple[str, str, str] = ("dq", "dq.norm", "uq")) -> None:
        super().__init__(dtype=dtype, device=device)
        if min(hidden_size, num_heads, head_dim, value_dim, rank) < 1 or rot_dim < 0:
            raise ValueError("every size of the latent attention must be >= 1 (rot_dim >= 0)")
        if window is not None and window < 1:
            raise ValueError(f"window must be >= 1, got {window}")
        self.hidden_size, self.num_heads = int(hidden_size), int(num_heads)
        self.head_dim, self.rot_dim, self.value_dim, self.rank = int(head_dim), int(rot_dim), int(value_dim), int(rank)
        # the cached key [latent | rotated part] and the cached value (the latent), as the pages are laid out
        self.key_size, self.value_size = ops.padded_sizes(self.rank + self.rot_dim, self.rank)
        if max(self.key_size, self.value_size) > 512 or self.head_dim + self.rot_dim > 1024:
            raise ValueError(f"rank + rot_dim must be at most 512 and head_dim + rot_dim at most 1,024; got "
                             f"{rank}, {rot_dim}, {head_dim}")
        self.softmax_scale, self.norm_eps = float(softmax_scale), float(norm_eps)
        self.window = None if window is None else int(window)
        self.has_sink = bool(sink)
        self.names = tuple(names)
        self.q_rank = None if q_rank is None else int(q_rank)
        if self.q_rank is not None and not 1 <= self.q_rank <= 1024:
            raise ValueError(f"q_rank must be 1 to 1,024, got {q_rank}")
        if self.q_rank is not None and self.rot_dim:
            raise ValueError("queries through a latent have no rotated part here (rot_dim must be 0)")
        self.own_latent = bool(own_latent)
        self.q_names = tuple(q_names)
        self.q_dkv = self.latent_norm = self.uk_t = self.uv = self.o = self.sink = None
        self.q_norm = self.uq = None

    def expected_tensors(self, prefix: str) -> dict[str, TensorSpec]:
        h, nh, hd, rd, vd, r = self.hidden_size, self.num_heads, self.head_dim, self.rot_dim, self.value_dim, self.rank
        q, dkv, norm, uk, uv, o, sink = self.names
        out = {prefix + uk: TensorSpec((nh * hd, r)), prefix + uv: TensorSpec((nh * vd, r)), prefix + o: TensorSpec((h, nh * vd))}
        if self.own_latent:
            out.update({prefix + dkv: TensorSpec((r + rd, h)), prefix + norm: TensorSpec((r,), role="vector")})
        if self.q_rank is None:
            out[prefix + q] = TensorSpec((nh * (hd + rd), h))
        else:
            dq, dq_norm, uq = self.q_names
            out.update({prefix + dq: TensorSpec((self.q_rank, h)), prefix + dq_norm: TensorSpec((self.q_rank,), role="vector"),
                        prefix + uq: TensorSpec((nh * (hd + rd), self.q_rank))})
        if self.has_sink:
            out[prefix + sink] = TensorSpec((nh,), role="vector")
        return out

    def bind(self, prefix: str, fetch: Fetch) -> None:
        q, dkv, norm, uk, uv, o, sink = self.names
        nh, hd, vd, r = self.num_heads, self.head_dim, self.value_dim, self.rank
        # one product yields the queries (or their latent), the latent and the rotated key part
        first = fetch(prefix + q) if self.q_rank is None else fetch(prefix + self.q_names[0])
        self.q_dkv = torch.cat([first, fetch(prefix + dkv)], dim=0).contiguous() if self.own_latent else first
        self.latent_norm = fetch(prefix + norm) if self.own_latent else None
        if self.q_rank is not None:
            self.q_norm = fetch(prefix + self.q_names[1])
            self.uq = fetch(prefix + self.q_names[2])
        # W_uk per head, transposed: [heads, rank, head_dim] takes a query into the latent's space
        self.uk_t = fetch(prefix + uk).view(nh, hd, r).transpose(1, 2).contiguous()
        self.uv = fetch(prefix + uv).view(nh, vd, r).contiguous()
        self.o = fetch(prefix + o)
        if self.has_sink:
            self.sink = fetch(prefix + sink)

    def cache_request(self) -> CacheRequest | None:
        if not self.own_latent:
            return None
        return CacheRequest.of(window=self.window, k=self.key_size, v=self.value_size)

    def step_planner(self):
        return ATTENTION_WORK

    def check_page_size(self, page_size: int) -> None:
        check_page_size(page_size)

    def pair_flops(self) -> float:
        return 2.0 * self.num_heads * (self.rank + self.rot_dim + self.rank)

    def visible_keys(self, position: int) -> int:
        return position + 1 if self.window is None else min(position + 1, self.window)

    def forward(self, h, batch, store, writes_cache: bool = True, position: PositionData | None = None):
        nh, hd, rd, vd, r = self.num_heads, self.head_dim, self.rot_dim, self.value_dim, self.rank
        n = h.shape[0]
        if writes_cache and not self.own_latent:
            raise ops.KernelError("a latent attention without a latent of its own reads another layer's cache slot")
        q_rows = nh * (hd + rd) if self.q_rank is None else self.q_rank
        weight = self.q_dkv if writes_cache or not self.own_latent else self.q_dkv[:q_rows]
        proj = linear(h, weight, allow_partials=True)
        cos = sin = None
        rotary_dim, interleaved = 0, False
        if position is not None:
            if position.score_slopes is not None:
                raise ops.KernelError("this attention part has no kernel for a bias on the scores")
            cos, sin, rotary_dim, interleaved = position.cos, position.sin, position.rotary_dim, position.interleaved
        tables = batch.block_tables[store.group]
        q_full = torch.empty((n, nh, self.key_size), dtype=h.dtype, device=h.device)
        if self.q_rank is None:
            q_plain = torch.empty((n, nh, hd), dtype=h.dtype, device=h.device)
            ops.latent_prepare(proj, self.latent_norm, cos, sin, batch.positions, batch.req_of_token, tables, q_plain, q_full,
                               store.arrays["k"], store.arrays["v"], num_heads=nh, head_dim=hd, rot_dim=rd, rank=r,
                               rotary_dim=rotary_dim, interleaved=interleaved, page_size=store.page_size, eps=self.norm_eps,
                               store=writes_cache)
        else:
            # the query's latent is one unit that is normed like the keys' latent, which goes into the pages
            c_q = torch.empty((n, self.q_rank), dtype=h.dtype, device=h.device)
            ops.latent_prepare(proj, self.latent_norm, None, None, batch.positions, batch.req_of_token, tables, c_q, None,
                               store.arrays["k"], store.arrays["v"], num_heads=1, head_dim=self.q_rank, rot_dim=0, rank=r,
                               rotary_dim=0, interleaved=False, page_size=store.page_size, eps=self.norm_eps,
                               store=writes_cache, q_weight=self.q_norm)
            q = linear(c_q, self.uq)
            if self.key_size == r:
                q_plain = q.view(n, nh, hd)
            else:
                q_plain = torch.empty((n, nh, hd), dtype=h.dtype, device=h.device)
                ops.latent_prepare(q, None, cos, sin, batch.positions, batch.req_of_token, tables, q_plain, q_full,
                                   None, None, num_heads=nh, head_dim=hd, rot_dim=rd, rank=r, rotary_dim=rotary_dim,
                                   interleaved=interleaved, page_size=store.page_size, eps=self.norm_eps, store=False)
        ops.head_linear(q_plain, self.uk_t, q_full[:, :, :r])
        attended = torch.empty((n, nh, self.value_size), dtype=h.dtype, device=h.device)
        paged_attention(q_full, store.arrays["k"], store.arrays["v"], tables, batch, attended, num_heads=nh,
                        num_kv_heads=1, head_dim=self.key_size, value_dim=self.value_size, page_size=store.page_size,
                        scale=self.softmax_scale, window=self.window, sinks=self.sink)
        values = torch.empty((n, nh, vd), dtype=h.dtype, device=h.device)
        ops.head_linear(attended[:, :, :r], self.uv, values)
        return linear(values.view(n, nh * vd), self.o, allow_partials=True)


register_part("mixer", "latent_attention", LatentAttention)
