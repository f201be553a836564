"""Plain, slow implementation of the Supinex design, one function per mechanism.

Written from the design's equations with torch on the CPU, a query at a time; it shares no
code with the engine.  ``cfg`` is the ``config.json`` dict itself and ``w`` a dict of tensors by
checkpoint name.  Everything runs in the dtype of the tensors it is given (the tests use
float64 or float32).

A layer is x <- x + (mixer(h) + ff(h)) with h = layer_norm(x): one norm, both sub-layers read
its output.  The mixers keep what a later call needs in ``past`` (keys and values, or latents
and the shared rotated key part), so a prompt can be fed in portions.
"""

from __future__ import annotations

import math

import torch


def layer_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """(x - mean) / sqrt(variance + eps) * weight, the variance being the mean squared deviation."""
    d = x - x.mean(-1, keepdim=True)
    return d / torch.sqrt((d * d).mean(-1, keepdim=True) + eps) * weight


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def rotary_frequencies(rot: dict) -> tuple[torch.Tensor, float]:
    """(f_i for i < dims / 2 in float64, the amplitude that multiplies cos and sin).

    f_i = base^(-2i/dims).  With a ``scaling`` entry (factor s, original length L, fast, slow):
    d(t) = dims ln(L / (2 pi t)) / (2 ln base), lo = max(floor(d(fast)), 0), hi = min(ceil(d(slow)), dims - 1),
    r_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1), f_i <- f_i / s * r_i + f_i (1 - r_i); amplitude 0.1 ln s + 1."""
    dims, base = int(rot["dims"]), float(rot["base"])
    f = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    amplitude = 1.0
    s = rot.get("scaling")
    if s:
        factor, original = float(s["factor"]), float(s["original"])

        def d(turns: float) -> float:
            return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

        lo = max(math.floor(d(float(s["fast"]))), 0)
        hi = min(math.ceil(d(float(s["slow"]))), dims - 1)
        for i in range(dims // 2):
            r = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
            f[i] = f[i] / factor * r + f[i] * (1.0 - r)
        amplitude = 0.1 * math.log(factor) + 1.0
    return torch.tensor(f, dtype=torch.float64), amplitude


def rotate(x: torch.Tensor, positions: torch.Tensor, rot: dict | None) -> torch.Tensor:
    """x [T, heads, dim]: the first rot.dims dimensions of every head are rotated, dimension 2i
    paired with 2i + 1; the rest pass."""
    if not rot or int(rot["dims"]) == 0:
        return x
    f, amplitude = rotary_frequencies(rot)
    n = 2 * f.numel()
    angle = positions.to(torch.float64)[:, None] * f[None, :]
    cos = (torch.cos(angle) * amplitude).to(x.dtype)[:, None, :]
    sin = (torch.sin(angle) * amplitude).to(x.dtype)[:, None, :]
    u, v = x[..., 0:n:2], x[..., 1:n:2]
    out = x.clone()
    out[..., 0:n:2] = u * cos - v * sin
    out[..., 1:n:2] = v * cos + u * sin
    return out


def sink_softmax(scores: torch.Tensor, sink: torch.Tensor | float | None) -> torch.Tensor:
    """Weights exp(s_j) / (sum_j exp(s_j) + exp(sink)): the sink has no key and no value."""
    if sink is None:
        return torch.softmax(scores, dim=0)
    top = torch.maximum(scores.max(), torch.as_tensor(sink, dtype=scores.dtype))
    e = torch.exp(scores - top)
    return e / (e.sum() + torch.exp(torch.as_tensor(sink, dtype=scores.dtype) - top))


def attention(h, w, prefix, m, first_position=0, past=None, v_first=None):
    """Grouped-query attention, causal, a sink per head, values mixed with another layer's.

    h [T, width].  ``past`` = (keys, values) of the positions before.  ``v_first``: None, or the
    values [T, kv, vdim] that the first value-mixing layer made for the same tokens; then
    v <- (1 - lambda) v + lambda v_first with lambda = the layer's ``vmix``.
    Returns (output [T, width], (keys, values), this layer's own new values before any mixing)."""
    heads, kv, dim, vdim = int(m["heads"]), int(m.get("kv_heads") or m["heads"]), int(m["dim"]), int(m["vdim"])
    t = h.shape[0]
    positions = torch.arange(first_position, first_position + t)
    q = rotate((h @ w[prefix + "q"].T).view(t, heads, dim), positions, m.get("rot"))
    k = rotate((h @ w[prefix + "k"].T).view(t, kv, dim), positions, m.get("rot"))
    v_own = (h @ w[prefix + "v"].T).view(t, kv, vdim)
    v = v_own
    if v_first is not None:
        lam = w[prefix + "vmix"]
        v = (1.0 - lam) * v_own + lam * v_first
    if past is not None:
        k, v = torch.cat([past[0], k]), torch.cat([past[1], v])
    group = heads // kv
    size = int(m["mask"]["size"]) if m.get("mask") else None       # (a window, should a layer of this kind have one)
    out = torch.zeros(t, heads, vdim, dtype=h.dtype)
    for a in range(t):
        i = first_position + a
        seen = [j for j in range(i + 1) if window_visible(i, j, size)]
        for head in range(heads):
            scores = (k[seen, head // group] @ q[a, head]) * float(m["scale"])
            p = sink_softmax(scores, w[prefix + "sink"][head] if prefix + "sink" in w else None)
            out[a, head] = p @ v[seen, head // group]
    return out.reshape(t, heads * vdim) @ w[prefix + "o"].T, (k, v), v_own


def window_visible(i: int, j: int, size: int | None) -> bool:
    return j <= i and (size is None or i - j < size)


def latent_attention(h, w, prefix, m, eps, first_position=0, past=None):
    """Attention whose keys and values are made from a cached latent.

    Of W_dkv h the first kv_rank numbers, RMS-normed with a weight, are the latent c, the last
    rot_dim one rotated key part for all heads.  Head a: key = [W_uk c (its rows), rotated part],
    value = W_uv c (its rows), query = [dim unrotated, rot_dim rotated].  A sliding window, a sink
    per head.  ``past`` = (latents, rotated key parts) of the positions before.
    Returns (output [T, width], (latents, rotated key parts))."""
    heads, dim, rot_dim, vdim, rank = (int(m[k]) for k in ("heads", "dim", "rot_dim", "vdim", "kv_rank"))
    t = h.shape[0]
    positions = torch.arange(first_position, first_position + t)
    q = (h @ w[prefix + "q"].T).view(t, heads, dim + rot_dim)
    q_plain, q_rot = q[..., :dim], rotate(q[..., dim:], positions, m.get("rot"))
    dkv = h @ w[prefix + "dkv"].T
    c = rms(dkv[:, :rank], eps) * w[prefix + "dkv.norm"]
    k_rot = rotate(dkv[:, None, rank:], positions, m.get("rot"))[:, 0]
    if past is not None:
        c, k_rot = torch.cat([past[0], c]), torch.cat([past[1], k_rot])
    keys = (c @ w[prefix + "uk"].T).view(-1, heads, dim)
    values = (c @ w[prefix + "uv"].T).view(-1, heads, vdim)
    size = int(m["mask"]["size"]) if m.get("mask") else None
    out = torch.zeros(t, heads, vdim, dtype=h.dtype)
    for a in range(t):
        i = first_position + a
        seen = [j for j in range(i + 1) if window_visible(i, j, size)]
        for head in range(heads):
            scores = (keys[seen, head] @ q_plain[a, head] + k_rot[seen] @ q_rot[a, head]) * float(m["scale"])
            p = sink_softmax(scores, w[prefix + "sink"][head] if prefix + "sink" in w else None)
            out[a, head] = p @ values[seen, head]
    return out.reshape(t, heads * vdim) @ w[prefix + "o"].T, (c, k_rot)


def dense_ff(h, w, prefix):
    return (gelu_tanh(h @ w[prefix + "gate"].T) * (h @ w[prefix + "up"].T)) @ w[prefix + "down"].T


def routed_experts(h, w, prefix, mlp, margins: list | None = None):
    """Softmax router over all experts; the ``top`` largest scores are chosen and weigh the chosen
    experts' OUTPUTS as they are (not renormalised).  ``margins`` receives, per token, how far the
    last chosen expert's logit lies above the first one left out (infinite if all are chosen)."""
    experts, top = int(mlp["router"]["experts"]), int(mlp["router"]["top"])
    z = h @ w[prefix + "router"].T
    scores = torch.softmax(z, dim=-1)
    out = torch.zeros_like(h)
    for a in range(h.shape[0]):
        order = sorted(range(experts), key=lambda e: (-float(z[a, e]), e))
        if margins is not None:
            margins.append(float(z[a, order[top - 1]] - z[a, order[top]]) if top < experts else math.inf)
        for e in order[:top]:
            base = f"{prefix}e{e}."
            x = h[a]
            y = (silu(w[base + "gate"] @ x) * (w[base + "up"] @ x))
            out[a] += scores[a, e] * (w[base + "down"] @ y)
    return out


def feed_forward(h, w, prefix, mlp, margins=None):
    if mlp is None:
        return torch.zeros_like(h)
    if mlp["kind"] == "dense":
        return dense_ff(h, w, prefix)
    if mlp["kind"] == "moe":
        return routed_experts(h, w, prefix, mlp, margins)
    raise ValueError(mlp["kind"])


def value_mix_source(cfg: dict) -> int | None:
    """Index of the first layer whose mixer says ``v_mix``."""
    for i, L in enumerate(cfg["layers"]):
        if L["type"] == "attention" and L["mixer"].get("v_mix"):
            return i
    return None


def forward(cfg, w, tokens, first_position=0, past=None, layers_out: list | None = None, margins: list | None = None):
    """Logits [T, vocab] of ``tokens`` at positions first_position ...; ``past`` is what an earlier
    call returned for the positions before.  Returns (logits, past).  ``layers_out`` receives the
    residual stream after every layer."""
    eps = float(cfg["norm"]["eps"])
    x = w["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    past = list(past) if past is not None else [None] * len(cfg["layers"])
    source = value_mix_source(cfg)
    v_first = None
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = layer_norm(x, w[p + "norm1"], eps)
        if L["type"] == "attention":
            mixes = bool(L["mixer"].get("v_mix"))
            mixed, past[i], v_own = attention(h, w, p + "mix.", L["mixer"], first_position, past[i],
                                              v_first if mixes and i != source else None)
            if i == source:
                v_first = v_own
        elif L["type"] == "latent_attention":
            mixed, past[i] = latent_attention(h, w, p + "mix.", L["mixer"], eps, first_position, past[i])
        else:
            raise ValueError(L["type"])
        x = x + (mixed + feed_forward(h, w, p + "mlp.", L.get("mlp"), margins))
        if layers_out is not None:
            layers_out.append(x.clone())
    return layer_norm(x, w["final.norm"], eps) @ w["head"].T, past
