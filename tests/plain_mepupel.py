"""A plain, slow implementation of the Mepupel design, written from its equations: one function
per mechanism, whole sequences at a time, no cache, no kernels, nothing shared with the engine.

``cfg`` is the parsed ``config.json`` (a dict), ``w`` maps tensor names to torch tensors.  Everything
is computed in the dtype of ``DTYPE`` (float64 by default).
"""

from __future__ import annotations

import math

import torch

DTYPE = torch.float64


def _f(t: torch.Tensor) -> torch.Tensor:
    return t.to(DTYPE)


def rms_norm(x: torch.Tensor, weight: torch.Tensor | None, eps: float) -> torch.Tensor:
    y = x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)
    return y if weight is None else y * _f(weight)


def silu(x: torch.Tensor) -> torch.Tensor:
    return x / (1.0 + torch.exp(-x))


def softplus(x: torch.Tensor) -> torch.Tensor:
    return torch.where(x > 30.0, x, torch.log1p(torch.exp(torch.clamp(x, max=30.0))))


# ---------------------------------------------------------------------------------------------
# positions
def stretched_frequencies(dims: int, base: float, scaling: dict | None) -> tuple[list[float], float]:
    """(frequency of pair i for i < dims / 2, amplitude of cos and sin)."""
    freqs = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    if not scaling:
        return freqs, 1.0
    factor, original = float(scaling["factor"]), float(scaling["original"])

    def where(turns: float) -> float:
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(where(float(scaling["fast"]))), 0)
    hi = min(math.ceil(where(float(scaling["slow"]))), dims - 1)
    out = []
    for i, f in enumerate(freqs):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(f / factor * ramp + f * (1.0 - ramp))
    return out, 0.1 * math.log(factor) + 1.0


def rotate(x: torch.Tensor, positions: torch.Tensor, rot: dict | None) -> torch.Tensor:
    """x [T, heads, dim]; the first rot.dims dimensions rotated, dimension i paired with i + dims / 2."""
    if not rot or not rot.get("dims"):
        return x
    dims = int(rot["dims"])
    half = dims // 2
    freqs, amp = stretched_frequencies(dims, float(rot["base"]), rot.get("scaling"))
    angle = positions.to(DTYPE)[:, None] * torch.tensor(freqs, dtype=DTYPE)[None, :]      # [T, half]
    cos, sin = (torch.cos(angle) * amp)[:, None, :], (torch.sin(angle) * amp)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * cos - v * sin, v * cos + u * sin, x[..., dims:]], dim=-1)


# ---------------------------------------------------------------------------------------------
# mixers
def visible(i: int, j: int, mask: dict | None) -> bool:
    if j > i:
        return False
    if not mask:
        return True
    return i - j < int(mask["size"]) or j < int(mask.get("keep_first", 0))


def softmax_attention(q, k, v, scale: float, mask: dict | None) -> torch.Tensor:
    """q [T, H, d], k [T, G, d], v [T, G, dv] -> [T, H, dv]; query head a reads kv head a // (H / G)."""
    t, heads, _ = q.shape
    per = heads // k.shape[1]
    allowed = torch.tensor([[visible(i, j, mask) for j in range(t)] for i in range(t)])
    out = torch.zeros((t, heads, v.shape[-1]), dtype=DTYPE)
    for a in range(heads):
        g = a // per
        scores = (q[:, a, :] @ k[:, g, :].T) * scale
        scores = scores.masked_fill(~allowed, float("-inf"))
        out[:, a, :] = torch.softmax(scores, dim=-1) @ v[:, g, :]
    return out


def attention(h: torch.Tensor, w: dict, p: str, m: dict) -> torch.Tensor:
    t = h.shape[0]
    heads, kv = int(m["heads"]), int(m.get("kv_heads") or m["heads"])
    dim, vdim = int(m["dim"]), int(m["vdim"])
    pos = torch.arange(t)
    q = rotate((h @ _f(w[p + "q"]).T).view(t, heads, dim), pos, m.get("rot"))
    k = rotate((h @ _f(w[p + "k"]).T).view(t, kv, dim), pos, m.get("rot"))
    v = (h @ _f(w[p + "v"]).T).view(t, kv, vdim)
    o = softmax_attention(q, k, v, float(m["scale"]), m.get("mask"))
    return o.reshape(t, heads * vdim) @ _f(w[p + "o"]).T


def latent(h: torch.Tensor, w: dict, p: str, eps: float) -> torch.Tensor:
    """The cached latent of a latent-attention layer: [T, kv_rank]."""
    return rms_norm(h @ _f(w[p + "dkv"]).T, w[p + "dkv.norm"], eps)


def latent_attention(h: torch.Tensor, c: torch.Tensor, w: dict, p: str, m: dict, eps: float) -> torch.Tensor:
    """``c``: the latent this layer attends over (its own, or the one of the layer it names)."""
    t = h.shape[0]
    heads, dim, vdim = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    cq = rms_norm(h @ _f(w[p + "dq"]).T, w[p + "dq.norm"], eps)
    q = (cq @ _f(w[p + "uq"]).T).view(t, heads, dim)
    k = (c @ _f(w[p + "uk"]).T).view(t, heads, dim)
    v = (c @ _f(w[p + "uv"]).T).view(t, heads, vdim)
    o = softmax_attention(q, k, v, float(m["scale"]), None)
    return o.reshape(t, heads * vdim) @ _f(w[p + "o"]).T


def causal_conv(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor) -> torch.Tensor:
    """x [T, C], weight [C, taps] whose last column meets the current token, zeros before the start."""
    t, taps = x.shape[0], weight.shape[1]
    padded = torch.cat([torch.zeros((taps - 1, x.shape[1]), dtype=DTYPE), x], dim=0)
    out = _f(bias)[None, :].expand(t, -1).clone()
    for j in range(taps):
        out = out + padded[j:j + t, :] * _f(weight)[:, j][None, :]
    return out


def mamba2(h: torch.Tensor, w: dict, p: str, m: dict, eps: float, return_state: bool = False):
    t = h.shape[0]
    heads, vdim, n, groups = int(m["heads"]), int(m["vdim"]), int(m["state"]), int(m["groups"])
    parts = int(m.get("norm_groups", 1))
    inner = heads * vdim
    proj = h @ _f(w[p + "in"]).T
    z, xbc, dt = proj[:, :inner], proj[:, inner:2 * inner + 2 * groups * n], proj[:, 2 * inner + 2 * groups * n:]
    xbc = silu(causal_conv(xbc, w[p + "conv"], w[p + "conv.b"]))
    x = xbc[:, :inner].view(t, heads, vdim)
    b = xbc[:, inner:inner + groups * n].view(t, groups, n)
    c = xbc[:, inner + groups * n:].view(t, groups, n)
    dt = softplus(dt + _f(w[p + "dt_bias"])[None, :])                  # [T, heads]
    decay = torch.exp(-torch.exp(_f(w[p + "A_log"]))[None, :] * dt)    # [T, heads]
    skip = _f(w[p + "D"])
    per = heads // groups
    state = torch.zeros((heads, n, vdim), dtype=DTYPE)
    y = torch.zeros((t, heads, vdim), dtype=DTYPE)
    for i in range(t):
        for a in range(heads):
            g = a // per
            state[a] = decay[i, a] * state[a] + dt[i, a] * torch.outer(b[i, g], x[i, a])
            y[i, a] = state[a].T @ c[i, g] + skip[a] * x[i, a]
    y = y.reshape(t, inner) * silu(z)
    y = rms_norm(y.view(t, parts, inner // parts), None, eps).reshape(t, inner) * _f(w[p + "norm"])
    out = y @ _f(w[p + "o"]).T
    return (out, state) if return_state else out


# ---------------------------------------------------------------------------------------------
# feed-forwards
def gated(h: torch.Tensor, w: dict, p: str, biases: bool) -> torch.Tensor:
    g, u = h @ _f(w[p + "gate"]).T, h @ _f(w[p + "up"]).T
    if biases:
        g, u = g + _f(w[p + "gate.b"]), u + _f(w[p + "up.b"])
    out = (silu(g) * u) @ _f(w[p + "down"]).T
    return out + _f(w[p + "down.b"]) if biases else out


def route(h: torch.Tensor, w: dict, p: str, router: dict, margins: list | None = None) -> tuple[torch.Tensor, torch.Tensor]:
    """(chosen experts [T, top], their weights [T, top]).  ``margins`` receives, per token, the narrowest
    gap of a choice score (of a group or of an expert) between what was taken and what was not."""
    experts, top = int(router["experts"]), int(router["top"])
    gap = torch.full((h.shape[0],), float("inf"), dtype=DTYPE)
    s = torch.sigmoid(h @ _f(w[p + "router"]).T)
    choice = s + _f(w[p + "correction"])[None, :] if p + "correction" in w else s.clone()
    groups = router.get("groups")
    if groups:
        count, keep = int(groups["count"]), int(groups["keep"])
        size = experts // count
        grouped = choice.view(-1, count, size)
        score = grouped.topk(min(2, size), dim=-1).values.sum(dim=-1)          # [T, count]
        if keep < count:
            ordered = score.sort(dim=-1, descending=True).values
            gap = torch.minimum(gap, ordered[:, keep - 1] - ordered[:, keep])
        kept = torch.zeros_like(score, dtype=torch.bool)
        kept.scatter_(1, score.topk(keep, dim=-1).indices, True)
        choice = choice.masked_fill(~kept[:, :, None].expand(-1, -1, size).reshape(-1, experts), float("-inf"))
    chosen = choice.topk(top, dim=-1).indices
    if top < experts:
        ordered = choice.sort(dim=-1, descending=True).values
        gap = torch.minimum(gap, ordered[:, top - 1] - ordered[:, top])     # (inf where nothing else may be chosen)
    if margins is not None:
        margins.extend(gap.tolist())
    weight = s.gather(1, chosen)
    weight = weight / (weight.sum(dim=-1, keepdim=True) + 1e-20) * float(router.get("scale", 1.0))
    return chosen, weight


def experts_ff(h: torch.Tensor, w: dict, p: str, mlp: dict, margins: list | None = None) -> torch.Tensor:
    chosen, weight = route(h, w, p, mlp["router"], margins)
    out = torch.zeros_like(h)
    for i in range(h.shape[0]):
        for e, x in zip(chosen[i].tolist(), weight[i]):
            out[i] += x * gated(h[i:i + 1], w, f"{p}e{e}.", False)[0]
    if mlp.get("shared"):
        out = out + gated(h, w, p + "shared.", False)
    return out


def feed_forward(h: torch.Tensor, w: dict, p: str, mlp: dict | None, margins: list | None = None) -> torch.Tensor | None:
    if mlp is None:
        return None
    if mlp["kind"] == "dense":
        return gated(h, w, p, True)
    return experts_ff(h, w, p, mlp, margins)


# ---------------------------------------------------------------------------------------------
def forward(cfg: dict, w: dict, tokens: list[int], margins: list | None = None) -> tuple[torch.Tensor, torch.Tensor]:
    """(logits [T, vocab], the residual stream after every layer [layers, T, width]).  ``margins`` receives the
    routers' narrowest choices, T numbers for every layer with a mixture of experts, in layer order."""
    eps = float(cfg["norm"]["eps"])
    mult = float(cfg.get("residual_mult", 1.0))
    x = _f(w["embed"])[torch.tensor(tokens, dtype=torch.long)]
    latents: dict[int, torch.Tensor] = {}
    after = []
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        h = rms_norm(x, w[p + "norm1"], eps)
        if layer["type"] == "mamba2":
            mixed = mamba2(h, w, p + "mix.", m, eps)
        elif layer["type"] == "attention":
            mixed = attention(h, w, p + "mix.", m)
        elif layer["type"] == "latent_attention":
            if m.get("kv_from") is None:
                latents[i] = latent(h, w, p + "mix.", eps)
                c = latents[i]
            else:
                c = latents[int(m["kv_from"])]
            mixed = latent_attention(h, c, w, p + "mix.", m, eps)
        else:
            raise ValueError(layer["type"])
        if layer.get("mlp") is not None:
            mixed = mixed + feed_forward(rms_norm(x, w[p + "norm2"], eps), w, p + "mlp.", layer["mlp"], margins)
        x = x + mult * mixed
        after.append(x)
    logits = rms_norm(x, w["final.norm"], eps) @ _f(w["head"]).T
    return logits, torch.stack(after)
