"""Test-side helpers for the Mepupel design: small ``config.json`` dicts written by hand, random
weights under the design's tensor names (listed here independently of the engine), model
folders, and the plain implementation's logits."""

from __future__ import annotations

import json
from pathlib import Path

import torch
from safetensors.torch import save_file

import plain_mepupel as plain


def experts(n=8, top=2, ff=32, scale=1.5, groups=(4, 2), shared=24):
    router = {"experts": n, "top": top}
    if scale is not None:
        router["scale"] = scale
    if groups is not None:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    out = {"kind": "moe", "router": router, "expert": {"ff": ff}}
    if shared is not None:
        out["shared"] = {"ff": shared}
    return out


def dense(ff=48):
    return {"kind": "dense", "ff": ff}


def mamba(heads=4, vdim=16, state=16, groups=2, conv=4, norm_groups=2, mlp="default"):
    return {"type": "mamba2", "mixer": {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv,
                                        "norm_groups": norm_groups}, "mlp": experts() if mlp == "default" else mlp}


def attention(heads=4, kv_heads=2, dim=16, vdim=16, rot=8, scale=None, base=10000.0, yarn=None, window=24, keep_first=3,
              mlp="default"):
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": float(dim) ** -0.5 if scale is None else scale}
    if rot:
        mixer["rot"] = {"base": base, "dims": rot}
        if yarn is not None:
            mixer["rot"]["scaling"] = dict(zip(("factor", "original", "fast", "slow"), yarn))
    if window is not None:
        mixer["mask"] = {"size": window, "keep_first": keep_first}
    return {"type": "attention", "mixer": mixer, "mlp": experts() if mlp == "default" else mlp}


def latent(heads=2, dim=16, vdim=16, kv_rank=32, q_rank=24, scale=None, kv_from=None, mlp="default"):
    mixer = {"heads": heads, "dim": dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank,
             "scale": float(dim) ** -0.5 if scale is None else scale}
    if kv_from is not None:
        mixer["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": mixer, "mlp": experts() if mlp == "default" else mlp}


def model_json(layers, vocab=200, width=64, eps=1e-5, mult=0.5):
    out = {"architecture": "Mepupel", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": list(layers)}
    if mult is not None:
        out["residual_mult"] = mult
    return out


def tensor_shapes(cfg, correction=True) -> dict[str, tuple]:
    """Every tensor of a model, by name, written from the design's description."""
    W = cfg["width"]
    out = {"embed": (cfg["vocab"], W), "final.norm": (W,), "head": (cfg["vocab"], W)}
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        out[p + "norm1"] = (W,)
        if L["type"] == "mamba2":
            inner, gn = m["heads"] * m["vdim"], m["groups"] * m["state"]
            out.update({p + "mix.in": (2 * inner + 2 * gn + m["heads"], W), p + "mix.conv": (inner + 2 * gn, m["conv"]),
                        p + "mix.conv.b": (inner + 2 * gn,), p + "mix.dt_bias": (m["heads"],), p + "mix.A_log": (m["heads"],),
                        p + "mix.D": (m["heads"],), p + "mix.norm": (inner,), p + "mix.o": (W, inner)})
        elif L["type"] == "attention":
            kv = m.get("kv_heads") or m["heads"]
            out.update({p + "mix.q": (m["heads"] * m["dim"], W), p + "mix.k": (kv * m["dim"], W),
                        p + "mix.v": (kv * m["vdim"], W), p + "mix.o": (W, m["heads"] * m["vdim"])})
        else:
            out.update({p + "mix.dq": (m["q_rank"], W), p + "mix.dq.norm": (m["q_rank"],),
                        p + "mix.uq": (m["heads"] * m["dim"], m["q_rank"]),
                        p + "mix.uk": (m["heads"] * m["dim"], m["kv_rank"]), p + "mix.uv": (m["heads"] * m["vdim"], m["kv_rank"]),
                        p + "mix.o": (W, m["heads"] * m["vdim"])})
            if m.get("kv_from") is None:
                out.update({p + "mix.dkv": (m["kv_rank"], W), p + "mix.dkv.norm": (m["kv_rank"],)})
        mlp = L["mlp"]
        if mlp is None:
            continue
        out[p + "norm2"] = (W,)
        if mlp["kind"] == "dense":
            out.update({p + "mlp.gate": (mlp["ff"], W), p + "mlp.up": (mlp["ff"], W), p + "mlp.down": (W, mlp["ff"]),
                        p + "mlp.gate.b": (mlp["ff"],), p + "mlp.up.b": (mlp["ff"],), p + "mlp.down.b": (W,)})
        else:
            ff = mlp["expert"]["ff"]
            out[p + "mlp.router"] = (mlp["router"]["experts"], W)
            if correction:
                out[p + "mlp.correction"] = (mlp["router"]["experts"],)
            for e in range(mlp["router"]["experts"]):
                out.update({p + f"mlp.e{e}.gate": (ff, W), p + f"mlp.e{e}.up": (ff, W), p + f"mlp.e{e}.down": (W, ff)})
            if mlp.get("shared"):
                s = mlp["shared"]["ff"]
                out.update({p + "mlp.shared.gate": (s, W), p + "mlp.shared.up": (s, W), p + "mlp.shared.down": (W, s)})
    return out


def random_weights(cfg, seed, correction=True):
    """name -> float32 tensor holding bfloat16-representable values.  Biases, corrections and the state
    space's constants are large enough that leaving one out moves the output."""
    g = torch.Generator().manual_seed(seed)
    w = {}
    for name, shape in tensor_shapes(cfg, correction).items():
        last = name.rsplit(".", 1)[-1]
        if name == "final.norm" or last in ("norm1", "norm2", "norm"):
            t = 1.0 + 0.2 * torch.randn(shape, generator=g)
        elif name == "embed":
            t = torch.randn(shape, generator=g)
        elif last == "correction":
            t = 0.3 * torch.randn(shape, generator=g)
        elif last == "b":
            t = 0.5 * torch.randn(shape, generator=g)
        elif last == "dt_bias":
            t = -1.0 + torch.randn(shape, generator=g)
        elif last == "A_log":
            t = -1.0 + 0.7 * torch.randn(shape, generator=g)
        elif last == "D":
            t = 0.5 + 0.5 * torch.randn(shape, generator=g)
        elif last == "conv":
            t = torch.randn(shape, generator=g) * 0.5
        else:
            gain = 2.0 if last in ("router", "gate", "up", "in") else 1.0
            t = torch.randn(shape, generator=g) * gain * shape[1] ** -0.5
        w[name] = t.to(torch.bfloat16).float()
    return w


def write_folder(folder, cfg, weights) -> Path:
    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    (folder / "config.json").write_text(json.dumps(cfg, indent=1))
    save_file({n: t.to(torch.bfloat16).contiguous() for n, t in weights.items()}, str(folder / "model.safetensors"))
    return folder


def double(w):
    return {k: v.double() for k, v in w.items()}


def oracle_logits(cfg, weights, tokens):
    return plain.forward(cfg, double(weights), list(tokens))[0].float().numpy()


def oracle_with_margins(cfg, weights, tokens):
    """(logits, per position the narrowest choice of a router in any layer)."""
    margins: list[float] = []
    logits = plain.forward(cfg, double(weights), list(tokens), margins=margins)[0].float().numpy()
    routed = sum(1 for L in cfg["layers"] if L["mlp"] is not None and L["mlp"]["kind"] == "moe")
    n = len(tokens)
    per_position = [min((margins[layer * n + t] for layer in range(routed)), default=float("inf")) for t in range(n)]
    return logits, per_position


def every_expert(cfg):
    """The same model with every expert chosen for every token: no choice that rounding could turn."""
    out = json.loads(json.dumps(cfg))
    for layer in out["layers"]:
        if layer["mlp"] is not None and layer["mlp"]["kind"] == "moe":
            router = layer["mlp"]["router"]
            router["top"] = router["experts"]
            if "groups" in router:
                router["groups"]["keep"] = router["groups"]["count"]
    return out


def tokens(vocab, n, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()
