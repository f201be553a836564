"""Test-side helpers for the Supinex design: small ``config.json`` dicts written by hand, random
weights under the design's tensor names (listed here independently of the engine), model
folders, and the plain implementation's logits."""

from __future__ import annotations

import json
from pathlib import Path

import torch
from safetensors.torch import save_file

import plain_supinex as plain


def experts(n=4, top=2, ff=32):
    return {"kind": "moe", "router": {"experts": n, "top": top}, "expert": {"ff": ff}}


def dense(ff=48):
    return {"kind": "dense", "ff": ff}


def _rot(dims, base, yarn):
    rot = {"base": base, "dims": dims}
    if yarn is not None:
        rot["scaling"] = dict(zip(("factor", "original", "fast", "slow"), yarn))
    return rot


def attention(heads=4, kv_heads=2, dim=16, vdim=16, rot=8, scale=None, base=10000.0, yarn=None, v_mix=False,
              window=None, mlp="default"):
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
             "scale": float(dim) ** -0.5 if scale is None else scale, "v_mix": v_mix}
    if rot:
        mixer["rot"] = _rot(rot, base, yarn)
    if window is not None:
        mixer["mask"] = {"size": window}
    return {"type": "attention", "mixer": mixer, "mlp": experts() if mlp == "default" else mlp}


def latent(heads=2, dim=16, rot_dim=8, vdim=16, kv_rank=24, window=20, rot="all", scale=None, base=10000.0, yarn=None,
           mlp="default"):
    mixer = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank,
             "scale": float(dim + rot_dim) ** -0.5 if scale is None else scale}
    dims = rot_dim if rot == "all" else rot
    if dims:
        mixer["rot"] = _rot(dims, base, yarn)
    if window is not None:
        mixer["mask"] = {"size": window}
    return {"type": "latent_attention", "mixer": mixer, "mlp": experts() if mlp == "default" else mlp}


def model_json(layers, vocab=200, width=64, eps=1e-5):
    return {"architecture": "Supinex", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": list(layers)}


def tensor_shapes(cfg) -> dict[str, tuple]:
    """Every tensor of a model, by name, written from the design's description."""
    W = cfg["width"]
    out = {"embed": (cfg["vocab"], W), "final.norm": (W,), "head": (cfg["vocab"], W)}
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        out[p + "norm1"] = (W,)
        if L["type"] == "attention":
            kv = m.get("kv_heads") or m["heads"]
            out.update({p + "mix.q": (m["heads"] * m["dim"], W), p + "mix.k": (kv * m["dim"], W),
                        p + "mix.v": (kv * m["vdim"], W), p + "mix.o": (W, m["heads"] * m["vdim"]),
                        p + "mix.sink": (m["heads"],)})
            if m.get("v_mix"):
                out[p + "mix.vmix"] = ()
        else:
            out.update({p + "mix.q": (m["heads"] * (m["dim"] + m["rot_dim"]), W),
                        p + "mix.dkv": (m["kv_rank"] + m["rot_dim"], W), p + "mix.dkv.norm": (m["kv_rank"],),
                        p + "mix.uk": (m["heads"] * m["dim"], m["kv_rank"]), p + "mix.uv": (m["heads"] * m["vdim"], m["kv_rank"]),
                        p + "mix.o": (W, m["heads"] * m["vdim"]), p + "mix.sink": (m["heads"],)})
        mlp = L["mlp"]
        if mlp is None:
            continue
        if mlp["kind"] == "dense":
            out.update({p + "mlp.gate": (mlp["ff"], W), p + "mlp.up": (mlp["ff"], W), p + "mlp.down": (W, mlp["ff"])})
        else:
            ff = mlp["expert"]["ff"]
            out[p + "mlp.router"] = (mlp["router"]["experts"], W)
            for e in range(mlp["router"]["experts"]):
                out.update({p + f"mlp.e{e}.gate": (ff, W), p + f"mlp.e{e}.up": (ff, W), p + f"mlp.e{e}.down": (W, ff)})
    return out


def random_weights(cfg, seed, sink=1.0):
    """name -> float32 tensor holding bfloat16-representable values.  Sinks lie around ``sink`` so that
    leaving them out moves every head's weights; mixing weights lie between 0.2 and 0.8."""
    g = torch.Generator().manual_seed(seed)
    w = {}
    for name, shape in tensor_shapes(cfg).items():
        last = name.rsplit(".", 1)[-1]
        if name in ("final.norm",) or last in ("norm1", "norm"):
            t = 1.0 + 0.2 * torch.randn(shape, generator=g)
        elif last == "sink":
            t = sink + torch.randn(shape, generator=g)
        elif last == "vmix":
            t = 0.2 + 0.6 * torch.rand(shape, generator=g)
        elif name == "embed":
            t = torch.randn(shape, generator=g)
        else:
            gain = 2.0 if last in ("router", "gate", "up") else 1.0
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
    """(logits, per position the narrowest choice of experts in any layer)."""
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
            layer["mlp"]["router"]["top"] = layer["mlp"]["router"]["experts"]
    return out


def tokens(vocab, n, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()
