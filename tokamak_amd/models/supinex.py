"""Supinex: typed config from its ``config.json`` keys, and its model plan.

A decoder-only model whose layers are parallel: one layer norm (a weight, no bias) whose output
both the mixer and the feed-forward read, x <- x + (mixer(h) + ff(h)).  The mixer is, layer by
layer, grouped-query attention (causal, partial interleaved rotary positions, a learned sink per
head in the softmax's denominator, values optionally mixed with those of the first such layer) or
attention over a cached latent (a low-rank latent and one rotated key part per token, keys and
values made from the latent per head; a sliding window, a sink, frequencies stretched for long
contexts).  The feed-forward is a gated one with the tanh form of gelu, a mixture of small SiLU-gated
experts with a softmax router whose scores weigh the chosen experts' outputs, or absent.

    {"architecture": "Supinex", "vocab": V, "width": W, "norm": {"eps": e},
     "layers": [{"type": "attention",
                 "mixer": {"heads", "kv_heads", "dim", "vdim", "scale", "v_mix": bool,
                           "rot": {"base", "dims", "scaling": {"factor", "original", "fast", "slow"}},
                           "mask": {"size"}},
                 "mlp": M},
                {"type": "latent_attention",
                 "mixer": {"heads", "dim", "rot_dim", "vdim", "kv_rank", "scale", "mask": {"size"},
                           "rot": {"base", "dims", "scaling": {...}}},
                 "mlp": M}, ...]}
    M = {"kind": "dense", "ff": F} | {"kind": "moe", "router": {"experts", "top"}, "expert": {"ff"}} | null

Tensor names: ``embed``, ``l<i>.norm1``, ``l<i>.mix.{q,k,v,o,sink,vmix}`` or
``l<i>.mix.{q,dkv,dkv.norm,uk,uv,o,sink}``, ``l<i>.mlp.{gate,up,down}`` or ``l<i>.mlp.router`` and
``l<i>.mlp.e<j>.{gate,up,down}``, ``final.norm``, ``head``.
"""

from __future__ import annotations

from dataclasses import dataclass, replace
from typing import Any

from tokamak_amd.config.model_config import LayerSpec, ModelPlan, PartSpec, SubPart, default_order
from tokamak_amd.config.registry import Architecture, register_architecture

NAME = "Supinex"
# the design has no position table and no length of its own: the cache is the only limit
MAX_POSITIONS = 1 << 20


@dataclass(frozen=True)
class YarnScaling:
    factor: float
    original: float
    fast: float
    slow: float


@dataclass(frozen=True)
class RotaryConfig:
    base: float
    dims: int
    scaling: YarnScaling | None = None


@dataclass(frozen=True)
class AttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot: RotaryConfig | None = None     # None: no rotation
    window: int | None = None           # None: every earlier position is seen
    v_mix: bool = False


@dataclass(frozen=True)
class LatentConfig:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    scale: float
    rot: RotaryConfig | None = None
    window: int | None = None


@dataclass(frozen=True)
class DenseConfig:
    ff: int


@dataclass(frozen=True)
class ExpertsConfig:
    experts: int
    top: int
    ff: int


@dataclass(frozen=True)
class SupinexLayer:
    mixer: AttentionConfig | LatentConfig
    mlp: DenseConfig | ExpertsConfig | None     # None: the layer has no feed-forward

    @property
    def type(self) -> str:
        return "attention" if isinstance(self.mixer, AttentionConfig) else "latent_attention"


@dataclass(frozen=True)
class SupinexConfig:
    architecture: str
    vocab_size: int
    width: int
    norm_eps: float
    layers: tuple[SupinexLayer, ...]
    eos_token_ids: tuple[int, ...] = ()
    max_position_embeddings: int = MAX_POSITIONS

    def __post_init__(self) -> None:
        if self.vocab_size < 1 or self.width < 1 or not self.layers:
            raise ValueError("vocab, width and the number of layers must be >= 1")
        mixing = None
        for i, layer in enumerate(self.layers):
            m = layer.mixer
            if min(m.heads, m.dim, m.vdim) < 1:
                raise ValueError(f"layer {i}: every size must be >= 1")
            if m.window is not None and m.window < 1:
                raise ValueError(f"layer {i}: mask.size must be >= 1")
            rotated = m.dim if isinstance(m, AttentionConfig) else m.rot_dim
            if m.rot is not None and (m.rot.dims % 2 or not 0 <= m.rot.dims <= rotated):
                raise ValueError(f"layer {i}: rot.dims must be even and at most {rotated}")
            if isinstance(m, AttentionConfig):
                if m.kv_heads < 1 or m.heads % m.kv_heads:
                    raise ValueError(f"layer {i}: heads ({m.heads}) must be a multiple of kv_heads ({m.kv_heads})")
                if m.v_mix:
                    if mixing is not None and mixing != (m.kv_heads, m.vdim):
                        raise ValueError(f"layer {i}: layers that mix values need equal kv_heads and vdim")
                    mixing = (m.kv_heads, m.vdim)
            elif m.kv_rank < 1 or m.rot_dim < 0:
                raise ValueError(f"layer {i}: kv_rank >= 1 and rot_dim >= 0 are required")
            if isinstance(layer.mlp, ExpertsConfig) and (layer.mlp.ff < 1 or not 1 <= layer.mlp.top <= layer.mlp.experts):
                raise ValueError(f"layer {i}: ff >= 1 and 1 <= top <= experts are required")
            if isinstance(layer.mlp, DenseConfig) and layer.mlp.ff < 1:
                raise ValueError(f"layer {i}: ff must be >= 1")

    @property
    def hidden_size(self) -> int:
        return self.width

    @property
    def num_layers(self) -> int:
        return len(self.layers)


def _need(raw: Any, key: str, where: str) -> Any:
    if not isinstance(raw, dict) or key not in raw or raw[key] is None:
        raise ValueError(f"config.json lacks required key {key!r} in {where}")
    return raw[key]


def _mlp(raw: Any, where: str) -> DenseConfig | ExpertsConfig | None:
    if raw is None:
        return None
    kind = _need(raw, "kind", where)
    if kind == "dense":
        return DenseConfig(ff=int(_need(raw, "ff", where)))
    if kind == "moe":
        router = _need(raw, "router", where)
        return ExpertsConfig(experts=int(_need(router, "experts", where + ".router")),
                             top=int(_need(router, "top", where + ".router")),
                             ff=int(_need(_need(raw, "expert", where), "ff", where + ".expert")))
    raise ValueError(f"{where}: unknown feed-forward kind {kind!r}; this design has 'dense' and 'moe'")


def _rot(raw: Any, where: str) -> RotaryConfig | None:
    if raw is None:
        return None
    scaling = raw.get("scaling")
    if scaling is not None:
        scaling = YarnScaling(*(float(_need(scaling, k, where + ".scaling")) for k in ("factor", "original", "fast", "slow")))
    return RotaryConfig(base=float(_need(raw, "base", where)), dims=int(_need(raw, "dims", where)), scaling=scaling)


def _window(m: dict, where: str) -> int | None:
    mask = m.get("mask")
    return None if mask is None else int(_need(mask, "size", where + ".mask"))


def _layer(raw: Any, i: int) -> SupinexLayer:
    where = f"layers[{i}]"
    kind = _need(raw, "type", where)
    m = _need(raw, "mixer", where)
    mw = where + ".mixer"
    if kind == "attention":
        heads = int(_need(m, "heads", mw))
        mixer: AttentionConfig | LatentConfig = AttentionConfig(
            heads=heads, kv_heads=int(m["kv_heads"]) if m.get("kv_heads") is not None else heads,
            dim=int(_need(m, "dim", mw)), vdim=int(_need(m, "vdim", mw)), scale=float(_need(m, "scale", mw)),
            rot=_rot(m.get("rot"), mw + ".rot"), window=_window(m, mw), v_mix=bool(m.get("v_mix", False)))
    elif kind == "latent_attention":
        mixer = LatentConfig(
            heads=int(_need(m, "heads", mw)), dim=int(_need(m, "dim", mw)), rot_dim=int(_need(m, "rot_dim", mw)),
            vdim=int(_need(m, "vdim", mw)), kv_rank=int(_need(m, "kv_rank", mw)), scale=float(_need(m, "scale", mw)),
            rot=_rot(m.get("rot"), mw + ".rot"), window=_window(m, mw))
    else:
        raise ValueError(f"{where}: unknown layer type {kind!r}; this design has 'attention' and 'latent_attention'")
    return SupinexLayer(mixer=mixer, mlp=_mlp(raw.get("mlp"), where + ".mlp"))


def parse(raw: dict[str, Any], eos_token_ids: tuple[int, ...] = ()) -> SupinexConfig:
    name = raw.get("architecture")
    if name != NAME:
        raise ValueError(f"Unsupported architecture {name!r}; supported: {NAME}")
    layers = _need(raw, "layers", "config.json")
    return SupinexConfig(
        architecture=NAME,
        vocab_size=int(_need(raw, "vocab", "config.json")),
        width=int(_need(raw, "width", "config.json")),
        norm_eps=float(_need(_need(raw, "norm", "config.json"), "eps", "norm")),
        layers=tuple(_layer(layer, i) for i, layer in enumerate(layers)),
        eos_token_ids=tuple(int(t) for t in eos_token_ids),
    )


def _rot_json(rot: RotaryConfig | None) -> dict[str, Any] | None:
    if rot is None:
        return None
    out: dict[str, Any] = {"base": rot.base, "dims": rot.dims}
    if rot.scaling is not None:
        s = rot.scaling
        out["scaling"] = {"factor": s.factor, "original": s.original, "fast": s.fast, "slow": s.slow}
    return out


def _mixer_json(m: AttentionConfig | LatentConfig) -> dict[str, Any]:
    if isinstance(m, AttentionConfig):
        out: dict[str, Any] = {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim, "scale": m.scale,
                               "v_mix": m.v_mix}
    else:
        out = {"heads": m.heads, "dim": m.dim, "rot_dim": m.rot_dim, "vdim": m.vdim, "kv_rank": m.kv_rank, "scale": m.scale}
    if m.rot is not None:
        out["rot"] = _rot_json(m.rot)
    if m.window is not None:
        out["mask"] = {"size": m.window}
    return out


def _mlp_json(mlp: DenseConfig | ExpertsConfig | None) -> dict[str, Any] | None:
    if mlp is None:
        return None
    if isinstance(mlp, DenseConfig):
        return {"kind": "dense", "ff": mlp.ff}
    return {"kind": "moe", "router": {"experts": mlp.experts, "top": mlp.top}, "expert": {"ff": mlp.ff}}


def to_config_json(cfg: SupinexConfig) -> dict[str, Any]:
    """The ``config.json`` dict that parses back to ``cfg``."""
    return {
        "architecture": cfg.architecture,
        "vocab": cfg.vocab_size,
        "width": cfg.width,
        "norm": {"eps": cfg.norm_eps},
        "layers": [{"type": L.type, "mixer": _mixer_json(L.mixer), "mlp": _mlp_json(L.mlp)} for L in cfg.layers],
    }


def _position(rot: RotaryConfig | None) -> SubPart | None:
    if rot is None or rot.dims == 0:
        return None
    s = rot.scaling
    return SubPart("position", PartSpec.of(
        "rotary_interleaved", rotary_dim=rot.dims, theta=rot.base,
        yarn=None if s is None else (s.factor, s.original, s.fast, s.slow)), shared=True)


def plan(cfg: SupinexConfig) -> ModelPlan:
    width = cfg.width
    norm = PartSpec.of("layernorm", dim=width, eps=cfg.norm_eps, tensor="")
    # the first layer that mixes values is the others' source
    source = next((i for i, L in enumerate(cfg.layers) if isinstance(L.mixer, AttentionConfig) and L.mixer.v_mix), None)
    layers = []
    for i, L in enumerate(cfg.layers):
        m = L.mixer
        parts = dict(norm=SubPart("norm", norm, "norm1"))
        if isinstance(m, AttentionConfig):
            parts["mixer"] = SubPart("mixer", PartSpec.of(
                "rotated_unit_attention", hidden_size=width, num_heads=m.heads, num_kv_heads=m.kv_heads, head_dim=m.dim,
                value_dim=m.vdim, softmax_scale=m.scale, norm_eps=None, chunk=None, window=m.window, sink=True,
                value_mix=None if not m.v_mix else "source" if i == source else "mix"), "mix.")
        else:
            parts["mixer"] = SubPart("mixer", PartSpec.of(
                "latent_attention", hidden_size=width, num_heads=m.heads, head_dim=m.dim, rot_dim=m.rot_dim,
                value_dim=m.vdim, rank=m.kv_rank, softmax_scale=m.scale, norm_eps=cfg.norm_eps, window=m.window,
                sink=True), "mix.")
        position = _position(m.rot)
        if position is not None:
            parts["position"] = position
        if isinstance(L.mlp, DenseConfig):
            parts["feed_forward"] = SubPart("feed_forward", PartSpec.of(
                "swiglu", hidden_size=width, intermediate_size=L.mlp.ff, names=("gate", "up", "down"),
                activation="gelu_tanh"), "mlp.")
        elif isinstance(L.mlp, ExpertsConfig):
            parts["feed_forward"] = SubPart("feed_forward", PartSpec.of(
                "routed_experts", hidden_size=width, intermediate_size=L.mlp.ff, num_experts=L.mlp.experts,
                top=L.mlp.top, weight_on="output", scoring="softmax"), "mlp.")
        layers.append(LayerSpec.of(PartSpec.of("parallel_sublayers"), **parts))
    return ModelPlan(
        vocab_size=cfg.vocab_size,
        hidden_size=width,
        max_position_embeddings=cfg.max_position_embeddings,
        tie_word_embeddings=False,
        embedding=PartSpec.of("token_embedding", vocab_size=cfg.vocab_size, dim=width, tensor=""),
        layers=tuple(layers),
        order=default_order(len(layers)),
        final_norm=norm,
        head=PartSpec.of("linear_head", vocab_size=cfg.vocab_size, dim=width, tied=False, tensor=""),
        embedding_prefix="embed",
        layer_prefix="l{}.",
        final_norm_prefix="final.norm",
        head_prefix="head",
        eos_token_ids=cfg.eos_token_ids,
    )


def _shape(vocab, width, pairs, *, heads, kv, dim, latent_heads, latent_dim, rot_dim, rank, window, ff, experts, top,
           expert_ff) -> SupinexConfig:
    """``pairs`` times an attention layer followed by a latent-attention layer; the first layer's
    feed-forward is dense, the others are mixtures of experts."""
    att = AttentionConfig(heads, kv, dim, dim, float(dim) ** -0.5, RotaryConfig(5e5, dim // 2), None, True)
    lat = LatentConfig(latent_heads, latent_dim, rot_dim, latent_dim, rank, float(latent_dim + rot_dim) ** -0.5,
                       RotaryConfig(1e4, rot_dim, YarnScaling(8.0, 4096.0, 24.0, 2.0)), window)
    moe = ExpertsConfig(experts, top, expert_ff)
    layers = [SupinexLayer(att, DenseConfig(ff)), SupinexLayer(lat, moe)] + [SupinexLayer(att, moe), SupinexLayer(lat, moe)] * (pairs - 1)
    return SupinexConfig(NAME, vocab, width, 1e-5, tuple(layers))


# Shapes for the random-weights mode (sizes only; no trained weights exist here): a tiny one, and
# layers of the widths of 0.6B- and 8B-class models for measurements (a token's experts together are
# as wide as the dense feed-forward of that class; the cached key of the latent layers, latent and
# rotated part, fills the 512 channels the attention kernels take).
PRESETS = {
    "supinex-tiny": _shape(256, 64, 2, heads=4, kv=2, dim=16, latent_heads=2, latent_dim=16, rot_dim=8, rank=24,
                           window=40, ff=96, experts=4, top=2, expert_ff=32),
    "supinex-0.6b": _shape(151936, 1024, 14, heads=16, kv=8, dim=128, latent_heads=16, latent_dim=64, rot_dim=32,
                           rank=224, window=1024, ff=3072, experts=16, top=2, expert_ff=1536),
    "supinex-8b": _shape(151936, 4096, 18, heads=32, kv=8, dim=128, latent_heads=32, latent_dim=128, rot_dim=64,
                         rank=448, window=1024, ff=12288, experts=16, top=2, expert_ff=6144),
}


def shorten(cfg: SupinexConfig, num_layers: int) -> SupinexConfig:
    return replace(cfg, layers=cfg.layers[:num_layers])


register_architecture(Architecture(name=NAME, parse=parse, plan=plan, to_json=to_config_json, presets=PRESETS,
                                   shorten=shorten))
