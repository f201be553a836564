"""Mepupel: typed config from its ``config.json`` keys, and its model plan.

A decoder-only model whose layers are parallel with a norm each for the two sub-layers over the
same stream: x <- x + m (mixer(norm1(x)) + ff(norm2(x))), m = ``residual_mult``, RMS norms.  The
mixer is, layer by layer, one of three:

* ``mamba2``: a selective state-space mixer (scalar decay per head, a short causal convolution over
  x, B and C, a gate before a grouped RMS norm);
* ``attention``: grouped-query attention, the first ``rot.dims`` dimensions of every head rotated
  in half-split pairs with optionally stretched frequencies, a sliding window that keeps the first
  ``mask.keep_first`` positions of the sequence visible;
* ``latent_attention``: attention without positions over a cached latent; the queries go through a
  normed latent of their own; a layer with ``kv_from``: j has no latent of its own and attends over
  layer j's, with its own up-projections.

The feed-forward is a gated one with biases on every projection, a mixture of small gated experts
(sigmoid scores, a correction for the choice only, groups of experts of which the best are kept,
weights renormalised and scaled, a shared expert), or absent.

    {"architecture": "Mepupel", "vocab": V, "width": W, "norm": {"eps": e}, "residual_mult": m,
     "layers": [{"type": "mamba2",
                 "mixer": {"heads", "vdim", "state", "groups", "conv", "norm_groups"}, "mlp": M},
                {"type": "attention",
                 "mixer": {"heads", "kv_heads", "dim", "vdim", "scale", "mask": {"size", "keep_first"},
                           "rot": {"base", "dims", "scaling": {"factor", "original", "fast", "slow"}}}, "mlp": M},
                {"type": "latent_attention",
                 "mixer": {"heads", "dim", "vdim", "kv_rank", "q_rank", "scale", "kv_from": j}, "mlp": M}, ...]}
    M = {"kind": "dense", "ff": F}
      | {"kind": "moe", "router": {"experts", "top", "scale", "groups": {"count", "keep"}},
         "expert": {"ff"}, "shared": {"ff"}} | null

Tensor names: ``embed``, ``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.mix.{in,conv,conv.b,dt_bias,A_log,D,norm,o}``
or ``l<i>.mix.{q,k,v,o}`` or ``l<i>.mix.{dq,dq.norm,uq,dkv,dkv.norm,uk,uv,o}``, ``l<i>.mlp.{gate,up,down}``
with ``.b`` biases, or ``l<i>.mlp.{router,correction}``, ``l<i>.mlp.e<j>.{gate,up,down}`` and
``l<i>.mlp.shared.{gate,up,down}``, ``final.norm``, ``head``.
"""

from __future__ import annotations

from dataclasses import dataclass, replace
from typing import Any

from tokamak_amd.config.model_config import LayerCall, LayerSpec, ModelPlan, PartSpec, SubPart
from tokamak_amd.config.registry import Architecture, register_architecture

NAME = "Mepupel"
# the design has no position table and no length of its own: the cache is the only limit
MAX_POSITIONS = 1 << 20


@dataclass(frozen=True)
class StretchedFrequencies:
    factor: float
    original: float
    fast: float
    slow: float


@dataclass(frozen=True)
class RotationConfig:
    base: float
    dims: int
    scaling: StretchedFrequencies | None = None


@dataclass(frozen=True)
class StateSpaceConfig:
    heads: int
    vdim: int
    state: int
    groups: int
    conv: int
    norm_groups: int = 1


@dataclass(frozen=True)
class WindowAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot: RotationConfig | None = None     # None: no rotation
    window: int | None = None             # None: every earlier position is seen
    keep_first: int = 0                   # with a window: the first positions that stay visible


@dataclass(frozen=True)
class LatentAttentionConfig:
    heads: int
    dim: int
    vdim: int
    kv_rank: int
    q_rank: int
    scale: float
    kv_from: int | None = None            # the layer whose cached latent this one attends over


@dataclass(frozen=True)
class DenseFeedForward:
    ff: int


@dataclass(frozen=True)
class ExpertsFeedForward:
    experts: int
    top: int
    ff: int
    scale: float = 1.0
    groups: tuple[int, int] | None = None   # (count, keep)
    shared_ff: int | None = None


Mixer = StateSpaceConfig | WindowAttentionConfig | LatentAttentionConfig
KINDS = {StateSpaceConfig: "mamba2", WindowAttentionConfig: "attention", LatentAttentionConfig: "latent_attention"}


@dataclass(frozen=True)
class MepupelLayer:
    mixer: Mixer
    mlp: DenseFeedForward | ExpertsFeedForward | None

    @property
    def type(self) -> str:
        return KINDS[type(self.mixer)]


@dataclass(frozen=True)
class MepupelConfig:
    architecture: str
    vocab_size: int
    width: int
    norm_eps: float
    residual_mult: float
    layers: tuple[MepupelLayer, ...]
    eos_token_ids: tuple[int, ...] = ()
    max_position_embeddings: int = MAX_POSITIONS

    def __post_init__(self) -> None:
        if self.vocab_size < 1 or self.width < 1 or not self.layers:
            raise ValueError("vocab, width and the number of layers must be >= 1")
        for i, layer in enumerate(self.layers):
            m = layer.mixer
            if isinstance(m, StateSpaceConfig):
                if min(m.heads, m.vdim, m.state, m.groups, m.conv, m.norm_groups) < 1:
                    raise ValueError(f"layer {i}: every size must be >= 1")
                if m.heads % m.groups or (m.heads * m.vdim) % m.norm_groups:
                    raise ValueError(f"layer {i}: groups must divide heads, norm_groups must divide heads * vdim")
            elif isinstance(m, WindowAttentionConfig):
                if min(m.heads, m.kv_heads, m.dim, m.vdim) < 1 or m.heads % m.kv_heads:
                    raise ValueError(f"layer {i}: heads ({m.heads}) must be a multiple of kv_heads ({m.kv_heads})")
                if m.window is not None and m.window < 1:
                    raise ValueError(f"layer {i}: mask.size must be >= 1")
                if m.keep_first < 0 or (m.keep_first and m.window is None):
                    raise ValueError(f"layer {i}: mask.keep_first goes with mask.size")
                if m.rot is not None and (m.rot.dims % 2 or not 0 <= m.rot.dims <= m.dim):
                    raise ValueError(f"layer {i}: rot.dims must be even and at most {m.dim}")
            else:
                if min(m.heads, m.dim, m.vdim, m.kv_rank, m.q_rank) < 1:
                    raise ValueError(f"layer {i}: every size must be >= 1")
                if m.kv_from is not None:
                    src = self.layers[m.kv_from].mixer if 0 <= m.kv_from < i else None
                    if not isinstance(src, LatentAttentionConfig) or src.kv_from is not None or src.kv_rank != m.kv_rank:
                        raise ValueError(f"layer {i}: kv_from must name an earlier latent-attention layer with a latent "
                                         f"of its own and the same kv_rank")
            f = layer.mlp
            if isinstance(f, DenseFeedForward) and f.ff < 1:
                raise ValueError(f"layer {i}: ff must be >= 1")
            if isinstance(f, ExpertsFeedForward):
                if f.ff < 1 or not 1 <= f.top <= f.experts or (f.shared_ff is not None and f.shared_ff < 1):
                    raise ValueError(f"layer {i}: ff >= 1 and 1 <= top <= experts are required")
                if f.groups is not None:
                    count, keep = f.groups
                    if count < 1 or f.experts % count or not 1 <= keep <= count or keep * (f.experts // count) < f.top:
                        raise ValueError(f"layer {i}: groups.count must divide the experts, and the kept groups must "
                                         f"hold at least `top` of them")

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


def _mlp(raw: Any, where: str) -> DenseFeedForward | ExpertsFeedForward | None:
    if raw is None:
        return None
    kind = _need(raw, "kind", where)
    if kind == "dense":
        return DenseFeedForward(ff=int(_need(raw, "ff", where)))
    if kind == "moe":
        router = _need(raw, "router", where)
        groups = router.get("groups")
        shared = raw.get("shared")
        return ExpertsFeedForward(
            experts=int(_need(router, "experts", where + ".router")), top=int(_need(router, "top", where + ".router")),
            ff=int(_need(_need(raw, "expert", where), "ff", where + ".expert")),
            scale=float(router["scale"]) if router.get("scale") is not None else 1.0,
            groups=None if groups is None else (int(_need(groups, "count", where + ".router.groups")),
                                                int(_need(groups, "keep", where + ".router.groups"))),
            shared_ff=None if shared is None else int(_need(shared, "ff", where + ".shared")))
    raise ValueError(f"{where}: unknown feed-forward kind {kind!r}; this design has 'dense' and 'moe'")


def _rot(raw: Any, where: str) -> RotationConfig | None:
    if raw is None:
        return None
    scaling = raw.get("scaling")
    if scaling is not None:
        scaling = StretchedFrequencies(*(float(_need(scaling, k, where + ".scaling")) for k in ("factor", "original", "fast", "slow")))
    return RotationConfig(base=float(_need(raw, "base", where)), dims=int(_need(raw, "dims", where)), scaling=scaling)


def _layer(raw: Any, i: int) -> MepupelLayer:
    where = f"layers[{i}]"
    kind = _need(raw, "type", where)
    m = _need(raw, "mixer", where)
    mw = where + ".mixer"
    if kind == "mamba2":
        mixer: Mixer = StateSpaceConfig(
            heads=int(_need(m, "heads", mw)), vdim=int(_need(m, "vdim", mw)), state=int(_need(m, "state", mw)),
            groups=int(m["groups"]) if m.get("groups") is not None else 1, conv=int(_need(m, "conv", mw)),
            norm_groups=int(m["norm_groups"]) if m.get("norm_groups") is not None else 1)
    elif kind == "attention":
        heads = int(_need(m, "heads", mw))
        dim = int(_need(m, "dim", mw))
        mask = m.get("mask")
        mixer = WindowAttentionConfig(
            heads=heads, kv_heads=int(m["kv_heads"]) if m.get("kv_heads") is not None else heads, dim=dim,
            vdim=int(m["vdim"]) if m.get("vdim") is not None else dim, scale=float(_need(m, "scale", mw)),
            rot=_rot(m.get("rot"), mw + ".rot"),
            window=None if mask is None else int(_need(mask, "size", mw + ".mask")),
            keep_first=0 if mask is None or mask.get("keep_first") is None else int(mask["keep_first"]))
    elif kind == "latent_attention":
        dim = int(_need(m, "dim", mw))
        mixer = LatentAttentionConfig(
            heads=int(_need(m, "heads", mw)), dim=dim, vdim=int(m["vdim"]) if m.get("vdim") is not None else dim,
            kv_rank=int(_need(m, "kv_rank", mw)), q_rank=int(_need(m, "q_rank", mw)), scale=float(_need(m, "scale", mw)),
            kv_from=None if m.get("kv_from") is None else int(m["kv_from"]))
    else:
        raise ValueError(f"{where}: unknown layer type {kind!r}; this design has 'mamba2', 'attention' and 'latent_attention'")
    return MepupelLayer(mixer=mixer, mlp=_mlp(raw.get("mlp"), where + ".mlp"))


def parse(raw: dict[str, Any], eos_token_ids: tuple[int, ...] = ()) -> MepupelConfig:
    name = raw.get("architecture")
    if name != NAME:
        raise ValueError(f"Unsupported architecture {name!r}; supported: {NAME}")
    layers = _need(raw, "layers", "config.json")
    return MepupelConfig(
        architecture=NAME,
        vocab_size=int(_need(raw, "vocab", "config.json")),
        width=int(_need(raw, "width", "config.json")),
        norm_eps=float(_need(_need(raw, "norm", "config.json"), "eps", "norm")),
        residual_mult=float(raw["residual_mult"]) if raw.get("residual_mult") is not None else 1.0,
        layers=tuple(_layer(layer, i) for i, layer in enumerate(layers)),
        eos_token_ids=tuple(int(t) for t in eos_token_ids),
    )


def _mixer_json(m: Mixer) -> dict[str, Any]:
    if isinstance(m, StateSpaceConfig):
        return {"heads": m.heads, "vdim": m.vdim, "state": m.state, "groups": m.groups, "conv": m.conv,
                "norm_groups": m.norm_groups}
    if isinstance(m, WindowAttentionConfig):
        out: dict[str, Any] = {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim, "scale": m.scale}
        if m.window is not None:
            out["mask"] = {"size": m.window, "keep_first": m.keep_first}
        if m.rot is not None:
            out["rot"] = {"base": m.rot.base, "dims": m.rot.dims}
            if m.rot.scaling is not None:
                s = m.rot.scaling
                out["rot"]["scaling"] = {"factor": s.factor, "original": s.original, "fast": s.fast, "slow": s.slow}
        return out
    out = {"heads": m.heads, "dim": m.dim, "vdim": m.vdim, "kv_rank": m.kv_rank, "q_rank": m.q_rank, "scale": m.scale}
    if m.kv_from is not None:
        out["kv_from"] = m.kv_from
    return out


def _mlp_json(mlp: DenseFeedForward | ExpertsFeedForward | None) -> dict[str, Any] | None:
    if mlp is None:
        return None
    if isinstance(mlp, DenseFeedForward):
        return {"kind": "dense", "ff": mlp.ff}
    router: dict[str, Any] = {"experts": mlp.experts, "top": mlp.top, "scale": mlp.scale}
    if mlp.groups is not None:
        router["groups"] = {"count": mlp.groups[0], "keep": mlp.groups[1]}
    out: dict[str, Any] = {"kind": "moe", "router": router, "expert": {"ff": mlp.ff}}
    if mlp.shared_ff is not None:
        out["shared"] = {"ff": mlp.shared_ff}
    return out


def to_config_json(cfg: MepupelConfig) -> dict[str, Any]:
    """The ``config.json`` dict that parses back to ``cfg``."""
    return {
        "architecture": cfg.architecture,
        "vocab": cfg.vocab_size,
        "width": cfg.width,
        "norm": {"eps": cfg.norm_eps},
        "residual_mult": cfg.residual_mult,
        "layers": [{"type": L.type, "mixer": _mixer_json(L.mixer), "mlp": _mlp_json(L.mlp)} for L in cfg.layers],
    }


def run_order(cfg: MepupelConfig) -> tuple[LayerCall, ...]:
    """Each layer once; a latent-attention layer with ``kv_from`` reads the cache slot of the layer it
    names and writes none."""
    return tuple(
        LayerCall(i, L.mixer.kv_from, writes_cache=False)
        if isinstance(L.mixer, LatentAttentionConfig) and L.mixer.kv_from is not None else LayerCall(i, i)
        for i, L in enumerate(cfg.layers))


def plan(cfg: MepupelConfig) -> ModelPlan:
    width = cfg.width
    norm = PartSpec.of("rmsnorm", dim=width, eps=cfg.norm_eps, tensor="")
    layers = []
    for L in cfg.layers:
        m = L.mixer
        parts = dict(norm=SubPart("norm", norm, "norm1"))
        if isinstance(m, StateSpaceConfig):
            parts["mixer"] = SubPart("mixer", PartSpec.of(
                "selective_state_space", hidden_size=width, num_heads=m.heads, value_dim=m.vdim, state_size=m.state,
                groups=m.groups, conv_taps=m.conv, norm_groups=m.norm_groups, norm_eps=cfg.norm_eps), "mix.")
        elif isinstance(m, WindowAttentionConfig):
            parts["mixer"] = SubPart("mixer", PartSpec.of(
                "rotated_unit_attention", hidden_size=width, num_heads=m.heads, num_kv_heads=m.kv_heads, head_dim=m.dim,
                value_dim=m.vdim, softmax_scale=m.scale, norm_eps=None, chunk=None, window=m.window,
                keep_first=m.keep_first), "mix.")
            if m.rot is not None and m.rot.dims > 0:
                s = m.rot.scaling
                parts["position"] = SubPart("position", PartSpec.of(
                    "rotary_half", rotary_dim=m.rot.dims, theta=m.rot.base,
                    yarn=None if s is None else (s.factor, s.original, s.fast, s.slow)), shared=True)
        else:
            parts["mixer"] = SubPart("mixer", PartSpec.of(
                "latent_attention", hidden_size=width, num_heads=m.heads, head_dim=m.dim, rot_dim=0, value_dim=m.vdim,
                rank=m.kv_rank, softmax_scale=m.scale, norm_eps=cfg.norm_eps, window=None, sink=False, q_rank=m.q_rank,
                own_latent=m.kv_from is None), "mix.")
        if isinstance(L.mlp, DenseFeedForward):
            parts["feed_forward"] = SubPart("feed_forward", PartSpec.of(
                "swiglu", hidden_size=width, intermediate_size=L.mlp.ff, names=("gate", "up", "down"), bias_suffix=".b"), "mlp.")
        elif isinstance(L.mlp, ExpertsFeedForward):
            f = L.mlp
            parts["feed_forward"] = SubPart("feed_forward", PartSpec.of(
                "routed_experts", hidden_size=width, intermediate_size=f.ff, num_experts=f.experts, top=f.top,
                weight_on="output", scoring="sigmoid", correction="correction", groups=f.groups, normalise=True,
                weight_scale=f.scale, shared_size=f.shared_ff), "mlp.")
        if L.mlp is not None:
            parts["feed_forward_norm"] = SubPart("norm", norm, "norm2")
        layers.append(LayerSpec.of(PartSpec.of("parallel_sublayers", branch_scale=cfg.residual_mult), **parts))
    return ModelPlan(
        vocab_size=cfg.vocab_size,
        hidden_size=width,
        max_position_embeddings=cfg.max_position_embeddings,
        tie_word_embeddings=False,
        embedding=PartSpec.of("token_embedding", vocab_size=cfg.vocab_size, dim=width, tensor=""),
        layers=tuple(layers),
        order=run_order(cfg),
        final_norm=norm,
        head=PartSpec.of("linear_head", vocab_size=cfg.vocab_size, dim=width, tied=False, tensor=""),
        embedding_prefix="embed",
        layer_prefix="l{}.",
        final_norm_prefix="final.norm",
        head_prefix="head",
        eos_token_ids=cfg.eos_token_ids,
    )


def _shape(vocab, width, repeats, *, ssm_heads, ssm_vdim, state, groups, att_heads, att_kv, att_dim, rot_dims, window,
           keep_first, lat_heads, lat_dim, kv_rank, q_rank, ff, experts, top, expert_ff, expert_groups, shared_ff,
           norm_groups=1) -> MepupelConfig:
    """``repeats`` times (latent attention, state space, window attention, latent attention over the first
    one's latent of the same stretch, state space, window attention); the model's first feed-forward is
    dense, the others are mixtures of experts."""
    ssm = StateSpaceConfig(ssm_heads, ssm_vdim, state, groups, 4, norm_groups)
    att = WindowAttentionConfig(att_heads, att_kv, att_dim, att_dim, float(att_dim) ** -0.5,
                                RotationConfig(1e6, rot_dims, StretchedFrequencies(8.0, 4096.0, 32.0, 1.0)), window, keep_first)
    moe = ExpertsFeedForward(experts, top, expert_ff, 1.5, expert_groups, shared_ff)
    layers: list[MepupelLayer] = []
    for r in range(repeats):
        lat = LatentAttentionConfig(lat_heads, lat_dim, lat_dim, kv_rank, q_rank, float(lat_dim) ** -0.5)
        first = len(layers)
        layers += [MepupelLayer(lat, DenseFeedForward(ff) if r == 0 else moe), MepupelLayer(ssm, moe), MepupelLayer(att, moe),
                   MepupelLayer(replace(lat, kv_from=first), moe), MepupelLayer(ssm, moe), MepupelLayer(att, moe)]
    return MepupelConfig(NAME, vocab, width, 1e-5, 0.5, tuple(layers))


# Shapes for the random-weights mode (sizes only; no trained weights exist here): a tiny one, and
# layers of the widths of 0.6B- and 8B-class models for measurements (a token's experts together with
# the shared one are about as wide as the dense feed-forward of that class).
PRESETS = {
    "mepupel-tiny": _shape(256, 64, 1, ssm_heads=4, ssm_vdim=16, state=16, groups=2, att_heads=4, att_kv=2, att_dim=16,
                           rot_dims=8, window=24, keep_first=3, lat_heads=2, lat_dim=16, kv_rank=32, q_rank=24, ff=96,
                           experts=8, top=2, expert_ff=32, expert_groups=(4, 2), shared_ff=32, norm_groups=2),
    "mepupel-0.6b": _shape(151936, 1024, 5, ssm_heads=32, ssm_vdim=64, state=128, groups=1, att_heads=16, att_kv=8,
                           att_dim=128, rot_dims=64, window=1024, keep_first=4, lat_heads=16, lat_dim=64, kv_rank=256,
                           q_rank=384, ff=3072, experts=16, top=2, expert_ff=1024, expert_groups=(4, 2), shared_ff=1024),
    "mepupel-8b": _shape(151936, 4096, 6, ssm_heads=128, ssm_vdim=64, state=128, groups=8, att_heads=32, att_kv=8,
                         att_dim=128, rot_dims=64, window=1024, keep_first=4, lat_heads=32, lat_dim=128, kv_rank=512,
                         q_rank=1024, ff=12288, experts=16, top=2, expert_ff=4096, expert_groups=(4, 2), shared_ff=4096),
}


def shorten(cfg: MepupelConfig, num_layers: int) -> MepupelConfig:
    """The model's first ``num_layers`` layers (a layer whose latent's source is cut off cannot stay: the
    stretches are six layers long and the source is a stretch's first)."""
    return replace(cfg, layers=cfg.layers[:num_layers])


register_architecture(Architecture(name=NAME, parse=parse, plan=plan, to_json=to_config_json, presets=PRESETS,
                                   shorten=shorten))
