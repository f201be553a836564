"""The Supinex design in the engine against the plain implementation (plain_supinex.py): each
mechanism alone, then whole models of several small shapes through the step function: whole
prompts, tails one by one, portions down to two tokens, mixed batches with pages and state slots
used again, window edges with sharp attention, a far key among hundreds, long decoding through
recorded steps, greedy generation through ``LLM.generate``, and the trace runner.

float32 runs compare every row.  In bfloat16 a choice between two experts whose logits lie within
rounding of each other may fall the other way than in the plain implementation; so a bfloat16 run
compares a request's rows up to the first position where the plain implementation's choice was
that narrow, and every row of the same models with all experts chosen for every token."""

import json
import subprocess
import sys
from pathlib import Path

import numpy as np
import pytest
import torch

import plain_supinex as plain
from kernel_util import make_batch, pack_pages_whole
from replay_util import mixed, portions, tail_one_by_one, whole
from rorosun_util import run_steps
from supinex_util import (attention, dense, double, every_expert, experts, latent, model_json, oracle_logits,
                          oracle_with_margins, random_weights, tokens, write_folder)

pytestmark = pytest.mark.gpu
DEV = "cuda"
ROOT = Path(__file__).resolve().parent.parent
REL = {torch.float32: 3e-5, torch.bfloat16: 2.5e-2}
LIMIT = {"float32": 2e-4, "bfloat16": 1e-1}
NARROW = 0.15      # a choice of experts that bfloat16 rounding may turn (distance of the router's logits)
BOTH = pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])


def close(got, want, dtype, slack=1.0):
    err = float((got - want).abs().max() / want.abs().max())
    assert err <= REL[dtype] * slack, err


def row_errors(steps, got, expected):
    cursor = {rid: 0 for rid in expected}
    out = []
    for rec in steps:
        row = 0
        for e in rec["entries"]:
            start = cursor[e["id"]]
            for w in e.get("want", []):
                want = expected[e["id"]][start + w]
                err = float(np.abs(got[rec["step"]][row] - want).max() / max(1e-6, np.abs(want).max()))
                out.append((err if err == err else float("inf"), (rec["step"], e["id"], start + w, len(e["tokens"]))))
                row += 1
            cursor[e["id"]] = start + len(e["tokens"])
    return out


def check_rows(steps, got, expected, dtype, what="", margins=None):
    errors = row_errors(steps, got, expected)
    if dtype == "bfloat16" and margins is not None:
        sure = {rid: next((i for i, m in enumerate(ms) if m < NARROW), len(ms)) for rid, ms in margins.items()}
        errors = [(e, where) for e, where in errors if where[2] < sure[where[1]]]
    over = [(e, where) for e, where in errors if not e <= LIMIT[dtype]]
    assert not over, (what, dtype, len(over), len(errors), sorted(over)[-1])
    return len(errors)


def fetcher(tensors, dtype):
    def fetch(name):
        t = tensors[name]
        held = dtype if t.dim() == 2 and not name.endswith("router") else torch.float32
        return t.to(DEV, held).contiguous()
    return fetch


def summed(out):
    return (out.sum(0) if out.dim() == 3 else out).float().cpu()


def fresh_store(part, page, pages, dtype, fill):
    from tokamak_amd.engine.storage import SlotStore

    return SlotStore(0, page, {name: torch.full((pages, array.elems_per_token * page), fill, dtype=dtype, device=DEV)
                               for name, array in part.cache_request().arrays})


# -- mechanisms alone -------------------------------------------------------------
@BOTH
@pytest.mark.parametrize("width", [64, 50, 328, 4100])
def test_layer_norm_adds_both_branches_once(dtype, width):
    """x + (a + b) with a in the compute dtype and b as float32 partial sums, the stream written back;
    rows picked by index leave the stream alone; a norm without anything to add."""
    from tokamak_amd.config import get_part
    from tokamak_amd.parts.base import BranchPair

    g = torch.Generator().manual_seed(width)
    n = 9
    weight = 1.0 + 0.3 * torch.randn(width, generator=g)
    part = get_part("norm", "layernorm")(dim=width, eps=1e-5, tensor="", dtype=dtype, device=DEV)
    part.bind("n", lambda name: weight.to(DEV))
    x = 3.0 + 2.0 * torch.randn(n, width, generator=g)         # (a mean far from zero: the centring shows)
    a = torch.randn(n, width, generator=g).to(dtype)
    b = torch.randn(3, n, width, generator=g)
    total = x.double() + (a.double() + b.double().sum(0))
    resid = x.to(DEV)
    out = part.forward(resid, BranchPair(a.to(DEV), b.to(DEV)))
    close(out.float().cpu(), plain.layer_norm(total, weight.double(), 1e-5).float(), dtype)
    assert torch.allclose(resid.cpu().double(), total, atol=1e-5)
    rows = torch.tensor([7, 0, 7, 3], dtype=torch.int32, device=DEV)
    before = resid.clone()
    picked = part.forward(resid, BranchPair(a.to(DEV), None), rows=rows, write_resid=False)
    want = plain.layer_norm(total + a.double(), weight.double(), 1e-5)[rows.cpu().long()]
    close(picked.float().cpu(), want.float(), dtype)
    assert torch.equal(resid, before)
    close(part.forward(resid, None).float().cpu(), plain.layer_norm(total, weight.double(), 1e-5).float(), dtype)
    # the same kernel without the centring is the RMS norm of the two branches' sum
    rms = get_part("norm", "rmsnorm")(dim=width, eps=1e-5, tensor="", dtype=dtype, device=DEV)
    rms.bind("n", lambda name: weight.to(DEV))
    resid = x.to(DEV)
    got = rms.forward(resid, BranchPair(b.to(DEV), a.to(DEV)))
    close(got.float().cpu(), (plain.rms(total, 1e-5) * weight.double()).float(), dtype)


@pytest.mark.parametrize("rot", [dict(base=10000.0, dims=16), dict(base=5e4, dims=24, scaling=dict(factor=4.0, original=64, fast=8.0, slow=1.0))])
def test_interleaved_rotary_tables(rot):
    from tokamak_amd.config import get_part

    s = rot.get("scaling")
    part = get_part("position", "rotary_interleaved")(
        rotary_dim=rot["dims"], theta=rot["base"], dtype=torch.float32, device=DEV,
        yarn=None if s is None else (s["factor"], s["original"], s["fast"], s["slow"]))
    batch = make_batch([(5, 0, [0]), (3, 1000, list(range(70))), (1, 41, [1, 2, 3])])
    data = part.prepare(batch)
    assert data.interleaved and data.rotary_dim == rot["dims"]
    f, amplitude = plain.rotary_frequencies(rot)
    positions = torch.tensor([0, 1, 2, 3, 4, 1000, 1001, 1002, 41], dtype=torch.float64)
    angle = positions[:, None] * f.float().double()[None, :]
    assert torch.allclose(data.cos.cpu().double(), torch.cos(angle) * amplitude, atol=2e-4)   # float32 angles at position 1,000
    assert torch.allclose(data.sin.cpu().double(), torch.sin(angle) * amplitude, atol=2e-4)
    assert torch.allclose(data.cos[:5].cpu().double(), (torch.cos(angle) * amplitude)[:5], atol=1e-6)


ATTENTIONS = {
    "g2": dict(heads=4, kv_heads=2, dim=16, vdim=16, rot=8),
    "g3-yarn": dict(heads=3, kv_heads=1, dim=24, vdim=48, rot=24, yarn=(4.0, 32.0, 8.0, 1.0)),
    "norot-window": dict(heads=2, kv_heads=2, dim=40, vdim=16, rot=0, window=33),
    "wide": dict(heads=8, kv_heads=2, dim=128, vdim=128, rot=64, base=1e5),
    "mid": dict(heads=4, kv_heads=1, dim=64, vdim=64, rot=64),
    "pad": dict(heads=3, kv_heads=1, dim=20, vdim=36, rot=10, window=50),
    "tiny": dict(heads=2, kv_heads=2, dim=6, vdim=2, rot=6),
    "g9": dict(heads=18, kv_heads=2, dim=24, vdim=32, rot=8),
}


def attention_part(m, width, dtype, value_mix=None):
    from tokamak_amd.config import get_part

    part = get_part("mixer", "rotated_unit_attention")(
        hidden_size=width, num_heads=m["heads"], num_kv_heads=m["kv_heads"], head_dim=m["dim"], value_dim=m["vdim"],
        softmax_scale=m["scale"], norm_eps=None, chunk=None, window=(m.get("mask") or {}).get("size"), sink=True,
        value_mix=value_mix, dtype=dtype, device=DEV)
    position = None
    if m.get("rot"):
        s = m["rot"].get("scaling")
        position = get_part("position", "rotary_interleaved")(
            rotary_dim=m["rot"]["dims"], theta=m["rot"]["base"], dtype=dtype, device=DEV,
            yarn=None if s is None else (s["factor"], s["original"], s["fast"], s["slow"]))
    return part, position


@BOTH
@pytest.mark.parametrize("name", list(ATTENTIONS))
def test_sink_attention_alone_with_mixed_values(dtype, name):
    """Two layers over the same tokens, the second mixing the first one's values into its own: a
    portion from position zero, one that ends inside a page, two tokens, then single tokens; pages
    scattered.  Heads of 64 and 128 with pages of 16 run on the tuned matrix-core kernels in bfloat16, other
    sizes with pages of 16 on the ones that take any size (nine heads a kv head: single tokens too)."""
    a = ATTENTIONS[name]
    width = 64
    page = 16 if a["dim"] >= 64 or name in ("g9", "pad") else 8
    cfg = model_json([attention(**a, v_mix=True), attention(**a, v_mix=True)], width=width)
    m = cfg["layers"][0]["mixer"]
    w = random_weights(cfg, seed=a["dim"])
    T = 150
    g = torch.Generator().manual_seed(2)
    h0, h1 = torch.randn(T, width, generator=g).to(dtype), torch.randn(T, width, generator=g).to(dtype)
    want0, _, v_first = plain.attention(h0.double(), double(w), "l0.mix.", m)
    want1, _, _ = plain.attention(h1.double(), double(w), "l1.mix.", m, v_first=v_first)
    # the sinks and the mixing matter: without them the outputs move by far more than the tolerance
    no_sink = {k: v for k, v in double(w).items() if not k.endswith("sink")}
    assert float((plain.attention(h0.double(), no_sink, "l0.mix.", m)[0] - want0).abs().max() / want0.abs().max()) > 0.05
    assert float((plain.attention(h1.double(), double(w), "l1.mix.", m)[0] - want1).abs().max() / want1.abs().max()) > 0.05
    parts = []
    for i, mix in enumerate(("source", "mix")):
        part, position = attention_part(m, width, dtype, mix)
        assert set(part.expected_tensors(f"l{i}.mix.")) == {n for n in w if n.startswith(f"l{i}.mix.")}
        part.bind(f"l{i}.mix.", fetcher(w, dtype))
        padded = (part.key_size, part.value_size) != (m["dim"], m["vdim"])
        parts.append((part, position, fresh_store(part, page, 40, dtype, 0.0 if padded else float("nan"))))
    table = [(7 * i + 3) % 40 for i in range(-(-T // page))]
    got0, got1, at = [], [], 0
    for n in [37, 30, 2] + [1] * (T - 69):
        batch = make_batch([(n, at, table)])
        for (part, position, store), h, got in ((parts[0], h0, got0), (parts[1], h1, got1)):
            data = None if position is None else position.prepare(batch)
            got.append(summed(part.forward(h[at:at + n].to(DEV), batch, store, True, data)))
        at += n
    close(torch.cat(got0), want0.float(), dtype)
    close(torch.cat(got1), want1.float(), dtype)


@pytest.mark.parametrize("nh,nkv,hd", [(8, 2, 128), (4, 4, 64), (6, 2, 64)])
def test_sinks_in_every_form_of_the_matrix_core_kernels(nh, nkv, hd):
    """Decode tokens whose keys are split over blocks and merged, tiles of 16 with and without split
    keys, tiles of 32 in the wide and the group form: the sink is added once, where a row's sums
    are complete."""
    from tokamak_amd.kernels import ops

    ps, T = 16, 1400
    g = torch.Generator().manual_seed(nh * hd)
    k, v = torch.randn(T, nkv, hd, generator=g), torch.randn(T, nkv, hd, generator=g)
    pages = -(-T // ps)
    table = torch.randperm(pages, generator=g).tolist()
    kc = torch.zeros(pages, nkv * hd * ps, dtype=torch.bfloat16)
    vc = torch.zeros_like(kc)
    pack_pages_whole(kc, vc, k, v, table, ps)
    kc, vc = kc.to(DEV), vc.to(DEV)
    sinks = (8.0 + torch.randn(nh, generator=g)).to(DEV)      # (as heavy as a thousand keys together)
    scale = hd ** -0.5
    kd, vd = k.bfloat16().double(), v.bfloat16().double()

    def reference(q, positions):
        out = torch.zeros(len(positions), nh, hd, dtype=torch.float64)
        for i, p in enumerate(positions):
            for a in range(nh):
                s = (kd[: p + 1, a // (nh // nkv)] @ q[i, a].double()) * scale
                out[i, a] = plain.sink_softmax(s, sinks[a].double().cpu()) @ vd[: p + 1, a // (nh // nkv)]
        return out

    def run(mode, spans, **kw):
        batch = make_batch(spans)
        n = batch.num_tokens
        q = torch.randn(n, nh, hd, generator=g).bfloat16()
        out = torch.full((n, nh * hd), float("nan"), dtype=torch.bfloat16, device=DEV)
        lists = {"heads": ("single", None, "num_single"), "tokens": ("tile_first", "tile_count", "num_tiles"),
                 "tokens_wide": ("wide_first", "wide_count", "num_wide"), "tokens_group": ("wide_first", "wide_count", "num_wide")}[mode]
        count = batch.lists["attention." + lists[1]] if lists[1] else None
        assert ops.attention_mfma(mode, q.to(DEV).view(n, -1), kc, vc, batch.block_tables[0], batch.positions, batch.req_of_token,
                                  batch.lists["attention." + lists[0]], count, batch.facts["attention." + lists[2]], out,
                                  num_heads=nh, num_kv_heads=nkv, head_dim=hd, page_size=ps, scale=scale, sinks=sinks, **kw)
        positions = [c + i for n_, c, _ in spans for i in range(n_)]
        want = reference(q, positions)
        plain_softmax = torch.stack([torch.stack([torch.softmax((kd[: p + 1, a // (nh // nkv)] @ q[i, a].double()) * scale, 0)
                                                  @ vd[: p + 1, a // (nh // nkv)] for a in range(nh)]) for i, p in enumerate(positions[:2])])
        assert float((plain_softmax - want[:2]).abs().max()) > 0.02        # (the sink is no small term here)
        close(out.float().cpu().view(n, nh, hd), want.float(), torch.bfloat16)

    run("heads", [(1, 1399, table), (1, 700, table)], split_keys=1536)      # (one split that holds every key)
    run("heads", [(1, 1399, table), (1, 5, table)], split_keys=512, num_splits=3)
    run("tokens", [(40, 1300, table)], split_keys=1536)
    run("tokens", [(20, 1300, table)], split_keys=512, num_splits=3)
    run("tokens_wide", [(64, 1200, table)])
    run("tokens_group", [(64, 1200, table)])


LATENTS = {
    "base": dict(heads=2, dim=16, rot_dim=8, vdim=16, kv_rank=24, window=20),
    "odd": dict(heads=3, dim=20, rot_dim=12, vdim=36, kv_rank=45, window=33, rot=6, yarn=(4.0, 32.0, 8.0, 1.0)),
    "one-head": dict(heads=1, dim=8, rot_dim=4, vdim=8, kv_rank=16, window=1),
    "no-window": dict(heads=5, dim=32, rot_dim=16, vdim=24, kv_rank=80, window=None, base=1e5),
    "no-rot": dict(heads=2, dim=16, rot_dim=8, vdim=8, kv_rank=12, window=64, rot=0),
    "big": dict(heads=4, dim=64, rot_dim=32, vdim=64, kv_rank=160, window=100),
    "many-heads": dict(heads=20, dim=16, rot_dim=8, vdim=16, kv_rank=40, window=70),
}


@BOTH
@pytest.mark.parametrize("name", list(LATENTS))
def test_latent_attention_alone(dtype, name):
    """Scattered pages, portions that end inside a page and inside a window, then single tokens; a
    window one position longer or shorter moves the output by far more than the tolerance."""
    from tokamak_amd.config import get_part

    a = LATENTS[name]
    width, eps, page = 64, 1e-5, 16 if name in ("big", "many-heads", "odd") else 8
    cfg = model_json([latent(**a)], width=width, eps=eps)
    m = cfg["layers"][0]["mixer"]
    w = random_weights(cfg, seed=a["kv_rank"])
    part = get_part("mixer", "latent_attention")(
        hidden_size=width, num_heads=m["heads"], head_dim=m["dim"], rot_dim=m["rot_dim"], value_dim=m["vdim"],
        rank=m["kv_rank"], softmax_scale=m["scale"], norm_eps=eps, window=a["window"], sink=True, dtype=dtype, device=DEV)
    assert set(part.expected_tensors("l0.mix.")) == {n for n in w if n.startswith("l0.mix.")}
    part.bind("l0.mix.", fetcher(w, dtype))
    position = None
    if m.get("rot"):
        s = m["rot"].get("scaling")
        position = get_part("position", "rotary_interleaved")(
            rotary_dim=m["rot"]["dims"], theta=m["rot"]["base"], dtype=dtype, device=DEV,
            yarn=None if s is None else (s["factor"], s["original"], s["fast"], s["slow"]))
    T = 150
    h = torch.randn(T, width, generator=torch.Generator().manual_seed(4)).to(dtype)
    want = plain.latent_attention(h.double(), double(w), "l0.mix.", m, eps)[0].float()
    if a["window"] not in (None,):
        for size in (a["window"] + 1, max(1, a["window"] - 1)):
            if size != a["window"]:
                near = plain.latent_attention(h.double(), double(w), "l0.mix.", dict(m, mask={"size": size}), eps)[0].float()
                assert float((near - want).abs().max() / want.abs().max()) > 0.02
    # only the latent and the rotated key part are cached: one key/value head, whatever the heads
    request = dict(part.cache_request().arrays)
    assert request["k"].elems_per_token == -(-(m["kv_rank"] + m["rot_dim"]) // 8) * 8
    assert request["v"].elems_per_token == -(-m["kv_rank"] // 16) * 16 and part.cache_request().window == a["window"]
    padded = (part.key_size, part.value_size) != (m["kv_rank"] + m["rot_dim"], m["kv_rank"])
    store = fresh_store(part, page, 40, dtype, 0.0 if padded else float("nan"))
    table = [(7 * i + 3) % 40 for i in range(-(-T // page))]
    got, at = [], 0
    for n in [37, 30, 2] + [1] * (T - 69):
        batch = make_batch([(n, at, table)])
        data = None if position is None else position.prepare(batch)
        got.append(summed(part.forward(h[at:at + n].to(DEV), batch, store, True, data)))
        at += n
    close(torch.cat(got), want, dtype, slack=2.0 if dtype == torch.bfloat16 else 1.0)


@BOTH
@pytest.mark.parametrize("n,heads,m,k", [(1, 3, 20, 45), (37, 2, 64, 16), (200, 5, 130, 70), (64, 4, 448, 128)])
def test_per_head_product_with_strides(dtype, n, heads, m, k):
    from tokamak_amd.kernels import ops

    g = torch.Generator().manual_seed(n + m)
    x = torch.randn(n, heads, k + 8, generator=g).to(dtype)
    w = (torch.randn(heads, m, k, generator=g) * k ** -0.5).to(dtype)
    out = torch.full((n, heads, m + 5), float("nan"), dtype=dtype, device=DEV)
    ops.head_linear(x.to(DEV)[:, :, :k], w.to(DEV), out[:, :, 2:2 + m])
    want = torch.einsum("nhk,hmk->nhm", x[:, :, :k].double(), w.double()).float()
    close(out[:, :, 2:2 + m].float().cpu(), want, dtype)
    assert torch.isnan(out[:, :, :2]).all() and torch.isnan(out[:, :, 2 + m:]).all()


@BOTH
@pytest.mark.parametrize("rows,width,ff", [(5, 64, 48), (70, 72, 40), (300, 256, 136)])
def test_dense_feed_forward_with_the_tanh_gelu(dtype, rows, width, ff):
    from tokamak_amd.config import get_part

    cfg = model_json([attention(mlp=dense(ff))], width=width)
    w = random_weights(cfg, seed=ff)
    part = get_part("feed_forward", "swiglu")(hidden_size=width, intermediate_size=ff, names=("gate", "up", "down"),
                                              activation="gelu_tanh", dtype=dtype, device=DEV)
    part.bind("l0.mlp.", fetcher(w, dtype))
    h = (2.0 * torch.randn(rows, width, generator=torch.Generator().manual_seed(1))).to(dtype)
    want = plain.dense_ff(h.double(), double(w), "l0.mlp.").float()
    silu = (plain.silu(h.double() @ double(w)["l0.mlp.gate"].T) * (h.double() @ double(w)["l0.mlp.up"].T)) @ double(w)["l0.mlp.down"].T
    assert float((silu.float() - want).abs().max() / want.abs().max()) > 0.01      # (another gate would show)
    close(summed(part.forward(h.to(DEV), None)), want, dtype)


def clear_of(h, w, top, n):
    """Rows whose choice of experts no rounding turns."""
    z = h.double() @ w["l0.mlp.router"].double().T
    s = torch.sort(z, dim=-1, descending=True).values
    return torch.ones(h.shape[0], dtype=torch.bool) if top == n else (s[:, top - 1] - s[:, top]) > NARROW


@BOTH
@pytest.mark.parametrize("width,ff,n,top", [(64, 32, 4, 2), (48, 24, 12, 1), (72, 40, 5, 5), (36, 20, 7, 3), (256, 136, 3, 2)])
def test_routed_experts_with_softmax_scores_on_the_outputs(dtype, width, ff, n, top):
    """Few tokens (a block a pair) and many (grouped on the matrix cores in bfloat16); the weights are the
    softmax's scores over ALL experts, not renormalised, and act on the experts' outputs."""
    from tokamak_amd.config import get_part

    cfg = model_json([attention(mlp=experts(n, top, ff))], width=width)
    w = random_weights(cfg, seed=width + top)
    part = get_part("feed_forward", "routed_experts")(hidden_size=width, intermediate_size=ff, num_experts=n, top=top,
                                                      weight_on="output", scoring="softmax", dtype=dtype, device=DEV)
    part.bind("l0.mlp.", fetcher(w, dtype))
    for rows in (3, 200):
        h = (2.0 * torch.randn(rows, width, generator=torch.Generator().manual_seed(rows))).to(dtype)
        want = plain.routed_experts(h.double(), double(w), "l0.mlp.", cfg["layers"][0]["mlp"]).float()
        got = summed(part.forward(h.to(DEV), None))
        keep = clear_of(h, w, top, n)
        assert int(keep.sum()) >= rows // 2
        close(got[keep], want[keep], dtype)
    if top < n:
        # renormalised weights, or weights on the input, would be another function
        z = torch.softmax(h.double() @ double(w)["l0.mlp.router"].T, -1)
        assert float(torch.sort(z, -1, descending=True).values[:, :top].sum(-1).min()) < 0.95


# -- whole models -------------------------------------------------------------------
SHAPES = {
    "base": dict(cfg=model_json([attention(v_mix=True, mlp=dense(40)), latent(), attention(v_mix=True), latent(heads=9, window=150, mlp=dense(24)),
                                 attention(v_mix=True, rot=16)]), page=16),
    "odd": dict(cfg=model_json([latent(heads=3, dim=20, rot_dim=12, vdim=36, kv_rank=45, window=7, rot=6, yarn=(4.0, 32.0, 8.0, 1.0),
                                       mlp=experts(5, 1, 24)),
                                attention(heads=3, kv_heads=3, dim=20, vdim=40, rot=12, yarn=(2.0, 16.0, 4.0, 1.0), mlp=None),
                                attention(heads=6, kv_heads=2, dim=8, vdim=16, rot=8, v_mix=True, window=19, mlp=experts(3, 3, 40)),
                                attention(heads=2, kv_heads=2, dim=24, vdim=16, rot=0, v_mix=True, mlp=dense(50))],
                               vocab=131, width=72, eps=1e-6), page=8),
    "ones": dict(cfg=model_json([attention(heads=5, kv_heads=1, dim=8, vdim=16, rot=2, mlp=experts(7, 2, 16)),
                                 latent(heads=1, dim=8, rot_dim=2, vdim=8, kv_rank=16, window=1, mlp=None),
                                 latent(heads=4, dim=16, rot_dim=16, vdim=32, kv_rank=40, window=None, mlp=experts(2, 1, 48)),
                                 attention(heads=2, kv_heads=1, dim=64, vdim=64, rot=32, v_mix=True, window=64, mlp=dense(16))],
                                vocab=97, width=40, eps=1e-4), page=16),
}


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    root = tmp_path_factory.mktemp("supinex")
    out = {}
    for name, spec in SHAPES.items():
        w = random_weights(spec["cfg"], seed=len(name))
        out[name] = (write_folder(root / name, spec["cfg"], w), spec["cfg"], w, spec["page"])
        all_cfg = every_expert(spec["cfg"])
        out[name + "-all"] = (write_folder(root / (name + "-all"), all_cfg, w), all_cfg, w, spec["page"])
    return out


def runner_for(models, name, dtype, pool_tokens=1024, max_requests=4, **kw):
    from tokamak_amd.engine.runner import ModelRunner

    folder, cfg, w, page = models[name]
    return ModelRunner.from_folder(folder, dtype=dtype, page_size=page, kv_pool_tokens=pool_tokens,
                                   max_requests=max_requests, **kw), cfg, w


LENGTHS = [1, 2, 23, 61, 150]


def requests_for(cfg, seed=0):
    return {f"r{i}": tokens(cfg["vocab"], n, 100 * seed + i) for i, n in enumerate(LENGTHS)}


def expected_and_margins(cfg, w, requests):
    both = {rid: oracle_with_margins(cfg, w, toks) for rid, toks in requests.items()}
    return {rid: b[0] for rid, b in both.items()}, {rid: b[1] for rid, b in both.items()}


@pytest.fixture(scope="module")
def oracle(models):
    out = {}
    for name, (folder, cfg, w, page) in models.items():
        for seed in (0, 1):
            requests = requests_for(cfg, seed)
            if seed == 1:
                requests.update({f"s{i}": tokens(cfg["vocab"], n, 900 + i) for i, n in enumerate([40, 64, 17])})
            out[name, seed] = (requests, *expected_and_margins(cfg, w, requests))
    return out


ALL_SHAPES = [n + tail for n in SHAPES for tail in ("", "-all")]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ALL_SHAPES)
def test_every_cutting(models, oracle, name, dtype):
    """Whole prompts; most of a prompt and its tail token by token (prefill against decoding through
    the cache); portions of 16 down to 2 tokens."""
    runner, cfg, w = runner_for(models, name, dtype)
    requests, expected, margins = oracle[name, 0]
    checked = 0
    for steps in [whole(requests)] + [f(rid, toks) for rid, toks in requests.items() for f in (tail_one_by_one, portions)]:
        checked += check_rows(steps, run_steps(runner, steps), expected, dtype, name, margins)
    assert checked >= (3 * sum(LENGTHS) if name.endswith("-all") or dtype == "float32" else 3)
    runner.manager.check()
    assert runner.manager.num_free_pages() == runner.manager.num_pages()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ALL_SHAPES)
def test_mixed_batches_with_pages_and_slots_used_again(models, oracle, name, dtype):
    """Up to four live requests, portions beside single tokens, requests left out of steps; eight
    requests over four state slots and a pool that only holds what is live."""
    requests, expected, margins = oracle[name, 1]
    steps, peak = mixed(requests, seed=5)
    assert max(len(s["entries"]) for s in steps) >= 3
    runner, _, _ = runner_for(models, name, dtype, pool_tokens=peak, max_requests=4)
    check_rows(steps, run_steps(runner, steps), expected, dtype, name, margins)
    runner.manager.check()
    alone = whole({"r4": requests["r4"]})
    check_rows(alone, run_steps(runner, alone), expected, dtype, name, margins)


def test_window_edges_sinks_and_a_far_key_show(tmp_path):
    """Attention so sharp (scores times eight) that a key one position inside or outside a window moves
    the logits by far more than the tolerance, in a prompt, in portions and in decoding; a window
    longer than several pages and a layer that sees everything, hundreds of positions back."""
    from tokamak_amd.engine.runner import ModelRunner

    cfg = model_json([latent(window=11, scale=1.6, mlp=None), attention(heads=2, kv_heads=1, rot=16, scale=2.0, v_mix=True),
                      latent(heads=3, window=200, scale=1.6), attention(heads=2, kv_heads=1, rot=16, scale=2.0, v_mix=True, window=37, mlp=dense(32))],
                     width=64)
    w = random_weights(cfg, seed=3, sink=3.0)
    folder = write_folder(tmp_path / "sharp", cfg, w)
    toks = tokens(cfg["vocab"], 450, 7)
    expected = {"x": oracle_logits(cfg, w, toks)}
    for layer, size in ((0, 12), (0, 10), (2, 201), (2, 199), (3, 38), (3, 36)):
        other = json.loads(json.dumps(cfg))
        other["layers"][layer]["mixer"]["mask"]["size"] = size
        assert np.abs(oracle_logits(other, w, toks) - expected["x"]).max() > 0.1
    flat = {k: (v - 3.0 if k.endswith("sink") else v) for k, v in w.items()}
    assert np.abs(oracle_logits(cfg, flat, toks) - expected["x"]).max() > 0.1
    first = list(toks)
    first[0] = (first[0] + 1) % cfg["vocab"]
    assert np.abs(oracle_logits(cfg, w, first)[-1] - expected["x"][-1]).max() > 1e-3      # the far key is seen
    runner = ModelRunner.from_folder(folder, dtype="float32", page_size=16, kv_pool_tokens=512, max_requests=2)
    for steps in (whole({"x": toks}), tail_one_by_one("x", toks, tail=64), portions("x", toks)):
        check_rows(steps, run_steps(runner, steps), expected, "float32")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_through_recorded_steps(models, dtype):
    """One prompt token, then 260 tokens one by one (the recorded step of each shape replayed many
    times, two requests side by side at different lengths); and the same without recorded steps and
    without recorded layers gives the same bits."""
    shape = "base" if dtype == "float32" else "base-all"
    runner, cfg, w = runner_for(models, shape, dtype)
    assert runner.use_graphs
    a, b = tokens(cfg["vocab"], 261, 11), tokens(cfg["vocab"], 200, 12)
    expected = {"a": oracle_logits(cfg, w, a), "b": oracle_logits(cfg, w, b)}
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:1], "want": [0]}], "end": []}]
    for i in range(1, 261):
        entries = [{"id": "a", "tokens": [a[i]], "want": [0]}]
        if i >= 61:
            entries.append({"id": "b", "tokens": [b[i - 61]], "want": [0]})
        steps.append({"step": i, "entries": entries, "end": []})
    got = run_steps(runner, steps)
    check_rows(steps, got, expected, dtype)
    plain_runner, _, _ = runner_for(models, shape, dtype, use_graphs=False)
    plain_runner.model.replay_layers = False
    again = run_steps(plain_runner, steps)
    for step in got:
        assert np.array_equal(got[step], again[step]), step


def test_greedy_generation_through_the_entry_point(models):
    """``LLM.generate``: scheduler, portions of prompts, batched decoding, greedy sampling; a pool so
    tight that requests are evicted and computed again."""
    from tokamak_amd import LLM, SamplingParams

    folder, cfg, w, page = models["base"]
    prompts = [tokens(cfg["vocab"], n, 40 + n) for n in (3, 30, 17, 9, 1)]
    new = 14

    def greedy(prompt):
        ids = list(prompt)
        for _ in range(new):
            ids.append(int(np.argmax(oracle_logits(cfg, w, ids)[-1])))
        return ids[len(prompt):]

    want = [greedy(p) for p in prompts]
    params = SamplingParams(temperature=0.0, max_new_tokens=new)
    for kwargs in (dict(kv_pool_tokens=512), dict(kv_pool_tokens=64, prefill_chunk=8, max_batch_size=3)):
        llm = LLM(folder, dtype="float32", max_seq_len=64, block_size=page, **kwargs)
        out = llm.generate(prompt_token_ids=prompts, sampling_params=params)
        assert [o.output_token_ids for o in out] == want, kwargs


def test_trace_runner_and_command_line(models, tmp_path):
    from test_gpu_rorosun import run_trace_any

    folder, cfg, w, page = models["odd"]
    requests = {f"r{i}": tokens(cfg["vocab"], n, 300 + i) for i, n in enumerate([5, 33, 70, 12, 41])}
    steps, peak = mixed(requests, seed=2)
    expected = {rid: oracle_logits(cfg, w, toks) for rid, toks in requests.items()}
    got = run_trace_any(folder, "float32", steps, peak, tmp_path / "out", page, cfg["vocab"])
    check_rows(steps, got, expected, "float32")
    done = subprocess.run([sys.executable, "-m", "tokamak_amd.cli", "--model", str(folder), "--prompt-ids", "5,6,7",
                           "--max-new-tokens", "4", "--dtype", "float32", "--temperature", "0", "--max-seq-len", "64",
                           "--page-size", str(page), "--quiet"], cwd=ROOT, capture_output=True, text=True, timeout=240)
    assert done.returncode == 0, done.stderr[-2000:]
    ids = [5, 6, 7]
    for _ in range(4):
        ids.append(int(np.argmax(oracle_logits(cfg, w, ids)[-1])))
    assert ",".join(map(str, ids[3:])) in done.stdout.replace(" ", ""), done.stdout
    done = subprocess.run([sys.executable, "-m", "tokamak_amd.cli", "--random-weights", "supinex-tiny", "--prompt-ids",
                           "1,2,3", "--max-new-tokens", "3", "--quiet"], cwd=ROOT, capture_output=True, text=True, timeout=240)
    assert done.returncode == 0, done.stderr[-2000:]
