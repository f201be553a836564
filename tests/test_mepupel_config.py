"""The Mepupel design without a GPU: configuration, plan, tensor names, cache groups, and properties of
the plain implementation that the GPU tests compare the engine with."""

import json
import math

import pytest
import torch

import plain_mepupel as plain
from mepupel_util import (attention, dense, double, experts, latent, mamba, model_json, random_weights, tensor_shapes,
                          tokens, write_folder)

CFG = model_json([latent(mlp=dense(40)), mamba(), attention(), latent(kv_from=0), mamba(mlp=None),
                  attention(rot=16, yarn=(4.0, 64.0, 16.0, 2.0), window=44, keep_first=5)])


def test_a_folder_is_found_by_its_architecture_key_and_round_trips(tmp_path):
    from tokamak_amd.config.registry import load_model_description
    from tokamak_amd.models.mepupel import MepupelConfig, parse, to_config_json

    folder = write_folder(tmp_path / "m", CFG, random_weights(CFG, 1))
    arch, cfg, made = load_model_description(folder)
    assert arch.name == "Mepupel" and isinstance(cfg, MepupelConfig) and cfg.residual_mult == 0.5
    assert parse(to_config_json(cfg)) == cfg
    assert [L.type for L in cfg.layers] == [L["type"] for L in CFG["layers"]]
    assert made.vocab_size == CFG["vocab"] and len(made.layers) == 6


def test_run_order_and_cache_slots_of_borrowed_latents():
    from tokamak_amd.models.mepupel import parse, plan

    made = plan(parse(CFG))
    assert [(c.layer, c.cache, c.writes_cache) for c in made.order] == [
        (0, 0, True), (1, 1, True), (2, 2, True), (3, 0, False), (4, 4, True), (5, 5, True)]
    assert made.layers[3].role("mixer").spec["own_latent"] is False and made.layers[0].role("mixer").spec["own_latent"] is True
    # every layer has a second norm exactly if it has a feed-forward, and the block scales the branches' sum
    for spec, layer in zip(made.layers, CFG["layers"]):
        roles = dict(spec.parts)
        assert ("feed_forward_norm" in roles) == (layer["mlp"] is not None) == ("feed_forward" in roles)
        assert spec.block.kind == "parallel_sublayers" and spec.block["branch_scale"] == 0.5
    assert "position" in dict(made.layers[2].parts) and "position" not in dict(made.layers[0].parts)
    assert made.layers[5].role("position").spec["yarn"] == (4.0, 64.0, 16.0, 2.0)


def test_tensor_names_and_shapes_match_a_list_written_independently():
    from tokamak_amd.models.mepupel import parse, plan
    from tokamak_amd.weights.random_init import expected_tensors_of

    for cfg in (CFG, model_json([mamba(heads=3, vdim=20, state=24, groups=1, conv=3, norm_groups=5, mlp=experts(5, 1, 24, None, None, None)),
                                 latent(heads=3, dim=20, vdim=36, kv_rank=45, q_rank=17, mlp=None)], width=72)):
        expected = expected_tensors_of(plan(parse(cfg)))
        shapes = tensor_shapes(cfg)
        assert set(expected) == set(shapes)
        assert all(expected[n].fits(shape) for n, shape in shapes.items())
        optional = {n for n, s in expected.items() if s.optional}
        assert optional == {n for n in shapes if n.endswith("correction")}


def test_optional_keys_may_be_absent():
    from tokamak_amd.models.mepupel import parse, plan

    cfg = model_json([attention(rot=0, window=None), latent(mlp=experts(4, 2, 16, None, None, None)), mamba(mlp=None)], mult=None)
    cfg["layers"][0]["mixer"].pop("kv_heads")
    cfg["layers"][0]["mixer"].pop("vdim")
    cfg["layers"][2]["mixer"].pop("norm_groups")
    cfg["layers"][2]["mixer"].pop("groups")
    parsed = parse(cfg)
    made = plan(parsed)
    assert parsed.residual_mult == 1.0 and parsed.layers[2].mixer.norm_groups == 1 and parsed.layers[2].mixer.groups == 1
    mixer = made.layers[0].role("mixer").spec
    assert mixer["num_kv_heads"] == 4 and mixer["value_dim"] == 16 and mixer["window"] is None and mixer["keep_first"] == 0
    ff = made.layers[1].role("feed_forward").spec
    assert ff["groups"] is None and ff["shared_size"] is None and ff["weight_scale"] == 1.0 and ff["normalise"] is True
    only_size = model_json([attention(window=9, keep_first=0)])
    only_size["layers"][0]["mixer"]["mask"].pop("keep_first")
    assert plan(parse(only_size)).layers[0].role("mixer").spec["keep_first"] == 0


@pytest.mark.parametrize("change,message", [
    (lambda c: c.update(architecture="Other"), "Unsupported architecture"),
    (lambda c: c["layers"][0].update(type="conv"), "unknown layer type"),
    (lambda c: c["layers"][0]["mlp"].update(kind="sparse"), "unknown feed-forward kind"),
    (lambda c: c["layers"][3]["mixer"].update(kv_from=1), "kv_from"),
    (lambda c: c["layers"][3]["mixer"].update(kv_from=3), "kv_from"),
    (lambda c: c["layers"][3]["mixer"].update(kv_rank=16), "kv_from"),
    (lambda c: c["layers"][2]["mixer"].update(heads=3), "multiple of kv_heads"),
    (lambda c: c["layers"][1]["mixer"].update(groups=3), "groups must divide"),
    (lambda c: c["layers"][1]["mlp"]["router"]["groups"].update(count=3), "groups.count"),
    (lambda c: c["layers"][1]["mlp"]["router"]["groups"].update(keep=0), "groups.count"),
    (lambda c: c["layers"][1]["mlp"]["router"].update(top=9), "top <= experts"),
    (lambda c: c["layers"][2]["mixer"]["rot"].update(dims=7), "rot.dims"),
    (lambda c: c.pop("width"), "width"),
    (lambda c: c["layers"][0]["mixer"].pop("q_rank"), "q_rank"),
    (lambda c: c["layers"][1]["mixer"].pop("state"), "state"),
])
def test_what_cannot_be_a_model_is_refused(change, message):
    from tokamak_amd.models.mepupel import parse

    cfg = json.loads(json.dumps(CFG))
    change(cfg)
    with pytest.raises(ValueError, match=message):
        parse(cfg)


def test_presets_build_and_shorten():
    from tokamak_amd.config.registry import find_preset

    for name in ("mepupel-tiny", "mepupel-0.6b", "mepupel-8b"):
        arch, cfg = find_preset(name)
        made = arch.plan(arch.shorten(cfg, 4))
        assert len(made.layers) == 4 and arch.parse(arch.to_json(cfg)) == cfg
        assert made.order[3].cache == 0 and not made.order[3].writes_cache


def test_cache_groups_keep_the_pages_of_the_first_positions():
    """A window group with kept first positions gives back what lies behind the window, never the pages that
    hold the first positions; groups are told apart by both numbers."""
    from tokamak_amd.cache.manager import CacheManager
    from tokamak_amd.cache.pages import RELEASED, CacheGroupSpec

    groups = [CacheGroupSpec("full", (0,)), CacheGroupSpec("a", (1,), window=10, keep_first=0),
              CacheGroupSpec("b", (2,), window=10, keep_first=5), CacheGroupSpec("c", (3,), window=10, keep_first=17)]
    manager = CacheManager(groups, 64, 8, 2)
    manager.admit("r")
    manager.ensure_capacity("r", 100)
    assert manager.release_behind_window("r", 100) == 11 + 10 + 8       # first needed position 91: pages 0..10 lie behind it
    tables = [manager.block_table("r", g) for g in range(4)]
    assert all(p != RELEASED for p in tables[0])
    assert [i for i, p in enumerate(tables[1]) if p == RELEASED] == list(range(0, 11))
    assert [i for i, p in enumerate(tables[2]) if p == RELEASED] == list(range(1, 11))
    assert [i for i, p in enumerate(tables[3]) if p == RELEASED] == list(range(3, 11))
    assert manager.release_behind_window("r", 100) == 0
    manager.ensure_capacity("r", 130)
    assert manager.release_behind_window("r", 130) == 3 * 4
    manager.check()
    manager.free("r")
    manager.check()
    assert all(manager.num_free_pages(g) == 64 for g in range(4))
    # a request shorter than the kept positions gives nothing back
    manager.admit("s")
    manager.ensure_capacity("s", 12)
    assert manager.release_behind_window("s", 12) == 0 and manager.groups[3].live_pages("s") == 2


def test_the_model_asks_for_one_group_per_window_and_kept_count():
    from tokamak_amd.engine.model import LayeredModel
    from tokamak_amd.models.mepupel import parse, plan

    cfg = model_json([attention(window=24, keep_first=3), attention(window=24, keep_first=3), attention(window=24, keep_first=4),
                      attention(window=None), latent(), latent(kv_from=4), mamba()])
    model = LayeredModel(plan(parse(cfg)), dtype=torch.float32, device="meta")
    groups, slots = model.cache_layout()
    assert [(g.window, g.keep_first, g.slots) for g in groups] == [(None, 0, (3, 4)), (24, 3, (0, 1)), (24, 4, (2,))]
    assert 5 not in slots and 6 not in slots
    assert set(model.state_requests()) == {6} and set(model.state_requests()[6]) == {"S", "conv"}


# -- properties of the plain implementation -----------------------------------------------
def test_plain_visibility_by_brute_force():
    mask = {"size": 5, "keep_first": 3}
    for i in range(20):
        seen = [j for j in range(25) if plain.visible(i, j, mask)]
        assert seen == sorted(set(range(min(3, i + 1))) | set(range(max(0, i - 4), i + 1)))
    assert [j for j in range(9) if plain.visible(6, j, None)] == list(range(7))
    assert [j for j in range(9) if plain.visible(6, j, {"size": 2})] == [5, 6]


def test_plain_rotation_pairs_halves_and_stretches_slow_frequencies():
    x = torch.randn(3, 2, 10, dtype=torch.float64)
    rot = {"base": 100.0, "dims": 6}
    out = plain.rotate(x, torch.tensor([0, 5, 9]), rot)
    assert torch.equal(out[0], x[0]) and torch.equal(out[..., 6:], x[..., 6:])
    lengths = lambda t: t[..., 0:3] ** 2 + t[..., 3:6] ** 2
    assert torch.allclose(lengths(out), lengths(x), atol=1e-12)            # each pair (i, i + 3) keeps its length
    angle = 5 * 100.0 ** (-2.0 / 6)
    u, v = x[1, 0, 1], x[1, 0, 4]
    assert float(out[1, 0, 1]) == pytest.approx(float(u * math.cos(angle) - v * math.sin(angle)))
    assert float(out[1, 0, 4]) == pytest.approx(float(v * math.cos(angle) + u * math.sin(angle)))
    scaling = dict(factor=4.0, original=8, fast=4.0, slow=1.0)
    scaled = plain.rotate(x, torch.tensor([0, 5, 9]), dict(rot, scaling=scaling))
    assert torch.allclose(lengths(scaled), lengths(x) * (0.1 * math.log(4.0) + 1.0) ** 2, atol=1e-12)
    freqs, _ = plain.stretched_frequencies(64, 1e6, dict(factor=40.0, original=4096, fast=24.0, slow=2.0))
    ratios = [f / 1e6 ** (-2.0 * i / 64) for i, f in enumerate(freqs)]
    assert ratios[0] == pytest.approx(1.0) and ratios[-1] == pytest.approx(1 / 40.0)
    assert all(a >= b - 1e-12 for a, b in zip(ratios, ratios[1:]))


@pytest.mark.parametrize("rot", [dict(base=10000.0, dims=16), dict(base=2e5, dims=20, scaling=dict(factor=6.0, original=512, fast=16.0, slow=2.0)),
                                 dict(base=500.0, dims=8, scaling=dict(factor=8.0, original=16, fast=4.0, slow=0.5))])
def test_the_engines_frequencies_match_the_plain_ones(rot):
    from tokamak_amd.parts.rotary import yarn_frequencies

    s = rot.get("scaling")
    got, amplitude = yarn_frequencies(rot["dims"], rot["base"], None if s is None else (s["factor"], s["original"], s["fast"], s["slow"]))
    want, want_amplitude = plain.stretched_frequencies(rot["dims"], rot["base"], s)
    assert got == pytest.approx(want, rel=1e-12) and amplitude == pytest.approx(want_amplitude, rel=1e-12)


def test_plain_state_space_against_its_closed_form_and_convolution():
    cfg = model_json([mamba(heads=2, vdim=4, state=3, groups=1, conv=3, norm_groups=2, mlp=None)], width=16)
    w = double(random_weights(cfg, 2))
    m = cfg["layers"][0]["mixer"]
    h = torch.randn(7, 16, dtype=torch.float64)
    out, state = plain.mamba2(h, w, "l0.mix.", m, 1e-5, return_state=True)
    # the same by unrolling: S_T = sum_s (prod_{r > s} a_r) dt_s B_s x_s^T
    proj = h @ w["l0.mix.in"].T
    u = plain.silu(plain.causal_conv(proj[:, 8:8 + 14], w["l0.mix.conv"], w["l0.mix.conv.b"]))
    dt = plain.softplus(proj[:, 22:] + w["l0.mix.dt_bias"])
    a = torch.exp(-torch.exp(w["l0.mix.A_log"]) * dt)
    want = torch.zeros(2, 3, 4, dtype=torch.float64)
    for s in range(7):
        for head in range(2):
            want[head] += a[s + 1:, head].prod() * dt[s, head] * torch.outer(u[s, 8:11], u[s, 4 * head:4 * head + 4])
    assert torch.allclose(state, want, atol=1e-12)
    # the convolution is causal with zeros before the start, and its last tap meets the token itself
    x = torch.randn(5, 2, dtype=torch.float64)
    k = torch.tensor([[1.0, 10.0, 100.0], [0.0, 0.0, 1.0]], dtype=torch.float64)
    y = plain.causal_conv(x, k, torch.tensor([0.5, 0.0], dtype=torch.float64))
    assert torch.allclose(y[:, 1], x[:, 1]) and float(y[0, 0]) == pytest.approx(0.5 + 100.0 * float(x[0, 0]))
    assert float(y[2, 0]) == pytest.approx(0.5 + float(x[0, 0]) + 10.0 * float(x[1, 0]) + 100.0 * float(x[2, 0]))
    # a later token changes nothing before it
    other = h.clone()
    other[5] += 1.0
    assert torch.allclose(plain.mamba2(other, w, "l0.mix.", m, 1e-5)[:5], out[:5], atol=1e-12)


def test_plain_router_groups_correction_and_weights():
    router = {"experts": 6, "top": 2, "scale": 2.0, "groups": {"count": 3, "keep": 1}}
    w = {"r.router": torch.eye(6, dtype=torch.float64), "r.correction": torch.tensor([0.0, 0.0, 0.0, 0.0, 0.0, 0.0], dtype=torch.float64)}
    logit = lambda s: math.log(s / (1 - s))
    # scores: group 0 = (.9, .1), group 1 = (.6, .6), group 2 = (.2, .3): the sum of two picks group 1 over the single best
    h = torch.tensor([[logit(0.9), logit(0.1), logit(0.6), logit(0.6), logit(0.2), logit(0.3)]], dtype=torch.float64)
    chosen, weight = plain.route(h, w, "r.", router)
    assert sorted(chosen[0].tolist()) == [2, 3] and weight[0].tolist() == pytest.approx([1.0, 1.0])
    # a correction moves the choice, not the weights: group 0 now wins, its weights are the plain scores renormalised
    w["r.correction"] = torch.tensor([0.0, 0.5, 0.0, 0.0, 0.0, 0.0], dtype=torch.float64)
    chosen, weight = plain.route(h, w, "r.", router)
    assert sorted(chosen[0].tolist()) == [0, 1]
    assert sorted(weight[0].tolist()) == pytest.approx([2.0 * 0.1 / 1.0, 2.0 * 0.9 / 1.0])
    # negative choice scores: an expert outside the kept groups is never chosen, however few are left
    w["r.correction"] = torch.tensor([-5.0, -5.0, -7.0, -7.0, -9.0, -9.0], dtype=torch.float64)
    assert sorted(plain.route(h, w, "r.", router)[0][0].tolist()) == [0, 1]
    no_groups = {"experts": 6, "top": 2}
    w["r.correction"] = torch.zeros(6, dtype=torch.float64)
    chosen, weight = plain.route(h, w, "r.", no_groups)
    assert sorted(chosen[0].tolist()) in ([0, 2], [0, 3]) and float(weight.sum()) == pytest.approx(1.0)


def test_plain_model_runs_and_a_borrowed_latent_is_the_sources():
    w = random_weights(CFG, 4)
    toks = tokens(CFG["vocab"], 12, 2)
    logits, after = plain.forward(CFG, double(w), toks)
    assert logits.shape == (12, CFG["vocab"]) and after.shape == (6, 12, CFG["width"])
    # layer 3 reads layer 0's latent: changing layer 0's W_dkv moves layer 3's output even with layer 0's own
    # attention taken out of the picture (its o projection zeroed)
    changed = dict(double(w))
    changed["l0.mix.o"] = torch.zeros_like(changed["l0.mix.o"])
    base = plain.forward(CFG, changed, toks)[1]
    changed["l0.mix.dkv"] = changed["l0.mix.dkv"] * 1.5 + 0.1
    moved = plain.forward(CFG, changed, toks)[1]
    assert torch.allclose(moved[2], base[2], atol=1e-12) and not torch.allclose(moved[3], base[3], atol=1e-6)
