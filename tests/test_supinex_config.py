"""Supinex on the CPU: configuration, plan, tensor names, the stretched frequencies, and properties
of the plain implementation (no GPU, no kernels)."""

import json
import math

import pytest
import torch

import plain_supinex as plain
from supinex_util import (attention, dense, experts, latent, model_json, oracle_logits, random_weights, tensor_shapes,
                          tokens, write_folder)

CFG = model_json([
    attention(v_mix=False, mlp=dense(40)),
    attention(heads=6, kv_heads=3, dim=12, vdim=20, rot=4, v_mix=True, yarn=(4.0, 64.0, 8.0, 1.0)),
    latent(heads=3, dim=8, rot_dim=4, vdim=12, kv_rank=20, window=9, yarn=(2.0, 32.0, 16.0, 2.0)),
    attention(heads=3, kv_heads=3, dim=12, vdim=20, rot=12, v_mix=True, window=30, mlp=None),
    latent(window=None, rot=4, mlp=experts(5, 1, 24)),
], vocab=131, width=72, eps=1e-6)


def test_a_folder_is_found_by_its_architecture_key(tmp_path):
    from tokamak_amd.config.registry import load_model_description
    from tokamak_amd.models.supinex import parse, to_config_json

    folder = write_folder(tmp_path / "m", CFG, random_weights(CFG, 1))
    arch, cfg, plan = load_model_description(folder)
    assert arch.name == "Supinex" and cfg.width == 72 and len(plan.layers) == 5
    assert parse(json.loads(json.dumps(to_config_json(cfg)))) == cfg
    # every layer its own cache slot: two groups of slots with a window (9, 30), the rest keep everything
    kinds = [spec.role("mixer").spec.kind for spec in plan.layers]
    assert kinds == ["rotated_unit_attention", "rotated_unit_attention", "latent_attention", "rotated_unit_attention",
                     "latent_attention"]
    mixes = [spec.role("mixer").spec.as_dict().get("value_mix") for spec in plan.layers]
    assert mixes == [None, "source", None, "mix", None]        # the first layer that says v_mix is the source
    assert plan.layers[3].role("mixer").spec["window"] == 30 and plan.layers[2].role("mixer").spec["window"] == 9
    assert all(spec.block.kind == "parallel_sublayers" for spec in plan.layers)
    assert "feed_forward" not in dict(plan.layers[3].parts)


def test_tensor_names_and_shapes_match_a_list_written_independently():
    from tokamak_amd.engine.model import LayeredModel
    from tokamak_amd.models.supinex import parse, plan

    model = LayeredModel(plan(parse(CFG)), dtype=torch.float32, device="cpu")
    expected = {n: tuple(s.shape) for n, s in model.expected_tensors().items()}
    assert expected == tensor_shapes(CFG)


@pytest.mark.parametrize("change,message", [
    (lambda c: c.__setitem__("architecture", "Other"), "Unsupported"),
    (lambda c: c["layers"][0].__setitem__("type", "conv"), "unknown layer type"),
    (lambda c: c["layers"][0]["mlp"].__setitem__("kind", "sparse"), "unknown feed-forward kind"),
    (lambda c: c["layers"][1]["mixer"].__setitem__("kv_heads", 4), "multiple of kv_heads"),
    (lambda c: c["layers"][1]["mixer"]["rot"].__setitem__("dims", 14), "rot.dims"),
    (lambda c: c["layers"][2]["mixer"]["rot"].__setitem__("dims", 6), "rot.dims"),
    (lambda c: c["layers"][3]["mixer"].__setitem__("vdim", 24), "mix values"),
    (lambda c: c["layers"][4]["mlp"]["router"].__setitem__("top", 6), "top"),
    (lambda c: c.pop("width"), "width"),
    (lambda c: c["layers"][2]["mixer"].pop("kv_rank"), "kv_rank"),
])
def test_what_cannot_be_a_model_is_refused(change, message):
    from tokamak_amd.models.supinex import parse

    cfg = json.loads(json.dumps(CFG))
    change(cfg)
    with pytest.raises(ValueError, match=message):
        parse(cfg)


def test_optional_keys_may_be_absent():
    from tokamak_amd.models.supinex import parse, plan

    cfg = model_json([attention(rot=0), latent(rot=0, window=None, mlp=None)])
    cfg["layers"][0]["mixer"].pop("kv_heads")
    cfg["layers"][0]["mixer"].pop("v_mix")
    made = plan(parse(cfg))
    assert "position" not in dict(made.layers[0].parts) and "position" not in dict(made.layers[1].parts)
    assert made.layers[0].role("mixer").spec["num_kv_heads"] == 4


@pytest.mark.parametrize("rot", [dict(base=10000.0, dims=16), dict(base=120000.0, dims=40, scaling=dict(factor=3.0, original=256, fast=16.0, slow=2.0)),
                                 dict(base=500.0, dims=8, scaling=dict(factor=8.0, original=16, fast=4.0, slow=0.5)),
                                 dict(base=1e6, dims=64, scaling=dict(factor=40.0, original=4096, fast=24.0, slow=2.0))])
def test_stretched_frequencies_match_the_plain_ones(rot):
    from tokamak_amd.parts.rotary import yarn_frequencies

    s = rot.get("scaling")
    got, amplitude = yarn_frequencies(rot["dims"], rot["base"], None if s is None else (s["factor"], s["original"], s["fast"], s["slow"]))
    want, want_amplitude = plain.rotary_frequencies(rot)
    assert torch.allclose(torch.tensor(got, dtype=torch.float64), want, rtol=1e-12, atol=0)
    assert amplitude == pytest.approx(want_amplitude, rel=1e-12)
    if s is not None:
        plain_f = [rot["base"] ** (-2.0 * i / rot["dims"]) for i in range(rot["dims"] // 2)]
        ratios = [g / p for g, p in zip(got, plain_f)]
        # fast dimensions are kept, slow ones divided by the factor, and the ramp between them is monotone
        assert ratios[0] == pytest.approx(1.0) and all(a >= b - 1e-12 for a, b in zip(ratios, ratios[1:]))
        assert min(ratios) >= 1.0 / s["factor"] - 1e-12


def test_presets_build_and_shorten():
    from tokamak_amd.config.registry import find_preset

    for name in ("supinex-tiny", "supinex-0.6b", "supinex-8b"):
        arch, cfg = find_preset(name)
        made = arch.plan(arch.shorten(cfg, 3))
        assert len(made.layers) == 3 and arch.parse(arch.to_json(cfg)) == cfg


# -- properties of the plain implementation -----------------------------------------------
def test_plain_sink_softmax_and_layer_norm():
    s = torch.tensor([0.3, -1.0, 2.0], dtype=torch.float64)
    p = plain.sink_softmax(s, torch.tensor(0.5, dtype=torch.float64))
    assert float(p.sum()) == pytest.approx(float(torch.exp(s).sum() / (torch.exp(s).sum() + math.exp(0.5))))
    assert float(plain.sink_softmax(s, -1e30).sum()) == pytest.approx(1.0)      # a sink far below adds nothing
    assert float(plain.sink_softmax(s, 800.0).sum()) == 0.0                     # and one far above takes everything
    x = torch.randn(5, 12, dtype=torch.float64)
    w = torch.rand(12, dtype=torch.float64)
    want = torch.nn.functional.layer_norm(x, (12,), w, None, 1e-5)
    assert torch.allclose(plain.layer_norm(x, w, 1e-5), want, atol=1e-12)
    z = torch.linspace(-4, 4, 9, dtype=torch.float64)
    assert torch.allclose(plain.gelu_tanh(z), torch.nn.functional.gelu(z, approximate="tanh"), atol=1e-12)


def test_plain_rotation_pairs_neighbours_and_keeps_the_rest():
    x = torch.randn(3, 2, 10, dtype=torch.float64)
    rot = {"base": 100.0, "dims": 6}
    out = plain.rotate(x, torch.tensor([0, 5, 9]), rot)
    assert torch.equal(out[0], x[0]) and torch.equal(out[..., 6:], x[..., 6:])
    norms = lambda t: (t[..., 0:6:2] ** 2 + t[..., 1:6:2] ** 2)
    assert torch.allclose(norms(out), norms(x), atol=1e-12)            # each pair keeps its length
    angle = 5 * 100.0 ** (-2.0 / 6)
    u, v = x[1, 0, 2], x[1, 0, 3]
    assert float(out[1, 0, 2]) == pytest.approx(float(u * math.cos(angle) - v * math.sin(angle)))
    assert float(out[1, 0, 3]) == pytest.approx(float(v * math.cos(angle) + u * math.sin(angle)))
    scaled = plain.rotate(x, torch.tensor([0, 5, 9]), dict(rot, scaling=dict(factor=4.0, original=8, fast=4.0, slow=1.0)))
    assert torch.allclose(norms(scaled), norms(x) * (0.1 * math.log(4.0) + 1.0) ** 2, atol=1e-12)


def test_plain_portions_equal_the_whole_and_windows_hide_keys():
    cfg = model_json([attention(v_mix=True, mlp=dense(24)), latent(window=5), attention(v_mix=True, window=7, mlp=None)], width=32)
    w = {k: v.double() for k, v in random_weights(cfg, 3).items()}
    toks = tokens(cfg["vocab"], 19, 1)
    whole = plain.forward(cfg, w, toks)[0]
    past, rows, at = None, [], 0
    for n in (6, 2, 1, 7, 3):
        out, past = plain.forward(cfg, w, toks[at:at + n], first_position=at, past=past)
        rows.append(out)
        at += n
    assert torch.allclose(torch.cat(rows), whole, atol=1e-10)
    # a token that the windows have left behind changes nothing later, one just inside does
    other = list(toks)
    other[2] = (other[2] + 1) % cfg["vocab"]
    moved = plain.forward(cfg, w, other)[0]
    reach = 2 + (5 - 1) + (7 - 1)          # through both windowed layers at most; the first layer sees everything
    assert not torch.allclose(moved[reach], whole[reach], atol=1e-6)
    assert (moved[3] - whole[3]).abs().max() > 1e-6
    wide = json.loads(json.dumps(cfg))
    wide["layers"][1]["mixer"]["mask"]["size"] = 6
    assert (plain.forward(wide, w, toks)[0][8:] - whole[8:]).abs().max() > 1e-6
    assert torch.allclose(plain.forward(wide, w, toks)[0][:5], whole[:5], atol=1e-10)


def test_plain_experts_with_all_chosen_is_the_softmax_weighted_sum():
    cfg = model_json([attention(mlp=experts(3, 3, 8))], width=16)
    w = {k: v.double() for k, v in random_weights(cfg, 5).items()}
    h = torch.randn(4, 16, dtype=torch.float64)
    got = plain.routed_experts(h, w, "l0.mlp.", cfg["layers"][0]["mlp"])
    scores = torch.softmax(h @ w["l0.mlp.router"].T, -1)
    want = sum(scores[:, e:e + 1] * ((plain.silu(h @ w[f"l0.mlp.e{e}.gate"].T) * (h @ w[f"l0.mlp.e{e}.up"].T)) @ w[f"l0.mlp.e{e}.down"].T)
               for e in range(3))
    assert torch.allclose(got, want, atol=1e-12)
    assert oracle_logits(cfg, random_weights(cfg, 5), [1, 2, 3]).shape == (3, cfg["vocab"])


def test_key_splits_of_single_tokens_with_many_heads():
    """Blocks that share a token's keys in the heads-as-columns form: none for short contexts, more the
    fewer tokens there are, a wave never under two steps of 16 keys, at most 16 (the merge's 64 parts)."""
    from tokamak_amd.kernels.attention import heads_form_splits

    assert heads_form_splits(1, 1, 8, 20, 30, None) == 1
    # the context counts as recorded steps round it, so a step splits alike recorded or not
    assert heads_form_splits(1, 1, 8, 20, None, None) == heads_form_splits(1, 1, 8, 256, None, None)
    assert heads_form_splits(2, 1, 8, 257, None, None) == heads_form_splits(2, 1, 8, 320, None, None)
    assert heads_form_splits(8, 1, 32, 2112, 1024, None) == 9          # 65 steps of the window, two pieces of 16 heads
    assert heads_form_splits(8, 1, 32, 2112, None, None) == 16
    assert heads_form_splits(1, 1, 16, 100000, None, None) == 16
    assert heads_form_splits(64, 2, 16, 4000, None, None) == 2
    assert heads_form_splits(300, 4, 8, 4000, None, None) == 1
    for tokens in (1, 3, 17, 200):
        for keys in (1, 15, 16, 17, 500, 5000):
            n = heads_form_splits(tokens, 2, 12, keys, None, 64)
            assert 1 <= n <= 16 and (n == 1 or n * 8 <= min(keys, 64) // 16 + 2 + 8)
