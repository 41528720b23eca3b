"""Retudra's configuration, recipe and cache needs, and the plain implementation's own consistency (no GPU)."""
import copy

import pytest
import torch

import plain_retudra as plain
from arle_amd.cache.manager import PagedNeed, StateNeed
from arle_amd.cache.pages import PageGroup
from arle_amd.config import ConfigError, RetudraConfig, detect_architecture
from arle_amd.models.decoder import declared_cache_needs, expected_checkpoint_tensors
from arle_amd.weights.loader import WeightsError, compare_with_expected
from tiny_retudra import TINY, attn, layer


@pytest.mark.parametrize("name", list(TINY))
def test_a_configuration_reads_back_equal_and_names_its_tensors(name):
    raw = TINY[name][0]
    config = RetudraConfig.from_dict(raw)
    assert RetudraConfig.from_dict(config.to_dict()) == config
    arch = detect_architecture(raw)
    assert arch.name == "Retudra"
    spec = arch.recipe(config, ())
    expected = expected_checkpoint_tensors(spec)
    W, V, side = raw["width"], raw["vocab"], raw.get("token_side")
    assert expected["embed"].shape == (V, W) and expected["head"].shape == (V, W)
    assert expected["final.norm"].shape == (W,) and expected["final.norm.b"].shape == (W,)
    assert ("side.embed" in expected) == (side is not None)
    if side:
        assert expected["side.embed"].shape == (V, len(raw["layers"]) * side["dim"])
    for i, lay in enumerate(raw["layers"]):
        m, p = lay["mixer"], f"l{i}."
        assert expected[p + "norm1"].shape == (W,) and expected[p + "norm1.b"].shape == (W,)
        assert (p + "norm2" in expected) == (lay["mlp"] is not None) == (p + "norm2.b" in expected)
        assert (p + "side.gate" in expected) == (side is not None)
        if side:
            assert expected[p + "side.gate"].shape == (side["dim"], W) and expected[p + "side.proj"].shape == (W, side["dim"])
            assert expected[p + "side.norm"].shape == (W,)
        if lay["type"] == "attention":
            kv = m.get("kv_heads") or m["heads"]
            assert expected[p + "mix.q.norm"].shape == (m["heads"] * m["dim"],)
            assert expected[p + "mix.k.norm"].shape == (kv * m["dim"],)
            assert expected[p + "mix.v"].shape == (kv * m["vdim"], W) and expected[p + "mix.o"].shape == (W, m["heads"] * m["vdim"])
        elif lay["type"] == "latent_attention":
            assert expected[p + "mix.q"].shape == (m["heads"] * (m["dim"] + m["rot_dim"]), W)
            assert expected[p + "mix.dkv"].shape == (m["kv_rank"] + m["rot_dim"], W)
            assert expected[p + "mix.uk"].shape == (m["heads"] * m["dim"], m["kv_rank"])
            assert expected[p + "mix.g"].shape == (m["heads"] * m["vdim"], W) and p + "mix.sink" not in expected
        else:
            kv = m.get("kv_heads") or m["heads"]
            assert expected[p + "mix.q.conv"].shape == (kv * m["dim"], m["conv"])
            assert expected[p + "mix.a1"].shape == (m["decay_rank"], W)
            assert expected[p + "mix.a2"].shape == (m["heads"] * m["dim"], m["decay_rank"])
            assert expected[p + "mix.dt_bias"].shape == (m["heads"] * m["dim"],) and expected[p + "mix.A_log"].shape == (m["heads"],)
            assert expected[p + "mix.g2"].shape == (m["heads"] * m["vdim"], m["gate_rank"]) and p + "mix.g" not in expected
        if lay["mlp"] and lay["mlp"]["kind"] == "moe":
            r = lay["mlp"]["router"]
            outputs = r["experts"] + r.get("identity", 0)
            assert expected[p + "mlp.router"].shape == (outputs, W) and expected[p + "mlp.correction"].shape == (outputs,)
            assert p + f"mlp.e{r['experts'] - 1}.down" in expected and p + f"mlp.e{r['experts']}.down" not in expected


def test_the_middle_widths_of_the_delta_rules_projections_come_from_the_tensors_where_the_configuration_is_silent():
    raw = copy.deepcopy(TINY["P"][0])
    for key in ("decay_rank", "gate_rank"):
        del raw["layers"][1]["mixer"][key]
    config = RetudraConfig.from_dict(raw)
    assert RetudraConfig.from_dict(config.to_dict()) == config
    expected = expected_checkpoint_tensors(detect_architecture(raw).recipe(config, ()))
    W = raw["width"]
    assert expected["l1.mix.a1"].shape == (None, W) and expected["l1.mix.a2"].shape == (4 * 16, None)
    found = {n: tuple(7 if d is None else d for d in decl.shape) for n, decl in expected.items()}
    assert compare_with_expected(found, expected) == []
    found["l1.mix.a2"] = (4 * 16 + 1, 7)
    with pytest.raises(WeightsError):
        compare_with_expected(found, expected)
    from arle_amd.weights.random_init import random_tensor
    with pytest.raises(ValueError, match="configuration"):
        random_tensor("l1.mix.a1", expected["l1.mix.a1"], 1, 0.1, 0.1, torch.float32)


def test_cache_needs_follow_the_mixers():
    raw = TINY["P"][0]
    spec = detect_architecture(raw).recipe(RetudraConfig.from_dict(raw), ())
    needs = declared_cache_needs(spec)
    assert isinstance(needs[0], PagedNeed) and needs[0].window == 24 and needs[0].keep_first == 5
    assert isinstance(needs[1]["S"], StateNeed) and needs[1]["S"].shape == (4, 16, 12) and needs[1]["S"].dtype == torch.float32
    assert needs[1]["conv"].shape[0] == 3       # taps - 1 inputs of every channel of q, k and v
    assert isinstance(needs[2], PagedNeed) and needs[2].window is None and needs[2].keep_first == 0
    assert [t.shape for t in needs[2].tensors] == [(1, "page", 24 + 8), (1, 24, "page")]
    assert needs[3].window == 9 and needs[3].keep_first == 3
    # an attention without a window keeps everything, whatever it would keep first
    q = TINY["Q"][0]
    needs = declared_cache_needs(detect_architecture(q).recipe(RetudraConfig.from_dict(q), ()))
    assert needs[1].window is None and needs[1].keep_first == 0 and needs[3].window == 7 and needs[3].keep_first == 0


def test_pages_of_the_kept_first_keys_never_go_back():
    g = PageGroup(num_pages=12, page_size=4, window=6, keep_first=5)
    g.open("a")
    g.append("a", 9)
    assert g.trim("a") == []                  # the window's first page is page 1, which holds kept key 4
    g.append("a", 11)                         # length 20: keys <= 14 are behind the window: pages 2 (keys 8..11); page 3 holds 15
    assert g.trim("a") == [2]
    assert [p >= 0 for p in g.tables["a"].pages] == [True, True, False, True, True]
    g.append("a", 9)                          # length 29: keys <= 23 are dead: pages 3..5
    assert g.trim("a") == [3, 4, 5]
    g.check()
    g.close("a")
    assert g.pool.free_count == 12
    none = PageGroup(num_pages=4, page_size=4, window=6)
    none.open("b")
    none.append("b", 16)
    assert none.trim("b") == [0, 1]
    with pytest.raises(ValueError):
        PageGroup(num_pages=4, page_size=4, window=6, keep_first=-1)


BAD = [
    (lambda r: r["layers"][0].update(type="attention_9"), "unknown layer type"),
    (lambda r: r["layers"][0]["mixer"].update(kv_heads=4), "divisible"),
    (lambda r: r["layers"][0]["mixer"]["rot"].update(dims=11), "even"),
    (lambda r: r["layers"][0]["mixer"]["rot"].update(dims=18), "at most"),
    (lambda r: r["layers"][0]["mixer"]["mask"].update(size=0), "positive"),
    (lambda r: r["layers"][0]["mixer"]["mask"].update(keep_first=-1), "negative"),
    (lambda r: r["layers"][0]["mlp"].update(kind="sparse"), "unknown kind"),
    (lambda r: r["layers"][1]["mlp"]["router"].update(top=5), "top"),
    (lambda r: r["layers"][1]["mlp"]["router"]["groups"].update(count=3), "divide"),
    (lambda r: r["layers"][1]["mlp"]["router"]["groups"].update(keep=5), "at most"),
    (lambda r: r["layers"][1]["mlp"]["router"].update(identity=-1), "negative"),
    (lambda r: r["layers"][1]["mlp"].pop("expert"), "expert"),
    (lambda r: r["layers"][2]["mixer"].pop("kv_rank"), "kv_rank"),
    (lambda r: r["layers"][2]["mixer"]["rot"].update(dims=10), "at most"),
    (lambda r: r["layers"][1]["mixer"].update(conv=0), "positive"),
    (lambda r: r.update(logit_softcap=-1.0), "positive"),
    (lambda r: r["token_side"].update(dim=0), "positive"),
    (lambda r: r.update(layers=[]), "at least one"),
    (lambda r: r.pop("width"), "width"),
]


@pytest.mark.parametrize("case", range(len(BAD)))
def test_a_configuration_that_cannot_be_used_is_refused_with_its_key(case):
    change, word = BAD[case]
    raw = copy.deepcopy(TINY["P"][0])
    change(raw)
    with pytest.raises(ConfigError, match=word):
        RetudraConfig.from_dict(raw)


def test_what_the_configuration_leaves_out_is_not_there():
    raw = {"architecture": "Retudra", "vocab": 30, "width": 16, "norm": {"eps": 1e-6},
           "layers": [layer("attention", attn(2, None, 8, 8), None)]}
    c = RetudraConfig.from_dict(raw)
    assert c.residual_mult == 1.0 and c.side_dim is None and c.logit_softcap is None
    m = c.layers[0].mixer
    assert m.kv_heads == 2 and m.window is None and m.keep_first == 0 and m.rot is None and c.layers[0].mlp is None
    spec = detect_architecture(raw).recipe(c, ())
    assert not spec.layers[0].parts and "side_out" not in spec.layers[0].norms and not spec.head.params.get("softcap")


def test_the_plain_implementation_agrees_with_itself():
    """The mask, the rotation and the router written a second way."""
    see = plain.visible(12, 4, 2)
    for i in range(12):
        for j in range(12):
            assert bool(see[i, j]) == (j <= i and (i - j < 4 or j < 2))
    assert bool(plain.visible(5).equal(torch.tril(torch.ones(5, 5, dtype=torch.bool))))
    x = torch.randn(3, 2, 10, dtype=torch.float64)
    y = plain.rotate_half(x, torch.tensor([0, 1, 7]), 6, 100.0)
    assert torch.equal(y[0], x[0]) and torch.equal(y[..., 6:], x[..., 6:])
    for i in range(3):
        a = 7 * 100.0 ** (-2.0 * i / 6)
        u, v = x[2, :, i], x[2, :, i + 3]
        assert torch.allclose(y[2, :, i], u * torch.cos(torch.tensor(a)) - v * torch.sin(torch.tensor(a)))
        assert torch.allclose(y[2, :, i + 3], v * torch.cos(torch.tensor(a)) + u * torch.sin(torch.tensor(a)))
    h, router = torch.randn(20, 8, dtype=torch.float64), torch.randn(6, 8, dtype=torch.float64)
    corr = torch.randn(6, dtype=torch.float64) * 0.1
    chosen, weights = plain.route(h, {"top": 2, "groups": {"count": 3, "keep": 1}}, router, corr)
    s = torch.softmax(h @ router.T, -1)
    for t in range(20):
        c = s[t] + corr
        best = max(range(3), key=lambda g: max(c[2 * g], c[2 * g + 1]))
        pair = sorted([2 * best, 2 * best + 1], key=lambda e: -c[e])
        assert chosen[t].tolist() == pair and torch.allclose(weights[t], s[t][pair])
    conv = plain.causal_conv(torch.arange(1.0, 6.0, dtype=torch.float64)[:, None], torch.tensor([[10.0, 1.0]], dtype=torch.float64))
    assert conv[:, 0].tolist() == [1.0, 12.0, 23.0, 34.0, 45.0]
