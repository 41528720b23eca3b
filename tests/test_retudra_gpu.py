"""Retudra on the GPU against the plain implementation (`plain_retudra.py`): every mechanism alone as the part the
engine runs, in cuts of every size, and whole models through `Engine.step`, the scheduler and `LLM.generate`.

Tolerances.  float32: 5e-5 of the largest plain logit for whole models (the test models' routers have logits of order
ten, so that few choices are close calls, and a softmax of such logits carries their rounding on), 5e-5 of the largest
plain output for a mechanism alone (the plain side is float64; the engine adds in 32 bits).  bfloat16: 3e-2 of the largest plain logit
for whole models, 2.5e-2 of the largest plain output for a mechanism alone.
"""
import pytest
import torch

import plain_retudra as plain
import replay
from arle_amd import LLM
from arle_amd.cache import CacheManager
from arle_amd.config import RetudraConfig
from arle_amd.engine import Engine, StepEntry
from arle_amd.engine.batch import build_step_batch
from arle_amd.kernels import ops
from arle_amd.models.retudra import retudra_spec
from arle_amd.parts.base import Runtime, build_part, expected_tensors
from tiny import random_tokens, read_folder
from tiny_retudra import ARCH, TINY, attn, delta, dense, latent, layer, make_model_dir, moe, rot

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
F32, BF16 = torch.float32, torch.bfloat16
TOL = {F32: 5e-5, BF16: 2.5e-2}
EPS = 1e-5


def rnd(shape, seed, std=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * std).to(BF16).float()     # values that bfloat16 holds exactly


def close(got, want, dtype, what, tol=None):
    got, want = got.double().cpu(), want.double()
    assert torch.isfinite(got).all(), what
    err = float((got - want).abs().max()) / float(want.abs().max())
    assert err <= (tol or TOL[dtype]), f"{what}: {err:.3e}"


def one_layer(kind, mixer, mlp=None, width=40, **top):
    """(config dictionary, ModelSpec) of a model of one layer."""
    raw = dict({"architecture": ARCH, "vocab": 50, "width": width, "norm": {"eps": EPS},
                "layers": [layer(kind, mixer, mlp)]}, **top)
    return raw, retudra_spec(RetudraConfig.from_dict(raw))


def random_part(role, spec, dtype, seed, std=0.3, fills=None):
    """A part of `spec` with random tensors; returns (part, {checkpoint name: float32 CPU tensor})."""
    tensors = {}
    for i, (name, decl) in enumerate(sorted(expected_tensors(role, spec).items())):
        t = rnd(tuple(decl.shape), seed + i, std)
        if decl.init == "ones":
            t = 1 + rnd(tuple(decl.shape), seed + i, 0.3)
        for suffix, fill in (fills or {}).items():
            if name.endswith(suffix):
                t = fill(t, seed + i)
        tensors[name] = t
    rt = Runtime(device=torch.device(DEV), act_dtype=dtype)
    held = {k: v.to(DEV, dtype) for k, v in tensors.items()}
    return build_part(role, spec, held.__getitem__, rt), tensors


def run_mixer(part, x, cuts, *, page=4, dtype=F32, tokens=None):
    """Feed x [T, W] of one request to a mixer in portions of the given sizes (repeating), through a cache in which
    another request's pages and slot lie between, every page starts as NaN and the other request's state is rubbish.
    Returns the concatenated outputs."""
    T = x.shape[0]
    part.prepare(T + page)
    cache = CacheManager([part.cache_need()], page_size=page, num_pages=2 * (-(-T // page)) + 4, max_slots=3,
                         max_request_tokens=T + page, device=torch.device(DEV), dtype=dtype)
    cache.admit("other")
    cache.append([("other", page + 1)])
    for group in cache.page_buffers:
        for t in group.values():
            t.fill_(float("nan"))
    cache.admit("r")
    outs, at, k = [], 0, 0
    xd = x.to(DEV, dtype)
    while at < T:
        n = min(cuts[k % len(cuts)], T - at)
        k += 1
        before = cache.length("r")
        cache.append([("r", n)])
        cache.sync_tables()
        batch = build_step_batch([StepEntry("r", [0] * n, [])], cache.slot_of.__getitem__, lambda _r, b=before: b, 10, DEV)
        y = part.forward(xd[at:at + n].contiguous(), batch, cache.view(0))
        outs.append((y.float().sum(0) if y.dim() == 3 else y.float()).cpu())
        cache.trim_windows("r")
        cache.sync_tables()
        at += n
    cache.check()
    return torch.cat(outs)


CUTS = [(1000,), (1,), (2,), (5, 2, 7, 3, 1, 16, 2)]


def mixer_case(kind, mixer, dtype, seed, T, *, page=4, loud=(), std=0.3, fills=None, cuts=CUTS, tol=None, what=""):
    """A mixer alone against its plain function, in every cutting; in float32 the cuttings agree bit for bit.
    loud: positions whose input dwarfs the others', so that a key seen or hidden by mistake shows."""
    raw, spec = one_layer(kind, mixer)
    part, tensors = random_part("mixer", spec.layers[0].mixer, dtype, seed, std, fills)
    x = rnd((T, raw["width"]), seed + 100)
    for p in loud:
        if 0 <= p < T:
            x[p] *= 6.0
    w = lambda name: tensors["l0.mix." + name].double() if ("l0.mix." + name) in tensors else None
    want = plain.MIXERS[kind](x.double(), mixer, w, EPS)
    first = None
    for c in cuts:
        got = run_mixer(part, x, c, page=page, dtype=dtype)
        close(got, want, dtype, f"{what or kind} {dtype} cut {c}", tol)
        if dtype == F32:
            first = got if first is None else first
            assert torch.equal(got, first), f"{what or kind}: cut {c} differs in bits from the whole prompt"


# ----------------------------------------------------------------------------------- mechanisms alone

@pytest.mark.parametrize("width,rows", [(72, 5), (1001, 3), (4096, 2), (42, 4)])
def test_a_layer_norm_on_a_sublayers_output_is_added_times_the_factor(width, rows):
    res = rnd((rows, width), 1, 2.0)
    w, b = 1 + rnd((width,), 2, 0.3), rnd((width,), 3, 0.5)
    y = rnd((rows, width), 4, 3.0) + 2.0      # a mean that is not zero: taking it off shows
    stack = rnd((3, rows, width), 5)
    outs, coefs = rnd((rows, 2, width), 6), rnd((rows, 2), 7).abs()
    for mult in (1.0, 0.5):
        for terms, total in ((y, y), (stack, stack.sum(0)), ([y, stack], y + stack.sum(0)),
                             ((outs, coefs), (outs * coefs[:, :, None]).sum(1))):
            want = res.double() + mult * plain.layer_norm(total.double(), w.double(), b.double(), EPS)
            dev = [tuple(t.to(DEV) for t in terms)] if isinstance(terms, tuple) else \
                  [t.to(DEV) for t in (terms if isinstance(terms, list) else [terms])]
            r32 = res.to(DEV).clone()
            act = ops.norm_add(r32, dev, w.to(DEV), EPS, center=True, bias=b.to(DEV), mult=mult, act_dtype=BF16)
            close(r32, want, F32, f"layer norm added, factor {mult}")
            assert torch.equal(act, r32.to(BF16))
            r16 = res.to(DEV).clone()
            ops.norm_add(r16, dev, w.to(DEV, BF16), EPS, center=True, bias=b.to(DEV, BF16), mult=mult)
            rounded = res.double() + mult * plain.layer_norm(total.double(), w.to(BF16).double(), b.to(BF16).double(), EPS)
            close(r16, rounded, F32, "bfloat16 weight and bias", tol=1e-5)
    # without a bias, and the root-mean-square norm with a factor: what the token-side sublayer adds
    r32 = res.to(DEV).clone()
    ops.norm_add(r32, y.to(DEV), w.to(DEV), EPS, center=True, mult=0.25)
    close(r32, res.double() + 0.25 * plain.layer_norm(y.double(), w.double(), 0.0, EPS), F32, "no bias")
    r32 = res.to(DEV).clone()
    ops.norm_add(r32, y.to(DEV), w.to(DEV), EPS, mult=0.25)
    close(r32, res.double() + 0.25 * plain.rms_norm(y.double(), w.double(), EPS), F32, "rms norm with a factor")
    # that taking the mean off would show
    assert float((plain.layer_norm(y.double(), w.double(), b.double(), EPS) - plain.rms_norm(y.double(), w.double(), EPS)).abs().max()) > 0.1


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("width", [72, 1001, 4096])
def test_the_last_layer_norm_has_a_bias_and_reads_picked_rows(dtype, width):
    res = rnd((6, width), 1, 2.0) + 1.0
    w, b = 1 + rnd((width,), 2, 0.3), rnd((width,), 3, 0.5)
    picks = torch.tensor([5, 0, 3], dtype=torch.int32, device=DEV)
    got = ops.add_layernorm(res.to(DEV), [], w.to(DEV, dtype), EPS, dtype, rows=picks, bias=b.to(DEV, dtype))
    close(got, plain.layer_norm(res.double(), w.double(), b.double(), EPS)[[5, 0, 3]], dtype, "picked rows")
    got = ops.add_layernorm(res.to(DEV), [], w.to(DEV, dtype), EPS, dtype)
    close(got, plain.layer_norm(res.double(), w.double(), 0.0, EPS), dtype, "no bias")


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("width,dim,layers,which", [(40, 12, 3, 1), (72, 5, 2, 0), (96, 24, 4, 3), (50, 1, 1, 0)])
def test_the_token_side_input_reads_its_own_slice_of_the_second_embedding(dtype, width, dim, layers, which):
    vocab = 37
    raw = {"architecture": ARCH, "vocab": vocab, "width": width, "norm": {"eps": EPS}, "token_side": {"dim": dim},
           "layers": [layer("attention", attn(1, 1, 8, 8), None)] * layers}
    spec = retudra_spec(RetudraConfig.from_dict(raw))
    role, side = spec.layers[which].parts["side"]
    part, tensors = random_part(role, side, dtype, 11, 0.5)
    tokens = random_tokens(9, vocab, 3)
    x = rnd((9, width), 5)
    batch = build_step_batch([StepEntry("r", tokens, [])], lambda _r: 0, lambda _r: 0, vocab, DEV)
    y = part.forward(x.to(DEV, dtype), batch)
    y = y.float().sum(0) if y.dim() == 3 else y.float()
    e = tensors["side.embed"].double()[tokens][:, which * dim:(which + 1) * dim]
    g = plain.gelu_tanh(x.double() @ tensors[f"l{which}.side.gate"].double().T) * e
    close(y, g @ tensors[f"l{which}.side.proj"].double().T, dtype, "token side")
    # and through the block's norm: the plain function with the norm's weight
    named = dict(tensors, **{f"l{which}.side.norm": torch.ones(width)})
    want = plain.token_side(x.double(), torch.tensor(tokens), which, dim, named, EPS)
    close(plain.rms_norm(y.double().cpu(), 1.0, EPS), want, dtype, "token side, normed")


ATTENTIONS = [
    # (mixer, page, rows, positions made loud)
    (attn(6, 2, 16, 24, scale=0.35, rot=rot(10000.0, 12), mask=(24, 5)), 4, 70, (4, 5, 70 - 24, 70 - 25, 30, 31)),
    (attn(2, 2, 32, 8, scale=0.2, rot=rot(100.0, 32), mask=(9, 3)), 4, 40, (2, 3, 40 - 9, 40 - 10)),
    (attn(5, 1, 12, 6, scale=0.5), 8, 33, (0, 16)),                                        # no window, no rotation
    (attn(1, None, 10, 14, scale=0.6, rot=rot(20.0, 6), mask=(7, 0)), 8, 30, (22, 23)),      # a window that keeps nothing
    (attn(3, 1, 24, 16, scale=0.3, rot=rot(300.0, 8), mask=(5, 40)), 4, 36, (0, 30)),        # keeps more than it has
    (attn(6, 2, 64, 64, scale=0.125, rot=rot(250000.0, 16), mask=(40, 18)), 16, 150, (17, 18, 109, 110, 31, 32)),
    (attn(2, 1, 128, 64, scale=0.09, rot=rot(800.0, 64), mask=(33, 32)), 16, 120, (31, 32, 86, 87)),
    (attn(8, 2, 64, 32, scale=0.125, rot=rot(1000.0, 64), mask=(16, 16)), 16, 100, (15, 16, 83, 84)),
    (attn(4, 4, 48, 80, scale=0.15, rot=rot(1000.0, 16), mask=(64, 1)), 32, 200, (0, 1, 135, 136)),
]


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("case", range(len(ATTENTIONS)))
def test_the_windowed_attention_keeps_the_first_keys_in_every_cut(dtype, case):
    mixer, page, T, loud = ATTENTIONS[case]
    mixer_case("attention", mixer, dtype, 20 + case, T, page=page, loud=loud)


@pytest.mark.parametrize("dtype", [F32, BF16])
def test_a_far_kept_key_is_found_and_the_one_behind_it_is_not(dtype):
    """One query at the end of 400 rows; the key at position keep_first - 1 is made the only one its score can find
    (query and key share one large direction), and its value is loud.  The same with the key at keep_first: hidden."""
    keep, T, W = 6, 400, 48
    mixer = attn(2, 1, 16, 16, scale=1.0, mask=(10, keep))
    raw, spec = one_layer("attention", mixer, width=W)
    for target, seen in ((keep - 1, True), (keep, False)):
        part, tensors = random_part("mixer", spec.layers[0].mixer, dtype, 77, 0.2)
        x = rnd((T, W), 3, 0.5)
        x[target] = 8.0 * x[T - 1]          # the same direction as the last row: its key meets the last query
        w = lambda name: tensors["l0.mix." + name].double()
        want = plain.attention(x.double(), mixer, w, EPS)
        hidden = plain.attention(torch.cat([x[:target], x[target + 1:]]).double(), mixer, w, EPS)
        differs = float((want[-1] - hidden[-1]).abs().max()) / float(want.abs().max())
        assert (differs > 0.05) == seen, "the test's own inputs must make the key matter exactly where it is seen"
        for c in ((1000,), (7, 1)):
            close(run_mixer(part, x, c, page=4, dtype=dtype), want, dtype, f"far key at {target}, cut {c}")


LATENTS = [
    (latent(4, 16, 8, 12, 24, scale=0.3, rot=rot(500.0, 8)), 4, 50),
    (latent(1, 10, 6, 14, 18, scale=0.4, rot=rot(50.0, 4)), 8, 40),          # one head; only part of the rotated part turns
    (latent(4, 32, 32, 48, 64, scale=0.12, rot=rot(250000.0, 32)), 16, 130),
    (latent(8, 64, 32, 48, 112, scale=0.1, rot=rot(100000.0, 32)), 16, 90),
    (latent(3, 8, 2, 8, 6, scale=0.5, rot=rot(10.0, 2)), 4, 30),
]


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("case", range(len(LATENTS)))
def test_the_latent_attention_rotates_halves_and_gates_its_heads(dtype, case):
    mixer, page, T = LATENTS[case]
    # (the folded form rounds W_uk^T q and the summed latents, eight heads over a latent of 112: 2.8e-2 measured)
    mixer_case("latent_attention", mixer, dtype, 40 + case, T, page=page, loud=(0, T // 2),
               tol=4e-2 if (dtype == BF16 and case == 3) else None)
    if case == 0 and dtype == F32:      # that the other pairing and a missing gate would show
        raw, spec = one_layer("latent_attention", mixer)
        part, tensors = random_part("mixer", spec.layers[0].mixer, dtype, 40, 0.3)
        x = rnd((20, raw["width"]), 140)
        w = lambda name: tensors["l0.mix." + name].double()
        want = plain.latent_attention(x.double(), mixer, w, EPS)
        no_gate = lambda name: torch.zeros_like(w(name)) if name == "g" else w(name)
        assert float((2 * plain.latent_attention(x.double(), mixer, no_gate, EPS) - want).abs().max()) > 0.01 * float(want.abs().max())


DELTAS = [
    (delta(4, 2, 16, 12), 50),
    (delta(3, None, 10, 6, conv=2, decay_rank=3, gate_rank=5), 40),
    (delta(4, 2, 64, 48, conv=4, decay_rank=16, gate_rank=8), 70),
    (delta(4, 1, 128, 16, conv=5, decay_rank=12, gate_rank=4), 45),
    (delta(2, 1, 130, 20, conv=1, decay_rank=1, gate_rank=1), 37),
    (delta(5, 5, 24, 40, conv=3, decay_rank=7, gate_rank=9), 66),
]
DELTA_FILLS = {".A_log": lambda t, s: rnd(t.shape, s) - 1.0, ".dt_bias": lambda t, s: rnd(t.shape, s) - 1.0,
               ".conv": lambda t, s: rnd(t.shape, s, 0.5) + 0.2, ".a2": lambda t, s: t * 4.0, ".g2": lambda t, s: t * 4.0}


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("case", range(len(DELTAS)))
def test_the_delta_rule_decays_every_key_channel_by_itself(dtype, case):
    mixer, T = DELTAS[case]
    # a loud token: the next taps - 1 rows hear it through the convolution, later ones only through the state
    mixer_case("channel_delta", mixer, dtype, 60 + case, T, loud=(9,), fills=DELTA_FILLS, std=0.25,
               cuts=CUTS + [(9, 1, 1, 1, 30), (10, 1)], tol=2e-4 if dtype == F32 else None)


def test_the_delta_rule_over_long_decoding_and_that_one_decay_a_head_would_differ():
    mixer = delta(2, 1, 32, 16, conv=4, decay_rank=6, gate_rank=6)
    raw, spec = one_layer("channel_delta", mixer)
    part, tensors = random_part("mixer", spec.layers[0].mixer, F32, 90, 0.25, DELTA_FILLS)
    x = rnd((460, raw["width"]), 91)
    w = lambda name: tensors["l0.mix." + name].double()
    want = plain.channel_delta(x.double(), mixer, w, EPS)
    got = run_mixer(part, x, (60,) + (1,) * 400, dtype=F32)
    close(got, want, F32, "400 rows decoded one by one", tol=2e-4)
    # a decay that is the same for every channel of a head (the first channel's) gives another result
    same = lambda name: w(name).view(2, 32, -1)[:, :1].expand(2, 32, -1).reshape(64, -1) if name == "a2" else \
        (w(name).view(2, 32)[:, :1].expand(2, 32).reshape(64) if name == "dt_bias" else w(name))
    other = plain.channel_delta(x.double(), mixer, same, EPS)
    assert float((other - want).abs().max()) > 0.02 * float(want.abs().max())


ROUTERS = [
    # (experts, identity, top, groups, width, ff)
    (6, 2, 2, (4, 2), 72, 40), (5, 0, 3, None, 40, 24), (4, 0, 1, None, 42, 30), (7, 1, 3, (2, 1), 96, 48),
    (7, 2, 2, (3, 2), 80, 40), (2, 1, 2, None, 64, 16), (30, 2, 6, (8, 3), 128, 64), (1, 3, 2, (2, 1), 48, 32),
]


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("case", range(len(ROUTERS)))
def test_the_softmax_router_chooses_within_groups_and_identity_experts_hand_back_the_input(dtype, case):
    experts, identity, top, groups, width, ff = ROUTERS[case]
    mlp = moe(experts, top, ff, identity=identity, groups=groups)
    raw, spec = one_layer("attention", attn(1, 1, 8, 8), mlp, width=width)
    fills = {".router": lambda t, s: t * 4.0, ".correction": lambda t, s: rnd(t.shape, s, 0.1)}
    part, tensors = random_part("feed_forward", spec.layers[0].feed_forward, dtype, 300 + case, 0.3, fills)
    for rows in (1, 9, 70, 300):
        x = rnd((rows, width), 7 + rows)
        w = lambda name: tensors["l0.mlp." + name].double() if ("l0.mlp." + name) in tensors else None
        # the choice itself, where no two choice numbers are close
        chosen, weights = plain.route(x.double(), mlp["router"], w("router"), w("correction"))
        ids, got_w = ops.moe_route(x.to(DEV, dtype), tensors["l0.mlp.router"].to(DEV, dtype),
                                   tensors["l0.mlp.correction"].to(DEV, dtype), top=top, scale=1.0, score="softmax",
                                   groups=groups[0] if groups else 1, keep_groups=groups[1] if groups else 1,
                                   normalize=False)
        s = torch.softmax(x.double() @ w("router").T, -1) + w("correction")
        gaps = (s[:, :, None] - s[:, None, :]).abs() + 10.0 * torch.eye(s.shape[1])
        clear = gaps.flatten(1).min(1).values > 1e-5      # (the router's sums are 32-bit in both modes, from the same inputs)
        assert clear.sum() >= rows // 2 or rows == 1
        assert torch.equal(ids.cpu().long()[clear], chosen[clear]), "the chosen experts, in the order they were chosen"
        close(got_w.cpu()[clear], weights[clear], dtype, "their weights are the scores themselves")
        if bool(clear.all()):
            outs = part.forward(x.to(DEV, dtype))
            (y, coef), = outs
            got = (y.double() * coef.double()[:, :, None]).sum(1)
            close(got, plain.mixture(x.double(), mlp, w), dtype, f"the mixture's output at {rows} rows")
    if identity:
        assert float(plain.mixture(x.double(), mlp, w).abs().max()) > 0


def test_a_group_that_is_not_kept_counts_as_minus_infinity_not_zero():
    """Corrections below zero make every choice number of the kept groups negative: experts of a dropped group (whose
    numbers, were they counted as 0, would be the largest) must still not be chosen."""
    width, experts = 32, 8
    router = rnd((experts, width), 1, 0.5)
    correction = torch.full((experts,), -2.0)
    correction[5] = -1.0          # group 2 of four groups of two wins; only its experts 4 and 5 may be chosen
    x = rnd((50, width), 2)
    ids, _ = ops.moe_route(x.to(DEV), router.to(DEV), correction.to(DEV), top=2, scale=1.0, score="softmax", groups=4,
                           keep_groups=1, normalize=False)
    assert set(ids.cpu().flatten().tolist()) == {4, 5}
    chosen, _ = plain.route(x.double(), {"top": 2, "groups": {"count": 4, "keep": 1}}, router.double(), correction.double())
    assert set(chosen.flatten().tolist()) == {4, 5}


# ----------------------------------------------------------------------------------- whole models

@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    base = tmp_path_factory.mktemp("retudra")
    return {name: make_model_dir(base, name) for name in TINY}


def requests_for(cfg, lengths, seed):
    return {f"r{i}": random_tokens(n, cfg["vocab"], seed + i) for i, n in enumerate(lengths)}


def engine_for(folder, name, dtype, tokens, slots=4, **kw):
    return Engine.from_folder(folder, dtype=dtype, page_size=TINY[name][1], max_tokens=tokens, max_slots=slots, **kw)


def references(cfg, weights, reqs):
    return {rid: plain.forward(cfg, weights, toks) for rid, toks in reqs.items()}


OWN_MARGIN, EARLIER_MARGIN = 0.1, 0.05


def close_calls(cfg, weights, reqs):
    """{request: bool [T]}: rows that bfloat16 is not held to, because a router's choice there, or at an earlier row
    of the request that this one attends to or carries in its state, was a close call in the plain implementation:
    the last chosen and the first unchosen number (of experts or of groups) less than a tenth of the two rivals' scores
    apart at the row itself, or less than a twentieth of them at an earlier row.  Rounding moves the hidden state by about a
    hundredth, which decides such a call the other way, and another expert is another function.  float32 is held to
    every row."""
    out = {}
    for rid, toks in reqs.items():
        plain.route_margins.clear()
        plain.forward(cfg, weights, toks)
        if not plain.route_margins:
            out[rid] = torch.zeros(len(toks), dtype=torch.bool)
            continue
        own = torch.stack(plain.route_margins).min(0).values
        earlier = torch.cat([torch.full((1,), float("inf"), dtype=own.dtype), torch.cummin(own, 0).values[:-1]])
        out[rid] = (own < OWN_MARGIN) | (earlier < EARLIER_MARGIN)
    return out


MODEL_TOL = {"float32": 5e-5, "bfloat16": 3e-2}
UNIT = {"float32": 2.0 ** -24, "bfloat16": 2.0 ** -9}     # half a unit in the last place


def row_limits(cfg, weights, reqs, ref, dtype, floor=None):
    """What rounding may do to each row.  The norms on the sublayers' outputs and the norm on the delta rule's
    read-out magnify the rounding of what lies in front where terms nearly cancel (a read-out whose q.k is near zero
    keeps only its sign through the norm; a router's close call changes an expert), row by row differently and most at
    a sequence's first tokens.  A row's limit is eight times what the plain logits of that row change by when every
    matrix entry, or every entry of every matrix product, moves by up to half a unit in the last place of the type,
    and no less than the usual tolerance."""
    limits = {rid: torch.full((len(toks),), floor or MODEL_TOL[dtype], dtype=torch.float64) for rid, toks in reqs.items()}
    jitter = lambda t, g: t * (1 + (torch.rand(t.shape, generator=g, dtype=torch.float64) - 0.5) * 2.0 * UNIT[dtype])
    for trial in range(3):
        g = torch.Generator().manual_seed(1000 + trial)
        moved = weights
        if trial == 0:
            moved = {k: (jitter(v.double(), g) if v.dim() == 2 else v) for k, v in weights.items()}
        else:
            plain.after_product = lambda y: jitter(y, g)
        try:
            for rid, toks in reqs.items():
                err = (plain.forward(cfg, moved, toks) - ref[rid]).abs().max(1).values / ref[rid].abs().max()
                limits[rid] = torch.maximum(limits[rid], 8.0 * err)
        finally:
            plain.after_product = None
    return limits


def check(got, ref, limits, dtype, what, floor=None, exempt=None):
    """Every row within its limit, and the median row within the usual tolerance.  exempt {request: bool [T]}: rows
    that only have to be finite (bfloat16 behind a router's close call)."""
    errors = []
    for rid, want in ref.items():
        scale = float(want.abs().max())
        for p in range(want.shape[0]):
            row = got[(rid, p)].double()
            assert torch.isfinite(row).all(), f"{what}: non-finite logits at {rid}:{p}"
            err = float((row - want[p]).abs().max()) / scale
            if exempt is not None and dtype == "bfloat16" and bool(exempt[rid][p]):
                continue
            errors.append(err)
            assert err <= float(limits[rid][p]), f"{what}: row {rid}:{p} is off by {err:.3e}, its limit is {float(limits[rid][p]):.3e}"
    assert sorted(errors)[len(errors) // 2] <= (floor or MODEL_TOL[dtype]), f"{what}: the median row is off by more than the tolerance"


CASES = [(name, dtype) for name in TINY for dtype in ("float32", "bfloat16")]


@pytest.mark.parametrize("name,dtype", CASES)
def test_whole_prompts_decoding_and_portions_equal_the_plain_logits(folders, name, dtype):
    cfg, weights = read_folder(folders[name])
    reqs = requests_for(cfg, (1, 2, 23, 61, 130), 100)
    ref = references(cfg, weights, reqs)
    eng = engine_for(folders[name], name, dtype, 160)
    limits = row_limits(cfg, weights, reqs, ref, dtype)
    exempt = close_calls(cfg, weights, reqs)
    assert sum(int((~e).sum()) for e in exempt.values()) >= 40, "too few rows are left for bfloat16 to be held to"
    for how, make in (("whole", replay.whole), ("decode", lambda r, t: replay.prefill_then_decode(r, t, tail=80)),
                      ("portions", replay.portions), ("pairs", lambda r, t: replay.portions(r, t, sizes=(2,))),
                      ("single tokens", lambda r, t: replay.portions(r, t, sizes=(1,)))):
        got = {}
        for rid, toks in reqs.items():
            got.update(replay.run_steps(eng, make(rid, toks)))
        check(got, ref, limits, dtype, f"retudra {name} {dtype} {how}", exempt=exempt)
        assert eng.cache.free_tokens() == eng.cache.pool_tokens()


@pytest.mark.parametrize("name,dtype", CASES)
def test_mixed_batches_with_pages_and_slots_used_again(folders, name, dtype):
    cfg, weights = read_folder(folders[name])
    reqs = requests_for(cfg, (40, 7, 75, 2, 33, 58, 19, 90), 210)
    ref = references(cfg, weights, reqs)
    # three slots and a pool that just holds the three longest live requests: every slot and page is used again
    eng = engine_for(folders[name], name, dtype, 90 + 75 + 58 + 3 * TINY[name][1], slots=3)
    alone = engine_for(folders[name], name, dtype, 128, slots=1)
    limits = row_limits(cfg, weights, reqs, ref, dtype)
    exempt = close_calls(cfg, weights, reqs)
    for seed in (1, 2):
        steps = replay.mixed(reqs, max_live=3, seed=seed, decode_tail=12, max_portion=17)
        got = replay.run_steps(eng, steps)
        check(got, ref, limits, dtype, f"retudra {name} {dtype} mixed {seed}", exempt=exempt)
        assert eng.cache.free_slot_count == 3 and eng.cache.free_tokens() == eng.cache.pool_tokens()
    if dtype == "float32":      # in 32 bits a row is the same bits in a batch and alone
        for rid in ("r0", "r3", "r5"):
            solo = replay.run_steps(alone, replay.whole(rid, reqs[rid]))
            for key, row in solo.items():
                assert torch.equal(row, got[key]), f"{key} differs between the batch and the request alone"


def test_a_long_prompt_and_long_decoding_stay_with_the_plain_logits(folders):
    # (R in bfloat16 would be held to next to nothing: among 700 rows a router's close call comes early)
    for name, dtype in (("R", "float32"), ("Q", "float32"), ("Q", "bfloat16")):
        cfg, weights = read_folder(folders[name])
        toks = random_tokens(700, cfg["vocab"], 31)
        ref = {"a": plain.forward(cfg, weights, toks)}
        eng = engine_for(folders[name], name, dtype, 720)
        got = replay.run_steps(eng, replay.prefill_then_decode("a", toks, tail=300))
        floor = 1e-4 if dtype == "float32" else None      # a thousand steps of a 32-bit recurrence
        check(got, ref, row_limits(cfg, weights, {"a": toks}, ref, dtype, floor), dtype, f"long {name} {dtype}", floor,
              exempt=close_calls(cfg, weights, {"a": toks}))


def test_pages_that_the_window_has_passed_go_back_and_the_first_ones_stay(folders):
    cfg, _ = read_folder(folders["R"])      # a window of 40 that keeps 18 keys, pages of 16
    eng = engine_for(folders["R"], "R", "float32", 400)
    free = eng.cache.free_tokens()
    toks = random_tokens(300, cfg["vocab"], 5)
    replay.run_steps(eng, [{"entries": [("a", toks[:200], [199])], "end": []}] +
                     [{"entries": [("a", toks[i:i + 1], [0])], "end": []} for i in range(200, 300)])
    windowed = [g for g in eng.cache.groups if g.window is not None]
    assert len(windowed) == 1 and windowed[0].keep_first == 18
    table = windowed[0].tables["a"]
    held = [i for i, p in enumerate(table.pages) if p >= 0]
    # the two pages of the 18 kept keys, and the pages from the one that holds key 300 - 40 + 1 on
    assert held == [0, 1] + list(range((300 - 40 + 1) // 16, -(-300 // 16)))
    eng.end_request("a")
    assert eng.cache.free_tokens() == free


def test_captured_steps_give_the_bits_of_eager_ones(folders):
    cfg, _ = read_folder(folders["P"])
    reqs = requests_for(cfg, (30, 30, 41), 300)
    steps = []
    for rid, toks in reqs.items():      # equal portions, then decoding: shapes repeat and are captured
        steps += [{"entries": [(rid, toks[i:i + 6], list(range(len(toks[i:i + 6]))))], "end": []} for i in range(0, 24, 6)]
    live = list(reqs)
    for i in range(24, 30):
        steps.append({"entries": [(rid, reqs[rid][i:i + 1], [0]) for rid in live], "end": live if i == 29 else []})
    out = {}
    for graphs in (False, True):
        eng = engine_for(folders["P"], "P", "bfloat16", 160, cuda_graph=graphs)
        out[graphs] = replay.run_steps(eng, steps)
        assert (eng.graph_replays > 0) == graphs
    assert all(torch.equal(out[True][k], out[False][k]) for k in out[False])


def _plain_greedy(cfg, weights, prompt, n):
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(plain.forward(cfg, weights, toks)[-1].argmax()))
    return toks[len(prompt):]


@pytest.mark.parametrize("name", ["P", "Q"])
def test_greedy_generation_through_the_scheduler_equals_the_plain_implementation(folders, name):
    cfg, weights = read_folder(folders[name])
    prompts = [random_tokens(n, cfg["vocab"], 400 + n) for n in (3, 12, 29, 18, 7)]
    want = [_plain_greedy(cfg, weights, p, 24) for p in prompts]
    # two slots for five requests, portions of at most eight tokens: slots and pages are used again
    llm = LLM(folders[name], dtype="float32", page_size=TINY[name][1], kv_cache_tokens=160, max_seq_len=64, num_slots=2,
              chunked_prefill_size=8)
    outs = llm.generate(prompts, max_tokens=24)
    assert [o.response_token_ids for o in outs] == want
    assert all(o.finish_reason == "length" for o in outs)
