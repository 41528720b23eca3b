"""Tazitar on the GPU against the plain implementation (`plain_tazitar.py`): every mechanism alone as the part the
engine runs, in cuts of every size, and whole models through `Engine.step`, the scheduler and `LLM.generate`.

Tolerances.  float32: 2e-5 of the largest plain logit for whole models, 5e-5 of the largest plain output for a
mechanism alone (the plain side is float64; the engine adds in 32 bits).  bfloat16: 3e-2 of the largest plain logit
for whole models, 2.5e-2 of the largest plain output for a mechanism alone.
"""
import pytest
import torch

import plain_tazitar as plain
import replay
from arle_amd import LLM
from arle_amd.cache import CacheManager
from arle_amd.engine import Engine, StepEntry
from arle_amd.engine.batch import build_step_batch
from arle_amd.kernels import ops
from arle_amd.parts import PartSpec
from arle_amd.parts.base import Runtime, build_part
from arle_amd.parts.hyper import StreamWrite
from tiny import random_tokens, read_folder
from tiny_tazitar import TINY, attn, delta, make_model_dir, rot

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
F32, BF16 = torch.float32, torch.bfloat16
TOL = {F32: 5e-5, BF16: 2.5e-2}


def rnd(shape, seed, std=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * std).to(BF16).float()     # values that bfloat16 holds exactly


def close(got, want, dtype, what, tol=None):
    got, want = got.double().cpu(), want.double()
    assert torch.isfinite(got).all(), what
    err = float((got - want).abs().max()) / float(want.abs().max())
    assert err <= (tol or TOL[dtype]), f"{what}: {err:.3e}"


def make_part(role, kind, params, tensors, dtype, weights=None):
    rt = Runtime(device=torch.device(DEV), act_dtype=dtype)
    held = {k: v.to(DEV, dtype) for k, v in tensors.items()}
    return build_part(role, PartSpec(kind, params, weights or {k: k for k in tensors}), held.__getitem__, rt)


def run_mixer(part, x, cuts, *, page=4, dtype=F32):
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
        at += n
    cache.check()
    return torch.cat(outs)


CUTS = [(1000,), (1,), (2,), (5, 2, 7, 3, 1, 16, 2)]


# ----------------------------------------------------------------------------------- mechanisms alone

def plain_streams(x, y, mix, out_w):
    """x [T, S, W] float64 -> the streams once y is written through (mix, out_w)."""
    return torch.einsum("tsw,sk->tkw", x, mix) + out_w[None, :, None] * y[:, None, :]


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("streams,width,rows", [(4, 72, 5), (3, 1000, 3), (1, 64, 4), (5, 101, 6), (2, 4100, 2), (9, 40, 3)])
def test_residual_streams_are_written_and_read_through_their_connections(dtype, streams, width, rows):
    S = streams
    emb = rnd((rows, width), 1, 2.0)
    conn = lambda seed: {"weight": 1 + rnd((width,), seed, 0.3), "in": 1.0 / S + rnd((S,), seed + 1, 0.3),
                         "out": 1 + rnd((S,), seed + 2, 0.3), "mix": torch.eye(S) + rnd((S, S), seed + 3, 0.3)}
    params = {"width": width, "eps": 1e-5, "streams": S}
    a, b = conn(10), conn(20)
    # the connections' numbers stay 32-bit in both modes (they are converted when the part is built)
    pa = make_part("norm", "hyper_rmsnorm", params, a, F32)
    pb = make_part("norm", "hyper_rmsnorm", params, b, F32)
    last = make_part("norm", "hyper_rmsnorm", dict(params, connect=False), {"weight": a["weight"]}, F32)
    for p in (pa, pb, last):
        p.rt = Runtime(device=torch.device(DEV), act_dtype=dtype)
    norm = lambda u, w: plain.rms_unit(u, 1e-5) * w.double()
    # the first read makes the streams out of the embedding's output
    x, got = pa.read(emb.to(DEV))
    want_x = emb.double()[:, None, :].expand(rows, S, width)
    assert x.shape == (rows, S, width) and got.dtype == dtype
    close(x, want_x, F32, "the streams at the start", tol=0)
    close(got, norm(torch.einsum("tsw,s->tw", want_x, a["in"].double()), a["weight"]), dtype, "the first read")
    # a write and the next read in one pass: the output as a tensor of the activation type, then as a stack
    y1 = rnd((rows, width), 2)
    x, got = pb.read(x, StreamWrite(y1.to(DEV, dtype), pa))
    want_x = plain_streams(want_x, y1.double(), a["mix"].double(), a["out"].double())
    close(x, want_x, F32, "the streams after a write")
    close(got, norm(torch.einsum("tsw,s->tw", want_x, b["in"].double()), b["weight"]), dtype, "the read behind a write")
    y2 = rnd((3, rows, width), 3)
    pending = StreamWrite(y2.to(DEV), pb)
    close(pending.settled(x), plain_streams(want_x, y2.double().sum(0), b["mix"].double(), b["out"].double()).sum(1), F32,
          "the sum of the streams as the debugging dump forms it")
    # the last norm reads the plain sum of picked rows, behind a pending write, and writes nothing
    before = x.clone()
    picks = torch.tensor([rows - 1, 0], dtype=torch.int32, device=DEV)
    got = last.add_norm(x, pending, rows=picks)
    want_x = plain_streams(want_x, y2.double().sum(0), b["mix"].double(), b["out"].double())
    close(got, norm(want_x.sum(1), a["weight"])[[rows - 1, 0]], dtype, "the last norm")
    assert torch.equal(x, before)
    # in place: a write of all rows leaves what the plain formula leaves
    x2, _ = pa.read(x, pending)
    assert x2.data_ptr() == x.data_ptr()
    close(x2, want_x, F32, "the streams after a second write")


@pytest.mark.parametrize("width,rows", [(72, 5), (1001, 3), (4096, 2)])
def test_two_outputs_are_normed_each_and_averaged(width, rows):
    a, b = rnd((rows, width), 1, 3.0), rnd((2, rows, width), 2, 0.1)
    wa, wb = 1 + rnd((width,), 3, 0.3), 1 + rnd((width,), 4, 0.3)
    want = 0.5 * (plain.rms_unit(a.double(), 1e-5) * wa.double() + plain.rms_unit(b.double().sum(0), 1e-5) * wb.double())
    got = ops.pair_norm(a.to(DEV), b.to(DEV), wa.to(DEV), wb.to(DEV), 1e-5, 0.5)
    close(got, want, F32, "a tensor and a stack")
    got = ops.pair_norm(a.to(DEV, BF16), b.sum(0).to(DEV, BF16), wa.to(DEV), wb.to(DEV), 1e-5, 0.5)
    want = 0.5 * (plain.rms_unit(a.double(), 1e-5) * wa.double()
                  + plain.rms_unit(b.sum(0).to(BF16).double(), 1e-5) * wb.double())
    close(got, want, F32, "two bfloat16 tensors")


KINDS = {"attention": ("weighted_before", None, False), "sink0": ("unit_after", "zero", False),
         "attention_2": ("unit_after", "learned", True)}


def attention_part(width, m, kind, dtype, seed, eps=1e-5):
    qk_norm, sink, inter = KINDS[kind]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    t = {"q": rnd((H * D, width), seed, 0.3), "k": rnd((G * D, width), seed + 1, 0.3), "v": rnd((G * Dv, width), seed + 2, 0.3),
         "o": rnd((width, H * Dv), seed + 3, 0.3)}
    names = {k: k for k in t}
    if qk_norm == "weighted_before":
        t.update(q_norm=1 + rnd((D,), seed + 4, 0.4), k_norm=1 + rnd((D,), seed + 5, 0.4))
        names.update(q_norm="q.norm", k_norm="k.norm")
    if sink == "learned":
        t["sink"] = 1.0 + rnd((H,), seed + 6)
        names["sink"] = "sink"
    position = None
    if m.get("rot"):
        r = m["rot"]
        sc = r.get("scaling")
        position = PartSpec("rope_interleaved" if inter else "rope_neox",
                            {"head_dim": D, "rotary_dim": r["dims"], "theta": r["base"], "max_positions": 1,
                             "scaling": tuple(sc[k] for k in ("factor", "original", "fast", "slow")) if sc else None})
    params = {"hidden_size": width, "num_q_heads": H, "num_kv_heads": G, "key_dim": D, "value_dim": Dv, "eps": eps,
              "scale": m["scale"], "softcap": m.get("softcap") or 0.0, "qk_norm": qk_norm, "sink": sink,
              "position": position, "window": None}
    part = make_part("mixer", "rotary_attention", params, t, dtype)
    return part, {names[k]: v.double() for k, v in t.items()}


ATTENTIONS = [("attention", attn(6, 2, 16, 24, 0.35, 6.0, rot(10000.0, 12)), 4),
              ("attention", attn(5, 1, 12, 6, 0.5), 8),                                            # no rotation, no cap
              ("attention", attn(6, 2, 48, 80, 0.15, 20.0, rot(5000.0, 48)), 16),                  # the matrix-core kernel's sizes
              ("sink0", attn(4, 2, 24, 16, 0.5, None, rot(500.0, 8)), 4),
              ("sink0", attn(4, 1, 96, 80, 0.15, None, rot(10000.0, 48)), 16),
              ("sink0", attn(1, 1, 10, 14, 0.6, None, rot(50.0, 6)), 8),
              ("attention_2", attn(6, 3, 16, 8, 0.4, None, rot(3000.0, 16, (4.0, 40, 8.0, 1.0))), 4),
              ("attention_2", attn(4, 2, 64, 64, 0.2, None, rot(250000.0, 64, (2.0, 64, 16.0, 2.0))), 16),
              ("attention_2", attn(3, 3, 24, 40, 0.3, None, rot(10000.0, 10)), 16),
              # head groups that are a multiple of eight: the matrix-core kernel then deals them to the chip's dies
              ("sink0", attn(32, 8, 64, 64, 0.2, None, rot(10000.0, 64)), 16),
              ("attention", attn(16, 16, 32, 32, 0.3, 10.0, rot(100.0, 16)), 16)]


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("kind,m,page", ATTENTIONS)
def test_an_attention_norms_rotates_caps_and_sinks_in_every_cut(dtype, kind, m, page):
    width, T = 40, 70
    part, w = attention_part(width, m, kind, dtype, 30)
    x = rnd((T, width), 7)
    # tokens whose input dwarfs the others right behind a page's border and at the very start
    x[page] *= 4.0
    x[0] *= 3.0
    want = plain.attention(x.double(), w, "", m, 1e-5, torch.arange(T), kind)
    first = None
    for cuts in CUTS:
        got = run_mixer(part, x, cuts, page=page, dtype=dtype)
        close(got, want, dtype, f"{kind} {m} cuts {cuts}")
        if dtype == F32:
            if first is None:
                first = got
            assert torch.equal(got, first), f"{kind}: cuts {cuts} change the bits"


def test_a_sink_takes_its_share_and_leaving_it_out_would_show():
    m = attn(4, 2, 32, 16, 0.3, None, rot(1000.0, 32))
    x = rnd((12, 40), 3)
    for kind in ("sink0", "attention_2"):
        part, w = attention_part(40, m, kind, F32, 50)
        got = run_mixer(part, x, (5, 2), page=4)
        close(got, plain.attention(x.double(), w, "", m, 1e-5, torch.arange(12), kind), F32, kind)
        part.sink = None
        without = run_mixer(part, x, (5, 2), page=4)
        assert float((without - got).abs().max()) > 1e-2 * float(got.abs().max())


@pytest.mark.parametrize("kind", ["attention", "attention_2"])
def test_a_far_key_among_hundreds_is_found(kind):
    # one early token and the last token get inputs that make their key and query line up; the rotation must turn the
    # score by exactly the distance for the attention to find it among 400 others
    T, far, width = 400, 37, 48
    m = attn(2, 1, 32, 16, 1.0, None, rot(10000.0, 32, (4.0, 64, 8.0, 1.0) if kind == "attention_2" else None))
    if kind == "attention":
        m["softcap"] = 50.0
    for dtype in (F32, BF16):
        part, w = attention_part(width, m, kind, dtype, 60)
        x = rnd((T, width), 9, 0.05)
        x[far] = rnd((width,), 10, 3.0)
        x[T - 1] = rnd((width,), 11, 3.0)
        want = plain.attention(x.double(), w, "", m, 1e-5, torch.arange(T), kind)
        for cuts in ((1000,), (390, 1), (64, 3)):
            got = run_mixer(part, x, cuts, page=16, dtype=dtype)
            close(got[-40:], want[-40:], dtype, f"{kind} far key, cuts {cuts}", tol=None if dtype == F32 else 4e-2)


def delta_part(width, m, dtype, seed, eps=1e-5):
    H, G, D, Dv, taps = m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["conv"]
    t = {"q": rnd((G * D, width), seed, 0.3), "k": rnd((G * D, width), seed + 1, 0.3), "v": rnd((H * Dv, width), seed + 2, 0.3),
         "g": rnd((H * Dv, width), seed + 3, 0.3), "o": rnd((width, H * Dv), seed + 4, 0.3),
         "q_conv": 0.2 + rnd((G * D, taps), seed + 5, 0.5), "k_conv": 0.2 + rnd((G * D, taps), seed + 6, 0.5),
         "v_conv": 0.2 + rnd((H * Dv, taps), seed + 7, 0.5), "b": rnd((H, width), seed + 8, 0.3), "a": rnd((H, width), seed + 9, 0.3),
         "A_log": rnd((H,), seed + 10) - 1.0, "dt_bias": rnd((H,), seed + 11) - 1.0, "norm": 1 + rnd((Dv,), seed + 12, 0.3)}
    params = {"hidden_size": width, "heads": H, "kv_heads": G, "key_dim": D, "value_dim": Dv, "conv_taps": taps, "eps": eps}
    part = make_part("mixer", "gated_delta", params, t, dtype)
    return part, {k.replace("_conv", ".conv"): v.double() for k, v in t.items()}


DELTAS = [delta(4, 2, 16, 12), delta(3, 3, 10, 6, conv=2), delta(4, 2, 64, 32, conv=5), delta(5, 1, 40, 10, conv=3),
          delta(2, 1, 24, 20), delta(2, 2, 130, 36, conv=4), delta(1, 1, 8, 70, conv=1),
          delta(32, 8, 64, 144, conv=2)]      # many heads over few q/k heads, nine column tiles a head


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("m", DELTAS)
def test_the_delta_rule_carries_its_state_and_its_taps_through_every_cut(dtype, m):
    width, T = 40, 75
    part, w = delta_part(width, m, dtype, 80)
    x = rnd((T, width), 8)
    # a token whose input dwarfs the others: the taps - 1 tokens behind it still hear it, the next one only through the state
    x[33] *= 5.0
    want = plain.gated_delta_rule(x.double(), w, "", m, 1e-5)
    first = None
    for cuts in CUTS + [(33, 1, 1, 1, 1, 1, 40), (34, 2, 2, 40), (31, 32)]:
        got = run_mixer(part, x, cuts, dtype=dtype)
        close(got, want, dtype, f"delta rule {m} cuts {cuts}", tol=None if dtype == F32 else 3e-2)
        if dtype == F32:
            if first is None:
                first = got
            assert torch.equal(got, first), f"delta rule: cuts {cuts} change the bits"


def test_the_delta_rule_decodes_for_long_and_forgets_at_its_own_rate():
    m = delta(2, 1, 32, 16)
    part, w = delta_part(40, m, F32, 90)
    x = rnd((600, 40), 12)
    want = plain.gated_delta_rule(x.double(), w, "", m, 1e-5)
    got = run_mixer(part, x, (200, 1), page=16)
    close(got, want, F32, "400 tokens decoded one by one behind a portion", tol=2e-4)
    # a head that does not decay (A_log very negative) and one that forgets at once are different heads
    w2 = dict(w)
    w2["A_log"] = torch.tensor([-20.0, 6.0], dtype=torch.float64)
    part.a_log = w2["A_log"].float().to(DEV)
    close(run_mixer(part, x[:90], (7, 2, 1), page=16), plain.gated_delta_rule(x[:90].double(), w2, "", m, 1e-5), F32,
          "extreme decays", tol=2e-4)


@pytest.mark.parametrize("dtype", [F32, BF16])
def test_a_pair_of_mixers_runs_side_by_side_on_their_own_caches(dtype):
    width, T = 40, 50
    left, right = attn(4, 2, 24, 16, 0.5, None, rot(500.0, 8)), delta(4, 2, 16, 12)
    lp, lw = attention_part(width, left, "sink0", dtype, 100)
    rp, rw = delta_part(width, right, dtype, 120)
    rt = Runtime(device=torch.device(DEV), act_dtype=dtype)
    from arle_amd.parts.mixer_pair import MixerPair

    wl, wr = 1 + rnd((width,), 140, 0.3), 1 + rnd((width,), 141, 0.3)
    pair = MixerPair({"width": width, "eps": 1e-5}, {"left_out": wl.to(DEV, dtype), "right_out": wr.to(DEV, dtype)}, rt,
                     {"left": lp, "right": rp})
    need = pair.cache_need()
    assert set(need) == {"left", "right"} and set(need["right"]) == {"S", "conv"}
    w = {"left." + k: v for k, v in lw.items()}
    w.update({"right." + k: v for k, v in rw.items()})
    w.update({"left.out": wl.double(), "right.out": wr.double()})
    x = rnd((T, width), 13)
    want = plain.parallel_mixer(x.double(), w, "", {"left": left, "right": right}, 1e-5, torch.arange(T))
    for cuts in CUTS:
        close(run_mixer(pair, x, cuts, dtype=dtype), want, dtype, f"pair, cuts {cuts}", tol=None if dtype == F32 else 3e-2)


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("width,ff,rows", [(72, 96, 5), (42, 50, 3), (256, 1024, 70), (96, 112, 300)])
def test_the_feed_forward_gates_with_the_tanh_form_of_gelu(dtype, width, ff, rows):
    t = {"gate": rnd((ff, width), 1, 0.3), "up": rnd((ff, width), 2, 0.3), "down": rnd((width, ff), 3, 0.3)}
    part = make_part("feed_forward", "swiglu", {"hidden_size": width, "intermediate_size": ff, "activation": "gelu_tanh",
                                                "float32_out": True}, t, dtype)
    x = rnd((rows, width), 4, 2.0)
    y = part.forward(x.to(DEV, dtype))
    y = y.float().sum(0) if y.dim() == 3 else y.float()
    want = plain.feed_forward(x.double(), {k: v.double() for k, v in t.items()}, "")
    close(y, want, dtype, f"feed-forward {width}x{ff}, {rows} rows")
    silu = make_part("feed_forward", "swiglu", {"hidden_size": width, "intermediate_size": ff}, t, dtype).forward(x.to(DEV, dtype))
    silu = silu.float().sum(0) if silu.dim() == 3 else silu.float()
    assert float((silu.cpu().double() - want).abs().max()) > 1e-2 * float(want.abs().max())      # the two activations differ
    z = torch.linspace(-6, 6, 97)
    assert torch.allclose(plain.gelu_tanh(z.double()), torch.nn.functional.gelu(z.double(), approximate="tanh"), atol=1e-12)


# ----------------------------------------------------------------------------------- whole models

@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    base = tmp_path_factory.mktemp("tazitar")
    return {name: make_model_dir(base, name) for name in TINY}


def requests_for(cfg, lengths, seed):
    return {f"r{i}": random_tokens(n, cfg["vocab"], seed + i) for i, n in enumerate(lengths)}


def engine_for(folder, name, dtype, tokens, slots=4, **kw):
    return Engine.from_folder(folder, dtype=dtype, page_size=TINY[name][1], max_tokens=tokens, max_slots=slots, **kw)


def references(cfg, weights, reqs):
    return {rid: plain.forward(cfg, weights, toks) for rid, toks in reqs.items()}


MODEL_TOL = {"float32": 2e-5, "bfloat16": 3e-2}


UNIT = {"float32": 2.0 ** -24, "bfloat16": 2.0 ** -9}     # half a unit in the last place


def row_limits(cfg, weights, reqs, ref, dtype, floor=None):
    """What rounding may do to each row.  The stream connections, the norms on the two mixers' outputs and the norm on
    the delta rule's read-out magnify the rounding of what lies in front where terms nearly cancel (a read-out whose
    q.k is near zero keeps only its sign through the norm), row by row differently and most at a sequence's first
    tokens.  A row's limit is eight times what the plain logits of that row change by when every matrix entry, or every
    entry of every matrix product, moves by up to half a unit in the last place of the type, and no less than the
    usual tolerance."""
    limits = {rid: torch.full((len(toks),), floor or MODEL_TOL[dtype], dtype=torch.float64) for rid, toks in reqs.items()}
    jitter = lambda t, g: t * (1 + (torch.rand(t.shape, generator=g, dtype=torch.float64) - 0.5) * 2.0 * UNIT[dtype])
    for trial in range(3):
        g = torch.Generator().manual_seed(1000 + trial)
        moved = weights
        if trial == 0:
            moved = {k: (jitter(v.double(), g) if v.dim() == 2 and ".hc" not in k else v) for k, v in weights.items()}
        else:
            plain.after_product = lambda y: jitter(y, g)
        try:
            for rid, toks in reqs.items():
                err = (plain.forward(cfg, moved, toks) - ref[rid]).abs().max(1).values / ref[rid].abs().max()
                limits[rid] = torch.maximum(limits[rid], 8.0 * err)
        finally:
            plain.after_product = None
    return limits


def check(got, ref, limits, dtype, what, floor=None):
    """Every row within its limit, and the median row within the usual tolerance."""
    errors = []
    for rid, want in ref.items():
        scale = float(want.abs().max())
        for p in range(want.shape[0]):
            row = got[(rid, p)].double()
            assert torch.isfinite(row).all(), f"{what}: non-finite logits at {rid}:{p}"
            err = float((row - want[p]).abs().max()) / scale
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
    for how, make in (("whole", replay.whole), ("decode", lambda r, t: replay.prefill_then_decode(r, t, tail=80)),
                      ("portions", replay.portions), ("pairs", lambda r, t: replay.portions(r, t, sizes=(2,))),
                      ("single tokens", lambda r, t: replay.portions(r, t, sizes=(1,)))):
        got = {}
        for rid, toks in reqs.items():
            got.update(replay.run_steps(eng, make(rid, toks)))
        check(got, ref, limits, dtype, f"tazitar {name} {dtype} {how}")


@pytest.mark.parametrize("name,dtype", CASES)
def test_mixed_batches_with_pages_and_slots_used_again(folders, name, dtype):
    cfg, weights = read_folder(folders[name])
    reqs = requests_for(cfg, (40, 7, 75, 2, 33, 58, 19, 90), 210)
    ref = references(cfg, weights, reqs)
    # three slots and a pool that just holds the three longest live requests: every slot and page is used again
    eng = engine_for(folders[name], name, dtype, 90 + 75 + 58 + 3 * TINY[name][1], slots=3)
    alone = engine_for(folders[name], name, dtype, 128, slots=1)
    limits = row_limits(cfg, weights, reqs, ref, dtype)
    for seed in (1, 2):
        steps = replay.mixed(reqs, max_live=3, seed=seed, decode_tail=12, max_portion=17)
        got = replay.run_steps(eng, steps)
        check(got, ref, limits, dtype, f"tazitar {name} {dtype} mixed {seed}")
        assert eng.cache.free_slot_count == 3 and eng.cache.free_tokens() == eng.cache.pool_tokens()
    if dtype == "float32":      # in 32 bits a row is the same bits in a batch and alone
        for rid in ("r0", "r3", "r5"):
            solo = replay.run_steps(alone, replay.whole(rid, reqs[rid]))
            for key, row in solo.items():
                assert torch.equal(row, got[key]), f"{key} differs between the batch and the request alone"


def test_a_long_prompt_and_long_decoding_stay_with_the_plain_logits(folders):
    cfg, weights = read_folder(folders["R"])
    toks = random_tokens(700, cfg["vocab"], 31)
    ref = {"a": plain.forward(cfg, weights, toks)}
    for dtype in ("float32", "bfloat16"):
        eng = engine_for(folders["R"], "R", dtype, 720)
        got = replay.run_steps(eng, replay.prefill_then_decode("a", toks, tail=300))
        floor = 1e-4 if dtype == "float32" else None      # a thousand steps of a 32-bit recurrence
        check(got, ref, row_limits(cfg, weights, {"a": toks}, ref, dtype, floor), dtype, f"long {dtype}", floor)


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
