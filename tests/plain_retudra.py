"""A plain, slow implementation of the Retudra decoder in float64 on the CPU: one function a mechanism, whole
sequences at once, no cache, no kernels.  It shares no code with the engine; the tests compare the two.

`config` is the config.json body as a dictionary, `tensors` a dictionary name -> torch tensor (any float type).
"""
from __future__ import annotations

import math

import torch

F = torch.float64

# a test may set this to a function of a matrix product's result (to move every entry by a rounding, say)
after_product = None


def t64(x):
    return x.to(F)


def mm(x, w):
    """x [.., K] times w [N, K] transposed: every projection goes through here."""
    y = x @ w.T
    return after_product(y) if after_product is not None else y


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def rms_norm(x, weight, eps):
    """x / sqrt(mean(x^2) + eps) * weight over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * weight


def layer_norm(x, weight, bias, eps):
    mean = x.mean(-1, keepdim=True)
    var = ((x - mean) ** 2).mean(-1, keepdim=True)
    return (x - mean) / torch.sqrt(var + eps) * weight + bias


def rotate_half(x, positions, dims, base):
    """x [T, heads, D]: the first `dims` entries of every head turn, entry i with entry i + dims / 2."""
    if not dims:
        return x
    half = dims // 2
    freq = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=F)
    ang = positions.to(F)[:, None] * freq[None, :]            # [T, half]
    cos, sin = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * cos - v * sin, v * cos + u * sin, x[..., dims:]], dim=-1)


def visible(n, size=None, keep_first=0):
    """[n, n] bool: row i sees column j if j <= i and (i - j < size or j < keep_first); size None: every j <= i."""
    i = torch.arange(n)[:, None]
    j = torch.arange(n)[None, :]
    ok = j <= i
    if size is not None:
        ok = ok & ((i - j < size) | (j < keep_first))
    return ok


def softmax_attention(q, k, v, scale, mask):
    """q [T, H, Dk], k [T, H, Dk], v [T, H, Dv] (keys and values already given to every query head) -> [T, H, Dv]."""
    s = torch.einsum("ihd,jhd->hij", q, k) * scale
    s = s.masked_fill(~mask[None], float("-inf"))
    p = torch.softmax(s, dim=-1)
    return torch.einsum("hij,jhd->ihd", p, v)


def attention(h, m, w, eps):
    """The windowed grouped-query attention.  m: the layer's `mixer` dictionary, w(name) -> tensor of the mixer."""
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m.get("kv_heads") or m["heads"], m["dim"], m["vdim"]
    q, k, v = mm(h, w("q")), mm(h, w("k")), mm(h, w("v"))
    q = rms_norm(q, w("q.norm"), eps).view(T, H, D)           # over all heads' entries at once
    k = rms_norm(k, w("k.norm"), eps).view(T, G, D)
    pos = torch.arange(T)
    rot = m.get("rot")
    if rot:
        q, k = rotate_half(q, pos, rot["dims"], rot["base"]), rotate_half(k, pos, rot["dims"], rot["base"])
    rep = H // G
    k = k.repeat_interleave(rep, dim=1)
    v = v.view(T, G, Dv).repeat_interleave(rep, dim=1)
    mask = m.get("mask")
    see = visible(T, mask["size"], mask.get("keep_first", 0)) if mask else visible(T)
    o = softmax_attention(q, k, v, m["scale"], see)
    return mm(o.reshape(T, H * Dv), w("o"))


def latent_attention(h, m, w, eps):
    """Attention whose keys and values are linear maps of one compressed vector a token, with a rotated key part
    that all heads share and a sigmoid gate on the heads' outputs."""
    T = h.shape[0]
    H, D, R, Dv, C = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    q = mm(h, w("q")).view(T, H, D + R)
    d = mm(h, w("dkv"))
    c = rms_norm(d[:, :C], w("dkv.norm"), eps)
    k_rot = d[:, C:].view(T, 1, R)
    pos = torch.arange(T)
    rot = m["rot"]
    q_rot = rotate_half(q[..., D:], pos, rot["dims"], rot["base"])
    k_rot = rotate_half(k_rot, pos, rot["dims"], rot["base"]).expand(T, H, R)
    k_plain = mm(c, w("uk")).view(T, H, D)
    v = mm(c, w("uv")).view(T, H, Dv)
    qq = torch.cat([q[..., :D], q_rot], dim=-1)
    kk = torch.cat([k_plain, k_rot], dim=-1)
    o = softmax_attention(qq, kk, v, m["scale"], visible(T)).reshape(T, H * Dv)
    o = o * torch.sigmoid(mm(h, w("g")))
    return mm(o, w("o"))


def causal_conv(x, taps):
    """x [T, C], taps [C, n] (last column the current token's), zeros in front of the start."""
    T, n = x.shape[0], taps.shape[1]
    padded = torch.cat([torch.zeros(n - 1, x.shape[1], dtype=x.dtype), x], dim=0)
    out = torch.zeros_like(x)
    for j in range(n):
        out = out + padded[j:j + T] * taps[:, j][None, :]
    return out


def channel_delta(h, m, w, eps):
    """The gated delta rule with a decay for every head and key channel."""
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m.get("kv_heads") or m["heads"], m["dim"], m["vdim"]
    q = silu(causal_conv(mm(h, w("q")), w("q.conv"))).view(T, G, D)
    k = silu(causal_conv(mm(h, w("k")), w("k.conv"))).view(T, G, D)
    v = silu(causal_conv(mm(h, w("v")), w("v.conv"))).view(T, H, Dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(mm(h, w("b")))                                        # [T, H]
    a = mm(mm(h, w("a1")), w("a2")) + w("dt_bias")                             # [T, H * D]
    decay = torch.exp(-torch.exp(w("A_log"))[None, :, None] * torch.nn.functional.softplus(a.view(T, H, D)))
    gate = torch.sigmoid(mm(mm(h, w("g1")), w("g2"))).view(T, H, Dv)
    rep = H // G
    out = torch.zeros(T, H, Dv, dtype=F)
    S = torch.zeros(H, D, Dv, dtype=F)
    for t in range(T):
        for j in range(H):
            kt, qt = k[t, j // rep], q[t, j // rep]
            Sj = S[j] * decay[t, j][:, None]
            u = beta[t, j] * (v[t, j] - Sj.T @ kt)
            Sj = Sj + kt[:, None] * u[None, :]
            S[j] = Sj
            out[t, j] = Sj.T @ qt
    out = rms_norm(out, w("norm"), eps) * gate
    return mm(out.reshape(T, H * Dv), w("o"))


def gated_ff(h, gate, up, down):
    return mm(silu(mm(h, gate)) * mm(h, up), down)


# every call of `route` leaves here, a token, how far its choice was from another one: the gap between the last
# chosen and the first unchosen number (experts, and groups), as a fraction of the two rivals' own scores (what moves
# when the router's input moves is the scores; the corrections stand still)
route_margins: list = []


def _gap(numbers, scores, taken):
    """[T]: the taken-th largest of numbers [T, n] less the next one, over the sum of the two rivals' scores
    (infinity where there is no next one, or where the next one cannot be chosen at all)."""
    if taken >= numbers.shape[1]:
        return torch.full((numbers.shape[0],), float("inf"), dtype=numbers.dtype)
    ordered, order = torch.sort(numbers, dim=-1, descending=True)
    rivals = torch.gather(scores, 1, order[:, taken - 1:taken + 1]).sum(-1)
    gap = (ordered[:, taken - 1] - ordered[:, taken]) / (rivals + 1e-30)
    return torch.nan_to_num(gap, nan=float("inf"))


def route(h, r, router, correction):
    """-> (chosen [T, top] indices, weights [T, top]) of a softmax router with grouped choice."""
    E = router.shape[0]
    s = torch.softmax(mm(h, router), dim=-1)
    choice = s + (correction if correction is not None else 0.0)
    groups = r.get("groups")
    margin = torch.full((h.shape[0],), float("inf"), dtype=F)
    if groups:
        per = E // groups["count"]
        best, where = choice.view(-1, groups["count"], per).max(-1)
        best_scores = torch.gather(s.view(-1, groups["count"], per), 2, where[..., None])[..., 0]
        margin = _gap(best, best_scores, groups["keep"])
        kept = torch.topk(best, groups["keep"], dim=-1).indices
        allow = torch.zeros_like(best, dtype=torch.bool).scatter_(1, kept, True)
        choice = choice.masked_fill(~allow.repeat_interleave(per, dim=1), float("-inf"))
    chosen = torch.topk(choice, r["top"], dim=-1).indices
    route_margins.append(torch.minimum(margin, _gap(choice, s, r["top"])))
    return chosen, torch.gather(s, 1, chosen)


def mixture(h, mlp, w):
    """Experts e0.. with a router; the last `identity` outputs of the router stand for experts that hand back h."""
    r = mlp["router"]
    E, ident = r["experts"], r.get("identity", 0)
    chosen, weights = route(h, r, w("router"), w("correction"))
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, f in zip(chosen[t].tolist(), weights[t]):
            y = h[t] if e >= E else gated_ff(h[t], w(f"e{e}.gate"), w(f"e{e}.up"), w(f"e{e}.down"))
            out[t] = out[t] + f * y
    assert ident + E == w("router").shape[0]
    return out


def feed_forward(h, mlp, w):
    if mlp["kind"] == "dense":
        return gated_ff(h, w("gate"), w("up"), w("down"))
    return mixture(h, mlp, w)


def token_side(x, tokens, i, dim, tensors, eps):
    """The layer's own slice of a second embedding, gated by the residual, projected back and RMS-normed."""
    e = t64(tensors["side.embed"])[tokens][:, i * dim:(i + 1) * dim]
    g = gelu_tanh(mm(x, t64(tensors[f"l{i}.side.gate"]))) * e
    y = mm(g, t64(tensors[f"l{i}.side.proj"]))
    return rms_norm(y, t64(tensors[f"l{i}.side.norm"]), eps)


MIXERS = {"attention": attention, "latent_attention": latent_attention, "channel_delta": channel_delta}


def forward(config, tensors, tokens, return_layers=False):
    """tokens: a list of ids -> float64 logits [T, vocab] (and the residual after every layer)."""
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    eps, m = config["norm"]["eps"], config.get("residual_mult", 1.0)
    side = config.get("token_side")
    x = t64(tensors["embed"])[tokens]
    seen = []
    for i, layer in enumerate(config["layers"]):
        p = f"l{i}."
        w_mix = lambda name, p=p: t64(tensors[p + "mix." + name]) if (p + "mix." + name) in tensors else None
        w_mlp = lambda name, p=p: t64(tensors[p + "mlp." + name]) if (p + "mlp." + name) in tensors else None
        y = MIXERS[layer["type"]](x, layer["mixer"], w_mix, eps)
        x = x + m * layer_norm(y, t64(tensors[p + "norm1"]), t64(tensors[p + "norm1.b"]), eps)
        if layer.get("mlp") is not None:
            y = feed_forward(x, layer["mlp"], w_mlp)
            x = x + m * layer_norm(y, t64(tensors[p + "norm2"]), t64(tensors[p + "norm2.b"]), eps)
        if side:
            x = x + m * token_side(x, tokens, i, side["dim"], tensors, eps)
        seen.append(x)
    x = layer_norm(x, t64(tensors["final.norm"]), t64(tensors["final.norm.b"]), eps)
    logits = mm(x, t64(tensors["head"]))
    cap = config.get("logit_softcap")
    if cap:
        logits = cap * torch.tanh(logits / cap)
    return (logits, torch.stack(seen)) if return_layers else logits
