"""A plain, slow implementation of the Tazitar decoder in PyTorch on the CPU, one function per
mechanism, written from the design's equations.  It shares no code with the engine: it reads
config.json as a dictionary and the tensors by name, and keeps nothing between calls.

Notation: T tokens, W model width, S residual streams.  A layer is pre-norm, x += mixer(N1(x)),
x += ff(N2(x)); with residual streams x_1..x_S a sublayer reads N(sum_s a_s x_s) and its output y is
written as x_t <- sum_s M[s, t] x_s + b_t y.  Mixers: a grouped-query attention with weighted q/k norm,
rotate-half rotary positions and tanh-capped scores; a pair of mixers side by side (an attention
whose softmax has a sink of score 0, and a gated delta rule with short convolutions), each normed
over the width and averaged; an attention with interleaved rotary pairs under YaRN scaling and a
learned sink per head.  The feed-forward is gated with the tanh form of gelu.  Layers start..stop-1
of the list may run several times in a row with the same weights.
"""
from __future__ import annotations

import math

import torch
import torch.nn.functional as F


def rms_unit(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


# A test may set this to a function of a matrix product's output (to model the rounding of activations); None in
# ordinary use.
after_product = None


def lin(h, weight):
    """weight [out, in] applied to the rows of h."""
    y = h @ weight.T
    return y if after_product is None else after_product(y)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def rotary_frequencies(rot, dtype=torch.float32):
    """(f_i for i < dims/2, factor on cos and sin).  With `scaling` (YaRN) the slow dimensions are divided by
    `factor`, the fast ones kept, with a linear ramp between the two border dimensions."""
    dims, base = int(rot["dims"]), float(rot["base"])
    half = dims // 2
    i = torch.arange(half, dtype=dtype)
    f = torch.pow(torch.tensor(base, dtype=dtype), -2.0 * i / dims)
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    factor, original = float(sc["factor"]), float(sc["original"])
    at = lambda turns: dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo = max(math.floor(at(float(sc["fast"]))), 0)
    hi = min(math.ceil(at(float(sc["slow"]))), dims - 1)
    ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate(x, positions, rot, interleaved):
    """x [T, heads, D]: the first rot.dims entries of every head are rotated by the angle p f_i; pairs are
    (i, i + dims/2) or, interleaved, (2i, 2i + 1).  rot None: nothing rotates."""
    if rot is None:
        return x
    dims = int(rot["dims"])
    f, mag = rotary_frequencies(rot, x.dtype)
    angle = positions.to(x.dtype)[:, None] * f[None, :]
    cos, sin = (torch.cos(angle) * mag)[:, None, :], (torch.sin(angle) * mag)[:, None, :]
    half = dims // 2
    if interleaved:
        u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    else:
        u, v = x[..., :half], x[..., half:dims]
    a, b = u * cos - v * sin, v * cos + u * sin
    out = x.clone()
    if interleaved:
        out[..., 0:dims:2], out[..., 1:dims:2] = a, b
    else:
        out[..., :half], out[..., half:dims] = a, b
    return out


def causal_softmax_attention(q, k, v, scale, softcap=None, sink=None):
    """q [T, H, D], k [T, G, D], v [T, G, Dv] -> [T, H * Dv].  sink [H]: a term exp(sink_h) in the denominator."""
    T, H, _ = q.shape
    G = k.shape[1]
    rep = H // G
    k = k.repeat_interleave(rep, dim=1)
    v = v.repeat_interleave(rep, dim=1)
    s = torch.einsum("ihd,jhd->hij", q, k) * scale
    if softcap:
        s = softcap * torch.tanh(s / softcap)
    seen = torch.arange(T)[None, :] <= torch.arange(T)[:, None]
    s = s.masked_fill(~seen[None], float("-inf"))
    m = s.max(-1, keepdim=True).values
    if sink is not None:
        m = torch.maximum(m, sink[:, None, None].to(s.dtype))
    e = torch.exp(s - m)
    denom = e.sum(-1, keepdim=True)
    if sink is not None:
        denom = denom + torch.exp(sink[:, None, None].to(s.dtype) - m)
    o = torch.einsum("hij,jhd->ihd", e / denom, v)
    return o.reshape(T, -1)


def attention(h, w, p, m, eps, positions, kind):
    """kind "attention": weighted q/k norm, then rotate-half rotation, capped scores, plain softmax.
    kind "sink0": rotate-half rotation, then unit-rms q and k, a sink of score 0.
    kind "attention_2": interleaved rotation (YaRN), then unit-rms q and k, a learned sink."""
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m.get("kv_heads") or m["heads"], m["dim"], m["vdim"]
    q = lin(h, w[p + "q"]).view(T, H, D)
    k = lin(h, w[p + "k"]).view(T, G, D)
    v = lin(h, w[p + "v"]).view(T, G, Dv)
    sink = None
    if kind == "attention":
        q = rms_unit(q, eps) * w[p + "q.norm"]
        k = rms_unit(k, eps) * w[p + "k.norm"]
        q, k = rotate(q, positions, m.get("rot"), False), rotate(k, positions, m.get("rot"), False)
    else:
        inter = kind == "attention_2"
        q, k = rotate(q, positions, m.get("rot"), inter), rotate(k, positions, m.get("rot"), inter)
        q, k = rms_unit(q, eps), rms_unit(k, eps)
        sink = w[p + "sink"] if inter else torch.zeros(H, dtype=h.dtype)
    o = causal_softmax_attention(q, k, v, m["scale"], m.get("softcap"), sink)
    return lin(o, w[p + "o"])


def short_conv(x, weight):
    """x [T, C], weight [C, taps]: y_t = sum_j weight[:, j] x_(t - taps + 1 + j), zeros before the start."""
    taps = weight.shape[1]
    padded = torch.cat([x.new_zeros(taps - 1, x.shape[1]), x], dim=0)
    return sum(padded[j:j + x.shape[0]] * weight[:, j] for j in range(taps))


def gated_delta_rule(h, w, p, m, eps):
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m.get("kv_heads") or m["heads"], m["dim"], m["vdim"]
    q = F.silu(short_conv(lin(h, w[p + "q"]), w[p + "q.conv"])).view(T, G, D)
    k = F.silu(short_conv(lin(h, w[p + "k"]), w[p + "k.conv"])).view(T, G, D)
    v = F.silu(short_conv(lin(h, w[p + "v"]), w[p + "v.conv"])).view(T, H, Dv)
    unit = lambda x: x / torch.sqrt((x * x).sum(-1, keepdim=True) + 1e-6)
    q, k = unit(q) * D ** -0.5, unit(k)
    q, k = q.repeat_interleave(H // G, dim=1), k.repeat_interleave(H // G, dim=1)
    beta = torch.sigmoid(lin(h, w[p + "b"]))                                               # [T, H]
    decay = torch.exp(-torch.exp(w[p + "A_log"]) * F.softplus(lin(h, w[p + "a"]) + w[p + "dt_bias"]))
    S = h.new_zeros(H, D, Dv)
    out = h.new_zeros(T, H, Dv)
    for t in range(T):
        S = S * decay[t][:, None, None]
        u = beta[t][:, None] * (v[t] - torch.einsum("hdv,hd->hv", S, k[t]))
        S = S + k[t][:, :, None] * u[:, None, :]
        out[t] = torch.einsum("hdv,hd->hv", S, q[t])
    gate = F.silu(lin(h, w[p + "g"])).view(T, H, Dv)
    y = rms_unit(out, eps) * w[p + "norm"] * gate
    return lin(y.reshape(T, -1), w[p + "o"])


def parallel_mixer(h, w, p, m, eps, positions):
    left = attention(h, w, p + "left.", m["left"], eps, positions, "sink0")
    right = gated_delta_rule(h, w, p + "right.", m["right"], eps)
    return 0.5 * (rms_unit(left, eps) * w[p + "left.out"] + rms_unit(right, eps) * w[p + "right.out"])


def feed_forward(h, w, p):
    return lin(gelu_tanh(lin(h, w[p + "gate"])) * lin(h, w[p + "up"]), w[p + "down"])


def layer_order(config):
    n = len(config["layers"])
    loop = config.get("loop")
    if not loop:
        return list(range(n))
    body = list(range(loop["start"], loop["stop"]))
    return list(range(loop["start"])) + body * loop["times"] + list(range(loop["stop"], n))


def forward(config, tensors, tokens, dtype=torch.float64, layer_outputs=None):
    """Logits [T, vocab] of one sequence, every position from 0."""
    w = {n: t.to(dtype) for n, t in tensors.items()}
    eps = float(config["norm"]["eps"])
    positions = torch.arange(len(tokens))
    x = w["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    S = config.get("streams")
    streams = [x.clone() for _ in range(S)] if S else None

    def sublayer(x, streams, prefix, which, fn):
        norm = w[f"{prefix}norm{which}"]
        if streams is None:
            return x + fn(rms_unit(x, eps) * norm), None
        hc = f"{prefix}hc{which}."
        u = sum(w[hc + "in"][s] * streams[s] for s in range(S))
        y = fn(rms_unit(u, eps) * norm)
        new = [sum(w[hc + "mix"][s, t] * streams[s] for s in range(S)) + w[hc + "out"][t] * y for t in range(S)]
        return None, new

    for i in layer_order(config):
        layer, prefix = config["layers"][i], f"l{i}."
        kind, m = layer["type"], layer["mixer"]
        if kind == "parallel":
            mix = lambda a: parallel_mixer(a, w, prefix + "mix.", m, eps, positions)
        else:
            mix = lambda a: attention(a, w, prefix + "mix.", m, eps, positions, kind)
        x, streams = sublayer(x, streams, prefix, 1, mix)
        if layer.get("mlp") is not None:
            x, streams = sublayer(x, streams, prefix, 2, lambda a: feed_forward(a, w, prefix + "mlp."))
        if layer_outputs is not None:
            layer_outputs.append(sum(streams) if streams is not None else x)
    if streams is not None:
        x = sum(streams)
    return (rms_unit(x, eps) * w["final.norm"]) @ w["head"].T
