"""Tiny Tazitar configurations for tests, and helpers that make model folders from them.

P: all three mixers over three streams, layers 1..2 run twice; key and value sizes differ, rotary dims below the key size,
   three q heads a kv head in the attentions and two value heads a q/k head in the delta rule, a YaRN ramp that lies
   inside the pairs.
Q: what models often make equal differs and what is often large is 1: one plain residual (no streams), no loop, a parallel
   layer first, an attention without rotation and without a cap, a layer without feed-forward, one head, one kv head for
   five q heads, a delta rule with as many q/k heads as value heads, two taps, sizes that are no multiples of 4 or 8.
R: sizes the matrix-core attention takes (keys of 64 and 96, values of 64 and 80), pages of 16, one stream, the whole
   model inside the loop and run three times, five taps.
S: two streams, a loop that runs once and one that could be left out (times 1), a loop body of one layer, widths that
   are no multiple of 4, a key size of 40, three taps, no scaling on the interleaved rotation.
T: sizes of a small real model, on the kernels such a model runs on: heads of 64 and 128 for the matrix cores and the
   eight-entries-a-lane preparation, sixteen q heads (head groups that are a multiple of eight), a delta rule with key
   size 128, two streams, the first two layers looped twice, pages of 32.
"""
from __future__ import annotations

import os

import torch
from safetensors.torch import load_file, save_file

from arle_amd.config import TazitarConfig
from arle_amd.weights import write_random_model

ARCH = "Tazitar"


def attn(heads, kv_heads, dim, vdim, scale=0.3, softcap=None, rot=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if softcap is not None:
        m["softcap"] = softcap
    if rot is not None:
        m["rot"] = rot
    return m


def rot(base, dims, scaling=None):
    r = {"base": base, "dims": dims}
    if scaling is not None:
        r["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    return r


def delta(heads, kv_heads, dim, vdim, conv=4):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}


def layer(kind, mixer, ff):
    return {"type": kind, "mixer": mixer, "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


TINY_P = {"architecture": ARCH, "vocab": 211, "width": 72, "norm": {"eps": 2e-5}, "streams": 3,
          "loop": {"start": 1, "stop": 3, "times": 2},
          "layers": [layer("attention", attn(6, 2, 16, 24, scale=0.35, softcap=6.0, rot=rot(10000.0, 12)), 96),
                     layer("parallel", {"left": attn(4, 2, 24, 16, scale=0.5, rot=rot(500.0, 8)),
                                        "right": delta(4, 2, 16, 12)}, 80),
                     layer("attention_2", attn(6, 3, 16, 8, scale=0.4, rot=rot(3000.0, 16, (4.0, 40, 8.0, 1.0))), 96),
                     layer("attention", attn(2, 2, 32, 8, scale=0.2, softcap=15.0, rot=rot(100.0, 32)), 64)]}

TINY_Q = {"architecture": ARCH, "vocab": 97, "width": 42, "norm": {"eps": 1e-6},
          "layers": [layer("parallel", {"left": attn(1, 1, 10, 14, scale=0.6, rot=rot(50.0, 6)),
                                        "right": delta(3, 3, 10, 6, conv=2)}, 50),
                     layer("attention", attn(5, 1, 12, 6, scale=0.5), None),
                     layer("attention_2", attn(2, 2, 8, 20, scale=0.7, rot=rot(20.0, 4, (8.0, 16, 4.0, 2.0))), 30),
                     layer("parallel", {"left": attn(4, 4, 8, 8, scale=0.4, rot=rot(1000.0, 8)),
                                        "right": delta(2, 1, 24, 20, conv=4)}, None)]}

TINY_R = {"architecture": ARCH, "vocab": 300, "width": 96, "norm": {"eps": 1e-5}, "streams": 1,
          "loop": {"start": 0, "stop": 3, "times": 3},
          "layers": [layer("attention_2", attn(4, 2, 64, 64, scale=0.2, rot=rot(250000.0, 64, (2.0, 64, 16.0, 2.0))), 128),
                     layer("parallel", {"left": attn(4, 1, 96, 80, scale=0.15, rot=rot(10000.0, 48)),
                                        "right": delta(4, 2, 64, 32, conv=5)}, 112),
                     layer("attention", attn(6, 2, 64, 80, scale=0.125, softcap=20.0, rot=rot(5000.0, 32)), 128)]}

TINY_S = {"architecture": ARCH, "vocab": 150, "width": 54, "norm": {"eps": 1e-5}, "streams": 2,
          "loop": {"start": 2, "stop": 3, "times": 1},
          "layers": [layer("attention", attn(3, 1, 40, 24, scale=0.3, softcap=4.0, rot=rot(800.0, 20)), 70),
                     layer("attention_2", attn(3, 3, 24, 40, scale=0.3, rot=rot(10000.0, 24)), 46),
                     layer("parallel", {"left": attn(2, 1, 48, 16, scale=0.25, rot=rot(200.0, 48)),
                                        "right": delta(5, 1, 40, 10, conv=3)}, 70)]}

TINY_T = {"architecture": ARCH, "vocab": 500, "width": 256, "norm": {"eps": 1e-6}, "streams": 2,
          "loop": {"start": 0, "stop": 2, "times": 2},
          "layers": [layer("parallel", {"left": attn(8, 2, 128, 64, scale=0.09, rot=rot(1000000.0, 64)),
                                        "right": delta(8, 2, 128, 64, conv=4)}, 384),
                     layer("attention_2", attn(8, 8, 128, 128, scale=0.09, rot=rot(50000.0, 128, (4.0, 256, 32.0, 1.0))), 384),
                     layer("attention", attn(16, 4, 64, 64, scale=0.125, softcap=30.0, rot=rot(500000.0, 64)), 384)]}

# name -> (config, page size, weight std, norm std, seed)
TINY = {"P": (TINY_P, 4, 0.2, 0.2, 5), "Q": (TINY_Q, 8, 0.25, 0.3, 6), "R": (TINY_R, 16, 0.12, 0.2, 7),
        "S": (TINY_S, 16, 0.2, 0.2, 9), "T": (TINY_T, 32, 0.08, 0.2, 11)}


def make_model_dir(tmp_path, name: str) -> str:
    raw, _, std, norm_std, seed = TINY[name]
    d = os.path.join(str(tmp_path), f"tazitar_{name}")
    write_random_model(d, ARCH, TazitarConfig.from_dict(raw), seed=seed, std=std, norm_std=norm_std)
    # Constants as a trained model may have them, large enough that leaving one out or misplacing one shows: sinks of
    # the size of the scores, decays and step biases of several tenths, convolution taps of order one, stream
    # connections that mix every stream into every other.
    path = os.path.join(d, "model.safetensors")
    tensors = load_file(path)
    g = torch.Generator().manual_seed(seed)
    for key, t in tensors.items():
        r = lambda s=1.0: torch.randn(t.shape, generator=g) * s
        if key.endswith(".sink"):
            tensors[key] = (r() + 1.5).to(t.dtype)
        elif key.endswith(".A_log"):
            tensors[key] = (r() - 1.0).to(t.dtype)
        elif key.endswith(".dt_bias"):
            tensors[key] = (r() - 1.5).to(t.dtype)
        elif key.endswith(".conv"):
            tensors[key] = (r(0.5) + 0.2).to(t.dtype)
        elif key.endswith((".hc1.mix", ".hc2.mix")):
            tensors[key] = (torch.eye(t.shape[0]) + r(0.25)).to(t.dtype)
        elif key.endswith((".hc1.in", ".hc2.in")):
            tensors[key] = (1.0 / t.shape[0] + r(0.2)).to(t.dtype)
        elif key.endswith((".hc1.out", ".hc2.out")):
            tensors[key] = (1.0 + r(0.2)).to(t.dtype)
        elif key.endswith((".right.b", ".right.a")):
            tensors[key] = (t.float() * 3.0).to(t.dtype)
    save_file(tensors, path)
    return d
