"""Tiny Retudra configurations for tests, and helpers that make model folders from them.

P: all three mixers and both feed-forwards: a window of 24 that keeps 5 first keys, rotary dims below the key size,
   three q heads a kv head, key and value sizes that differ everywhere, a delta rule with two value heads a q/k head and
   four taps, experts in four groups of which two are kept with two identity experts, a layer without feed-forward, a
   token-side input of 12 columns, a factor of 0.5 on what is added, capped logits.
Q: what models often make equal differs and what is often large is 1: no token side, no cap, no factor (1), one head,
   one kv head for five q heads, an attention without window and one without rotation, a window that keeps nothing, a
   delta rule with as many q/k heads as heads and two taps, an expert choice of one among all (no groups, no identity
   experts), sizes that are no multiples of 4 or 8, a latent whose rotated part turns only in its first entries.
R: sizes the matrix cores take (keys and values of 64, three q heads a kv head, a latent of 64 + 32), pages of 16, a
   window of 40 that keeps 18 (neither a multiple of a tile), seven experts and one identity expert in two groups of which one is kept, three
   choices, a factor of 0.25.
S: heads of 128 over values of 64, a window of 33 that keeps a whole page of 32, a delta rule with key size 128 and one
   q/k head for four heads, nine router outputs in three groups of which two are kept, five taps.
"""
from __future__ import annotations

import os

import torch
from safetensors.torch import load_file, save_file

from arle_amd.config import RetudraConfig
from arle_amd.weights import write_random_model

ARCH = "Retudra"


def rot(base, dims):
    return {"base": base, "dims": dims}


def attn(heads, kv_heads, dim, vdim, scale=0.3, rot=None, mask=None):
    m = {"heads": heads, "dim": dim, "vdim": vdim, "scale": scale}
    if kv_heads is not None:
        m["kv_heads"] = kv_heads
    if rot is not None:
        m["rot"] = rot
    if mask is not None:
        m["mask"] = {"size": mask[0], "keep_first": mask[1]}
    return m


def latent(heads, dim, rot_dim, vdim, rank, scale=0.3, rot=None):
    return {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": rank, "scale": scale, "rot": rot}


def delta(heads, kv_heads, dim, vdim, conv=4, decay_rank=8, gate_rank=6):
    m = {"heads": heads, "dim": dim, "vdim": vdim, "conv": conv, "decay_rank": decay_rank, "gate_rank": gate_rank}
    if kv_heads is not None:
        m["kv_heads"] = kv_heads
    return m


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, identity=0, groups=None):
    router = {"experts": experts, "top": top, "identity": identity}
    if groups is not None:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    return {"kind": "moe", "expert": {"ff": ff}, "router": router}


def layer(kind, mixer, mlp):
    return {"type": kind, "mixer": mixer, "mlp": mlp}


TINY_P = {"architecture": ARCH, "vocab": 211, "width": 72, "norm": {"eps": 2e-5}, "residual_mult": 0.5,
          "token_side": {"dim": 12}, "logit_softcap": 25.0,
          "layers": [layer("attention", attn(6, 2, 16, 24, scale=0.35, rot=rot(10000.0, 12), mask=(24, 5)), dense(96)),
                     layer("channel_delta", delta(4, 2, 16, 12), moe(6, 2, 40, identity=2, groups=(4, 2))),
                     layer("latent_attention", latent(4, 16, 8, 12, 24, scale=0.3, rot=rot(500.0, 8)), None),
                     layer("attention", attn(2, 2, 32, 8, scale=0.2, rot=rot(100.0, 32), mask=(9, 3)), moe(5, 3, 24))]}

TINY_Q = {"architecture": ARCH, "vocab": 97, "width": 42, "norm": {"eps": 1e-6},
          "layers": [layer("channel_delta", delta(3, None, 10, 6, conv=2, decay_rank=3, gate_rank=5), moe(4, 1, 30)),
                     layer("attention", attn(5, 1, 12, 6, scale=0.5), None),
                     layer("latent_attention", latent(1, 10, 6, 14, 18, scale=0.4, rot=rot(50.0, 4)), dense(50)),
                     layer("attention", attn(1, None, 10, 14, scale=0.6, rot=rot(20.0, 6), mask=(7, 0)), dense(30))]}

TINY_R = {"architecture": ARCH, "vocab": 300, "width": 96, "norm": {"eps": 1e-5}, "residual_mult": 0.25,
          "token_side": {"dim": 16}, "logit_softcap": 40.0,
          "layers": [layer("latent_attention", latent(4, 32, 32, 48, 64, scale=0.12, rot=rot(250000.0, 32)), dense(128)),
                     layer("attention", attn(6, 2, 64, 64, scale=0.125, rot=rot(250000.0, 16), mask=(40, 18)),
                           moe(7, 3, 48, identity=1, groups=(2, 1))),
                     layer("channel_delta", delta(4, 2, 64, 48, conv=4, decay_rank=16, gate_rank=8),
                           moe(7, 3, 48, identity=1, groups=(2, 1)))]}

TINY_S = {"architecture": ARCH, "vocab": 150, "width": 80, "norm": {"eps": 1e-5}, "residual_mult": 0.7,
          "token_side": {"dim": 5},
          "layers": [layer("attention", attn(2, 1, 128, 64, scale=0.09, rot=rot(800.0, 64), mask=(33, 32)),
                           moe(7, 2, 40, identity=2, groups=(3, 2))),
                     layer("channel_delta", delta(4, 1, 128, 16, conv=5, decay_rank=12, gate_rank=4), dense(70)),
                     layer("latent_attention", latent(2, 24, 16, 40, 40, scale=0.2, rot=rot(10000.0, 16)),
                           moe(2, 2, 40, identity=1))]}

# name -> (config, page size, weight std, norm std, seed)
TINY = {"P": (TINY_P, 4, 0.2, 0.2, 5), "Q": (TINY_Q, 8, 0.25, 0.3, 6), "R": (TINY_R, 16, 0.12, 0.2, 7),
        "S": (TINY_S, 16, 0.12, 0.2, 9)}


def make_model_dir(tmp_path, name: str) -> str:
    raw, _, std, norm_std, seed = TINY[name]
    d = os.path.join(str(tmp_path), f"retudra_{name}")
    write_random_model(d, ARCH, RetudraConfig.from_dict(raw), seed=seed, std=std, norm_std=norm_std)
    # Constants as a trained model may have them, large enough that leaving one out or misplacing one shows: decays
    # and step biases of several tenths, convolution taps of order one, corrections of the router that change who is
    # chosen, norm biases, a second embedding of order one.
    path = os.path.join(d, "model.safetensors")
    tensors = load_file(path)
    g = torch.Generator().manual_seed(seed)
    for key, t in tensors.items():
        r = lambda s=1.0: torch.randn(t.shape, generator=g) * s
        if key.endswith(".A_log"):
            tensors[key] = (r() - 1.0).to(t.dtype)
        elif key.endswith(".dt_bias"):
            tensors[key] = (r() - 1.5).to(t.dtype)
        elif key.endswith(".conv"):
            tensors[key] = (r(0.5) + 0.2).to(t.dtype)
        elif key.endswith(".correction"):
            tensors[key] = r(0.15).to(t.dtype)
        elif key.endswith((".norm1.b", ".norm2.b", "final.norm.b")):
            tensors[key] = r(0.3).to(t.dtype)
        elif key == "side.embed":
            tensors[key] = r(1.0).to(t.dtype)
        elif key.endswith(".mlp.router"):
            tensors[key] = (t.float() * 8.0).to(t.dtype)      # decisive routers: fewer choices that rounding can turn
        elif key.endswith((".mix.b", ".mix.a2", ".mix.g2")):
            tensors[key] = (t.float() * 3.0).to(t.dtype)
    save_file(tensors, path)
    return d
