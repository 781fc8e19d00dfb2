"""Tiny Sipilorn configurations for the tests, and their model folders.

Sizes differ from layer to layer and between the configurations: key sizes of 4 to 192 and value
sizes of 4 to 64 that are no multiples of each other (values wider and narrower than keys), widths and
feed-forwards that are no multiples of 8, one to seven heads, grouped and ungrouped kv heads, windows of
1 to 70 and an attention without a window, rotations of a part of the head and of the whole head,
convolutions of one to five taps, one expert a token to all of them, a layer without a feed-forward, loops
over a part of the layers, over all of them, three passes, one pass, and no loop at all, with and without a cap on the logits.  The random weights
are made *sharp* after they are drawn so that a wrong window edge, a lost state or a wrong expert
moves the logits by far more than bfloat16 rounding.
"""
from __future__ import annotations

import json
import os

import torch


def delta(heads, kv_heads, dim, vdim, conv):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}


def attn(heads, kv_heads, dim, vdim, scale, window=None, rot=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if window:
        m["mask"] = {"size": window}
    if rot:
        m["rot"] = {"dims": rot[0], "base": rot[1]}
    return m


def pair(left, right, left_scale, right_scale):
    return {"left": left, "right": right, "left_scale": left_scale, "right_scale": right_scale}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def layer(kind, mixer, mlp):
    return {"type": kind, "mixer": mixer, "mlp": mlp}


def model(width, vocab, eps, layers, loop=None, softcap=None):
    d = {"architecture": "Sipilorn", "width": width, "vocab": vocab, "norm": {"eps": eps}, "layers": layers}
    if loop:
        d["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    if softcap:
        d["logit_softcap"] = softcap
    return d


# a pair first, values wider than keys, a part of the head rotated, a window that is no multiple of anything,
# a layer without a feed-forward, the last two layers three times
SP_A = model(64, 300, 1e-6, [
    layer("parallel", pair(attn(4, 2, 16, 24, 0.3, window=13, rot=(8, 10000.0)), delta(2, 1, 16, 8, 3), 0.7, 1.3), dense(72)),
    layer("delta", delta(4, 2, 24, 16, 4), moe(5, 2, 24)),
    layer("delta", delta(3, 3, 8, 40, 2), None),
], loop=(1, 3, 3), softcap=20.0)
# no loop, one head, every expert chosen, a window of one page, the whole head rotated (of a size that decoding
# steps take in one kernel), keys of 64 channels and more
SP_B = model(96, 257, 1e-5, [
    layer("delta", delta(1, 1, 64, 64, 4), moe(3, 3, 16)),
    layer("parallel", pair(attn(2, 1, 64, 64, 0.2, window=8, rot=(64, 500.0)), delta(6, 2, 32, 16, 5), 1.0, 0.5), moe(4, 1, 32)),
    layer("delta", delta(2, 2, 100, 24, 1), dense(40)),
])
# two pairs in a row with caches of their own, one attention without a window and without a rotation, values
# narrower than keys, all layers looped, no cap
SP_C = model(72, 128, 1e-4, [
    layer("parallel", pair(attn(6, 2, 32, 16, 0.25), delta(2, 2, 48, 24, 4), 1.0, 1.0), dense(40)),
    layer("parallel", pair(attn(3, 3, 24, 40, 0.3, window=70, rot=(24, 1000000.0)), delta(1, 1, 192, 8, 2), 1.5, 0.6), moe(2, 2, 16)),
], loop=(0, 2, 2))
# recurrences only, a loop over the first layer alone
SP_D = model(48, 90, 1e-6, [
    layer("delta", delta(6, 3, 8, 8, 4), dense(56)),
    layer("delta", delta(2, 1, 128, 32, 3), moe(4, 1, 8)),
], loop=(0, 1, 2), softcap=8.0)
# sizes that are no multiples of 8 (width, heads' sizes, feed-forwards), a window of one token (a token sees
# itself alone), a loop of one pass, seven heads of four channels, every expert chosen
SP_E = model(132, 500, 1e-6, [
    layer("parallel", pair(attn(2, 2, 40, 24, 0.15, window=1, rot=(4, 10000.0)), delta(1, 1, 44, 12, 4), 1.0, 1.0), moe(4, 4, 28)),
    layer("delta", delta(7, 7, 4, 4, 4), dense(52)),
    layer("delta", delta(3, 1, 20, 12, 3), moe(5, 2, 20)),
], loop=(0, 1, 1), softcap=30.0)
SIPILORN_CONFIGS = {"spA": (SP_A, 3), "spB": (SP_B, 5), "spC": (SP_C, 7), "spD": (SP_D, 9), "spE": (SP_E, 14)}
SIPILORN_PAGE = {"spA": 16, "spB": 8, "spC": 32, "spD": 16, "spE": 16}
SIPILORN_LENGTHS = {"spA": [1, 2, 12, 13, 14, 40, 61], "spB": [3, 8, 9, 17, 75, 130], "spC": [5, 69, 70, 71, 100],
                    "spD": [1, 2, 33, 80], "spE": [2, 35, 66]}

#: factors on the drawn weights by the tensor's last name (matrices only)
SHARP = {"q": 12.0, "k": 12.0, "v": 10.0, "g": 8.0, "o": 5.0, "b": 15.0, "a": 15.0, "up": 6.0, "down": 6.0,
         "gate": 10.0, "embed": 40.0, "head": 3.0}


def make_sipilorn_dir(path: str, cfg: dict, seed: int, sharp: bool = True) -> str:
    from safetensors import safe_open
    from safetensors.torch import save_file
    from tffinfer_amd.weights import write_random_model
    write_random_model(path, json.loads(json.dumps(cfg)), seed, dtype="bfloat16")
    if sharp:
        f = os.path.join(path, "model.safetensors")
        W = {}
        with safe_open(f, "pt") as fh:
            for k in fh.keys():
                W[k] = fh.get_tensor(k)
        for k in list(W):
            last = k.split(".")[-1]
            if last in SHARP and W[k].dim() == 2 and W[k].is_floating_point():
                W[k] = (W[k].float() * SHARP[last]).to(W[k].dtype)
        save_file(W, f)
    return path
