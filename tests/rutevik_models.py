"""Tiny Rutevik configurations for the tests, and their model folders.

Sizes differ from layer to layer and between the configurations: one to eight heads, grouped and ungrouped kv
heads, maps of 8 to 64 channels with values wider and narrower than two maps, ranks and widths that are no
multiples of 8, a rotation of a part of a map and of all of it, with and without slowed-down long waves, with
and without a cap on the scores, one expert a token to all of them, a layer without a feed-forward, layers
that read the cache of an earlier layer (one reader, two readers of one cache, none), a scale on the logits
of 1 and of other values.  The random weights are made *sharp* after they are drawn so that a wrong key, a
lost page, a wrong map or a wrong expert moves the logits by far more than bfloat16 rounding.
"""
from __future__ import annotations

import functools
import json
import os

import torch


def latent(heads, dim, rot_dim, vdim, kv_rank, q_rank, scale, base, kv_from=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank,
         "scale": scale, "rot": {"dims": rot_dim, "base": base}}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def attn(heads, kv_heads, dim, vdim, scale, diff, rot, softcap=None, scaling=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "diff": diff,
         "rot": {"dims": rot[0], "base": rot[1]}}
    if softcap:
        m["softcap"] = softcap
    if scaling:
        m["rot"]["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    return m


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def layer(kind, mixer, mlp):
    return {"type": kind, "mixer": mixer, "mlp": mlp}


def model(width, vocab, eps, logit_scale, layers):
    return {"architecture": "Rutevik", "width": width, "vocab": vocab, "norm": {"eps": eps}, "logit_scale": logit_scale,
            "layers": layers}


# two readers of the first layer's cache, a part of every map rotated with slowed-down long waves, a cap, two
# experts a token, a layer without a feed-forward
RV_A = model(64, 300, 1e-6, 0.5, [
    layer("latent_attention", latent(3, 16, 8, 24, 40, 24, 0.2, 10000.0), dense(72)),
    layer("attention", attn(4, 2, 16, 24, 0.3, 0.2, (8, 500.0), softcap=5.0, scaling=(4.0, 1.0, 2.0, 32)), moe(5, 2, 24)),
    layer("latent_attention", latent(2, 24, 8, 16, 40, 32, 0.25, 10000.0, kv_from=0), moe(4, 1, 16)),
    layer("latent_attention", latent(3, 8, 8, 32, 40, 16, 0.3, 10000.0, kv_from=0), None),
])
# attention first, one kv head, values narrower than two maps, no cap and no scaling; one latent head whose
# rotated part is half the key; every expert chosen; heads that are not grouped; a scale of 1 on the logits
RV_B = model(96, 257, 1e-5, 1.0, [
    layer("attention", attn(2, 1, 32, 48, 0.2, 0.5, (32, 1000000.0)), dense(40)),
    layer("latent_attention", latent(1, 64, 32, 64, 64, 16, 0.1, 300.0), moe(3, 3, 16)),
    layer("attention", attn(6, 6, 8, 8, 0.4, 0.1, (8, 50.0), softcap=2.0), None),
])
# sizes that are no multiples of 8 (width, ranks, heads' sizes, feed-forwards), two caches of different ranks,
# each with a reader, five heads and three on one kv head
RV_C = model(132, 500, 1e-4, 3.0, [
    layer("latent_attention", latent(5, 12, 6, 20, 30, 18, 0.3, 777.0), moe(4, 4, 28)),
    layer("attention", attn(3, 1, 12, 20, 0.35, 0.3, (4, 10000.0), softcap=12.0, scaling=(2.0, 1.0, 3.0, 16)), dense(52)),
    layer("latent_attention", latent(2, 20, 10, 12, 22, 26, 0.2, 50000.0), moe(6, 2, 20)),
    layer("latent_attention", latent(4, 12, 10, 20, 22, 10, 0.2, 50000.0, kv_from=2), dense(36)),
    layer("latent_attention", latent(1, 28, 6, 44, 30, 30, 0.15, 777.0, kv_from=0), moe(2, 1, 12)),
])
# head sizes of real models: prompts run on the blocks of the matrix-core attention, eight heads on two kv heads
# (eight query heads of 128 on each), a latent key of 192
RV_D = model(256, 400, 1e-5, 1.5, [
    layer("attention", attn(8, 2, 64, 128, 0.125, 0.4, (64, 10000.0), softcap=20.0, scaling=(8.0, 1.0, 4.0, 64)), moe(8, 3, 32)),
    layer("latent_attention", latent(8, 64, 32, 64, 160, 96, 0.1, 10000.0), dense(128)),
    layer("latent_attention", latent(4, 32, 32, 128, 160, 64, 0.12, 10000.0, kv_from=1), moe(4, 2, 64)),
])
RUTEVIK_CONFIGS = {"rvA": (RV_A, 3), "rvB": (RV_B, 5), "rvC": (RV_C, 7), "rvD": (RV_D, 9)}
RUTEVIK_PAGE = {"rvA": 16, "rvB": 8, "rvC": 32, "rvD": 16}
RUTEVIK_LENGTHS = {"rvA": [1, 2, 15, 16, 17, 40, 61], "rvB": [3, 8, 9, 17, 75, 130], "rvC": [5, 31, 33, 64, 100],
                   "rvD": [1, 2, 33, 150]}

#: factors on the drawn weights by the tensor's last name (matrices only)
SHARP = {"q": 12.0, "k": 12.0, "v": 10.0, "g": 8.0, "o": 5.0, "dq": 12.0, "uq": 10.0, "dkv": 12.0, "uk": 10.0, "uv": 10.0,
         "up": 6.0, "down": 6.0, "gate": 10.0, "router": 8.0, "embed": 40.0, "head": 3.0}
#: factors on vectors: the biases of q, k and v (tensors '...q.b'), and the four vectors of lambda
SHARP_VECTORS = {"q.b": 5.0, "k.b": 5.0, "v.b": 5.0, "lq1": 6.0, "lk1": 6.0, "lq2": 6.0, "lk2": 6.0}
#: the smallest gap between a token's last chosen expert score and its first rejected one in the test sequences
MIN_MARGIN = 0.004


def make_rutevik_dir(path: str, cfg: dict, seed: int, sharp: bool = True) -> str:
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
            for tail, f_ in SHARP_VECTORS.items():
                if k.endswith(".mix." + tail):
                    W[k] = (W[k].float() * f_).to(W[k].dtype)
        save_file(W, f)
    return path


@functools.lru_cache(maxsize=None)
def clear_tokens(model_dir: str, n: int, vocab: int, seed: int) -> tuple:
    """``n`` random tokens whose sequence makes no close call in any mixture of experts.  A token's routers see
    the tokens up to it and no later one, so the first token with a close call is drawn again until none is left."""
    import plain_rutevik as plain
    from helpers import random_tokens
    cfg, W = plain.load(model_dir)
    toks = random_tokens(n, vocab, seed)
    g = torch.Generator().manual_seed(seed + 1)
    for _ in range(60 + 4 * n):
        margins = []
        plain.forward(cfg, W, toks, margins=margins)
        if not margins:
            return tuple(toks)
        close = (torch.stack(margins, 0).min(0).values < MIN_MARGIN).nonzero()
        if close.numel() == 0:
            return tuple(toks)
        toks[int(close[0])] = int(torch.randint(0, vocab, (1,), generator=g))
    raise AssertionError(f"no sequence of {n} tokens without a close call")
