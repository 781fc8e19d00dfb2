"""Plain, slow implementation of the Rutevik decoder, used only by tests.

Whole sequences, no cache, no batching, one function per mechanism, float64.  It shares no code
with the package: config.json is read with ``json``, the weights with the ``safetensors`` library,
every head's keys and values are expanded from the latent vectors (the long way round), and the
two maps of a differential attention are two attentions computed one after the other.
"""
from __future__ import annotations

import json
import math
import os

import torch


# ---------------------------------------------------------------- small pieces ---
def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last dimension."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def sigmoid(z):
    return 1.0 / (1.0 + torch.exp(-z))


def silu(z):
    return z * sigmoid(z)


def dyt(x: torch.Tensor, alpha, w: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """The norm without statistics: tanh(alpha x) w + b, element by element."""
    return torch.tanh(alpha * x) * w + b


def frequencies(dims: int, base: float, scaling: dict | None = None) -> torch.Tensor:
    """f_i = base^(-2i/dims) for i < dims/2; with ``scaling`` long waves are slowed down: a wave
    longer than original/low turns ``factor`` times slower, one shorter than original/high as it
    is, and between the two the frequency goes over smoothly."""
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = base ** (-2.0 * i / dims)
    if not scaling:
        return f
    factor, low, high, orig = scaling["factor"], scaling["low"], scaling["high"], scaling["original"]
    out = f.clone()
    for n in range(f.numel()):
        wave = 2.0 * math.pi / f[n].item()
        if wave < orig / high:
            continue
        if wave > orig / low:
            out[n] = f[n] / factor
        else:
            s = (orig / wave - low) / (high - low)
            out[n] = (1.0 - s) * f[n] / factor + s * f[n]
    return out


def rotate(x: torch.Tensor, freq: torch.Tensor, first_pos: int = 0) -> torch.Tensor:
    """x [T, ..., D]: of the last dimension's first 2 len(freq) elements, element i and element
    i + len(freq) turn by the angle pos * freq[i]; the other elements stay."""
    half = freq.numel()
    if not half:
        return x
    T = x.shape[0]
    ang = torch.arange(first_pos, first_pos + T, dtype=torch.float64)[:, None] * freq[None, :]
    shape = [T] + [1] * (x.dim() - 2) + [half]
    c, s = torch.cos(ang).reshape(shape), torch.sin(ang).reshape(shape)
    u, v = x[..., :half], x[..., half:2 * half]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., 2 * half:]], -1)


def causal_softmax(s: torch.Tensor) -> torch.Tensor:
    """s [T, T] scores; row i over the columns j <= i."""
    T = s.shape[0]
    vis = torch.arange(T)[None, :] <= torch.arange(T)[:, None]
    return torch.softmax(s.masked_fill(~vis, -math.inf), -1)


# ---------------------------------------------------------------- mixers ---
def latent_cache(m: dict, P: dict, h: torch.Tensor, eps: float):
    """What a latent attention keeps of its tokens: the normed latent vectors [T, kv_rank] and the
    rotated key part [T, rot_dim] that all heads share."""
    rank = m["kv_rank"]
    a = h @ P["dkv"].T
    c = unit_rms(a[:, :rank], eps) * P["dkv.norm"]
    kr = rotate(a[:, rank:], frequencies(m["rot"]["dims"], m["rot"]["base"]))
    return c, kr


def latent_attention(m: dict, P: dict, h: torch.Tensor, eps: float, cache) -> torch.Tensor:
    """``cache`` = (c, kr) of this layer or of the layer it borrows from."""
    T = h.shape[0]
    H, D, R, E = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
    c, kr = cache
    cq = unit_rms(h @ P["dq"].T, eps) * P["dq.norm"]
    q = (cq @ P["uq"].T).reshape(T, H, D + R)
    qn = q[..., :D]
    qr = rotate(q[..., D:], frequencies(m["rot"]["dims"], m["rot"]["base"]))
    kn = (c @ P["uk"].T).reshape(T, H, D)
    v = (c @ P["uv"].T).reshape(T, H, E)
    out = torch.zeros(T, H, E, dtype=h.dtype)
    for a in range(H):
        s = (qn[:, a] @ kn[:, a].T + qr[:, a] @ kr.T) * m["scale"]
        out[:, a] = causal_softmax(s) @ v[:, a]
    return out.reshape(T, H * E) @ P["o"].T


def differential_attention(m: dict, P: dict, h: torch.Tensor, eps: float) -> torch.Tensor:
    T = h.shape[0]
    H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    freq = frequencies(m["rot"]["dims"], m["rot"]["base"], m["rot"].get("scaling"))
    q = rotate((h @ P["q"].T + P["q.b"]).reshape(T, H, 2, D), freq)
    k = rotate((h @ P["k"].T + P["k.b"]).reshape(T, G, 2, D), freq)
    v = (h @ P["v"].T + P["v.b"]).reshape(T, G, E)
    cap, diff = m.get("softcap"), m["diff"]
    lam = math.exp((P["lq1"] * P["lk1"]).sum().item()) - math.exp((P["lq2"] * P["lk2"]).sum().item()) + diff
    out = torch.zeros(T, H, E, dtype=h.dtype)
    for a in range(H):
        g = a // (H // G)
        maps = []
        for n in range(2):
            s = (q[:, a, n] @ k[:, g, n].T) * m["scale"]
            if cap:
                s = cap * torch.tanh(s / cap)
            maps.append(causal_softmax(s) @ v[:, g])
        o = maps[0] - lam * maps[1]
        out[:, a] = unit_rms(o, eps) * (1.0 - diff)
    out = out.reshape(T, H * E) * sigmoid(h @ P["g"].T)
    return out @ P["o"].T


# ---------------------------------------------------------------- feed-forwards ---
def dense_ff(P: dict, h: torch.Tensor) -> torch.Tensor:
    return (torch.relu(h @ P["up"].T) ** 2) @ P["down"].T


def routed_experts(m: dict, P: dict, h: torch.Tensor) -> torch.Tensor:
    """Each token's ``top`` experts by the largest sigmoid of the router's logits; the score is the
    expert's weight as it is, and it multiplies what goes *into* the expert."""
    top = m["router"]["top"]
    s = sigmoid(h @ P["router"].T)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e in torch.topk(s[t], top).indices.tolist():
            z = s[t, e] * h[t]
            out[t] += P[f"e{e}.down"] @ (silu(P[f"e{e}.gate"] @ z) * (P[f"e{e}.up"] @ z))
    return out


def router_margins(m: dict, P: dict, h: torch.Tensor) -> torch.Tensor:
    """Per token, the gap between its last chosen score and its first rejected one."""
    top, E = m["router"]["top"], m["router"]["experts"]
    if top >= E:
        return torch.full((h.shape[0],), math.inf, dtype=h.dtype)
    s = torch.sort(sigmoid(h @ P["router"].T), -1, descending=True).values
    return s[:, top - 1] - s[:, top]


def feed_forward(m, P: dict, h: torch.Tensor):
    if m["kind"] == "dense":
        return dense_ff(P, h)
    if m["kind"] == "moe":
        return routed_experts(m, P, h)
    raise ValueError(m["kind"])


# ---------------------------------------------------------------- the model ---
def load(model_dir: str):
    from safetensors import safe_open
    with open(os.path.join(model_dir, "config.json")) as f:
        cfg = json.load(f)
    P = {}
    with safe_open(os.path.join(model_dir, "model.safetensors"), "pt") as f:
        for name in f.keys():
            t = f.get_tensor(name)
            P[name] = t.to(torch.float64) if t.is_floating_point() else t.to(torch.int64)
    return cfg, P


def sub(P: dict, prefix: str) -> dict:
    return {k[len(prefix):]: v for k, v in P.items() if k.startswith(prefix)}


def norm(P: dict, name: str, x: torch.Tensor) -> torch.Tensor:
    return dyt(x, P[name + ".alpha"], P[name], P[name + ".b"])


def forward(cfg: dict, P: dict, tokens: list, streams: list | None = None, margins: list | None = None) -> torch.Tensor:
    """float64 logits [T, vocab] of a whole sequence; ``streams`` collects the stream after every
    layer, ``margins`` every router's gaps, a tensor [T] per mixture of experts."""
    eps = cfg["norm"]["eps"]
    x = P["embed"][torch.tensor(tokens)]
    caches = {}
    for i, L in enumerate(cfg["layers"]):
        W = sub(P, f"l{i}.")
        M, m = sub(W, "mix."), L["mixer"]
        h = norm(W, "norm1", x)
        if L["type"] == "latent_attention":
            src = m.get("kv_from")
            if src is None:
                caches[i] = latent_cache(m, M, h, eps)
                src = i
            a = latent_attention(m, M, h, eps, caches[src])
        elif L["type"] == "attention":
            a = differential_attention(m, M, h, eps)
        else:
            raise ValueError(L["type"])
        x = x + a
        if L.get("mlp") is not None:
            z = norm(W, "norm2", x)
            if margins is not None and L["mlp"]["kind"] == "moe":
                margins.append(router_margins(L["mlp"], sub(W, "mlp."), z))
            x = x + feed_forward(L["mlp"], sub(W, "mlp."), z)
        if streams is not None:
            streams.append(x.clone())
    return (norm(P, "final.norm", x) @ P["head"].T) * cfg.get("logit_scale", 1.0)
