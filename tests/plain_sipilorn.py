"""Plain, slow implementation of the Sipilorn decoder, used only by tests.

Whole sequences, no cache, no state slots, no batching, one function per mechanism, float64.
It shares no code with the package: config.json is read with ``json``, the weights with the
``safetensors`` library, and every recurrence is the loop over tokens that its definition is.
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


def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    return unit_rms(x, eps) * w


def silu(z):
    return z / (1.0 + torch.exp(-z))


def sigmoid(z):
    return 1.0 / (1.0 + torch.exp(-z))


def softplus(z):
    return torch.logaddexp(z, torch.zeros_like(z))


def rotate_half_layout(x: torch.Tensor, dims: int, base: float, first_pos: int = 0) -> torch.Tensor:
    """x [T, heads, D]: of each head's first ``dims`` elements, element i and element i + dims/2 turn
    by the angle pos * base^(-2i/dims); the other elements stay."""
    if not dims:
        return x
    T = x.shape[0]
    half = dims // 2
    i = torch.arange(half, dtype=torch.float64)
    ang = torch.arange(first_pos, first_pos + T, dtype=torch.float64)[:, None] * base ** (-2.0 * i / dims)[None, :]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    a, b = x[..., :half], x[..., half:dims]
    return torch.cat([a * c - b * s, b * c + a * s, x[..., dims:]], -1)


def window_visible(T: int, size: int | None) -> torch.Tensor:
    """[T, T] bool: query i sees key j when j <= i and, with a window, i - j < size."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    vis = j <= i
    if size:
        vis &= (i - j) < size
    return vis


def causal_conv_silu(x: torch.Tensor, taps: torch.Tensor) -> torch.Tensor:
    """x [T, C], taps [C, K]: y[t, c] = silu(sum_k taps[c, k] x[t - (K - 1) + k, c]), rows before the
    first being zero."""
    T, C = x.shape
    K = taps.shape[1]
    padded = torch.cat([torch.zeros(K - 1, C, dtype=x.dtype), x], 0)
    y = torch.zeros_like(x)
    for k in range(K):
        y = y + padded[k:k + T] * taps[:, k]
    return silu(y)


def unit_vectors(x: torch.Tensor) -> torch.Tensor:
    return x / torch.sqrt((x * x).sum(-1, keepdim=True) + 1e-6)


def delta_rule(q, k, v, beta, decay):
    """q, k [T, H, D], v [T, H, E], beta, decay [T, H].  Per head, with S [D, E] starting at zero:
    S <- decay S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q.  Returns o [T, H, E]."""
    T, H, D = q.shape
    E = v.shape[2]
    S = torch.zeros(H, D, E, dtype=q.dtype)
    o = torch.zeros(T, H, E, dtype=q.dtype)
    for t in range(T):
        for h in range(H):
            S[h] = decay[t, h] * S[h]
            u = beta[t, h] * (v[t, h] - S[h].T @ k[t, h])
            S[h] = S[h] + torch.outer(k[t, h], u)
            o[t, h] = S[h].T @ q[t, h]
    return o


# ---------------------------------------------------------------- mixers ---
def delta_mixer(m: dict, P: dict, h: torch.Tensor, eps: float) -> torch.Tensor:
    T = h.shape[0]
    H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = causal_conv_silu(h @ P["q"].T, P["q.conv"]).reshape(T, G, D)
    k = causal_conv_silu(h @ P["k"].T, P["k.conv"]).reshape(T, G, D)
    v = causal_conv_silu(h @ P["v"].T, P["v.conv"]).reshape(T, H, E)
    q = unit_vectors(q) * D ** -0.5
    k = unit_vectors(k)
    rep = H // G
    q = q.repeat_interleave(rep, 1)
    k = k.repeat_interleave(rep, 1)
    beta = sigmoid(h @ P["b"].T)
    decay = torch.exp(-torch.exp(P["A_log"]) * softplus(h @ P["a"].T + P["dt_bias"]))
    o = delta_rule(q, k, v, beta, decay)
    o = unit_rms(o, eps) * P["norm"] * silu(h @ P["g"].T).reshape(T, H, E)
    return o.reshape(T, H * E) @ P["o"].T


def window_attention(m: dict, P: dict, h: torch.Tensor, eps: float) -> torch.Tensor:
    T = h.shape[0]
    H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rms_norm((h @ P["q"].T).reshape(T, H, D), P["q.norm"], eps)
    k = rms_norm((h @ P["k"].T).reshape(T, G, D), P["k.norm"], eps)
    v = (h @ P["v"].T).reshape(T, G, E)
    rot = m.get("rot")
    if rot:
        q = rotate_half_layout(q, rot["dims"], rot["base"])
        k = rotate_half_layout(k, rot["dims"], rot["base"])
    vis = window_visible(T, (m.get("mask") or {}).get("size"))
    out = torch.zeros(T, H, E, dtype=h.dtype)
    for a in range(H):
        g = a // (H // G)
        s = (q[:, a] @ k[:, g].T) * m["scale"]
        s = s.masked_fill(~vis, -math.inf)
        out[:, a] = torch.softmax(s, -1) @ v[:, g]
    out = out.reshape(T, H * E) * sigmoid(h @ P["g"].T)
    return out @ P["o"].T


def sub(P: dict, prefix: str) -> dict:
    return {k[len(prefix):]: v for k, v in P.items() if k.startswith(prefix)}


def mixer(kind: str, m: dict, P: dict, h: torch.Tensor, eps: float) -> torch.Tensor:
    if kind == "delta":
        return delta_mixer(m, P, h, eps)
    if kind == "parallel":
        left = window_attention(m["left"], sub(P, "left."), h, eps)
        right = delta_mixer(m["right"], sub(P, "right."), h, eps)
        return m["left_scale"] * left + m["right_scale"] * right
    raise ValueError(kind)


# ---------------------------------------------------------------- feed-forwards ---
def dense_ff(P: dict, h: torch.Tensor) -> torch.Tensor:
    return (silu(h @ P["gate"].T) * (h @ P["up"].T)) @ P["down"].T


def table_experts(m: dict, P: dict, h: torch.Tensor, tokens: list) -> torch.Tensor:
    """Every token id has its experts in a table; each counts 1/top.  An expert is down(relu(up h)^2)."""
    top = m["router"]["top"]
    out = torch.zeros_like(h)
    for t, tok in enumerate(tokens):
        for e in P["table"][tok].tolist():
            a = torch.relu(P[f"e{e}.up"] @ h[t]) ** 2
            out[t] += (P[f"e{e}.down"] @ a) / top
    return out


def feed_forward(m, P: dict, h: torch.Tensor, tokens: list):
    if m["kind"] == "dense":
        return dense_ff(P, h)
    if m["kind"] == "moe":
        return table_experts(m, P, h, tokens)
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


def run_order(cfg: dict):
    """(layer, pass or None) in the order the layers run: the looped span ``times`` times in a row."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, None) for i in range(n)]
    order = [(i, None) for i in range(loop["start"])]
    for t in range(loop["times"]):
        order += [(i, t) for i in range(loop["start"], loop["stop"])]
    return order + [(i, None) for i in range(loop["stop"], n)]


def forward(cfg: dict, P: dict, tokens: list, streams: list | None = None) -> torch.Tensor:
    """float64 logits [T, vocab] of a whole sequence; ``streams`` collects the stream after every layer run."""
    eps = cfg["norm"]["eps"]
    x = rms_norm(P["embed"][torch.tensor(tokens)], P["embed.norm"], eps)
    loop = cfg.get("loop")
    for i, t in run_order(cfg):
        L = cfg["layers"][i]
        if t is not None and i == loop["start"]:
            x = x + P["loop.step"][t]
        W = sub(P, f"l{i}.")
        a = mixer(L["type"], L["mixer"], sub(W, "mix."), rms_norm(x, W["norm1"], eps), eps)
        if L.get("mlp") is not None:
            a = a + feed_forward(L["mlp"], sub(W, "mlp."), rms_norm(x, W["norm2"], eps), tokens)
        x = x + a
        if streams is not None:
            streams.append(x.clone())
    z = rms_norm(x, P["final.norm"], eps) @ P["head"].T
    cap = cfg.get("logit_softcap")
    return cap * torch.tanh(z / cap) if cap else z
