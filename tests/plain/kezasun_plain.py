"""Plain, slow Kezasun implementation: the oracle of the Kezasun tests.

Whole sequences, no cache, no state carried between calls, one function per
mechanism, nothing shared with the engine's code.  Everything runs on the CPU
in float64 (or the dtype of the weights handed in).  `cfg` is the dictionary of
config.json; `w` maps tensor names to tensors.

Notation: h is a layer's normed input [T, width]; W x means `x @ W.T` with W
stored [out, in]; positions count from 0.
"""
from __future__ import annotations

import json
import math
import os
from typing import Dict, List, Optional, Sequence

import torch


# --------------------------------------------------------------------------
# small pieces
# --------------------------------------------------------------------------
def rms_unit(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last axis (eps inside the root)."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def one_plus_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """RMS norm whose stored weight lies around zero: the gain is 1 + weight."""
    return rms_unit(x, eps) * (1.0 + weight)


def sigmoid(x: torch.Tensor) -> torch.Tensor:
    return 1.0 / (1.0 + torch.exp(-x))


def silu(x: torch.Tensor) -> torch.Tensor:
    return x * sigmoid(x)


# --------------------------------------------------------------------------
# wkv mixer: a per-head matrix state with data-dependent decay
# --------------------------------------------------------------------------
def token_shift(h: torch.Tensor, first: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Row t holds h[t - 1]; row 0 holds `first` (zeros where a sequence starts)."""
    prev = torch.zeros_like(h)
    prev[1:] = h[:-1]
    if first is not None:
        prev[0] = first
    return prev


def wkv_decay(mix_w: torch.Tensor, w: Dict[str, torch.Tensor], p: str) -> torch.Tensor:
    """exp(-exp(W_w2 tanh(W_w1 x) + w0)): one number in (0, 1) per head and key channel."""
    return torch.exp(-torch.exp(torch.tanh(mix_w @ w[p + "w1"].T) @ w[p + "w2"].T + w[p + "w0"]))


def wkv_recurrence(r, k, v, decay, u, state=None):
    """One head.  r, k, v, decay [T, d]; u [d]; state [d (key), d (value)] or None for zeros.
        o_t = (S + diag(u) k_t v_t^T)^T r_t        (the bonus u counts for the current token only)
        S  <- diag(decay_t) S + k_t v_t^T
    Returns o [T, d] and the last state."""
    T, d = r.shape
    S = torch.zeros((d, d), dtype=r.dtype) if state is None else state.clone()
    out = []
    for t in range(T):
        kv = torch.outer(k[t], v[t])
        out.append((S + u[:, None] * kv).T @ r[t])
        S = decay[t][:, None] * S + kv
    return torch.stack(out), S


def wkv_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, heads: int, dim: int, eps: float) -> torch.Tensor:
    prev = token_shift(h)
    mix = {s: h + (prev - h) * w[p + "mu." + s] for s in "rkvgw"}
    T = h.shape[0]
    r = (mix["r"] @ w[p + "r"].T).view(T, heads, dim)
    k = (mix["k"] @ w[p + "k"].T).view(T, heads, dim)
    v = (mix["v"] @ w[p + "v"].T).view(T, heads, dim)
    gate = silu(mix["g"] @ w[p + "g"].T)
    decay = wkv_decay(mix["w"], w, p).view(T, heads, dim)
    u = w[p + "u"].view(heads, dim)
    o = torch.stack([wkv_recurrence(r[:, a], k[:, a], v[:, a], decay[:, a], u[a])[0] for a in range(heads)], dim=1)
    o = rms_unit(o, eps).reshape(T, heads * dim)  # every head by its own root mean square
    return (o * w[p + "norm"] * gate) @ w[p + "o"].T


# --------------------------------------------------------------------------
# attention mixer
# --------------------------------------------------------------------------
def scaled_frequencies(base: float, dims: int, scaling: Optional[dict]) -> List[float]:
    """f_i = base^(-2i/dims), i < dims / 2; with `scaling` (factor, low, high, original) long
    wavelengths are stretched: l = 2 pi / f; l < original / high keeps f; l > original / low
    gives f / factor; between the two, s = (original / l - low) / (high - low) and the
    frequency is (1 - s) f / factor + s f."""
    out = []
    for i in range(dims // 2):
        f = float(base) ** (-2.0 * i / dims)
        if scaling:
            factor, low, high = float(scaling["factor"]), float(scaling["low"]), float(scaling["high"])
            original = float(scaling["original"])
            l = 2.0 * math.pi / f
            if l < original / high:
                pass
            elif l > original / low:
                f = f / factor
            else:
                s = (original / l - low) / (high - low)
                f = (1.0 - s) * f / factor + s * f
        out.append(f)
    return out


def rotate_half(x: torch.Tensor, positions: Sequence[int], freqs: Sequence[float]) -> torch.Tensor:
    """x [T, heads, d]: element i < len(freqs) pairs with i + len(freqs); the pair (a, b) at
    position p becomes (a cos - b sin, b cos + a sin) with the angle p * f_i; elements from
    2 len(freqs) on pass unchanged."""
    y = x.clone()
    half = len(freqs)
    pos = torch.tensor([float(p) for p in positions], dtype=torch.float64)
    for i, f in enumerate(freqs):
        ang = pos * f
        c, s = torch.cos(ang).to(x.dtype)[:, None], torch.sin(ang).to(x.dtype)[:, None]
        a, b = x[:, :, i], x[:, :, i + half]
        y[:, :, i] = a * c - b * s
        y[:, :, i + half] = b * c + a * s
    return y


def attention_keys_values(h: torch.Tensor, w, p: str, m: dict, eps: float):
    """Keys (normed over the whole projection, then rotated) [T, G, dim] and values [T, G, vdim]."""
    T = h.shape[0]
    G = int(m["kv_heads"])
    k = h @ w[p + "k"].T + w[p + "k.b"]
    k = rms_unit(k, eps) * w[p + "k.norm"]
    v = h @ w[p + "v"].T + w[p + "v.b"]
    freqs = scaled_frequencies(m["rot"]["base"], int(m["rot"]["dims"]), m["rot"].get("scaling"))
    k = rotate_half(k.view(T, G, int(m["dim"])), range(T), freqs)
    return k, v.view(T, G, int(m["vdim"]))


def sink_softmax(scores: torch.Tensor, seen: torch.Tensor) -> torch.Tensor:
    """Row by row over the places where `seen`: exp(s_j) / (1 + sum_j exp(s_j)), a softmax with one more
    place whose score is 0 and whose share is dropped."""
    scores = scores.masked_fill(~seen, -math.inf)  # (exp(-inf) = 0: what is not seen has no share)
    big = torch.clamp(scores.max(dim=-1, keepdim=True).values, min=0.0)
    e = torch.exp(scores - big)
    return e / (torch.exp(-big) + e.sum(dim=-1, keepdim=True))


def attention_mixer(h: torch.Tensor, w, p: str, m: dict, eps: float, keys=None, values=None) -> torch.Tensor:
    """`keys`, `values`: those of another layer (this one then has none of its own)."""
    T = h.shape[0]
    H, G, dim, vdim = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    if keys is None:
        keys, values = attention_keys_values(h, w, p, m, eps)
    q = h @ w[p + "q"].T + w[p + "q.b"]
    q = rms_unit(q, eps) * w[p + "q.norm"]
    freqs = scaled_frequencies(m["rot"]["base"], int(m["rot"]["dims"]), m["rot"].get("scaling"))
    q = rotate_half(q.view(T, H, dim), range(T), freqs)
    i, j = torch.arange(T)[:, None], torch.arange(T)[None, :]
    seen = j <= i  # a position sees itself and what came before ...
    if m.get("mask"):
        seen = seen & (i - j < int(m["mask"]["size"]))  # ... as far back as the window reaches
    gate = sigmoid(h @ w[p + "g"].T)  # [T, H]
    out = torch.zeros((T, H, vdim), dtype=h.dtype)
    for a in range(H):
        g = a // (H // G)
        s = (q[:, a] @ keys[:, g].T) * float(m["scale"])
        out[:, a] = (sink_softmax(s, seen) @ values[:, g]) * gate[:, a : a + 1]
    return out.reshape(T, H * vdim) @ w[p + "o"].T


# --------------------------------------------------------------------------
# routed feed-forward
# --------------------------------------------------------------------------
def router_choice(z: torch.Tensor, correction: torch.Tensor, top: int, groups: int, keep: int):
    """z: one token's logits over experts and identity experts alike.  Scores are the softmax
    over all of them; the choice is made on score + correction, among the `keep` groups (of
    `groups` equal groups of neighbours) whose best choice score is largest; the gains are
    the chosen scores (without the correction) divided by their sum.  Returns (ids, gains)."""
    s = torch.softmax(z, dim=-1)
    c = s + correction
    n = z.shape[0]
    size = n // groups
    best = torch.stack([c[g * size : (g + 1) * size].max() for g in range(groups)])
    kept = sorted(range(groups), key=lambda g: (-float(best[g]), g))[:keep]
    allowed = torch.full((n,), -math.inf, dtype=z.dtype)
    for g in kept:
        allowed[g * size : (g + 1) * size] = c[g * size : (g + 1) * size]
    ids = sorted(range(n), key=lambda e: (-float(allowed[e]), e))[:top]
    gains = s[ids] / (s[ids].sum() + 1e-20)
    return ids, gains


def routed_ff(h: torch.Tensor, w, p: str, f: dict) -> torch.Tensor:
    r = f["router"]
    E, I, top = int(r["experts"]), int(r.get("identity", 0)), int(r["top"])
    groups = r.get("groups") or {"count": 1, "keep": 1}
    z = h @ w[p + "router"].T
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        ids, gains = router_choice(z[t], w[p + "correction"], top, int(groups["count"]), int(groups["keep"]))
        for e, g in zip(ids, gains):
            if e >= E:  # an identity expert hands its input on
                out[t] += g * h[t]
            else:
                q = f"{p}e{e}."
                out[t] += g * ((silu(h[t] @ w[q + "gate"].T) * (h[t] @ w[q + "up"].T)) @ w[q + "down"].T)
    return out


# --------------------------------------------------------------------------
# layers and the model
# --------------------------------------------------------------------------
def residual_streams(ids: Sequence[int], w, cfg) -> List[torch.Tensor]:
    """The residual stream after every layer, [T, width] each.  A layer is
    x <- x + m (mixer(h) + ff(h)) with h = norm1(x): both sublayers read the same norm."""
    eps = float(cfg["norm"]["eps"])
    mult = float(cfg["residual_mult"])
    x = w["embed"][torch.tensor(list(ids), dtype=torch.long)]
    kv = {}
    out = []
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        m = layer["mixer"]
        h = one_plus_norm(x, w[p + "norm1"], eps)
        if layer["type"] == "wkv":
            y = wkv_mixer(h, w, p + "mix.", int(m["heads"]), int(m["dim"]), eps)
        elif layer["type"] == "attention":
            src = m.get("kv_from")
            if src is None:
                kv[i] = attention_keys_values(h, w, p + "mix.", m, eps)
                y = attention_mixer(h, w, p + "mix.", m, eps, *kv[i])
            else:
                y = attention_mixer(h, w, p + "mix.", m, eps, *kv[int(src)])
        else:
            raise ValueError(layer["type"])
        if layer.get("mlp") is not None:
            y = y + routed_ff(h, w, p + "mlp.", layer["mlp"])
        x = x + mult * y
        out.append(x)
    return out


def model_logits(ids: Sequence[int], w, cfg) -> torch.Tensor:
    """Logits at every position, [T, vocab]."""
    x = residual_streams(ids, w, cfg)[-1] if cfg["layers"] else w["embed"][torch.tensor(list(ids), dtype=torch.long)]
    return one_plus_norm(x, w["final.norm"], float(cfg["norm"]["eps"])) @ w["head"].T


def generate_greedy(ids: Sequence[int], w, cfg, max_new: int, eos: int = -1) -> List[int]:
    """New tokens, the first maximum of the last position's logits each time (recomputed whole)."""
    ids, new = list(ids), []
    for _ in range(max_new):
        t = int(torch.argmax(model_logits(ids, w, cfg)[-1]))
        new.append(t)
        ids.append(t)
        if t == eos:
            break
    return new


def read_model_dir(path: str, dtype=torch.float64):
    from safetensors import safe_open

    with open(os.path.join(path, "config.json")) as f:
        cfg = json.load(f)
    w = {}
    with safe_open(os.path.join(path, "model.safetensors"), framework="pt") as f:
        for name in f.keys():
            t = f.get_tensor(name)
            w[name] = t if not t.is_floating_point() else t.to(dtype)
    return cfg, w
