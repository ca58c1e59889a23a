"""Plain, slow Visadra implementation: the oracle of the Visadra tests.

Whole sequences, no cache, no state carried between calls, one function per
mechanism, nothing shared with the engine's code.  Everything runs on the CPU
in float64 (or the dtype of the weights handed in).  `cfg` is the dictionary of
config.json; `w` maps tensor names to tensors.

Notation: h is a sublayer's input [T, width]; W x means `x @ W.T` with W stored
[out, in]; positions count from 0.
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


def scalar_norm(x: torch.Tensor, gain: torch.Tensor, eps: float) -> torch.Tensor:
    """RMS norm whose gain is one number for all coordinates."""
    return rms_unit(x, eps) * gain.reshape(())


def sigmoid(x: torch.Tensor) -> torch.Tensor:
    return 1.0 / (1.0 + torch.exp(-x))


def silu(x: torch.Tensor) -> torch.Tensor:
    return x * sigmoid(x)


def gated_ff(h: torch.Tensor, w_gate: torch.Tensor, w_up: torch.Tensor, w_down: torch.Tensor) -> torch.Tensor:
    """down(silu(gate h) * (up h)), no biases."""
    return (silu(h @ w_gate.T) * (h @ w_up.T)) @ w_down.T


# --------------------------------------------------------------------------
# minGRU mixer
# --------------------------------------------------------------------------
def mingru_candidate(u: torch.Tensor) -> torch.Tensor:
    """u + 1/2 where u >= 0, sigmoid(u) where u < 0 (continuous at 0, always positive)."""
    return torch.where(u >= 0, u + 0.5, sigmoid(u))


def mingru(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, state: Optional[torch.Tensor] = None) -> torch.Tensor:
    """S_t = (1 - z_t) S_(t-1) + z_t c_t, element by element, S_(-1) = 0 (or `state`);
    z = sigmoid(W_z h + b_z), c = candidate(W_x h + b_x); output W_o (S_t * silu(W_g h))."""
    z = sigmoid(h @ w[p + "z"].T + w[p + "z.b"])
    c = mingru_candidate(h @ w[p + "x"].T + w[p + "x.b"])
    gate = silu(h @ w[p + "g"].T)
    s = torch.zeros(z.shape[1], dtype=h.dtype) if state is None else state.clone()
    rows = []
    for t in range(h.shape[0]):
        s = (1.0 - z[t]) * s + z[t] * c[t]
        rows.append(s * gate[t])
    return torch.stack(rows) @ w[p + "o"].T


# --------------------------------------------------------------------------
# latent attention mixer
# --------------------------------------------------------------------------
def rotate_interleaved(x: torch.Tensor, positions: Sequence[int], base: float, dims: int) -> torch.Tensor:
    """Rotary encoding on the first `dims` elements of the last axis of x [T, ..., d]:
    element 2i pairs with 2i + 1; angle a = p * base^(-2i/dims);
    (u, v) -> (u cos a - v sin a, v cos a + u sin a).  The rest passes unchanged."""
    y = x.clone()
    for t in range(x.shape[0]):
        for i in range(dims // 2):
            a = float(positions[t]) * base ** (-2.0 * i / dims)
            c, s = math.cos(a), math.sin(a)
            u, v = x[t, ..., 2 * i], x[t, ..., 2 * i + 1]
            y[t, ..., 2 * i] = u * c - v * s
            y[t, ..., 2 * i + 1] = v * c + u * s
    return y


def sink_softmax_attention(scores: torch.Tensor, values: torch.Tensor, sink: torch.Tensor,
                           window: Optional[int] = None) -> torch.Tensor:
    """scores [T, T] (query, key; already scaled), values [T, dv], `sink` one number: causal
    softmax whose denominator also holds exp(sink), which has no value.  -> [T, dv]."""
    T = scores.shape[0]
    out = torch.zeros(T, values.shape[1], dtype=values.dtype)
    for i in range(T):
        lo = 0 if window is None else max(0, i - window + 1)
        s = scores[i, lo : i + 1]
        m = torch.maximum(s.max(), sink)
        e = torch.exp(s - m)
        out[i] = (e[:, None] * values[lo : i + 1]).sum(0) / (e.sum() + torch.exp(sink - m))
    return out


def latent_attention(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: dict, eps: float,
                     positions: Optional[Sequence[int]] = None) -> torch.Tensor:
    """Keys and values of every head are made from one small latent vector per token.
    q = W_q h, per head [dim plain | rot_dim rotated]; W_dkv h = [kv_rank latent | rot_dim shared
    rotated key]; latent c = RMS norm with weight; per head k_plain = W_uk c, v = W_uv c;
    score = (q_plain . k_plain + q_rot . k_rot) * scale; softmax with a sink per head; W_o on the heads."""
    T = h.shape[0]
    H, d, r, dv, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    base, dims = float(m["rot"]["base"]), int(m["rot"]["dims"])
    positions = list(range(T)) if positions is None else positions
    q = (h @ w[p + "q"].T).reshape(T, H, d + r)
    dkv = h @ w[p + "dkv"].T
    c = rms_unit(dkv[:, :rank], eps) * w[p + "dkv.norm"]
    k_rot = rotate_interleaved(dkv[:, rank:], positions, base, dims)  # [T, r], shared by the heads
    q_rot = rotate_interleaved(q[:, :, d:], positions, base, dims)  # [T, H, r]
    k_plain = (c @ w[p + "uk"].T).reshape(T, H, d)
    v = (c @ w[p + "uv"].T).reshape(T, H, dv)
    heads = []
    for hd in range(H):
        scores = (q[:, hd, :d] @ k_plain[:, hd].T + q_rot[:, hd] @ k_rot.T) * float(m["scale"])
        heads.append(sink_softmax_attention(scores, v[:, hd], w[p + "sink"][hd], m.get("window")))
    return torch.cat(heads, dim=1) @ w[p + "o"].T


# --------------------------------------------------------------------------
# feed-forwards
# --------------------------------------------------------------------------
def route(h: torch.Tensor, w_router: torch.Tensor, b_router: torch.Tensor, top: int):
    """(chosen experts [T, top], their weights [T, top]): the `top` largest logits of
    W_router h + b, weights = softmax over the chosen logits only."""
    logits = h @ w_router.T + b_router
    vals, idx = torch.topk(logits, top, dim=-1)
    return idx, torch.softmax(vals, dim=-1)


def moe_ff(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, mlp: dict) -> torch.Tensor:
    """Weighted sum of the chosen experts' outputs, plus the shared expert for every token."""
    E, top = mlp["router"]["experts"], mlp["router"]["top"]
    idx, wt = route(h, w[p + "router"], w[p + "router.b"], top)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for k in range(top):
            e = int(idx[t, k])
            q = f"{p}e{e}."
            out[t] += wt[t, k] * gated_ff(h[t : t + 1], w[q + "gate"], w[q + "up"], w[q + "down"])[0]
    if mlp.get("shared"):
        q = p + "shared."
        out = out + gated_ff(h, w[q + "gate"], w[q + "up"], w[q + "down"])
    return out


def feed_forward(h, w, p, mlp):
    if mlp["kind"] == "dense":
        return gated_ff(h, w[p + "gate"], w[p + "up"], w[p + "down"])
    if mlp["kind"] == "moe":
        return moe_ff(h, w, p, mlp)
    raise ValueError(mlp["kind"])


# --------------------------------------------------------------------------
# the model
# --------------------------------------------------------------------------
def mixer(h, w, i, layer, eps, positions=None):
    p = f"l{i}.mix."
    if layer["type"] in ("mingru", "mingru_2"):
        return mingru(h, w, p)
    if layer["type"] == "latent_attention":
        return latent_attention(h, w, p, layer["mixer"], eps, positions)
    raise ValueError(layer["type"])


def layer_forward(x, w, i, layer, eps, positions=None):
    """x <- x + norm1(mixer(x)); x <- x + norm2(ff(x)): the norm sits on the sublayer's output."""
    x = x + scalar_norm(mixer(x, w, i, layer, eps, positions), w[f"l{i}.norm1"], eps)
    if layer.get("mlp"):
        x = x + scalar_norm(feed_forward(x, w, f"l{i}.mlp.", layer["mlp"]), w[f"l{i}.norm2"], eps)
    return x


def residual_streams(ids: Sequence[int], w, cfg) -> List[torch.Tensor]:
    """The residual stream after every layer, [T, width] each."""
    eps = float(cfg["norm"]["eps"])
    x = w["embed"][torch.tensor(list(ids), dtype=torch.long)] * float(cfg["embedding"]["scale"])
    out = []
    for i, layer in enumerate(cfg["layers"]):
        x = layer_forward(x, w, i, layer, eps)
        out.append(x)
    return out


def model_logits(ids: Sequence[int], w, cfg) -> torch.Tensor:
    """Logits at every position, [T, vocab]."""
    eps = float(cfg["norm"]["eps"])
    x = residual_streams(ids, w, cfg)[-1] if cfg["layers"] else (
        w["embed"][torch.tensor(list(ids), dtype=torch.long)] * float(cfg["embedding"]["scale"]))
    return (scalar_norm(x, w["final.norm"], eps) @ w["head"].T) * float(cfg["logit_scale"])


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
