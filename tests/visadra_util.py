"""Tiny Visadra configurations and helpers for the tests.  Between them every size and option
differs: rotated elements fewer than the rotated part or all of it, heads whose widths do or do
not add up to the model's, one or several chosen experts, a shared expert or none, layers without
a feed-forward, a window on some attention layers, scales equal to 1 or not."""
from __future__ import annotations

import io
import os
import subprocess
import sys
from typing import Dict, List

import torch

from litellmengine_amd.config import VisadraConfig
from litellmengine_amd.weights import write_model_dir
from tests.plain import visadra_plain as plain
from tests.trace_util import ROOT, TraceBuilder


def _latent(heads, dim, rot_dim, dims, vdim, rank, scale, base, window=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": rank, "scale": scale,
         "rot": {"base": base, "dims": dims}}
    if window:
        m["window"] = window
    return m


def _moe(experts, top, ff, shared):
    m = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff}}
    if shared:
        m["shared"] = {"ff": shared}
    return m


V_A = {
    "architecture": "Visadra", "vocab": 131, "width": 72, "embedding": {"scale": 0.7}, "logit_scale": 1.5,
    "norm": {"eps": 1e-5},
    "layers": [
        {"type": "latent_attention", "mixer": _latent(3, 20, 12, 8, 28, 40, 0.2, 500.0), "mlp": _moe(5, 1, 24, 40)},
        {"type": "mingru", "mixer": {"width": 56}, "mlp": {"kind": "dense", "ff": 100}},
        {"type": "latent_attention", "mixer": _latent(3, 20, 12, 8, 28, 40, 0.2, 500.0, window=19), "mlp": None},
        {"type": "mingru_2", "mixer": {"width": 72}, "mlp": _moe(4, 3, 16, 0)},
    ],
}
# sizes that are multiples of 16: what the matrix-core kernels take
V_B = {
    "architecture": "Visadra", "vocab": 256, "width": 128, "embedding": {"scale": 1.0}, "logit_scale": 1.0,
    "norm": {"eps": 1e-6},
    "layers": [
        {"type": "mingru_2", "mixer": {"width": 192}, "mlp": {"kind": "dense", "ff": 256}},
        {"type": "latent_attention", "mixer": _latent(4, 32, 16, 16, 32, 64, 0.15, 10000.0), "mlp": _moe(8, 2, 32, 64)},
        {"type": "latent_attention", "mixer": _latent(8, 16, 32, 32, 16, 128, 0.15, 10000.0, window=48),
         "mlp": {"kind": "dense", "ff": 64}},
        {"type": "mingru", "mixer": {"width": 128}, "mlp": None},
    ],
}
# one head, one expert of one, a rotation of nothing but a pair
V_C = {
    "architecture": "Visadra", "vocab": 77, "width": 48, "embedding": {"scale": 2.0}, "logit_scale": 0.5,
    "norm": {"eps": 3e-5},
    "layers": [
        {"type": "latent_attention", "mixer": _latent(1, 48, 6, 2, 10, 24, 0.1, 50.0), "mlp": _moe(1, 1, 20, 12)},
        {"type": "latent_attention", "mixer": _latent(5, 8, 4, 4, 8, 16, 0.3, 2000.0), "mlp": {"kind": "dense", "ff": 40}},
        {"type": "mingru", "mixer": {"width": 20}, "mlp": _moe(6, 6, 8, 0)},
    ],
}
CONFIGS = {"A": V_A, "B": V_B, "C": V_C}
PAGE_SIZES = {"A": 4, "B": 16, "C": 8}


def make_model_dir(tmp_path, which, seed: int = 77, dtype=torch.float32, config=None) -> str:
    cfg = VisadraConfig.from_dict(config or CONFIGS[which])
    path = os.path.join(str(tmp_path), f"visadra_{which}_{seed}")
    write_model_dir(cfg, path, seed, dtype)
    return path


def rewrite(model_dir: str, change) -> None:
    """`change(name, tensor) -> tensor or None` over the folder's tensors."""
    from safetensors.torch import load_file, save_file

    path = os.path.join(model_dir, "model.safetensors")
    tensors = load_file(path)
    for name in list(tensors):
        new = change(name, tensors[name])
        if new is not None:
            tensors[name] = new.to(tensors[name].dtype).contiguous()
    save_file(tensors, path, metadata={"format": "pt"})


def sharpen(model_dir: str, factor: float = 1.0, sink: float = None, gates: float = 1.0,
            fixed_routes: bool = False) -> None:
    """Random weights average everything: attention weights are flat, gates sit at one half, routers
    barely prefer anybody.  Here the query projections, the plain keys' up projections and the rotated
    key's rows grow by `factor` (scores by its square, so single keys, near or hundreds back, carry
    the softmax and a lost one moves the logits), the recurrences' gate and candidate projections by
    `gates` (states that remember far back or forget at once), and with `sink` the first head's sink
    is set to it.  Routers and the embedding grow 50-fold (clear choices, gains far from equal; a first
    layer whose input is as large as the later ones').  `fixed_routes`: the
    routers' biases are spread so far that they alone decide which experts are chosen (the gains still
    follow the tokens): for runs in bfloat16, where a close call between two experts may fall either
    way and nothing could be compared after it; which expert a token gets is pinned in 32-bit."""
    from safetensors import safe_open

    with safe_open(os.path.join(model_dir, "model.safetensors"), framework="pt") as f:
        ranks = {n[: -len("dkv.norm")]: f.get_slice(n).get_shape()[0] for n in f.keys() if n.endswith(".mix.dkv.norm")}

    def change(name, t):
        if name.endswith(".mix.q") or name.endswith(".mix.uk"):
            return t.float() * factor
        if name.endswith(".mix.dkv"):
            t = t.float().clone()
            t[ranks[name[: -len("dkv")]] :] *= factor
            return t
        if name == "embed":
            return t.float() * 50.0  # rows of about unit size, like everything that the layers add to them
        if name.endswith(".mix.z") or name.endswith(".mix.x"):
            return t.float() * gates
        if name.endswith(".mlp.router"):
            return t.float() * 50.0
        if name.endswith(".mlp.router.b") and fixed_routes:
            g = torch.Generator().manual_seed(len(name) + t.shape[0])
            return torch.randperm(t.shape[0], generator=g).float() * 3000.0
        if sink is not None and name.endswith(".mix.sink"):
            s = t.float().clone()
            s[0] = sink
            return s
        return None

    rewrite(model_dir, change)


def plain_logits(model_dir: str, requests: Dict[str, List[int]]) -> Dict[str, torch.Tensor]:
    cfg, w = plain.read_model_dir(model_dir)
    return {rid: plain.model_logits(tokens, w, cfg) for rid, tokens in requests.items()}


def run_tool(model_dir: str, dtype: str, out_dir: str, trace: TraceBuilder, page_size: int = None, max_requests: int = 4,
             in_process_ops=None, max_tokens: int = None) -> None:
    """bin/trace_run over the trace as a child process, as a user would run it; with
    `in_process_ops` its loop runs here on the CPU with substitute kernels."""
    max_tokens = max_tokens or trace.max_tokens
    if in_process_ops is not None:
        from litellmengine_amd.entrypoints.trace_run import replay
        from litellmengine_amd.models import load_model

        out = io.StringIO()
        model = load_model(model_dir, dtype, device="cpu", ops=in_process_ops)
        replay(model, out_dir, max_tokens, page_size or 16, max_requests, io.StringIO(trace.text()), out)
        done = out.getvalue().split("\n")
    else:
        argv = ["--model", model_dir, "--dtype", dtype, "--out", out_dir, "--max-tokens", str(max_tokens),
                "--max-requests", str(max_requests)]
        if page_size:
            argv += ["--page-size", str(page_size)]
        proc = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run")] + argv, input=trace.text(),
                              text=True, capture_output=True, timeout=600)
        assert proc.returncode == 0, proc.stderr[-3000:]
        done = proc.stdout.split("\n")
    assert [l for l in done if l] == [f"done {i}" for i in range(len(trace.steps))]


def attention_peaks(model_dir: str, tokens: List[int]) -> float:
    """Share of the queries past the first few, over the heads of the plain model's first
    latent-attention layer, that give one key more than half of the weight."""
    cfg, w = plain.read_model_dir(model_dir)
    i = next(k for k, layer in enumerate(cfg["layers"]) if layer["type"] == "latent_attention")
    m, eps = cfg["layers"][i]["mixer"], float(cfg["norm"]["eps"])
    x = w["embed"][torch.tensor(tokens)] * float(cfg["embedding"]["scale"])
    if i:
        x = plain.residual_streams(tokens, w, {**cfg, "layers": cfg["layers"][:i]})[-1]
    p, T, H, d, rank = f"l{i}.mix.", len(tokens), m["heads"], m["dim"], m["kv_rank"]
    q = (x @ w[p + "q"].T).reshape(T, H, d + m["rot_dim"])
    dkv = x @ w[p + "dkv"].T
    c = plain.rms_unit(dkv[:, :rank], eps) * w[p + "dkv.norm"]
    pos = list(range(T))
    kr = plain.rotate_interleaved(dkv[:, rank:], pos, float(m["rot"]["base"]), int(m["rot"]["dims"]))
    qr = plain.rotate_interleaved(q[:, :, d:], pos, float(m["rot"]["base"]), int(m["rot"]["dims"]))
    k = (c @ w[p + "uk"].T).reshape(T, H, d)
    peaked = total = 0
    for h in range(H):
        sc = (q[:, h, :d] @ k[:, h].T + qr[:, h] @ kr.T) * float(m["scale"])
        for t in range(8, T):
            lo = max(0, t - m["window"] + 1) if m.get("window") else 0
            e = torch.exp(sc[t, lo : t + 1] - sc[t, lo : t + 1].max())
            peaked += int(float(e.max() / (e.sum() + torch.exp(w[p + "sink"][h] - sc[t, lo : t + 1].max()))) > 0.5)
            total += 1
    return peaked / total
