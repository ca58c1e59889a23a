"""Tiny Kezasun configurations and helpers for the tests.  Between them every size and option differs:
keys and values of equal or unequal width, rotations over a few elements or the whole head, with and
without stretched frequencies, windows or none, layers that read another layer's keys and values through
a wider or a narrower window, one head or several, recurrence heads whose widths do or do not add up to
the model's, routers with one group or several, with or without identity experts, all experts chosen or
one, layers without a feed-forward, a residual multiplier of 1 or not."""
from __future__ import annotations

import os
from typing import Dict, List

import torch

from litellmengine_amd.config import KezasunConfig
from litellmengine_amd.weights import write_model_dir
from tests.plain import kezasun_plain as plain
from tests.visadra_util import rewrite, run_tool  # noqa: F401  (the same tool, whatever the architecture)


def attn(heads, kv_heads, dim, vdim, scale, base, dims, window=None, scaling=None, kv_from=None):
    rot = {"base": base, "dims": dims}
    if scaling:
        rot["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "rot": rot}
    if window:
        m["mask"] = {"size": window}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def moe(experts, identity, top, ff, groups=1, keep=1):
    return {"kind": "moe", "expert": {"ff": ff},
            "router": {"experts": experts, "identity": identity, "top": top, "groups": {"count": groups, "keep": keep}}}


def wkv(heads, dim, rank):
    return {"heads": heads, "dim": dim, "decay_rank": rank}


# odd sizes: what only the generic kernels take
K_A = {
    "architecture": "Kezasun", "vocab": 131, "width": 72, "residual_mult": 0.5, "norm": {"eps": 1e-5},
    "layers": [
        {"type": "attention", "mixer": attn(6, 2, 24, 40, 0.2, 500.0, 8, window=19, scaling=(4.0, 2.0, 5.0, 64)),
         "mlp": moe(5, 1, 2, 24, groups=3, keep=2)},
        {"type": "wkv", "mixer": wkv(3, 24, 8), "mlp": None},
        {"type": "attention", "mixer": attn(6, 2, 24, 40, 0.3, 500.0, 8, window=37, scaling=(4.0, 2.0, 5.0, 64), kv_from=0),
         "mlp": moe(4, 0, 4, 16)},
        {"type": "wkv", "mixer": wkv(2, 36, 5), "mlp": moe(3, 3, 3, 20, groups=2, keep=1)},
        {"type": "attention", "mixer": attn(3, 3, 16, 16, 0.25, 10000.0, 16), "mlp": None},
    ],
}
# sizes that the matrix-core kernels take
K_B = {
    "architecture": "Kezasun", "vocab": 256, "width": 128, "residual_mult": 1.0, "norm": {"eps": 1e-6},
    "layers": [
        {"type": "wkv", "mixer": wkv(2, 64, 16), "mlp": moe(8, 8, 6, 32, groups=4, keep=2)},
        {"type": "attention", "mixer": attn(8, 2, 32, 32, 0.15, 10000.0, 32, window=48), "mlp": moe(6, 2, 3, 64, groups=2, keep=2)},
        {"type": "attention", "mixer": attn(8, 2, 32, 32, 0.2, 10000.0, 32, window=16, kv_from=1), "mlp": None},
        {"type": "wkv", "mixer": wkv(4, 32, 4), "mlp": None},
        {"type": "attention", "mixer": attn(4, 4, 64, 32, 0.1, 250000.0, 16, scaling=(8.0, 1.0, 4.0, 128)),
         "mlp": moe(4, 4, 4, 48, groups=4, keep=3)},
        {"type": "attention", "mixer": attn(4, 4, 64, 32, 0.1, 250000.0, 16, scaling=(8.0, 1.0, 4.0, 128), kv_from=4),
         "mlp": moe(2, 0, 1, 16)},
    ],
}
# one head, one expert, a rotation of nothing but a pair, a wide recurrence head
K_C = {
    "architecture": "Kezasun", "vocab": 77, "width": 48, "residual_mult": 0.3, "norm": {"eps": 3e-5},
    "layers": [
        {"type": "attention", "mixer": attn(1, 1, 48, 10, 0.1, 50.0, 2, window=7), "mlp": moe(1, 0, 1, 20)},
        {"type": "wkv", "mixer": wkv(1, 100, 3), "mlp": moe(1, 5, 2, 12, groups=6, keep=3)},
        {"type": "attention", "mixer": attn(5, 1, 8, 12, 0.3, 2000.0, 4), "mlp": None},
        {"type": "wkv", "mixer": wkv(6, 8, 2), "mlp": moe(6, 0, 6, 8, groups=3, keep=3)},
    ],
}
# recurrences alone (no cache group at all), and attention alone (no state rows)
K_D = {
    "architecture": "Kezasun", "vocab": 50, "width": 32, "residual_mult": 0.7, "norm": {"eps": 1e-5},
    "layers": [
        {"type": "wkv", "mixer": wkv(2, 16, 4), "mlp": moe(3, 1, 2, 8, groups=2, keep=1)},
        {"type": "wkv", "mixer": wkv(1, 32, 2), "mlp": None},
    ],
}
K_E = {
    "architecture": "Kezasun", "vocab": 50, "width": 32, "residual_mult": 0.7, "norm": {"eps": 1e-5},
    "layers": [
        {"type": "attention", "mixer": attn(2, 1, 16, 16, 0.25, 100.0, 8, window=5), "mlp": None},
        {"type": "attention", "mixer": attn(2, 1, 16, 16, 0.25, 100.0, 8, kv_from=0), "mlp": moe(2, 0, 1, 8)},
    ],
}
CONFIGS = {"A": K_A, "B": K_B, "C": K_C, "D": K_D, "E": K_E}
PAGE_SIZES = {"A": 4, "B": 16, "C": 8, "D": 4, "E": 16}


def make_model_dir(tmp_path, which, seed: int = 77, dtype=torch.float32, config=None) -> str:
    cfg = KezasunConfig.from_dict(config or CONFIGS[which])
    path = os.path.join(str(tmp_path), f"kezasun_{which}_{seed}")
    write_model_dir(cfg, path, seed, dtype)
    return path


def sharpen(model_dir: str, factor: float = 1.0, fixed_routes: bool = False, memory: float = 1.0) -> None:
    """Random weights average everything and hide faults: attention is flat, the mixing weights and the norms'
    stored weights sit at zero, every decay is the same, routers barely prefer anybody.  Here the query and key
    norms' weights grow by `factor` (scores by its square: single keys, near or far back, carry the softmax, the
    sink takes a real share where all scores are low), biases grow tenfold, the norms' stored weights spread to
    +-0.3, the mixing weights spread over (0, 1), the decays' offsets over (-5 memory, 1) (channels that remember
    for hundreds of tokens beside channels that forget at once), the bonus and the decays' projections grow, the
    routers and the embedding grow 50-fold (clear choices, gains far from equal; a first layer whose input is as
    large as the later ones').  `fixed_routes`: the corrections are spread so far that they alone decide which
    experts are chosen (the gains still follow the tokens): for runs in bfloat16, where a close call between two
    experts may fall either way and nothing could be compared after it; which expert a token gets is pinned in
    32-bit."""

    def spread(t, lo, hi, salt):
        g = torch.Generator().manual_seed(salt + t.numel())
        return torch.rand(t.shape, generator=g) * (hi - lo) + lo

    def change(name, t):
        if name.endswith(".q.norm") or name.endswith(".k.norm"):
            return t.float() * factor
        if name.endswith(".b"):
            return t.float() * 10.0
        if name.endswith("norm1") or name == "final.norm":
            return spread(t, -0.3, 0.3, 1)
        if ".mix.mu." in name:
            return spread(t, 0.05, 0.95, 2 + ord(name[-1]))
        if name.endswith(".mix.w0"):
            return spread(t, -5.0 * memory, 1.0, 3)
        if name.endswith(".mix.w1") or name.endswith(".mix.w2"):
            return t.float() * 15.0
        if name.endswith(".mix.u"):
            return t.float() * 25.0
        if name == "embed":
            return t.float() * 50.0
        if name.endswith(".mlp.router"):
            return t.float() * 50.0
        if name.endswith(".mlp.correction"):
            if fixed_routes:
                g = torch.Generator().manual_seed(len(name) + t.shape[0])
                return torch.randperm(t.shape[0], generator=g).float() * 30.0
            return t.float() * 5.0  # (about a tenth: of the size of the scores)
        return None

    rewrite(model_dir, change)


def plain_logits(model_dir: str, requests: Dict[str, List[int]]) -> Dict[str, torch.Tensor]:
    cfg, w = plain.read_model_dir(model_dir)
    return {rid: plain.model_logits(tokens, w, cfg) for rid, tokens in requests.items()}
