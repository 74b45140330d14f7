"""Tiny Malilorn configurations and helpers for the tests.  Between them every size and option differs:
keys and values of equal or unequal width (values wider and narrower than keys), convolutions of two to five
taps or none, rotations over a pair, a few elements or the whole head, with and without stretched
frequencies, one key/value head or several or as many as query heads, recurrence heads whose widths do or do
not add up to the model's, dense and routed feed-forwards in either order, with and without a shared expert,
one expert chosen or several or all, layers without a feed-forward, with and without a cap on the logits,
mixer constants of one and other values."""
from __future__ import annotations

import os
from typing import Dict, List

import torch

from litellmengine_amd.config import MalilornConfig
from litellmengine_amd.weights import write_model_dir
from tests.plain import malilorn_plain as plain
from tests.visadra_util import rewrite, run_tool  # noqa: F401  (the same tool, whatever the architecture)


def left(heads, kv_heads, dim, vdim, scale, conv, base=10000.0, dims=0, scaling=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if conv:
        m["conv"] = conv
    if dims:
        m["rot"] = {"base": base, "dims": dims}
        if scaling:
            m["rot"]["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    return m


def par(l, heads, dim, rank, left_scale=1.0, right_scale=1.0):
    return {"left": l, "right": {"heads": heads, "dim": dim, "decay_rank": rank}, "left_scale": left_scale,
            "right_scale": right_scale}


def moe(experts, top, ff, shared=None):
    m = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if shared:
        m["shared"] = {"ff": shared}
    return m


def dense(ff):
    return {"kind": "dense", "ff": ff}


# odd sizes: what only the generic kernels take
M_A = {
    "architecture": "Malilorn", "vocab": 131, "width": 72, "norm": {"eps": 1e-5}, "logit_softcap": 40.0,
    "layers": [
        {"type": "parallel", "mlp": moe(5, 2, 24, shared=20),
         "mixer": par(left(6, 2, 24, 40, 0.2, 3, 500.0, 8, scaling=(4.0, 2.0, 5.0, 64)), 3, 24, 8, 0.7, 1.3)},
        {"type": "parallel", "mlp": dense(52),
         "mixer": par(left(3, 3, 16, 16, 0.25, 5, 10000.0, 16), 2, 36, 5, 1.0, 1.0)},
        {"type": "parallel", "mlp": None,
         "mixer": par(left(4, 1, 40, 24, 0.15, 2, 300.0, 6, scaling=(8.0, 1.0, 4.0, 32)), 1, 20, 3, 2.0, 0.25)},
        {"type": "parallel", "mlp": moe(4, 4, 16),
         "mixer": par(left(6, 2, 24, 40, 0.3, 3, 500.0, 8, scaling=(4.0, 2.0, 5.0, 64)), 3, 24, 8, 1.1, 0.9)},
    ],
}
# sizes that the matrix-core kernels take
M_B = {
    "architecture": "Malilorn", "vocab": 256, "width": 128, "norm": {"eps": 1e-6},
    "layers": [
        {"type": "parallel", "mlp": dense(96),
         "mixer": par(left(8, 2, 32, 64, 0.15, 4, 10000.0, 32), 2, 64, 16, 1.5, 0.5)},
        {"type": "parallel", "mlp": moe(8, 3, 32),
         "mixer": par(left(4, 4, 64, 32, 0.1, 3, 250000.0, 16, scaling=(8.0, 1.0, 4.0, 128)), 4, 32, 4, 0.8, 0.8)},
        {"type": "parallel", "mlp": moe(6, 1, 64, shared=40),
         "mixer": par(left(16, 1, 32, 32, 0.2, 2, 10000.0, 8), 2, 64, 8, 1.0, 2.0)},
    ],
}
# one head, one expert, no convolution, a rotation of nothing but a pair and none at all, a wide recurrence head
M_C = {
    "architecture": "Malilorn", "vocab": 77, "width": 48, "norm": {"eps": 3e-5}, "logit_softcap": 30.0,
    "layers": [
        {"type": "parallel", "mlp": moe(1, 1, 20, shared=12),
         "mixer": par(left(1, 1, 48, 10, 0.1, 0, 50.0, 2), 1, 100, 3, 0.5, 0.5)},
        {"type": "parallel", "mlp": None,
         "mixer": par(left(5, 1, 8, 12, 0.3, 4), 6, 8, 2, 1.0, 3.0)},
        {"type": "parallel", "mlp": dense(8),
         "mixer": par(left(2, 2, 12, 12, 0.3, 1, 2000.0, 4), 2, 16, 6)},
    ],
}
CONFIGS = {"A": M_A, "B": M_B, "C": M_C}
PAGE_SIZES = {"A": 4, "B": 16, "C": 8}


def make_model_dir(tmp_path, which, seed: int = 77, dtype=torch.float32, config=None) -> str:
    cfg = MalilornConfig.from_dict(config or CONFIGS[which])
    path = os.path.join(str(tmp_path), f"malilorn_{which}_{seed}")
    write_model_dir(cfg, path, seed, dtype)
    return path


def sharpen(model_dir: str, factor: float = 1.0, same_experts: bool = False, memory: float = 1.0) -> None:
    """Random weights average everything and hide faults: attention is flat, the mixing weights sit at zero,
    every decay is the same, routers barely prefer anybody, the logits never reach their cap.  Here the query and
    key norms' weights grow by `factor` (scores by its square: single keys, near or far back, carry the softmax),
    biases grow fiftyfold, the norms' weights spread over (0.5, 1.5), the mixing weights over (0, 1), the decays'
    offsets over (-5 memory, 1) (channels that remember for hundreds of tokens beside channels that forget at
    once), the bonus and the decays' projections grow, the routers, the shared experts' gates and the embedding grow
    (clear choices, weights far from equal, a first layer whose input is as large as the later ones').
    `same_experts`: every routed expert of a layer gets the first one's weights, so that the choice itself moves
    nothing (the weights still follow the tokens): for runs in bfloat16, where a close call between two experts
    may fall either way and nothing could be compared after it; which expert a token gets is pinned in 32-bit."""

    def spread(t, lo, hi, salt):
        g = torch.Generator().manual_seed(salt + t.numel())
        return torch.rand(t.shape, generator=g) * (hi - lo) + lo

    from safetensors.torch import load_file

    first = {}
    if same_experts:
        for name, t in load_file(os.path.join(model_dir, "model.safetensors")).items():
            if ".mlp.e0." in name:
                first[name] = t

    def change(name, t):
        if name.endswith(".q.norm") or name.endswith(".k.norm"):
            return t.float() * factor
        if name.endswith(".b"):
            return t.float() * 10.0
        if name.endswith("norm1") or name.endswith("norm2") or name.endswith("norm1b") or name.endswith("norm2b") \
                or name == "final.norm":
            return spread(t, 0.5, 1.5, 1 + len(name))
        if ".right.mu." in name:
            return spread(t, 0.05, 0.95, 2 + ord(name[-1]))
        if name.endswith(".right.w0"):
            return spread(t, -5.0 * memory, 1.0, 3)
        if name.endswith(".right.w1") or name.endswith(".right.w2"):
            return t.float() * 15.0
        if name.endswith(".right.u"):
            return t.float() * 25.0
        if name == "embed":
            return t.float() * 30.0
        if name.endswith(".mlp.router") or name.endswith(".shared.sg"):
            return t.float() * 10.0
        if same_experts and ".mlp.e" in name:
            i = name.index(".mlp.e")
            return first[name[:i] + ".mlp.e0." + name.split(".")[-1]].float()
        return None

    rewrite(model_dir, change)


def read(model_dir: str):
    return plain.load(model_dir)


def plain_logits(model_dir: str, requests: Dict[str, List[int]]) -> Dict[str, torch.Tensor]:
    cfg, w = plain.load(model_dir)
    return {rid: plain.forward(cfg, w, tokens) for rid, tokens in requests.items()}


def residual_streams(model_dir: str, tokens: List[int]) -> List[torch.Tensor]:
    cfg, w = plain.load(model_dir)
    out: List[torch.Tensor] = []
    plain.forward(cfg, w, tokens, out)
    return out
