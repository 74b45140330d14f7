"""Tiny Birelix configurations and helpers for the tests.  Between them every size and option differs: latent
attention with rotated parts of a pair or many elements, ranks that are or are not multiples of 16, one head or
many, values wider and narrower than keys; window attention with one key/value head, several, or as many as
query heads, windows from 3 tokens to none, values of another width than keys; delta layers with one to five
taps, as many value heads as query/key heads or several times as many, heads of 8 to 100 channels; dense and
routed feed-forwards in any order, one group or several, one kept or all, one expert chosen or all, groups of a
single expert, layers without a feed-forward, an embedding scale of one and others."""
from __future__ import annotations

import os
from typing import Dict, List

import torch

from litellmengine_amd.config import BirelixConfig
from litellmengine_amd.weights import write_model_dir
from tests.plain import birelix_plain as plain
from tests.visadra_util import rewrite, run_tool  # noqa: F401  (the same tool, whatever the architecture)


def latent(heads, dim, rot_dim, vdim, kv_rank, q_rank, scale, base=10000.0, dims=None):
    return {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank, "scale": scale,
            "rot": {"base": base, "dims": rot_dim if dims is None else dims}}


def window(heads, kv_heads, dim, vdim, scale, size=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if size:
        m["mask"] = {"size": size}
    return m


def delta(heads, kv_heads, dim, vdim, conv):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}


def moe(experts, top, ff, limit, count=1, keep=1):
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit},
            "router": {"experts": experts, "top": top, "groups": {"count": count, "keep": keep}}}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def layer(kind, mixer, mlp):
    return {"type": kind, "mixer": mixer, "mlp": mlp}


# odd sizes: what only the generic kernels take
B_A = {
    "architecture": "Birelix", "vocab": 131, "width": 72, "embedding": {"scale": 3.0}, "norm": {"eps": 1e-5},
    "layers": [
        layer("delta", delta(6, 2, 24, 20, 3), moe(6, 2, 24, 1.5, count=3, keep=2)),
        layer("latent_attention", latent(3, 20, 12, 28, 40, 24, 0.2, 500.0), dense(52)),
        layer("attention", window(6, 2, 24, 40, 0.3, size=19), None),
        layer("delta", delta(3, 3, 36, 44, 5), moe(4, 4, 16, 0.5)),
        layer("attention", window(3, 3, 40, 24, 0.2, size=5), moe(5, 1, 20, 2.0, count=5, keep=3)),
    ],
}
# sizes that the matrix-core kernels take
B_B = {
    "architecture": "Birelix", "vocab": 256, "width": 128, "embedding": {"scale": 11.0}, "norm": {"eps": 1e-6},
    "layers": [
        layer("latent_attention", latent(8, 32, 16, 32, 64, 48, 0.15, 100000.0), dense(96)),
        layer("delta", delta(4, 2, 64, 48, 3), moe(8, 3, 32, 1.5, count=2, keep=1)),
        layer("attention", window(8, 2, 64, 64, 0.12, size=48), moe(12, 3, 64, 3.0, count=4, keep=2)),
        layer("latent_attention", latent(4, 64, 32, 64, 128, 96, 0.1, 10000.0), moe(10, 2, 32, 1.0, count=5, keep=2)),
        layer("delta", delta(8, 8, 32, 64, 2), dense(64)),
        layer("attention", window(4, 4, 32, 32, 0.2), None),
    ],
}
# one head, one expert, one tap, a rotation of nothing but a pair, a window of three tokens, a wide delta head
B_C = {
    "architecture": "Birelix", "vocab": 77, "width": 48, "embedding": {"scale": 1.0}, "norm": {"eps": 3e-5},
    "layers": [
        layer("attention", window(1, 1, 48, 10, 0.1, size=3), moe(1, 1, 20, 1.0)),
        layer("delta", delta(1, 1, 100, 12, 1), None),
        layer("latent_attention", latent(1, 8, 2, 12, 10, 6, 0.4, 50.0), moe(6, 2, 8, 0.7, count=6, keep=3)),
        layer("delta", delta(4, 1, 8, 100, 2), dense(8)),
        layer("latent_attention", latent(5, 12, 6, 8, 20, 30, 0.3, 2000.0, dims=4), None),
    ],
}
CONFIGS = {"A": B_A, "B": B_B, "C": B_C}
PAGE_SIZES = {"A": 4, "B": 16, "C": 8}


def make_model_dir(tmp_path, which, seed: int = 77, dtype=torch.float32, config=None) -> str:
    cfg = BirelixConfig.from_dict(config or CONFIGS[which])
    path = os.path.join(str(tmp_path), f"birelix_{which}_{seed}")
    write_model_dir(cfg, path, seed, dtype)
    return path


def sharpen(model_dir: str, factor: float = 1.0, same_experts: bool = False, memory: float = 1.0, skip=()) -> None:
    """Random weights average everything and hide faults: attention is flat, every decay is the same, the
    corrections are halves, routers barely prefer anybody, and sublayers of N(0, 0.02) weights whisper beside the
    residual stream.  Here the latent attention's query and key projections and the window attention's score scale
    grow with `factor` (single keys, near or far back, carry the softmax, or no key does and the sum's extra place
    takes the weight), biases grow tenfold, the norms' weights spread over (0.5, 1.5), the decays' logarithms over
    (-6 memory, 1) (heads that remember for hundreds of tokens beside heads that forget at once), their offsets
    over (-2, 2), beta's and the decay's projections grow, the heads' gates, the routers and every projection back
    into the stream grow (clear choices, weights far from equal, sublayers as loud as the stream).
    `same_experts`: every routed expert of a layer gets the first one's weights, so that the choice itself moves
    nothing (the weights still follow the tokens): for runs in bfloat16, where a close call between two experts
    may fall either way and nothing could be compared after it; which expert a token gets is pinned in 32-bit.
    `skip`: endings of tensor names that stay as they are."""

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
        if any(name.endswith(x) for x in skip):
            return None
        if same_experts and ".mlp.e" in name:
            i = name.index(".mlp.e")
            t = first[name[:i] + ".mlp.e0." + name.split(".")[-1]]
        if name.endswith(".mix.uq"):
            return t.float() * 2.0 * factor * factor
        if name.endswith(".mix.uk") or name.endswith(".mix.dkv"):
            return t.float() * 2.0 * factor
        if name.endswith(".mix.q.b") or name.endswith(".mix.k.b") or name.endswith(".mix.v.b"):
            return t.float() * 10.0
        if name.endswith("norm1") or name.endswith("norm2") or name == "final.norm" or name.endswith(".mix.norm"):
            return spread(t, 0.5, 1.5, 1 + len(name))
        if name.endswith(".mix.A_log"):
            return spread(t, -6.0 * memory, 1.0, 3)
        if name.endswith(".mix.dt_bias"):
            return spread(t, -2.0, 2.0, 4)
        if name.endswith(".mix.b") or name.endswith(".mix.a"):
            return t.float() * 30.0
        if name.endswith(".mix.g") or name.endswith(".mlp.router"):
            return t.float() * 15.0
        if name.endswith(".mix.o") or name.endswith(".down"):
            return t.float() * 8.0
        if name.endswith(".mix.v") or name.endswith(".mix.uv"):
            return t.float() * 4.0
        return t.float() if same_experts and ".mlp.e" in name else None

    rewrite(model_dir, change)
    if factor != 1.0:  # the window attention's q and k are unit vectors times sqrt(dim): its scores grow with `scale`
        import json

        path = os.path.join(model_dir, "config.json")
        with open(path) as f:
            cfg = json.load(f)
        for spec in cfg["layers"]:
            if spec["type"] == "attention":
                spec["mixer"]["scale"] = spec["mixer"]["scale"] * factor
        with open(path, "w") as f:
            json.dump(cfg, f)


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
