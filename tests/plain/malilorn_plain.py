"""Plain, slow Malilorn implementation: the oracle of the Malilorn tests.

Whole sequences, no cache, no state carried between calls, one function per
mechanism, nothing shared with the engine's code.  Everything runs on the CPU
in float64 (or the dtype of the weights handed in).  `cfg` is the dictionary of
config.json; `w` maps tensor names to tensors.

Notation: h is a sublayer's normed input [T, width]; W x means `x @ W.T` with W
stored [out, in]; positions count from 0.
"""
from __future__ import annotations

import json
import math
import os
from typing import Dict, List, Optional

import torch


# --------------------------------------------------------------------------
# small pieces
# --------------------------------------------------------------------------
def rms_unit(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last axis (eps inside the root)."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    return rms_unit(x, eps) * weight


def sigmoid(x: torch.Tensor) -> torch.Tensor:
    return 1.0 / (1.0 + torch.exp(-x))


def silu(x: torch.Tensor) -> torch.Tensor:
    return x * sigmoid(x)


def relu(x: torch.Tensor) -> torch.Tensor:
    return torch.clamp(x, min=0.0)


def relu_squared(x: torch.Tensor) -> torch.Tensor:
    return relu(x) ** 2


# --------------------------------------------------------------------------
# left mixer: attention behind a short convolution
# --------------------------------------------------------------------------
def short_conv(u: torch.Tensor, taps: torch.Tensor) -> torch.Tensor:
    """u [T, C], taps [C, J]: y_t = sum_j taps[:, j] * u_(t - J + 1 + j), zeros before the start.
    The last tap meets the token itself, the first one the token J - 1 places back."""
    T, C = u.shape
    J = taps.shape[1]
    padded = torch.cat([torch.zeros((J - 1, C), dtype=u.dtype), u], dim=0)
    y = torch.zeros_like(u)
    for j in range(J):
        y = y + padded[j : j + T] * taps[:, j]
    return y


def rotary_frequencies(base: float, dims: int, scaling: Optional[dict]) -> torch.Tensor:
    """f_i = base^(-2i/dims), i < dims / 2; with `scaling` the long wavelengths are stretched:
    kept below original / high, divided by factor above original / low, blended in between."""
    out = []
    for i in range(dims // 2):
        f = float(base) ** (-2.0 * i / dims)
        if scaling:
            factor, low, high, original = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
            wavelength = 2.0 * math.pi / f
            if wavelength < original / high:
                pass
            elif wavelength > original / low:
                f = f / factor
            else:
                s = (original / wavelength - low) / (high - low)
                f = (1.0 - s) * f / factor + s * f
        out.append(f)
    return torch.tensor(out, dtype=torch.float64)


def rotate_half_split(x: torch.Tensor, positions: torch.Tensor, freqs: torch.Tensor) -> torch.Tensor:
    """x [T, heads, d]; the first 2 len(freqs) elements of every head turn, element i with i + len(freqs)."""
    half = freqs.shape[0]
    if half == 0:
        return x
    angle = positions.to(torch.float64)[:, None] * freqs[None, :]
    cos, sin = torch.cos(angle).to(x.dtype)[:, None, :], torch.sin(angle).to(x.dtype)[:, None, :]
    a, b, rest = x[..., :half], x[..., half : 2 * half], x[..., 2 * half :]
    return torch.cat([a * cos - b * sin, b * cos + a * sin, rest], dim=-1)


def causal_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float) -> torch.Tensor:
    """q [T, H, d], k [T, G, d], v [T, G, dv]; query head h reads key/value head h // (H / G); token i sees j <= i."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros((T, H, v.shape[2]), dtype=q.dtype)
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        s = s.masked_fill(torch.ones((T, T), dtype=torch.bool).triu(1), float("-inf"))
        out[:, h] = torch.softmax(s, dim=-1) @ v[:, g]
    return out


def left_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: dict, eps: float) -> torch.Tensor:
    T = h.shape[0]
    H, G, d, dv = m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m.get("vdim", m["dim"])
    q, k, v = h @ w[p + "q"].T, h @ w[p + "k"].T, h @ w[p + "v"].T
    if m.get("conv"):
        q, k, v = short_conv(q, w[p + "q.conv"]), short_conv(k, w[p + "k.conv"]), short_conv(v, w[p + "v.conv"])
    q = rms_norm(q.view(T, H, d), w[p + "q.norm"], eps)
    k = rms_norm(k.view(T, G, d), w[p + "k.norm"], eps)
    rot = m.get("rot")
    if rot and rot.get("dims"):
        f = rotary_frequencies(rot["base"], rot["dims"], rot.get("scaling"))
        pos = torch.arange(T)
        q, k = rotate_half_split(q, pos, f), rotate_half_split(k, pos, f)
    o = causal_attention(q, k, v.view(T, G, dv), m["scale"])
    return o.reshape(T, H * dv) @ w[p + "o"].T


# --------------------------------------------------------------------------
# right mixer: a per-head matrix state with data-dependent decay
# --------------------------------------------------------------------------
def matrix_state_walk(r, k, v, decay, u):
    """One head.  r, k, v, decay [T, d]; u [d].  o_t = (S + diag(u) k_t v_t^T)^T r_t, then
    S <- diag(decay_t) S + k_t v_t^T; S starts at zero."""
    T, d = r.shape
    S = torch.zeros((d, d), dtype=r.dtype)
    out = []
    for t in range(T):
        kv = torch.outer(k[t], v[t])
        out.append((S + u[:, None] * kv).T @ r[t])
        S = decay[t][:, None] * S + kv
    return torch.stack(out)


def right_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: dict, eps: float) -> torch.Tensor:
    T = h.shape[0]
    heads, dim = m["heads"], m["dim"]
    prev = torch.zeros_like(h)
    prev[1:] = h[:-1]
    mix = {s: h + (prev - h) * w[p + "mu." + s] for s in "rkvgw"}
    r = (mix["r"] @ w[p + "r"].T).view(T, heads, dim)
    k = (mix["k"] @ w[p + "k"].T).view(T, heads, dim)
    v = (mix["v"] @ w[p + "v"].T).view(T, heads, dim)
    gate = silu(mix["g"] @ w[p + "g"].T)
    decay = torch.exp(-torch.exp(torch.tanh(mix["w"] @ w[p + "w1"].T) @ w[p + "w2"].T + w[p + "w0"])).view(T, heads, dim)
    u = w[p + "u"].reshape(heads, dim)
    o = torch.stack([matrix_state_walk(r[:, i], k[:, i], v[:, i], decay[:, i], u[i]) for i in range(heads)], dim=1)
    o = rms_unit(o, eps).reshape(T, heads * dim) * w[p + "norm"] * gate
    return o @ w[p + "o"].T


def parallel_mixer(h, w, p: str, m: dict, eps: float) -> torch.Tensor:
    left = left_mixer(h, w, p + "left.", m["left"], eps)
    right = right_mixer(h, w, p + "right.", m["right"], eps)
    return m.get("left_scale", 1.0) * left + m.get("right_scale", 1.0) * right


# --------------------------------------------------------------------------
# feed-forwards
# --------------------------------------------------------------------------
def dense_ff(h, w, p: str) -> torch.Tensor:
    gate = h @ w[p + "gate"].T + w[p + "gate.b"]
    up = h @ w[p + "up"].T + w[p + "up.b"]
    return (relu(gate) * up) @ w[p + "down"].T + w[p + "down.b"]


def small_expert(x, w, p: str) -> torch.Tensor:
    return relu_squared(x @ w[p + "up"].T) @ w[p + "down"].T


def routed_choice(h, w, p: str, top: int):
    """(ids [T, top], weights [T, top]): the `top` largest sigmoid scores, as they are."""
    s = sigmoid(h @ w[p + "router"].T)
    weights, ids = torch.topk(s, top, dim=-1)
    return ids, weights


def moe_ff(h, w, p: str, f: dict) -> torch.Tensor:
    ids, weights = routed_choice(h, w, p, f["router"]["top"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, g in zip(ids[t].tolist(), weights[t]):
            out[t] = out[t] + small_expert(g * h[t], w, f"{p}e{e}.")  # the weight meets the expert's input
    if f.get("shared"):
        out = out + small_expert(h, w, p + "shared.") * sigmoid(h @ w[p + "shared.sg"].T)
    return out


def feed_forward(h, w, p: str, f: dict) -> torch.Tensor:
    return dense_ff(h, w, p) if f.get("kind") == "dense" else moe_ff(h, w, p, f)


# --------------------------------------------------------------------------
# the model
# --------------------------------------------------------------------------
def layer(x, w, i: int, spec: dict, eps: float) -> torch.Tensor:
    p = f"l{i}."
    x = x + rms_norm(parallel_mixer(rms_norm(x, w[p + "norm1"], eps), w, p + "mix.", spec["mixer"], eps), w[p + "norm1b"], eps)
    if spec.get("mlp"):
        x = x + rms_norm(feed_forward(rms_norm(x, w[p + "norm2"], eps), w, p + "mlp.", spec["mlp"]), w[p + "norm2b"], eps)
    return x


def forward(cfg: dict, w: Dict[str, torch.Tensor], tokens, layers_out: Optional[List[torch.Tensor]] = None) -> torch.Tensor:
    """Logits [T, vocab] of one whole sequence; `layers_out` collects the residual stream after every layer."""
    eps = cfg["norm"]["eps"]
    x = w["embed"][torch.as_tensor(list(tokens), dtype=torch.long)]
    for i, spec in enumerate(cfg["layers"]):
        x = layer(x, w, i, spec, eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    logits = rms_norm(x, w["final.norm"], eps) @ w["embed"].T
    cap = cfg.get("logit_softcap")
    return cap * torch.tanh(logits / cap) if cap else logits


def router_margins(cfg: dict, w: Dict[str, torch.Tensor], tokens) -> torch.Tensor:
    """[T]: per position the smallest gap, over the routed layers, between the last chosen expert's logit and the
    best one left out (infinity where nothing is left out): where it is tiny, rounding decides the choice."""
    eps = cfg["norm"]["eps"]
    x = w["embed"][torch.as_tensor(list(tokens), dtype=torch.long)]
    gap = torch.full((x.shape[0],), float("inf"), dtype=x.dtype)
    for i, spec in enumerate(cfg["layers"]):
        p = f"l{i}."
        x = x + rms_norm(parallel_mixer(rms_norm(x, w[p + "norm1"], eps), w, p + "mix.", spec["mixer"], eps), w[p + "norm1b"], eps)
        f = spec.get("mlp")
        if not f:
            continue
        h = rms_norm(x, w[p + "norm2"], eps)
        if f.get("kind") != "dense" and f["router"]["experts"] > f["router"]["top"]:
            z = torch.sort(h @ w[p + "mlp.router"].T, dim=-1, descending=True).values
            top = f["router"]["top"]
            gap = torch.minimum(gap, z[:, top - 1] - z[:, top])
        x = x + rms_norm(feed_forward(h, w, p + "mlp.", f), w[p + "norm2b"], eps)
    return gap


def load(model_dir: str, dtype=torch.float64):
    from safetensors.torch import load_file

    with open(os.path.join(model_dir, "config.json")) as f:
        cfg = json.load(f)
    w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in load_file(os.path.join(model_dir, "model.safetensors")).items()}
    return cfg, w


def greedy(cfg, w, prompt, new_tokens: int) -> List[int]:
    ids = list(prompt)
    for _ in range(new_tokens):
        ids.append(int(torch.argmax(forward(cfg, w, ids)[-1])))
    return ids[len(prompt):]
