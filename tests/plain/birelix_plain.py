"""Plain, slow Birelix implementation: the oracle of the Birelix tests.

Whole sequences, no cache, no state carried between calls, one function per
mechanism, nothing shared with the engine's code.  Everything runs on the CPU
in float64 (or the dtype of the weights handed in).  `cfg` is the dictionary of
config.json; `w` maps tensor names to tensors.

Notation: h is a sublayer's normed input [T, width]; W x means `x @ W.T` with W
stored [out, in]; positions count from 0; `p` is a tensor-name prefix.
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


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    return rms_unit(x, eps) * weight


def sigmoid(x: torch.Tensor) -> torch.Tensor:
    return 1.0 / (1.0 + torch.exp(-x))


def silu(x: torch.Tensor) -> torch.Tensor:
    return x * sigmoid(x)


def softplus(x: torch.Tensor) -> torch.Tensor:
    """log(1 + e^x), written so that large x do not overflow."""
    return torch.clamp(x, min=0.0) + torch.log1p(torch.exp(-x.abs()))


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def rotate_neighbours(x: torch.Tensor, positions: torch.Tensor, dims: int, base: float) -> torch.Tensor:
    """x [T, ..., n >= dims]: elements 2i and 2i+1 (i < dims/2) turn by the angle pos * base^(-2i/dims);
    elements from `dims` on pass."""
    out = x.clone()
    T = x.shape[0]
    shape = [T] + [1] * (x.dim() - 2)
    for i in range(dims // 2):
        a = positions.to(x.dtype) * (float(base) ** (-2.0 * i / dims))
        c, s = torch.cos(a).view(shape), torch.sin(a).view(shape)
        u, v = x[..., 2 * i], x[..., 2 * i + 1]
        out[..., 2 * i] = u * c - v * s
        out[..., 2 * i + 1] = v * c + u * s
    return out


# --------------------------------------------------------------------------
# latent attention
# --------------------------------------------------------------------------
def latent_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: dict, eps: float,
                 positions: Optional[torch.Tensor] = None) -> torch.Tensor:
    T = h.shape[0]
    H, dim, rot, vdim = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
    rank = w[p + "dkv.norm"].shape[0]  # the latent's size (config `kv_rank`, where it says it)
    pos = torch.arange(T) if positions is None else positions
    rdims, base = m["rot"]["dims"], m["rot"]["base"]
    cq = rms_norm(h @ w[p + "dq"].T, w[p + "dq.norm"], eps)
    q = (cq @ w[p + "uq"].T).view(T, H, dim + rot)
    q_plain, q_rot = q[..., :dim], rotate_neighbours(q[..., dim:], pos, rdims, base)
    down = h @ w[p + "dkv"].T
    c = rms_norm(down[:, :rank], w[p + "dkv.norm"], eps)
    k_rot = rotate_neighbours(down[:, rank:], pos, rdims, base)  # [T, rot], one for all heads
    k_plain = (c @ w[p + "uk"].T).view(T, H, dim)
    v = (c @ w[p + "uv"].T).view(T, H, vdim)
    gate = sigmoid(h @ w[p + "g"].T)  # [T, H]
    seen = torch.tril(torch.ones(T, T, dtype=torch.bool))
    heads = []
    for a in range(H):
        s = (q_plain[:, a] @ k_plain[:, a].T + q_rot[:, a] @ k_rot.T) * m["scale"]
        s = s.masked_fill(~seen, -math.inf)
        prob = torch.softmax(s, dim=-1)
        heads.append((prob @ v[:, a]) * gate[:, a : a + 1])
    return torch.cat(heads, dim=-1) @ w[p + "o"].T


# --------------------------------------------------------------------------
# windowed attention with one more place in the softmax's sum
# --------------------------------------------------------------------------
def sink_softmax(scores: torch.Tensor, seen: torch.Tensor) -> torch.Tensor:
    """p_j = exp(s_j) / (1 + sum over seen j of exp(s_j))."""
    s = scores.masked_fill(~seen, -math.inf)
    top = torch.clamp(s.max(dim=-1, keepdim=True).values, min=0.0)
    e = torch.exp(s - top)
    return e / (torch.exp(-top) + e.sum(dim=-1, keepdim=True))


def window_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: dict, eps: float) -> torch.Tensor:
    T = h.shape[0]
    H, G, dim, vdim = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rms_unit((h @ w[p + "q"].T + w[p + "q.b"]).view(T, H, dim), eps)
    k = rms_unit((h @ w[p + "k"].T + w[p + "k.b"]).view(T, G, dim), eps)
    v = (h @ w[p + "v"].T + w[p + "v.b"]).view(T, G, vdim)
    i = torch.arange(T)
    back = i[:, None] - i[None, :]
    seen = back >= 0
    size = (m.get("mask") or {}).get("size")
    if size is not None:
        seen = seen & (back < size)
    heads = []
    for a in range(H):
        g = a // (H // G)
        prob = sink_softmax((q[:, a] @ k[:, g].T) * m["scale"], seen)
        heads.append(prob @ v[:, g])
    return torch.cat(heads, dim=-1) @ w[p + "o"].T


# --------------------------------------------------------------------------
# gated delta rule
# --------------------------------------------------------------------------
def short_conv(u: torch.Tensor, taps: torch.Tensor) -> torch.Tensor:
    """Per channel over time: y[t, c] = sum_j taps[c, j] u[t - (J - 1) + j, c]; rows before 0 are zeros."""
    T, J = u.shape[0], taps.shape[1]
    padded = torch.cat([torch.zeros((J - 1, u.shape[1]), dtype=u.dtype), u])
    y = torch.zeros_like(u)
    for j in range(J):
        y = y + padded[j : j + T] * taps[:, j]
    return y


def unit_vector(x: torch.Tensor) -> torch.Tensor:
    return x / torch.sqrt((x * x).sum(dim=-1, keepdim=True) + 1e-6)


def delta_walk(q, k, v, beta, g, state=None):
    """One head.  q, k [T, d]; v [T, e]; beta, g [T]; the state S [d, e] starts at zero.
        S <- g_t S;  u = beta_t (v_t - S^T k_t);  S <- S + k_t u^T;  o_t = S^T q_t."""
    T, d = q.shape
    S = torch.zeros((d, v.shape[1]), dtype=q.dtype) if state is None else state.clone()
    out = []
    for t in range(T):
        S = g[t] * S
        u = beta[t] * (v[t] - S.T @ k[t])
        S = S + torch.outer(k[t], u)
        out.append(S.T @ q[t])
    return torch.stack(out), S


def delta_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: dict, eps: float) -> torch.Tensor:
    T = h.shape[0]
    H, G, dim, vdim = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(short_conv(h @ w[p + "q"].T, w[p + "q.conv"])).view(T, G, dim)
    k = silu(short_conv(h @ w[p + "k"].T, w[p + "k.conv"])).view(T, G, dim)
    v = silu(short_conv(h @ w[p + "v"].T, w[p + "v.conv"])).view(T, H, vdim)
    q = unit_vector(q) * dim ** -0.5
    k = unit_vector(k)
    beta = sigmoid(h @ w[p + "b"].T)  # [T, H]
    g = torch.exp(-torch.exp(w[p + "A_log"]) * softplus(h @ w[p + "a"].T + w[p + "dt_bias"]))  # [T, H]
    gate = silu(h @ w[p + "g"].T).view(T, H, vdim)
    heads = []
    for a in range(H):
        j = a // (H // G)
        o, _ = delta_walk(q[:, j], k[:, j], v[:, a], beta[:, a], g[:, a])
        heads.append(rms_unit(o, eps) * w[p + "norm"] * gate[:, a])
    return torch.cat(heads, dim=-1) @ w[p + "o"].T


# --------------------------------------------------------------------------
# feed-forwards
# --------------------------------------------------------------------------
def dense_ff(h, w, p: str) -> torch.Tensor:
    return (gelu_tanh(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def clamped_expert(x, w, p: str, limit: float) -> torch.Tensor:
    g = torch.clamp(x @ w[p + "gate"].T, max=limit)
    u = torch.clamp(x @ w[p + "up"].T, min=-limit, max=limit)
    return (g * sigmoid(1.702 * g) * (u + 1.0)) @ w[p + "down"].T


def router_choice(z: torch.Tensor, top: int, groups: int, keep: int):
    """z [E] router logits -> (chosen expert ids, their weights).  Scores are sigmoids; a group of
    neighbours is worth the sum of its two largest scores; the choice is among the `keep` best groups."""
    s = sigmoid(z)
    E = s.shape[0]
    per = E // groups
    worth = torch.stack([torch.topk(s[a * per : (a + 1) * per], min(2, per)).values.sum() for a in range(groups)])
    kept = torch.topk(worth, keep).indices.tolist()
    allowed = torch.full((E,), -math.inf, dtype=s.dtype)
    for a in kept:
        allowed[a * per : (a + 1) * per] = s[a * per : (a + 1) * per]
    ids = torch.topk(allowed, top).indices
    return ids, s[ids] / (s[ids].sum() + 1e-20)


def routed_ff(h, w, p: str, f: dict) -> torch.Tensor:
    r = f["router"]
    groups = r.get("groups") or {}
    count = groups.get("count", 1)
    keep = groups.get("keep", count)
    z = h @ w[p + "router"].T
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        ids, weights = router_choice(z[t], r["top"], count, keep)
        for e, a in zip(ids.tolist(), weights):
            out[t] = out[t] + a * clamped_expert(h[t : t + 1], w, f"{p}e{e}.", f["expert"]["limit"])[0]
    return out


def feed_forward(h, w, p: str, f: dict) -> torch.Tensor:
    return dense_ff(h, w, p) if f["kind"] == "dense" else routed_ff(h, w, p, f)


# --------------------------------------------------------------------------
# the model
# --------------------------------------------------------------------------
MIXERS = {"latent_attention": latent_mixer, "attention": window_mixer, "delta": delta_mixer}


def forward(cfg: dict, w: Dict[str, torch.Tensor], tokens: Sequence[int],
            layers_out: Optional[List[torch.Tensor]] = None) -> torch.Tensor:
    """Logits [T, vocab] of one sequence; with `layers_out`, the residual stream after every layer is appended."""
    eps = cfg["norm"]["eps"]
    x = w["embed"][torch.as_tensor(list(tokens), dtype=torch.long)] * cfg["embedding"]["scale"]
    for i, spec in enumerate(cfg["layers"]):
        p = f"l{i}."
        x = x + MIXERS[spec["type"]](rms_norm(x, w[p + "norm1"], eps), w, p + "mix.", spec["mixer"], eps)
        if spec.get("mlp") is not None:
            x = x + feed_forward(rms_norm(x, w[p + "norm2"], eps), w, p + "mlp.", spec["mlp"])
        if layers_out is not None:
            layers_out.append(x.clone())
    return rms_norm(x, w["final.norm"], eps) @ w["embed"].T


def router_margins(cfg: dict, w: Dict[str, torch.Tensor], tokens: Sequence[int]) -> torch.Tensor:
    """For every token the smallest gap, over the routed layers, between the last chosen expert's score and the
    best score left out among the experts that could have been chosen, and between the last kept group and the
    best group left out: where it is tiny, rounding may choose otherwise."""
    eps = cfg["norm"]["eps"]
    T = len(tokens)
    margin = torch.full((T,), math.inf, dtype=torch.float64)
    x = w["embed"][torch.as_tensor(list(tokens), dtype=torch.long)] * cfg["embedding"]["scale"]
    for i, spec in enumerate(cfg["layers"]):
        p = f"l{i}."
        x = x + MIXERS[spec["type"]](rms_norm(x, w[p + "norm1"], eps), w, p + "mix.", spec["mixer"], eps)
        f = spec.get("mlp")
        if f is None:
            continue
        h = rms_norm(x, w[p + "norm2"], eps)
        if f["kind"] == "moe":
            r = f["router"]
            groups = r.get("groups") or {}
            count = groups.get("count", 1)
            keep = groups.get("keep", count)
            s = sigmoid(h @ w[p + "mlp.router"].T).double()
            per = s.shape[1] // count
            for t in range(T):
                worth = torch.stack([torch.topk(s[t, a * per : (a + 1) * per], min(2, per)).values.sum()
                                     for a in range(count)])
                order = torch.sort(worth, descending=True).values
                if keep < count:
                    margin[t] = min(margin[t], float(order[keep - 1] - order[keep]))
                kept = torch.topk(worth, keep).indices.tolist()
                inside = torch.sort(torch.cat([s[t, a * per : (a + 1) * per] for a in kept]), descending=True).values
                if r["top"] < inside.shape[0]:
                    margin[t] = min(margin[t], float(inside[r["top"] - 1] - inside[r["top"]]))
        x = x + feed_forward(h, w, p + "mlp.", f)
    return margin


def load(model_dir: str, dtype=torch.float64):
    from safetensors.torch import load_file

    with open(os.path.join(model_dir, "config.json")) as f:
        cfg = json.load(f)
    w = {k: v.to(dtype) for k, v in load_file(os.path.join(model_dir, "model.safetensors")).items()}
    return cfg, w


def greedy(cfg, w, prompt: Sequence[int], new_tokens: int) -> List[int]:
    ids = list(prompt)
    for _ in range(new_tokens):
        ids.append(int(torch.argmax(forward(cfg, w, ids)[-1])))
    return ids[len(prompt):]
