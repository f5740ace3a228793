"""A plain, slow Dokulix decoder in 32-bit torch on the CPU, one function per mechanism.

It is the oracle of the tests: written from the design's equations, sharing no code with the
library (it reads the configuration dictionary and the checkpoint's tensor names directly, and
keeps no cache: every call runs whole sequences).

Notation: ``h`` a mixer's input ``[T, width]``, positions ``0 .. T-1``, ``W x`` for a matrix
stored ``[out, in]``.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

F = torch.float32


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def norm_plain(x, w, eps):
    return rms(x, eps) * w


def norm_one_plus(x, w, eps):
    """The layers' and the model's norm: the stored weight lies around zero."""
    return rms(x, eps) * (1.0 + w)


def rotate_halves(x: torch.Tensor, positions: torch.Tensor, base: float, dims: Optional[int] = None) -> torch.Tensor:
    """Rotates the pairs ``(i, i + n/2)`` of the first ``n = dims`` numbers of the last axis of
    ``x [T, ..., width]`` by ``p * base^(-2i/n)``; the rest passes unchanged."""
    n = x.shape[-1] if dims is None else dims
    if n < x.shape[-1]:
        return torch.cat([rotate_halves(x[..., :n], positions, base), x[..., n:]], dim=-1)
    half = n // 2
    freq = torch.tensor([base ** (-2.0 * i / n) for i in range(half)], dtype=torch.float64)
    ang = positions.to(torch.float64)[:, None] * freq[None, :]
    cos, sin = torch.cos(ang).to(F), torch.sin(ang).to(F)
    while cos.dim() < x.dim():
        cos, sin = cos.unsqueeze(1), sin.unsqueeze(1)
    u, v = x[..., :half], x[..., half:]
    return torch.cat([u * cos - v * sin, v * cos + u * sin], dim=-1)


def window_mask(n: int, size: int) -> torch.Tensor:
    """visible[i, j]: 0 <= i - j < size."""
    i = torch.arange(n)[:, None]
    j = torch.arange(n)[None, :]
    return (i - j >= 0) & (i - j < size)


def chunk_mask(n: int, size: int) -> torch.Tensor:
    """visible[i, j]: j <= i and both in the same block of ``size`` positions counted from 0."""
    i = torch.arange(n)[:, None]
    j = torch.arange(n)[None, :]
    return (j <= i) & (i // size == j // size)


def softmax_visible(scores: torch.Tensor, visible: torch.Tensor, sink: bool) -> torch.Tensor:
    """Weights over the visible keys; with ``sink`` the denominator has one more term, exp(0)."""
    s = scores.masked_fill(~visible, float("-inf"))
    m = s.max(dim=-1, keepdim=True).values
    if sink:
        m = torch.clamp(m, min=0.0)
    e = torch.exp(s - m)
    den = e.sum(dim=-1, keepdim=True)
    if sink:
        den = den + torch.exp(-m)
    return e / den


def latent_attention(h: torch.Tensor, t: Dict[str, torch.Tensor], pre: str, m: Dict, eps: float) -> torch.Tensor:
    """Queries through a normed latent; keys and values expanded from one normed latent per
    position plus one rotated key part shared by the heads; sliding window; gated output."""
    T = h.shape[0]
    H, d, r, dv, kr = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    pos = torch.arange(T)
    cq = norm_plain(h @ t[pre + "dq"].T, t[pre + "dq.norm"], eps)
    q = (cq @ t[pre + "uq"].T).view(T, H, d + r)
    q_nope, q_rot = q[..., :d], rotate_halves(q[..., d:], pos, m["rot"]["base"], m["rot"]["dims"])
    dkv = h @ t[pre + "dkv"].T
    c = norm_plain(dkv[:, :kr], t[pre + "dkv.norm"], eps)
    k_rot = rotate_halves(dkv[:, kr:], pos, m["rot"]["base"], m["rot"]["dims"])          # [T, r], one for all heads
    k_nope = (c @ t[pre + "uk"].T).view(T, H, d)
    v = (c @ t[pre + "uv"].T).view(T, H, dv)
    scores = (torch.einsum("ihd,jhd->hij", q_nope, k_nope) + torch.einsum("ihd,jd->hij", q_rot, k_rot)) * m["scale"]
    p = softmax_visible(scores, window_mask(T, m["mask"]["size"])[None], sink=False)
    o = torch.einsum("hij,jhd->ihd", p, v).reshape(T, H * dv)
    o = o * torch.sigmoid(h @ t[pre + "g"].T)
    return o @ t[pre + "o"].T


def biased_attention(h: torch.Tensor, t: Dict[str, torch.Tensor], pre: str, m: Dict, eps: float) -> torch.Tensor:
    """Grouped heads with biased projections, per-head norm of q and k, no rotation, a distance
    penalty per head, blocks of positions as the mask and a sink in the softmax."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ t[pre + "q"].T + t[pre + "q.b"]).view(T, H, d)
    k = (h @ t[pre + "k"].T + t[pre + "k.b"]).view(T, G, d)
    v = (h @ t[pre + "v"].T + t[pre + "v.b"]).view(T, G, dv)
    q = norm_plain(q, t[pre + "q.norm"], eps)
    k = norm_plain(k, t[pre + "k.norm"], eps)
    rep = H // G
    k = k.repeat_interleave(rep, dim=1)
    v = v.repeat_interleave(rep, dim=1)
    scores = torch.einsum("ihd,jhd->hij", q, k) * m["scale"]
    slopes = torch.tensor([2.0 ** (-8.0 * (x + 1) / H) for x in range(H)], dtype=F)
    dist = (torch.arange(T)[:, None] - torch.arange(T)[None, :]).to(F)
    scores = scores - slopes[:, None, None] * dist[None]
    p = softmax_visible(scores, chunk_mask(T, m["mask"]["size"])[None], sink=True)
    o = torch.einsum("hij,jhd->ihd", p, v).reshape(T, H * dv)
    return o @ t[pre + "o"].T + t[pre + "o.b"]


def gated_relu_ff(h, t, pre):
    return (torch.relu(h @ t[pre + "gate"].T) * (h @ t[pre + "up"].T)) @ t[pre + "down"].T


MIXERS = {"latent_attention": latent_attention, "attention": biased_attention}


def layer_order(cfg: Dict) -> List[tuple]:
    """``(layer, pass number or None)`` in the order the layers run; the pass number is set on
    the first layer of each pass of the loop."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, None) for i in range(n)]
    start, stop, times = loop["start"], loop["stop"], loop["times"]
    order = [(i, None) for i in range(start)]
    for p in range(times):
        order += [(i, p if i == start else None) for i in range(start, stop)]
    order += [(i, None) for i in range(stop, n)]
    return order


def forward(cfg: Dict, tensors: Dict[str, torch.Tensor], tokens, return_layers: bool = False):
    """Logits ``[T, vocab]`` of one sequence (and the residual stream after every layer run)."""
    t = {k: v.to(F) for k, v in tensors.items() if v.dtype != torch.int32}
    eps = cfg["norm"]["eps"]
    x = t["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    seen = []
    for i, loop_pass in layer_order(cfg):
        layer = cfg["layers"][i]
        if loop_pass is not None:
            x = x + t["loop.step"][loop_pass]
        pre = f"l{i}."
        x = x + MIXERS[layer["type"]](norm_one_plus(x, t[pre + "norm1"], eps), t, pre + "mix.", layer["mixer"], eps)
        if layer.get("mlp") is not None:
            x = x + gated_relu_ff(norm_one_plus(x, t[pre + "norm2"], eps), t, pre + "mlp.")
        seen.append(x)
    logits = norm_one_plus(x, t["final.norm"], eps) @ t["head"].T
    if return_layers:
        return logits, torch.stack(seen)
    return logits


def greedy(cfg: Dict, tensors: Dict[str, torch.Tensor], prompt, n_new: int, stop=()) -> List[int]:
    """Greedy continuation, every step a whole forward pass; a stop token ends it and is not kept."""
    tokens, out = list(prompt), []
    for _ in range(n_new):
        nxt = int(torch.argmax(forward(cfg, tensors, tokens)[-1]))
        if nxt in stop:
            break
        out.append(nxt)
        tokens.append(nxt)
    return out
