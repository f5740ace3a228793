"""A plain, slow Felovik decoder in torch on the CPU, one function per mechanism.

It is the oracle of the tests: written from the design's equations, sharing no code with the
library (it reads the configuration dictionary and the checkpoint's tensor names directly, and
keeps no cache: every call runs whole sequences, the recurrence token by token).

Notation: ``h`` a sublayer's input ``[T, width]``, positions ``0 .. T-1``, ``W x`` for a matrix
stored ``[out, in]``.  The arithmetic type is the type of the tensors handed in (the tests use
64-bit floats so that the oracle's own rounding does not count).
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional, Sequence

import torch


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def norm(x, w, eps):
    return rms(x, eps) * w


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.log1p(torch.exp(-z.abs())) + torch.clamp(z, min=0.0)


def embed(t: Dict[str, torch.Tensor], tokens: Sequence[int], scale: float, first: int = 0) -> torch.Tensor:
    """A token's row times ``scale`` plus the learned row of its position (not scaled)."""
    ids = torch.tensor(list(tokens), dtype=torch.long)
    pos = torch.arange(first, first + len(ids))
    return t["embed"][ids] * scale + t["pos"][pos]


def query_temperature(positions: torch.Tensor, coef: float, every: int) -> torch.Tensor:
    """1 + coef * ln(floor((p + 1) / every) + 1)."""
    steps = torch.div(positions + 1, every, rounding_mode="floor")
    return 1.0 + coef * torch.log(steps.to(torch.float64) + 1.0)


def gated_attention(h: torch.Tensor, t: Dict[str, torch.Tensor], pre: str, m: Dict, eps: float) -> torch.Tensor:
    """Causal softmax attention with grouped key/value heads and no rotation: queries and keys
    are divided by their root mean square per head, the query is stretched with its position,
    and the heads are gated by a sigmoid of a projection of ``h`` before the output matrix."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ t[pre + "q"].T).reshape(T, H, d)
    k = (h @ t[pre + "k"].T).reshape(T, G, d)
    v = (h @ t[pre + "v"].T).reshape(T, G, dv)
    q, k = rms(q, eps), rms(k, eps)
    if m.get("q_temp") is not None:
        temp = query_temperature(torch.arange(T), m["q_temp"]["coef"], m["q_temp"]["every"]).to(h.dtype)
        q = q * temp[:, None, None]
    out = torch.zeros(T, H, dv, dtype=h.dtype)
    visible = torch.arange(T)[None, :] <= torch.arange(T)[:, None]
    for a in range(H):
        g = a // (H // G)
        s = (q[:, a] @ k[:, g].T) * m["scale"]
        s = s.masked_fill(~visible, float("-inf"))
        p = torch.softmax(s, dim=-1)
        out[:, a] = p @ v[:, g]
    gate = torch.sigmoid(h @ t[pre + "g"].T)
    return (out.reshape(T, H * dv) * gate) @ t[pre + "o"].T


def causal_conv(u: torch.Tensor, w: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """Per channel: ``out[t] = b + sum_j w[:, j] * u[t - (taps - 1) + j]``, zeros before the
    start; the last column of ``w`` multiplies the current token."""
    T, taps = u.shape[0], w.shape[1]
    padded = torch.cat([torch.zeros(taps - 1, u.shape[1], dtype=u.dtype), u], dim=0)
    out = b[None, :].expand(T, -1).clone()
    for j in range(taps):
        out = out + padded[j:j + T] * w[:, j][None, :]
    return out


def state_space(h: torch.Tensor, t: Dict[str, torch.Tensor], pre: str, m: Dict, eps: float) -> torch.Tensor:
    """The recurrence with a scalar decay per head: ``S <- exp(-exp(A_log) dt) S + dt B x^T``,
    ``y = S^T C + D x``; inputs through a short causal convolution and silu; the output gated by
    silu(z), normed in equal parts, and projected."""
    T = h.shape[0]
    Hs, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = Hs * P
    proj = h @ t[pre + "in"].T
    z, xbc, dt = proj[:, :inner], proj[:, inner:2 * inner + 2 * G * N], proj[:, 2 * inner + 2 * G * N:]
    xbc = silu(causal_conv(xbc, t[pre + "conv"], t[pre + "conv.b"]))
    x = xbc[:, :inner].reshape(T, Hs, P)
    B = xbc[:, inner:inner + G * N].reshape(T, G, N)
    C = xbc[:, inner + G * N:].reshape(T, G, N)
    dt = softplus(dt + t[pre + "dt_bias"])
    decay = torch.exp(-torch.exp(t[pre + "A_log"])[None, :] * dt)        # [T, Hs]
    y = torch.zeros(T, Hs, P, dtype=h.dtype)
    for a in range(Hs):
        g = a // (Hs // G)
        S = torch.zeros(N, P, dtype=h.dtype)
        for r in range(T):
            S = decay[r, a] * S + dt[r, a] * torch.outer(B[r, g], x[r, a])
            y[r, a] = S.T @ C[r, g] + t[pre + "D"][a] * x[r, a]
    y = y.reshape(T, inner) * silu(z)
    parts = m["norm_groups"]
    y = rms(y.reshape(T, parts, inner // parts), eps).reshape(T, inner) * t[pre + "norm"]
    return y @ t[pre + "o"].T


def parallel_mixer(h: torch.Tensor, t: Dict[str, torch.Tensor], pre: str, m: Dict, eps: float) -> torch.Tensor:
    """Half the sum of the two mixers' outputs, each normed over the width with a weight of its own."""
    left = gated_attention(h, t, pre + "left.", m["left"], eps)
    right = state_space(h, t, pre + "right.", m["right"], eps)
    return 0.5 * (norm(left, t[pre + "left.out"], eps) + norm(right, t[pre + "right.out"], eps))


def dense_ff(h: torch.Tensor, t: Dict[str, torch.Tensor], pre: str, m: Dict) -> torch.Tensor:
    """``g = min(W_gate h, limit)``, ``u = clamp(W_up h, -limit, limit)``,
    ``W_down (g sigmoid(1.702 g) (u + 1))``."""
    limit = m["limit"]
    g = torch.clamp(h @ t[pre + "gate"].T, max=limit)
    u = torch.clamp(h @ t[pre + "up"].T, min=-limit, max=limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ t[pre + "down"].T


def route(h: torch.Tensor, w_router: torch.Tensor, r: Dict):
    """Softmax over all experts; only experts of the ``keep`` best groups (a group's score is its
    largest) can be chosen; the ``top`` best of those, their scores divided by their sum."""
    s = torch.softmax(h @ w_router.T, dim=-1)
    T, E = s.shape
    allowed = torch.ones(T, E, dtype=torch.bool)
    groups = r.get("groups")
    if groups is not None:
        per = E // groups["count"]
        best = s.reshape(T, groups["count"], per).max(dim=-1).values
        kept = torch.topk(best, groups["keep"], dim=-1).indices
        allowed = torch.zeros(T, groups["count"], dtype=torch.bool)
        allowed.scatter_(1, kept, True)
        allowed = allowed[:, :, None].expand(T, groups["count"], per).reshape(T, E)
    chosen = torch.topk(s.masked_fill(~allowed, -1.0), r["top"], dim=-1).indices
    picked = torch.gather(s, 1, chosen)
    return chosen, picked / (picked.sum(dim=-1, keepdim=True) + 1e-20)


def expert_ff(h, t, pre):
    return (silu(h @ t[pre + "gate"].T) * (h @ t[pre + "up"].T)) @ t[pre + "down"].T


def routed_ff(h: torch.Tensor, t: Dict[str, torch.Tensor], pre: str, m: Dict) -> torch.Tensor:
    chosen, weight = route(h, t[pre + "router"], m["router"])
    out = torch.zeros_like(h)
    for r in range(h.shape[0]):
        for e, w in zip(chosen[r].tolist(), weight[r]):
            out[r] = out[r] + w * expert_ff(h[r:r + 1], t, f"{pre}e{e}.")[0]
    return out


def layer(x: torch.Tensor, t: Dict[str, torch.Tensor], i: int, spec: Dict, alpha: float, eps: float) -> torch.Tensor:
    """Each sublayer is fed the residual stream as it is, and the norm is applied to the scaled sum:
    ``x <- norm1(alpha x + mixer(x))``, ``x <- norm2(alpha x + ff(x))``."""
    pre = f"l{i}."
    if spec["type"] != "parallel":
        raise ValueError(f"unknown layer type {spec['type']!r}")
    x = norm(alpha * x + parallel_mixer(x, t, pre + "mix.", spec["mixer"], eps), t[pre + "norm1"], eps)
    mlp = spec.get("mlp")
    if mlp is None:
        return x
    if mlp["kind"] == "dense":
        y = dense_ff(x, t, pre + "mlp.", mlp)
    elif mlp["kind"] == "moe":
        y = routed_ff(x, t, pre + "mlp.", mlp)
    else:
        raise ValueError(f"unknown feed-forward kind {mlp['kind']!r}")
    return norm(alpha * x + y, t[pre + "norm2"], eps)


def forward(cfg: Dict, t: Dict[str, torch.Tensor], tokens: Sequence[int], streams: Optional[List] = None) -> torch.Tensor:
    """Logits at every position ``[T, vocab]``; with ``streams`` a list, the residual stream
    after every layer is appended to it."""
    eps = cfg["norm"]["eps"]
    x = embed(t, tokens, cfg["embedding"]["scale"])
    for i, spec in enumerate(cfg["layers"]):
        x = layer(x, t, i, spec, cfg["postln_alpha"], eps)
        if streams is not None:
            streams.append(x)
    return norm(x, t["final.norm"], eps) @ t["head"].T


def greedy(cfg: Dict, t: Dict[str, torch.Tensor], prompt: Sequence[int], n_new: int) -> List[int]:
    ids, out = list(prompt), []
    for _ in range(n_new):
        nxt = int(torch.argmax(forward(cfg, t, ids)[-1]))
        out.append(nxt)
        ids.append(nxt)
    return out
