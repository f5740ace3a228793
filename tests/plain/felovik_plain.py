"""A plain, slow Felovik decoder in torch on the CPU, one function per mechanism.

It is the oracle of the tests: written from the design's equations, sharing no code with the
library (it reads the configuration dictionary and the checkpoint's tensor names directly, and
keeps no cache: every call runs whole sequences, the recurrence token by token).

Notation: ``h`` a sublayer's input ``[T, width]``, positions ``0 .. T-1``, ``W x`` for a matrix
stored ``[out, in]``.  The arithmetic type is the type of the tensors handed in (the tests use
64-bit floats so that the oracle's own rounding does not count).
"""
from __future__ import annotations

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


def attend(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float) -> torch.Tensor:
    """Causal softmax attention of one sequence: ``q [T, H, d]``, ``k [T, G, d]``, ``v [T, G, dv]``; query
    head ``a`` uses key/value head ``a // (H / G)``; position ``i`` sees every ``j <= i``."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[2], dtype=q.dtype)
    visible = torch.arange(T)[None, :] <= torch.arange(T)[:, None]
    for a in range(H):
        g = a // (H // G)
        s = (q[:, a] @ k[:, g].T) * scale
        s = s.masked_fill(~visible, float("-inf"))
        out[:, a] = torch.softmax(s, dim=-1) @ v[:, g]
    return out


def gated_attention(h: torch.Tensor, t: Dict[str, torch.Tensor], pre: str, m: Dict, eps: float) -> torch.Tensor:
    """Attention without rotation: queries and keys are divided by their root mean square per head,
    the query is stretched with its position, and the heads are gated by a sigmoid of a projection
    of ``h`` before the output matrix."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ t[pre + "q"].T).reshape(T, H, d)
    k = (h @ t[pre + "k"].T).reshape(T, G, d)
    v = (h @ t[pre + "v"].T).reshape(T, G, dv)
    q, k = rms(q, eps), rms(k, eps)
    if m.get("q_temp") is not None:
        temp = query_temperature(torch.arange(T), m["q_temp"]["coef"], m["q_temp"]["every"]).to(h.dtype)
        q = q * temp[:, None, None]
    out = attend(q, k, v, m["scale"])
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


def recurrence(x: torch.Tensor, B: torch.Tensor, C: torch.Tensor, dt_raw: torch.Tensor, dt_bias: torch.Tensor,
               a_log: torch.Tensor, d_skip: torch.Tensor) -> torch.Tensor:
    """``x [T, H, P]``, ``B`` and ``C [T, G, N]``, ``dt_raw [T, H]``.  Per head ``a`` (group
    ``a // (H / G)``): ``dt = softplus(dt_raw + dt_bias)``, ``S <- exp(-exp(A_log) dt) S + dt B x^T``
    (``S`` is ``N x P``, zero at the start), ``y = S^T C + D x``."""
    T, Hs, P = x.shape
    G, N = B.shape[1], B.shape[2]
    dt = softplus(dt_raw + dt_bias)
    decay = torch.exp(-torch.exp(a_log)[None, :] * dt)        # [T, H]
    y = torch.zeros(T, Hs, P, dtype=x.dtype)
    for a in range(Hs):
        g = a // (Hs // G)
        S = torch.zeros(N, P, dtype=x.dtype)
        for r in range(T):
            S = decay[r, a] * S + dt[r, a] * torch.outer(B[r, g], x[r, a])
            y[r, a] = S.T @ C[r, g] + d_skip[a] * x[r, a]
    return y


def gated_part_norm(y: torch.Tensor, z: torch.Tensor, w: torch.Tensor, parts: int, eps: float) -> torch.Tensor:
    """``y * silu(z)`` first, then every one of the ``parts`` equal parts of a row divided by its own root
    mean square, times ``w``."""
    T, n = y.shape
    v = y * silu(z)
    return rms(v.reshape(T, parts, n // parts), eps).reshape(T, n) * w


def state_space(h: torch.Tensor, t: Dict[str, torch.Tensor], pre: str, m: Dict, eps: float) -> torch.Tensor:
    """The input projection gives ``[z | x | B | C | dt]``; x, B and C pass the short causal convolution
    and silu, then the recurrence; its output is gated by z, normed in parts and projected."""
    T = h.shape[0]
    Hs, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = Hs * P
    proj = h @ t[pre + "in"].T
    z, xbc, dt = proj[:, :inner], proj[:, inner:2 * inner + 2 * G * N], proj[:, 2 * inner + 2 * G * N:]
    xbc = silu(causal_conv(xbc, t[pre + "conv"], t[pre + "conv.b"]))
    y = recurrence(xbc[:, :inner].reshape(T, Hs, P), xbc[:, inner:inner + G * N].reshape(T, G, N),
                   xbc[:, inner + G * N:].reshape(T, G, N), dt, t[pre + "dt_bias"], t[pre + "A_log"], t[pre + "D"])
    return gated_part_norm(y.reshape(T, inner), z, t[pre + "norm"], m["norm_groups"], eps) @ t[pre + "o"].T


def parallel_mixer(h: torch.Tensor, t: Dict[str, torch.Tensor], pre: str, m: Dict, eps: float) -> torch.Tensor:
    """Half the sum of the two mixers' outputs, each normed over the width with a weight of its own."""
    left = gated_attention(h, t, pre + "left.", m["left"], eps)
    right = state_space(h, t, pre + "right.", m["right"], eps)
    return 0.5 * (norm(left, t[pre + "left.out"], eps) + norm(right, t[pre + "right.out"], eps))


def limited_gate(g: torch.Tensor, u: torch.Tensor, limit: Optional[float]) -> torch.Tensor:
    """``g <- min(g, limit)``, ``u <- clamp(u, -limit, limit)``, then ``g sigmoid(1.702 g) (u + 1)``."""
    if limit is not None:
        g, u = torch.clamp(g, max=limit), torch.clamp(u, min=-limit, max=limit)
    return g * torch.sigmoid(1.702 * g) * (u + 1.0)


def dense_ff(h: torch.Tensor, t: Dict[str, torch.Tensor], pre: str, m: Dict) -> torch.Tensor:
    return limited_gate(h @ t[pre + "gate"].T, h @ t[pre + "up"].T, m.get("limit")) @ t[pre + "down"].T


def route(h: torch.Tensor, w_router: torch.Tensor, r: Dict):
    return choose(h @ w_router.T, r)


def choose(logits: torch.Tensor, r: Dict):
    """Softmax over all experts; only experts of the ``keep`` best groups (a group's score is its
    largest) can be chosen; the ``top`` best of those, their scores divided by their sum."""
    s = torch.softmax(logits, dim=-1)
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
