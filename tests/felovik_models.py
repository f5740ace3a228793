"""Small Felovik configurations and random weights for the tests.

The weights are drawn here and not by the library's own initialiser, with spreads that keep
activations of order one and make every mechanism count: attention scales well above 1/sqrt(dim) so
that single keys stand out, decays between a few percent and almost one, step sizes around a half,
norm weights clearly away from one, router matrices that spread the tokens over the experts.
"""
from __future__ import annotations

import json
import os
from typing import Dict

import torch


def left(heads, kv_heads, dim, vdim, scale, q_temp=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if q_temp is not None:
        m["q_temp"] = {"coef": q_temp[0], "every": q_temp[1]}
    return m


def right(heads, vdim, state, groups, conv, norm_groups):
    return {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv, "norm_groups": norm_groups}


def dense(ff, limit):
    return {"kind": "dense", "ff": ff, "limit": limit}


def moe(experts, ff, top, groups=None):
    router = {"experts": experts, "top": top}
    if groups is not None:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    return {"kind": "moe", "expert": {"ff": ff}, "router": router}


def layer(l, r, mlp):
    return {"type": "parallel", "mixer": {"left": l, "right": r}, "mlp": mlp}


def config(vocab, width, layers, alpha, scale, eps=1e-5, max_positions=1024) -> Dict:
    return {"architecture": "Felovik", "vocab": vocab, "width": width, "max_positions": max_positions, "norm": {"eps": eps},
            "embedding": {"scale": scale}, "postln_alpha": alpha, "layers": layers}


# A: every size differs from its neighbours and none is a multiple of 8 where it need not be: value heads
# narrower and wider than key heads, query stretches that change every 16 and every 5 positions and a
# layer without one, convolutions of 4, 2 and 3 taps, one group and several, a layer without a
# feed-forward, experts with and without groups, one chosen expert and several.
CFG_A = config(211, 72, [
    layer(left(4, 2, 24, 16, 0.9, (0.7, 16)), right(4, 12, 20, 2, 4, 2), dense(80, 0.8)),
    layer(left(3, 3, 16, 40, 1.1), right(2, 24, 33, 1, 2, 1), moe(6, 24, 2, (3, 2))),
    layer(left(6, 1, 12, 12, 1.3, (1.5, 5)), right(3, 20, 17, 3, 3, 4), None),
    layer(left(2, 1, 40, 24, 0.6, (0.25, 64)), right(6, 8, 48, 2, 4, 3), moe(5, 40, 1)),
], alpha=2.0, scale=5.0, eps=3e-6)

# B: sizes the matrix-core kernels know: key heads of 64 and 128 with value heads of the same size, widths
# that are multiples of 8 (the experts' products then run on the matrix cores in bfloat16), states of 64
# and 128, more experts, a stretch that changes every 64 positions (inside the prompts).  Its attention
# scales are twice 1/sqrt(dim), not eight times: it is the model that bfloat16 runs are judged on.
CFG_B = config(300, 128, [
    layer(left(4, 1, 64, 64, 0.25, (0.45, 64)), right(4, 32, 64, 2, 4, 2), dense(224, 1.25)),
    layer(left(2, 2, 128, 128, 0.18, (0.4, 100)), right(2, 64, 128, 1, 4, 1), moe(8, 64, 3, (4, 2))),
    layer(left(4, 2, 64, 64, 0.3), right(8, 16, 16, 4, 3, 8), moe(16, 32, 4, (4, 3))),
    layer(left(8, 4, 32, 32, 0.35, (1.0, 7)), right(4, 32, 40, 4, 2, 4), dense(192, 4.0)),
], alpha=2.5, scale=9.0)

# C: the values that make mechanisms vanish or coincide: one head everywhere, a convolution of one tap (no
# inputs are kept), a state of one number, every expert chosen, all groups kept, a residual scale and an
# embedding scale of one, a stretch that grows with every position.
CFG_C = config(131, 36, [
    layer(left(1, 1, 10, 10, 1.0, (1.0, 1)), right(1, 12, 1, 1, 1, 1), moe(2, 20, 2, (1, 1))),
    layer(left(2, 2, 12, 6, 0.8), right(2, 6, 9, 2, 2, 12), dense(28, 100.0)),
    layer(left(1, 1, 20, 20, 0.5, (0.1, 1000)), right(4, 4, 5, 1, 8, 2), moe(3, 12, 3)),
], alpha=1.0, scale=1.0, eps=1e-3, max_positions=400)

CONFIGS = {"A": (CFG_A, 21), "B": (CFG_B, 22), "C": (CFG_C, 23)}


def tensor_shapes(cfg: Dict) -> Dict[str, tuple]:
    w = cfg["width"]
    shapes = {"embed": (cfg["vocab"], w), "pos": (cfg["max_positions"], w), "final.norm": (w,), "head": (cfg["vocab"], w)}
    for i, lay in enumerate(cfg["layers"]):
        l, r, p = lay["mixer"]["left"], lay["mixer"]["right"], f"l{i}."
        H, G, d, dv = l["heads"], l["kv_heads"], l["dim"], l["vdim"]
        inner, bc = r["heads"] * r["vdim"], r["groups"] * r["state"]
        shapes.update({p + "norm1": (w,), p + "mix.left.q": (H * d, w), p + "mix.left.k": (G * d, w), p + "mix.left.v": (G * dv, w),
                       p + "mix.left.g": (H * dv, w), p + "mix.left.o": (w, H * dv), p + "mix.left.out": (w,),
                       p + "mix.right.in": (2 * inner + 2 * bc + r["heads"], w), p + "mix.right.conv": (inner + 2 * bc, r["conv"]),
                       p + "mix.right.conv.b": (inner + 2 * bc,), p + "mix.right.dt_bias": (r["heads"],),
                       p + "mix.right.A_log": (r["heads"],), p + "mix.right.D": (r["heads"],), p + "mix.right.norm": (inner,),
                       p + "mix.right.o": (w, inner), p + "mix.right.out": (w,)})
        mlp = lay.get("mlp")
        if mlp is None:
            continue
        shapes[p + "norm2"] = (w,)
        if mlp["kind"] == "dense":
            shapes.update({p + "mlp.gate": (mlp["ff"], w), p + "mlp.up": (mlp["ff"], w), p + "mlp.down": (w, mlp["ff"])})
        else:
            ff = mlp["expert"]["ff"]
            shapes[p + "mlp.router"] = (mlp["router"]["experts"], w)
            for e in range(mlp["router"]["experts"]):
                shapes.update({p + f"mlp.e{e}.gate": (ff, w), p + f"mlp.e{e}.up": (ff, w), p + f"mlp.e{e}.down": (w, ff)})
    return shapes


def random_tensors(cfg: Dict, seed: int) -> Dict[str, torch.Tensor]:
    """Values that bfloat16 holds exactly (so both compute types read the same weights)."""
    gen = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        def n(std=1.0, mean=0.0):
            return mean + std * torch.randn(shape, generator=gen)
        if name.endswith(("norm1", "norm2", ".norm", ".out")):
            t = n(0.3, 1.0)
        elif name == "embed":
            t = n(1.0)
        elif name == "pos":
            t = n(1.0 * cfg["embedding"]["scale"] * 0.5)
        elif name.endswith("conv"):
            t = n(0.6)
        elif name.endswith("conv.b"):
            t = n(0.3)
        elif name.endswith("dt_bias"):
            t = n(1.0, -0.5)
        elif name.endswith("A_log"):
            t = n(0.8, -0.5)
        elif name.endswith(".D"):
            t = n(0.4, 1.0)
        elif name.endswith("router"):
            t = n(3.0 / shape[-1] ** 0.5)
        else:
            t = n(1.5 / shape[-1] ** 0.5)
        out[name] = t.to(torch.bfloat16).to(torch.float32)
    return out


def write_model(path: str, cfg: Dict, tensors: Dict[str, torch.Tensor], dtype=torch.bfloat16) -> str:
    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.to(dtype).contiguous() for k, v in tensors.items()}, os.path.join(path, "model.safetensors"))
    return path


def as_double(tensors: Dict[str, torch.Tensor]) -> Dict[str, torch.Tensor]:
    return {k: v.double() for k, v in tensors.items()}
