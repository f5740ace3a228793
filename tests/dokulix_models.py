"""Small Dokulix configurations and random weights for the tests.

The weights are drawn here and not by the library's own initialiser, with spreads that keep
activations of order one: attention scores then differ between keys, a key more or less inside a
window changes the logits far beyond rounding, and norm weights stored around zero differ clearly
from plain ones.
"""
from __future__ import annotations

import json
import os
from typing import Dict

import torch


def latent(heads, dim, rot_dim, vdim, q_rank, kv_rank, window, base=10000.0, dims=None, scale=None):
    return {"type": "latent_attention",
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank,
                      "mask": {"size": window}, "rot": {"base": base, "dims": rot_dim if dims is None else dims},
                      "scale": (dim + rot_dim) ** -0.5 if scale is None else scale}}


def biased(heads, kv_heads, dim, vdim, chunk, scale=None):
    return {"type": "attention",
            "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "mask": {"size": chunk},
                      "scale": dim ** -0.5 if scale is None else scale}}


def with_mlp(layer: Dict, ff) -> Dict:
    return dict(layer, mlp=None if ff is None else {"kind": "dense", "ff": ff})


def config(vocab, width, layers, loop=None, eps=1e-5) -> Dict:
    cfg = {"architecture": "Dokulix", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}
    if loop is not None:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg


# P: every size differs from its neighbours; value heads narrower and wider than key heads, a rotated
# part of which only the first half turns, a window shorter than a page and one that crosses pages, blocks
# that are no multiple of a page, a layer without a feed-forward, a loop of three passes that
# starts after the first layer.
CFG_P = config(257, 64, [
    with_mlp(latent(4, 16, 8, 24, 48, 40, 20, base=100.0), 96),
    with_mlp(biased(4, 2, 32, 16, 24), 80),
    with_mlp(latent(2, 24, 16, 8, 32, 24, 70, base=5000.0, dims=8), None),
    with_mlp(biased(3, 3, 16, 48, 65, scale=0.4), 72),
], loop=(1, 3, 3), eps=3e-6)

# Q: no loop; one key/value head under six query heads, blocks longer than two pages, head sizes the
# matrix-core kernels know (64, and a latent row of 64 + 32).
CFG_Q = config(300, 96, [
    with_mlp(biased(6, 1, 64, 64, 130), 128),
    with_mlp(latent(8, 32, 32, 32, 64, 64, 100), 128),
    with_mlp(biased(4, 2, 64, 64, 64), 128),
    with_mlp(latent(4, 64, 64, 64, 96, 128, 33), 160),
])

# R: the values that make mechanisms vanish: one head, a window and blocks of one position, a loop
# of one pass over the only layers, widths that are no multiple of 8.
CFG_R = config(131, 36, [
    with_mlp(latent(1, 10, 6, 10, 12, 14, 1), 20),
    with_mlp(biased(1, 1, 12, 12, 1), None),
    with_mlp(biased(2, 2, 20, 12, 7), 28),
    with_mlp(latent(3, 8, 4, 12, 20, 10, 5), 44),
], loop=(0, 4, 1), eps=1e-3)

CONFIGS = {"P": (CFG_P, 11), "Q": (CFG_Q, 12), "R": (CFG_R, 13)}


def tensor_shapes(cfg: Dict) -> Dict[str, tuple]:
    w = cfg["width"]
    shapes = {"embed": (cfg["vocab"], w), "final.norm": (w,), "head": (cfg["vocab"], w)}
    if cfg.get("loop"):
        shapes["loop.step"] = (cfg["loop"]["times"], w)
    for i, layer in enumerate(cfg["layers"]):
        m, p = layer["mixer"], f"l{i}."
        shapes[p + "norm1"] = (w,)
        if layer["type"] == "attention":
            H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            shapes.update({p + "mix.q": (H * d, w), p + "mix.q.b": (H * d,), p + "mix.k": (G * d, w),
                           p + "mix.k.b": (G * d,), p + "mix.v": (G * dv, w), p + "mix.v.b": (G * dv,),
                           p + "mix.q.norm": (d,), p + "mix.k.norm": (d,), p + "mix.o": (w, H * dv), p + "mix.o.b": (w,)})
        else:
            H, d, r, dv = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
            shapes.update({p + "mix.dq": (m["q_rank"], w), p + "mix.dq.norm": (m["q_rank"],),
                           p + "mix.uq": (H * (d + r), m["q_rank"]), p + "mix.dkv": (m["kv_rank"] + r, w),
                           p + "mix.dkv.norm": (m["kv_rank"],), p + "mix.uk": (H * d, m["kv_rank"]),
                           p + "mix.uv": (H * dv, m["kv_rank"]), p + "mix.g": (H * dv, w), p + "mix.o": (w, H * dv)})
        if layer.get("mlp") is not None:
            ff = layer["mlp"]["ff"]
            shapes.update({p + "norm2": (w,), p + "mlp.gate": (ff, w), p + "mlp.up": (ff, w), p + "mlp.down": (w, ff)})
    return shapes


def random_tensors(cfg: Dict, seed: int) -> Dict[str, torch.Tensor]:
    """Values that bfloat16 holds exactly (so both compute types read the same weights)."""
    gen = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        if name.endswith((".norm", "norm1", "norm2")) and not name.endswith(("q.norm", "k.norm", "dq.norm", "dkv.norm")):
            t = 0.3 * torch.randn(shape, generator=gen)                 # stored around zero
        elif name.endswith(".norm"):
            t = 1.0 + 0.3 * torch.randn(shape, generator=gen)           # plain weights
        elif name.endswith(".b"):
            t = 0.3 * torch.randn(shape, generator=gen)
        elif name == "embed" or name == "loop.step":
            t = torch.randn(shape, generator=gen)
        else:
            t = torch.randn(shape, generator=gen) * (1.5 / shape[-1] ** 0.5)
        out[name] = t.to(torch.bfloat16).to(torch.float32)
    return out


def write_model(path: str, cfg: Dict, tensors: Dict[str, torch.Tensor], dtype=torch.bfloat16) -> str:
    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.to(dtype).contiguous() for k, v in tensors.items()}, os.path.join(path, "model.safetensors"))
    return path
