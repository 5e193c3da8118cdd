"""Small Dazapel configurations and model folders with random weights for the tests.  The weights
are drawn here (not by the engine) and written with the safetensors package."""

from __future__ import annotations

import json
import os
from typing import Dict, Optional

import torch


def attention(heads, kv_heads, dim, vdim, rot_dims, base=10000.0, scaling=None, scale=None, mask=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale or dim ** -0.5,
         "rot": {"base": base, "dims": rot_dims, "scaling": scaling}}
    if mask is not None:
        m["mask"] = {"size": mask[0], "keep_first": mask[1]}
    return m


def moe(experts, top, ff, limit, groups=(1, 1), scale=1.0, shared=None):
    mlp = {"kind": "moe", "expert": {"ff": ff, "limit": limit},
           "router": {"experts": experts, "top": top, "scale": scale, "groups": {"count": groups[0], "keep": groups[1]}}}
    if shared is not None:
        mlp["shared"] = {"ff": shared[0], "limit": shared[1]}
    return mlp


def layer(mixer, mlp=None):
    return {"type": "attention", "mixer": mixer, "mlp": mlp}


def config(width, vocab, layers, eps=1e-5, mult=0.5, loop=None):
    cfg = {"architecture": "Dazapel", "width": width, "vocab": vocab, "norm": {"eps": eps}, "residual_mult": mult,
           "layers": layers}
    if loop is not None:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg


RAMP = {"factor": 8.0, "original": 32, "fast": 4.0, "slow": 0.5}

# Sizes that all differ from one another; value heads wider and narrower than key heads; head sizes on
# and off the matrix-core steps of 16; partial and full rotation, with and without the ramp; windows
# with and without kept first tokens and a layer that sees everything; layers with different experts,
# one without a feed-forward, one without a shared expert; the middle two layers run three times.
MIXED = config(72, 203, [
    layer(attention(4, 2, 16, 24, 8, base=500.0, scaling=RAMP, scale=0.7, mask=(9, 3)),
          moe(6, 2, 40, 1.0, groups=(3, 2), scale=1.5, shared=(56, 0.8))),
    layer(attention(6, 2, 20, 12, 20, base=10000.0, scale=0.5, mask=(21, 0)),
          moe(8, 3, 24, 2.0, groups=(4, 2), scale=0.7)),
    layer(attention(2, 2, 32, 32, 16, base=80.0, scaling={"factor": 2.0, "original": 16, "fast": 2.0, "slow": 1.0},
                    scale=0.4)),
    layer(attention(3, 1, 48, 16, 48, base=2000.0, scale=0.3, mask=(37, 18)),
          moe(4, 4, 32, 0.6, groups=(1, 1), scale=2.0, shared=(16, 1.5))),
], eps=1e-5, mult=0.4, loop=(1, 3, 3))

# The same shapes with score scales so large that the softmax picks single keys: a key lost at a
# window's edge, a page's border or among the kept first tokens moves the logits.
SHARP = json.loads(json.dumps(MIXED))
for _l, _s in zip(SHARP["layers"], (5.0, 4.0, 3.0, 2.5)):
    _l["mixer"]["scale"] = _s

# Values that happen to be 1 or equal: one head, one key/value head, one expert chosen of one group,
# every expert chosen, a window of one token, one kept token, a loop that runs once, a factor of one
# on the residual, equal key and value sizes.
ONES = config(32, 61, [
    layer(attention(1, 1, 16, 16, 2, base=100.0, scale=1.0, mask=(1, 1)), moe(1, 1, 16, 1.0, shared=(16, 1.0))),
    layer(attention(2, 1, 16, 16, 16, base=100.0, scale=1.0, mask=(16, 16)), moe(2, 2, 8, 1.0, groups=(2, 2))),
    layer(attention(2, 2, 8, 8, 4, base=9.0, scale=0.25), moe(3, 1, 8, 3.0, groups=(3, 1), scale=1.0)),
], eps=1e-6, mult=1.0, loop=(0, 1, 1))

# Sizes that no vector width divides: an odd width and vocabulary, head sizes of 6 and 10, odd expert
# sizes, a group of three experts, no loop at all.
ODD = config(50, 101, [
    layer(attention(3, 3, 10, 7, 6, base=77.0, scaling=RAMP, scale=0.4, mask=(5, 2)),
          moe(9, 2, 11, 1.2, groups=(3, 2), scale=1.1, shared=(13, 0.9))),
    layer(attention(2, 1, 6, 9, 6, base=30.0, scale=0.6), moe(2, 1, 7, 2.0)),
], eps=1e-5, mult=0.7)


def tensor_shapes(cfg: dict) -> Dict[str, tuple]:
    w = cfg["width"]
    shapes = {"embed": (cfg["vocab"], w), "final.norm": (w,)}
    if cfg.get("loop"):
        shapes["loop.step"] = (cfg["loop"]["times"], w)
    for i, lay in enumerate(cfg["layers"]):
        p, m = f"l{i}.", lay["mixer"]
        h, g, d, v = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        shapes.update({p + "norm1": (w,), p + "norm1b": (w,),
                       p + "mix.q": (h * d, w), p + "mix.q.b": (h * d,), p + "mix.k": (g * d, w), p + "mix.k.b": (g * d,),
                       p + "mix.v": (g * v, w), p + "mix.v.b": (g * v,), p + "mix.g": (h * v, w),
                       p + "mix.o": (w, h * v), p + "mix.o.b": (w,)})
        mlp = lay.get("mlp")
        if mlp:
            shapes.update({p + "norm2": (w,), p + "norm2b": (w,), p + "mlp.router": (mlp["router"]["experts"], w)})
            names = [(f"e{e}", mlp["expert"]["ff"]) for e in range(mlp["router"]["experts"])]
            if mlp.get("shared"):
                names.append(("shared", mlp["shared"]["ff"]))
            for name, ff in names:
                shapes.update({f"{p}mlp.{name}.gate": (ff, w), f"{p}mlp.{name}.up": (ff, w), f"{p}mlp.{name}.down": (w, ff)})
    return shapes


def random_tensors(cfg: dict, seed: int) -> Dict[str, torch.Tensor]:
    """bfloat16 tensors.  Matrices N(0, 1/in) (the router's and the gates' larger, so that choices are
    clear and clamps bite); norm weights around 1; biases and pass vectors of the size of the activations."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        if "norm" in name:
            t = 1.0 + 0.2 * torch.randn(shape, generator=g)
        elif name.endswith(".b") or name == "loop.step":
            t = 0.5 * torch.randn(shape, generator=g)
        elif name == "embed":
            t = torch.randn(shape, generator=g)
        else:
            boost = 3.0 if name.endswith("router") else (1.5 if name.endswith((".gate", ".up")) else 1.0)
            t = torch.randn(shape, generator=g) * boost / shape[1] ** 0.5
        out[name] = t.to(torch.bfloat16)
    return out


def write_model(folder: str, cfg: dict, seed: int, tensors: Optional[Dict[str, torch.Tensor]] = None) -> str:
    from safetensors.torch import save_file

    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as fh:
        json.dump(cfg, fh)
    save_file(tensors if tensors is not None else random_tensors(cfg, seed), os.path.join(folder, "model.safetensors"))
    return folder
