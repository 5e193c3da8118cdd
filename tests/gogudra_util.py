"""Small Gogudra configurations and model folders with random weights for the tests.  The weights
are drawn here (not by the engine) and written with the safetensors package."""

from __future__ import annotations

import json
import os
from typing import Dict, Optional

import torch


def attention_layer(heads, kv_heads, dim, rot_dims, base=10000.0, scaling=None, scale=None, mlp=None):
    return {"type": "attention",
            "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale or dim ** -0.5,
                      "rot": {"base": base, "dims": rot_dims, "scaling": scaling}},
            "mlp": mlp}


def lightning_layer(heads, dim, vdim, decay, mlp=None):
    return {"type": "lightning", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay)}, "mlp": mlp}


def gla_layer(heads, dim, vdim, tau, mlp=None):
    return {"type": "gla", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau}, "mlp": mlp}


def dense(ff, limit):
    return {"kind": "dense", "ff": ff, "limit": limit}


def config(width, vocab, layers, eps=1e-5, softcap=9.0):
    cfg = {"architecture": "Gogudra", "width": width, "vocab": vocab, "norm": {"eps": eps}, "layers": layers}
    if softcap is not None:
        cfg["logit_softcap"] = softcap
    return cfg


# Sizes that are all different from one another; head sizes off and on the matrix-core steps of 16;
# partial and full rotation, with and without frequency scaling; a layer without feed-forward; two
# attention shapes (two cache groups).
MIXED = config(80, 211, [
    gla_layer(2, 12, 24, 5.0, dense(136, 1.0)),
    attention_layer(6, 2, 24, 10, base=1000.0, scale=0.3),
    lightning_layer(3, 20, 40, [0.5, 0.93, 0.999], dense(72, 2.5)),
    attention_layer(4, 4, 32, 32, base=50000.0, scaling={"factor": 8.0, "low": 1.0, "high": 4.0, "original": 64},
                    scale=0.2, mlp=dense(48, 0.7)),
    gla_layer(1, 64, 8, 1.0),
], eps=1e-5, softcap=9.0)

# Values that happen to be 1 or equal: one head, one key/value head, tau 1, a decay of exactly 1,
# equal key and value sizes, no soft cap, rotation of two channels only.
ONES = config(48, 97, [
    lightning_layer(1, 16, 16, [1.0], dense(48, 1.0)),
    attention_layer(1, 1, 16, 2, base=100.0, scale=1.0, mlp=dense(16, 3.0)),
    gla_layer(1, 16, 16, 1.0, dense(24, 0.25)),
], eps=1e-6, softcap=None)

# Only recurrent layers: no pages at all.
NO_PAGES = config(40, 64, [
    gla_layer(2, 8, 12, 3.0, dense(56, 1.5)),
    lightning_layer(2, 12, 8, [0.8, 0.97]),
], eps=1e-6, softcap=4.0)


# Odd everything: a width that eight does not divide, key sizes that four (or two) does not divide, value
# sizes below a wave, an odd inner size of the decay projection, an odd vocabulary.
ODD = config(50, 101, [
    gla_layer(3, 6, 7, 2.0, dense(30, 1.2)),
    lightning_layer(2, 5, 9, [0.9, 0.6]),
    attention_layer(3, 3, 10, 6, base=77.0, scale=0.4, mlp=dense(22, 2.0)),
], eps=1e-5, softcap=6.0)


def tensor_shapes(cfg: dict, rank: int = 6) -> Dict[str, tuple]:
    w = cfg["width"]
    shapes = {"embed": (cfg["vocab"], w), "final.norm": (w,)}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        h, d, v = m["heads"], m["dim"], m["vdim"]
        shapes[p + "norm1"] = (w,)
        if layer["type"] == "attention":
            shapes.update({p + "mix.q": (h * d, w), p + "mix.k": (m["kv_heads"] * d, w), p + "mix.q.norm": (d,),
                           p + "mix.k.norm": (d,), p + "mix.g": (h, w), p + "mix.o": (w, h * d)})
        else:
            shapes.update({p + "mix.q": (h * d, w), p + "mix.k": (h * d, w), p + "mix.v": (h * v, w),
                           p + "mix.g": (h * v, w), p + "mix.o": (w, h * v)})
            if layer["type"] == "lightning":
                shapes[p + "mix.norm"] = (h * v,)
            else:
                shapes.update({p + "mix.norm": (v,), p + "mix.a1": (rank, w), p + "mix.a2": (h * d, rank),
                               p + "mix.a2.b": (h * d,)})
        if layer.get("mlp"):
            ff = layer["mlp"]["ff"]
            shapes.update({p + "mlp.gate": (ff, w), p + "mlp.up": (ff, w), p + "mlp.down": (w, ff)})
    return shapes


def random_tensors(cfg: dict, seed: int, rank: int = 6, sharp: float = 1.0) -> Dict[str, torch.Tensor]:
    """bfloat16 tensors.  Matrices N(0, 1/in); norm weights around 0 (layer norms) or 1 (inner norms);
    the decay bias around +2 so that states remember.  ``sharp`` scales the attention's query norm
    weight: scores grow with it and the softmax picks single keys, so a wrong key shows."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg, rank).items():
        if name.endswith("norm1") or name == "final.norm":
            t = 0.1 * torch.randn(shape, generator=g)
        elif name.endswith(".norm"):
            t = 1.0 + 0.1 * torch.randn(shape, generator=g)
            if name.endswith("q.norm"):
                t = t * sharp
        elif name.endswith(".b"):
            t = 2.0 + torch.randn(shape, generator=g)
        elif name == "embed":
            t = torch.randn(shape, generator=g)
        else:
            t = torch.randn(shape, generator=g) * (1.5 if name.endswith(("mlp.gate", "mlp.up")) else 1.0) / shape[1] ** 0.5
        out[name] = t.to(torch.bfloat16)
    return out


def write_model(folder: str, cfg: dict, seed: int, rank: int = 6, sharp: float = 1.0,
                tensors: Optional[Dict[str, torch.Tensor]] = None) -> str:
    from safetensors.torch import save_file

    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as fh:
        json.dump(cfg, fh)
    save_file(tensors if tensors is not None else random_tensors(cfg, seed, rank, sharp),
              os.path.join(folder, "model.safetensors"))
    return folder
