"""A plain, slow implementation of the Dazapel decoder: whole sequences, no cache, dense masks, one
function per mechanism, on the CPU.  It reads config.json and the safetensors file by itself and
shares no code with the engine; the engine's logits are compared with it.

Notation: ``x`` is ``[T, width]``, a linear weight is ``[out, in]`` and applied as ``x @ W.T``.
``store`` is applied to whatever the engine may keep in bfloat16 (matrix products and their
activations); norms, angles, scores, the router and the residual sum stay in the working precision.
"""

from __future__ import annotations

import json
import math
import os
from typing import Callable, Dict, List, Optional

import torch

SLOPE = 1.702          # g * sigmoid(1.702 g)
SHIFT = 1.0            # (u + 1)
WEIGHT_FLOOR = 1e-20   # added to the sum the routing weights are divided by


def _keep(x: torch.Tensor) -> torch.Tensor:
    return x


def to_bfloat16_and_back(x: torch.Tensor) -> torch.Tensor:
    return x.to(torch.bfloat16).to(x.dtype)


def dazapel_read(model_dir: str, dtype=torch.float64):
    """``(config dict, {tensor name: tensor})`` with the names the file uses."""
    from safetensors import safe_open

    with open(os.path.join(model_dir, "config.json")) as fh:
        cfg = json.load(fh)
    tensors = {}
    with safe_open(os.path.join(model_dir, "model.safetensors"), framework="pt", device="cpu") as f:
        for name in f.keys():
            tensors[name] = f.get_tensor(name).to(dtype)
    return cfg, tensors


# --------------------------------------------------------------------------------------------
# small pieces
# --------------------------------------------------------------------------------------------
def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """Each row divided by its root mean square, eps inside the root."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    return unit_rms(x, eps) * w


# --------------------------------------------------------------------------------------------
# rotation
# --------------------------------------------------------------------------------------------
def yarn_frequencies(dims: int, base: float, scaling: Optional[dict]):
    """``(frequencies [dims/2], factor on cos and sin)``.  Without scaling: ``base^(-2i/dims)``, 1."""
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=torch.float64)
    if not scaling:
        return f, 1.0
    factor, original = float(scaling["factor"]), float(scaling["original"])

    def dim_of(turns: float) -> float:
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(dim_of(float(scaling["fast"]))), 0)
    hi = min(math.ceil(dim_of(float(scaling["slow"]))), dims - 1)
    ramp = torch.tensor([min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0) for i in range(half)], dtype=torch.float64)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate_half_layout(x: torch.Tensor, positions: torch.Tensor, dims: int, base: float, scaling: Optional[dict]):
    """``x [T, heads, dim]``: channel i < dims/2 is paired with channel i + dims/2; channels from
    ``dims`` on pass unchanged."""
    freqs, mult = yarn_frequencies(dims, base, scaling)
    ang = positions.to(torch.float64)[:, None] * freqs[None, :]
    cos = (torch.cos(ang) * mult).to(x.dtype)[:, None, :]
    sin = (torch.sin(ang) * mult).to(x.dtype)[:, None, :]
    half = dims // 2
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * cos - v * sin, v * cos + u * sin, x[..., dims:]], dim=-1)


# --------------------------------------------------------------------------------------------
# attention
# --------------------------------------------------------------------------------------------
def visible(T: int, size: Optional[int], keep_first: int) -> torch.Tensor:
    """``[T, T]`` bool: query i sees key j."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    causal = j <= i
    if size is None:
        return causal
    return causal & ((i - j < size) | (j < keep_first))


def attention_mixer(h: torch.Tensor, t: Dict[str, torch.Tensor], p: str, m: dict, eps: float,
                    store: Callable = _keep) -> torch.Tensor:
    T = h.shape[0]
    H, G, D, V = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q = (h @ t[p + "q"].T + t[p + "q.b"]).view(T, H, D)
    k = (h @ t[p + "k"].T + t[p + "k.b"]).view(T, G, D)
    v = store(h @ t[p + "v"].T + t[p + "v.b"]).view(T, G, V)
    gate = store(h @ t[p + "g"].T)
    pos = torch.arange(T)
    rot = m["rot"]
    q = rotate_half_layout(q, pos, int(rot["dims"]), float(rot["base"]), rot.get("scaling"))
    k = rotate_half_layout(k, pos, int(rot["dims"]), float(rot["base"]), rot.get("scaling"))
    q, k = store(unit_rms(q, eps)), store(unit_rms(k, eps))
    mask = m.get("mask")
    see = visible(T, None if not mask else int(mask["size"]), 0 if not mask else int(mask["keep_first"]))
    out = torch.empty(T, H, V, dtype=h.dtype)
    for head in range(H):
        g = head // (H // G)
        s = (q[:, head] @ k[:, g].T) * float(m["scale"])
        s = s.masked_fill(~see, float("-inf"))
        out[:, head] = torch.softmax(s, dim=-1) @ v[:, g]
    out = store(out.reshape(T, H * V) * torch.sigmoid(gate))
    return out @ t[p + "o"].T + t[p + "o.b"]


# --------------------------------------------------------------------------------------------
# feed-forward
# --------------------------------------------------------------------------------------------
def expert(h: torch.Tensor, t: Dict[str, torch.Tensor], p: str, limit: float, store: Callable = _keep) -> torch.Tensor:
    g = store(h @ t[p + "gate"].T).clamp(max=limit)
    u = store(h @ t[p + "up"].T).clamp(-limit, limit)
    return store(g * torch.sigmoid(SLOPE * g) * (u + SHIFT)) @ t[p + "down"].T


def route(z: torch.Tensor, top: int, groups: int, keep: int, scale: float):
    """Router logits ``[T, E]`` -> ``(chosen [T, top], weights [T, top])``."""
    T, E = z.shape
    s = torch.sigmoid(z)
    per = E // groups
    grouped = s.view(T, groups, per)
    gscore = grouped.topk(min(2, per), dim=-1).values.sum(-1)
    best = gscore.topk(keep, dim=-1).indices
    allowed = torch.zeros(T, groups, dtype=torch.bool)
    allowed.scatter_(1, best, True)
    masked = torch.where(allowed[:, :, None].expand(T, groups, per).reshape(T, E), s, torch.full_like(s, -1.0))
    chosen = masked.topk(top, dim=-1).indices
    w = s.gather(1, chosen)
    return chosen, w / (w.sum(-1, keepdim=True) + WEIGHT_FLOOR) * scale


def choice_margin(z: torch.Tensor, top: int, groups: int, keep: int) -> torch.Tensor:
    """Per token, by how much the router's choice is clear: the gap between the last group kept and
    the first one left out, and between the last expert chosen and the best allowed one left out
    (infinite where nothing is left out)."""
    T, E = z.shape
    s = torch.sigmoid(z)
    per = E // groups
    gscore = s.view(T, groups, per).topk(min(2, per), dim=-1).values.sum(-1).sort(dim=-1, descending=True)
    margin = torch.full((T,), float("inf"), dtype=z.dtype)
    if keep < groups:
        margin = gscore.values[:, keep - 1] - gscore.values[:, keep]
    allowed = torch.zeros(T, groups, dtype=torch.bool).scatter_(1, gscore.indices[:, :keep], True)
    masked = torch.where(allowed[:, :, None].expand(T, groups, per).reshape(T, E), s, torch.full_like(s, -1.0))
    if top < keep * per:
        ranked = masked.sort(dim=-1, descending=True).values
        margin = torch.minimum(margin, ranked[:, top - 1] - ranked[:, top])
    return margin


def moe(h: torch.Tensor, t: Dict[str, torch.Tensor], p: str, mlp: dict, store: Callable = _keep,
        margins: Optional[list] = None) -> torch.Tensor:
    r = mlp["router"]
    z = h @ t[p + "router"].T
    if margins is not None:
        margins.append(choice_margin(z, int(r["top"]), int(r["groups"]["count"]), int(r["groups"]["keep"])))
    chosen, w = route(z, int(r["top"]), int(r["groups"]["count"]), int(r["groups"]["keep"]), float(r["scale"]))
    out = torch.zeros(h.shape[0], t[p + "e0.down"].shape[0], dtype=h.dtype)
    limit = float(mlp["expert"]["limit"])
    for e in range(int(r["experts"])):
        hit = chosen == e
        rows = hit.any(-1).nonzero().flatten()
        if rows.numel():
            we = (w * hit).sum(-1)[rows]
            out[rows] += we[:, None] * expert(h[rows], t, f"{p}e{e}.", limit, store)
    if mlp.get("shared"):
        out = out + expert(h, t, p + "shared.", float(mlp["shared"]["limit"]), store)
    return out


# --------------------------------------------------------------------------------------------
# the model
# --------------------------------------------------------------------------------------------
def run_order(cfg: dict) -> List[tuple]:
    """``(layer, pass number or None)`` in the order the layers run; the pass number stands at the
    first layer of each pass through the looped range."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, None) for i in range(n)]
    start, stop, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    order = [(i, None) for i in range(start)]
    for t in range(times):
        order += [(i, t if i == start else None) for i in range(start, stop)]
    return order + [(i, None) for i in range(stop, n)]


def dazapel_forward(cfg: dict, t: Dict[str, torch.Tensor], tokens, store: Callable = _keep,
                    trace: Optional[list] = None, margins: Optional[list] = None) -> torch.Tensor:
    """Logits ``[T, vocab]`` of a whole sequence.  ``trace`` collects the residual after every layer
    run, ``margins`` every router's :func:`choice_margin` per token."""
    eps, mult = float(cfg["norm"]["eps"]), float(cfg["residual_mult"])
    x = t["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    for i, pass_no in run_order(cfg):
        if pass_no is not None:
            x = x + t["loop.step"][pass_no]
        layer, p = cfg["layers"][i], f"l{i}."
        if layer["type"] != "attention":
            raise ValueError(layer["type"])
        y = attention_mixer(store(rms_norm(x, t[p + "norm1"], eps)), t, p + "mix.", layer["mixer"], eps, store)
        x = x + mult * rms_norm(y, t[p + "norm1b"], eps)
        if layer.get("mlp") is not None:
            y = moe(store(rms_norm(x, t[p + "norm2"], eps)), t, p + "mlp.", layer["mlp"], store, margins)
            x = x + mult * rms_norm(y, t[p + "norm2b"], eps)
        if trace is not None:
            trace.append(x.clone())
    return store(rms_norm(x, t["final.norm"], eps)) @ t["embed"].T
