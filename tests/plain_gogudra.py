"""A plain, slow implementation of the Gogudra decoder: whole sequences, no cache, token-by-token
recurrences, one function per mechanism, on the CPU.  It reads config.json and the safetensors
file by itself and shares no code with the engine; the engine's logits are compared with it.

Notation: ``x`` is ``[T, width]``, a linear weight is ``[out, in]`` and applied as ``x @ W.T``.
``store`` is applied to whatever the engine may keep in bfloat16 (matrix products and their
activations); norms, scores, decays, states and the residual sum stay in the working precision.
"""

from __future__ import annotations

import json
import math
import os
from typing import Callable, Dict, List, Optional, Sequence

import torch


def _keep(x: torch.Tensor) -> torch.Tensor:
    return x


def to_bfloat16_and_back(x: torch.Tensor) -> torch.Tensor:
    return x.to(torch.bfloat16).to(x.dtype)


def gogudra_read(model_dir: str, dtype=torch.float64):
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


def layer_norm_one_plus(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """The layers' norm: the weight is stored around zero and used as a gain of 1 + w."""
    return unit_rms(x, eps) * (1.0 + w)


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def scaled_frequencies(rot: dict) -> List[float]:
    """Rotation frequency of every pair: base^(-2i/dims), then long wavelengths slowed down by
    ``factor``, short ones kept, the band between blended linearly in original/wavelength."""
    dims, base = int(rot["dims"]), float(rot["base"])
    freqs = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    sc = rot.get("scaling")
    if not sc:
        return freqs
    factor, low, high, orig = float(sc["factor"]), float(sc["low"]), float(sc["high"]), float(sc["original"])
    out = []
    for f in freqs:
        wavelength = 2.0 * math.pi / f
        if wavelength < orig / high:
            out.append(f)
        elif wavelength > orig / low:
            out.append(f / factor)
        else:
            s = (orig / wavelength - low) / (high - low)
            out.append((1.0 - s) * f / factor + s * f)
    return out


def rotate_interleaved(x: torch.Tensor, positions: torch.Tensor, freqs: Sequence[float]) -> torch.Tensor:
    """``x [T, heads, dim]``: channel 2i is paired with channel 2i+1 for i below len(freqs); the
    remaining channels pass unchanged.  Angles are formed in float32 like the engine's."""
    out = x.clone()
    f = torch.tensor(list(freqs), dtype=torch.float32)
    ang = (positions.to(torch.float32)[:, None] * f[None, :]).to(x.dtype)      # [T, pairs]
    cos, sin = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    n = 2 * len(freqs)
    u, v = x[..., 0:n:2], x[..., 1:n:2]
    out[..., 0:n:2] = u * cos - v * sin
    out[..., 1:n:2] = v * cos + u * sin
    return out


# --------------------------------------------------------------------------------------------
# mixers
# --------------------------------------------------------------------------------------------
def attention_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], p: dict, eps: float, start: int = 0,
                    store: Callable = _keep) -> torch.Tensor:
    """Softmax attention with grouped key/value heads whose values are the projected keys (taken
    before the key norm and the rotation), a per-head norm on queries and keys, partial interleaved
    rotation, a fixed score scale and a per-head sigmoid gate on the output."""
    T = h.shape[0]
    H, G, D = int(p["heads"]), int(p["kv_heads"]), int(p["dim"])
    q = store(h @ w["q"].T).view(T, H, D)
    k_raw = store(h @ w["k"].T).view(T, G, D)
    v = k_raw
    q = unit_rms(q, eps) * w["q.norm"]
    k = unit_rms(k_raw, eps) * w["k.norm"]
    pos = torch.arange(start, start + T)
    freqs = scaled_frequencies(p["rot"])
    q, k = store(rotate_interleaved(q, pos, freqs)), store(rotate_interleaved(k, pos, freqs))
    gate = torch.sigmoid(h @ w["g"].T)                      # [T, H]
    out = torch.zeros(T, H, D, dtype=h.dtype)
    rep = H // G
    causal = torch.tril(torch.ones(T, T, dtype=torch.bool))
    for head in range(H):
        g = head // rep
        scores = (q[:, head] @ k[:, g].T) * float(p["scale"])
        scores = scores.masked_fill(~causal, float("-inf"))
        out[:, head] = torch.softmax(scores, dim=-1) @ v[:, g]
    out = store(out) * gate[:, :, None]
    return store(out.reshape(T, H * D)) @ w["o"].T


def decayed_outer_product_scan(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, decay: torch.Tensor,
                               state: Optional[torch.Tensor] = None):
    """One head: ``S_t = diag(decay_t) S_(t-1) + k_t v_t^T``, ``o_t = S_t^T q_t``, token by token.
    ``q, k [T, dim]``, ``v [T, vdim]``, ``decay [T, dim]``.  Returns ``(o [T, vdim], S)``."""
    T, dim = k.shape
    S = torch.zeros(dim, v.shape[1], dtype=q.dtype) if state is None else state.clone()
    o = torch.zeros(T, v.shape[1], dtype=q.dtype)
    for t in range(T):
        S = decay[t][:, None] * S + k[t][:, None] * v[t][None, :]
        o[t] = S.T @ q[t]
    return o, S


def lightning_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], p: dict, eps: float,
                    store: Callable = _keep) -> torch.Tensor:
    """Linear attention with one fixed decay per head; silu on q, k and v; the heads' outputs are
    normed together, gated by a sigmoid and projected."""
    T = h.shape[0]
    H, D, V = int(p["heads"]), int(p["dim"]), int(p["vdim"])
    q = store(silu(h @ w["q"].T)).view(T, H, D)
    k = store(silu(h @ w["k"].T)).view(T, H, D)
    v = store(silu(h @ w["v"].T)).view(T, H, V)
    out = torch.zeros(T, H, V, dtype=h.dtype)
    for head in range(H):
        decay = torch.full((T, D), float(p["decay"][head]), dtype=torch.float32).to(h.dtype)
        out[:, head], _ = decayed_outer_product_scan(q[:, head], k[:, head], v[:, head], decay)
    y = unit_rms(out.reshape(T, H * V), eps) * w["norm"]
    y = y * torch.sigmoid(store(h @ w["g"].T))
    return store(y) @ w["o"].T


def gla_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], p: dict, eps: float, store: Callable = _keep) -> torch.Tensor:
    """Gated linear attention: a decay per key channel and token from a low-rank projection,
    ``sigmoid(z)^(1/tau)``; each head's output normed by itself, gated by silu, projected."""
    T = h.shape[0]
    H, D, V = int(p["heads"]), int(p["dim"]), int(p["vdim"])
    q = store((h @ w["q"].T) * D ** -0.5).view(T, H, D)
    k = store(h @ w["k"].T).view(T, H, D)
    v = store(h @ w["v"].T).view(T, H, V)
    z = store(store(h @ w["a1"].T) @ w["a2"].T) + w["a2.b"]
    decay = torch.exp(torch.nn.functional.logsigmoid(z) / float(p["tau"])).view(T, H, D)
    out = torch.zeros(T, H, V, dtype=h.dtype)
    for head in range(H):
        out[:, head], _ = decayed_outer_product_scan(q[:, head], k[:, head], v[:, head], decay[:, head])
    y = unit_rms(out, eps) * w["norm"]
    y = y.reshape(T, H * V) * silu(store(h @ w["g"].T))
    return store(y) @ w["o"].T


# --------------------------------------------------------------------------------------------
# feed-forward, head, model
# --------------------------------------------------------------------------------------------
def clamped_gated_ff(h: torch.Tensor, w: Dict[str, torch.Tensor], p: dict, store: Callable = _keep) -> torch.Tensor:
    """``down(g sigmoid(1.702 g) (u + 1))`` with the gate capped from above and the linear branch
    clamped on both sides."""
    limit = float(p["limit"])
    g = torch.clamp(store(h @ w["gate"].T), max=limit)
    u = torch.clamp(store(h @ w["up"].T), -limit, limit)
    return store(g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ w["down"].T


def _sub(tensors: Dict[str, torch.Tensor], prefix: str) -> Dict[str, torch.Tensor]:
    return {k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)}


MIXERS = {"attention": attention_mixer, "lightning": lightning_mixer, "gla": gla_mixer}


def gogudra_logits(cfg: dict, tensors: Dict[str, torch.Tensor], tokens: Sequence[int], store: Callable = _keep,
                   layers_out: Optional[list] = None) -> torch.Tensor:
    """Logits ``[T, vocab]`` of a whole sequence.  ``layers_out`` collects the residual stream
    after every layer."""
    eps = float(cfg["norm"]["eps"])
    embed = tensors["embed"]
    x = embed[torch.tensor(list(tokens), dtype=torch.long)]
    for i, layer in enumerate(cfg["layers"]):
        pre = f"l{i}."
        h = store(layer_norm_one_plus(x, tensors[pre + "norm1"], eps))
        y = MIXERS[layer["type"]](h, _sub(tensors, pre + "mix."), layer["mixer"], eps, store=store)
        if layer.get("mlp") is not None:
            if layer["mlp"]["kind"] != "dense":
                raise ValueError(f"feed-forward kind {layer['mlp']['kind']!r}")
            y = y + clamped_gated_ff(h, _sub(tensors, pre + "mlp."), layer["mlp"], store=store)
        x = x + y
        if layers_out is not None:
            layers_out.append(x.clone())
    xn = store(layer_norm_one_plus(x, tensors["final.norm"], eps))
    logits = xn @ embed.T
    cap = cfg.get("logit_softcap")
    if cap:
        logits = float(cap) * torch.tanh(logits / float(cap))
    return logits


def gogudra_model_logits(model_dir: str, tokens: Sequence[int], store: Callable = _keep, dtype=torch.float64,
                         layers_out: Optional[list] = None) -> torch.Tensor:
    cfg, tensors = gogudra_read(model_dir, dtype)
    return gogudra_logits(cfg, tensors, tokens, store, layers_out)
