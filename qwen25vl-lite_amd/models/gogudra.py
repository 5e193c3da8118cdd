"""The Gogudra decoder as a model spec.

A stack of parallel layers (one norm whose output feeds both the mixer and the feed-forward;
the norm's weight is stored around zero and used as ``1 + w``), each with one of three mixers:

* ``lightning``: linear attention with a fixed decay per head, silu on q, k and v, the heads normed
  together, a sigmoid gate;
* ``gla``: gated linear attention, a decay per key channel and token ``sigmoid(z)^(1/tau)`` from a
  low-rank projection, queries scaled by ``dim^-0.5``, each head normed by itself, a silu gate;
* ``attention``: softmax attention over grouped key/value heads whose values are the keys as
  projected, a per-head norm of queries and keys, interleaved rotation of the first ``rot.dims``
  channels with wavelength-dependent frequency scaling, a fixed score scale, a sigmoid gate per head.

The feed-forward is ``down(g sigmoid(1.702 g) (u + 1))`` with the gate capped at ``limit`` and the
linear branch clamped to ``[-limit, limit]``.  The output head is the embedding table, and the
logits pass through ``c tanh(. / c)``.

``config.json``: ``architecture``, ``width``, ``vocab``, ``norm.eps``, ``logit_softcap``, and
``layers``, a list of ``{"type", "mixer": {sizes and constants}, "mlp": {"kind", "ff", "limit"} | null}``.
Tensors are named ``embed``, ``final.norm``, ``l<i>.norm1``, ``l<i>.mix.<name>``, ``l<i>.mlp.<name>``;
a bias ends in ``.b``.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

from ..config.model_config import ConfigError
from ..config.registry import register_architecture
from ..parts.base import PartSpec
from .spec import LayerSpec, ModelSpec, RunEntry

__all__ = ["GogudraConfig", "gogudra_spec", "GELU_SIGMOID_SLOPE"]

# constants the design fixes
GELU_SIGMOID_SLOPE = 1.702      # g * sigmoid(1.702 g)
LINEAR_BRANCH_SHIFT = 1.0       # (u + 1)
MIXER_TYPES = ("lightning", "gla", "attention")


def _need(block: Dict[str, Any], keys, where: str) -> None:
    missing = [k for k in keys if k not in block]
    if missing:
        raise ConfigError(f"config.json: {where} lacks {', '.join(missing)}")


@dataclass
class GogudraConfig:
    """The parsed ``config.json``.  Sizes and constants have no defaults: what the file does not
    give is an error."""

    width: int
    vocab: int
    eps: float
    layers: List[Dict[str, Any]]
    logit_softcap: Optional[float] = None
    architecture: str = "Gogudra"
    eos_token_id: Optional[int] = None
    raw: Dict[str, Any] = field(default_factory=dict, repr=False)

    @classmethod
    def from_dict(cls, raw: Dict[str, Any]) -> "GogudraConfig":
        _need(raw, ("width", "vocab", "norm", "layers"), "the top level")
        _need(raw["norm"], ("eps",), "norm")
        layers = raw["layers"]
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json: layers must be a non-empty list")
        for i, layer in enumerate(layers):
            where = f"layers[{i}]"
            _need(layer, ("type", "mixer"), where)
            kind, m = layer["type"], layer["mixer"]
            if kind not in MIXER_TYPES:
                raise ConfigError(f"config.json: {where} has type {kind!r}; known: {', '.join(MIXER_TYPES)}")
            _need(m, ("heads", "dim", "vdim"), f"{where}.mixer")
            if kind == "lightning":
                _need(m, ("decay",), f"{where}.mixer")
                if len(m["decay"]) != int(m["heads"]):
                    raise ConfigError(f"config.json: {where}.mixer.decay needs one value per head")
            elif kind == "gla":
                _need(m, ("tau",), f"{where}.mixer")
            else:
                _need(m, ("kv_heads", "scale", "rot"), f"{where}.mixer")
                _need(m["rot"], ("base", "dims"), f"{where}.mixer.rot")
                if m["rot"].get("scaling"):
                    _need(m["rot"]["scaling"], ("factor", "low", "high", "original"), f"{where}.mixer.rot.scaling")
                if int(m["vdim"]) != int(m["dim"]):
                    raise ConfigError(f"config.json: {where}: the values are the keys, so vdim must equal dim")
                if int(m["heads"]) % int(m["kv_heads"]):
                    raise ConfigError(f"config.json: {where}: heads must be a multiple of kv_heads")
            mlp = layer.get("mlp")
            if mlp is not None:
                _need(mlp, ("kind", "ff", "limit"), f"{where}.mlp")
                if mlp["kind"] != "dense":
                    raise ConfigError(f"config.json: {where}.mlp has kind {mlp['kind']!r}; known: dense")
        cap = raw.get("logit_softcap")
        return cls(width=int(raw["width"]), vocab=int(raw["vocab"]), eps=float(raw["norm"]["eps"]), layers=layers,
                   logit_softcap=None if not cap else float(cap),
                   architecture=str(raw.get("architecture") or "Gogudra"), eos_token_id=raw.get("eos_token_id"),
                   raw=dict(raw))

    def to_dict(self) -> Dict[str, Any]:
        return dict(self.raw)


def _store_name(name: str) -> str:
    """Canonical name (``l0.mix.q.weight``, ``l0.mix.a2.bias``) -> the file's (``l0.mix.q``, ``l0.mix.a2.b``)."""
    if name.endswith(".weight"):
        return name[:-len(".weight")]
    if name.endswith(".bias"):
        return name[:-len(".bias")] + ".b"
    return name


def _map_name(name: str) -> str:
    return name[:-2] + ".bias" if name.endswith(".b") else name + ".weight"


def _mixer_spec(kind: str, m: Dict[str, Any], width: int, eps: float, rank: Optional[int]) -> PartSpec:
    heads, dim, vdim = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    if kind == "attention":
        rot = m["rot"]
        position = PartSpec("rope", {"theta": float(rot["base"]), "rotary_dim": int(rot["dims"]),
                                     "scaling": rot.get("scaling") or None, "interleaved": True})
        return PartSpec("paged_attention", {
            "hidden_size": width, "num_heads": heads, "num_kv_heads": int(m["kv_heads"]), "head_dim": dim,
            "qkv_bias": False, "window": None, "scale": float(m["scale"]), "position": position,
            "qk_norm_eps": eps, "values_are_keys": True, "head_gate": True,
            "names": {"q": "q", "k": "k", "o": "o", "g": "g", "q_norm": "q.norm", "k_norm": "k.norm"},
        })
    common = {"hidden_size": width, "num_heads": heads, "key_dim": dim, "value_dim": vdim, "eps": eps}
    if kind == "lightning":
        return PartSpec("linear_attention", {
            **common, "decay": {"kind": "head", "values": [float(a) for a in m["decay"]]},
            "activation": "silu", "q_scale": 1.0, "norm": "all_heads", "gate": "sigmoid"})
    return PartSpec("linear_attention", {
        **common, "decay": {"kind": "channel", "rank": rank, "tau": float(m["tau"])},
        "activation": None, "q_scale": dim ** -0.5, "norm": "per_head", "gate": "silu"})


def gogudra_spec(config: GogudraConfig) -> ModelSpec:
    width, eps = config.width, config.eps
    norm = PartSpec("rms_norm", {"size": width, "eps": eps, "offset": 1.0})
    layers: List[LayerSpec] = []
    for i, layer in enumerate(config.layers):
        m = layer["mixer"]
        # the decay projection's inner size is a tensor's shape, not a key of config.json
        rank = m.get("rank")
        if layer["type"] == "gla" and rank is None:
            rank = _tensor_rows(config, f"l{i}.mix.a1")
        mixer = _mixer_spec(layer["type"], m, width, eps, rank)
        mlp = layer.get("mlp")
        ffn = None if mlp is None else PartSpec("clamped_gated", {
            "hidden_size": width, "intermediate_size": int(mlp["ff"]), "alpha": GELU_SIGMOID_SLOPE,
            "limit": float(mlp["limit"]), "shift": LINEAR_BRANCH_SHIFT,
            "names": {"gate": "gate", "up": "up", "down": "down"}})
        block = PartSpec("parallel", {"norm": norm, "mixer": mixer, "ffn": ffn,
                                      "names": {"norm": "norm1", "mixer": "mix", "ffn": "mlp"}})
        layers.append(LayerSpec(block, f"l{i}."))
    sizes = {"vocab_size": config.vocab, "hidden_size": width}
    return ModelSpec(
        hidden_size=width, vocab_size=config.vocab, layers=layers, run=[RunEntry(i) for i in range(len(layers))],
        final_norm=norm, tie_word_embeddings=True, position_rows=1,
        embed_name="embed.weight", final_norm_prefix="final.norm.", head_name="lm_head.weight",
        map_name=_map_name, store_name=_store_name, eos_token_id=config.eos_token_id,
        head=PartSpec("linear", {**sizes, "softcap": config.logit_softcap}),
    )


def _tensor_rows(config: GogudraConfig, name: str) -> int:
    """Rows of a tensor of the model's safetensors file (read from its header), for a size that only
    a shape gives.  A configuration that came without a folder must give the size itself."""
    import os

    folder = getattr(config, "name_or_path", None)
    path = os.path.join(folder, "model.safetensors") if folder else None
    if not path or not os.path.isfile(path):
        raise ConfigError(f"the size of {name} comes from the tensor's shape: load the configuration from a model "
                          "folder, or give the mixer a 'rank'")
    from ..weights.safetensors_io import SafetensorsFile

    with SafetensorsFile(path) as f:
        if name not in f.keys():
            raise ConfigError(f"{path} holds no tensor {name}")
        return int(f.shape(name)[0])


register_architecture("Gogudra", gogudra_spec, GogudraConfig.from_dict)
