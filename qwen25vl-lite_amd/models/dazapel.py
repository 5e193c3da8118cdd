"""The Dazapel decoder as a model spec.

A stack of layers with a norm before and behind each sublayer and a fixed factor on what joins the
residual sum: ``x += m norm1b(mixer(norm1(x)))``, ``x += m norm2b(ff(norm2(x)))``.  A range of the layers
may run several times in a row with the same weights; each pass has a cache of its own and starts
by adding its vector (a row of ``loop.step``) to the sum.

* mixer ``attention``: grouped key/value heads, biased projections, values of their own width, rotation
  of the first ``rot.dims`` channels of every head in halves (channel i with i + dims/2) with
  frequencies stretched by a ramp over the channel index and cosines and sines scaled (``rot.scaling``:
  ``factor``, ``original``, ``fast``, ``slow``), then queries and keys divided by their root mean square
  per head, a fixed score scale, a sliding window that also keeps a request's first tokens visible
  (``mask``: ``size``, ``keep_first``), every channel of the heads' joined output scaled by the sigmoid of its own channel of a
  projection of the mixer's input, a biased output projection.
* feed-forward ``moe``: routed experts with sigmoid scores, a choice limited to the best groups of
  neighbouring experts, weights normalised over the choice and scaled, plus a shared expert.  Every
  expert is ``down(g sigmoid(1.702 g) (u + 1))`` with the gate capped at ``limit`` and the linear
  branch clamped to ``[-limit, limit]``.

The output head is the embedding table.

``config.json``: ``architecture``, ``width``, ``vocab``, ``norm.eps``, ``residual_mult``, ``loop``
(``start``, ``stop``, ``times``; optional) and ``layers``, a list of ``{"type", "mixer": {...}, "mlp": {...} | null}``.
Tensors are named ``embed``, ``final.norm``, ``loop.step``, ``l<i>.norm1|norm1b|norm2|norm2b``, ``l<i>.mix.<name>``,
``l<i>.mlp.router``, ``l<i>.mlp.e<j>.gate|up|down``, ``l<i>.mlp.shared.gate|up|down``; a bias ends in ``.b``.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

from ..config.model_config import ConfigError
from ..config.registry import register_architecture
from ..parts.base import PartSpec
from .spec import LayerSpec, ModelSpec, RunEntry

__all__ = ["DazapelConfig", "dazapel_spec", "dazapel_run_list"]

# constants the design fixes
GATE_SLOPE = 1.702              # g * sigmoid(1.702 g)
LINEAR_BRANCH_SHIFT = 1.0       # (u + 1)
WEIGHT_SUM_FLOOR = 1e-20        # added to the sum the routing weights are divided by
MIXER_TYPES = ("attention",)
MLP_KINDS = ("moe",)


def _need(block: Any, keys, where: str) -> None:
    if not isinstance(block, dict):
        raise ConfigError(f"config.json: {where} must be an object")
    missing = [k for k in keys if k not in block]
    if missing:
        raise ConfigError(f"config.json: {where} lacks {', '.join(missing)}")


def _positive(value, what: str) -> None:
    if not (isinstance(value, (int, float)) and value > 0):
        raise ConfigError(f"config.json: {what} must be positive")


@dataclass
class DazapelConfig:
    """The parsed ``config.json``.  Sizes and constants have no defaults: what the file does not
    give is an error (``loop``, a mixer's ``mask`` and ``rot.scaling``, and an ``mlp``'s ``shared`` may be
    absent or null: then the model has none)."""

    width: int
    vocab: int
    eps: float
    residual_mult: float
    layers: List[Dict[str, Any]]
    loop: Optional[Dict[str, int]] = None
    architecture: str = "Dazapel"
    eos_token_id: Optional[int] = None
    raw: Dict[str, Any] = field(default_factory=dict, repr=False)

    @classmethod
    def from_dict(cls, raw: Dict[str, Any]) -> "DazapelConfig":
        _need(raw, ("width", "vocab", "norm", "residual_mult", "layers"), "the top level")
        _need(raw["norm"], ("eps",), "norm")
        layers = raw["layers"]
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json: layers must be a non-empty list")
        for i, layer in enumerate(layers):
            where = f"layers[{i}]"
            _need(layer, ("type", "mixer"), where)
            if layer["type"] not in MIXER_TYPES:
                raise ConfigError(f"config.json: {where} has type {layer['type']!r}; known: {', '.join(MIXER_TYPES)}")
            m = layer["mixer"]
            _need(m, ("heads", "kv_heads", "dim", "vdim", "scale", "rot"), f"{where}.mixer")
            for key in ("heads", "kv_heads", "dim", "vdim"):
                _positive(m[key], f"{where}.mixer.{key}")
            if int(m["heads"]) % int(m["kv_heads"]):
                raise ConfigError(f"config.json: {where}: heads must be a multiple of kv_heads")
            _need(m["rot"], ("base", "dims"), f"{where}.mixer.rot")
            dims = int(m["rot"]["dims"])
            if dims < 0 or dims % 2 or dims > int(m["dim"]):
                raise ConfigError(f"config.json: {where}.mixer.rot.dims must be even and at most dim")
            if m["rot"].get("scaling"):
                _need(m["rot"]["scaling"], ("factor", "original", "fast", "slow"), f"{where}.mixer.rot.scaling")
            if m.get("mask"):
                _need(m["mask"], ("size", "keep_first"), f"{where}.mixer.mask")
                _positive(m["mask"]["size"], f"{where}.mixer.mask.size")
                if int(m["mask"]["keep_first"]) < 0:
                    raise ConfigError(f"config.json: {where}.mixer.mask.keep_first cannot be negative")
            mlp = layer.get("mlp")
            if mlp is not None:
                _need(mlp, ("kind", "expert", "router"), f"{where}.mlp")
                if mlp["kind"] not in MLP_KINDS:
                    raise ConfigError(f"config.json: {where}.mlp has kind {mlp['kind']!r}; known: {', '.join(MLP_KINDS)}")
                _need(mlp["expert"], ("ff", "limit"), f"{where}.mlp.expert")
                r = mlp["router"]
                _need(r, ("experts", "top", "scale"), f"{where}.mlp.router")
                groups = r.get("groups") or {"count": 1, "keep": 1}
                _need(groups, ("count", "keep"), f"{where}.mlp.router.groups")
                e, top, count, keep = int(r["experts"]), int(r["top"]), int(groups["count"]), int(groups["keep"])
                if count <= 0 or e <= 0 or e % count or not 0 < keep <= count or not 0 < top <= keep * (e // count):
                    raise ConfigError(f"config.json: {where}.mlp.router: {e} experts in {count} groups, {keep} kept, "
                                      f"{top} chosen do not fit together")
                if mlp.get("shared"):
                    _need(mlp["shared"], ("ff", "limit"), f"{where}.mlp.shared")
        loop = raw.get("loop") or None
        if loop is not None:
            _need(loop, ("start", "stop", "times"), "loop")
            start, stop, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
            if not (0 <= start < stop <= len(layers)) or times < 1:
                raise ConfigError("config.json: loop needs 0 <= start < stop <= the number of layers and times >= 1")
            loop = {"start": start, "stop": stop, "times": times}
        return cls(width=int(raw["width"]), vocab=int(raw["vocab"]), eps=float(raw["norm"]["eps"]),
                   residual_mult=float(raw["residual_mult"]), layers=layers, loop=loop,
                   architecture=str(raw.get("architecture") or "Dazapel"), eos_token_id=raw.get("eos_token_id"),
                   raw=dict(raw))

    def to_dict(self) -> Dict[str, Any]:
        return dict(self.raw)


def _store_name(name: str) -> str:
    """Canonical name (``l0.mix.q.weight``, ``l0.mix.q.bias``) -> the file's (``l0.mix.q``, ``l0.mix.q.b``)."""
    if name.endswith(".weight"):
        return name[:-len(".weight")]
    if name.endswith(".bias"):
        return name[:-len(".bias")] + ".b"
    return name


def _map_name(name: str) -> str:
    return name[:-2] + ".bias" if name.endswith(".b") else name + ".weight"


def _attention_spec(m: Dict[str, Any], width: int, eps: float) -> PartSpec:
    rot = m["rot"]
    scaling = rot.get("scaling") or None
    if scaling:
        scaling = {"kind": "ramp", "factor": float(scaling["factor"]), "original": int(scaling["original"]),
                   "fast": float(scaling["fast"]), "slow": float(scaling["slow"])}
    position = PartSpec("rope", {"theta": float(rot["base"]), "rotary_dim": int(rot["dims"]), "scaling": scaling})
    mask = m.get("mask") or None
    return PartSpec("paged_attention", {
        "hidden_size": width, "num_heads": int(m["heads"]), "num_kv_heads": int(m["kv_heads"]), "head_dim": int(m["dim"]),
        "value_dim": int(m["vdim"]), "qkv_bias": True, "out_bias": True, "scale": float(m["scale"]), "position": position,
        "window": None if mask is None else int(mask["size"]), "keep_first": 0 if mask is None else int(mask["keep_first"]),
        "qk_norm_eps": eps, "qk_norm_where": "after", "qk_norm_weights": False, "element_gate": True,
        "names": {"q": "q", "k": "k", "v": "v", "o": "o", "g": "g"},
    })


def _expert_ff(width: int, sizes: Dict[str, Any]) -> PartSpec:
    return PartSpec("clamped_gated", {
        "hidden_size": width, "intermediate_size": int(sizes["ff"]), "alpha": GATE_SLOPE, "limit": float(sizes["limit"]),
        "shift": LINEAR_BRANCH_SHIFT, "names": {"gate": "gate", "up": "up", "down": "down"}})


def _moe_spec(mlp: Dict[str, Any], width: int) -> PartSpec:
    r = mlp["router"]
    groups = r.get("groups") or {"count": 1, "keep": 1}
    return PartSpec("routed_experts", {
        "hidden_size": width, "num_experts": int(r["experts"]), "top": int(r["top"]),
        "intermediate_size": int(mlp["expert"]["ff"]), "alpha": GATE_SLOPE, "limit": float(mlp["expert"]["limit"]),
        "shift": LINEAR_BRANCH_SHIFT, "groups": int(groups["count"]), "keep": int(groups["keep"]),
        "scale": float(r["scale"]), "score": "sigmoid", "normalize": True, "floor": WEIGHT_SUM_FLOOR,
        "shared": _expert_ff(width, mlp["shared"]) if mlp.get("shared") else None,
        "names": {"router": "router", "expert": "e{}", "gate": "gate", "up": "up", "down": "down", "shared": "shared"},
    })


def dazapel_run_list(num_layers: int, loop: Optional[Dict[str, int]]) -> List[RunEntry]:
    """The layers in the order they run: those before the looped range, the range ``times`` times
    (the first layer of pass t adds pass vector t), those after it."""
    if loop is None:
        return [RunEntry(i) for i in range(num_layers)]
    start, stop, times = loop["start"], loop["stop"], loop["times"]
    run = [RunEntry(i) for i in range(start)]
    for t in range(times):
        run += [RunEntry(i, add_vector=t if i == start else None) for i in range(start, stop)]
    return run + [RunEntry(i) for i in range(stop, num_layers)]


def dazapel_spec(config: DazapelConfig) -> ModelSpec:
    width, eps = config.width, config.eps
    norm = PartSpec("rms_norm", {"size": width, "eps": eps})
    layers: List[LayerSpec] = []
    for i, layer in enumerate(config.layers):
        mlp = layer.get("mlp")
        block = PartSpec("sandwich", {
            "norm1": norm, "mixer": _attention_spec(layer["mixer"], width, eps), "norm1b": norm,
            "norm2": norm, "ffn": None if mlp is None else _moe_spec(mlp, width), "norm2b": norm,
            "residual_mult": config.residual_mult,
            "names": {"norm1": "norm1", "mixer": "mix", "norm1b": "norm1b", "norm2": "norm2", "ffn": "mlp",
                      "norm2b": "norm2b"}})
        layers.append(LayerSpec(block, f"l{i}."))
    return ModelSpec(
        hidden_size=width, vocab_size=config.vocab, layers=layers, run=dazapel_run_list(len(layers), config.loop),
        final_norm=norm, tie_word_embeddings=True, position_rows=1,
        embed_name="embed.weight", final_norm_prefix="final.norm.", head_name="lm_head.weight",
        map_name=_map_name, store_name=_store_name, eos_token_id=config.eos_token_id,
        pass_vectors_name=None if config.loop is None else "loop.step.weight",
        pass_vectors_rows=0 if config.loop is None else config.loop["times"],
    )


register_architecture("Dazapel", dazapel_spec, DazapelConfig.from_dict)
