"""Typed configuration of the Taluvik decoder, read from ``config.json``, and the model it describes.

A Taluvik model is a list of layers, each with one of three token mixers (chunked attention with a
sink, the gated delta rule, a selective scan) and a gated feed-forward or none, all reading one layer
norm and added to a 32-bit residual stream with a common factor.  A layer may reuse the tensors of
another ("weights_of") while keeping a cache or state of its own.  Every size and constant comes from
config.json; nothing here knows a particular model.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional, Tuple

from .llama import ConfigError
from .spec import LayerRun, LayerSpec, ModelSpec, PartSpec

ARCHITECTURE = "Taluvik"
MIXER_TYPES = ("attention", "delta", "mamba1")
#: config.json names no longest context: angles, chunks and states are computed from positions, so the
#: bound is a matter of memory alone; an engine is given its own ``max_model_len`` or pool size
DEFAULT_MAX_POSITIONS = 1 << 20

_MIXER_KEYS = {
    "attention": ("heads", "kv_heads", "dim", "vdim", "scale", "softcap", "mask", "rot"),
    "delta": ("heads", "kv_heads", "dim", "vdim", "conv"),
    "mamba1": ("inner", "state", "dt_rank", "conv"),
}


def _positive_int(where: str, name: str, v) -> int:
    if not isinstance(v, int) or isinstance(v, bool) or v <= 0:
        raise ConfigError(f"{where}: {name} must be a positive integer, got {v!r}")
    return v


@dataclass(frozen=True)
class TaluvikLayer:
    """One entry of ``layers``: the mixer's type and sizes, the feed-forward's width (None: the layer
    has none) and, for a layer without tensors of its own, the layer whose tensors it uses."""

    type: str
    mixer: Dict[str, Any]
    ff: Optional[int] = None
    weights_of: Optional[int] = None

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {"type": self.type, "mixer": self.mixer,
                             "mlp": None if self.ff is None else {"kind": "dense", "ff": self.ff}}
        if self.weights_of is not None:
            d["weights_of"] = self.weights_of
        return d


@dataclass(frozen=True)
class TaluvikConfig:
    vocab: int
    width: int
    layers: Tuple[TaluvikLayer, ...]
    norm_eps: float
    residual_mult: float = 1.0
    embedding_scale: float = 1.0
    eos_token_id: Any = None
    architectures: tuple = (ARCHITECTURE,)

    # ------------------------------------------------------------------ reading / writing
    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "TaluvikConfig":
        missing = [k for k in ("vocab", "width", "layers", "norm") if k not in d]
        if missing:
            raise ConfigError(f"config.json lacks required keys {missing}")
        _positive_int("config", "vocab", d["vocab"])
        _positive_int("config", "width", d["width"])
        if not isinstance(d["layers"], list) or not d["layers"]:
            raise ConfigError("config.json: 'layers' must be a list with at least one layer")
        eps = d["norm"].get("eps") if isinstance(d["norm"], dict) else None
        if not isinstance(eps, (int, float)) or not eps > 0:
            raise ConfigError(f"config.json: norm.eps must be positive, got {eps!r}")
        layers = []
        for i, entry in enumerate(d["layers"]):
            layers.append(cls._layer_from_dict(i, entry, len(d["layers"])))
        # a layer that borrows tensors names a layer that owns them (chains are followed to their end)
        for i, layer in enumerate(layers):
            seen = {i}
            j = layer.weights_of
            while j is not None:
                if j in seen:
                    raise ConfigError(f"layers[{i}]: weights_of runs in a circle")
                seen.add(j)
                j = layers[j].weights_of
        emb = d.get("embedding") or {}
        return cls(
            vocab=d["vocab"],
            width=d["width"],
            layers=tuple(layers),
            norm_eps=float(eps),
            residual_mult=float(d.get("residual_mult", 1.0)),
            embedding_scale=float(emb.get("scale", 1.0)),
            eos_token_id=d.get("eos_token_id"),
        )

    @staticmethod
    def _layer_from_dict(i: int, entry: Dict[str, Any], n_layers: int) -> TaluvikLayer:
        where = f"layers[{i}]"
        kind = entry.get("type")
        if kind not in MIXER_TYPES:
            raise ConfigError(f"{where}: type {kind!r} is not one of {list(MIXER_TYPES)}")
        mixer = entry.get("mixer")
        if not isinstance(mixer, dict):
            raise ConfigError(f"{where}: no 'mixer' sizes")
        lacking = [k for k in _MIXER_KEYS[kind] if k not in mixer]
        if lacking:
            raise ConfigError(f"{where}: the {kind} mixer lacks {lacking}")
        for k in _MIXER_KEYS[kind]:
            if k not in ("scale", "softcap", "mask", "rot"):
                _positive_int(where, k, mixer[k])
        if kind in ("attention", "delta") and mixer["heads"] % mixer["kv_heads"]:
            raise ConfigError(f"{where}: {mixer['heads']} heads are not a multiple of {mixer['kv_heads']} kv_heads")
        if kind == "attention":
            _positive_int(where, "mask.size", (mixer["mask"] or {}).get("size"))
            rot = mixer["rot"]
            if not isinstance(rot, dict) or "dims" not in rot or "base" not in rot:
                raise ConfigError(f"{where}: rot needs 'dims' and 'base'")
            if not isinstance(rot["dims"], int) or rot["dims"] < 0 or rot["dims"] % 2 or rot["dims"] > mixer["dim"]:
                raise ConfigError(f"{where}: rot.dims={rot['dims']!r} must be even and at most dim={mixer['dim']}")
            sc = rot.get("scaling")
            if sc:
                lacking = [k for k in ("factor", "low", "high", "original") if k not in sc]
                if lacking:
                    raise ConfigError(f"{where}: rot.scaling lacks {lacking}")
                if sc["high"] == sc["low"]:
                    raise ConfigError(f"{where}: rot.scaling.high must differ from low")
            if not mixer["softcap"] > 0:
                raise ConfigError(f"{where}: softcap must be positive, got {mixer['softcap']!r}")
        mlp = entry.get("mlp")
        ff = None
        if mlp is not None:
            if mlp.get("kind") != "dense":
                raise ConfigError(f"{where}: mlp.kind {mlp.get('kind')!r} is not 'dense'")
            ff = _positive_int(where, "mlp.ff", mlp.get("ff"))
        owner = entry.get("weights_of")
        if owner is not None:
            if not isinstance(owner, int) or isinstance(owner, bool) or not 0 <= owner < n_layers or owner == i:
                raise ConfigError(f"{where}: weights_of={owner!r} must name another layer")
        return TaluvikLayer(type=kind, mixer=dict(mixer), ff=ff, weights_of=owner)

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {
            "architecture": ARCHITECTURE,
            "vocab": self.vocab,
            "width": self.width,
            "embedding": {"scale": self.embedding_scale},
            "norm": {"eps": self.norm_eps},
            "residual_mult": self.residual_mult,
            "layers": [layer.to_dict() for layer in self.layers],
        }
        if self.eos_token_id is not None:
            d["eos_token_id"] = self.eos_token_id
        return d

    def owner_of(self, i: int) -> int:
        """The layer whose tensors layer ``i`` uses (itself, unless it names another)."""
        while self.layers[i].weights_of is not None:
            i = self.layers[i].weights_of
        return i


def _mixer_spec(cfg: TaluvikConfig, layer: TaluvikLayer) -> PartSpec:
    m = layer.mixer
    if layer.type == "attention":
        rot = m["rot"]
        scaling = None
        if rot.get("scaling"):
            sc = rot["scaling"]
            scaling = {"rope_type": "llama3", "factor": sc["factor"], "low_freq_factor": sc["low"],
                       "high_freq_factor": sc["high"], "original_max_position_embeddings": sc["original"]}
        position = PartSpec("rope", dict(head_dim=m["dim"], rotary_dim=rot["dims"], theta=rot["base"], scaling=scaling,
                                         pairing="half")) if rot["dims"] > 0 else PartSpec("none", {})
        return PartSpec("attention", dict(
            hidden_size=cfg.width, num_heads=m["heads"], num_kv_heads=m["kv_heads"], head_dim=m["dim"], qkv_bias=False,
            softmax_scale=float(m["scale"]), window=0, position=position, v_head_dim=m["vdim"], qk_norm_eps=cfg.norm_eps,
            softcap=float(m["softcap"]), chunk=m["mask"]["size"], sinks=True,
        ))
    if layer.type == "delta":
        return PartSpec("gated_delta", dict(
            hidden_size=cfg.width, num_heads=m["heads"], num_key_heads=m["kv_heads"], head_dim=m["dim"], v_head_dim=m["vdim"],
            conv_taps=m["conv"], norm_eps=cfg.norm_eps,
        ))
    return PartSpec("selective_scan", dict(
        hidden_size=cfg.width, inner_size=m["inner"], state_size=m["state"], dt_rank=m["dt_rank"], conv_taps=m["conv"],
    ))


def taluvik_model_spec(cfg: TaluvikConfig) -> ModelSpec:
    """The model as data: one ``LayerSpec`` for every layer that owns tensors (named ``l<i>`` as its
    tensors are), and an execution order that runs a borrowing layer as a second run of its owner,
    with a cache entry of its own."""
    norm = PartSpec("layernorm", dict(size=cfg.width, eps=cfg.norm_eps))
    specs: List[LayerSpec] = []
    index_of: Dict[int, int] = {}
    for i, layer in enumerate(cfg.layers):
        if layer.weights_of is not None:
            continue
        parts = {"norm1": norm, "mix": _mixer_spec(cfg, layer)}
        if layer.ff is not None:
            parts["mlp"] = PartSpec("swiglu", dict(hidden_size=cfg.width, intermediate_size=layer.ff, activation="gelu_tanh"))
        index_of[i] = len(specs)
        specs.append(LayerSpec(name=f"l{i}", block="parallel" if layer.ff is not None else "parallel_mixer", parts=parts,
                               block_params=dict(residual_mult=cfg.residual_mult)))
    order = [LayerRun(index_of[cfg.owner_of(i)]) for i in range(len(cfg.layers))]
    spec = ModelSpec(
        architecture=ARCHITECTURE,
        hidden_size=cfg.width,
        vocab_size=cfg.vocab,
        max_positions=DEFAULT_MAX_POSITIONS,
        embedding=PartSpec("embedding", dict(vocab_size=cfg.vocab, hidden_size=cfg.width, scale=cfg.embedding_scale,
                                             stream_dtype="float32")),
        layers=specs,
        order=order,
        final_norm=norm,
        head=PartSpec("lm_head", dict(vocab_size=cfg.vocab, hidden_size=cfg.width, tied=False)),
    )
    spec.validate()
    return spec
