"""Typed configuration of the Vobolorn decoder, read from ``config.json``, and the model it describes.

A Vobolorn model is a list of layers over a 32-bit residual stream.  Every layer has one of three token
mixers and a gated feed-forward (or none); each branch reads the stream itself and is RMS-normed on its
way into it.  The mixers: grouped-query attention with biases and a gate per output channel
("attention"), grouped-query attention whose queries grow with the logarithm of the position
("attention_2"), and attention through a latent with a shared rotated key part and a gate per head
("latent_attention").  The grouped-query layers norm queries and keys per head with a weight, use no
rotation, and may lean their values on those of the first layer that says ``v_mix``.  The logits may be
capped.  Every size and constant comes from config.json; nothing here knows a particular model.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, List, Optional, Tuple

from .llama import ConfigError
from .spec import LayerSpec, LayerRun, ModelSpec, PartSpec

ARCHITECTURE = "Vobolorn"
MIXER_TYPES = ("attention", "attention_2", "latent_attention")
#: config.json names no longest context: nothing but memory bounds it
DEFAULT_MAX_POSITIONS = 1 << 20

_GQA_KEYS = ("heads", "kv_heads", "dim", "vdim", "scale")
_MIXER_KEYS = {
    "attention": _GQA_KEYS,
    "attention_2": _GQA_KEYS,
    "latent_attention": ("heads", "dim", "rot_dim", "vdim", "q_rank", "kv_rank", "scale", "rot"),
}


def _positive_int(where: str, name: str, v) -> int:
    if not isinstance(v, int) or isinstance(v, bool) or v <= 0:
        raise ConfigError(f"{where}: {name} must be a positive integer, got {v!r}")
    return v


def _number(where: str, name: str, v) -> float:
    if not isinstance(v, (int, float)) or isinstance(v, bool):
        raise ConfigError(f"{where}: {name} must be a number, got {v!r}")
    return float(v)


@dataclass(frozen=True)
class VobolornLayer:
    """One entry of ``layers``: the mixer's type and sizes and the feed-forward's width (None: none)."""

    type: str
    mixer: Dict[str, Any]
    ff: Optional[int] = None

    def to_dict(self) -> Dict[str, Any]:
        return {"type": self.type, "mixer": self.mixer, "mlp": None if self.ff is None else {"kind": "dense", "ff": self.ff}}


@dataclass(frozen=True)
class VobolornConfig:
    vocab: int
    width: int
    layers: Tuple[VobolornLayer, ...]
    norm_eps: float
    logit_softcap: float = 0.0
    eos_token_id: Any = None
    architectures: tuple = (ARCHITECTURE,)

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "VobolornConfig":
        missing = [k for k in ("vocab", "width", "layers", "norm") if k not in d]
        if missing:
            raise ConfigError(f"config.json lacks required keys {missing}")
        _positive_int("config", "vocab", d["vocab"])
        _positive_int("config", "width", d["width"])
        if not isinstance(d["layers"], list) or not d["layers"]:
            raise ConfigError("config.json: 'layers' must be a list with at least one layer")
        eps = d["norm"].get("eps") if isinstance(d["norm"], dict) else None
        if not isinstance(eps, (int, float)) or isinstance(eps, bool) or not eps > 0:
            raise ConfigError(f"config.json: norm.eps must be positive, got {eps!r}")
        cap = d.get("logit_softcap")
        if cap is not None and (_number("config", "logit_softcap", cap) <= 0):
            raise ConfigError(f"config.json: logit_softcap must be positive when given, got {cap!r}")
        layers = [cls._layer_from_dict(i, entry) for i, entry in enumerate(d["layers"])]
        mixing = [l for l in layers if l.mixer.get("v_mix")]
        if len({(l.mixer["kv_heads"], l.mixer["vdim"]) for l in mixing}) > 1:
            raise ConfigError("config.json: layers that mix their values (v_mix) must agree in kv_heads and vdim")
        return cls(vocab=d["vocab"], width=d["width"], layers=tuple(layers), norm_eps=float(eps),
                   logit_softcap=float(cap) if cap is not None else 0.0, eos_token_id=d.get("eos_token_id"))

    @staticmethod
    def _layer_from_dict(i: int, entry: Dict[str, Any]) -> VobolornLayer:
        where = f"layers[{i}]"
        if not isinstance(entry, dict):
            raise ConfigError(f"{where}: not an object")
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
            if k == "rot_dim":  # (a latent layer may rotate nothing)
                if not isinstance(mixer[k], int) or isinstance(mixer[k], bool) or mixer[k] < 0:
                    raise ConfigError(f"{where}: rot_dim must be an integer that is not negative, got {mixer[k]!r}")
            elif k not in ("scale", "rot"):
                _positive_int(where, k, mixer[k])
        if not _number(where, "scale", mixer["scale"]) > 0:
            raise ConfigError(f"{where}: scale must be positive, got {mixer['scale']!r}")
        if kind in ("attention", "attention_2"):
            if mixer["heads"] % mixer["kv_heads"]:
                raise ConfigError(f"{where}: {mixer['heads']} heads are not a multiple of {mixer['kv_heads']} kv_heads")
            qt = mixer.get("q_temp")
            if kind == "attention_2" and qt is None:
                raise ConfigError(f"{where}: the attention_2 mixer lacks ['q_temp']")
            if qt is not None:
                if not isinstance(qt, dict) or "coef" not in qt or "every" not in qt:
                    raise ConfigError(f"{where}: q_temp needs 'coef' and 'every'")
                _number(where, "q_temp.coef", qt["coef"])
                every = qt["every"]
                if isinstance(every, float) and every.is_integer():  # (64.0 is 64)
                    every = int(every)
                    mixer = dict(mixer, q_temp=dict(qt, every=every))
                _positive_int(where, "q_temp.every", every)
        else:
            rot = mixer["rot"]
            if not isinstance(rot, dict) or "dims" not in rot or "base" not in rot:
                raise ConfigError(f"{where}: rot needs 'dims' and 'base'")
            if rot["dims"] != mixer["rot_dim"] or mixer["rot_dim"] % 2:
                raise ConfigError(f"{where}: rot.dims={rot['dims']!r} must be rot_dim={mixer['rot_dim']!r}, and even")
            if not _number(where, "rot.base", rot["base"]) > 0:
                raise ConfigError(f"{where}: rot.base must be positive")
        mlp = entry.get("mlp")
        ff = None
        if mlp is not None:
            if not isinstance(mlp, dict) or mlp.get("kind") != "dense":
                raise ConfigError(f"{where}: mlp.kind {mlp.get('kind') if isinstance(mlp, dict) else mlp!r} is not 'dense'")
            ff = _positive_int(where, "mlp.ff", mlp.get("ff"))
        return VobolornLayer(type=kind, mixer=dict(mixer), ff=ff)

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {
            "architecture": ARCHITECTURE,
            "vocab": self.vocab,
            "width": self.width,
            "norm": {"eps": self.norm_eps},
            "layers": [layer.to_dict() for layer in self.layers],
        }
        if self.logit_softcap > 0:
            d["logit_softcap"] = self.logit_softcap
        if self.eos_token_id is not None:
            d["eos_token_id"] = self.eos_token_id
        return d

    def first_mixing_layer(self) -> Optional[int]:
        """The first layer that says ``v_mix``: the one whose values the later such layers lean on."""
        for i, layer in enumerate(self.layers):
            if layer.mixer.get("v_mix"):
                return i
        return None


def _mixer_spec(cfg: VobolornConfig, i: int) -> PartSpec:
    layer = cfg.layers[i]
    m = layer.mixer
    if layer.type == "latent_attention":
        position = PartSpec("rope", dict(head_dim=m["rot_dim"], rotary_dim=m["rot_dim"], theta=float(m["rot"]["base"]), scaling=None,
                                         pairing="interleaved")) if m["rot_dim"] > 0 else PartSpec("none", {})
        return PartSpec("latent_attention", dict(
            hidden_size=cfg.width, num_heads=m["heads"], head_dim=m["dim"], rot_dim=m["rot_dim"], v_head_dim=m["vdim"],
            q_rank=m["q_rank"], kv_rank=m["kv_rank"], softmax_scale=float(m["scale"]), norm_eps=cfg.norm_eps, position=position,
            head_gate=True,
        ))
    qt = m.get("q_temp") or {}
    mix = None
    if m.get("v_mix"):
        mix = "source" if cfg.first_mixing_layer() == i else "mix"
    return PartSpec("attention", dict(
        hidden_size=cfg.width, num_heads=m["heads"], num_kv_heads=m["kv_heads"], head_dim=m["dim"], qkv_bias=layer.type == "attention",
        softmax_scale=float(m["scale"]), window=0, position=PartSpec("none", {}), v_head_dim=m["vdim"], qk_norm_eps=cfg.norm_eps,
        qk_norm_weight=True, q_temp_coef=float(qt.get("coef", 0.0)), q_temp_every=int(qt.get("every", 1)), value_mix=mix,
        value_mix_key="first_values", out_gate="channel" if layer.type == "attention" else None,
    ))


def vobolorn_model_spec(cfg: VobolornConfig) -> ModelSpec:
    """The model as data: one ``LayerSpec`` per layer, named ``l<i>`` as its tensors are."""
    norm = PartSpec("rmsnorm", dict(size=cfg.width, eps=cfg.norm_eps, stream_dtype="float32"))
    specs: List[LayerSpec] = []
    for i, layer in enumerate(cfg.layers):
        parts = {"norm1": norm, "mix": _mixer_spec(cfg, i)}
        if layer.ff is not None:
            parts["norm2"] = norm
            parts["mlp"] = PartSpec("swiglu", dict(hidden_size=cfg.width, intermediate_size=layer.ff, activation="silu"))
        specs.append(LayerSpec(name=f"l{i}", block="branch_norm" if layer.ff is not None else "branch_norm_mixer", parts=parts))
    spec = ModelSpec(
        architecture=ARCHITECTURE,
        hidden_size=cfg.width,
        vocab_size=cfg.vocab,
        max_positions=DEFAULT_MAX_POSITIONS,
        embedding=PartSpec("embedding", dict(vocab_size=cfg.vocab, hidden_size=cfg.width, scale=1.0, stream_dtype="float32")),
        layers=specs,
        order=[LayerRun(i) for i in range(len(specs))],
        final_norm=norm,
        head=PartSpec("lm_head", dict(vocab_size=cfg.vocab, hidden_size=cfg.width, tied=False, softcap=cfg.logit_softcap)),
    )
    spec.validate()
    return spec
