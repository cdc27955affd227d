"""A plain, slow implementation of the Vobolorn decoder: whole sequences, no cache, one function per
mechanism, only ``torch`` tensor arithmetic.  It shares no code with ``torchllms_amd``; the tests compare
the engine against it.

Conventions: one sequence at a time; activations are [S, ...]; ``weights`` maps the checkpoint's own
tensor names (``l3.mix.q``, ``l3.mlp.up``, ``final.norm`` ...) to tensors; ``config`` is the dictionary
of config.json.  Everything is computed in the dtype the weights are given in (the tests pass 32-bit or
64-bit copies), so the functions state the formulas and nothing about rounding.
"""

from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch


# ----------------------------------------------------------------------------- small functions
def silu(z: torch.Tensor) -> torch.Tensor:
    return z / (1.0 + torch.exp(-z))


def sigmoid(z: torch.Tensor) -> torch.Tensor:
    return 1.0 / (1.0 + torch.exp(-z))


def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """x over its root mean square along the last axis (eps under the root), times w."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w


def gated_feed_forward(h: torch.Tensor, gate: torch.Tensor, up: torch.Tensor, down: torch.Tensor) -> torch.Tensor:
    return (silu(h @ gate.T) * (h @ up.T)) @ down.T


def capped_logits(z: torch.Tensor, cap: float) -> torch.Tensor:
    return cap * torch.tanh(z / cap)


# ----------------------------------------------------------------------------- positions
def query_temperature(S: int, coef: float, every: int, dtype) -> torch.Tensor:
    """The factor on the query at positions 0..S-1: 1 + coef * ln(floor((p + 1) / every) + 1)."""
    return torch.tensor([1.0 + coef * math.log((p + 1) // every + 1) for p in range(S)], dtype=dtype)


def rotate_pairs(x: torch.Tensor, base: float, dims: int) -> torch.Tensor:
    """x [S, ..., d]: channels (2i, 2i+1), i < dims/2, of the token at position p are turned by the angle
    p * base^(-2i/dims); channels from ``dims`` on pass."""
    S = x.shape[0]
    out = x.clone()
    for i in range(dims // 2):
        f = base ** (-2.0 * i / dims)
        ang = torch.arange(S, dtype=torch.float64) * f
        shape = (S,) + (1,) * (x.dim() - 2)
        c = torch.cos(ang).to(x.dtype).reshape(shape)
        s = torch.sin(ang).to(x.dtype).reshape(shape)
        a, b = x[..., 2 * i], x[..., 2 * i + 1]
        out[..., 2 * i] = a * c - b * s
        out[..., 2 * i + 1] = b * c + a * s
    return out


# ----------------------------------------------------------------------------- attention proper
def causal_softmax_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float) -> torch.Tensor:
    """q [S, H, d], k [S, G, d], v [S, G, dv]; query head h reads key/value head h // (H / G); token i
    sees tokens j <= i.  Returns [S, H, dv]."""
    S, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros((S, H, v.shape[2]), dtype=q.dtype)
    mask = torch.ones((S, S), dtype=torch.bool).tril()
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        s = s.masked_fill(~mask, float("-inf"))
        p = torch.softmax(s, dim=-1)
        out[:, h] = p @ v[:, g]
    return out


def mix_values(v: torch.Tensor, v_first: Optional[torch.Tensor], lam) -> torch.Tensor:
    """Values of a layer that mixes: the first such layer's values pass; later ones lean on them."""
    if v_first is None:
        return v
    return (1.0 - lam) * v + lam * v_first


# ----------------------------------------------------------------------------- mixers
def attention_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: dict, eps: float, shared: dict,
                    biases: bool, gate: bool) -> torch.Tensor:
    """The two grouped-query mixers.  ``biases``: q, k, v have them.  ``gate``: the heads' outputs are
    multiplied by sigmoid(W_g h), channel by channel.  ``m["q_temp"]``: the query grows with the logarithm
    of its position.  ``shared`` carries the first mixing layer's values through the model."""
    S = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q, k, v = h @ w[p + "q"].T, h @ w[p + "k"].T, h @ w[p + "v"].T
    if biases:
        q, k, v = q + w[p + "q.b"], k + w[p + "k.b"], v + w[p + "v.b"]
    q = rms_norm(q.reshape(S, H, d), w[p + "q.norm"], eps)
    k = rms_norm(k.reshape(S, G, d), w[p + "k.norm"], eps)
    v = v.reshape(S, G, dv)
    qt = m.get("q_temp")
    if qt:
        q = q * query_temperature(S, qt["coef"], qt["every"], q.dtype).reshape(S, 1, 1)
    if m.get("v_mix"):
        first = shared.get("v_first")
        v = mix_values(v, first, w[p + "vmix"] if first is not None else None)  # (the first such layer's factor is unused)
        shared.setdefault("v_first", v)
    o = causal_softmax_attention(q, k, v, m["scale"]).reshape(S, H * dv)
    if gate:
        o = o * sigmoid(h @ w[p + "g"].T)
    return o @ w[p + "o"].T


def latent_attention_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: dict, eps: float) -> torch.Tensor:
    """Queries through a normed latent; keys and values expanded from a second normed latent; one rotated
    key part for all heads; a gate per head."""
    S = h.shape[0]
    H, d, r, dv, kr = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    base = m["rot"]["base"]
    cq = rms_norm(h @ w[p + "dq"].T, w[p + "dq.norm"], eps)
    q = (cq @ w[p + "uq"].T).reshape(S, H, d + r)
    q_plain, q_rot = q[..., :d], rotate_pairs(q[..., d:], base, r)
    dkv = h @ w[p + "dkv"].T
    c = rms_norm(dkv[:, :kr], w[p + "dkv.norm"], eps)
    k_rot = rotate_pairs(dkv[:, kr:].reshape(S, 1, r), base, r)
    k_plain = (c @ w[p + "uk"].T).reshape(S, H, d)
    v = (c @ w[p + "uv"].T).reshape(S, H, dv)
    qq = torch.cat([q_plain, q_rot], dim=-1)
    kk = torch.cat([k_plain, k_rot.expand(S, H, r)], dim=-1)
    o = causal_softmax_attention(qq, kk, v, m["scale"])
    o = o * sigmoid(h @ w[p + "g"].T).reshape(S, H, 1)
    return o.reshape(S, H * dv) @ w[p + "o"].T


# ----------------------------------------------------------------------------- the model
def forward(config: dict, weights: Dict[str, torch.Tensor], tokens: List[int], return_layers: bool = False):
    """Logits [S, vocab] of one sequence; with ``return_layers`` also the residual stream after every layer."""
    eps = config["norm"]["eps"]
    x = weights["embed"][torch.tensor(tokens, dtype=torch.long)]
    shared: dict = {}
    after = []
    for i, layer in enumerate(config["layers"]):
        p = f"l{i}.mix."
        kind, m = layer["type"], layer["mixer"]
        if kind == "attention":
            y = attention_mixer(x, weights, p, m, eps, shared, biases=True, gate=True)
        elif kind == "attention_2":
            y = attention_mixer(x, weights, p, m, eps, shared, biases=False, gate=False)
        elif kind == "latent_attention":
            y = latent_attention_mixer(x, weights, p, m, eps)
        else:
            raise ValueError(f"layer {i}: unknown mixer {kind!r}")
        x = x + rms_norm(y, weights[f"l{i}.norm1"], eps)
        if layer.get("mlp") is not None:
            f = gated_feed_forward(x, weights[f"l{i}.mlp.gate"], weights[f"l{i}.mlp.up"], weights[f"l{i}.mlp.down"])
            x = x + rms_norm(f, weights[f"l{i}.norm2"], eps)
        after.append(x)
    z = rms_norm(x, weights["final.norm"], eps) @ weights["head"].T
    cap = config.get("logit_softcap")
    if cap:
        z = capped_logits(z, cap)
    return (z, torch.stack(after)) if return_layers else z
