"""A plain, slow implementation of the Taluvik decoder: whole sequences, no cache, no state carried
between calls, one function per mechanism, only ``torch`` tensor arithmetic.  It shares no code with
``torchllms_amd``; the tests compare the engine against it.

Conventions: one sequence at a time; activations are [S, ...]; ``weights`` maps the checkpoint's own
tensor names (``l3.mix.q``, ``l3.mlp.up``, ``final.norm.b`` ...) to tensors; ``config`` is the
dictionary of config.json.  Everything is computed in the dtype the weights are given in (the tests
pass 32-bit or 64-bit copies), so the functions state the formulas and nothing about rounding.
"""

from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch


# ----------------------------------------------------------------------------- small functions
def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z: torch.Tensor) -> torch.Tensor:
    return z / (1.0 + torch.exp(-z))


def softplus(z: torch.Tensor) -> torch.Tensor:
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


def layer_norm(x: torch.Tensor, w: torch.Tensor, b: torch.Tensor, eps: float) -> torch.Tensor:
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w + b


def rms_unit(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x over its root mean square along the last axis, eps under the root."""
    return x / torch.sqrt((x ** 2).mean(-1, keepdim=True) + eps)


def gated_feed_forward(h: torch.Tensor, gate: torch.Tensor, up: torch.Tensor, down: torch.Tensor) -> torch.Tensor:
    return (gelu_tanh(h @ gate.T) * (h @ up.T)) @ down.T


def causal_conv(x: torch.Tensor, taps: torch.Tensor, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x [S, C]; taps [C, K], the last column multiplies the current token, the one before it the
    previous token, and so on; inputs before the sequence's start are zero."""
    S, C = x.shape
    K = taps.shape[1]
    out = torch.zeros_like(x)
    for j in range(K):
        back = K - 1 - j  # how many tokens before the current one column j reads
        if back < S:
            out[back:] += taps[:, j] * x[: S - back]
    if bias is not None:
        out = out + bias
    return out


# ----------------------------------------------------------------------------- rotary positions
def rotary_frequencies(dims: int, base: float, scaling: Optional[dict]) -> List[float]:
    """One frequency per rotated pair, in double precision, with the long wavelengths stretched when
    ``scaling`` (factor, low, high, original) is given."""
    out = []
    for i in range(dims // 2):
        f = base ** (-2.0 * i / dims)
        if scaling:
            factor, low, high, original = scaling["factor"], scaling["low"], scaling["high"], scaling["original"]
            wavelength = 2.0 * math.pi / f
            if wavelength < original / high:
                pass
            elif wavelength > original / low:
                f = f / factor
            else:
                s = (original / wavelength - low) / (high - low)
                f = (1.0 - s) * f / factor + s * f
        out.append(f)
    return out


def rotate(x: torch.Tensor, positions: torch.Tensor, freqs: List[float], dims: int) -> torch.Tensor:
    """x [S, H, d]: channel i < dims/2 is paired with channel i + dims/2; channels from ``dims`` on pass."""
    half = dims // 2
    ang = positions.to(x.dtype)[:, None] * torch.tensor(freqs, dtype=x.dtype)[None, :]  # [S, half]
    cos, sin = ang.cos()[:, None, :], ang.sin()[:, None, :]
    a, b = x[..., :half], x[..., half:dims]
    out = x.clone()
    out[..., :half] = a * cos - b * sin
    out[..., half:dims] = b * cos + a * sin
    return out


# ----------------------------------------------------------------------------- mixers
def attention_scores_to_output(q, k, v, scale, softcap, chunk, sink, positions):
    """q [S, d], k [S, d], v [S, dv] of one head; ``positions`` [S] absolute.  Token i reads token
    j <= i of its own chunk of ``chunk`` positions; the softmax has one more term exp(sink) in its
    denominator that carries no value."""
    s = (q @ k.T) * scale
    s = softcap * torch.tanh(s / softcap)
    pi, pj = positions[:, None], positions[None, :]
    seen = (pj <= pi) & (torch.div(pj, chunk, rounding_mode="floor") == torch.div(pi, chunk, rounding_mode="floor"))
    s = s.masked_fill(~seen, float("-inf"))
    m = torch.clamp(s.max(dim=-1, keepdim=True).values, min=float(sink))
    e = torch.exp(s - m)
    denom = e.sum(dim=-1, keepdim=True) + torch.exp(sink - m)
    return (e / denom) @ v


def attention_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: dict, eps: float,
                    positions: torch.Tensor) -> torch.Tensor:
    S = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w[p + "q"].T).view(S, H, d)
    k = (h @ w[p + "k"].T).view(S, G, d)
    v = (h @ w[p + "v"].T).view(S, G, dv)
    rot = m["rot"]
    freqs = rotary_frequencies(rot["dims"], rot["base"], rot.get("scaling"))
    q = rms_unit(rotate(q, positions, freqs, rot["dims"]), eps)
    k = rms_unit(rotate(k, positions, freqs, rot["dims"]), eps)
    heads = []
    for head in range(H):
        g = head // (H // G)
        heads.append(attention_scores_to_output(q[:, head], k[:, g], v[:, g], m["scale"], m["softcap"],
                                                m["mask"]["size"], w[p + "sink"][head], positions))
    return torch.cat(heads, dim=-1) @ w[p + "o"].T


def delta_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: dict, eps: float) -> torch.Tensor:
    S = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(causal_conv(h @ w[p + "q"].T, w[p + "q.conv"])).view(S, G, d)
    k = silu(causal_conv(h @ w[p + "k"].T, w[p + "k.conv"])).view(S, G, d)
    v = silu(causal_conv(h @ w[p + "v"].T, w[p + "v.conv"])).view(S, H, dv)
    q = q / torch.sqrt((q ** 2).sum(-1, keepdim=True) + 1e-6) * d ** -0.5
    k = k / torch.sqrt((k ** 2).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ w[p + "b"].T)  # [S, H]
    decay = torch.exp(-torch.exp(w[p + "A_log"]) * softplus(h @ w[p + "a"].T + w[p + "dt_bias"]))  # [S, H]
    gate = silu(h @ w[p + "g"].T).view(S, H, dv)
    rep = H // G  # head h reads q/k head h // rep
    qh, kh = q.repeat_interleave(rep, dim=1), k.repeat_interleave(rep, dim=1)  # [S, H, d]
    out = torch.zeros((S, H, dv), dtype=h.dtype)
    state = torch.zeros((H, d, dv), dtype=h.dtype)
    for t in range(S):
        state = decay[t][:, None, None] * state
        u = beta[t][:, None] * (v[t] - torch.einsum("hij,hi->hj", state, kh[t]))
        state = state + torch.einsum("hi,hj->hij", kh[t], u)
        out[t] = torch.einsum("hij,hi->hj", state, qh[t])
    out = rms_unit(out, eps) * w[p + "norm"] * gate
    return out.reshape(S, H * dv) @ w[p + "o"].T


def mamba_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: dict) -> torch.Tensor:
    S = h.shape[0]
    inner, N, R = m["inner"], m["state"], m["dt_rank"]
    xz = h @ w[p + "in"].T
    x, z = xz[:, :inner], xz[:, inner:]
    x = silu(causal_conv(x, w[p + "conv"], w[p + "conv.b"]))
    proj = x @ w[p + "x"].T
    dt_in, B, C = proj[:, :R], proj[:, R : R + N], proj[:, R + N : R + 2 * N]
    dt = softplus(dt_in @ w[p + "dt"].T + w[p + "dt.b"])  # [S, inner]
    A = -torch.exp(w[p + "A_log"])  # [inner, N]
    state = torch.zeros((inner, N), dtype=h.dtype)
    ys = []
    for t in range(S):
        state = torch.exp(dt[t][:, None] * A) * state + (dt[t] * x[t])[:, None] * B[t][None, :]
        ys.append(state @ C[t] + w[p + "D"] * x[t])
    y = torch.stack(ys) * silu(z)
    return y @ w[p + "o"].T


# ----------------------------------------------------------------------------- the model
def forward(config: dict, weights: Dict[str, torch.Tensor], tokens, return_layers: bool = False):
    """Logits [S, vocab] of one sequence from position 0 (and, asked for, the residual stream after
    every layer run, [runs, S, width])."""
    w = weights
    eps = config["norm"]["eps"]
    mult = config["residual_mult"]
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    positions = torch.arange(tokens.numel())
    x = w["embed"][tokens] * config["embedding"]["scale"]
    streams = []
    for i, layer in enumerate(config["layers"]):
        owner = layer.get("weights_of", i)
        p = f"l{owner}."
        h = layer_norm(x, w[p + "norm1"], w[p + "norm1.b"], eps)
        kind, m = layer["type"], layer["mixer"]
        if kind == "attention":
            mixed = attention_mixer(h, w, p + "mix.", m, eps, positions)
        elif kind == "delta":
            mixed = delta_mixer(h, w, p + "mix.", m, eps)
        elif kind == "mamba1":
            mixed = mamba_mixer(h, w, p + "mix.", m)
        else:
            raise ValueError(f"layer {i}: unknown mixer {kind!r}")
        if layer.get("mlp") is not None:
            if layer["mlp"]["kind"] != "dense":
                raise ValueError(f"layer {i}: unknown feed-forward {layer['mlp']['kind']!r}")
            mixed = mixed + gated_feed_forward(h, w[p + "mlp.gate"], w[p + "mlp.up"], w[p + "mlp.down"])
        x = x + mult * mixed
        streams.append(x)
    logits = layer_norm(x, w["final.norm"], w["final.norm.b"], eps) @ w["head"].T
    if return_layers:
        return logits, torch.stack(streams)
    return logits
