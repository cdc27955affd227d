"""Mixers that carry a state of fixed size per request instead of keys and values: the selective scan
of a diagonal state-space layer and the gated delta rule, both behind a short causal convolution.

Everything such a mixer keeps for a request lies in one 32-bit row of its ``StateView`` (the
convolution's history first, then the recurrence's state); rows are zeroed when a request is admitted,
and a step reads and writes the rows of its requests' slots (``ctx.slot_ids``), so a sequence may be
cut into steps anywhere and batched with anything."""

from __future__ import annotations

from typing import Dict, Optional

import torch

from ..kernels import ops
from .base import MIXERS, Mixer, ParamSpec, StateNeed


@MIXERS.register("selective_scan")
class SelectiveScan(Mixer):
    """``[x | z] = W_in h``; x through a causal convolution over ``conv`` taps (with bias) and silu;
    ``[dt | B | C] = W_x x``; ``dt <- softplus(W_dt dt + b_dt)`` per channel; ``A = -exp(A_log)``;
    ``S[c, n] <- exp(dt_c A[c, n]) S[c, n] + dt_c x_c B_n``; ``y_c = sum_n S[c, n] C_n + D_c x_c``;
    the output is ``W_o (y * silu(z))``.  Step sizes, decays and the state are 32-bit."""

    graph_safe = True

    def __init__(self, hidden_size: int, inner_size: int, state_size: int, dt_rank: int, conv_taps: int):
        for name, v in (("inner_size", inner_size), ("state_size", state_size), ("dt_rank", dt_rank), ("conv_taps", conv_taps)):
            if not isinstance(v, int) or v <= 0:
                raise ValueError(f"selective_scan: {name} must be a positive integer, got {v!r}")
        self.hidden_size, self.inner, self.n_state, self.dt_rank, self.taps = hidden_size, inner_size, state_size, dt_rank, conv_taps
        self.w_in = self.w_x = self.w_dt = self.w_o = None
        self.conv_w = self.conv_b = self.dt_b = self.A = self.D = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        d, c, n, r = self.hidden_size, self.inner, self.n_state, self.dt_rank
        return {
            "in": ParamSpec((2 * c, d)),
            "conv": ParamSpec((c, self.taps), init="conv"),
            "conv.b": ParamSpec((c,), init="zeros"),
            "x": ParamSpec((r + 2 * n, c)),
            "dt": ParamSpec((c, r), init="wide"),
            "dt.b": ParamSpec((c,), init="zeros"),
            "A_log": ParamSpec((c, n), init="zeros"),
            "D": ParamSpec((c,), init="ones"),
            "o": ParamSpec((d, c)),
        }

    def check_sizes(self, dtype: torch.dtype) -> None:
        if self.n_state > 256:
            raise ValueError(f"selective_scan: {self.n_state} states a channel; the kernel takes up to 256")
        if self.taps > 64:
            raise ValueError(f"selective_scan: a convolution over {self.taps} taps; the kernel takes up to 64")

    def cache_need(self):
        return StateNeed(shape=((self.taps - 1) * self.inner + self.inner * self.n_state,), dtype="float32")

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.w_in = tensors["in"].contiguous()
        self.w_x = tensors["x"].contiguous()
        self.w_dt = tensors["dt"].contiguous()
        self.w_o = tensors["o"].contiguous()
        self.conv_w = tensors["conv"].float().t().contiguous()  # [taps, channels]: a tap's weights lie side by side
        self.conv_b = tensors["conv.b"].float().contiguous()
        self.dt_b = tensors["dt.b"].float().contiguous()
        self.A = (-torch.exp(tensors["A_log"].float())).contiguous()
        self.D = tensors["D"].float().contiguous()

    def linear_weights(self):
        return [self.w_in, self.w_x, (self.w_dt, "plain", torch.float32), (self.w_o, "sum")]

    def forward(self, x, ctx, cache):
        c, n, r = self.inner, self.n_state, self.dt_rank
        state = cache.tensor
        x = ops.resolved(x)
        xz = ops.linear(x, self.w_in)
        xc = ops.causal_conv(xz[:, :c], self.conv_w, self.conv_b, state, 0, ctx.token_seq, ctx.qo_indptr, ctx.slot_ids)
        proj = ops.linear(xc, self.w_x)
        dt_pre = ops.linear(proj[:, :r], self.w_dt, out_dtype=torch.float32)
        # a long prompt's recurrence is cut into segments that run side by side; in 32-bit every row is
        # walked in one piece, so that no bit depends on how the prompt was cut into steps
        segments = None
        if x.dtype != torch.float32 and ctx.host.max_q_len >= ops.SCAN_SEGMENTS_FROM:
            segments = ctx.scratch.get("scan_segments")
            if segments is None:
                segments = ctx.scratch["scan_segments"] = ops.ScanSegments(ctx.host.qo_indptr, x.device)
        y = ops.selective_scan(xc, dt_pre, proj, r, r + n, xz[:, c:], self.dt_b, self.A, self.D, state, (self.taps - 1) * c,
                               ctx.qo_indptr, ctx.slot_ids, segments=segments)
        return ops.linear_to_sum(y, self.w_o)


@MIXERS.register("gated_delta")
class GatedDelta(Mixer):
    """The gated delta rule.  ``q, k`` (``num_key_heads`` heads of ``head_dim``) and ``v`` (``num_heads``
    heads of ``v_head_dim``) are projections of the input, each through a causal convolution over
    ``conv_taps`` taps (no bias) and silu; head h reads q/k head ``h // (num_heads / num_key_heads)``.
    q and k become unit vectors (q also times head_dim^-1/2); ``beta = sigmoid(W_b h)``;
    ``decay = exp(-exp(A_log) softplus(W_a h + dt_bias))`` per head.  Per head and token
    ``S <- decay S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q``; o is divided by its root mean
    square over v_head_dim, multiplied by the weight ``norm`` and by ``silu(W_g h)``, then projected by
    W_o.  Gates, decays, unit norms and the state are 32-bit."""

    graph_safe = True

    def __init__(self, hidden_size: int, num_heads: int, num_key_heads: int, head_dim: int, v_head_dim: int, conv_taps: int,
                 norm_eps: float):
        if num_heads % num_key_heads:
            raise ValueError(f"gated_delta: {num_heads} heads are not a multiple of {num_key_heads} key heads")
        self.hidden_size, self.H, self.G, self.dk, self.dv, self.taps = hidden_size, num_heads, num_key_heads, head_dim, v_head_dim, conv_taps
        self.norm_eps = float(norm_eps)
        self.w_all = self.w_o = self.conv_w = self.A_log = self.dt_bias = self.norm_w = None

    @property
    def conv_channels(self) -> int:
        return 2 * self.G * self.dk + self.H * self.dv

    def param_specs(self) -> Dict[str, ParamSpec]:
        d, qk, v = self.hidden_size, self.G * self.dk, self.H * self.dv
        return {
            "q": ParamSpec((qk, d)), "q.conv": ParamSpec((qk, self.taps), init="conv"),
            "k": ParamSpec((qk, d)), "k.conv": ParamSpec((qk, self.taps), init="conv"),
            "v": ParamSpec((v, d)), "v.conv": ParamSpec((v, self.taps), init="conv"),
            "b": ParamSpec((self.H, d)), "a": ParamSpec((self.H, d)),
            "A_log": ParamSpec((self.H,), init="zeros"), "dt_bias": ParamSpec((self.H,), init="zeros"),
            "norm": ParamSpec((self.dv,), init="ones"),
            "g": ParamSpec((v, d)), "o": ParamSpec((d, v)),
        }

    def check_sizes(self, dtype: torch.dtype) -> None:
        if self.dk > 256:
            raise ValueError(f"gated_delta: keys of {self.dk} channels; the kernel takes up to 256 (values: any number)")
        if self.taps > 64:
            raise ValueError(f"gated_delta: a convolution over {self.taps} taps; the kernel takes up to 64")

    def cache_need(self):
        return StateNeed(shape=((self.taps - 1) * self.conv_channels + self.H * self.dv * self.dk,), dtype="float32")

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        # one projection [q | k | v | output gate | write strength | decay]: a single product per step
        self.w_all = torch.cat([tensors[n] for n in ("q", "k", "v", "g", "b", "a")], dim=0).contiguous()
        self.conv_w = torch.cat([tensors[n + ".conv"] for n in ("q", "k", "v")], dim=0).float().t().contiguous()  # [taps, channels]
        self.w_o = tensors["o"].contiguous()
        self.A_log = tensors["A_log"].float().contiguous()
        self.dt_bias = tensors["dt_bias"].float().contiguous()
        self.norm_w = tensors["norm"].float().contiguous()

    def linear_weights(self):
        return [self.w_all, (self.w_o, "sum")]

    def forward(self, x, ctx, cache):
        c, hv = self.conv_channels, self.H * self.dv
        state = cache.tensor
        proj = ops.linear(ops.resolved(x), self.w_all)
        qkv = ops.causal_conv(proj[:, :c], self.conv_w, None, state, 0, ctx.token_seq, ctx.qo_indptr, ctx.slot_ids)
        y = ops.gated_delta(qkv, proj, c, c + hv, c + hv + self.H, self.A_log, self.dt_bias, self.norm_w, self.norm_eps, state,
                            (self.taps - 1) * c, ctx.qo_indptr, ctx.slot_ids, self.H, self.G, self.dk, self.dv)
        return ops.linear_to_sum(y, self.w_o)
