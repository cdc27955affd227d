"""Kernels of layers that norm their branches on the way into a 32-bit residual stream and of attention
layers that prepare their heads before the scores: weighted RMS norm per head, rotation of a part of the
head, a query factor that grows with the logarithm of the position, values mixed with an earlier layer's,
gates on the heads' outputs, the packing of queries and outputs of attention through a latent, a cap on
the logits."""

from __future__ import annotations

from typing import Optional

import torch

from .base import KernelError, _gpu, _i32, _ptr, _stream, check, core, dtype_code

#: the widest head ``head_prepare`` takes (sixteen channels a lane)
HEAD_PREPARE_MAX_DIM = 1024


def _f32_vector(v: Optional[torch.Tensor], n: int, what: str) -> None:
    if v is not None and (not v.is_cuda or v.dtype != torch.float32 or v.numel() != n or not v.is_contiguous()):
        raise KernelError(f"{what} must be a contiguous float32 GPU vector of {n} entries")


def head_prepare(
    rows: torch.Tensor,
    n_q_heads: int,
    n_kv_heads: int,
    head_dim: int,
    v_head_dim: int,
    bias: Optional[torch.Tensor] = None,
    q_norm: Optional[torch.Tensor] = None,
    k_norm: Optional[torch.Tensor] = None,
    norm_dims: int = 0,
    eps: float = 0.0,
    cos_sin: Optional[torch.Tensor] = None,
    rot_offset: int = 0,
    rot_dims: int = 0,
    pairing: int = 0,
    positions: Optional[torch.Tensor] = None,
    temp_coef: float = 0.0,
    temp_every: int = 1,
    v_first: Optional[torch.Tensor] = None,
    v_mix: Optional[torch.Tensor] = None,
    k_pages: Optional[torch.Tensor] = None,
    v_pages: Optional[torch.Tensor] = None,
    slot_mapping: Optional[torch.Tensor] = None,
    page_size: int = 0,
) -> None:
    """Prepare the heads of ``rows`` [n, >= (Hq + Hkv) * dk + Hkv * dv] = query heads | key heads | value
    heads | anything else, in place and into the cache:

    * every head first takes its ``bias`` (one entry per column of the heads, in the rows' dtype; None: none);
    * query and key heads: the first ``norm_dims`` channels are divided by their root mean square
      (``eps`` under the root) and multiplied by ``q_norm`` / ``k_norm`` (32-bit vectors; None: no norm);
      then channels ``rot_offset .. rot_offset + rot_dims`` are rotated by ``cos_sin`` (the step's table);
      then queries are multiplied by ``1 + temp_coef * ln(floor((p + 1) / temp_every) + 1)``;
    * value heads (``v_head_dim`` 0: the rows hold none): with ``v_first`` [n, Hkv * dv] (a view will do)
      and ``v_mix`` (a 32-bit scalar on the device) they become ``(1 - v_mix) v + v_mix v_first``;
    * queries and mixed values are written back, keys and values go to their pages at ``slot_mapping``
      (keys back in place when there are no pages)."""
    _gpu(rows, bias, q_norm, k_norm, cos_sin, positions, v_first, v_mix, k_pages, v_pages, slot_mapping)
    _i32(positions, "positions")
    _i32(slot_mapping, "slot_mapping")
    n = rows.shape[0]
    width = (n_q_heads + n_kv_heads) * head_dim + n_kv_heads * v_head_dim
    if rows.dim() != 2 or rows.stride(1) != 1 or rows.shape[1] < width:
        raise KernelError(f"head_prepare: rows must be row-major with at least {width} columns, got {tuple(rows.shape)}")
    if bias is not None and (bias.dim() != 1 or bias.numel() != width or bias.dtype != rows.dtype or not bias.is_contiguous()):
        raise KernelError(f"head_prepare: bias must be a contiguous vector of {width} entries of the rows' dtype")
    if q_norm is not None or k_norm is not None:
        _f32_vector(q_norm, norm_dims, "head_prepare: q_norm")
        _f32_vector(k_norm, norm_dims, "head_prepare: k_norm")
    if rot_dims > 0 and (cos_sin is None or cos_sin.dtype != torch.float32 or tuple(cos_sin.shape) != (n, rot_dims // 2, 2)
                         or not cos_sin.is_contiguous()):
        raise KernelError(f"head_prepare: cos_sin must be contiguous float32 [{n}, {rot_dims // 2}, 2]")
    if temp_coef != 0.0 and (positions is None or positions.numel() != n):
        raise KernelError("head_prepare: a query factor needs one position per token")
    vf_stride = 0
    if v_first is not None:
        if (v_first.dim() != 2 or v_first.shape != (n, n_kv_heads * v_head_dim) or v_first.stride(1) != 1 or v_first.dtype != rows.dtype):
            raise KernelError(f"head_prepare: v_first must be row-major [{n}, {n_kv_heads * v_head_dim}] of the rows' dtype")
        if v_mix is None or v_mix.dtype != torch.float32 or v_mix.numel() != 1:
            raise KernelError("head_prepare: v_mix must be one float32 number on the device")
        vf_stride = v_first.stride(0)
    if k_pages is not None:
        if slot_mapping is None or slot_mapping.numel() != n:
            raise KernelError("head_prepare: pages need one slot per token")
        wanted = [(k_pages, head_dim)] + ([(v_pages, v_head_dim)] if v_head_dim > 0 else [])
        for pg, d in wanted:
            if pg is None or pg.dim() != 4 or pg.shape[1:] != (n_kv_heads, page_size, d) or pg.dtype != rows.dtype or not pg.is_contiguous():
                raise KernelError(f"head_prepare: pages must be contiguous [pages, {n_kv_heads}, {page_size}, {d}] of {rows.dtype}")
    check(
        core().tl_head_prepare(
            rows.data_ptr(), rows.stride(0), n, n_q_heads, n_kv_heads, head_dim, v_head_dim, _ptr(bias), _ptr(q_norm), _ptr(k_norm),
            int(norm_dims), float(eps), _ptr(cos_sin), int(rot_offset), int(rot_dims), int(pairing), _ptr(positions),
            float(temp_coef), int(temp_every), _ptr(v_first), vf_stride, _ptr(v_mix), _ptr(k_pages),
            _ptr(v_pages) if v_head_dim > 0 else None, _ptr(slot_mapping), int(page_size), dtype_code(rows.dtype), _stream(),
        )
    )


def branch_norm_add(stream: torch.Tensor, y: torch.Tensor, weight: torch.Tensor, eps: float, want_rows: bool = True):
    """``stream += y / sqrt(mean(y^2) + eps) * weight`` row by row, in place, all in 32-bit (``stream`` float32
    [n, hidden], ``weight`` float32).  Returns the new rows in ``y``'s dtype for whoever reads them next (the
    stream itself when that is float32; None with ``want_rows`` False)."""
    _gpu(stream, y, weight)
    if stream.dim() != 2 or stream.dtype != torch.float32 or not stream.is_contiguous():
        raise KernelError("branch_norm_add: the stream must be a contiguous float32 [rows, hidden] tensor")
    n, hidden = stream.shape
    if y.shape != stream.shape or not y.is_contiguous():
        raise KernelError("branch_norm_add: the branch must have the stream's shape")
    _f32_vector(weight, hidden, "branch_norm_add: weight")
    rows = None
    if want_rows and y.dtype != torch.float32:
        rows = torch.empty_like(y)
    check(core().tl_branch_norm_add(stream.data_ptr(), y.data_ptr(), weight.data_ptr(), _ptr(rows), n, hidden, float(eps),
                                    dtype_code(y.dtype), _stream()))
    if not want_rows:
        return None
    return stream if y.dtype == torch.float32 else rows


def rmsnorm_columns(x: torch.Tensor, weight: torch.Tensor, eps: float, out_dtype: torch.dtype,
                    rows: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``x / sqrt(mean(x^2) + eps) * weight`` row by row with one rounding at the end: ``x`` a row-major matrix
    (some columns of a wider one will do) of float32 or of ``out_dtype``, ``weight`` float32, optionally of
    the rows ``rows`` only; the result has ``out_dtype`` and may be written into ``out`` (row-major)."""
    _gpu(x, weight, rows, out)
    _i32(rows, "rows")
    if x.dim() != 2 or x.stride(1) != 1:
        raise KernelError("rmsnorm_columns: x must be a row-major matrix")
    width = x.shape[1]
    _f32_vector(weight, width, "rmsnorm_columns: weight")
    if x.dtype not in (torch.float32, out_dtype):
        raise KernelError(f"rmsnorm_columns: rows of {x.dtype} with results of {out_dtype}")
    n = x.shape[0] if rows is None else rows.numel()
    if out is None:
        out = torch.empty((n, width), dtype=out_dtype, device=x.device)
    elif out.shape != (n, width) or out.stride(1) != 1 or out.dtype != out_dtype:
        raise KernelError(f"rmsnorm_columns: out must be row-major [{n}, {width}] of {out_dtype}")
    check(core().tl_rmsnorm_columns(x.data_ptr(), x.stride(0), dtype_code(x.dtype), _ptr(rows), weight.data_ptr(),
                                    out.data_ptr(), out.stride(0), dtype_code(out_dtype), n, width, float(eps), _stream()))
    return out


def sigmoid_gate_(x: torch.Tensor, gate: torch.Tensor, per: int = 1) -> torch.Tensor:
    """In place ``x[t, c] *= sigmoid(gate[t, c // per])``: ``per`` 1 gates channel by channel, the head size
    gates head by head.  Both row-major (views of some columns will do), one dtype."""
    _gpu(x, gate)
    if x.dim() != 2 or gate.dim() != 2 or x.stride(1) != 1 or gate.stride(1) != 1 or x.dtype != gate.dtype or x.shape[0] != gate.shape[0]:
        raise KernelError("sigmoid_gate: x and gate must be row-major matrices of one dtype with the same rows")
    if per <= 0 or gate.shape[1] * per != x.shape[1]:
        raise KernelError(f"sigmoid_gate: {gate.shape[1]} gates of {per} channels do not cover {x.shape[1]} columns")
    check(core().tl_sigmoid_gate(x.data_ptr(), x.stride(0), gate.data_ptr(), gate.stride(0), x.shape[0], x.shape[1], int(per),
                                 dtype_code(x.dtype), _stream()))
    return x


def pack_heads(a: torch.Tensor, b: torch.Tensor, b_head: int, b_offset: int, nb: int) -> torch.Tensor:
    """``out[t, h] = a[h, t, :] | b[t, h * b_head + b_offset : ... + nb]`` as [n, heads * (na + nb)]: the two
    parts of every head's query against a latent (``a`` [heads, n, na] contiguous, ``b`` row-major)."""
    _gpu(a, b)
    if a.dim() != 3 or not a.is_contiguous() or b.dim() != 2 or b.stride(1) != 1 or a.dtype != b.dtype or a.shape[1] != b.shape[0]:
        raise KernelError("pack_heads: a must be contiguous [heads, n, na] and b row-major [n, ...] of the same dtype")
    heads, n, na = a.shape
    if b_offset < 0 or nb < 0 or b_offset + nb > b_head or heads * b_head > b.shape[1]:
        raise KernelError("pack_heads: the second part does not lie inside b's heads")
    out = torch.empty((n, heads * (na + nb)), dtype=a.dtype, device=a.device)
    check(core().tl_pack_heads(a.data_ptr(), na, b.data_ptr(), b.stride(0), int(b_head), int(b_offset), int(nb), out.data_ptr(), n,
                               heads, dtype_code(a.dtype), _stream()))
    return out


def unpack_heads_gate(a: torch.Tensor, gate: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``out[t, h * d + j] = a[h, t, j] * sigmoid(gate[t, h])`` as [n, heads * d] (``gate`` None: no gate)."""
    _gpu(a, gate)
    if a.dim() != 3 or not a.is_contiguous():
        raise KernelError("unpack_heads_gate: a must be contiguous [heads, n, d]")
    heads, n, d = a.shape
    if gate is not None and (gate.dim() != 2 or gate.shape != (n, heads) or gate.stride(1) != 1 or gate.dtype != a.dtype):
        raise KernelError(f"unpack_heads_gate: gate must be row-major [{n}, {heads}] of a's dtype")
    out = torch.empty((n, heads * d), dtype=a.dtype, device=a.device)
    check(core().tl_unpack_heads_gate(a.data_ptr(), out.data_ptr(), _ptr(gate), gate.stride(0) if gate is not None else 0, n, heads, d,
                                      dtype_code(a.dtype), _stream()))
    return out


def softcap_(z: torch.Tensor, cap: float) -> torch.Tensor:
    """In place ``z = cap * tanh(z / cap)`` on contiguous float32 values."""
    _gpu(z)
    if z.dtype != torch.float32 or not z.is_contiguous():
        raise KernelError("softcap: contiguous float32 values")
    check(core().tl_softcap(z.data_ptr(), z.numel(), float(cap), _stream()))
    return z
