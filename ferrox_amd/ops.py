"""Python faces of the HIP kernels: argument checks, then one ctypes call.

Tensors live on the GPU; the kernels run on torch's current stream.  There is no
other implementation behind these functions: a tensor on the CPU, or a missing
library, raises.
"""
from __future__ import annotations

import ctypes
from ctypes import c_float, c_int, c_long, c_void_p

import math

import torch

from .csrc.build import load_library

FX_F32, FX_BF16 = 0, 1
EPI_STORE, EPI_STORE_F32, EPI_RESID, EPI_GATED = 0, 1, 2, 3
# what the gate of a gated product goes through (EPI_GATED stores activation(gate) * up); ACT_* in csrc/gemm.hip
ACTIVATIONS = {"silu": 0, "gelu_tanh": 1, "gelu": 2, "relu": 3, "swiglu_clamped": 4}
# what a stored product (EPI_STORE) may go through on its way out, the activation of a feed-forward without a
# gate; SACT_* in csrc/gemm.hip
STORED_ACTIVATIONS = {None: 0, "relu2": 1, "relu": 2, "silu": 3, "gelu_tanh": 4}
GATE_SOFTMAX, GATE_SIGMOID = 0, 1
ROPE_NEOX, ROPE_INTERLEAVED = 0, 1


class KernelError(RuntimeError):
    pass


def dtype_code(dt: torch.dtype) -> int:
    if dt == torch.float32:
        return FX_F32
    if dt == torch.bfloat16:
        return FX_BF16
    raise KernelError(f"kernels take float32 and bfloat16 tensors, not {dt}")


def _p(t):
    if t is None:
        return None
    if not t.is_cuda:
        raise KernelError("kernel called with a tensor that is not on the GPU")
    return t.data_ptr()           # (a plain integer: ctypes turns it into the pointer argument itself)


# the current stream's handle, asked for before every launch: straight from the runtime's binding where this torch
# has it (a fifth of the host's time per launch went into the Stream object that the public call builds)
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_device_index = getattr(torch._C, "_cuda_getDevice", None)


def _stream():
    if _raw_stream is not None and _device_index is not None:
        return _raw_stream(_device_index())
    return torch.cuda.current_stream().cuda_stream


_sigs = {
    ("elementwise", "fx_embed"): [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_float, c_void_p, c_void_p, c_int],
    ("elementwise", "fx_layernorm"): [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_float, c_long],
    ("elementwise", "fx_gated_add"): [c_void_p, c_void_p, c_void_p, c_void_p, c_long],
    ("elementwise", "fx_gated_add_layernorm"): [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p,
                                                c_int, c_int, c_float],
    ("elementwise", "fx_temp_unit_kv_write"): [c_void_p, c_int, c_void_p, c_long, c_void_p, c_long, c_void_p, c_void_p, c_void_p,
                                               c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int,
                                               c_float, c_int, c_int, c_float],
    ("elementwise", "fx_latent_kv_write"): [c_void_p, c_int, c_void_p, c_long, c_void_p, c_int, c_float, c_void_p, c_void_p,
                                            c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p,
                                            c_float, c_void_p, c_long, c_void_p, c_float, c_void_p, c_long, c_int],
    ("elementwise", "fx_latent_q_rot"): [c_void_p, c_int, c_void_p, c_long, c_void_p, c_long, c_void_p, c_int, c_int, c_int,
                                         c_int, c_int, c_int, c_void_p, c_float],
    ("elementwise", "fx_span_norm_kv_write"): [c_void_p, c_int, c_void_p, c_long, c_void_p, c_long, c_void_p, c_void_p, c_int,
                                               c_float, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_int, c_int,
                                               c_int, c_int, c_int],
    ("elementwise", "fx_rmsnorm"): [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_float, c_long],
    ("elementwise", "fx_rope_kv_write"): [c_void_p, c_int, c_void_p, c_int, c_void_p, c_int, c_void_p, c_int,
                                          c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p,
                                          c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_int],
    ("elementwise", "fx_rmsnorm_add"): [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_float],
    ("elementwise", "fx_moe_combine_identity"): [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int,
                                                 c_int, c_int, c_int, c_int, c_void_p, c_int, c_float],
    ("recurrent", "fx_short_conv"): [c_void_p, c_void_p, c_int, c_long, c_void_p, c_int, c_long, c_void_p, c_int, c_int, c_void_p,
                                     c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_int, c_int],
    ("recurrent", "fx_gated_outer"): [c_void_p, c_void_p, c_long, c_void_p, c_long, c_void_p, c_long, c_void_p, c_int, c_void_p,
                                      c_void_p, c_long, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int,
                                      c_float],
    ("recurrent", "fx_exp_gate_scan"): [c_void_p, c_void_p, c_long, c_void_p, c_long, c_float, c_void_p, c_void_p, c_void_p,
                                        c_void_p, c_void_p, c_void_p, c_int, c_int],
    ("recurrent", "fx_rglru_gates"): [c_void_p, c_void_p, c_long, c_void_p, c_void_p, c_void_p, c_int, c_float,
                                      c_void_p, c_void_p, c_int, c_int, c_int],
    ("recurrent", "fx_rglru_scan"): [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_long, c_void_p, c_long, c_void_p, c_void_p,
                                     c_void_p, c_int, c_int, c_int],
    ("recurrent", "fx_delta_prepare"): [c_void_p, c_void_p, c_long, c_void_p, c_long, c_void_p, c_long, c_void_p, c_long,
                                        c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                        c_int, c_int, c_int, c_int, c_int],
    ("recurrent", "fx_channel_delta"): [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_long, c_void_p, c_long,
                                        c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int],
    ("recurrent", "fx_small_rows_pair"): [c_void_p, c_void_p, c_long, c_void_p, c_void_p, c_long, c_int, c_int,
                                          c_void_p, c_long, c_void_p, c_void_p, c_long, c_int, c_int, c_int],
    ("recurrent", "fx_small_rows_parts"): [c_void_p, c_void_p, c_long, c_void_p, c_void_p, c_int, c_int, c_int, c_int],
    ("recurrent", "fx_gated_head_norm"): [c_void_p, c_int, c_void_p, c_long, c_void_p, c_long, c_void_p, c_int, c_int, c_void_p,
                                          c_long, c_int, c_int, c_int, c_float, c_int, c_void_p, c_void_p],
    ("elementwise", "fx_head_norm_kv_write"): [c_void_p, c_int, c_void_p, c_long, c_void_p, c_long, c_void_p, c_int,
                                               c_void_p, c_void_p, c_int, c_float, c_void_p, c_void_p, c_void_p, c_int,
                                               c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int],
    ("elementwise", "fx_residual_add"): [c_void_p, c_int, c_void_p, c_void_p, c_long],
    ("elementwise", "fx_cast"): [c_void_p, c_int, c_void_p, c_int, c_void_p, c_long],
    ("elementwise", "fx_moe_combine"): [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                        c_int, c_int, c_int, c_int, c_void_p, c_int, c_void_p, c_int, c_void_p],
    ("elementwise", "fx_fill_u32"): [c_void_p, c_void_p, ctypes.c_uint, c_long],
    ("elementwise", "fx_feed_tokens"): [c_void_p, c_void_p, c_void_p, c_void_p, c_int],
    ("gemm", "fx_gemm"): [c_void_p, c_int, c_int, c_void_p, c_long, c_void_p, c_long, c_long, c_void_p, c_int,
                          c_void_p, c_long, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                          c_void_p, c_int, c_float, c_void_p, c_int, c_int, c_int, c_int, c_long, c_void_p, c_int, c_int, c_int,
                          c_float, c_float, c_void_p, c_void_p],
    ("gemm", "fx_qkv_rope"): [c_void_p, c_void_p, c_long, c_void_p, c_long, c_void_p, c_int, c_void_p, c_long, c_int, c_int,
                              c_void_p, c_int, c_float, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p,
                              c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p],
    ("attention", "fx_attn_tiles"): [c_void_p, c_int, c_void_p, c_long, c_void_p, c_long, c_void_p, c_void_p,
                                     c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p,
                                     c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_int, c_int,
                                     c_int, c_void_p, c_void_p, c_long, c_float, c_void_p, c_int],
    ("attention", "fx_attn_tile_queries"): [c_int, c_int, c_int],
    ("attention", "fx_attn_decode"): [c_void_p, c_int, c_void_p, c_long, c_void_p, c_long, c_void_p, c_void_p,
                                      c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int,
                                      c_int, c_int, c_int, c_int, c_int, c_float,
                                      c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int,
                                      c_int, c_void_p, c_void_p, c_long, c_float, c_void_p, c_int],
    ("moe", "fx_router_select"): [c_void_p, c_void_p, c_long, c_long, c_int, c_int, c_int, c_int, c_float, c_float, c_int,
                                  c_void_p, c_void_p, c_void_p, c_void_p],
    ("moe", "fx_router_select_align"): [c_void_p, c_void_p, c_long, c_int, c_int, c_int, c_int, c_float, c_float, c_int,
                                        c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p],
    ("moe", "fx_moe_front"): [c_void_p, c_void_p, c_long, c_void_p, c_int, c_float, c_void_p, c_void_p, c_int, c_int,
                              c_int, c_int, c_int, c_int, c_float, c_float, c_int] + [c_void_p] * 9 + [c_int],
    ("moe", "fx_moe_align"): [c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int],
    ("sampling", "fx_sample_greedy"): [c_void_p, c_void_p, c_long, c_int, c_int, c_void_p, c_void_p, c_void_p],
    ("sampling", "fx_sample"): [c_void_p, c_void_p, c_long, c_void_p, c_int, c_int] + [c_void_p] * 10,
}
_fns: dict = {}


def _fn(lib: str, name: str):
    key = (lib, name)
    entry = _fns.get(key)
    if entry is None:
        handle = load_library(lib)
        f = getattr(handle, name)
        f.argtypes = _sigs[key]
        f.restype = c_int
        entry = _fns[key] = (f, handle)
    return entry


def _call(lib: str, name: str, *args) -> None:
    f, handle = _fn(lib, name)
    if f(*args):
        raise KernelError(handle.fx_last_error().decode())


def _i32(t, what):
    if t is not None and t.dtype != torch.int32:
        raise KernelError(f"{what} must be int32, got {t.dtype}")
    return t


# ---------------------------------------------------------------------------
def embed(table: torch.Tensor, ids: torch.Tensor, out: torch.Tensor | None = None, scale: float = 1.0,
          position_table: torch.Tensor | None = None, positions: torch.Tensor | None = None) -> torch.Tensor:
    """h[t] = table[ids[t]] * scale (+ position_table[positions[t]], a learned vector per position) as float32."""
    V, H = table.shape
    T = ids.numel()
    if out is None:
        out = torch.empty((T, H), dtype=torch.float32, device=table.device)
    n_pos = 0
    if position_table is not None:
        if positions is None or positions.numel() < T or position_table.dtype != table.dtype or position_table.dim() != 2 \
                or position_table.shape[1] != H or not position_table.is_contiguous():
            raise KernelError(f"embed: a table of positions {tuple(position_table.shape)} ({position_table.dtype}) beside an "
                              f"embedding table {tuple(table.shape)} ({table.dtype}) needs the tokens' positions")
        n_pos = position_table.shape[0]
    _call("elementwise", "fx_embed", _stream(), dtype_code(table.dtype), _p(table), _p(_i32(ids, "ids")), _p(out), T, H, V,
          float(scale), _p(position_table), _p(_i32(positions, "positions")) if position_table is not None else None, n_pos)
    return out


def layernorm(h: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None, eps: float, out_dtype: torch.dtype,
              rows: torch.Tensor | None = None) -> torch.Tensor:
    """Rows of float32 `h` (all, or those in `rows`) through (x - mean) / sqrt(var + eps) * weight + bias, var the
    mean of the squared deviations, into `out_dtype`."""
    if h.dtype != torch.float32 or h.dim() != 2 or not h.is_contiguous():
        raise KernelError("layernorm reads contiguous float32 rows")
    H = h.shape[1]
    if weight.numel() != H or not weight.is_contiguous() or (bias is not None and (bias.numel() != H or bias.dtype != weight.dtype
                                                                                     or not bias.is_contiguous())):
        raise KernelError(f"layernorm: weight and bias must hold {H} elements of one type")
    R = h.shape[0] if rows is None else rows.numel()
    out = torch.empty((R, H), dtype=out_dtype, device=h.device)
    _call("elementwise", "fx_layernorm", _stream(), dtype_code(out_dtype), _p(h), _p(_i32(rows, "rows")), _p(weight), _p(bias),
          dtype_code(weight.dtype), _p(out), R, H, float(eps), h.stride(0))
    return out


def gated_add(h: torch.Tensor, y: torch.Tensor, gate_logits: torch.Tensor) -> None:
    """h += y * sigmoid(gate_logits), element by element (contiguous float32 tensors of one shape)."""
    for t in (h, y, gate_logits):
        if t.dtype != torch.float32 or not t.is_contiguous() or t.shape != h.shape:
            raise KernelError("gated_add wants contiguous float32 tensors of one shape")
    _call("elementwise", "fx_gated_add", _stream(), _p(h), _p(y), _p(gate_logits), h.numel())


GATED_ADD_NORM_MAX = 4096       # the widest row that the gated add keeps in registers for the norm behind it


def gated_add_layernorm(h: torch.Tensor, y: torch.Tensor, gate_logits: torch.Tensor, weight: torch.Tensor,
                        bias: torch.Tensor | None, eps: float, out_dtype: torch.dtype) -> torch.Tensor:
    """`gated_add(h, y, gate_logits)` and `layernorm(h, weight, bias, eps, out_dtype)` of the new rows in one launch
    (rows of up to GATED_ADD_NORM_MAX columns); returns the normed rows."""
    for t in (h, y, gate_logits):
        if t.dtype != torch.float32 or not t.is_contiguous() or t.shape != h.shape or t.dim() != 2:
            raise KernelError("gated_add_layernorm wants contiguous float32 matrices of one shape")
    T, H = h.shape
    if H > GATED_ADD_NORM_MAX or weight.numel() != H or not weight.is_contiguous() \
            or (bias is not None and (bias.numel() != H or bias.dtype != weight.dtype or not bias.is_contiguous())):
        raise KernelError(f"gated_add_layernorm: rows of {H} columns (up to {GATED_ADD_NORM_MAX}) with weight and bias of one type")
    out = torch.empty((T, H), dtype=out_dtype, device=h.device)
    _call("elementwise", "fx_gated_add_layernorm", _stream(), dtype_code(out_dtype), _p(h), _p(y), _p(gate_logits), _p(weight),
          _p(bias), dtype_code(weight.dtype), _p(out), T, H, float(eps))
    return out


def temp_unit_kv_write(qkv, q_out, positions, token_seq, block_table, k_pages, v_pages, n_heads: int, n_kv_heads: int,
                       head_dim: int, v_dim: int, block_size: int, n_gate: int = 0, temperature: tuple | None = None,
                       unit_values: bool = False, eps: float = 0.0) -> None:
    """For attention that rotates nothing: from the float32 product qkv [T, nh*hd | nkv*hd | nkv*vd | n_gate], q times the
    temperature of its position, 1 + coef ln(floor((p + 1) / every) + 1) with `temperature` = (coef, every), into
    q_out[:, :nh*hd]; the gate columns into q_out[:, nh*hd:]; k into its page; v, each head divided by its root mean
    square over v_dim (`unit_values`, eps inside the root), into its transposed page.  Pages None: nothing is cached."""
    T = qkv.shape[0]
    nh, nkv, hd, vd = int(n_heads), int(n_kv_heads), int(head_dim), int(v_dim)
    cols = (nh + nkv) * hd + nkv * vd + int(n_gate)
    _f32_rows(qkv, "temp_unit_kv_write: qkv", cols)
    if q_out.dim() != 2 or q_out.stride(1) != 1 or q_out.shape[0] < T or q_out.shape[1] < nh * hd + n_gate:
        raise KernelError(f"temp_unit_kv_write: q_out {tuple(q_out.shape)} for {T} rows of {nh * hd + n_gate}")
    if (k_pages is None) != (v_pages is None):
        raise KernelError("temp_unit_kv_write: key and value pages come together")
    if k_pages is not None and (tuple(k_pages.shape[1:]) != (nkv, block_size, hd) or tuple(v_pages.shape[1:]) != (nkv, vd, block_size)
                                or k_pages.dtype != q_out.dtype or v_pages.dtype != q_out.dtype):
        raise KernelError(f"temp_unit_kv_write: pages {tuple(k_pages.shape)}, {tuple(v_pages.shape)} for {nkv} heads of {hd} / {vd}")
    coef, every = (float(temperature[0]), int(temperature[1])) if temperature else (0.0, 1)
    if positions.numel() < T or token_seq.numel() < T:
        raise KernelError("temp_unit_kv_write: the step's index tensors are shorter than its tokens")
    _call("elementwise", "fx_temp_unit_kv_write", _stream(), dtype_code(q_out.dtype), _p(qkv), qkv.stride(0), _p(q_out),
          q_out.stride(0), _p(_i32(positions, "positions")), _p(_i32(token_seq, "token_seq")),
          _p(_i32(block_table, "block_table")), block_table.shape[1], _p(k_pages), _p(v_pages), T, nh, nkv, hd, vd,
          int(block_size), int(n_gate), coef, every, 1 if unit_values else 0, float(eps))


def rmsnorm(h: torch.Tensor, weight: torch.Tensor, eps: float, out_dtype: torch.dtype,
            rows: torch.Tensor | None = None, out: torch.Tensor | None = None, width: int | None = None) -> torch.Tensor:
    """Rows of float32 `h` (all, or those in `rows`) normed into `out_dtype`; `weight` None: brought to unit root
    mean square, no more.  `width`: the norm runs over the first so many columns of every row (the rows may then be
    any distance apart); the output is dense [rows, width]."""
    if h.dtype != torch.float32 or h.dim() != 2 or h.stride(1) != 1 or (width is None and not h.is_contiguous()):
        raise KernelError("rmsnorm reads float32 rows with unit inner stride (contiguous ones unless `width` is given)")
    H = h.shape[-1] if width is None else int(width)
    if not 0 < H <= h.shape[-1]:
        raise KernelError(f"rmsnorm: a width of {H} for rows of {h.shape[-1]}")
    if weight is not None and weight.numel() != H:
        raise KernelError(f"rmsnorm weight has {weight.numel()} elements for width {H}")
    R = h.shape[0] if rows is None else rows.numel()
    if out is None:
        out = torch.empty((R, H), dtype=out_dtype, device=h.device)
    _call("elementwise", "fx_rmsnorm", _stream(), dtype_code(out_dtype), _p(h), _p(_i32(rows, "rows")), _p(weight),
          dtype_code(weight.dtype) if weight is not None else FX_F32, _p(out), R, H, float(eps), h.stride(0))
    return out


def _freq_factors(freq_factors, rotary_dim):
    if freq_factors is None:
        return None
    if freq_factors.dtype != torch.float32 or not freq_factors.is_contiguous() or freq_factors.numel() != rotary_dim // 2:
        raise KernelError(f"rotary frequency factors must be {rotary_dim // 2} contiguous float32 values")
    return freq_factors


_inv_freq_tables: dict = {}


def rotary_frequencies(device, rotary_dim: int, theta: float, frequencies: tuple | None = None) -> torch.Tensor | None:
    """float32 [rotary_dim / 2] on the device: theta^(-2i/rotary_dim), worked out in float64 on the host and
    rounded once, so that the numbers do not depend on whose `powf` made them (the reference makes them in
    float32, ferrox-core/src/attention.rs:26: the last bit is its libm's).  The kernels multiply them by the
    position in float32, as the reference does (attention.rs:27).  Tables are kept for the life of the process:
    recorded steps hold their addresses."""
    if rotary_dim <= 0:
        return None
    if frequencies is not None:       # an encoding's own table (float64 numbers, rounded once here)
        frequencies = tuple(float(f) for f in frequencies)
        if len(frequencies) != rotary_dim // 2:
            raise KernelError(f"a table of {len(frequencies)} frequencies for {rotary_dim // 2} pairs")
    key = (torch.device(device), int(rotary_dim), float(theta), frequencies)
    if key not in _inv_freq_tables:
        values = list(frequencies) if frequencies is not None else \
            [1.0 / float(theta) ** (2.0 * i / rotary_dim) for i in range(rotary_dim // 2)]
        _inv_freq_tables[key] = torch.tensor(values, dtype=torch.float64).to(torch.float32).to(device)
    return _inv_freq_tables[key]


def rope_kv_write(q, k, v, positions, token_seq, block_table, k_pages, v_pages, n_heads, n_kv_heads,
                  head_dim, block_size, rotary_dim, theta, interleaved=False, freq_factors=None, frequencies=None,
                  v_dim=None) -> None:
    """Rotate q in place; rotate k and write it and v into the pages (skipped when k_pages is None).
    q, k, v are 2-D views [T, heads*head_dim] with unit inner stride.  `freq_factors` (float32
    [rotary_dim / 2] or None): the angle of pair i is divided by freq_factors[i].  `frequencies` (a tuple of
    rotary_dim / 2 numbers): the pairs' frequencies, instead of theta^(-2i/rotary_dim).  `v_dim`: size of a
    value head where it is not head_dim (v is then [T, n_kv_heads * v_dim])."""
    T = q.shape[0]
    v_dim = int(v_dim or head_dim)
    freq_factors = _freq_factors(freq_factors, rotary_dim)
    for t in (q, k, v):
        if t.stride(-1) != 1 or t.dtype != q.dtype:
            raise KernelError("rope_kv_write wants q, k, v of one dtype with unit inner stride")
    if k_pages is not None:
        if k_pages.dtype != q.dtype or v_pages.dtype != q.dtype:
            raise KernelError("cache pages and activations differ in dtype")
        if tuple(k_pages.shape[1:]) != (n_kv_heads, block_size, head_dim) or \
                tuple(v_pages.shape[1:]) != (n_kv_heads, v_dim, block_size):
            raise KernelError(f"cache pages have shapes {tuple(k_pages.shape)}, {tuple(v_pages.shape)}; expected "
                              f"[pages,{n_kv_heads},{block_size},{head_dim}] and [pages,{n_kv_heads},{v_dim},{block_size}]")
    if q.shape[1] < n_heads * head_dim or k.shape[1] < n_kv_heads * head_dim or v.shape[1] < n_kv_heads * v_dim:
        raise KernelError("rope_kv_write: q, k or v has fewer columns than its heads need")
    _call("elementwise", "fx_rope_kv_write", _stream(), dtype_code(q.dtype), _p(q), q.stride(0), _p(k), k.stride(0),
          _p(v), v.stride(0), _p(_i32(positions, "positions")), _p(_i32(token_seq, "token_seq")),
          _p(_i32(block_table, "block_table")), block_table.shape[1] if block_table is not None else 0,
          _p(k_pages), _p(v_pages), T, n_heads, n_kv_heads, head_dim, block_size, rotary_dim,
          1 if interleaved else 0, _p(rotary_frequencies(q.device, rotary_dim, theta, frequencies)), _p(freq_factors), v_dim)


def head_norm_kv_write(qk, q_out, v, q_weight, k_weight, eps, positions, token_seq, block_table, k_pages, v_pages,
                       n_heads, n_kv_heads, head_dim, block_size, v_dim=None) -> None:
    """For mixers that norm their heads and rotate nothing, in one launch: every head of the float32 q/k product
    `qk` [T, (n_heads + n_kv_heads) * head_dim] (or [T, n_heads * head_dim]: no keys) is divided by its root mean
    square (eps inside the root) and multiplied by `q_weight` / `k_weight` (head_dim elements each, or None); q goes
    to `q_out` [T, n_heads * head_dim], k into its page, `v` [T, n_kv_heads * v_dim] into its transposed page
    (`k_pages` None: q alone).  The norms are the bits of `rmsnorm` over gathered heads."""
    T = qk.shape[0]
    v_dim = int(v_dim or head_dim)
    with_keys = k_pages is not None
    if qk.dtype != torch.float32 or qk.stride(-1) != 1 or qk.shape[1] < (n_heads + (n_kv_heads if with_keys else 0)) * head_dim:
        raise KernelError(f"head_norm_kv_write: the q/k product must be float32 rows of all heads, got {tuple(qk.shape)} {qk.dtype}")
    if q_out.stride(-1) != 1 or q_out.shape[0] < T or q_out.shape[1] < n_heads * head_dim:
        raise KernelError(f"head_norm_kv_write: q_out {tuple(q_out.shape)} for {T} tokens of {n_heads} heads of {head_dim}")
    w_dtype = FX_F32
    for w in (q_weight, k_weight):
        if w is not None:
            if w.numel() != head_dim or not w.is_contiguous():
                raise KernelError(f"head_norm_kv_write: a weight of {w.numel()} elements for heads of {head_dim}")
            w_dtype = dtype_code(w.dtype)
    if q_weight is not None and k_weight is not None and q_weight.dtype != k_weight.dtype:
        raise KernelError("head_norm_kv_write: the two weights differ in dtype")
    if with_keys:
        if v is None or v.dtype != q_out.dtype or v.stride(-1) != 1 or v.shape[0] < T or v.shape[1] < n_kv_heads * v_dim:
            raise KernelError("head_norm_kv_write: values must come with the pages, in the type of q_out")
        if k_pages.dtype != q_out.dtype or v_pages.dtype != q_out.dtype:
            raise KernelError("cache pages and activations differ in dtype")
        if tuple(k_pages.shape[1:]) != (n_kv_heads, block_size, head_dim) or \
                tuple(v_pages.shape[1:]) != (n_kv_heads, v_dim, block_size):
            raise KernelError(f"cache pages have shapes {tuple(k_pages.shape)}, {tuple(v_pages.shape)}; expected "
                              f"[pages,{n_kv_heads},{block_size},{head_dim}] and [pages,{n_kv_heads},{v_dim},{block_size}]")
    _call("elementwise", "fx_head_norm_kv_write", _stream(), dtype_code(q_out.dtype), _p(qk), qk.stride(0), _p(q_out),
          q_out.stride(0), _p(v) if with_keys else None, v.stride(0) if with_keys else 0, _p(q_weight), _p(k_weight), w_dtype,
          float(eps), _p(_i32(positions, "positions")), _p(_i32(token_seq, "token_seq")),
          _p(_i32(block_table, "block_table")), block_table.shape[1] if block_table is not None else 0,
          _p(k_pages), _p(v_pages) if with_keys else None, T, n_heads, n_kv_heads, head_dim, block_size, v_dim)



def latent_kv_write(down, weight, eps, positions, token_seq, block_table, k_pages, v_pages, kv_rank: int, rot_dim: int,
                    rotary_dim: int, block_size: int, inv_freq, magnitude: float = 1.0, q_latent=None):
    """What a latent-attention layer keeps per position, from the float32 down-projection `down` [T, kv_rank +
    rot_dim]: the first kv_rank columns through an RMS norm with `weight` (the latent c), the last rot_dim with the
    pairs (2i, 2i+1), i < rotary_dim / 2, turned by pos * inv_freq[i] and stretched by `magnitude`.  The key page
    [pages, 1, block_size, kv_rank + rot_dim] receives (c | rotated part), the value page [pages, 1, kv_rank,
    block_size] c transposed.  `q_latent` = (rows, weight, eps): the same launch also norms the queries' latent, float32
    `rows` [T, q_rank] (any row distance, unit inner stride) with a weight of the keys' norm's type, and returns it
    [T, q_rank] in the pages' type (None without `q_latent`)."""
    T = down.shape[0]
    R, rd = int(kv_rank), int(rot_dim)
    _f32_rows(down, "latent_kv_write: the down-projection", R + rd)
    if weight.numel() != R or not weight.is_contiguous():
        raise KernelError(f"latent_kv_write: a norm weight of {weight.numel()} elements for a latent of {R}")
    if k_pages.dtype != v_pages.dtype or tuple(k_pages.shape[1:]) != (1, block_size, R + rd) or \
            tuple(v_pages.shape[1:]) != (1, R, block_size) or not k_pages.is_contiguous() or not v_pages.is_contiguous():
        raise KernelError(f"latent_kv_write: pages {tuple(k_pages.shape)}, {tuple(v_pages.shape)}; expected "
                          f"[pages,1,{block_size},{R + rd}] and [pages,1,{R},{block_size}]")
    if rotary_dim and (inv_freq is None or inv_freq.dtype != torch.float32 or inv_freq.numel() != rotary_dim // 2):
        raise KernelError(f"latent_kv_write: {rotary_dim} rotated dimensions need {rotary_dim // 2} float32 frequencies")
    if positions.numel() < T or token_seq.numel() < T:
        raise KernelError("latent_kv_write: the step's index tensors are shorter than its tokens")
    q_rows = q_w = q_out = None
    q_eps, Rq = 0.0, 0
    if q_latent is not None:
        q_rows, q_w, q_eps = q_latent
        Rq = q_w.numel()
        if q_rows.dtype != torch.float32 or q_rows.dim() != 2 or q_rows.stride(1) != 1 or q_rows.shape[0] < T or q_rows.shape[1] < Rq \
                or q_w.dtype != weight.dtype or not q_w.is_contiguous() or Rq < 1:
            raise KernelError(f"latent_kv_write: the queries' latent {tuple(q_rows.shape)} with a weight of {Rq} ({q_w.dtype})")
        q_out = torch.empty((T, Rq), dtype=k_pages.dtype, device=k_pages.device)
    _call("elementwise", "fx_latent_kv_write", _stream(), dtype_code(k_pages.dtype), _p(down), down.stride(0), _p(weight),
          dtype_code(weight.dtype), float(eps), _p(_i32(positions, "positions")), _p(_i32(token_seq, "token_seq")),
          _p(_i32(block_table, "block_table")), block_table.shape[1], _p(k_pages), _p(v_pages), T, R, rd, int(rotary_dim),
          int(block_size), _p(inv_freq), float(magnitude), _p(q_rows), q_rows.stride(0) if q_rows is not None else 0, _p(q_w),
          float(q_eps), _p(q_out), q_out.stride(0) if q_out is not None else 0, int(Rq))
    return q_out


def latent_q_rot(q, q_lat, positions, n_heads: int, dim: int, rot_dim: int, rotary_dim: int, kv_rank: int, inv_freq,
                 magnitude: float = 1.0) -> None:
    """The rotated part of latent attention's queries: the last rot_dim dimensions of every head of q [T, n_heads *
    (dim + rot_dim)], turned as `latent_kv_write` turns the shared key part, go behind the first kv_rank columns of
    that head's row of q_lat [T, n_heads * (kv_rank + rot_dim)]."""
    T = q.shape[0]
    for t, cols, what in ((q, n_heads * (dim + rot_dim), "q"), (q_lat, n_heads * (kv_rank + rot_dim), "q_lat")):
        if t.dim() != 2 or t.stride(1) != 1 or t.shape[1] < cols or t.shape[0] < T or t.dtype != q.dtype:
            raise KernelError(f"latent_q_rot: {what} {tuple(t.shape)} for {n_heads} heads")
    if rotary_dim and (inv_freq is None or inv_freq.dtype != torch.float32 or inv_freq.numel() != rotary_dim // 2):
        raise KernelError(f"latent_q_rot: {rotary_dim} rotated dimensions need {rotary_dim // 2} float32 frequencies")
    if positions.numel() < T:
        raise KernelError("latent_q_rot: fewer positions than tokens")
    _call("elementwise", "fx_latent_q_rot", _stream(), dtype_code(q.dtype), _p(q), q.stride(0), _p(q_lat), q_lat.stride(0),
          _p(_i32(positions, "positions")), T, int(n_heads), int(dim), int(rot_dim), int(rotary_dim), int(kv_rank),
          _p(inv_freq), float(magnitude))


def span_norm_kv_write(qk, q_out, q_weight, k_weight, eps, positions, token_seq, block_table, k_pages, v_pages,
                       n_heads: int, n_kv_heads: int, head_dim: int, block_size: int) -> None:
    """Queries and keys normed over their whole projection, keys that are their own values, in one launch: from the
    float32 product qk [T, (n_heads + n_kv_heads) * head_dim], the queries go, normed over all their columns with
    `q_weight` (one element a column), to q_out [T, n_heads * head_dim]; the keys, normed over all theirs with
    `k_weight`, into the key page, and as they are into the transposed value page (`k_pages` None: q alone, and qk
    may hold the queries only)."""
    T = qk.shape[0]
    qw, kw = int(n_heads) * int(head_dim), int(n_kv_heads) * int(head_dim)
    with_keys = k_pages is not None
    _f32_rows(qk, "span_norm_kv_write: the q/k product", qw + (kw if with_keys else 0))
    if q_out.stride(-1) != 1 or q_out.shape[0] < T or q_out.shape[1] < qw:
        raise KernelError(f"span_norm_kv_write: q_out {tuple(q_out.shape)} for {T} tokens of {qw} columns")
    if q_weight.numel() != qw or not q_weight.is_contiguous():
        raise KernelError(f"span_norm_kv_write: a query norm weight of {q_weight.numel()} elements for rows of {qw}")
    if with_keys:
        if k_weight is None or k_weight.numel() != kw or not k_weight.is_contiguous() or k_weight.dtype != q_weight.dtype:
            raise KernelError(f"span_norm_kv_write: the key norm's weight must hold {kw} elements of the query norm's type")
        if k_pages.dtype != q_out.dtype or v_pages.dtype != q_out.dtype or \
                tuple(k_pages.shape[1:]) != (n_kv_heads, block_size, head_dim) or \
                tuple(v_pages.shape[1:]) != (n_kv_heads, head_dim, block_size) or not k_pages.is_contiguous() or not v_pages.is_contiguous():
            raise KernelError(f"span_norm_kv_write: pages {tuple(k_pages.shape)}, {tuple(v_pages.shape)} ({k_pages.dtype})")
    if positions.numel() < T or token_seq.numel() < T:
        raise KernelError("span_norm_kv_write: the step's index tensors are shorter than its tokens")
    _call("elementwise", "fx_span_norm_kv_write", _stream(), dtype_code(q_out.dtype), _p(qk), qk.stride(0), _p(q_out),
          q_out.stride(0), _p(q_weight), _p(k_weight) if with_keys else None, dtype_code(q_weight.dtype), float(eps),
          _p(_i32(positions, "positions")), _p(_i32(token_seq, "token_seq")), _p(_i32(block_table, "block_table")),
          block_table.shape[1] if block_table is not None else 0, _p(k_pages), _p(v_pages) if with_keys else None, T,
          int(n_heads), int(n_kv_heads), int(head_dim), int(block_size))


_constant_rows: dict = {}


def constant_rows(device, value: float, n: int) -> torch.Tensor:
    """float32 [n] on the device, every element `value`: a row scale for products whose output is weighted by a
    constant (`gemm(..., row_scale=)`).  Tables are kept for the life of the process (recorded steps hold their
    addresses) and grow in powers of two."""
    key = (torch.device(device), float(value))
    have = _constant_rows.setdefault(key, [])
    for t in have:
        if t.numel() >= n:
            return t[:n]
    size = 1 << max(10, (int(n) - 1).bit_length())
    have.append(torch.full((size,), float(value), dtype=torch.float32, device=device))
    return have[-1][:n]


def residual_add(h: torch.Tensor, y: torch.Tensor) -> None:
    """h += y, summed in float32."""
    if h.dtype != torch.float32 or h.shape != y.shape or not h.is_contiguous() or not y.is_contiguous():
        raise KernelError("residual_add wants a contiguous float32 h and a y of the same shape")
    _call("elementwise", "fx_residual_add", _stream(), dtype_code(y.dtype), _p(h), _p(y), h.numel())


def cast(src: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    if src.dtype == dtype:
        return src
    src = src.contiguous()
    dst = torch.empty(src.shape, dtype=dtype, device=src.device)
    _call("elementwise", "fx_cast", _stream(), dtype_code(src.dtype), _p(src), dtype_code(dtype), _p(dst), src.numel())
    return dst


def fill_u32(t: torch.Tensor, value: int = 0) -> None:
    if not t.is_contiguous() or t.element_size() * t.numel() % 4:
        raise KernelError("fill_u32 wants a contiguous buffer of whole 32-bit words")
    _call("elementwise", "fx_fill_u32", _stream(), _p(t), value, t.element_size() * t.numel() // 4)


def feed_tokens(tokens: torch.Tensor, ids: torch.Tensor, pairs: torch.Tensor, n_tokens: int, n_ids: int) -> None:
    """tokens[pairs[i, 0]] = ids[pairs[i, 1]], all int32 on the device.  `pairs` [n, 2] was written by the host,
    which has checked it against `n_tokens` and `n_ids`; the ids come from the sampling kernel."""
    for t, name in ((tokens, "tokens"), (ids, "ids"), (pairs, "pairs")):
        if t.dtype != torch.int32 or not t.is_contiguous() or not t.is_cuda:
            raise KernelError(f"feed_tokens: {name} must be contiguous int32 on the GPU")
    if pairs.dim() != 2 or pairs.shape[1] != 2:
        raise KernelError("feed_tokens: pairs must be [n, 2]")
    if tokens.numel() < n_tokens or ids.numel() < n_ids:
        raise KernelError("feed_tokens: a buffer is shorter than the bound its pairs were checked against")
    _call("elementwise", "fx_feed_tokens", _stream(), _p(tokens), _p(ids), _p(pairs), pairs.shape[0])


class ScaleLater:
    """Rows x = round(h * w) of an RMSNorm whose scale is still to come: `ss` [T, n] holds sums of squares of
    parts of each row of h, and row t is to be scaled by rsqrt(sum(ss[t]) / width + eps).  `gemm(..., row_ss=)`
    applies the scale to its product, which is the rounding of the norm that `gemm(..., norm=)` applies itself."""
    __slots__ = ("x", "ss", "eps")

    def __init__(self, x, ss, eps):
        self.x, self.ss, self.eps = x, ss, eps


def moe_combine(h, y_sorted, inv, weights, top_k, shared=None, gate=None, scale_later=None):
    """h[t] += sum_j weights[t, j] * y_sorted[inv[t*k + j]] (inv None: y is in pair order t*k + j)
    + gate[t] * shared[t] if the float32 output of a shared expert is given; `shared` may also be
    [S, T, H], partial outputs that are summed first.
    `scale_later` = (norm weight, eps, dtype): also returns the new rows as a ScaleLater for that RMSNorm."""
    T, H = h.shape
    if y_sorted.dtype != torch.float32 or h.dtype != torch.float32:
        raise KernelError("moe_combine works on float32")
    slabs = 1
    if shared is not None:
        if shared.dtype != torch.float32 or not shared.is_contiguous() or shared.shape[-2:] != h.shape or shared.dim() > 3:
            raise KernelError("moe_combine: the shared expert's output must be float32 [T, H] or [S, T, H]")
        slabs = shared.shape[0] if shared.dim() == 3 else 1
    x, nw, eps, code, ss = None, None, 0.0, 0, None
    if scale_later is not None:
        nw, eps, dt = scale_later
        if nw.numel() != H or not nw.is_contiguous() or not h.is_contiguous():
            raise KernelError(f"moe_combine: norm weight of {nw.numel()} elements for width {H}")
        x, code = torch.empty((T, H), dtype=dt, device=h.device), dtype_code(dt)
        ss = torch.empty((T, (H + 255) // 256), dtype=torch.float32, device=h.device)
    _call("elementwise", "fx_moe_combine", _stream(), _p(h), _p(y_sorted), _p(_i32(inv, "inv")), _p(weights),
          _p(shared), _p(gate), T, H, top_k, slabs, _p(nw), dtype_code(nw.dtype) if nw is not None else 0,
          _p(x), code, _p(ss))
    return ScaleLater(x, ss, float(eps)) if ss is not None else None


def gemm(a: torch.Tensor, w: torch.Tensor, *, epilogue: int = EPI_STORE, out: torch.Tensor | None = None,
         bias: torch.Tensor | None = None, row_scale: torch.Tensor | None = None,
         a_rows: torch.Tensor | None = None, c_rows: torch.Tensor | None = None,
         expert_offsets: torch.Tensor | None = None,
         n_rows: int | None = None, n_out: int | None = None, up_offset: int = 0,
         norm: tuple | None = None, pair_ids: torch.Tensor | None = None, pair_div: int = 1,
         always: tuple | None = None, w_kblocked: bool = False, row_ss: tuple | None = None,
         activation: str = "silu", store_activation: str | None = None, activation_params: tuple = (0.0, 0.0),
         pre_scale: torch.Tensor | None = None, pre_scale_rows: torch.Tensor | None = None) -> torch.Tensor:
    """C[m, n] = sum_k a[m, k] * w[n, k] with an epilogue.

    `w` is [N, K], or [E, N, K] with `expert_offsets` [E+1] (rows sorted by expert).
    EPI_STORE stores in a's dtype (+bias); EPI_STORE_F32 stores float32; EPI_RESID adds the
    product (times row_scale[m]) into the float32 `out`; EPI_GATED multiplies two
    matrices (rows [0, n_out) and [up_offset/K, ...) of w) and stores activation(gate) * up,
    `activation` being one of ACTIVATIONS.
    `a_rows` gathers the rows of a; `n_rows` is the number of logical rows then.  `c_rows`
    scatters the rows of the output (row_scale stays indexed by the logical row).
    `pair_ids` (int32, up to 64 entries) replaces the sorted layout for
    few rows: logical row m belongs to expert pair_ids[m], reads row m // pair_div of `a` and
    writes row m of the output; the kernel groups the rows by expert itself.  `always` = (S, T,
    from_a): the last S experts of `w` are taken by each of T rows (a shared expert cut into S
    pieces); piece s writes output rows n_pairs + s*T + t and reads row t of `a` (from_a) or that
    same row of `a`.
    `w_kblocked`: `w` is stored as `to_kblocked` makes it, [.., K/64, N, 64] (bfloat16, K % 64 == 0).
    `norm` = (weight [K], eps): `a` is the float32 residual stream and RMSNorm is applied on the way
    in (bfloat16 weights, EPI_STORE, at most 32 rows; see `can_fuse_norm`).
    `row_ss` = (ss [M, n] float32, eps): row m of the product is scaled by rsqrt(sum(ss[m]) / K + eps)
    before the bias is added (the rows of `a` are a ScaleLater's; plain stored bfloat16 product, M <= 64).
    `store_activation` (one of STORED_ACTIVATIONS, EPI_STORE or EPI_STORE_F32 without bias): the product goes through
    it before it is stored, e.g. "relu2" = max(x, 0)^2.
    `activation_params` = (limit, alpha) for "swiglu_clamped": g = min(gate, limit), u = clamp(up, -limit, limit),
    stored g sigmoid(alpha g) (u + 1).
    `pre_scale` (EPI_GATED; float32): gate and up of logical row m are multiplied by pre_scale[m] (or by
    pre_scale[pre_scale_rows[m]]) before the activation, which is what the activation sees when row m of `a` is
    scaled by that number.
    """
    if store_activation not in STORED_ACTIVATIONS:
        raise KernelError(f"gemm: stored activation '{store_activation}' is not one of {sorted(k for k in STORED_ACTIVATIONS if k)}")
    if store_activation is not None and (epilogue not in (EPI_STORE, EPI_STORE_F32) or bias is not None):
        raise KernelError("gemm: a stored activation goes with the plain stored product without bias")
    if row_ss is not None:
        ss = row_ss[0]
        if ss.dtype != torch.float32 or ss.dim() != 2 or not ss.is_contiguous() or ss.shape[0] != a.shape[0]:
            raise KernelError("gemm: row_ss must be a contiguous float32 [rows, parts]")
    if norm is not None:
        if a.dtype != torch.float32 or w.dtype != torch.bfloat16 or epilogue != EPI_STORE:
            raise KernelError("gemm: the fused norm reads float32 rows for a stored bfloat16 product")
        if norm[0].numel() != a.shape[1] or not norm[0].is_contiguous():
            raise KernelError("gemm: the norm's weight does not fit the rows")
    elif a.dtype != w.dtype:
        raise KernelError(f"gemm: activations are {a.dtype}, weights {w.dtype}")
    if a.dim() != 2 or a.stride(1) != 1:
        raise KernelError("gemm: activations must be 2-D with unit inner stride")
    if not w.is_contiguous():
        raise KernelError("gemm: weights must be contiguous")
    K = a.shape[1]
    grouped = expert_offsets is not None or pair_ids is not None
    n_always, always_rows, always_from_a = (int(always[0]), int(always[1]), 1 if always[2] else 0) if always else (0, 0, 0)
    if pair_ids is not None:
        n_rows = pair_ids.numel()
    if w_kblocked:
        if w.dim() != (4 if grouped else 3) or w.shape[-1] != 64 or w.dtype != torch.bfloat16:
            raise KernelError("gemm: weights in slabs must be bfloat16 [(E,) K/64, N, 64]")
        n_w, kw = w.shape[-2], w.shape[-3] * 64
        E, w_stride = (w.shape[0] - n_always, n_w * kw) if grouped else (0, 0)
    elif grouped:
        if w.dim() != 3:
            raise KernelError("gemm: grouped weights must be [E, N, K]")
        E, n_w, kw = w.shape
        E -= n_always
        w_stride = n_w * kw
    else:
        if w.dim() != 2:
            raise KernelError("gemm: weights must be [N, K]")
        E, (n_w, kw), w_stride = 0, w.shape, 0
    if kw != K:
        raise KernelError(f"gemm: inner sizes differ, activations {K}, weights {kw}")
    M = n_rows if n_rows is not None else a.shape[0]
    if activation not in ACTIVATIONS:
        raise KernelError(f"gemm: activation '{activation}' is not one of {sorted(ACTIVATIONS)}")
    if epilogue == EPI_GATED:
        N = n_out if n_out is not None else n_w // 2
        if up_offset == 0:
            up_offset = N * K
        if up_offset // K + N > n_w:
            raise KernelError("gemm: gate/up rows exceed the weight matrix")
    else:
        N = n_out if n_out is not None else n_w
    out_dtype = w.dtype if epilogue in (EPI_STORE, EPI_GATED) else torch.float32
    out_rows = M + n_always * always_rows
    if out is None:
        if epilogue == EPI_RESID:
            raise KernelError("gemm: the residual epilogue needs `out`")
        out = torch.empty((out_rows, N), dtype=out_dtype, device=a.device)
    if out.dtype != out_dtype or out.dim() != 2 or out.stride(1) != 1 or out.shape[0] < out_rows or out.shape[1] < N:
        raise KernelError(f"gemm: output {tuple(out.shape)} {out.dtype} does not fit [{M},{N}] {out_dtype}")
    if bias is not None and bias.numel() != N:
        raise KernelError(f"gemm: bias has {bias.numel()} elements for {N} columns")
    if pre_scale is not None:
        if epilogue != EPI_GATED or pre_scale.dtype != torch.float32 or not pre_scale.is_contiguous() \
                or (pre_scale_rows is None and pre_scale.numel() < M) or (pre_scale_rows is not None and pre_scale_rows.numel() < M):
            raise KernelError("gemm: a scale in front of the activation is contiguous float32, one number per logical row, "
                              "with the gate/up epilogue")
    _call("gemm", "fx_gemm", _stream(), dtype_code(w.dtype), epilogue, _p(a), a.stride(0), _p(w), w_stride, up_offset,
          _p(bias), dtype_code(bias.dtype) if bias is not None else 0, _p(out), out.stride(0),
          _p(row_scale), _p(_i32(a_rows, "a_rows")), _p(_i32(c_rows, "c_rows")),
          _p(_i32(expert_offsets, "expert_offsets")), E, M, N, K,
          _p(norm[0]) if norm is not None else None, dtype_code(norm[0].dtype) if norm is not None else 0,
          float(norm[1]) if norm is not None else (float(row_ss[1]) if row_ss is not None else 0.0),
          _p(_i32(pair_ids, "pair_ids")), int(pair_div),
          n_always, always_rows, always_from_a, n_w if w_kblocked else 0,
          _p(row_ss[0]) if row_ss is not None else None, row_ss[0].shape[1] if row_ss is not None else 0,
          ACTIVATIONS[activation], STORED_ACTIVATIONS[store_activation], float(activation_params[0]),
          float(activation_params[1]), _p(pre_scale), _p(_i32(pre_scale_rows, "pre_scale_rows")))
    return out


def can_qkv_rope(x, w, n_rows: int, head_dim: int, rotary_dim: int, interleaved: bool) -> bool:
    """Whether qkv_rope takes these operands: up to 64 rows of bfloat16 (or a ScaleLater of them), split-half
    rotation, head and rotary dimensions that are multiples of 32, aligned rows."""
    xt = x.x if isinstance(x, ScaleLater) else x
    return (n_rows <= 64 and not interleaved and head_dim % 32 == 0 and rotary_dim % 32 == 0
            and xt.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and w.dim() == 2 and w.is_contiguous()
            and xt.dim() == 2 and xt.stride(1) == 1 and xt.stride(0) % 8 == 0 and xt.shape[1] % 8 == 0
            and xt.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0)


def qkv_rope(x, w, bias, positions, token_seq, block_table, k_pages, v_pages, n_heads, n_kv_heads, head_dim,
             block_size, rotary_dim, theta, freq_factors=None) -> torch.Tensor:
    """The q/k/v product of few tokens with the rotation and the cache write in its epilogue: returns
    [T, (n_heads + 2 n_kv_heads) head_dim] whose query columns are rotated (the others are not written); rotated
    keys and the values go into their pages (k_pages None: nowhere).  The bits are those of `gemm` followed by
    `rope_kv_write`.  `x` may be a ScaleLater."""
    later = x if isinstance(x, ScaleLater) else None
    xt = later.x if later else x
    T, K = xt.shape
    N = (n_heads + 2 * n_kv_heads) * head_dim
    if w.shape != (N, K):
        raise KernelError(f"qkv_rope: weights {tuple(w.shape)} for [{N}, {K}]")
    if bias is not None and bias.numel() != N:
        raise KernelError(f"qkv_rope: bias has {bias.numel()} elements for {N} columns")
    if k_pages is not None:
        if k_pages.dtype != xt.dtype or v_pages.dtype != xt.dtype:
            raise KernelError("cache pages and activations differ in dtype")
        if tuple(k_pages.shape[1:]) != (n_kv_heads, block_size, head_dim) or \
                tuple(v_pages.shape[1:]) != (n_kv_heads, head_dim, block_size):
            raise KernelError(f"cache pages have shapes {tuple(k_pages.shape)}, {tuple(v_pages.shape)}")
    out = torch.empty((T, N), dtype=xt.dtype, device=xt.device)
    _call("gemm", "fx_qkv_rope", _stream(), _p(xt), xt.stride(0), _p(w), 0, _p(bias),
          dtype_code(bias.dtype) if bias is not None else 0, _p(out), out.stride(0), T, K,
          _p(later.ss) if later else None, later.ss.shape[1] if later else 0, float(later.eps) if later else 0.0,
          _p(_i32(positions, "positions")), _p(_i32(token_seq, "token_seq")), _p(_i32(block_table, "block_table")),
          block_table.shape[1] if block_table is not None else 0, _p(k_pages), _p(v_pages),
          n_heads, n_kv_heads, head_dim, block_size, rotary_dim, _p(rotary_frequencies(xt.device, rotary_dim, theta)),
          _p(_freq_factors(freq_factors, rotary_dim)))
    return out


def to_kblocked(w: torch.Tensor) -> torch.Tensor:
    """[.., N, K] -> [.., K/64, N, 64]: 64 k of every row, then the next 64 k of every row.  A tile of
    rows then reads one contiguous stretch of memory per K step instead of a short piece of every
    row, which is what the memory likes when the weights are streamed."""
    *lead, N, K = w.shape
    if K % 64:
        raise KernelError(f"to_kblocked: K={K} is not a multiple of 64")
    return w.reshape(*lead, N, K // 64, 64).transpose(-3, -2).contiguous()


def can_fuse_norm(h: torch.Tensor, w: torch.Tensor, n_rows: int) -> bool:
    """Whether gemm(h, w, norm=...) takes these operands: few rows, bfloat16 weights, aligned rows."""
    return (h.dtype == torch.float32 and w.dtype == torch.bfloat16 and w.dim() == 2 and n_rows <= 32
            and h.shape[1] % 8 == 0 and h.stride(0) % 4 == 0 and h.stride(1) == 1
            and h.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0)


_compute_units: dict = {}


def compute_units(device) -> int:
    """CUs of the device (asked for once)."""
    key = torch.device(device) if device is not None else torch.device("cuda", torch.cuda.current_device())
    if key not in _compute_units:
        _compute_units[key] = int(torch.cuda.get_device_properties(key).multi_processor_count)
    return _compute_units[key]


def attention_tile_queries(dtype, head_dim: int, block_size: int) -> int:
    """The most consecutive queries of a sequence that one item of attention_tiles may cover at these sizes: 64,
    or 128 where the kernel has a block of eight waves for them."""
    f, _ = _fn("attention", "fx_attn_tile_queries")
    return int(f(dtype_code(dtype), int(head_dim), int(block_size)))


def attention_tiles(q, out, k_pages, v_pages, block_table, positions, item_seq, item_tok, item_n,
                    n_heads, n_kv_heads, head_dim, block_size, window, scale, tile_q: int = 64, mask_chunk: int = 0,
                    v_dim: int | None = None, keep_first: int = 0, sinks=None, gate=None, softcap: float = 0.0,
                    slopes=None, gate_per_head: bool = False) -> None:
    """Blocks of queries: item i is item_n[i] <= tile_q consecutive tokens of sequence item_seq[i] from token
    item_tok[i] on; tile_q is 64 or attention_tile_queries(...).  `mask_chunk` > 0: the chunked mask (a query sees
    the keys of its own chunk of that many positions) instead of a window.  `v_dim`: size of a value head where it
    is not head_dim; `out` is [T, n_heads * v_dim].  `keep_first` (with a window): the first so many keys of a
    sequence stay visible to every later query.  `sinks` (float32 [n_heads]): a logit per head that joins the
    softmax's denominator and has no value.  `gate` (shape and type of `out`): the output is multiplied by sigmoid(gate).
    `softcap` > 0: a scaled score s becomes softcap * tanh(s / softcap).  `slopes` (float32 [n_heads]): the score of
    key t for the query at position p then loses slopes[h] * (p - t)."""
    _check_attention_shapes(q, out, k_pages, v_pages, n_heads, n_kv_heads, head_dim, int(v_dim or head_dim), block_size)
    _check_attention_extras(out, n_heads, 1 if gate_per_head else int(v_dim or head_dim), window, keep_first, sinks, gate, softcap, slopes)
    _call("attention", "fx_attn_tiles", _stream(), dtype_code(q.dtype), _p(q), q.stride(0), _p(out), out.stride(0),
          _p(k_pages), _p(v_pages), _p(_i32(block_table, "block_table")), block_table.shape[1],
          _p(_i32(positions, "positions")), _p(_i32(item_seq, "item_seq")), _p(_i32(item_tok, "item_tok")),
          _p(_i32(item_n, "item_n")), item_seq.numel(), n_heads, n_kv_heads, head_dim, block_size,
          int(window or 0), float(scale), int(tile_q), int(v_dim or head_dim), int(mask_chunk or 0),
          int(keep_first or 0), _p(sinks), _p(gate), gate.stride(0) if gate is not None else 0, float(softcap or 0.0),
          _p(slopes), 1 if gate_per_head else 0)


def _check_attention_extras(out, n_heads, v_dim, window, keep_first, sinks, gate, softcap=0.0, slopes=None) -> None:
    if keep_first and not window:
        raise KernelError("attention: kept first keys go with a window")
    if not 0.0 <= float(softcap or 0.0) < math.inf:
        raise KernelError(f"attention: a cap of {softcap} on the scores")
    if slopes is not None and (slopes.dtype != torch.float32 or not slopes.is_contiguous() or slopes.numel() != n_heads):
        raise KernelError(f"attention: distance slopes must be {n_heads} contiguous float32 values")
    if sinks is not None and (sinks.dtype != torch.float32 or not sinks.is_contiguous() or sinks.numel() != n_heads):
        raise KernelError(f"attention: sinks must be {n_heads} contiguous float32 values")
    if gate is not None and (gate.dtype != out.dtype or gate.stride(-1) != 1 or gate.shape[0] < out.shape[0]
                             or gate.shape[1] < n_heads * v_dim):
        raise KernelError(f"attention: gate {tuple(gate.shape)} ({gate.dtype}) for an output {tuple(out.shape)} ({out.dtype})")


def _check_attention_shapes(q, out, k_pages, v_pages, n_heads, n_kv_heads, head_dim, v_dim, block_size) -> None:
    """The kernels index by these sizes: the operands must hold them."""
    if q.shape[1] < n_heads * head_dim or out.shape[1] < n_heads * v_dim or out.shape[0] < q.shape[0]:
        raise KernelError(f"attention: q {tuple(q.shape)} / out {tuple(out.shape)} for {n_heads} heads of {head_dim} / {v_dim}")
    if tuple(k_pages.shape[1:]) != (n_kv_heads, block_size, head_dim) or tuple(v_pages.shape[1:]) != (n_kv_heads, v_dim, block_size):
        raise KernelError(f"attention: cache pages have shapes {tuple(k_pages.shape)}, {tuple(v_pages.shape)}; expected "
                          f"[pages,{n_kv_heads},{block_size},{head_dim}] and [pages,{n_kv_heads},{v_dim},{block_size}]")
    if q.dtype != out.dtype or k_pages.dtype != q.dtype or v_pages.dtype != q.dtype:
        raise KernelError("attention: queries, output and cache pages differ in dtype")


SPLIT_PARTIAL_ROUNDS = True      # decode attention: more chunks where the blocks' last round over the CUs would be far from full


def decode_attention_chunk(n_items: int, n_heads: int, n_kv_heads: int, max_kv_len: int, cus: int) -> int:
    """Keys per chunk of the bfloat16 decode attention, where the caller names none: the fewest chunks that still put
    about eight waves on every CU (one chunk, and no merge launch, from as many (sequence, kv head) pairs as CUs
    on), unless the waves' last round over the CUs would be far from full."""
    pairs = n_items * n_kv_heads * (-(-(n_heads // n_kv_heads) // 16))
    want = max(1, 8 * cus // max(1, pairs * 8))
    # More (sequence, kv head) pairs than CUs: a CU holds eight waves of this kernel, which the launch groups
    # into blocks of eight or four (one chunk a sequence), so the waves run in rounds, and a last round that
    # is far from full (272 blocks of eight waves on 256 CUs: 17 sequences of 16 kv heads) costs nearly as much
    # as a full one.  Eight chunks a sequence, which the launch then gives to blocks of one wave, fill the CUs
    # evenly: 17 sequences at 2,060 keys 80 -> 58 us, 24 sequences 81 -> 77 us, 36 sequences 125 -> 108 us, 17 at
    # 8,200 keys 285 -> 192 us; where the last round is full (32, 64 sequences) one chunk is 2-4 % ahead, and
    # from four pairs a CU on one chunk is level with every other choice.
    if SPLIT_PARTIAL_ROUNDS and cus < pairs <= 4 * cus and max_kv_len >= 1024:
        per_block = 8                   # waves, as fx_attn_decode picks them for one chunk a sequence
        while per_block > 4 and pairs * (per_block // 2) >= 8 * cus:
            per_block //= 2
        rounds = pairs * per_block / (8 * cus)
        if (math.ceil(rounds) - rounds) / math.ceil(rounds) >= 0.10:
            want = 8
    return max(64, -(-(-(-max_kv_len // want)) // 64) * 64)


def attention_decode(q, out, k_pages, v_pages, block_table, positions, item_seq, item_tok,
                     n_heads, n_kv_heads, head_dim, block_size, window, scale, max_kv_len, chunk=None,
                     waves=0, mask_chunk: int = 0, v_dim: int | None = None, keep_first: int = 0, sinks=None,
                     gate=None, softcap: float = 0.0, slopes=None, gate_per_head: bool = False) -> None:
    """Single queries.  The keys go to ceil(max_kv_len / chunk) blocks whose results are merged in ascending
    order.  float32 cuts them at multiples of `chunk`, 256 by default (so that a result does not depend on the
    batch); bfloat16, whose blocks of up to eight waves share a chunk, cuts every sequence's own range of keys (from
    its window's first key to its position) into that many equal chunks of whole tiles of 64, `chunk` by default as
    `decode_attention_chunk` picks it.  `waves`: waves per block, 0 for the launch's own choice."""
    n = item_seq.numel()
    v_dim = int(v_dim or head_dim)
    _check_attention_shapes(q, out, k_pages, v_pages, n_heads, n_kv_heads, head_dim, v_dim, block_size)
    _check_attention_extras(out, n_heads, 1 if gate_per_head else v_dim, window, keep_first, sinks, gate, softcap, slopes)
    if chunk is None:
        chunk = 256
        if q.dtype == torch.bfloat16:
            chunk = decode_attention_chunk(n, n_heads, n_kv_heads, max_kv_len, compute_units(q.device))
    splits = max(1, -(-max_kv_len // chunk))
    part_o = torch.empty((n, n_heads, splits, v_dim), dtype=torch.float32, device=q.device)
    part_ml = torch.empty((n, n_heads, splits, 2), dtype=torch.float32, device=q.device)
    _call("attention", "fx_attn_decode", _stream(), dtype_code(q.dtype), _p(q), q.stride(0), _p(out), out.stride(0),
          _p(k_pages), _p(v_pages), _p(_i32(block_table, "block_table")), block_table.shape[1],
          _p(_i32(positions, "positions")), _p(_i32(item_seq, "item_seq")), _p(_i32(item_tok, "item_tok")), n,
          n_heads, n_kv_heads, head_dim, block_size, int(window or 0), float(scale),
          _p(part_o), _p(part_ml), splits, chunk, int(waves), v_dim, int(mask_chunk or 0),
          int(keep_first or 0), _p(sinks), _p(gate), gate.stride(0) if gate is not None else 0, float(softcap or 0.0),
          _p(slopes), 1 if gate_per_head else 0)


def router_select(logits, n_experts, top_k, renorm, gating=GATE_SOFTMAX, has_gate=False, selection_bias=None,
                  weighting=(0.0, 1.0)):
    """From float32 router logits [T, >= E (+1)] (any strides, so also the transpose of an
    [E (+1), T] product): (ids int32 [T,k], weights float32 [T,k], gate float32 [T] =
    sigmoid(logits[:, E]) or None).  `selection_bias` (float32 [E]): the experts are chosen by score + bias,
    the weights are the scores.  `weighting` = (eps, scale): a renormalised weight is score / (sum of the chosen
    scores + eps), and every weight is multiplied by scale."""
    if selection_bias is not None and (selection_bias.dtype != torch.float32 or not selection_bias.is_contiguous()
                                       or selection_bias.numel() != n_experts):
        raise KernelError(f"router_select: the selection bias must be {n_experts} contiguous float32 values")
    if logits.dtype != torch.float32 or logits.dim() != 2 or min(logits.stride()) < 1:
        raise KernelError("router_select: logits must be a float32 [T, E] matrix")
    T = logits.shape[0]
    ids = torch.empty((T, top_k), dtype=torch.int32, device=logits.device)
    weights = torch.empty((T, top_k), dtype=torch.float32, device=logits.device)
    gate = torch.empty((T,), dtype=torch.float32, device=logits.device) if has_gate else None
    if logits.shape[1] < n_experts + (1 if has_gate else 0):
        raise KernelError(f"router_select: {logits.shape[1]} columns for {n_experts} experts")
    _call("moe", "fx_router_select", _stream(), _p(logits), logits.stride(0), logits.stride(1), T, n_experts, top_k,
          1 if renorm else 0, float(weighting[0]), float(weighting[1]), gating, _p(ids), _p(weights), _p(gate),
          _p(selection_bias))
    return ids, weights, gate


def route(logits, n_experts, top_k, renorm, gating=GATE_SOFTMAX, has_gate=False, weighting=(0.0, 1.0)):
    """router_select followed by moe_align; one launch when the batch is small.
    Returns (ids, weights, gate, expert_offsets, sorted_token, sorted_pair, inv)."""
    if logits.dtype != torch.float32 or logits.dim() != 2:
        raise KernelError("route: logits must be a float32 [T, E] matrix")
    T = logits.shape[0]
    dev = logits.device
    if T <= 16 and logits.stride(1) == 1 and logits.shape[1] >= n_experts + (1 if has_gate else 0):
        n = T * top_k
        ids = torch.empty((T, top_k), dtype=torch.int32, device=dev)
        weights = torch.empty((T, top_k), dtype=torch.float32, device=dev)
        gate = torch.empty((T,), dtype=torch.float32, device=dev) if has_gate else None
        offsets = torch.empty((n_experts + 1,), dtype=torch.int32, device=dev)
        buf = torch.empty((3, n), dtype=torch.int32, device=dev)
        f, handle = _fn("moe", "fx_router_select_align")
        rc = f(_stream(), _p(logits), logits.stride(0), T, n_experts, top_k, 1 if renorm else 0, float(weighting[0]),
               float(weighting[1]), gating, _p(ids),
               _p(weights), _p(gate), _p(offsets), _p(buf[0]), _p(buf[1]), _p(buf[2]))
        if rc == 0:
            return ids, weights, gate, offsets, buf[0], buf[1], buf[2]
        if rc != 2:
            raise KernelError(handle.fx_last_error().decode())
    ids, weights, gate = router_select(logits, n_experts, top_k, renorm, gating, has_gate, weighting=weighting)
    return (ids, weights, gate) + moe_align(ids, n_experts)


_counters: dict = {}


def _counter(device, n: int = 1) -> torch.Tensor:
    """At least n zeroed words for kernels whose last block finishes the work; a kernel leaves its
    words at zero, so launches that follow each other on a stream share them.  Buffers are never
    freed: a recorded graph may hold their address."""
    key = torch.device(device)
    if key.index is None:
        key = torch.device(key.type, torch.cuda.current_device())
    held = _counters.setdefault(key, [])
    if not held or held[-1].numel() < n:
        held.append(torch.zeros(max(1024, 2 * n), dtype=torch.int32, device=key))
    return held[-1]


def moe_front(h, norm_weight, eps, router, n_experts, top_k, renorm, gating=GATE_SOFTMAX, has_gate=False,
              align: int | None = None, weighting=(0.0, 1.0)):
    """For up to 256 rows of the float32 residual stream, in one launch: RMSNorm into bfloat16, router
    products and selection.  Returns None for sizes the kernel does not take, else
    (x, ids, weights, gate, aligned).  `align` = S asks the same launch for what `moe_align(ids, n_experts,
    always=S)` returns (its last block sorts the pairs): `aligned`, else None."""
    T, H = h.shape
    if (T > 256 or h.dtype != torch.float32 or h.stride(1) != 1 or router.dtype != torch.bfloat16
            or not router.is_contiguous() or router.shape != (n_experts + (1 if has_gate else 0), H)
            or norm_weight.numel() != H):
        return None
    dev = h.device
    x = torch.empty((T, H), dtype=torch.bfloat16, device=dev)
    ids = torch.empty((T, top_k), dtype=torch.int32, device=dev)
    weights = torch.empty((T, top_k), dtype=torch.float32, device=dev)
    gate = torch.empty((T,), dtype=torch.float32, device=dev) if has_gate else None
    logits = torch.empty((T, router.shape[0]), dtype=torch.float32, device=dev)
    offsets = buf = None
    if align is not None:
        offsets = torch.empty((n_experts + 1 + align,), dtype=torch.int32, device=dev)
        buf = torch.empty((3, T * top_k + align * T), dtype=torch.int32, device=dev)
    f, handle = _fn("moe", "fx_moe_front")
    rc = f(_stream(), _p(h), h.stride(0), _p(norm_weight), dtype_code(norm_weight.dtype), float(eps), _p(x), _p(router),
           H, T, n_experts, 1 if has_gate else 0, top_k, 1 if renorm else 0, float(weighting[0]), float(weighting[1]),
           gating, _p(logits), _p(ids), _p(weights),
           _p(gate), _p(_counter(dev, T + 1)), _p(offsets), _p(buf[0]) if buf is not None else None,
           _p(buf[1]) if buf is not None else None, _p(buf[2]) if buf is not None else None, int(align or 0))
    if rc == 2 and align is not None:      # the sort's counters do not fit beside the front's: without it
        return moe_front(h, norm_weight, eps, router, n_experts, top_k, renorm, gating, has_gate, weighting=weighting)
    if rc == 2:
        return None
    if rc:
        raise KernelError(handle.fx_last_error().decode())
    return x, ids, weights, gate, (offsets, buf[0], buf[1], buf[2]) if buf is not None else None


def moe_align(ids: torch.Tensor, n_experts: int, always: int = 0):
    """For ids [T, k]: (expert_offsets [E+1], sorted_token [n], sorted_pair [n], inv [n]): sorted row i
    belongs to pair sorted_pair[i] = t*k + j of token sorted_token[i]; inv is the inverse map.
    `always` = S: S further experts follow that every token takes (a shared expert cut into pieces): the
    offsets have E+1+S entries and the sorted arrays n + S*T, piece s owning rows n + s*T + t (token t), whose
    output rows have the same numbers (up to 2048 pairs)."""
    T, k = ids.shape
    n = T * k
    dev = ids.device
    offsets = torch.empty((n_experts + 1 + always,), dtype=torch.int32, device=dev)
    buf = torch.empty((3, n + always * T), dtype=torch.int32, device=dev)
    # many pairs are sorted by many blocks, which hand each other the counts of every group of 64 pairs
    gcnt = torch.empty((-(-n // 64), n_experts), dtype=torch.int32, device=dev) if n > 2048 else None
    _call("moe", "fx_moe_align", _stream(), _p(_i32(ids, "ids")), n, k, n_experts, _p(offsets), _p(buf[0]), _p(buf[1]),
          _p(buf[2]), _p(gcnt), int(always))
    return offsets, buf[0], buf[1], buf[2]


def sample(logits: torch.Tensor, *, temperature=None, draw=None, top_k=None, top_p=None, rep_penalty=None,
           presence=None, frequency=None, hist=None, hist_start=None) -> torch.Tensor:
    """One token per row of float32 logits [R, V]; all per-row parameters are device tensors or None
    (None: greedy / option off)."""
    if logits.dtype != torch.float32 or logits.dim() != 2 or logits.stride(1) != 1:
        raise KernelError("sample: logits must be float32 [R, V] with unit inner stride")
    R, V = logits.shape
    out = torch.empty((R,), dtype=torch.int32, device=logits.device)
    if temperature is None and hist is None:      # plain greedy: many blocks per row
        part = torch.empty((R, 64, 2), dtype=torch.int32, device=logits.device)
        _call("sampling", "fx_sample_greedy", _stream(), _p(logits), logits.stride(0), R, V, _p(part),
              _p(_counter(logits.device, R)), _p(out))
        return out
    work = torch.empty((R, V), dtype=torch.float32, device=logits.device)
    _call("sampling", "fx_sample", _stream(), _p(logits), logits.stride(0), _p(work), R, V,
          _p(temperature), _p(_i32(top_k, "top_k")), _p(top_p), _p(rep_penalty), _p(presence), _p(frequency),
          _p(draw), _p(_i32(hist, "hist")), _p(_i32(hist_start, "hist_start")), _p(out))
    return out


# ---------------------------------------------------------------------------
# norms after a sublayer, identity experts, recurrent mixers
# ---------------------------------------------------------------------------
def rmsnorm_add(h: torch.Tensor, y: torch.Tensor, weight: torch.Tensor, eps: float) -> None:
    """h[t] += y[t] * rsqrt(mean(y[t]^2) + eps) * weight: float32 rows of a sublayer's output, normed as they join
    the residual stream."""
    if h.dtype != torch.float32 or y.dtype != torch.float32 or h.shape != y.shape or not h.is_contiguous() or not y.is_contiguous():
        raise KernelError("rmsnorm_add wants contiguous float32 h and y of one shape")
    T, H = h.shape
    if weight.numel() != H or not weight.is_contiguous():
        raise KernelError(f"rmsnorm_add: weight of {weight.numel()} elements for width {H}")
    _call("elementwise", "fx_rmsnorm_add", _stream(), _p(h), _p(y), _p(weight), dtype_code(weight.dtype), T, H, float(eps))


def moe_combine_identity(h, y, ids, weights, x, n_experts: int, post_norm=None) -> None:
    """h[t] += N(sum_j weights[t, j] * (y[t*k + j] if ids[t, j] < n_experts else x[t])), N the RMS norm
    `post_norm` = (weight, eps) or nothing.  y: float32 [T*k, H] in pair order (rows of pairs that chose an
    identity expert, ids >= n_experts, are never used: they need not have been written); x: the feed-forward's input rows [T, H]."""
    T, H = h.shape
    k = ids.shape[1]
    if h.dtype != torch.float32 or y.dtype != torch.float32 or weights.dtype != torch.float32 or not h.is_contiguous():
        raise KernelError("moe_combine_identity works on float32")
    if not y.is_contiguous() or y.shape[0] < T * k or y.shape[1] != H or tuple(x.shape) != (T, H) or not x.is_contiguous():
        raise KernelError(f"moe_combine_identity: y {tuple(y.shape)} / x {tuple(x.shape)} for {T} tokens, {k} choices, width {H}")
    if tuple(weights.shape) != (T, k) or not weights.is_contiguous() or not ids.is_contiguous():
        raise KernelError("moe_combine_identity: ids and weights must be contiguous [T, k]")
    nw, eps = post_norm if post_norm is not None else (None, 0.0)
    if nw is not None and (nw.numel() != H or not nw.is_contiguous()):
        raise KernelError(f"moe_combine_identity: norm weight of {nw.numel()} elements for width {H}")
    out = torch.empty((T, H), dtype=torch.float32, device=h.device)
    _call("elementwise", "fx_moe_combine_identity", _stream(), _p(h), _p(out), _p(y), _p(_i32(ids, "ids")), _p(weights), _p(x),
          dtype_code(x.dtype), T, int(n_experts), H, k, _p(nw), dtype_code(nw.dtype) if nw is not None else 0, float(eps))


def _f32_rows(t, what, cols):
    if t.dtype != torch.float32 or t.dim() != 2 or t.stride(1) != 1 or t.shape[1] < cols:
        raise KernelError(f"{what} must be float32 rows of at least {cols} columns with unit inner stride")
    return t


CONV_ACTIVATIONS = {None: 0, "silu": 1}


def short_conv(x, taps, state, token_seq, seq_starts, slot_ids, n_seqs: int, activation: str | None = "silu", bias=None,
               add_input: bool = False, out_dtype=torch.float32) -> torch.Tensor:
    """y[t, c] = act(sum_j taps[c, n-1-j] x[t-j, c] (+ bias[c])) (+ x[t, c] with `add_input`) over each sequence's own
    tokens, the n-1 inputs from before the step coming from state[slot, c, :] (oldest first), which afterwards holds
    the step's last n-1 inputs.  x: float32 or bfloat16 [T, C] rows (any row stride); taps [C, n] (and bias [C] of
    the taps' type); state float32 [slots, C, n-1]; sequence s owns tokens [seq_starts[s], seq_starts[s+1]) and slot
    slot_ids[s]; `activation` None or "silu".  Returns [T, C] in `out_dtype` (float32, or x's type); the sums are float32."""
    T, C = x.shape
    n = taps.shape[1]
    if activation not in CONV_ACTIVATIONS:
        raise KernelError(f"short_conv: activation '{activation}' is not one of {list(CONV_ACTIVATIONS)}")
    if x.dim() != 2 or x.stride(1) != 1 or out_dtype not in (torch.float32, x.dtype):
        raise KernelError("short_conv: x must be rows with unit inner stride, the output float32 or of x's type")
    if bias is not None and (bias.numel() != C or bias.dtype != taps.dtype or not bias.is_contiguous()):
        raise KernelError(f"short_conv: bias of {bias.numel()} elements ({bias.dtype}) for {C} channels of {taps.dtype} taps")
    if tuple(taps.shape) != (C, n) or not taps.is_contiguous():
        raise KernelError(f"short_conv: taps {tuple(taps.shape)} for {C} channels")
    if state.dtype != torch.float32 or not state.is_contiguous() or tuple(state.shape[1:]) != (C, max(n - 1, 0)):
        raise KernelError(f"short_conv: state {tuple(state.shape)} for [slots, {C}, {n - 1}]")
    if seq_starts.numel() < n_seqs + 1 or slot_ids.numel() < n_seqs or token_seq.numel() < T:
        raise KernelError("short_conv: the step's index tensors are shorter than its sequences and tokens")
    y = torch.empty((T, C), dtype=out_dtype, device=x.device)
    _call("recurrent", "fx_short_conv", _stream(), _p(x), dtype_code(x.dtype), x.stride(0), _p(y), dtype_code(out_dtype),
          y.stride(0), _p(taps), dtype_code(taps.dtype), n,
          _p(state), _p(_i32(token_seq, "token_seq")), _p(_i32(seq_starts, "seq_starts")), _p(_i32(slot_ids, "slot_ids")),
          T, int(n_seqs), C, _p(bias), CONV_ACTIVATIONS[activation], 1 if add_input else 0)
    return y


def delta_prepare(q, k, a, b, A_log, dt_bias, n_heads: int, n_kv_heads: int, key_dim: int, per_head: bool = False):
    """From convolved q, k [T, G*D], the decay's projection a [T, H*D] and the step size's b [T, H] (float32 rows):
    (q / |q| / sqrt(D), k / |k|, exp(-exp(A_log[h]) softplus(a + dt_bias)), sigmoid(b), the normed k . q per q/k head
    [T, G]), all float32 contiguous.  `per_head`: a is [T, H] and dt_bias [H], one decay per head, which all D
    channels of the head receive (the decays returned are [T, H*D] either way)."""
    T = q.shape[0]
    H, G, D = int(n_heads), int(n_kv_heads), int(key_dim)
    Dd = 1 if per_head else D
    _f32_rows(q, "delta_prepare: q", G * D), _f32_rows(k, "delta_prepare: k", G * D)
    _f32_rows(a, "delta_prepare: a", H * Dd), _f32_rows(b, "delta_prepare: b", H)
    if A_log.numel() != H or dt_bias.numel() != H * Dd or A_log.dtype != dt_bias.dtype or not A_log.is_contiguous() \
            or not dt_bias.is_contiguous():
        raise KernelError(f"delta_prepare: A_log {tuple(A_log.shape)} / dt_bias {tuple(dt_bias.shape)} for {H} heads of {D}")
    dev = q.device
    qn = torch.empty((T, G * D), dtype=torch.float32, device=dev)
    kn = torch.empty((T, G * D), dtype=torch.float32, device=dev)
    decay = torch.empty((T, H * D), dtype=torch.float32, device=dev)
    beta = torch.empty((T, H), dtype=torch.float32, device=dev)
    kq = torch.empty((T, G), dtype=torch.float32, device=dev)
    _call("recurrent", "fx_delta_prepare", _stream(), _p(q), q.stride(0), _p(k), k.stride(0), _p(a), a.stride(0), _p(b),
          b.stride(0), _p(A_log), _p(dt_bias), dtype_code(A_log.dtype), _p(qn), _p(kn), _p(decay), _p(beta), _p(kq), T, H, G, D,
          1 if per_head else 0)
    return qn, kn, decay, beta, kq


def channel_delta(qn, kn, decay, beta, kq, v, state, seq_starts, slot_ids, n_seqs: int, n_heads: int, n_kv_heads: int,
                  key_dim: int, v_dim: int) -> torch.Tensor:
    """The gated delta rule with a decay per key channel, over each sequence's tokens in order, from and into
    state[slot] (float32 [slots, H, V, D], the state's transpose: a column's key channels lie together):  S <- diag(decay_t) S;  u = beta_t (v_t - S^T k_t);  S <- S + k_t u^T;
    o_t = S^T q_t.  qn, kn, decay, beta, kq are what `delta_prepare` returns.  Returns o float32 [T, H*V]."""
    T = qn.shape[0]
    H, G, D, V = int(n_heads), int(n_kv_heads), int(key_dim), int(v_dim)
    for t, cols, what in ((qn, G * D, "q"), (kn, G * D, "k"), (decay, H * D, "decay"), (beta, H, "beta"), (kq, G, "k.q")):
        if t.dtype != torch.float32 or not t.is_contiguous() or tuple(t.shape) != (T, cols):
            raise KernelError(f"channel_delta: {what} must be contiguous float32 [{T}, {cols}]")
    _f32_rows(v, "channel_delta: v", H * V)
    if v.shape[0] != T or state.dtype != torch.float32 or not state.is_contiguous() or tuple(state.shape[1:]) != (H, V, D):
        raise KernelError(f"channel_delta: v {tuple(v.shape)} / state {tuple(state.shape)} for [slots, {H}, {V}, {D}]")
    if seq_starts.numel() < n_seqs + 1 or slot_ids.numel() < n_seqs:
        raise KernelError("channel_delta: the step's index tensors are shorter than its sequences")
    out = torch.empty((T, H * V), dtype=torch.float32, device=qn.device)
    _call("recurrent", "fx_channel_delta", _stream(), _p(qn), _p(kn), _p(decay), _p(beta), _p(kq), _p(v), v.stride(0), _p(out),
          out.stride(0), _p(state), _p(_i32(seq_starts, "seq_starts")), _p(_i32(slot_ids, "slot_ids")), int(n_seqs), H, G, D, V)
    return out


HEAD_GATES = {"sigmoid": 0, "silu": 1}


def gated_head_norm(o, gate, weight, eps: float, n_heads: int, v_dim: int, out_dtype, gate_activation: str = "sigmoid",
                    denominators: tuple | None = None) -> torch.Tensor:
    """y[t, h, :] = o[t, h, :] / rms(o[t, h, :]) * weight * act(gate[t, h, :]) in `out_dtype`, act being sigmoid or
    silu; o and gate are float32 rows [T, H*V]; weight is [V], shared by the heads, or [H*V], one per head and channel.
    `denominators` = (nq, m), float32 [T, H] each: o[t, h] is first divided by max(|nq|, exp(-m)) + 1e-6."""
    if gate_activation not in HEAD_GATES:
        raise KernelError(f"gated_head_norm: gate activation '{gate_activation}' is not one of {sorted(HEAD_GATES)}")
    T = o.shape[0]
    H, V = int(n_heads), int(v_dim)
    _f32_rows(o, "gated_head_norm: o", H * V), _f32_rows(gate, "gated_head_norm: gate", H * V)
    if gate.shape[0] != T or weight.numel() not in (V, H * V) or not weight.is_contiguous():
        raise KernelError(f"gated_head_norm: gate {tuple(gate.shape)} / weight {tuple(weight.shape)} for {T} x {H} heads of {V}")
    nq = m = None
    if denominators is not None:
        nq, m = denominators
        for t in (nq, m):
            if t.dtype != torch.float32 or not t.is_contiguous() or tuple(t.shape) != (T, H):
                raise KernelError(f"gated_head_norm: denominators must be contiguous float32 [{T}, {H}]")
    y = torch.empty((T, H * V), dtype=out_dtype, device=o.device)
    _call("recurrent", "fx_gated_head_norm", _stream(), dtype_code(out_dtype), _p(o), o.stride(0), _p(gate), gate.stride(0),
          _p(weight), dtype_code(weight.dtype), 1 if (weight.numel() == H * V and H > 1) else 0, _p(y), y.stride(0), T, H, V,
          float(eps), HEAD_GATES[gate_activation], _p(nq), _p(m))
    return y


def small_rows_parts(x, wt):
    """A block-diagonal float32 product of few rows, one launch: x float32 rows [T, parts * K] (any row stride), wt
    contiguous float32 [parts, K, N] (every part's matrix transposed); returns contiguous [T, parts, N] with
    out[t, j] = x[t, j K:(j + 1) K] @ wt[j], the sums over k ascending in one accumulator, as `gemm` does in float32."""
    T = x.shape[0]
    if wt.dtype != torch.float32 or wt.dim() != 3 or not wt.is_contiguous() or wt.shape[1] > SMALL_ROWS_MAX_K:
        raise KernelError(f"small_rows_parts: transposed weights {tuple(wt.shape)} ({wt.dtype})")
    parts, K, N = wt.shape
    _f32_rows(x, "small_rows_parts: x", parts * K)
    out = torch.empty((T, parts, N), dtype=torch.float32, device=x.device)
    _call("recurrent", "fx_small_rows_parts", _stream(), _p(x), x.stride(0), _p(wt), _p(out), K, N, parts, T)
    return out


def gated_outer(q, k, v, keep, take, state, seq_starts, slot_ids, n_seqs: int, n_heads: int, n_kv_heads: int, key_dim: int,
                v_dim: int, q_scale: float = 1.0, normalizer: bool = False):
    """A matrix memory with one forgetting and one writing factor per head and token, over each sequence's tokens in
    order, from and into state[slot]:  S <- keep_t S + take_t k_t v_t^T;  o_t = q_scale S^T q_t.  q, k: float32 rows
    [T, G*D]; v [T, H*V]; `keep` float32 [T, H], or [H] (the same factors at every token); `take` float32 [T, H] or
    None (1).  The state is float32 [slots, H, V, D] (transposed).  With `normalizer` it is [slots, H, V + 1, D]: its
    last column is n <- keep_t n + take_t k_t, and the call also returns nq [T, H] = q_scale n_t . q_t.
    Returns o float32 [T, H*V], or (o, nq)."""
    T = q.shape[0]
    H, G, D, V = int(n_heads), int(n_kv_heads), int(key_dim), int(v_dim)
    _f32_rows(q, "gated_outer: q", G * D), _f32_rows(k, "gated_outer: k", G * D), _f32_rows(v, "gated_outer: v", H * V)
    keep_const = keep.dim() == 1
    if keep.dtype != torch.float32 or not keep.is_contiguous() or tuple(keep.shape) not in ((H,), (T, H)):
        raise KernelError(f"gated_outer: forgetting factors {tuple(keep.shape)} for [{T}, {H}] or [{H}]")
    if take is not None and (take.dtype != torch.float32 or not take.is_contiguous() or tuple(take.shape) != (T, H)):
        raise KernelError(f"gated_outer: writing factors must be contiguous float32 [{T}, {H}]")
    VS = V + (1 if normalizer else 0)
    if k.shape[0] != T or v.shape[0] != T or state.dtype != torch.float32 or not state.is_contiguous() \
            or tuple(state.shape[1:]) != (H, VS, D):
        raise KernelError(f"gated_outer: k {tuple(k.shape)} / v {tuple(v.shape)} / state {tuple(state.shape)} for [slots, {H}, {VS}, {D}]")
    if seq_starts.numel() < n_seqs + 1 or slot_ids.numel() < n_seqs:
        raise KernelError("gated_outer: the step's index tensors are shorter than its sequences")
    out = torch.empty((T, H * V), dtype=torch.float32, device=q.device)
    nq = torch.empty((T, H), dtype=torch.float32, device=q.device) if normalizer else None
    _call("recurrent", "fx_gated_outer", _stream(), _p(q), q.stride(0), _p(k), k.stride(0), _p(v), v.stride(0), _p(keep),
          1 if keep_const else 0, _p(take), _p(out), out.stride(0), _p(nq), _p(state), _p(_i32(seq_starts, "seq_starts")),
          _p(_i32(slot_ids, "slot_ids")), int(n_seqs), H, G, D, V, float(q_scale))
    return (out, nq) if normalizer else out


def exp_gate_scan(x_in, x_forget, cap: float, state, seq_starts, slot_ids, n_seqs: int, n_heads: int):
    """Exponential gates under a running maximum, per head over each sequence's tokens in order.  From the float32
    rows x_in, x_forget [T, H]:  i = cap tanh(x_in / cap);  f = logsigmoid(cap tanh(x_forget / cap));
    m_t = max(f + m_(t-1), i);  keep_t = exp(f + m_(t-1) - m_t);  take_t = exp(i - m_t).  m is carried in
    state [slots, H] (float32).  Returns (keep, take, m), float32 [T, H] each."""
    T, H = x_in.shape[0], int(n_heads)
    _f32_rows(x_in, "exp_gate_scan: x_in", H), _f32_rows(x_forget, "exp_gate_scan: x_forget", H)
    if x_forget.shape[0] != T or state.dtype != torch.float32 or not state.is_contiguous() or tuple(state.shape[1:]) != (H,):
        raise KernelError(f"exp_gate_scan: state {tuple(state.shape)} for [slots, {H}]")
    if seq_starts.numel() < n_seqs + 1 or slot_ids.numel() < n_seqs:
        raise KernelError("exp_gate_scan: the step's index tensors are shorter than its sequences")
    keep, take, m = (torch.empty((T, H), dtype=torch.float32, device=x_in.device) for _ in range(3))
    _call("recurrent", "fx_exp_gate_scan", _stream(), _p(x_in), x_in.stride(0), _p(x_forget), x_forget.stride(0), float(cap),
          _p(keep), _p(take), _p(m), _p(state), _p(_i32(seq_starts, "seq_starts")), _p(_i32(slot_ids, "slot_ids")),
          int(n_seqs), H)
    return keep, take, m


def rglru(u, gate_logits, gate_bias, n_parts: int, lam, branch, state, seq_starts, slot_ids, n_seqs: int, longest: int,
          out_dtype, rate: float = 8.0) -> torch.Tensor:
    """The real-gated linear recurrent unit per channel, over each sequence's tokens in order, from and into
    state[slot] (float32 [slots, C]):  a = exp(-rate sigmoid(r) softplus(lam));
    S_t = a_t S_(t-1) + sqrt(1 - a_t^2) sigmoid(i) u_t;  y_t = S_t gelu_tanh(branch_t).  u, branch: float32 rows
    [T, C]; lam [C].  The gates' logits r and i come as the products of the channels' `n_parts` parts leave them:
    gate_logits contiguous float32 [T, n_parts, 2, C / n_parts] (recurrence gate, then input gate), plus gate_bias
    of shape [n_parts, 2, C / n_parts] (or None).  `longest`: the most tokens a sequence of the step brings (it picks
    how a sequence's tokens are dealt out to waves).  Returns y [T, C] in `out_dtype`."""
    T, C = u.shape
    for t, what in ((u, "u"), (branch, "branch")):
        _f32_rows(t, f"rglru: {what}", C)
        if t.shape[0] != T:
            raise KernelError(f"rglru: {what} has {t.shape[0]} rows, u {T}")
    if n_parts < 1 or C % n_parts or gate_logits.dtype != torch.float32 or not gate_logits.is_contiguous() \
            or gate_logits.numel() != 2 * T * C:
        raise KernelError(f"rglru: gate logits {tuple(gate_logits.shape)} for {T} tokens, {n_parts} parts of {C} channels")
    if gate_bias is not None and (gate_bias.dtype != torch.float32 or not gate_bias.is_contiguous() or gate_bias.numel() != 2 * C):
        raise KernelError(f"rglru: the gates' bias must hold {2 * C} contiguous float32 values")
    if lam.numel() != C or not lam.is_contiguous() or state.dtype != torch.float32 or not state.is_contiguous() \
            or tuple(state.shape[1:]) != (C,):
        raise KernelError(f"rglru: lam {tuple(lam.shape)} / state {tuple(state.shape)} for {C} channels")
    if seq_starts.numel() < n_seqs + 1 or slot_ids.numel() < n_seqs:
        raise KernelError("rglru: the step's index tensors are shorter than its sequences")
    a = torch.empty((T, C), dtype=torch.float32, device=u.device)
    x = torch.empty((T, C), dtype=torch.float32, device=u.device)
    _call("recurrent", "fx_rglru_gates", _stream(), _p(u), u.stride(0), _p(gate_logits), _p(gate_bias), _p(lam),
          dtype_code(lam.dtype), float(rate), _p(a), _p(x), T, C, int(n_parts))
    y = torch.empty((T, C), dtype=out_dtype, device=u.device)
    _call("recurrent", "fx_rglru_scan", _stream(), dtype_code(out_dtype), _p(a), _p(x), _p(branch), branch.stride(0), _p(y),
          y.stride(0), _p(state), _p(_i32(seq_starts, "seq_starts")), _p(_i32(slot_ids, "slot_ids")), int(n_seqs), C,
          int(longest))
    return y


SMALL_ROWS_MAX = 32          # up to so many rows the pair of small float32 products is one launch (more rows: the tiled product)
SMALL_ROWS_MAX_K = 512


def small_rows_pair(x0, wt0, x1, wt1):
    """(x0 @ wt0, x1 @ wt1) in float32 for few rows, one launch: x_i float32 rows [T, K_i] (any row stride),
    wt_i contiguous float32 [K_i, N_i] (the weights transposed).  The sums run over k ascending in one accumulator,
    as `gemm` does in float32."""
    T = x0.shape[0]
    for x, wt in ((x0, wt0), (x1, wt1)):
        _f32_rows(x, "small_rows_pair: x", wt.shape[0])
        if wt.dtype != torch.float32 or wt.dim() != 2 or not wt.is_contiguous() or x.shape[1] != wt.shape[0] \
                or wt.shape[0] > SMALL_ROWS_MAX_K or x.shape[0] != T:
            raise KernelError(f"small_rows_pair: rows {tuple(x.shape)} against transposed weights {tuple(wt.shape)}")
    out0 = torch.empty((T, wt0.shape[1]), dtype=torch.float32, device=x0.device)
    out1 = torch.empty((T, wt1.shape[1]), dtype=torch.float32, device=x0.device)
    _call("recurrent", "fx_small_rows_pair", _stream(), _p(x0), x0.stride(0), _p(wt0), _p(out0), out0.stride(0), wt0.shape[0],
          wt0.shape[1], _p(x1), x1.stride(0), _p(wt1), _p(out1), out1.stride(0), wt1.shape[0], wt1.shape[1], T)
    return out0, out1
