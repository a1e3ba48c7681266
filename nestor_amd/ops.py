"""``torch.library`` custom ops (namespace ``nestor_hip``) over the C ABI.

Each op allocates its outputs with torch, passes raw device pointers and the
current HIP stream to ``libnestor_hip.so`` and returns; none reads device memory
on the host, so a forward+backward enqueues without a single synchronisation.
Every op has a fake (meta) kernel, and the differentiable ones register their
backward as further custom ops, so the path traces under ``torch.compile``.

Ops only exist for CUDA/HIP tensors: calling one with CPU tensors raises.
"""

from __future__ import annotations

import ctypes

import torch
from torch import Tensor

from nestor_amd import _lib

_NS = "nestor_hip"


def _ptr(t: Tensor | None) -> ctypes.c_void_p | None:
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _stream(t: Tensor) -> ctypes.c_void_p:
    return ctypes.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def _code(dtype: torch.dtype) -> int:
    if dtype == torch.float32:
        return _lib.F32
    if dtype == torch.bfloat16:
        return _lib.BF16
    raise TypeError(f"nestor_hip kernels take float32 or bfloat16 here, got {dtype}")


def _bf16(t: Tensor, name: str) -> Tensor:
    if t.dtype != torch.bfloat16:
        raise TypeError(f"{name} must be bfloat16 (the GEMM dtype of the HIP path), got {t.dtype}")
    return t.contiguous()


def rows_pad_for(rows: int, num_banks: int) -> int:
    a = _lib.ROW_ALIGN
    return ((rows + a - 1) // a) * a + a * num_banks


def max_tiles_for(rows_pad: int, num_banks: int) -> int:
    return rows_pad // _lib.TILE_M + num_banks + 2


def tile_table_ints(rows_pad: int, num_banks: int) -> int:
    """int32 entries of a tile_table buffer: the 128-row table and the two balanced tables
    (tiles of up to 160 and up to 320 rows), each ``3 * cap + 1``
    (``nestor_hip_tile_table_ints``)."""

    cap = max_tiles_for(rows_pad, num_banks)
    caps = (cap, cap, rows_pad // 256 + num_banks + 2)
    return sum(3 * c + 1 for c in caps)


# --------------------------------------------------------------------------
# Index build
# --------------------------------------------------------------------------
@torch.library.custom_op(f"{_NS}::index_build", mutates_args=(), device_types="cuda")
def index_build(
    expert_ids: Tensor, num_banks: int, slots: int, capacity: int, valid_dtype: torch.dtype
) -> list[Tensor]:
    """[order, counts, raw_starts, padded_starts, offs, row_dest, pad_token,
    pad_src_row, eid_pad, pad_valid, row_kept, tile_table]."""

    ids = expert_ids.contiguous()
    assert ids.dtype == torch.long and ids.dim() == 1
    rows = ids.shape[0]
    dev = ids.device
    rows_pad = rows_pad_for(rows, num_banks)
    max_tiles = max_tiles_for(rows_pad, num_banks)
    i64 = dict(dtype=torch.long, device=dev)
    order = torch.empty(rows, **i64)
    counts = torch.empty(num_banks, **i64)
    raw_starts = torch.empty(num_banks, **i64)
    padded_starts = torch.empty(num_banks, **i64)
    offs = torch.empty(num_banks, dtype=torch.int32, device=dev)
    row_dest = torch.empty(rows, **i64)
    pad_token = torch.empty(rows_pad, **i64)
    pad_src_row = torch.empty(rows_pad, **i64)
    eid_pad = torch.empty(rows_pad, **i64)
    pad_valid = torch.empty(rows_pad, dtype=valid_dtype, device=dev)
    row_kept = torch.empty(rows, dtype=torch.uint8, device=dev)
    tile_table = torch.empty(tile_table_ints(rows_pad, num_banks), dtype=torch.int32, device=dev)
    ws_bytes = _lib.load().nestor_hip_index_build_workspace_bytes(rows, num_banks)
    workspace = torch.empty(max(ws_bytes, 4), dtype=torch.uint8, device=dev)
    _lib.call(
        "nestor_hip_index_build", _ptr(ids), rows, num_banks, slots, rows_pad, capacity,
        _code(valid_dtype), _ptr(order), _ptr(counts), _ptr(raw_starts), _ptr(padded_starts),
        _ptr(offs), _ptr(row_dest), _ptr(pad_token), _ptr(pad_src_row), _ptr(eid_pad),
        _ptr(pad_valid), _ptr(row_kept), _ptr(tile_table), max_tiles, _ptr(workspace),
        workspace.numel(), _stream(ids),
    )
    return [order, counts, raw_starts, padded_starts, offs, row_dest, pad_token,
            pad_src_row, eid_pad, pad_valid, row_kept, tile_table]


@index_build.register_fake
def _(expert_ids, num_banks, slots, capacity, valid_dtype):
    rows = expert_ids.shape[0]
    rows_pad = rows_pad_for(rows, num_banks)
    max_tiles = max_tiles_for(rows_pad, num_banks)
    new = expert_ids.new_empty
    return [
        new(rows), new(num_banks), new(num_banks), new(num_banks),
        new(num_banks, dtype=torch.int32), new(rows), new(rows_pad), new(rows_pad),
        new(rows_pad), new(rows_pad, dtype=valid_dtype), new(rows, dtype=torch.uint8),
        new(tile_table_ints(rows_pad, num_banks), dtype=torch.int32),
    ]


@torch.library.custom_op(f"{_NS}::build_dispatch_maps", mutates_args=(), device_types="cuda")
def build_dispatch_maps_op(
    expert_ids: Tensor, order: Tensor, padded_starts: Tensor, raw_starts: Tensor,
    slots: int, rows_pad: int, valid_dtype: torch.dtype,
) -> list[Tensor]:
    ids = expert_ids.contiguous()
    order = order.contiguous()
    padded_starts = padded_starts.contiguous()
    raw_starts = raw_starts.contiguous()
    rows = order.shape[0]
    dev = order.device
    num_banks = padded_starts.shape[0]
    row_dest = torch.empty(rows, dtype=torch.long, device=dev)
    pad_token = torch.empty(rows_pad, dtype=torch.long, device=dev)
    pad_src_row = torch.empty(rows_pad, dtype=torch.long, device=dev)
    eid_pad = torch.empty(rows_pad, dtype=torch.long, device=dev)
    pad_valid = torch.empty(rows_pad, dtype=valid_dtype, device=dev)
    _lib.call(
        "nestor_hip_build_dispatch_maps", _ptr(ids), _ptr(order), _ptr(padded_starts),
        _ptr(raw_starts), rows, num_banks, slots, rows_pad, _code(valid_dtype),
        _ptr(row_dest), _ptr(pad_token), _ptr(pad_src_row), _ptr(eid_pad), _ptr(pad_valid),
        _stream(order),
    )
    return [row_dest, pad_token, pad_src_row, eid_pad, pad_valid]


@build_dispatch_maps_op.register_fake
def _(expert_ids, order, padded_starts, raw_starts, slots, rows_pad, valid_dtype):
    rows = order.shape[0]
    new = order.new_empty
    return [new(rows), new(rows_pad), new(rows_pad), new(rows_pad),
            new(rows_pad, dtype=valid_dtype)]


@torch.library.custom_op(f"{_NS}::tile_schedule", mutates_args=(), device_types="cuda")
def tile_schedule(offs: Tensor, rows_pad: int) -> Tensor:
    offs = offs.contiguous()
    assert offs.dtype == torch.int32
    num_banks = offs.shape[0]
    max_tiles = max_tiles_for(rows_pad, num_banks)
    table = torch.empty(tile_table_ints(rows_pad, num_banks), dtype=torch.int32,
                        device=offs.device)
    _lib.call("nestor_hip_tile_schedule", _ptr(offs), num_banks, rows_pad, _ptr(table), max_tiles,
              _stream(offs))
    return table


@tile_schedule.register_fake
def _(offs, rows_pad):
    return offs.new_empty(tile_table_ints(rows_pad, offs.shape[0]))


def _table_max_tiles(tile_table: Tensor, rows_pad: int, num_banks: int) -> int:
    """Capacity of the buffer's first (128-row) table; the buffer must be the one built for
    these sizes (the GEMMs locate its other tables from the sizes alone)."""

    if tile_table.shape[0] != tile_table_ints(rows_pad, num_banks):
        raise ValueError(
            f"tile_table has {tile_table.shape[0]} entries; a table for rows_pad={rows_pad}, "
            f"{num_banks} banks has {tile_table_ints(rows_pad, num_banks)}"
        )
    return max_tiles_for(rows_pad, num_banks)


# --------------------------------------------------------------------------
# Row moves
# --------------------------------------------------------------------------
@torch.library.custom_op(f"{_NS}::dispatch_rows_fwd", mutates_args=(), device_types="cuda")
def dispatch_rows_fwd(
    x: Tensor, pad_token: Tensor, pad_valid: Tensor, row_dest: Tensor | None = None,
    slots: int = 0,
) -> Tensor:
    """``row_dest`` / ``slots`` (the inverse map) select the source-major kernel."""

    x = x.contiguous()
    rows_pad = pad_token.shape[0]
    out = torch.empty(rows_pad, x.shape[1], dtype=torch.bfloat16, device=x.device)
    scatter = row_dest is not None and slots > 0
    _lib.call(
        "nestor_hip_dispatch_rows_fwd", _ptr(x), _code(x.dtype), _ptr(pad_token.contiguous()),
        _ptr(pad_valid.contiguous()), _code(pad_valid.dtype), _ptr(out), rows_pad,
        x.shape[1], _ptr(row_dest.contiguous()) if scatter else None,
        x.shape[0] if scatter else 0, slots if scatter else 0, _stream(x),
    )
    return out


@dispatch_rows_fwd.register_fake
def _(x, pad_token, pad_valid, row_dest=None, slots=0):
    return x.new_empty(pad_token.shape[0], x.shape[1], dtype=torch.bfloat16)


@torch.library.custom_op(f"{_NS}::dispatch_rows_bwd", mutates_args=(), device_types="cuda")
def dispatch_rows_bwd(
    grad_pad: Tensor, row_dest: Tensor, num_tokens: int, slots: int, x_dtype: torch.dtype
) -> Tensor:
    grad_pad = _bf16(grad_pad, "grad_pad")
    dim = grad_pad.shape[1]
    out = torch.empty(num_tokens, dim, dtype=x_dtype, device=grad_pad.device)
    _lib.call(
        "nestor_hip_dispatch_rows_bwd", _ptr(grad_pad), _ptr(row_dest.contiguous()), _ptr(out),
        _code(x_dtype), num_tokens, slots, dim, _stream(grad_pad),
    )
    return out


@dispatch_rows_bwd.register_fake
def _(grad_pad, row_dest, num_tokens, slots, x_dtype):
    return grad_pad.new_empty(num_tokens, grad_pad.shape[1], dtype=x_dtype)


@torch.library.custom_op(f"{_NS}::dispatch_rows", mutates_args=(), device_types="cuda")
def dispatch_rows_op(
    x: Tensor, pad_token: Tensor, pad_valid: Tensor, row_dest: Tensor, slots: int,
    source_major: bool = True,
) -> Tensor:
    """``source_major``: the forward may walk the tokens and write each to the rows
    ``row_dest`` names (every token read once).  That form writes a real padded row only
    if ``row_dest`` points back at it, which holds for the plans of ``index_build``; with
    ``source_major=False`` the forward gathers every real row through ``pad_token`` alone
    and ``row_dest`` only serves the backward."""

    if source_major:
        return dispatch_rows_fwd(x, pad_token, pad_valid, row_dest, slots)
    return dispatch_rows_fwd(x, pad_token, pad_valid, None, 0)


@dispatch_rows_op.register_fake
def _(x, pad_token, pad_valid, row_dest, slots, source_major=True):
    return x.new_empty(pad_token.shape[0], x.shape[1], dtype=torch.bfloat16)


def _dispatch_setup(ctx, inputs, output):
    x, _pad_token, _pad_valid, row_dest, slots, _source_major = inputs
    ctx.save_for_backward(row_dest)
    ctx.slots = slots
    ctx.num_tokens = x.shape[0]
    ctx.x_dtype = x.dtype


def _dispatch_backward(ctx, grad_pad):
    (row_dest,) = ctx.saved_tensors
    gx = dispatch_rows_bwd(grad_pad, row_dest, ctx.num_tokens, ctx.slots, ctx.x_dtype)
    return gx, None, None, None, None, None


dispatch_rows_op.register_autograd(_dispatch_backward, setup_context=_dispatch_setup)


@torch.library.custom_op(f"{_NS}::swiglu_fwd", mutates_args=(), device_types="cuda")
def swiglu_fwd(up_gate: Tensor, hidden: int) -> Tensor:
    """``up_gate`` is ``[rows, 2*hidden]`` (up | gate)."""

    up_gate = _bf16(up_gate, "up_gate")
    rows = up_gate.shape[0]
    out = torch.empty(rows, hidden, dtype=torch.bfloat16, device=up_gate.device)
    base = up_gate.data_ptr()
    _lib.call(
        "nestor_hip_swiglu_fwd", ctypes.c_void_p(base), ctypes.c_void_p(base + 2 * hidden),
        _ptr(out), rows, hidden, 2 * hidden, hidden, _stream(up_gate),
    )
    return out


@swiglu_fwd.register_fake
def _(up_gate, hidden):
    return up_gate.new_empty(up_gate.shape[0], hidden)


@torch.library.custom_op(f"{_NS}::swiglu_bwd", mutates_args=(), device_types="cuda")
def swiglu_bwd(grad_out: Tensor, up_gate: Tensor, hidden: int) -> Tensor:
    grad_out = _bf16(grad_out, "grad_out")
    up_gate = _bf16(up_gate, "up_gate")
    rows = up_gate.shape[0]
    grad = torch.empty_like(up_gate)
    base = up_gate.data_ptr()
    gbase = grad.data_ptr()
    _lib.call(
        "nestor_hip_swiglu_bwd", _ptr(grad_out), ctypes.c_void_p(base),
        ctypes.c_void_p(base + 2 * hidden), ctypes.c_void_p(gbase),
        ctypes.c_void_p(gbase + 2 * hidden), rows, hidden, 2 * hidden, 2 * hidden, hidden,
        _stream(up_gate),
    )
    return grad


@swiglu_bwd.register_fake
def _(grad_out, up_gate, hidden):
    return torch.empty_like(up_gate)


@torch.library.custom_op(f"{_NS}::swiglu_fused", mutates_args=(), device_types="cuda")
def swiglu_fused_op(up_gate: Tensor, hidden: int) -> Tensor:
    return swiglu_fwd(up_gate, hidden)


@swiglu_fused_op.register_fake
def _(up_gate, hidden):
    return up_gate.new_empty(up_gate.shape[0], hidden)


def _swiglu_fused_setup(ctx, inputs, output):
    up_gate, hidden = inputs
    ctx.save_for_backward(up_gate)
    ctx.hidden = hidden


def _swiglu_fused_backward(ctx, grad_out):
    (up_gate,) = ctx.saved_tensors
    return swiglu_bwd(grad_out, up_gate, ctx.hidden), None


swiglu_fused_op.register_autograd(_swiglu_fused_backward, setup_context=_swiglu_fused_setup)


@torch.library.custom_op(f"{_NS}::swiglu_split_fwd", mutates_args=(), device_types="cuda")
def swiglu_split_fwd(up: Tensor, gate: Tensor) -> Tensor:
    up = _bf16(up, "up")
    gate = _bf16(gate, "gate")
    rows, hidden = up.shape
    out = torch.empty_like(up)
    _lib.call("nestor_hip_swiglu_fwd", _ptr(up), _ptr(gate), _ptr(out), rows, hidden, hidden,
              hidden, _stream(up))
    return out


@swiglu_split_fwd.register_fake
def _(up, gate):
    return torch.empty_like(up)


@torch.library.custom_op(f"{_NS}::swiglu_split_bwd", mutates_args=(), device_types="cuda")
def swiglu_split_bwd(grad_out: Tensor, up: Tensor, gate: Tensor) -> list[Tensor]:
    grad_out = _bf16(grad_out, "grad_out")
    up = _bf16(up, "up")
    gate = _bf16(gate, "gate")
    rows, hidden = up.shape
    gup = torch.empty_like(up)
    ggate = torch.empty_like(gate)
    _lib.call(
        "nestor_hip_swiglu_bwd", _ptr(grad_out), _ptr(up), _ptr(gate), _ptr(gup), _ptr(ggate),
        rows, hidden, hidden, hidden, hidden, _stream(up),
    )
    return [gup, ggate]


@swiglu_split_bwd.register_fake
def _(grad_out, up, gate):
    return [torch.empty_like(up), torch.empty_like(gate)]


@torch.library.custom_op(f"{_NS}::swiglu", mutates_args=(), device_types="cuda")
def swiglu_op(up: Tensor, gate: Tensor) -> Tensor:
    return swiglu_split_fwd(up, gate)


@swiglu_op.register_fake
def _(up, gate):
    return torch.empty_like(up)


def _swiglu_setup(ctx, inputs, output):
    ctx.save_for_backward(*inputs)


def _swiglu_backward(ctx, grad_out):
    up, gate = ctx.saved_tensors
    gup, ggate = swiglu_split_bwd(grad_out, up, gate)
    return gup, ggate


swiglu_op.register_autograd(_swiglu_backward, setup_context=_swiglu_setup)


@torch.library.custom_op(f"{_NS}::cat_cast_fwd", mutates_args=(), device_types="cuda")
def cat_cast_fwd(a: Tensor, b: Tensor) -> Tensor:
    a = a.contiguous()
    b = b.contiguous()
    assert a.dtype == torch.float32 and b.dtype == torch.float32
    hidden = a.shape[-1]
    rows = a.numel() // hidden
    out = torch.empty(*a.shape[:-1], 2 * hidden, dtype=torch.bfloat16, device=a.device)
    _lib.call("nestor_hip_cat_cast_fwd", _ptr(a), _ptr(b), _ptr(out), rows, hidden, _stream(a))
    return out


@cat_cast_fwd.register_fake
def _(a, b):
    return a.new_empty(*a.shape[:-1], 2 * a.shape[-1], dtype=torch.bfloat16)


@torch.library.custom_op(f"{_NS}::cat_cast_bwd", mutates_args=(), device_types="cuda")
def cat_cast_bwd(grad: Tensor) -> list[Tensor]:
    grad = _bf16(grad, "grad")
    hidden = grad.shape[-1] // 2
    rows = grad.numel() // (2 * hidden)
    shape = (*grad.shape[:-1], hidden)
    ga = torch.empty(shape, dtype=torch.float32, device=grad.device)
    gb = torch.empty(shape, dtype=torch.float32, device=grad.device)
    _lib.call("nestor_hip_cat_cast_bwd", _ptr(grad), _ptr(ga), _ptr(gb), rows, hidden,
              _stream(grad))
    return [ga, gb]


@cat_cast_bwd.register_fake
def _(grad):
    shape = (*grad.shape[:-1], grad.shape[-1] // 2)
    return [grad.new_empty(shape, dtype=torch.float32), grad.new_empty(shape, dtype=torch.float32)]


@torch.library.custom_op(f"{_NS}::cat_cast", mutates_args=(), device_types="cuda")
def cat_cast_op(a: Tensor, b: Tensor) -> Tensor:
    return cat_cast_fwd(a, b)


@cat_cast_op.register_fake
def _(a, b):
    return a.new_empty(*a.shape[:-1], 2 * a.shape[-1], dtype=torch.bfloat16)


def _cat_cast_backward(ctx, grad):
    ga, gb = cat_cast_bwd(grad)
    return ga, gb


cat_cast_op.register_autograd(_cat_cast_backward)


@torch.library.custom_op(f"{_NS}::combine_rows_fwd", mutates_args=(), device_types="cuda")
def combine_rows_fwd(
    y_pad: Tensor, row_dest: Tensor, weights: Tensor, group: int, out_dtype: torch.dtype,
    round_term: bool,
) -> Tensor:
    y_pad = _bf16(y_pad, "y_pad")
    weights = weights.contiguous()
    rows = row_dest.shape[0]
    n_out = rows // group
    dim = y_pad.shape[1]
    out = torch.empty(n_out, dim, dtype=out_dtype, device=y_pad.device)
    _lib.call(
        "nestor_hip_combine_rows_fwd", _ptr(y_pad), _ptr(row_dest.contiguous()), _ptr(weights),
        _code(weights.dtype), _ptr(out), _code(out_dtype), n_out, group, dim,
        1 if round_term else 0, _stream(y_pad),
    )
    return out


@combine_rows_fwd.register_fake
def _(y_pad, row_dest, weights, group, out_dtype, round_term):
    return y_pad.new_empty(row_dest.shape[0] // group, y_pad.shape[1], dtype=out_dtype)


@torch.library.custom_op(f"{_NS}::combine_rows_bwd", mutates_args=(), device_types="cuda")
def combine_rows_bwd(
    grad_out: Tensor, y_pad: Tensor, pad_src_row: Tensor, pad_valid: Tensor, weights: Tensor,
    group: int, need_w: bool, row_dest: Tensor | None = None,
) -> list[Tensor]:
    """``row_dest`` (the inverse map, optional) lets a gradient row that ``group > 1``
    routed rows share be read once for all of them; same values either way."""

    grad_out = grad_out.contiguous()
    y_pad = _bf16(y_pad, "y_pad")
    weights = weights.contiguous()
    rows_pad, dim = y_pad.shape
    grad_y = torch.empty_like(y_pad)
    # Rows that own no padded slot (dropped by a capacity limit) keep gradient 0.
    grad_w = torch.zeros(weights.shape[0], dtype=torch.float32, device=y_pad.device)
    _lib.call(
        "nestor_hip_combine_rows_bwd", _ptr(grad_out), _code(grad_out.dtype), _ptr(y_pad),
        _ptr(pad_src_row.contiguous()), _ptr(pad_valid.contiguous()), _code(pad_valid.dtype),
        _ptr(weights), _code(weights.dtype), _ptr(grad_y), _ptr(grad_w) if need_w else None,
        rows_pad, group, dim, _ptr(row_dest.contiguous()) if row_dest is not None else None,
        weights.shape[0] // group, _stream(y_pad),
    )
    return [grad_y, grad_w]


@combine_rows_bwd.register_fake
def _(grad_out, y_pad, pad_src_row, pad_valid, weights, group, need_w, row_dest=None):
    return [torch.empty_like(y_pad), y_pad.new_empty(weights.shape[0], dtype=torch.float32)]


@torch.library.custom_op(f"{_NS}::combine_rows", mutates_args=(), device_types="cuda")
def combine_rows_op(
    y_pad: Tensor, row_dest: Tensor, pad_src_row: Tensor, pad_valid: Tensor, weights: Tensor,
    group: int, out_dtype: torch.dtype,
) -> Tensor:
    promoted = torch.promote_types(y_pad.dtype, weights.dtype)
    round_term = promoted != torch.float32 or out_dtype != torch.float32
    return combine_rows_fwd(y_pad, row_dest, weights, group, out_dtype, round_term)


@combine_rows_op.register_fake
def _(y_pad, row_dest, pad_src_row, pad_valid, weights, group, out_dtype):
    return y_pad.new_empty(row_dest.shape[0] // group, y_pad.shape[1], dtype=out_dtype)


def _combine_setup(ctx, inputs, output):
    y_pad, row_dest, pad_src_row, pad_valid, weights, group, _out_dtype = inputs
    ctx.save_for_backward(y_pad, pad_src_row, pad_valid, weights, row_dest)
    ctx.group = group


def _combine_backward(ctx, grad_out):
    y_pad, pad_src_row, pad_valid, weights, row_dest = ctx.saved_tensors
    need_w = ctx.needs_input_grad[4]
    grad_y, grad_w = combine_rows_bwd(
        grad_out, y_pad, pad_src_row, pad_valid, weights, ctx.group, need_w, row_dest
    )
    return grad_y, None, None, None, grad_w.to(weights.dtype) if need_w else None, None, None


combine_rows_op.register_autograd(_combine_backward, setup_context=_combine_setup)


# --------------------------------------------------------------------------
# Grouped GEMMs
# --------------------------------------------------------------------------
@torch.library.custom_op(f"{_NS}::grouped_gemm_nn", mutates_args=(), device_types="cuda")
def grouped_gemm_nn(a: Tensor, b: Tensor, tile_table: Tensor) -> Tensor:
    a = _bf16(a, "a")
    b = _bf16(b, "b")
    rows_pad, k = a.shape
    num_banks, kb, n = b.shape
    assert kb == k
    out = torch.empty(rows_pad, n, dtype=torch.bfloat16, device=a.device)
    _lib.call(
        "nestor_hip_grouped_gemm_nn", _ptr(a), _ptr(b), _ptr(out), rows_pad, k, n, num_banks,
        _ptr(tile_table), _table_max_tiles(tile_table, rows_pad, num_banks), _stream(a),
    )
    return out


@grouped_gemm_nn.register_fake
def _(a, b, tile_table):
    return a.new_empty(a.shape[0], b.shape[2])


@torch.library.custom_op(f"{_NS}::grouped_gemm_nt", mutates_args=(), device_types="cuda")
def grouped_gemm_nt(a: Tensor, b: Tensor, tile_table: Tensor) -> Tensor:
    """``a [rows, K] @ b[bank]^T`` with ``b [E, N, K]``."""

    a = _bf16(a, "a")
    b = _bf16(b, "b")
    rows_pad, k = a.shape
    num_banks, n, kb = b.shape
    assert kb == k
    out = torch.empty(rows_pad, n, dtype=torch.bfloat16, device=a.device)
    _lib.call(
        "nestor_hip_grouped_gemm_nt", _ptr(a), _ptr(b), _ptr(out), rows_pad, k, n, num_banks,
        _ptr(tile_table), _table_max_tiles(tile_table, rows_pad, num_banks), _stream(a),
    )
    return out


@grouped_gemm_nt.register_fake
def _(a, b, tile_table):
    return a.new_empty(a.shape[0], b.shape[1])


@torch.library.custom_op(f"{_NS}::grouped_gemm_tn", mutates_args=(), device_types="cuda")
def grouped_gemm_tn(
    a: Tensor, g: Tensor, offs: Tensor, seg_start: Tensor | None, seg_count: Tensor | None,
    out_f32: bool = False,
) -> Tensor:
    """``out[e] = a[seg e]^T @ g[seg e]`` -> ``[E, M, N]``, bf16 or (``out_f32``) fp32
    straight from the fp32 accumulators.  ``a`` / ``g`` may be column slices of wider
    row-major tensors (unit inner stride)."""

    assert a.dtype == torch.bfloat16 and g.dtype == torch.bfloat16
    assert a.stride(1) == 1 and g.stride(1) == 1
    rows_pad, m = a.shape
    n = g.shape[1]
    num_banks = offs.shape[0]
    out_dtype = torch.float32 if out_f32 else torch.bfloat16
    out = torch.empty(num_banks, m, n, dtype=out_dtype, device=a.device)
    _lib.call(
        "nestor_hip_grouped_gemm_tn", _ptr(a), a.stride(0), _ptr(g), g.stride(0), _ptr(out), n,
        m * n, rows_pad, m, n, num_banks, _ptr(offs.contiguous()), _ptr(seg_start),
        _ptr(seg_count), _code(out_dtype), _stream(a),
    )
    return out


@grouped_gemm_tn.register_fake
def _(a, g, offs, seg_start, seg_count, out_f32=False):
    return a.new_empty(offs.shape[0], a.shape[1], g.shape[1],
                       dtype=torch.float32 if out_f32 else torch.bfloat16)


@torch.library.custom_op(f"{_NS}::grouped_gemm_tn_pair", mutates_args=(), device_types="cuda")
def grouped_gemm_tn_pair(
    a: Tensor, g: Tensor, offs: Tensor, seg_start: Tensor | None, seg_count: Tensor | None,
    out_f32: bool = False,
) -> list[Tensor]:
    """``[a_seg^T @ g_seg[:, :N], a_seg^T @ g_seg[:, N:]]`` for ``g [rows_pad, 2N]``: the
    weight gradients of the fused up|gate GEMM, one launch when ``N % 256 == 0``."""

    assert a.dtype == torch.bfloat16 and g.dtype == torch.bfloat16
    assert a.stride(1) == 1 and g.stride(1) == 1 and g.shape[1] % 2 == 0
    rows_pad, m = a.shape
    n = g.shape[1] // 2
    num_banks = offs.shape[0]
    out_dtype = torch.float32 if out_f32 else torch.bfloat16
    out0 = torch.empty(num_banks, m, n, dtype=out_dtype, device=a.device)
    out1 = torch.empty(num_banks, m, n, dtype=out_dtype, device=a.device)
    _lib.call(
        "nestor_hip_grouped_gemm_tn_pair", _ptr(a), a.stride(0), _ptr(g), g.stride(0), _ptr(out0),
        _ptr(out1), n, m * n, rows_pad, m, n, num_banks, _ptr(offs.contiguous()), _ptr(seg_start),
        _ptr(seg_count), _code(out_dtype), _stream(a),
    )
    return [out0, out1]


@grouped_gemm_tn_pair.register_fake
def _(a, g, offs, seg_start, seg_count, out_f32=False):
    dtype = torch.float32 if out_f32 else torch.bfloat16
    shape = (offs.shape[0], a.shape[1], g.shape[1] // 2)
    return [a.new_empty(shape, dtype=dtype), a.new_empty(shape, dtype=dtype)]


@torch.library.custom_op(f"{_NS}::upgate_swiglu_fwd", mutates_args=(), device_types="cuda")
def upgate_swiglu_fwd(
    x_pad: Tensor, w_up: Tensor, w_gate: Tensor, tile_table: Tensor
) -> list[Tensor]:
    """[up_gate ``[rows_pad, 2H]``, hidden ``[rows_pad, H]``]."""

    x_pad = _bf16(x_pad, "x_pad")
    w_up = _bf16(w_up, "w_up")
    w_gate = _bf16(w_gate, "w_gate")
    rows_pad, k = x_pad.shape
    num_banks, kb, h = w_up.shape
    assert kb == k and w_gate.shape == w_up.shape
    up_gate = torch.empty(rows_pad, 2 * h, dtype=torch.bfloat16, device=x_pad.device)
    hidden = torch.empty(rows_pad, h, dtype=torch.bfloat16, device=x_pad.device)
    _lib.call(
        "nestor_hip_grouped_gemm_upgate_swiglu", _ptr(x_pad), _ptr(w_up), _ptr(w_gate),
        _ptr(up_gate), _ptr(hidden), rows_pad, k, h, num_banks, _ptr(tile_table),
        _table_max_tiles(tile_table, rows_pad, num_banks), _stream(x_pad),
    )
    return [up_gate, hidden]


@upgate_swiglu_fwd.register_fake
def _(x_pad, w_up, w_gate, tile_table):
    h = w_up.shape[2]
    return [x_pad.new_empty(x_pad.shape[0], 2 * h), x_pad.new_empty(x_pad.shape[0], h)]


@torch.library.custom_op(f"{_NS}::grouped_gemm_nt_upgate", mutates_args=(), device_types="cuda")
def grouped_gemm_nt_upgate(
    g_up_gate: Tensor, w_up: Tensor, w_gate: Tensor, tile_table: Tensor
) -> Tensor:
    g_up_gate = _bf16(g_up_gate, "g_up_gate")
    w_up = _bf16(w_up, "w_up")
    w_gate = _bf16(w_gate, "w_gate")
    rows_pad = g_up_gate.shape[0]
    num_banks, k, h = w_up.shape
    out = torch.empty(rows_pad, k, dtype=torch.bfloat16, device=g_up_gate.device)
    _lib.call(
        "nestor_hip_grouped_gemm_nt_upgate", _ptr(g_up_gate), _ptr(w_up), _ptr(w_gate),
        _ptr(out), rows_pad, k, h, num_banks, _ptr(tile_table), _table_max_tiles(tile_table, rows_pad, num_banks),
        _stream(g_up_gate),
    )
    return out


@grouped_gemm_nt_upgate.register_fake
def _(g_up_gate, w_up, w_gate, tile_table):
    return g_up_gate.new_empty(g_up_gate.shape[0], w_up.shape[1])


def _fp8_bank_dims(b_q: Tensor, tiled: bool) -> tuple[int, int, int]:
    """(banks, K, N) of an e4m3 bank stored ``[E, K, N]`` or tiled ``[E, N/128, K, 128]``."""

    if tiled:
        num_banks, blocks, k, width = b_q.shape
        assert width == 128
        return num_banks, k, blocks * 128
    num_banks, k, n = b_q.shape
    return num_banks, k, n


@torch.library.custom_op(f"{_NS}::grouped_gemm_fp8w_nn", mutates_args=(), device_types="cuda")
def grouped_gemm_fp8w_nn(a: Tensor, b_q: Tensor, scale: Tensor, tile_table: Tensor,
                         tiled: bool = False) -> Tensor:
    a = _bf16(a, "a")
    b_q = b_q.contiguous()
    scale = scale.contiguous()
    assert b_q.dtype == torch.float8_e4m3fn and scale.dtype == torch.float32
    rows_pad, k = a.shape
    num_banks, kb, n = _fp8_bank_dims(b_q, tiled)
    assert kb == k and scale.shape == (num_banks, n)
    out = torch.empty(rows_pad, n, dtype=torch.bfloat16, device=a.device)
    _lib.call(
        "nestor_hip_grouped_gemm_fp8w_nn", _ptr(a), _ptr(b_q), _ptr(scale), _ptr(out), rows_pad,
        k, n, num_banks, _ptr(tile_table), _table_max_tiles(tile_table, rows_pad, num_banks),
        int(tiled), _stream(a),
    )
    return out


@grouped_gemm_fp8w_nn.register_fake
def _(a, b_q, scale, tile_table, tiled=False):
    return a.new_empty(a.shape[0], scale.shape[1])


@torch.library.custom_op(f"{_NS}::grouped_gemm_fp8w_upgate_swiglu", mutates_args=(),
                         device_types="cuda")
def grouped_gemm_fp8w_upgate_swiglu(
    a: Tensor, up_q: Tensor, gate_q: Tensor, scale_up: Tensor, scale_gate: Tensor,
    tile_table: Tensor, tiled: bool = False,
) -> Tensor:
    """``silu(gate) * up`` over e4m3 ``up_q`` / ``gate_q`` (``[E, K, H]``, or tiled
    ``[E, H/128, K, 128]``) in one weight-streaming launch (``K % 64 == 0``,
    ``H % 128 == 0``)."""

    a = _bf16(a, "a")
    up_q, gate_q = up_q.contiguous(), gate_q.contiguous()
    assert up_q.dtype == torch.float8_e4m3fn and gate_q.dtype == torch.float8_e4m3fn
    rows_pad, k = a.shape
    num_banks, kb, h = _fp8_bank_dims(up_q, tiled)
    assert kb == k and gate_q.shape == up_q.shape
    out = torch.empty(rows_pad, h, dtype=torch.bfloat16, device=a.device)
    _lib.call(
        "nestor_hip_grouped_gemm_fp8w_upgate_swiglu", _ptr(a), _ptr(up_q), _ptr(gate_q),
        _ptr(scale_up.contiguous()), _ptr(scale_gate.contiguous()), _ptr(out), rows_pad, k, h,
        num_banks, _ptr(tile_table), _table_max_tiles(tile_table, rows_pad, num_banks),
        int(tiled), _stream(a),
    )
    return out


@grouped_gemm_fp8w_upgate_swiglu.register_fake
def _(a, up_q, gate_q, scale_up, scale_gate, tile_table, tiled=False):
    return a.new_empty(a.shape[0], scale_up.shape[1])


# Differentiable grouped matmul: out = a @ b[bank] per segment.
@torch.library.custom_op(f"{_NS}::grouped_mm", mutates_args=(), device_types="cuda")
def grouped_mm_op(
    a: Tensor, b: Tensor, tile_table: Tensor, offs: Tensor, seg_start: Tensor | None,
    seg_count: Tensor | None,
) -> Tensor:
    return grouped_gemm_nn(a, b, tile_table)


@grouped_mm_op.register_fake
def _(a, b, tile_table, offs, seg_start, seg_count):
    return a.new_empty(a.shape[0], b.shape[2])


def _grouped_mm_setup(ctx, inputs, output):
    a, b, tile_table, offs, seg_start, seg_count = inputs
    ctx.save_for_backward(a, b, tile_table, offs, seg_start, seg_count)


def _grouped_mm_backward(ctx, grad):
    a, b, tile_table, offs, seg_start, seg_count = ctx.saved_tensors
    grad = grad.contiguous()
    ga = gb = None
    if ctx.needs_input_grad[0]:
        # b [E, K, N] read as [E, N', K'] with N' = K, K' = N: a @ b^T form.
        ga = grouped_gemm_nt(grad, b, tile_table)
    if ctx.needs_input_grad[1]:
        gb = grouped_gemm_tn(a, grad, offs, seg_start, seg_count)
    return ga, gb, None, None, None, None


grouped_mm_op.register_autograd(_grouped_mm_backward, setup_context=_grouped_mm_setup)


# The same product for a bank with fp32 owners that keeps a persistent bf16 copy for the
# GEMMs: ``b`` is the copy, ``owner`` the fp32 tensor it was made from.  The forward does
# not read ``owner``; the backward hands IT the weight gradient, in fp32 straight from the
# accumulators, and ``b`` gets none -- instead of a bf16 gradient for ``b`` that autograd
# then widens in another pass over the whole bank.
@torch.library.custom_op(f"{_NS}::grouped_mm_owned", mutates_args=(), device_types="cuda")
def grouped_mm_owned_op(
    a: Tensor, b: Tensor, owner: Tensor, tile_table: Tensor, offs: Tensor, seg_start: Tensor,
    seg_count: Tensor,
) -> Tensor:
    return grouped_gemm_nn(a, b, tile_table)


@grouped_mm_owned_op.register_fake
def _(a, b, owner, tile_table, offs, seg_start, seg_count):
    return a.new_empty(a.shape[0], b.shape[2])


def _grouped_mm_owned_setup(ctx, inputs, output):
    a, b, _owner, tile_table, offs, seg_start, seg_count = inputs
    ctx.save_for_backward(a, b, tile_table, offs, seg_start, seg_count)


def _grouped_mm_owned_backward(ctx, grad):
    a, b, tile_table, offs, seg_start, seg_count = ctx.saved_tensors
    grad = grad.contiguous()
    ga = gowner = None
    if ctx.needs_input_grad[0]:
        ga = grouped_gemm_nt(grad, b, tile_table)
    if ctx.needs_input_grad[2]:
        gowner = grouped_gemm_tn(a, grad, offs, seg_start, seg_count, True)
    return ga, None, gowner, None, None, None, None


grouped_mm_owned_op.register_autograd(_grouped_mm_owned_backward,
                                      setup_context=_grouped_mm_owned_setup)


# Differentiable fused up|gate projection + SwiGLU.
@torch.library.custom_op(f"{_NS}::upgate_swiglu", mutates_args=(), device_types="cuda")
def upgate_swiglu_op(
    x_pad: Tensor, w_up: Tensor, w_gate: Tensor, tile_table: Tensor, offs: Tensor,
    seg_start: Tensor | None, seg_count: Tensor | None,
) -> list[Tensor]:
    return upgate_swiglu_fwd(x_pad, w_up, w_gate, tile_table)


@upgate_swiglu_op.register_fake
def _(x_pad, w_up, w_gate, tile_table, offs, seg_start, seg_count):
    h = w_up.shape[2]
    return [x_pad.new_empty(x_pad.shape[0], 2 * h), x_pad.new_empty(x_pad.shape[0], h)]


def _upgate_setup(ctx, inputs, output):
    x_pad, w_up, w_gate, tile_table, offs, seg_start, seg_count = inputs
    up_gate, _hidden = output
    ctx.save_for_backward(x_pad, w_up, w_gate, tile_table, offs, seg_start, seg_count, up_gate)
    ctx.set_materialize_grads(False)


def _upgate_grad_rows(grads, up_gate, h):
    """Gradient of the ``[rows, 2H]`` up|gate rows from the gradients of both outputs."""

    grad_up_gate, grad_hidden = grads
    g = None
    if grad_hidden is not None:
        g = swiglu_bwd(grad_hidden.contiguous(), up_gate, h)
    if grad_up_gate is not None:
        g = grad_up_gate.contiguous() if g is None else g + grad_up_gate
    return g


def _upgate_backward(ctx, grads):
    x_pad, w_up, w_gate, tile_table, offs, seg_start, seg_count, up_gate = ctx.saved_tensors
    h = w_up.shape[2]
    g = _upgate_grad_rows(grads, up_gate, h)
    if g is None:
        return None, None, None, None, None, None, None
    gx = gup = ggate = None
    if ctx.needs_input_grad[0]:
        gx = grouped_gemm_nt_upgate(g, w_up, w_gate, tile_table)
    if ctx.needs_input_grad[1] and ctx.needs_input_grad[2]:
        gup, ggate = grouped_gemm_tn_pair(x_pad, g, offs, seg_start, seg_count)
    elif ctx.needs_input_grad[1]:
        gup = grouped_gemm_tn(x_pad, g[:, :h], offs, seg_start, seg_count)
    elif ctx.needs_input_grad[2]:
        ggate = grouped_gemm_tn(x_pad, g[:, h:], offs, seg_start, seg_count)
    return gx, gup, ggate, None, None, None, None


upgate_swiglu_op.register_autograd(_upgate_backward, setup_context=_upgate_setup)


# ... with fp32 owners behind persistent bf16 copies (see grouped_mm_owned).
@torch.library.custom_op(f"{_NS}::upgate_swiglu_owned", mutates_args=(), device_types="cuda")
def upgate_swiglu_owned_op(
    x_pad: Tensor, w_up: Tensor, w_gate: Tensor, owner_up: Tensor, owner_gate: Tensor,
    tile_table: Tensor, offs: Tensor, seg_start: Tensor, seg_count: Tensor,
) -> list[Tensor]:
    return upgate_swiglu_fwd(x_pad, w_up, w_gate, tile_table)


@upgate_swiglu_owned_op.register_fake
def _(x_pad, w_up, w_gate, owner_up, owner_gate, tile_table, offs, seg_start, seg_count):
    h = w_up.shape[2]
    return [x_pad.new_empty(x_pad.shape[0], 2 * h), x_pad.new_empty(x_pad.shape[0], h)]


def _upgate_owned_setup(ctx, inputs, output):
    x_pad, w_up, w_gate, _ou, _og, tile_table, offs, seg_start, seg_count = inputs
    up_gate, _hidden = output
    ctx.save_for_backward(x_pad, w_up, w_gate, tile_table, offs, seg_start, seg_count, up_gate)
    ctx.set_materialize_grads(False)


def _upgate_owned_backward(ctx, grads):
    x_pad, w_up, w_gate, tile_table, offs, seg_start, seg_count, up_gate = ctx.saved_tensors
    h = w_up.shape[2]
    g = _upgate_grad_rows(grads, up_gate, h)
    if g is None:
        return None, None, None, None, None, None, None, None, None
    gx = gown_up = gown_gate = None
    if ctx.needs_input_grad[0]:
        gx = grouped_gemm_nt_upgate(g, w_up, w_gate, tile_table)
    if ctx.needs_input_grad[3] and ctx.needs_input_grad[4]:
        gown_up, gown_gate = grouped_gemm_tn_pair(x_pad, g, offs, seg_start, seg_count, True)
    elif ctx.needs_input_grad[3]:
        gown_up = grouped_gemm_tn(x_pad, g[:, :h], offs, seg_start, seg_count, True)
    elif ctx.needs_input_grad[4]:
        gown_gate = grouped_gemm_tn(x_pad, g[:, h:], offs, seg_start, seg_count, True)
    return gx, None, None, gown_up, gown_gate, None, None, None, None


upgate_swiglu_owned_op.register_autograd(_upgate_owned_backward, setup_context=_upgate_owned_setup)


# --------------------------------------------------------------------------
# Router epilogue
# --------------------------------------------------------------------------
@torch.library.custom_op(f"{_NS}::router_topk", mutates_args=(), device_types="cuda")
def router_topk(
    scores: Tensor, choice_bias: Tensor, mask: Tensor | None, top_k: int, gate_mode: int
) -> list[Tensor]:
    """scores ``[n, C]``, choice_bias ``[rows_b, C]`` fp32 (row % rows_b), mask ``[n]``
    bool/uint8 -> [softmax_probs fp32, topk_indices int64, gates (scores dtype)]."""

    scores = scores.contiguous()
    n, c = scores.shape
    bias = choice_bias.contiguous().float().reshape(-1, c)
    m = None if mask is None else mask.contiguous().view(torch.uint8)
    probs = torch.empty(n, c, dtype=torch.float32, device=scores.device)
    topk = torch.empty(n, top_k, dtype=torch.long, device=scores.device)
    gates = torch.empty_like(scores)
    _lib.call(
        "nestor_hip_router_topk", _ptr(scores), _code(scores.dtype), _ptr(bias), bias.shape[0],
        _ptr(m), _ptr(probs), _ptr(topk), _ptr(gates), n, c, top_k, gate_mode, _stream(scores),
    )
    return [probs, topk, gates]


@router_topk.register_fake
def _(scores, choice_bias, mask, top_k, gate_mode):
    n, c = scores.shape
    return [scores.new_empty(n, c, dtype=torch.float32),
            scores.new_empty(n, top_k, dtype=torch.long), torch.empty_like(scores)]


@torch.library.custom_op(f"{_NS}::router_gates_bwd", mutates_args=(), device_types="cuda")
def router_gates_bwd(
    scores: Tensor, topk: Tensor, mask: Tensor | None, grad_gates: Tensor | None,
    grad_probs: Tensor | None, gate_mode: int,
) -> Tensor:
    scores = scores.contiguous()
    n, c = scores.shape
    m = None if mask is None else mask.contiguous().view(torch.uint8)
    gg = None if grad_gates is None else grad_gates.contiguous().to(scores.dtype)
    gp = None if grad_probs is None else grad_probs.contiguous().float()
    out = torch.empty_like(scores)
    _lib.call(
        "nestor_hip_router_gates_bwd", _ptr(scores), _code(scores.dtype), _ptr(topk.contiguous()),
        _ptr(m), _ptr(gg), _ptr(gp), _ptr(out), n, c, topk.shape[1], gate_mode, _stream(scores),
    )
    return out


@router_gates_bwd.register_fake
def _(scores, topk, mask, grad_gates, grad_probs, gate_mode):
    return torch.empty_like(scores)


def _router_setup(ctx, inputs, output):
    scores, _bias, mask, _top_k, gate_mode = inputs
    _probs, topk, _gates = output
    ctx.save_for_backward(scores, topk, mask)
    ctx.gate_mode = gate_mode
    ctx.set_materialize_grads(False)


def _router_backward(ctx, grads):
    grad_probs, _grad_topk, grad_gates = grads
    scores, topk, mask = ctx.saved_tensors
    if grad_probs is None and grad_gates is None:
        return None, None, None, None, None
    return (router_gates_bwd(scores, topk, mask, grad_gates, grad_probs, ctx.gate_mode),
            None, None, None, None)


router_topk.register_autograd(_router_backward, setup_context=_router_setup)


@torch.library.custom_op(f"{_NS}::router_choice_counts", mutates_args=(), device_types="cuda")
def router_choice_counts(topk: Tensor, mask: Tensor | None, num_choices: int) -> Tensor:
    """``[C]`` int32: how many (valid row, slot) pairs chose each entry."""

    topk = topk.contiguous()
    k = topk.shape[-1]
    n = topk.numel() // k
    m = None if mask is None else mask.contiguous().view(torch.uint8)
    counts = torch.zeros(num_choices, dtype=torch.int32, device=topk.device)
    _lib.call("nestor_hip_router_choice_counts", _ptr(topk), _ptr(m), _ptr(counts), n, k,
              num_choices, _stream(topk))
    return counts


@router_choice_counts.register_fake
def _(topk, mask, num_choices):
    return topk.new_empty(num_choices, dtype=torch.int32)


@torch.library.custom_op(f"{_NS}::private_slots", mutates_args=(), device_types="cuda")
def private_slots_op(
    column_gates: Tensor, gates: Tensor, choices: Tensor, selected: Tensor | None, k_a: int,
) -> list[Tensor]:
    """``column_gates [T, G]``, ``gates [T, G, Q]``, ``choices [T, G, k_q]`` ->
    ``[selected [T, k_a], ids [T, k_a*k_q], weights [T, k_a*k_q]]``; differentiable
    in both gate tensors."""

    cg = column_gates.contiguous()
    pg = gates.contiguous()
    if pg.dtype != cg.dtype:
        raise TypeError("column gates and private gates must share one dtype")
    ch = choices.contiguous()
    tokens, columns, experts = pg.shape
    k_q = ch.shape[2]
    sel_in = None if selected is None else selected.contiguous()
    sel = torch.empty(tokens, k_a, dtype=torch.long, device=cg.device)
    ids = torch.empty(tokens, k_a * k_q, dtype=torch.long, device=cg.device)
    weights = torch.empty(tokens, k_a * k_q, dtype=cg.dtype, device=cg.device)
    _lib.call("nestor_hip_private_slots_fwd", _ptr(cg), _ptr(pg), _code(cg.dtype), _ptr(ch),
              _ptr(sel_in), _ptr(sel), _ptr(ids), _ptr(weights), tokens, columns, experts, k_a,
              k_q, _stream(cg))
    return [sel, ids, weights]


@private_slots_op.register_fake
def _(column_gates, gates, choices, selected, k_a):
    tokens, k_q = gates.shape[0], choices.shape[2]
    return [gates.new_empty(tokens, k_a, dtype=torch.long),
            gates.new_empty(tokens, k_a * k_q, dtype=torch.long),
            gates.new_empty(tokens, k_a * k_q)]


@torch.library.custom_op(f"{_NS}::private_slots_bwd", mutates_args=(), device_types="cuda")
def private_slots_bwd(
    grad_weights: Tensor, column_gates: Tensor, gates: Tensor, choices: Tensor, selected: Tensor,
) -> list[Tensor]:
    cg = column_gates.contiguous()
    pg = gates.contiguous()
    ch = choices.contiguous()
    tokens, columns, experts = pg.shape
    g_cg = torch.empty_like(cg)
    g_pg = torch.empty_like(pg)
    _lib.call("nestor_hip_private_slots_bwd", _ptr(grad_weights.contiguous().to(cg.dtype)),
              _ptr(cg), _ptr(pg), _code(cg.dtype), _ptr(ch), _ptr(selected.contiguous()),
              _ptr(g_cg), _ptr(g_pg), tokens, columns, experts, selected.shape[1], ch.shape[2],
              _stream(cg))
    return [g_cg, g_pg]


@private_slots_bwd.register_fake
def _(grad_weights, column_gates, gates, choices, selected):
    return [torch.empty_like(column_gates), torch.empty_like(gates)]


def _private_slots_setup(ctx, inputs, output):
    column_gates, gates, choices, _selected, _k_a = inputs
    ctx.save_for_backward(column_gates, gates, choices, output[0])
    ctx.set_materialize_grads(False)


def _private_slots_backward(ctx, grads):
    grad_weights = grads[2]
    if grad_weights is None:
        return None, None, None, None, None
    column_gates, gates, choices, selected = ctx.saved_tensors
    g_cg, g_pg = private_slots_bwd(grad_weights, column_gates, gates, choices, selected)
    return g_cg, g_pg, None, None, None


private_slots_op.register_autograd(_private_slots_backward, setup_context=_private_slots_setup)


# --------------------------------------------------------------------------
# Biased banks
# --------------------------------------------------------------------------
@torch.library.custom_op(f"{_NS}::bias_rows_fwd", mutates_args=(), device_types="cuda")
def bias_rows_fwd(rows: Tensor, bias: Tensor, index: Tensor, valid: Tensor | None) -> Tensor:
    rows = _bf16(rows, "rows")
    bias = _bf16(bias, "bias")
    out = torch.empty_like(rows)
    v = None if valid is None else valid.contiguous()
    _lib.call("nestor_hip_bias_rows_fwd", _ptr(rows), _ptr(bias), _ptr(index.contiguous()),
              _ptr(v), 0 if v is None else _code(v.dtype), _ptr(out), rows.shape[0],
              rows.shape[1], _stream(rows))
    return out


@bias_rows_fwd.register_fake
def _(rows, bias, index, valid):
    return torch.empty_like(rows)


@torch.library.custom_op(f"{_NS}::segment_colsum", mutates_args=(), device_types="cuda")
def segment_colsum(grad: Tensor, row_index: Tensor | None, seg_start: Tensor,
                   seg_count: Tensor) -> Tensor:
    """``out[e] = sum of grad rows of bank e`` (bf16 ``[E, dim]``), deterministic."""

    grad = _bf16(grad, "grad")
    num_banks = seg_start.shape[0]
    dim = grad.shape[1]
    rows = grad.shape[0] if row_index is None else row_index.shape[0]
    # enough workgroups to fill the device (a few thousand), each with at least
    # ~128 rows to sum
    col_blocks = -(-dim // 512)
    want = -(-4096 // (num_banks * col_blocks))
    splits = max(1, min(64, want, rows // (128 * num_banks)))
    partial = None
    if splits > 1:
        partial = torch.empty(splits, num_banks, dim, dtype=torch.float32, device=grad.device)
    out = torch.empty(num_banks, dim, dtype=torch.bfloat16, device=grad.device)
    ri = None if row_index is None else row_index.contiguous()
    _lib.call("nestor_hip_segment_colsum", _ptr(grad), _ptr(ri), _ptr(seg_start.contiguous()),
              _ptr(seg_count.contiguous()), _ptr(partial), splits, _ptr(out), num_banks, dim,
              _stream(grad))
    return out


@segment_colsum.register_fake
def _(grad, row_index, seg_start, seg_count):
    return grad.new_empty(seg_start.shape[0], grad.shape[1])


@torch.library.custom_op(f"{_NS}::bias_rows", mutates_args=(), device_types="cuda")
def bias_rows_op(rows: Tensor, bias: Tensor, index: Tensor, valid: Tensor | None,
                 row_index: Tensor | None, seg_start: Tensor, seg_count: Tensor) -> Tensor:
    """``rows + bias[index]`` on the rows that hold an assignment.  ``row_index`` /
    ``seg_start`` / ``seg_count`` describe each bank's rows for the bias gradient
    (see :func:`segment_colsum`)."""

    return bias_rows_fwd(rows, bias, index, valid)


@bias_rows_op.register_fake
def _(rows, bias, index, valid, row_index, seg_start, seg_count):
    return torch.empty_like(rows)


def _bias_rows_setup(ctx, inputs, output):
    _rows, _bias, _index, _valid, row_index, seg_start, seg_count = inputs
    ctx.save_for_backward(row_index, seg_start, seg_count)


def _bias_rows_backward(ctx, grad):
    row_index, seg_start, seg_count = ctx.saved_tensors
    g_bias = None
    if ctx.needs_input_grad[1]:
        g_bias = segment_colsum(grad.contiguous(), row_index, seg_start, seg_count)
    return grad, g_bias, None, None, None, None, None


bias_rows_op.register_autograd(_bias_rows_backward, setup_context=_bias_rows_setup)


# --------------------------------------------------------------------------
# Path mix of the pool's summed layout
# --------------------------------------------------------------------------
def _mix_operands(alpha: Tensor, *tensors: Tensor) -> tuple[Tensor, ...]:
    dtype = tensors[0].dtype
    if any(t.dtype != dtype for t in tensors) or alpha.dtype != dtype:
        raise TypeError("path mix operands must share one dtype")
    if alpha.shape[-1] != 2 or alpha.numel() * tensors[0].shape[-1] != 2 * tensors[0].numel():
        raise ValueError("alpha must be [..., 2] over the leading axes of the updates")
    return tuple(t.contiguous() for t in (alpha, *tensors))


@torch.library.custom_op(f"{_NS}::path_mix_fwd", mutates_args=(), device_types="cuda")
def path_mix_fwd(public_update: Tensor, private_update: Tensor, alpha: Tensor) -> Tensor:
    alpha, pub, priv = _mix_operands(alpha, public_update, private_update)
    dim = pub.shape[-1]
    out = torch.empty_like(pub)
    _lib.call("nestor_hip_path_mix_fwd", _ptr(pub), _ptr(priv), _ptr(alpha), _ptr(out),
              _code(pub.dtype), pub.numel() // dim, dim, _stream(pub))
    return out


@path_mix_fwd.register_fake
def _(public_update, private_update, alpha):
    return torch.empty_like(public_update)


@torch.library.custom_op(f"{_NS}::path_mix_bwd", mutates_args=(), device_types="cuda")
def path_mix_bwd(grad_out: Tensor, public_update: Tensor, private_update: Tensor,
                 alpha: Tensor) -> list[Tensor]:
    alpha, g, pub, priv = _mix_operands(alpha, grad_out, public_update, private_update)
    dim = pub.shape[-1]
    g_pub = torch.empty_like(pub)
    g_priv = torch.empty_like(pub)
    g_alpha = torch.empty_like(alpha)
    _lib.call("nestor_hip_path_mix_bwd", _ptr(g), _ptr(pub), _ptr(priv), _ptr(alpha),
              _ptr(g_pub), _ptr(g_priv), _ptr(g_alpha), _code(pub.dtype), pub.numel() // dim,
              dim, _stream(pub))
    return [g_pub, g_priv, g_alpha]


@path_mix_bwd.register_fake
def _(grad_out, public_update, private_update, alpha):
    return [torch.empty_like(public_update), torch.empty_like(public_update),
            torch.empty_like(alpha)]


@torch.library.custom_op(f"{_NS}::path_mix", mutates_args=(), device_types="cuda")
def path_mix_op(public_update: Tensor, private_update: Tensor, alpha: Tensor) -> Tensor:
    """``alpha[..., 0:1] * public_update + alpha[..., 1:2] * private_update`` with the
    eager expression's roundings, one launch (and one for all three gradients)."""

    return path_mix_fwd(public_update, private_update, alpha)


@path_mix_op.register_fake
def _(public_update, private_update, alpha):
    return torch.empty_like(public_update)


def _path_mix_setup(ctx, inputs, output):
    ctx.save_for_backward(*inputs)


def _path_mix_backward(ctx, grad_out):
    pub, priv, alpha = ctx.saved_tensors
    g_pub, g_priv, g_alpha = path_mix_bwd(grad_out.contiguous(), pub, priv, alpha)
    return g_pub, g_priv, g_alpha


path_mix_op.register_autograd(_path_mix_backward, setup_context=_path_mix_setup)


@torch.library.custom_op(f"{_NS}::path_scale_fwd", mutates_args=(), device_types="cuda")
def path_scale_fwd(inp: Tensor, alpha: Tensor, which: int, dest: Tensor | None,
                   num_out: int) -> Tensor:
    inp = inp.contiguous()
    alpha = alpha.contiguous()
    if alpha.dtype != inp.dtype:
        raise TypeError("path scale operands must share one dtype")
    slots, dim = inp.shape[-2], inp.shape[-1]
    tokens = inp.numel() // (slots * dim)
    d = None if dest is None else dest.contiguous()
    out = torch.empty(*inp.shape[:-2], num_out, dim, dtype=inp.dtype, device=inp.device)
    _lib.call("nestor_hip_path_scale_fwd", _ptr(inp), _ptr(alpha), which, _ptr(d), _ptr(out),
              _code(inp.dtype), tokens, slots, num_out, dim, _stream(inp))
    return out


@path_scale_fwd.register_fake
def _(inp, alpha, which, dest, num_out):
    return inp.new_empty(*inp.shape[:-2], num_out, inp.shape[-1])


@torch.library.custom_op(f"{_NS}::path_scale_bwd", mutates_args=(), device_types="cuda")
def path_scale_bwd(grad_out: Tensor, inp: Tensor, alpha: Tensor, which: int,
                   dest: Tensor | None) -> list[Tensor]:
    grad_out = grad_out.contiguous()
    inp = inp.contiguous()
    alpha = alpha.contiguous()
    slots, dim = inp.shape[-2], inp.shape[-1]
    tokens = inp.numel() // (slots * dim)
    d = None if dest is None else dest.contiguous()
    g_in = torch.empty_like(inp)
    g_alpha = torch.empty(alpha.shape[:-1], dtype=torch.float32, device=inp.device)
    _lib.call("nestor_hip_path_scale_bwd", _ptr(grad_out), _ptr(inp), _ptr(alpha), which, _ptr(d),
              _ptr(g_in), _ptr(g_alpha), _code(inp.dtype), tokens, slots, grad_out.shape[-2], dim,
              _stream(inp))
    return [g_in, g_alpha]


@path_scale_bwd.register_fake
def _(grad_out, inp, alpha, which, dest):
    return [torch.empty_like(inp), alpha.new_empty(alpha.shape[:-1], dtype=torch.float32)]


@torch.library.custom_op(f"{_NS}::path_scale", mutates_args=(), device_types="cuda")
def path_scale_op(inp: Tensor, alpha: Tensor, which: int, dest: Tensor | None,
                  num_out: int) -> Tensor:
    """``alpha[..., which] * X`` for ``inp [..., slots, d]``: ``X = inp`` or, with ``dest
    [..., slots]``, ``zeros(..., num_out, d).scatter_add(-2, dest, inp)``."""

    return path_scale_fwd(inp, alpha, which, dest, num_out)


@path_scale_op.register_fake
def _(inp, alpha, which, dest, num_out):
    return inp.new_empty(*inp.shape[:-2], num_out, inp.shape[-1])


def _path_scale_setup(ctx, inputs, output):
    inp, alpha, which, dest, _num_out = inputs
    ctx.save_for_backward(inp, alpha, dest)
    ctx.which = which


def _path_scale_backward(ctx, grad_out):
    inp, alpha, dest = ctx.saved_tensors
    g_in, g_col = path_scale_bwd(grad_out, inp, alpha, ctx.which, dest)
    g_alpha = torch.zeros_like(alpha)
    g_alpha[..., ctx.which] = g_col.to(alpha.dtype)
    return g_in, g_alpha, None, None, None


path_scale_op.register_autograd(_path_scale_backward, setup_context=_path_scale_setup)


# --------------------------------------------------------------------------
# Packed column attention epilogue
# --------------------------------------------------------------------------
@torch.library.custom_op(f"{_NS}::gate_slots_fwd", mutates_args=(), device_types="cuda")
def gate_slots_fwd(out_c: Tensor, bias: Tensor | None, gid: Tensor | None, gates: Tensor,
                   slot_rows: Tensor, out_f32: bool) -> Tensor:
    out_c = _bf16(out_c, "out_c")
    dim = out_c.shape[1]
    n_out = slot_rows.shape[0]
    out_dtype = torch.float32 if out_f32 else torch.bfloat16
    out = torch.empty(n_out, dim, dtype=out_dtype, device=out_c.device)
    b = None if bias is None else bias.contiguous().float()
    gi = None if gid is None else gid.contiguous()
    _lib.call("nestor_hip_gate_slots_fwd", _ptr(out_c), _ptr(b), _ptr(gi),
              _ptr(gates.contiguous().float()), _ptr(slot_rows.contiguous()), _ptr(out),
              _code(out_dtype), n_out, dim, _stream(out_c))
    return out


@gate_slots_fwd.register_fake
def _(out_c, bias, gid, gates, slot_rows, out_f32):
    return out_c.new_empty(slot_rows.shape[0], out_c.shape[1],
                           dtype=torch.float32 if out_f32 else torch.bfloat16)


@torch.library.custom_op(f"{_NS}::gate_slots_bwd", mutates_args=(), device_types="cuda")
def gate_slots_bwd(grad_slots: Tensor, out_c: Tensor, bias: Tensor | None, gid: Tensor | None,
                   gates: Tensor, slot_packed: Tensor, need_gates: bool) -> list[Tensor]:
    grad_slots = grad_slots.contiguous()
    out_c = _bf16(out_c, "out_c")
    rows, dim = out_c.shape
    g_out_c = torch.empty_like(out_c)
    g_gates = torch.empty(rows if need_gates else 0, dtype=torch.float32, device=out_c.device)
    b = None if bias is None else bias.contiguous().float()
    gi = None if gid is None else gid.contiguous()
    _lib.call("nestor_hip_gate_slots_bwd", _ptr(grad_slots), _code(grad_slots.dtype), _ptr(out_c),
              _ptr(b), _ptr(gi), _ptr(gates.contiguous().float()), _ptr(slot_packed.contiguous()),
              _ptr(g_out_c), _ptr(g_gates) if need_gates else None, rows, dim, _stream(out_c))
    return [g_out_c, g_gates]


@gate_slots_bwd.register_fake
def _(grad_slots, out_c, bias, gid, gates, slot_packed, need_gates):
    return [torch.empty_like(out_c),
            out_c.new_empty(out_c.shape[0] if need_gates else 0, dtype=torch.float32)]


@torch.library.custom_op(f"{_NS}::gate_combine_slots", mutates_args=(), device_types="cuda")
def gate_combine_slots_op(out_c: Tensor, bias: Tensor | None, gid: Tensor | None, gates: Tensor,
                          slot_rows: Tensor, slot_packed: Tensor, out_f32: bool) -> Tensor:
    return gate_slots_fwd(out_c, bias, gid, gates, slot_rows, out_f32)


@gate_combine_slots_op.register_fake
def _(out_c, bias, gid, gates, slot_rows, slot_packed, out_f32):
    return out_c.new_empty(slot_rows.shape[0], out_c.shape[1],
                           dtype=torch.float32 if out_f32 else torch.bfloat16)


def _gate_slots_setup(ctx, inputs, output):
    out_c, bias, gid, gates, _slot_rows, slot_packed, _out_f32 = inputs
    ctx.save_for_backward(out_c, bias, gid, gates, slot_packed)


def _gate_slots_backward(ctx, grad_slots):
    out_c, bias, gid, gates, slot_packed = ctx.saved_tensors
    need_gates = ctx.needs_input_grad[3]
    g_out_c, g_gates = gate_slots_bwd(grad_slots, out_c, bias, gid, gates, slot_packed, need_gates)
    g_bias = None
    if bias is not None and ctx.needs_input_grad[1]:
        # rows of group e are those with gid == e: a stable sort groups them for the
        # segmented column sum (the reference's deterministic mask-GEMM)
        order = torch.argsort(gid, stable=True)
        counts = torch.bincount(gid, minlength=bias.shape[0])
        starts = torch.cumsum(counts, 0) - counts
        g_bias = segment_colsum(g_out_c, order, starts, counts).to(bias.dtype)
    return g_out_c, g_bias, None, (g_gates.to(gates.dtype) if need_gates else None), None, None, None


gate_combine_slots_op.register_autograd(_gate_slots_backward, setup_context=_gate_slots_setup)


# --------------------------------------------------------------------------
# Skinny score heads (router / path gate linear maps)
# --------------------------------------------------------------------------
@torch.library.custom_op(f"{_NS}::score_heads", mutates_args=(), device_types="cuda")
def score_heads_op(x: Tensor, weight: Tensor, bias: Tensor | None) -> Tensor:
    """``x [T, d] @ weight[C, d]^T (+ bias)`` in bf16, ``C`` a multiple of 8.

    The forward is a library GEMM.  The input gradient ``g [T, C] @ weight`` has a
    contraction of only ``C`` (tens to a few hundred) against ``T x d`` outputs: it is
    a write-bound pass over the activations, and runs on the grouped GEMM kernel
    with the whole batch as one bank."""

    x = _bf16(x, "x")
    weight = _bf16(weight, "weight")
    if bias is None:
        return x @ weight.t()
    return torch.addmm(_bf16(bias, "bias"), x, weight.t())


@score_heads_op.register_fake
def _(x, weight, bias):
    return x.new_empty(x.shape[0], weight.shape[0])


def _one_bank_table(like: Tensor, rows: int) -> Tensor:
    """Tile table of a single bank that owns rows ``0 .. rows`` (two tiny launches; built
    per call so that a traced graph holds it as nodes, not as a captured constant)."""

    offs = torch.full((1,), rows, dtype=torch.int32, device=like.device)
    return tile_schedule(offs, rows)


def _skinny_weight_grad(grad: Tensor, x: Tensor) -> Tensor:
    """``grad [T, C]^T @ x [T, d]``: few outputs, a contraction over every row.  As
    one GEMM it has ``C*d`` / tile-size workgroups (a few dozen) for the whole
    device; split over row chunks it is a batched GEMM that fills the device, and
    the chunk results (bf16) are summed in fp32."""

    rows = x.shape[0]
    chunks = 32
    while chunks > 1 and (rows % chunks or rows // chunks < 512):
        chunks //= 2
    if chunks == 1:
        return grad.t() @ x
    parts = torch.bmm(grad.view(chunks, rows // chunks, -1).transpose(1, 2),
                      x.view(chunks, rows // chunks, -1))
    return parts.sum(0)


def _score_heads_setup(ctx, inputs, output):
    x, weight, bias = inputs
    ctx.save_for_backward(x, weight)
    ctx.has_bias = bias is not None


def _score_heads_backward(ctx, grad):
    x, weight = ctx.saved_tensors
    grad = grad.contiguous()
    gx = gw = gb = None
    if ctx.needs_input_grad[0]:
        gx = grouped_gemm_nn(grad, weight.unsqueeze(0), _one_bank_table(grad, x.shape[0]))
    if ctx.needs_input_grad[1]:
        gw = _skinny_weight_grad(grad, x)
    if ctx.has_bias and ctx.needs_input_grad[2]:
        gb = grad.sum(0)
    return gx, gw, gb


score_heads_op.register_autograd(_score_heads_backward, setup_context=_score_heads_setup)


# --------------------------------------------------------------------------
# FLOP formulas for torch.utils.flop_counter.FlopCounterMode
# --------------------------------------------------------------------------
# The reference's MFU calibration counts ``aten._grouped_mm`` as ``2 * rows * K * N``
# over the rows of the row operand as passed, padding included
# (nestor/train/flop_formulas.py:28-91).  The ops below stand in for that GEMM and
# its autograd, so they carry the same formula; without it a calibration pass over
# this path would leave the expert GEMMs uncounted.  A mode only sees the ops that
# are called while it is active at the top level: the forward wrappers
# (``grouped_mm``, ``upgate_swiglu``, ``score_heads``) and whatever their backward
# functions call.  The kernels they run inside are not seen again, so nothing is
# counted twice.
def _rows(shape) -> int:
    n = 1
    for dim in shape[:-1]:
        n *= int(dim)
    return n


def _flops_rows_bank(a_shape, b_shape, *args, out_shape=None, **kwargs) -> int:
    """a ``[rows, K] @`` b ``[E, K, N]`` (or ``[E, N, K]`` transposed: same product)."""

    return 2 * _rows(a_shape) * int(b_shape[-2]) * int(b_shape[-1])


def _flops_upgate(x_shape, w_up_shape, *args, out_shape=None, **kwargs) -> int:
    """Both projections: rows ``[rows, K]`` (or gradients ``[rows, 2H]``) against two
    ``[E, K, H]`` banks."""

    return 2 * _rows(x_shape) * int(w_up_shape[-2]) * 2 * int(w_up_shape[-1])


def _flops_weight_grad(a_shape, g_shape, *args, out_shape=None, **kwargs) -> int:
    """``a [rows, M]^T @ g [rows, N]`` per segment."""

    return 2 * int(a_shape[0]) * int(a_shape[1]) * int(g_shape[1])


def _flops_score_heads(x_shape, w_shape, *args, out_shape=None, **kwargs) -> int:
    return 2 * _rows(x_shape) * int(w_shape[0]) * int(w_shape[1])


_FLOP_FORMULAS_REGISTERED = False


def register_flop_formulas() -> None:
    """Teach ``FlopCounterMode`` the expert GEMM ops.  Idempotent; never raises (a
    torch build with a different registration interface leaves them uncounted, as
    the reference's own registration does)."""

    global _FLOP_FORMULAS_REGISTERED
    if _FLOP_FORMULAS_REGISTERED:
        return
    try:
        from torch.utils.flop_counter import register_flop_formula

        ns = getattr(torch.ops, _NS)
        for names, formula in (
            (("grouped_mm", "grouped_mm_owned", "grouped_gemm_nn", "grouped_gemm_nt",
              "grouped_gemm_fp8w_nn"), _flops_rows_bank),
            (("upgate_swiglu", "upgate_swiglu_owned", "upgate_swiglu_fwd", "grouped_gemm_nt_upgate",
              "grouped_gemm_fp8w_upgate_swiglu"), _flops_upgate),
            (("grouped_gemm_tn", "grouped_gemm_tn_pair"), _flops_weight_grad),
            (("score_heads",), _flops_score_heads),
        ):
            for name in names:
                register_flop_formula(getattr(ns, name))(formula)
        _FLOP_FORMULAS_REGISTERED = True
    except Exception:  # noqa: BLE001 -- FLOP accounting must never break the path
        pass


register_flop_formulas()
