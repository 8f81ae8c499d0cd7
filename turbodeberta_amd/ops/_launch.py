"""Host-side plumbing shared by the two attention operators: dtype codes, the cached device copy
of the relative-position table, argument packing and the launch through the C ABI."""
from __future__ import annotations

import ctypes as C
import math
import threading
from typing import Optional

import torch

from .. import _lib

_DTYPES = {torch.float32: _lib.TDB_F32, torch.bfloat16: _lib.TDB_BF16, torch.float16: _lib.TDB_F16}

_lut_lock = threading.Lock()
_lut_cache: dict = {}


def dtype_code(t: torch.Tensor) -> int:
    try:
        return _DTYPES[t.dtype]
    except KeyError:
        raise ValueError(f"unsupported dtype {t.dtype}; expected float32, bfloat16 or float16") from None


def att_span(position_buckets: int, max_relative_distance: int) -> int:
    """Half-width of the relative-position axis, as the reference derives ATT_SPAN
    (ops/flash_attention.py:274-277)."""
    return position_buckets if position_buckets > 0 else max_relative_distance


def delta_lut(device: torch.device, max_len: int, position_buckets: int, max_relative_distance: int):
    """Device int32 table of delta(r) for |r| < half+1, and its half-width.  Built on the host by
    tdb_delta_table once per (device, size class, bucket configuration) and then reused."""
    size = 512
    while size < max_len:
        size *= 2
    key = (device.type, device.index, size, int(position_buckets), int(max_relative_distance))
    hit = _lut_cache.get(key)
    if hit is not None:
        return hit
    with _lut_lock:
        hit = _lut_cache.get(key)
        if hit is None:
            table = torch.from_numpy(_lib.delta_table(size, int(position_buckets), int(max_relative_distance)))
            hit = (table.to(device), size - 1)
            _lut_cache[key] = hit
    return hit


def require_gpu(*tensors) -> torch.device:
    dev = tensors[0].device
    if dev.type != "cuda":
        raise RuntimeError("turbodeberta_amd operators run HIP kernels only: tensors must live on a GPU "
                           f"(got {dev}); there is no CPU implementation")
    for t in tensors:
        if t is not None and t.device != dev:
            raise ValueError("all tensors must be on the same device")
    return dev


def rows_ok(t: torch.Tensor) -> bool:
    """Last dim contiguous, base and every outer stride 16-byte aligned."""
    es = t.element_size()
    return (t.stride(-1) == 1 and t.data_ptr() % 16 == 0
            and all(s >= 0 and (s * es) % 16 == 0 for s in t.stride()[:-1]))


def as_rows(t: torch.Tensor) -> torch.Tensor:
    return t if rows_ok(t) else t.contiguous()


def fused_table(t: Optional[torch.Tensor], heads: int, span: int, head_dim: int, name: str):
    """Normalise a fused position table to [H, >=2*span, D]; accepts a leading singleton dim
    (the reference's transform() output, model.py:94-110, is [1, H, 2*span, D])."""
    if t is None:
        return None
    if t.dim() == 4:
        if t.shape[0] != 1:
            raise ValueError(f"{name}: leading dim must be 1, got {tuple(t.shape)}")
        t = t[0]
    if t.dim() != 3 or t.shape[0] != heads or t.shape[2] != head_dim or t.shape[1] < 2 * span:
        raise ValueError(f"{name}: expected [H={heads}, >=2*span={2 * span}, D={head_dim}], got {tuple(t.shape)}")
    return as_rows(t)


def fill_pos(pos: _lib.PosArgs, *, dev, max_len, span, position_buckets, max_relative_distance,
             pos_key, pos_query, c2p_strip, p2c_strip, varlen: bool, keep: list) -> None:
    if pos_key is None and pos_query is None and c2p_strip is None and p2c_strip is None:
        return
    if span < 1:
        raise ValueError("position terms need position_buckets > 0 or max_relative_distance > 0")
    lut, half = delta_lut(dev, max_len, position_buckets, max_relative_distance)
    keep.append(lut)
    pos.span = span
    pos.lut_half = half
    pos.delta_lut = lut.data_ptr()
    if pos_key is not None:
        pos.pos_key = pos_key.data_ptr()
        pos.pos_key_stride_h, pos.pos_key_stride_r = pos_key.stride(0), pos_key.stride(1)
    if pos_query is not None:
        pos.pos_query = pos_query.data_ptr()
        pos.pos_query_stride_h, pos.pos_query_stride_r = pos_query.stride(0), pos_query.stride(1)
    for name, strip in (("c2p", c2p_strip), ("p2c", p2c_strip)):
        if strip is None:
            continue
        if strip.shape[-1] != 2 * span:
            raise ValueError(f"{name} strip: last dim {strip.shape[-1]} != 2*span {2 * span}")
        setattr(pos, name + "_strip", strip.data_ptr())
        if varlen:
            setattr(pos, name + "_stride_l", strip.stride(0))
            setattr(pos, name + "_stride_h", strip.stride(1))
        else:
            setattr(pos, name + "_stride_b", strip.stride(0))
            setattr(pos, name + "_stride_h", strip.stride(1))
            setattr(pos, name + "_stride_l", strip.stride(2))


def default_scale(sm_scale, head_dim: int) -> float:
    """``sm_scale=None`` means 1/sqrt(D) (ops/flash_attention.py:329-330)."""
    return 1.0 / math.sqrt(head_dim) if sm_scale is None else float(sm_scale)


class PreparedLaunch:
    """A fully validated call: the packed argument block, the output tensor and every tensor the
    block points into.  ``launch()`` issues the kernel on the current stream of the tensors' device
    and can be repeated (same inputs, same output buffer) at the cost of one C call."""

    __slots__ = ("_fn", "args", "out", "_keep", "_dev")

    def __init__(self, fn, args, out, keep, dev):
        self._fn, self.args, self.out, self._keep, self._dev = fn, args, out, keep, dev

    def launch(self) -> torch.Tensor:
        if torch.cuda.current_device() != self._dev.index:      # HIP launches on the current device
            with torch.cuda.device(self._dev):
                return self.launch()
        rc = self._fn(C.byref(self.args), torch.cuda.current_stream(self._dev).cuda_stream)
        if rc:
            _lib.check(rc)
        return self.out


BACKWARD_MESSAGE = "Backward pass is not implemented for FlashAttentionDisentangled"
