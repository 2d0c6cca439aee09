"""Python glue between torch tensors and the backend descriptors.

Counterparts of the helpers pybuda keeps in ``pybuda/pybuda/tensor.py`` (dtype/format maps
``:563-651``, descriptor building ``:653-745``, tile padding ``:805-954``) and of
``DirectPusherDeviceConnector._convert_tensor_for_tilize``
(``pybuda/pybuda/device_connector.py:177-201``), with the same names, argument meaning and errors.
"""
from functools import reduce
from operator import mul
from typing import List, Optional, Sequence

import torch

from ._C import DataFormat
from ._C.backend_api import PytorchTensorDesc, TilizedTensorDesc

TILE_DIM = 32  # pybuda/pybuda/pybudaglobal.py:22

_B_QUEUE_FORMATS = (DataFormat.Float16_b, DataFormat.Bfp8_b, DataFormat.Bfp4_b, DataFormat.Bfp2_b)
_A_QUEUE_FORMATS = (DataFormat.Float16, DataFormat.Bfp8, DataFormat.Bfp4, DataFormat.Bfp2)

_DTYPE_TO_FORMAT = {
    torch.float16: DataFormat.Float16,
    torch.bfloat16: DataFormat.Float16_b,
    torch.float32: DataFormat.Float32,
    torch.int8: DataFormat.Int8,
    torch.bool: DataFormat.Bfp2_b,
    torch.int32: DataFormat.Int32,
    torch.int64: DataFormat.Int8,  # the reference narrows int64 parameters to Int8 (tensor.py:604-606)
}

_FORMAT_TO_DTYPE = {
    DataFormat.Float32: torch.float32,
    DataFormat.Float16: torch.float16,
    DataFormat.Float16_b: torch.bfloat16,
    DataFormat.Bfp8_b: torch.bfloat16,
    DataFormat.Bfp4_b: torch.bfloat16,
    DataFormat.Bfp2_b: torch.bfloat16,
    DataFormat.Bfp8: torch.float16,
    DataFormat.Bfp4: torch.float16,
    DataFormat.Bfp2: torch.float16,
    DataFormat.Int8: torch.int8,
    DataFormat.RawUInt32: torch.int,
    DataFormat.UInt16: torch.int,
    DataFormat.Int32: torch.int32,
}


def pytorch_dtype_to_buda_dataformat(dtype, fp32_fallback: Optional[DataFormat] = None) -> DataFormat:
    if isinstance(dtype, DataFormat):
        return dtype
    assert isinstance(dtype, torch.dtype)
    if dtype == torch.float32 and fp32_fallback is not None:
        return fp32_fallback
    try:
        return _DTYPE_TO_FORMAT[dtype]
    except KeyError:
        raise RuntimeError("Unsupported torch dtype " + str(dtype))


def buda_dataformat_to_pytorch_dtype(data_format: DataFormat) -> torch.dtype:
    assert isinstance(data_format, DataFormat)
    try:
        return _FORMAT_TO_DTYPE[data_format]
    except KeyError:
        raise RuntimeError("Unsupported DataFormat for conversion to torch dtype: " + str(data_format))


def is_equivalent_data_format(pt_df: torch.dtype, tt_df: DataFormat) -> bool:
    """True only when the torch dtype and the queue format are bit-for-bit the same encoding."""
    exact = {DataFormat.Float32: torch.float32, DataFormat.Float16: torch.float16,
             DataFormat.Float16_b: torch.bfloat16, DataFormat.Int8: torch.int8}
    return exact.get(tt_df) == pt_df


def convert_tensor_for_tilize(tensor: torch.Tensor, queue_format: DataFormat) -> torch.Tensor:
    """Legalise a source dtype for a queue: 8-bit-exponent queues take fp32 or bf16 as they are and
    anything else as bf16; 5-bit-exponent queues need fp16; non-float tensors take the queue's own
    torch dtype (device_connector.py:177-201)."""
    if is_equivalent_data_format(tensor.dtype, queue_format):
        return tensor
    if not tensor.is_floating_point():
        return tensor.type(buda_dataformat_to_pytorch_dtype(queue_format))
    if queue_format in _A_QUEUE_FORMATS:
        return tensor if tensor.dtype == torch.float16 else tensor.type(torch.float16)
    if queue_format in _B_QUEUE_FORMATS:
        return tensor if tensor.dtype in (torch.float32, torch.bfloat16) else tensor.type(torch.bfloat16)
    return tensor


def pytorch_tensor_to_tensor_desc(t, df: DataFormat = None, element_size=None):
    """Describe a torch tensor as a 4-D (w, z, r, c) view with byte strides (tensor.py:653-727)."""
    if isinstance(t, (PytorchTensorDesc, TilizedTensorDesc)):
        return t
    if not t.is_contiguous():
        t = t.contiguous()
    if df is None:
        by_dtype = {torch.float32: DataFormat.Float32, torch.bfloat16: DataFormat.Float16_b,
                    torch.float16: DataFormat.Float16, torch.int32: DataFormat.Int32, torch.int8: DataFormat.Int8}
        if t.dtype == torch.int64:
            t = t.to(torch.int32)
            fmt = DataFormat.RawUInt32
        elif t.dtype in by_dtype:
            fmt = by_dtype[t.dtype]
        else:
            raise RuntimeError("Unsupported torch tensor type for tilization: " + str(t.dtype))
    else:
        fmt = df
        wanted = buda_dataformat_to_pytorch_dtype(fmt)
        if t.dtype != wanted:
            t = t.type(wanted)

    shape = list(t.shape)
    dim = 3 if len(shape) == 2 else len(shape)
    while len(shape) > 4:
        if shape[0] != 1:
            raise RuntimeError("Dropping a dimension that's not 1 to reduce shape to 4D: " + str(t.shape))
        shape.pop(0)
    shape = [1] * (4 - len(shape)) + shape

    strides = list(t.stride())[-4:]
    strides = [strides[0]] * (4 - len(strides)) + strides
    if element_size is None:
        element_size = t.element_size()
    return PytorchTensorDesc(t, element_size, fmt, dim, shape, [s * element_size for s in strides])


def tensor_desc_to_pytorch_tensor(desc) -> torch.Tensor:
    """Zero-copy torch view of a descriptor's memory (tensor.py:730-745)."""
    by_format = {DataFormat.Float32: torch.float32, DataFormat.Float16_b: torch.bfloat16,
                 DataFormat.Float16: torch.float16, DataFormat.RawUInt32: torch.int,
                 # beyond the reference, which reads back RawUInt32 only: the other integer queues, as they were pushed
                 DataFormat.Int32: torch.int32, DataFormat.Int8: torch.int8, DataFormat.UInt16: torch.int16,
                 DataFormat.RawUInt16: torch.int16, DataFormat.RawUInt8: torch.uint8}
    if desc.format not in by_format:
        raise RuntimeError(f"Unsupported tensor type({desc.format}) for untilization")
    return torch.frombuffer(desc, dtype=by_format[desc.format]).reshape(list(desc.shape))


def is_buda_shape(tensor: torch.Tensor, min_dim: int = -1) -> bool:
    rank_ok = len(tensor.shape) >= min_dim if min_dim > 0 else len(tensor.shape) == 4
    if not rank_ok or len(tensor.shape) > 4:
        return False
    return tensor.shape[-1] % TILE_DIM == 0 and tensor.shape[-2] % TILE_DIM == 0


def _snap(n: int, tile: int) -> int:
    return (tile - n % tile) % tile


def pad_pytorch_tensor_to_buda(tensor: torch.Tensor, tile_broadcast_dims: Sequence[int], squeeze: bool = False,
                               microbatch: int = 1, tile_r: int = TILE_DIM, tile_c: int = TILE_DIM) -> torch.Tensor:
    """Bring a tensor to 4-D with rows/columns snapped up to the tile size; padding is zeros, or a
    replica of the single row/column for dims listed in ``tile_broadcast_dims`` (tensor.py:805-877)."""
    min_dim = 2 if squeeze and tensor.shape[0] != microbatch and len(tensor.shape) > 2 else 4
    if is_buda_shape(tensor, min_dim):
        return tensor
    out = tensor
    while len(out.shape) < min_dim:
        out = out.unsqueeze(1 if out.shape[0] == microbatch else 0)
    while len(out.shape) > 5:
        assert out.shape[0] == 1, "Invalid dimension size above dim 5"
        out = out.squeeze(0)
    if out.shape[0] < microbatch:
        out = out.broadcast_to([microbatch, *out.shape[1:]]).contiguous()
    if is_buda_shape(out):
        return out.detach().contiguous()

    rows, cols = out.shape[-2], out.shape[-1]
    bcast_c = -1 in tile_broadcast_dims or 3 in tile_broadcast_dims
    bcast_r = -2 in tile_broadcast_dims or 2 in tile_broadcast_dims
    if bcast_c:
        assert cols == 1, "Trying to broadcast to tile dim a dimension that's not 1"
    if bcast_r:
        assert rows == 1, "Trying to broadcast to tile dim a dimension that's not 1"
    dtype, rank = out.dtype, len(out.shape)
    work = out.type(torch.float32) if dtype != torch.float32 else out
    while len(work.shape) < 3:
        work = work.unsqueeze(0)
    work = torch.nn.functional.pad(work, (0, _snap(cols, tile_c), 0, 0), mode="replicate" if bcast_c else "constant")
    work = torch.nn.functional.pad(work, (0, 0, 0, _snap(rows, tile_r)), mode="replicate" if bcast_r else "constant")
    while len(work.shape) > rank:
        work = work.squeeze(0)
    work = work.type(dtype).detach()
    work.requires_grad = tensor.requires_grad
    return work


def narrow_buda_tensor_to_pytorch(tensor: torch.Tensor, shape: List[int], has_microbatch_dim: bool = False) -> torch.Tensor:
    """Cut the tile padding off again and restore the original shape (tensor.py:879-954, dense case)."""
    out = tensor
    if len(shape) == 0:
        return out.narrow(-1, 0, 1).narrow(-2, 0, 1).squeeze()
    if len(shape) == 1:
        if len(out.shape) == 1:
            out = out.narrow(0, 0, shape[0])
        elif len(out.shape) > 2 and out.shape[0] == shape[0]:
            out = out.narrow(-1, 0, 1).narrow(-2, 0, 1)
        else:
            out = out.narrow(-1, 0, shape[0]).narrow(-2, 0, 1)
    elif reduce(mul, shape) != reduce(mul, out.shape):
        swapped = len(out.shape) == 4 and len(shape) == 4 and out.shape[-3] != shape[-3]
        if swapped:
            out = out.transpose(-3, -2)
        inner = shape[1:] if has_microbatch_dim else shape
        out = out.narrow(-2, 0, 1 if len(inner) == 1 else inner[-2])
        out = out.narrow(-1, 0, inner[-1])
        if swapped:
            out = out.transpose(-3, -2)
    return out.reshape(shape)


def _prestride_shape(tensor: torch.Tensor, stride_height: int, stride_width: int, queue):
    """The Prestride runtime transform (pybuda/pybuda/tensor.py:1413-1420): the tensor goes to ``push_input`` as it is and
    the queue descriptor tells the backend to rearrange it, ``[w, C, H, W] -> [w, 1, stride*stride*C, H/stride * W/stride]``,
    while it tilizes.  Returns ``(tensor, queue)`` like the reference."""
    from ._C.backend_api import StrideDescriptor

    assert stride_height == stride_width, "Backend supports only square strides for prestriding transform"
    stride = stride_height
    stride_desc = StrideDescriptor()
    stride_desc.stride = stride
    stride_desc.xy_offsets = [(x, y) for y in range(stride) for x in range(stride)]
    queue.s_descriptor = stride_desc
    return tensor, queue


def _embedding_index(tensor: torch.Tensor, original_shape: Sequence[int], queue) -> torch.Tensor:
    """The EmbeddingIndex runtime transform (pybuda/pybuda/tensor.py:1382-1408): the index vector(s) of an embedding lookup
    in the layout its RawUInt queue takes.  The vector is zero-padded to whole rows of 32, every position from the original
    length on is then set to all-ones (in that order, as the reference does: positions between the end of a vector that is
    shorter than its original shape and that shape's length stay zero), and the result is dealt in order to the queue's ``q_rt`` tile rows, and each tile row's share, read as rows
    of 32, is laid out column-block by column-block: ``[w, 1, q_rt * 32, cols]``."""
    from ._C import DataFormat as DF

    assert queue.data_format in (DF.RawUInt8, DF.RawUInt16, DF.RawUInt32)
    assert tensor.dim() <= 2, "Must be a 1d tensor"
    assert all(d == 1 for d in list(original_shape)[-3:-1]), "Must be a 1d tensor"
    q_rt = queue.bufq_grid_dim_r * queue.mblock_m * queue.ublock_rt
    w = tensor.shape[0] if tensor.dim() > 1 else 1
    n = tensor.shape[-1]
    ones = ~torch.zeros((), dtype=tensor.dtype)
    flat = torch.zeros((w, n + _snap(n, 32)), dtype=tensor.dtype)
    flat[:, :n] = tensor.reshape(w, n)
    flat[:, int(original_shape[-1]):] = ones
    rows = flat.shape[1] // (q_rt * 32)                      # rows of 32 per tile row of the queue
    assert rows * q_rt * 32 == flat.shape[1], "_embedding_index: the padded vector does not divide over the queue's tile rows"
    blocks = (rows + _snap(rows, 32)) // 32                  # column blocks of 32 rows each
    grouped = torch.zeros((w, q_rt, blocks * 32, 32), dtype=tensor.dtype)
    grouped[:, :, :rows] = flat.reshape(w, q_rt, rows, 32)
    out = grouped.reshape(w, q_rt, blocks, 32, 32).permute(0, 1, 3, 2, 4).reshape(w, 1, q_rt * 32, blocks * 32)
    assert out.shape[1] == queue.t, "_embedding_index: t changed"
    assert out.shape[2] == queue.bufq_grid_dim_r * queue.mblock_m * queue.ublock_rt * 32, "_embedding_index: tensor dims mismatch q dims"
    assert out.shape[3] == queue.bufq_grid_dim_c * queue.mblock_n * queue.ublock_ct * 32, "_embedding_index: tensor dims mismatch q dims"
    return out.contiguous()
