"""ctypes view of the C ABI in ``include/ttbfp.h`` (``libttbfp.so``), on torch device tensors.

torch is used for device memory and for its current stream only; every conversion and the GEMM
run in the HIP library.  There is no CPU fallback: a missing library or a failing call raises.
"""
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libttbfp.so")

SUCCESS, RUNTIME_ERROR, TIMEOUT_ERROR = 0, 1, 2
ROUND_TRUNCATE, ROUND_NEAREST = 0, 1
EPILOGUE_NONE, EPILOGUE_GELU, EPILOGUE_GELU_TANH = 0, 1, 2
EPILOGUE_BIAS_F32 = 0x100  # ORed into the epilogue: the bias vector is fp32


class DataFormatCode:
    """Numeric tt::DataFormat values (pybuda/csrc/lower_to_buda/common.hpp:92-111) the library accepts."""

    Float32 = 0
    Float16_b = 5
    Bfp8_b = 6
    Bfp4_b = 7
    Bfp2_b = 15
    # the family with the 5-bit exponent of IEEE half: half sources and results only
    Float16 = 1
    Bfp8 = 2
    Bfp4 = 3
    Bfp2 = 11
    # integer tensors (embedding indices as RawUInt32; int32 / int8 tensors as Int32 / Int8): tiled as they are, to and from
    # tiles of the same format only
    RawUInt32 = 0xF2
    RawUInt16 = 0xF1
    RawUInt8 = 0xF0
    Int32 = 8
    UInt16 = 12
    Int8 = 14


_U32x4 = ctypes.c_uint32 * 4
_U64x4 = ctypes.c_uint64 * 4

class QueueLayout(ctypes.Structure):
    """ttbfp_queue_layout: grid / mblock / ublock geometry of a queue; ublock_order 0 = r, 1 = c."""

    _fields_ = [(n, ctypes.c_uint32) for n in
                ("grid_r", "grid_c", "mblock_m", "mblock_n", "ublock_rt", "ublock_ct", "ublock_order", "tile_header")]


_LAYOUT_P = ctypes.POINTER(QueueLayout)

# name -> (restype, argtypes): every symbol include/ttbfp.h declares
SYMBOLS = {
    "ttbfp_last_error": (ctypes.c_char_p, []),
    "ttbfp_init": (ctypes.c_int32, [ctypes.c_int32]),
    "ttbfp_device_count": (ctypes.c_int32, []),
    "ttbfp_tile_bytes": (ctypes.c_uint32, [ctypes.c_uint8]),
    "ttbfp_packed_size": (ctypes.c_uint64, [ctypes.c_uint8, _U32x4]),
    "ttbfp_alloc": (ctypes.c_int32, [ctypes.c_uint64, ctypes.POINTER(ctypes.c_void_p)]),
    "ttbfp_free": (ctypes.c_int32, [ctypes.c_void_p]),
    "ttbfp_host_alloc": (ctypes.c_int32, [ctypes.c_uint64, ctypes.POINTER(ctypes.c_void_p)]),
    "ttbfp_host_free": (ctypes.c_int32, [ctypes.c_void_p]),
    "ttbfp_memcpy_h2d": (ctypes.c_int32, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_uint64, ctypes.c_void_p]),
    "ttbfp_memcpy_d2h": (ctypes.c_int32, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_uint64, ctypes.c_void_p]),
    "ttbfp_memcpy_d2d": (ctypes.c_int32, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_uint64, ctypes.c_void_p]),
    "ttbfp_pointer_is_device": (ctypes.c_int32, [ctypes.c_void_p]),
    "ttbfp_stream_create": (ctypes.c_int32, [ctypes.POINTER(ctypes.c_void_p)]),
    "ttbfp_stream_destroy": (ctypes.c_int32, [ctypes.c_void_p]),
    "ttbfp_device_synchronize": (ctypes.c_int32, []),
    "ttbfp_stream_synchronize": (ctypes.c_int32, [ctypes.c_void_p, ctypes.c_int32]),
    "ttbfp_tilize_pack": (ctypes.c_int32, [ctypes.c_void_p, ctypes.c_uint8, _U32x4, _U64x4, ctypes.c_uint8,
                                           ctypes.c_int32, ctypes.c_void_p, ctypes.c_uint64, ctypes.c_void_p]),
    "ttbfp_unpack_untilize": (ctypes.c_int32, [ctypes.c_void_p, ctypes.c_uint8, _U32x4, ctypes.c_uint8, _U64x4,
                                               ctypes.c_void_p, ctypes.c_void_p]),
    "ttbfp_queue_buffer_bytes": (ctypes.c_uint64, [ctypes.c_uint8, _U32x4, _LAYOUT_P]),
    "ttbfp_tilize_pack_queue": (ctypes.c_int32, [ctypes.c_void_p, ctypes.c_uint8, _U32x4, _U64x4, ctypes.c_uint8, ctypes.c_int32,
                                                 _LAYOUT_P, ctypes.c_uint64, ctypes.c_void_p, ctypes.c_uint64, ctypes.c_void_p]),
    "ttbfp_unpack_untilize_queue": (ctypes.c_int32, [ctypes.c_void_p, ctypes.c_uint8, _U32x4, _LAYOUT_P, ctypes.c_uint64,
                                                     ctypes.c_uint8, _U64x4, ctypes.c_void_p, ctypes.c_void_p]),
    "ttbfp_tilize_pack_padded": (ctypes.c_int32, [ctypes.c_void_p, ctypes.c_uint8, _U32x4, _U64x4, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint8,
                                                  ctypes.c_int32, _LAYOUT_P, ctypes.c_uint64, ctypes.c_void_p, ctypes.c_uint64, ctypes.c_void_p]),
    "ttbfp_unpack_untilize_narrow": (ctypes.c_int32, [ctypes.c_void_p, ctypes.c_uint8, _U32x4, _LAYOUT_P, ctypes.c_uint64,
                                                      ctypes.c_uint8, _U64x4, ctypes.c_void_p, ctypes.c_void_p]),
    "ttbfp_unpack_untilize_sized": (ctypes.c_int32, [ctypes.c_void_p, ctypes.c_uint64, ctypes.c_uint8, _U32x4, _LAYOUT_P, ctypes.c_uint64,
                                                     ctypes.c_uint8, _U64x4, ctypes.c_void_p, ctypes.c_uint64, ctypes.c_void_p]),
    "ttbfp_prestride_shape": (ctypes.c_uint64, [ctypes.c_uint32, _U32x4, ctypes.c_uint32, ctypes.POINTER(ctypes.c_uint32 * 2)]),
    "ttbfp_prestride": (ctypes.c_int32, [ctypes.c_void_p, ctypes.c_uint32, _U32x4, _U64x4, ctypes.c_uint32, ctypes.c_void_p,
                                         ctypes.c_uint64, ctypes.c_void_p]),
    "ttbfp_gemm_bfp8b_bf16": (ctypes.c_int32, [ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_void_p,
                                               ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int32, ctypes.c_void_p,
                                               ctypes.c_uint8, ctypes.c_void_p]),
    "ttbfp_gemm_bfp8b_workspace_bytes": (ctypes.c_uint64, [ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint32]),
    "ttbfp_gemm_bfp8b_bf16_ws": (ctypes.c_int32, [ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_void_p,
                                                  ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int32, ctypes.c_void_p,
                                                  ctypes.c_uint8, ctypes.c_void_p, ctypes.c_uint64, ctypes.c_void_p]),
    "ttbfp_gemm_bfp8b_bf16_sized": (ctypes.c_int32, [ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_void_p, ctypes.c_uint64,
                                                     ctypes.c_void_p, ctypes.c_uint64, ctypes.c_void_p, ctypes.c_uint64, ctypes.c_int32,
                                                     ctypes.c_void_p, ctypes.c_uint64, ctypes.c_uint8, ctypes.c_void_p, ctypes.c_uint64,
                                                     ctypes.c_void_p]),
    "ttbfp_gemm_f32": (ctypes.c_int32, [ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                        ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p]),
    "ttbfp_static_scratch_bytes": (ctypes.c_uint64, []),
    "ttbfp_gemm_bfp8b_bf16_static": (ctypes.c_int32, [ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_void_p,
                                                      ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int32, ctypes.c_void_p,
                                                      ctypes.c_uint8, ctypes.c_void_p]),
    "ttbfp_tilize_pack_cpu": (ctypes.c_int32, [ctypes.c_void_p, ctypes.c_uint8, _U32x4, _U64x4, ctypes.c_uint8, ctypes.c_int32,
                                               ctypes.c_void_p, ctypes.c_uint64]),
    "ttbfp_unpack_untilize_cpu": (ctypes.c_int32, [ctypes.c_void_p, ctypes.c_uint8, _U32x4, ctypes.c_uint8, _U64x4, ctypes.c_void_p]),
    "ttbfp_gemm_bfp8b_bf16_cpu": (ctypes.c_int32, [ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_void_p, ctypes.c_void_p,
                                                   ctypes.c_void_p, ctypes.c_int32, ctypes.c_void_p, ctypes.c_uint8]),
}

_lib = None


def lib():
    """The loaded C-ABI library.  Raises if it has not been built (``__graft_entry__.build()``)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build the HIP library first (python -c 'import __graft_entry__ as g; g.build()')")
        L = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SYMBOLS.items():
            fn = getattr(L, name)
            fn.restype, fn.argtypes = res, args
        _lib = L
    return _lib


class BackendError(RuntimeError):
    def __init__(self, status, text):
        super().__init__(text)
        self.status = status


def check(status):
    if status != SUCCESS:
        raise BackendError(status, lib().ttbfp_last_error().decode() or f"status {status}")


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


_TORCH_FMT = {torch.float32: DataFormatCode.Float32, torch.bfloat16: DataFormatCode.Float16_b,
              torch.float16: DataFormatCode.Float16, torch.int32: DataFormatCode.RawUInt32, torch.int16: DataFormatCode.UInt16,
              torch.int8: DataFormatCode.Int8, torch.uint8: DataFormatCode.RawUInt8}
_FMT_TORCH = {v: k for k, v in _TORCH_FMT.items()}
_INTEGER_ITEMSIZE = {DataFormatCode.RawUInt32: 4, DataFormatCode.Int32: 4, DataFormatCode.RawUInt16: 2, DataFormatCode.UInt16: 2,
                     DataFormatCode.RawUInt8: 1, DataFormatCode.Int8: 1}


def _fmt_of(tensor, tile_fmt):
    """Format code of a row-major tensor that goes into / comes out of tiles of ``tile_fmt``: an integer format pairs with
    itself, so an integer tensor of matching item size takes the tiles' own code, whatever its signedness."""
    if tile_fmt in _INTEGER_ITEMSIZE and not tensor.dtype.is_floating_point and tensor.element_size() == _INTEGER_ITEMSIZE[tile_fmt]:
        return tile_fmt
    return _TORCH_FMT[tensor.dtype]


def tile_bytes(fmt):
    return lib().ttbfp_tile_bytes(fmt)


def packed_size(fmt, shape):
    return lib().ttbfp_packed_size(fmt, _U32x4(*shape))


def tilize_pack(src, dst_fmt, rounding=ROUND_TRUNCATE, out=None):
    """4-D fp32/bf16 device tensor (any strides) -> uint8 device tensor of tiles in ``dst_fmt``."""
    assert src.is_cuda and src.dim() == 4, "tilize_pack takes a 4-D device tensor [w, z, r, c]"
    if src.dtype not in _TORCH_FMT:
        raise BackendError(RUNTIME_ERROR, f"unsupported source dtype {src.dtype}")
    nbytes = packed_size(dst_fmt, src.shape)
    if out is None:
        out = torch.empty(nbytes, dtype=torch.uint8, device=src.device)
    else:
        assert out.is_cuda and out.device == src.device and out.dtype == torch.uint8 and out.is_contiguous(), "out must be a contiguous uint8 device tensor"
    strides = _U64x4(*[s * src.element_size() for s in src.stride()])
    check(lib().ttbfp_tilize_pack(src.data_ptr(), _fmt_of(src, dst_fmt), _U32x4(*src.shape), strides, dst_fmt, rounding,
                                  out.data_ptr(), out.numel(), _stream()))
    return out


def unpack_untilize(packed, src_fmt, shape, dtype=torch.float32, out=None):
    """uint8 device tensor of tiles -> row-major 4-D device tensor of ``dtype`` (fp32 or bf16; fp16 for the
    formats with a 5-bit exponent)."""
    assert packed.is_cuda and packed.dtype == torch.uint8 and packed.is_contiguous()
    if out is None:
        out = torch.empty(tuple(shape), dtype=dtype, device=packed.device)
    else:  # the C ABI takes strides but no size for the destination
        assert out.is_cuda and out.device == packed.device and tuple(out.shape) == tuple(shape), "out must be a device tensor of the given shape"
        assert out.dtype in _TORCH_FMT, "unsupported result dtype"
    need = packed_size(src_fmt, shape)
    if packed.numel() < need:
        raise BackendError(RUNTIME_ERROR, f"packed buffer holds {packed.numel()} bytes, {need} needed")
    strides = _U64x4(*[s * out.element_size() for s in out.stride()])
    check(lib().ttbfp_unpack_untilize(packed.data_ptr(), src_fmt, _U32x4(*shape), _fmt_of(out, src_fmt), strides,
                                      out.data_ptr(), _stream()))
    return out


def _bytes_from(t):
    """Bytes between a tensor's first element and the end of the memory it lives in."""
    return t.untyped_storage().nbytes() - t.storage_offset() * t.element_size()


def unpack_untilize_sized(packed, src_fmt, shape, dtype=torch.float32, layout=None, pitch=None, out=None):
    """``unpack_untilize`` / ``_queue`` / ``_narrow`` through the entry point that is told how much memory both sides hold
    and refuses, before any launch, a source too small for the tiles or a destination the strided result would overrun."""
    assert packed.is_cuda and packed.dtype == torch.uint8 and packed.is_contiguous()
    if out is None:
        out = torch.empty(tuple(shape), dtype=dtype, device=packed.device)
    strides = _U64x4(*[s * out.element_size() for s in out.stride()])
    if layout is not None and pitch is None:
        pitch = queue_buffer_bytes(src_fmt, _tiled(shape), layout)
    check(lib().ttbfp_unpack_untilize_sized(packed.data_ptr(), packed.numel(), src_fmt, _U32x4(*shape),
                                            ctypes.byref(layout) if layout is not None else None, pitch or 0, _fmt_of(out, src_fmt), strides,
                                            out.data_ptr(), _bytes_from(out), _stream()))
    return out


def _tiled(shape):
    return (shape[0], shape[1], (shape[2] + 31) // 32 * 32, (shape[3] + 31) // 32 * 32)


def tilize_pack_padded(src, dst_fmt, replicate_rows=False, replicate_cols=False, rounding=ROUND_TRUNCATE, layout=None, pitch=None, out=None):
    """``tilize_pack`` of a 4-D device tensor whose rows / columns need not be multiples of 32: the padding to whole tiles
    (zeros, or copies of a single row / column with ``replicate_*``) happens inside the launch."""
    assert src.is_cuda and src.dim() == 4
    if src.dtype not in _TORCH_FMT:
        raise BackendError(RUNTIME_ERROR, f"unsupported source dtype {src.dtype}")
    tiled = _tiled(src.shape)
    if layout is None:
        nbytes, pitch = packed_size(dst_fmt, tiled), 0
    else:
        per = queue_buffer_bytes(dst_fmt, tiled, layout)
        pitch = per if pitch is None else pitch
        nbytes = max(layout.grid_r * layout.grid_c - 1, 0) * pitch + per
    if out is None:
        out = torch.zeros(nbytes, dtype=torch.uint8, device=src.device)
    else:
        assert out.is_cuda and out.device == src.device and out.dtype == torch.uint8 and out.is_contiguous()
    strides = _U64x4(*[s * src.element_size() for s in src.stride()])
    check(lib().ttbfp_tilize_pack_padded(src.data_ptr(), _fmt_of(src, dst_fmt), _U32x4(*src.shape), strides, int(replicate_rows), int(replicate_cols),
                                         dst_fmt, rounding, ctypes.byref(layout) if layout is not None else None, pitch, out.data_ptr(),
                                         out.numel(), _stream()))
    return out


def unpack_untilize_narrow(packed, src_fmt, shape, dtype=torch.float32, layout=None, pitch=None, out=None):
    """``unpack_untilize`` writing only ``shape`` (rows / columns need not be multiples of 32) out of tiles that cover it
    rounded up: the narrowing happens inside the launch."""
    assert packed.is_cuda and packed.dtype == torch.uint8 and packed.is_contiguous()
    tiled = _tiled(shape)
    if layout is None:
        need, pitch = packed_size(src_fmt, tiled), 0
    else:
        per = queue_buffer_bytes(src_fmt, tiled, layout)
        pitch = per if pitch is None else pitch
        need = max(layout.grid_r * layout.grid_c - 1, 0) * pitch + per
    if packed.numel() < need:
        raise BackendError(RUNTIME_ERROR, f"packed buffer holds {packed.numel()} bytes, {need} needed")
    if out is None:
        out = torch.empty(tuple(shape), dtype=dtype, device=packed.device)
    else:
        assert out.is_cuda and out.device == packed.device and tuple(out.shape) == tuple(shape) and out.dtype in _TORCH_FMT
    strides = _U64x4(*[s * out.element_size() for s in out.stride()])
    check(lib().ttbfp_unpack_untilize_narrow(packed.data_ptr(), src_fmt, _U32x4(*shape), ctypes.byref(layout) if layout is not None else None,
                                             pitch, _fmt_of(out, src_fmt), strides, out.data_ptr(), _stream()))
    return out


def queue_buffer_bytes(fmt, shape, layout):
    return lib().ttbfp_queue_buffer_bytes(fmt, _U32x4(*shape), ctypes.byref(layout))


def tilize_pack_queue(src, dst_fmt, layout, pitch=None, rounding=ROUND_TRUNCATE, out=None):
    """``tilize_pack`` with the tiles laid into the buffers of a queue with geometry ``layout``; buffers ``pitch`` bytes apart
    (default: back to back).  A fresh result is zero-filled, so bytes between buffers read as zero."""
    assert src.is_cuda and src.dim() == 4, "tilize_pack_queue takes a 4-D device tensor [w, t, r, c]"
    if src.dtype not in _TORCH_FMT:
        raise BackendError(RUNTIME_ERROR, f"unsupported source dtype {src.dtype}")
    per = queue_buffer_bytes(dst_fmt, src.shape, layout)
    pitch = per if pitch is None else pitch
    if out is None:
        out = torch.zeros(max(layout.grid_r * layout.grid_c - 1, 0) * pitch + per, dtype=torch.uint8, device=src.device)
    else:
        assert out.is_cuda and out.device == src.device and out.dtype == torch.uint8 and out.is_contiguous(), "out must be a contiguous uint8 device tensor"
    strides = _U64x4(*[s * src.element_size() for s in src.stride()])
    check(lib().ttbfp_tilize_pack_queue(src.data_ptr(), _fmt_of(src, dst_fmt), _U32x4(*src.shape), strides, dst_fmt, rounding,
                                        ctypes.byref(layout), pitch, out.data_ptr(), out.numel(), _stream()))
    return out


def unpack_untilize_queue(queue, src_fmt, shape, layout, pitch=None, dtype=torch.float32, out=None):
    """``unpack_untilize`` reading the tiles from the buffers of a queue with geometry ``layout``."""
    assert queue.is_cuda and queue.dtype == torch.uint8
    per = queue_buffer_bytes(src_fmt, shape, layout)
    pitch = per if pitch is None else pitch
    need = max(layout.grid_r * layout.grid_c - 1, 0) * pitch + per
    if queue.numel() < need:
        raise BackendError(RUNTIME_ERROR, f"queue memory holds {queue.numel()} bytes, {need} needed")
    if out is None:
        out = torch.empty(tuple(shape), dtype=dtype, device=queue.device)
    else:
        assert out.is_cuda and out.device == queue.device and tuple(out.shape) == tuple(shape) and out.dtype in _TORCH_FMT
    strides = _U64x4(*[s * out.element_size() for s in out.stride()])
    check(lib().ttbfp_unpack_untilize_queue(queue.data_ptr(), src_fmt, _U32x4(*shape), ctypes.byref(layout), pitch,
                                            _fmt_of(out, src_fmt), strides, out.data_ptr(), _stream()))
    return out


def prestride(src, stride):
    """[w, C, H, W] device tensor -> [w, 1, rows, cols]: the prestriding transform of a strided convolution's activation,
    zero-padded to whole tiles (what ``push_input`` does for a queue whose descriptor carries a stride)."""
    assert src.is_cuda and src.dim() == 4 and src.element_size() in (2, 4)
    rc = (ctypes.c_uint32 * 2)()
    nbytes = lib().ttbfp_prestride_shape(src.element_size(), _U32x4(*src.shape), stride, ctypes.byref(rc))
    out = torch.empty((src.shape[0], 1, rc[0], rc[1]), dtype=src.dtype, device=src.device)
    strides = _U64x4(*[s * src.element_size() for s in src.stride()])
    check(lib().ttbfp_prestride(src.data_ptr(), src.element_size(), _U32x4(*src.shape), strides, stride, out.data_ptr(), nbytes, _stream()))
    return out


def gemm_workspace_bytes(M, N, K):
    """Scratch bytes that ``gemm_bfp8b(..., workspace=...)`` can use for this shape: a bf16 panel of W converted once (many rows)
    or fp32 partial sums of a split over K (few macro tiles); 0 if neither applies."""
    return lib().ttbfp_gemm_bfp8b_workspace_bytes(M, N, K)


def gemm_bfp8b(x, w_packed, N, bias=None, epilogue=EPILOGUE_NONE, out_dtype=torch.bfloat16, out=None, workspace=None, sized=False):
    """Y = epilogue(X @ dequant(W) + bias).  x: [M, K] bf16 device tensor; w_packed: Bfp8_b tiles of W[K, N]; bias: [N] in bf16,
    or in fp32 (the sum of a bias over a weight stack).  ``workspace``: an optional uint8 device tensor of
    ``gemm_workspace_bytes(M, N, K)`` bytes.  ``sized``: go through the entry point that is told the size of every buffer."""
    assert x.is_cuda and x.dtype == torch.bfloat16 and x.dim() == 2 and x.is_contiguous()
    M, K = x.shape
    assert w_packed.is_cuda and w_packed.dtype == torch.uint8 and w_packed.is_contiguous()
    if w_packed.numel() < packed_size(DataFormatCode.Bfp8_b, (1, 1, K, N)):
        raise BackendError(RUNTIME_ERROR, "packed weight buffer too small for [K, N]")
    if out is None:
        out = torch.empty((M, N), dtype=out_dtype, device=x.device)
    else:  # the C ABI takes no size for y: a wrong one would be an out-of-bounds device write
        assert out.is_cuda and out.device == x.device and out.is_contiguous() and tuple(out.shape) == (M, N), "out must be a contiguous [M, N] device tensor"
        assert out.dtype in (torch.bfloat16, torch.float32), "out must be bf16 or fp32"
    if bias is not None:
        assert bias.is_cuda and bias.dtype in (torch.bfloat16, torch.float32) and bias.numel() == N and bias.is_contiguous()
        if bias.dtype == torch.float32:
            epilogue |= EPILOGUE_BIAS_F32
    if workspace is not None:
        assert workspace.is_cuda and workspace.dtype == torch.uint8 and workspace.is_contiguous()
    if sized:
        check(lib().ttbfp_gemm_bfp8b_bf16_sized(M, N, K, x.data_ptr(), _bytes_from(x), w_packed.data_ptr(), w_packed.numel(),
                                                bias.data_ptr() if bias is not None else None, _bytes_from(bias) if bias is not None else 0,
                                                epilogue, out.data_ptr(), _bytes_from(out), _TORCH_FMT[out.dtype],
                                                workspace.data_ptr() if workspace is not None else None,
                                                workspace.numel() if workspace is not None else 0, _stream()))
        return out
    if workspace is not None:
        check(lib().ttbfp_gemm_bfp8b_bf16_ws(M, N, K, x.data_ptr(), w_packed.data_ptr(),
                                             bias.data_ptr() if bias is not None else None, epilogue, out.data_ptr(),
                                             _TORCH_FMT[out.dtype], workspace.data_ptr(), workspace.numel(), _stream()))
        return out
    check(lib().ttbfp_gemm_bfp8b_bf16(M, N, K, x.data_ptr(), w_packed.data_ptr(),
                                      bias.data_ptr() if bias is not None else None, epilogue, out.data_ptr(),
                                      _TORCH_FMT[out.dtype], _stream()))
    return out


def gemm_f32(x, w, bias=None, epilogue=EPILOGUE_NONE, out=None):
    """Y = epilogue(X @ W + bias) on fp32 row-major device tensors: the matmul of the unquantized (full-precision) mode."""
    assert x.is_cuda and x.dtype == torch.float32 and x.dim() == 2 and x.is_contiguous()
    assert w.is_cuda and w.dtype == torch.float32 and w.dim() == 2 and w.is_contiguous() and w.shape[0] == x.shape[1]
    M, K = x.shape
    N = w.shape[1]
    if out is None:
        out = torch.empty((M, N), dtype=torch.float32, device=x.device)
    else:
        assert out.is_cuda and out.dtype == torch.float32 and out.is_contiguous() and tuple(out.shape) == (M, N)
    if bias is not None:
        assert bias.is_cuda and bias.dtype == torch.float32 and bias.numel() == N and bias.is_contiguous()
    check(lib().ttbfp_gemm_f32(M, N, K, x.data_ptr(), w.data_ptr(), bias.data_ptr() if bias is not None else None, epilogue,
                               out.data_ptr(), _stream()))
    return out


# ---- host-memory twins: CPU tensors in, CPU tensors out, no device --------------------------------------------------

def tilize_pack_cpu(src, dst_fmt, rounding=ROUND_TRUNCATE):
    """``tilize_pack`` on a 4-D tensor in host memory (any strides): the library's CPU twin of the conversion."""
    assert not src.is_cuda and src.dim() == 4
    if src.dtype not in _TORCH_FMT:
        raise BackendError(RUNTIME_ERROR, f"unsupported source dtype {src.dtype}")
    out = torch.empty(packed_size(dst_fmt, src.shape), dtype=torch.uint8)
    strides = _U64x4(*[s * src.element_size() for s in src.stride()])
    check(lib().ttbfp_tilize_pack_cpu(src.data_ptr(), _fmt_of(src, dst_fmt), _U32x4(*src.shape), strides, dst_fmt, rounding, out.data_ptr(), out.numel()))
    return out


def unpack_untilize_cpu(packed, src_fmt, shape, dtype=torch.float32):
    """``unpack_untilize`` on tiles in host memory."""
    assert not packed.is_cuda and packed.dtype == torch.uint8 and packed.is_contiguous()
    need = packed_size(src_fmt, shape)
    if packed.numel() < need:
        raise BackendError(RUNTIME_ERROR, f"packed buffer holds {packed.numel()} bytes, {need} needed")
    out = torch.empty(tuple(shape), dtype=dtype)
    strides = _U64x4(*[s * out.element_size() for s in out.stride()])
    check(lib().ttbfp_unpack_untilize_cpu(packed.data_ptr(), src_fmt, _U32x4(*shape), _fmt_of(out, src_fmt), strides, out.data_ptr()))
    return out


def gemm_bfp8b_cpu(x, w_packed, N, bias=None, epilogue=EPILOGUE_NONE, out_dtype=torch.bfloat16):
    """``gemm_bfp8b`` on host memory: dequantize-then-fp32-matmul, the library's CPU twin of the matmul."""
    assert not x.is_cuda and x.dtype == torch.bfloat16 and x.dim() == 2 and x.is_contiguous()
    assert not w_packed.is_cuda and w_packed.dtype == torch.uint8 and w_packed.is_contiguous()
    M, K = x.shape
    assert w_packed.numel() >= packed_size(DataFormatCode.Bfp8_b, (1, 1, K, N))
    if bias is not None:
        assert not bias.is_cuda and bias.is_contiguous() and bias.numel() >= N and bias.dtype in (torch.bfloat16, torch.float32)
        if bias.dtype == torch.float32:
            epilogue |= EPILOGUE_BIAS_F32
    out = torch.empty(M, N, dtype=out_dtype)
    check(lib().ttbfp_gemm_bfp8b_bf16_cpu(M, N, K, x.data_ptr(), w_packed.data_ptr(), bias.data_ptr() if bias is not None else None, epilogue,
                                          out.data_ptr(), _TORCH_FMT[out_dtype]))
    return out
