"""ctypes binding of the CPU oracle (``libttbfp_oracle.so``).  TEST INFRASTRUCTURE ONLY.

Imported by ``tests/``, by ``__graft_entry__.smoke()`` and by the ``cpu_baseline`` leg of
``bench.py``; the product package never imports it.  Arrays are numpy: fp32 tensors as
``float32``, bf16 tensors as ``uint16`` bit patterns, packed tiles as ``uint8``.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libttbfp_oracle.so")

Float32, Float16_b, Bfp8_b, Bfp4_b, Bfp2_b = 0, 5, 6, 7, 15
Float16, Bfp8, Bfp4, Bfp2 = 1, 2, 3, 11  # the family with the 5-bit exponent of IEEE half
RawUInt32 = 0xF2  # integer tensors (embedding indices): tiled as they are
Int32, UInt16, Int8, RawUInt8, RawUInt16 = 8, 12, 14, 0xF0, 0xF1  # the other integer formats, tiled as they are too
TRUNCATE, NEAREST = 0, 1
MANTISSA_BITS = {Bfp8_b: 7, Bfp4_b: 3, Bfp2_b: 1, Bfp8: 7, Bfp4: 3, Bfp2: 1}
_U32x4 = ctypes.c_uint32 * 4
_U64x4 = ctypes.c_uint64 * 4


def build(force=False):
    """Compile the oracle with gcc (a few hundred lines of C: about a second)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.run(["make", "-B", "-C", _HERE], check=True, capture_output=True)
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_LIB_PATH)
        vp, u8p = ctypes.c_void_p, ctypes.c_void_p
        L.oracle_tile_bytes.restype = ctypes.c_uint32
        L.oracle_tile_bytes.argtypes = [ctypes.c_int]
        L.oracle_packed_size.restype = ctypes.c_uint64
        L.oracle_packed_size.argtypes = [ctypes.c_int, _U32x4]
        for name in ("oracle_tilize", "oracle_untilize"):
            f = getattr(L, name)
            f.restype = ctypes.c_int
            f.argtypes = [vp, ctypes.c_uint32, _U32x4, _U64x4, vp]
        L.oracle_quantize_block.restype = ctypes.c_uint8
        L.oracle_quantize_block.argtypes = [vp, ctypes.c_int, ctypes.c_int, u8p]
        L.oracle_dequantize_datum.restype = ctypes.c_uint32
        L.oracle_dequantize_datum.argtypes = [ctypes.c_uint8, ctypes.c_uint8, ctypes.c_int]
        L.oracle_quantize_block_a.restype = ctypes.c_uint8
        L.oracle_quantize_block_a.argtypes = [vp, ctypes.c_int, ctypes.c_int, u8p]
        L.oracle_dequantize_datum_a.restype = ctypes.c_uint16
        L.oracle_dequantize_datum_a.argtypes = [ctypes.c_uint8, ctypes.c_uint8, ctypes.c_int]
        L.oracle_pack_tiles.restype = ctypes.c_int
        L.oracle_pack_tiles.argtypes = [vp, ctypes.c_int, ctypes.c_uint64, ctypes.c_int, ctypes.c_int, u8p]
        L.oracle_unpack_tiles.restype = ctypes.c_int
        L.oracle_unpack_tiles.argtypes = [u8p, ctypes.c_int, ctypes.c_uint64, ctypes.c_int, vp]
        L.oracle_queue_map.restype = ctypes.c_int
        L.oracle_queue_map.argtypes = [vp, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint32, vp, vp, vp]
        L.oracle_queue_unmap.restype = ctypes.c_int
        L.oracle_queue_unmap.argtypes = [vp, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint64, vp, vp, vp]
        for name in ("oracle_tiles_to_queue", "oracle_queue_to_tiles"):
            f = getattr(L, name)
            f.restype = ctypes.c_int
            f.argtypes = [u8p, ctypes.c_int, _U32x4, vp, ctypes.c_uint64, u8p]
        L.oracle_embedding_index.restype = ctypes.c_int
        L.oracle_embedding_index.argtypes = [vp, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint32, vp, vp]
        L.oracle_prestride.restype = ctypes.c_int
        L.oracle_prestride.argtypes = [vp, ctypes.c_uint32, _U32x4, _U64x4, ctypes.c_uint32, vp, vp]
        L.oracle_tilize_pack.restype = ctypes.c_int
        L.oracle_tilize_pack.argtypes = [vp, ctypes.c_int, _U32x4, _U64x4, ctypes.c_int, ctypes.c_int, vp,
                                         ctypes.c_int]
        L.oracle_unpack_untilize.restype = ctypes.c_int
        L.oracle_unpack_untilize.argtypes = [vp, ctypes.c_int, _U32x4, ctypes.c_int, _U64x4, vp, ctypes.c_int]
        L.oracle_dequant_weight.restype = ctypes.c_int
        L.oracle_dequant_weight.argtypes = [u8p, ctypes.c_int, ctypes.c_uint32, ctypes.c_uint32, vp]
        L.oracle_gemm_bfp.restype = ctypes.c_int
        L.oracle_gemm_bfp.argtypes = [ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint32, vp, u8p, ctypes.c_int,
                                      vp, ctypes.c_int, vp]
        L.oracle_f32_to_bf16_rne.restype = ctypes.c_uint16
        L.oracle_f32_to_bf16_rne.argtypes = [ctypes.c_uint32]
        _lib = L
    return _lib


def _ptr(a):
    return ctypes.c_void_p(a.ctypes.data)


def _fmt_of(a):
    if a.dtype == np.float32:
        return Float32
    if a.dtype == np.uint16:
        return Float16_b
    if a.dtype == np.float16:
        return Float16
    if a.dtype == np.uint32:
        return RawUInt32
    if a.dtype == np.int32:
        return Int32
    if a.dtype == np.int16:
        return UInt16
    if a.dtype == np.int8:
        return Int8
    if a.dtype == np.uint8:
        return RawUInt8
    raise TypeError("oracle takes float32, float16, uint16 (bf16 bit pattern) or integer arrays, got %s" % a.dtype)


_INTEGER_ITEMSIZE = {RawUInt32: 4, Int32: 4, RawUInt16: 2, UInt16: 2, RawUInt8: 1, Int8: 1}


def _dtype_of(fmt):
    return {Float32: np.float32, Float16_b: np.uint16, Float16: np.float16, RawUInt32: np.uint32, Int32: np.int32, UInt16: np.int16,
            RawUInt16: np.int16, Int8: np.int8, RawUInt8: np.uint8}[fmt]


def _shape4(a):
    assert a.ndim == 4, "oracle works on 4-D [w, z, r, c] arrays"
    return _U32x4(*a.shape), _U64x4(*a.strides)


def tile_bytes(fmt):
    return lib().oracle_tile_bytes(fmt)


def packed_size(fmt, shape):
    return lib().oracle_packed_size(fmt, _U32x4(*shape))


def tilize(a):
    shape, strides = _shape4(a)
    out = np.empty(a.size, dtype=a.dtype)
    rc = lib().oracle_tilize(_ptr(a), a.itemsize, shape, strides, _ptr(out))
    assert rc == 0, "oracle_tilize failed"
    return out


def untilize(tiles, shape):
    out = np.empty(shape, dtype=tiles.dtype)
    s, st = _shape4(out)
    rc = lib().oracle_untilize(_ptr(tiles), tiles.itemsize, s, st, _ptr(out))
    assert rc == 0, "oracle_untilize failed"
    return out


def quantize_block(block_bits, mant_bits, rounding=TRUNCATE):
    """block_bits: 16 uint32 fp32 bit patterns -> (shared exponent, 16 datums)."""
    block_bits = np.ascontiguousarray(block_bits, dtype=np.uint32)
    assert block_bits.shape == (16,)
    datums = np.empty(16, dtype=np.uint8)
    e = lib().oracle_quantize_block(_ptr(block_bits), mant_bits, rounding, _ptr(datums))
    return int(e), datums


def quantize_block_a(block_half, mant_bits, rounding=TRUNCATE):
    """block_half: 16 float16 values -> (shared 5-bit exponent, 16 datums)."""
    block_half = np.ascontiguousarray(block_half, dtype=np.float16)
    assert block_half.shape == (16,)
    datums = np.empty(16, dtype=np.uint8)
    e = lib().oracle_quantize_block_a(_ptr(block_half), mant_bits, rounding, _ptr(datums))
    return int(e), datums


def dequantize_datum_a(datum, shared_exp, mant_bits):
    """float16 value of one A-family datum."""
    return np.array([lib().oracle_dequantize_datum_a(int(datum), int(shared_exp), mant_bits)], dtype=np.uint16).view(np.float16)[0]


def dequantize_datum(datum, shared_exp, mant_bits):
    return int(lib().oracle_dequantize_datum(int(datum), int(shared_exp), mant_bits))


def pack_tiles(tiles, dst_fmt, rounding=TRUNCATE):
    tiles = np.ascontiguousarray(tiles)
    ntiles = tiles.size // 1024
    out = np.empty(ntiles * tile_bytes(dst_fmt), dtype=np.uint8)
    rc = lib().oracle_pack_tiles(_ptr(tiles), _fmt_of(tiles), ntiles, dst_fmt, rounding, _ptr(out))
    assert rc == 0, "oracle_pack_tiles failed"
    return out


def unpack_tiles(packed, src_fmt, dst_fmt):
    ntiles = packed.size // tile_bytes(src_fmt)
    out = np.empty(ntiles * 1024, dtype=_dtype_of(dst_fmt))
    rc = lib().oracle_unpack_tiles(_ptr(packed), src_fmt, ntiles, dst_fmt, _ptr(out))
    assert rc == 0, "oracle_unpack_tiles failed"
    return out


def tilize_pack(a, dst_fmt, rounding=TRUNCATE, nthreads=1):
    """Row-major 4-D array (any strides) -> packed/tilized bytes in ``dst_fmt``."""
    shape, strides = _shape4(a)
    nbytes = packed_size(dst_fmt, a.shape)
    assert nbytes, "shape must be tile aligned and the format supported"
    out = np.empty(nbytes, dtype=np.uint8)
    # an integer format pairs with itself: the array's item size has to match, its signedness does not matter
    src_fmt = dst_fmt if dst_fmt in _INTEGER_ITEMSIZE and a.itemsize == _INTEGER_ITEMSIZE[dst_fmt] and a.dtype.kind in "iu" else _fmt_of(a)
    rc = lib().oracle_tilize_pack(_ptr(a), src_fmt, shape, strides, dst_fmt, rounding, _ptr(out), nthreads)
    assert rc == 0, "oracle_tilize_pack failed"
    return out


def unpack_untilize(packed, src_fmt, shape, dst_fmt, nthreads=1):
    out = np.empty(shape, dtype=_dtype_of(dst_fmt))
    s, st = _shape4(out)
    rc = lib().oracle_unpack_untilize(_ptr(packed), src_fmt, s, dst_fmt, st, _ptr(out), nthreads)
    assert rc == 0, "oracle_unpack_untilize failed"
    return out


class QueueLayout(ctypes.Structure):
    """grid / mblock / ublock geometry of a queue; ublock_order 0 = r, 1 = c."""
    _fields_ = [(n, ctypes.c_uint32) for n in
                ("grid_r", "grid_c", "mblock_m", "mblock_n", "ublock_rt", "ublock_ct", "ublock_order", "tile_header")]

    def tiles(self):
        return self.grid_r * self.mblock_m * self.ublock_rt, self.grid_c * self.mblock_n * self.ublock_ct

    def buffer_bytes(self, fmt, w, t):
        return w * t * self.mblock_m * self.mblock_n * self.ublock_rt * self.ublock_ct * (tile_bytes(fmt) + 32 * self.tile_header)


def queue_map(layout, t, r, c):
    """(t, tile row, tile column) -> (grid row, grid column, address in tiles inside the buffer's entry)."""
    gr, gc, a = ctypes.c_uint32(), ctypes.c_uint32(), ctypes.c_uint64()
    rc = lib().oracle_queue_map(ctypes.byref(layout), t, r, c, ctypes.byref(gr), ctypes.byref(gc), ctypes.byref(a))
    assert rc == 0, "oracle_queue_map failed"
    return gr.value, gc.value, a.value


def queue_unmap(layout, grid_r, grid_c, address):
    t, r, c = ctypes.c_uint32(), ctypes.c_uint32(), ctypes.c_uint32()
    rc = lib().oracle_queue_unmap(ctypes.byref(layout), grid_r, grid_c, address, ctypes.byref(t), ctypes.byref(r), ctypes.byref(c))
    assert rc == 0, "oracle_queue_unmap failed"
    return t.value, r.value, c.value


def tiles_to_queue(tiles, fmt, shape, layout, pitch=None):
    """Header-less packed tiles of a [w,t,R,C] tensor -> the bytes of the queue's buffers (gaps stay zero)."""
    nbuf = layout.grid_r * layout.grid_c
    per = layout.buffer_bytes(fmt, shape[0], shape[1])
    pitch = per if pitch is None else pitch
    out = np.zeros((nbuf - 1) * pitch + per, dtype=np.uint8)
    rc = lib().oracle_tiles_to_queue(_ptr(np.ascontiguousarray(tiles, dtype=np.uint8)), fmt, _U32x4(*shape), ctypes.byref(layout), pitch, _ptr(out))
    assert rc == 0, "oracle_tiles_to_queue failed"
    return out


def queue_to_tiles(queue, fmt, shape, layout, pitch=None):
    per = layout.buffer_bytes(fmt, shape[0], shape[1])
    pitch = per if pitch is None else pitch
    out = np.empty(packed_size(fmt, shape), dtype=np.uint8)
    rc = lib().oracle_queue_to_tiles(_ptr(np.ascontiguousarray(queue, dtype=np.uint8)), fmt, _U32x4(*shape), ctypes.byref(layout), pitch, _ptr(out))
    assert rc == 0, "oracle_queue_to_tiles failed"
    return out


def prestride(a, stride):
    """[w, C, H, W] array of 2- or 4-byte elements -> prestrided, tile-padded [w, 1, rows, cols]."""
    shape, strides = _shape4(a)
    rows = -(-stride * stride * a.shape[1] // 32) * 32
    cols = -(-(-(-a.shape[2] // stride)) * -(-a.shape[3] // stride) // 32) * 32
    out = np.empty((a.shape[0], 1, rows, cols), dtype=a.dtype)
    rc = (ctypes.c_uint32 * 2)()
    r = lib().oracle_prestride(_ptr(a), a.itemsize, shape, strides, stride, _ptr(out), rc)
    assert r == 0 and (rc[0], rc[1]) == (rows, cols), "oracle_prestride failed"
    return out


def embedding_index(index, valid, q_rt):
    """[w, n] (or [n]) integer index vectors, the first ``valid`` entries real -> the [w, 1, q_rt*32, cols] uint32 tensor an
    embedding queue takes (pybuda/pybuda/tensor.py:1382-1408)."""
    idx = np.ascontiguousarray(np.atleast_2d(index)).astype(np.uint32)
    w, n = idx.shape
    n_pad = -(-n // 32) * 32
    rows = n_pad // (q_rt * 32)
    width = -(-rows // 32) * 32
    out = np.empty((w, 1, q_rt * 32, width), dtype=np.uint32)
    cols = ctypes.c_uint32()
    rc = lib().oracle_embedding_index(_ptr(idx), w, n, valid, q_rt, _ptr(out), ctypes.byref(cols))
    assert rc == 0 and cols.value == width, "oracle_embedding_index failed"
    return out


def dequant_weight(w_packed, K, N, w_fmt=Bfp8_b):
    out = np.empty((K, N), dtype=np.float32)
    rc = lib().oracle_dequant_weight(_ptr(w_packed), w_fmt, K, N, _ptr(out))
    assert rc == 0, "oracle_dequant_weight failed"
    return out


def gemm_bfp(x_bf16, w_packed, N, bias_bf16=None, epilogue=0, w_fmt=Bfp8_b):
    M, K = x_bf16.shape
    x_bf16 = np.ascontiguousarray(x_bf16, dtype=np.uint16)
    out = np.empty((M, N), dtype=np.float32)
    bias_p = _ptr(np.ascontiguousarray(bias_bf16, dtype=np.uint16)) if bias_bf16 is not None else None
    rc = lib().oracle_gemm_bfp(M, N, K, _ptr(x_bf16), _ptr(w_packed), w_fmt, bias_p, epilogue, _ptr(out))
    assert rc == 0, "oracle_gemm_bfp failed"
    return out


def f32_to_bf16_bits(a, rounding=NEAREST):
    """float32 array -> uint16 bf16 bit patterns (round-to-nearest-even, or truncation)."""
    bits = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)
    if rounding == TRUNCATE:
        return (bits >> 16).astype(np.uint16)
    nan = ((bits & 0x7F800000) == 0x7F800000) & ((bits & 0x007FFFFF) != 0)
    rounded = ((bits.astype(np.uint64) + 0x7FFF + ((bits >> 16) & 1)) >> 16).astype(np.uint16)
    return np.where(nan, ((bits >> 16) | 0x40).astype(np.uint16), rounded)


def bf16_bits_to_f32(a):
    return (np.ascontiguousarray(a, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)
