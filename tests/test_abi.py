"""CPU-side checks of the C-ABI library: it loads, exports every function include/ttbfp.h declares,
and its pure (no-GPU) functions follow the reference's size rules."""
import ctypes
import os
import re

import pytest

from tt_buda_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "ttbfp.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ttbfp_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = declared_functions()
    assert len(names) >= 15
    L = ctypes.CDLL(capi.LIB_PATH)
    for n in names:
        assert hasattr(L, n), f"{n} is declared in include/ttbfp.h but not exported"
    assert sorted(capi.SYMBOLS) == names, "the ctypes table and the header must list the same functions"


def test_tile_bytes_match_data_format_byte_size():
    # pybuda/csrc/lower_to_buda/common.cpp:167-190 with 1024 elements
    F = capi.DataFormatCode
    assert capi.tile_bytes(F.Float32) == 4096
    assert capi.tile_bytes(F.Float16_b) == 2048
    assert capi.tile_bytes(F.Bfp8_b) == 1088
    assert capi.tile_bytes(F.Bfp4_b) == 576
    assert capi.tile_bytes(F.Bfp2_b) == 320
    # the family with the 5-bit exponent has the same sizes (common.cpp:174-179 does not distinguish)
    assert (capi.tile_bytes(F.Float16), capi.tile_bytes(F.Bfp8), capi.tile_bytes(F.Bfp4), capi.tile_bytes(F.Bfp2)) == (2048, 1088, 576, 320)
    # integer formats: common.cpp:180-186
    assert (capi.tile_bytes(F.Int32), capi.tile_bytes(F.RawUInt32)) == (4096, 4096)
    assert (capi.tile_bytes(F.UInt16), capi.tile_bytes(F.RawUInt16)) == (2048, 2048)
    assert (capi.tile_bytes(F.Int8), capi.tile_bytes(F.RawUInt8)) == (1024, 1024)
    for unsupported in (4, 9, 10, 13, 0xF3, 0xFF):  # Lf8 and codes that name no format
        assert capi.tile_bytes(unsupported) == 0


def test_packed_sizes_of_the_benchmark_configs():
    F = capi.DataFormatCode
    assert capi.packed_size(F.Bfp8_b, (1, 1, 1024, 1024)) == 1_114_112
    assert capi.packed_size(F.Bfp4_b, (1, 1, 4096, 4096)) == 9_437_184
    assert capi.packed_size(F.Bfp2_b, (1, 1, 4096, 4096)) == 5_242_880
    assert capi.packed_size(F.Bfp8_b, (8, 1, 8192, 8192)) == 570_425_344
    assert capi.packed_size(F.Bfp8_b, (1, 1, 31, 32)) == 0


def test_argument_errors_are_reported_without_a_gpu():
    L = capi.lib()
    shape = (ctypes.c_uint32 * 4)(1, 1, 33, 32)
    strides = (ctypes.c_uint64 * 4)(4224, 4224, 128, 4)
    st = L.ttbfp_tilize_pack(None, 0, shape, strides, 6, 0, None, 0, None)
    assert st == capi.RUNTIME_ERROR and b"multiples of the 32x32 tile" in L.ttbfp_last_error()
    st = L.ttbfp_gemm_bfp8b_bf16(32, 32, 48, None, None, None, 0, None, 5, None)
    assert st == capi.RUNTIME_ERROR and b"multiples of 32" in L.ttbfp_last_error()
    with pytest.raises(capi.BackendError):
        capi.check(L.ttbfp_unpack_untilize(None, 0, (ctypes.c_uint32 * 4)(1, 1, 32, 32), 5,
                                           (ctypes.c_uint64 * 4)(2048, 2048, 64, 2), None, None))


def test_queue_buffer_bytes_follow_the_geometry():
    # get_io_size_in_bytes: tiles per buffer x (tile bytes + 32 with headers), backend_api.cpp:710-722,
    # balancer_utils.hpp:24-27
    F = capi.DataFormatCode
    lay = capi.QueueLayout(2, 3, 2, 1, 1, 2, 0, 0)  # 4 x 6 tiles over 2 x 3 buffers of 2 x 2 tiles
    assert capi.queue_buffer_bytes(F.Bfp8_b, (5, 3, 128, 192), lay) == 5 * 3 * 4 * 1088
    lay.tile_header = 1
    assert capi.queue_buffer_bytes(F.Bfp8_b, (5, 3, 128, 192), lay) == 5 * 3 * 4 * 1120
    assert capi.queue_buffer_bytes(F.Bfp2_b, (1, 1, 128, 192), lay) == 4 * 352
    assert capi.queue_buffer_bytes(F.Bfp8_b, (1, 1, 128, 160), lay) == 0  # shape does not match the geometry
    assert capi.queue_buffer_bytes(9, (1, 1, 128, 192), lay) == 0


def test_queue_argument_errors_are_reported_without_a_gpu():
    L = capi.lib()
    shape = (ctypes.c_uint32 * 4)(1, 1, 64, 64)
    strides = (ctypes.c_uint64 * 4)(16384, 16384, 256, 4)
    lay = capi.QueueLayout(1, 1, 2, 1, 1, 1, 0, 0)  # covers 2 x 1 tiles, the tensor has 2 x 2
    st = L.ttbfp_tilize_pack_queue(None, 0, shape, strides, 6, 0, ctypes.byref(lay), 4352, None, 0, None)
    assert st == capi.RUNTIME_ERROR and b"covers 2 x 1 tiles" in L.ttbfp_last_error()
    lay = capi.QueueLayout(1, 2, 2, 1, 1, 1, 2, 0)
    st = L.ttbfp_tilize_pack_queue(None, 0, shape, strides, 6, 0, ctypes.byref(lay), 4352, None, 0, None)
    assert st == capi.RUNTIME_ERROR and b"ublock_order" in L.ttbfp_last_error()
    lay.ublock_order = 1
    st = L.ttbfp_tilize_pack_queue(None, 0, shape, strides, 6, 0, ctypes.byref(lay), 2176 - 16, None, 0, None)
    assert st == capi.RUNTIME_ERROR and b"below the 2176 bytes" in L.ttbfp_last_error()
    st = L.ttbfp_tilize_pack_queue(None, 0, shape, strides, 6, 0, ctypes.byref(lay), 2184, None, 0, None)
    assert st == capi.RUNTIME_ERROR and b"multiple of 16" in L.ttbfp_last_error()
    st = L.ttbfp_tilize_pack_queue(None, 0, shape, strides, 6, 0, ctypes.byref(lay), 2176, None, 4351, None)
    assert st == capi.RUNTIME_ERROR and b"4352 needed" in L.ttbfp_last_error()
    st = L.ttbfp_unpack_untilize_queue(None, 6, shape, None, 2176, 0, strides, None, None)
    assert st == capi.RUNTIME_ERROR and b"layout is NULL" in L.ttbfp_last_error()


def test_sized_entry_points_refuse_short_buffers_without_a_gpu():
    """The entry points that are told the size of every buffer fail before any launch when one is too small."""
    L = capi.lib()
    shape = (ctypes.c_uint32 * 4)(1, 1, 64, 64)
    strides = (ctypes.c_uint64 * 4)(16384, 16384, 256, 4)
    tiles = 4 * 1088
    st = L.ttbfp_unpack_untilize_sized(None, tiles - 1, 6, shape, None, 0, 0, strides, None, 16384, None)
    assert st == capi.RUNTIME_ERROR and b"source holds 4351 bytes" in L.ttbfp_last_error()
    st = L.ttbfp_unpack_untilize_sized(None, tiles, 6, shape, None, 0, 0, strides, None, 16383, None)
    assert st == capi.RUNTIME_ERROR and b"reaches 16384" in L.ttbfp_last_error()
    wide = (ctypes.c_uint64 * 4)(32768, 32768, 512, 4)  # rows 512 bytes apart: the last element ends at 63 * 512 + 256
    st = L.ttbfp_unpack_untilize_sized(None, tiles, 6, shape, None, 0, 0, wide, None, 63 * 512 + 255, None)
    assert st == capi.RUNTIME_ERROR and b"reaches 32512" in L.ttbfp_last_error()
    ragged = (ctypes.c_uint32 * 4)(1, 1, 40, 33)  # tiles cover 64 x 64; the result is 40 rows of 33 floats
    st = L.ttbfp_unpack_untilize_sized(None, tiles - 1, 6, ragged, None, 0, 0, (ctypes.c_uint64 * 4)(5280, 5280, 132, 4), None, 5280, None)
    assert st == capi.RUNTIME_ERROR and b"source holds" in L.ttbfp_last_error()
    # with both sizes right the call gets as far as the pointer check
    st = L.ttbfp_unpack_untilize_sized(None, tiles, 6, shape, None, 0, 0, strides, None, 16384, None)
    assert st == capi.RUNTIME_ERROR and b"NULL device pointer" in L.ttbfp_last_error()

    M, N, K = 64, 96, 128
    w_need = capi.packed_size(capi.DataFormatCode.Bfp8_b, (1, 1, K, N))
    args = dict(x=M * K * 2, w=w_need, b=N * 2, y=M * N * 2)

    def call(**short):
        a = dict(args, **short)
        return L.ttbfp_gemm_bfp8b_bf16_sized(M, N, K, None, a["x"], None, a["w"], ctypes.c_void_p(16), a["b"], 0, None, a["y"], 5, None, 0, None)

    assert call(x=args["x"] - 1) == capi.RUNTIME_ERROR and b"x holds" in L.ttbfp_last_error()
    assert call(w=w_need - 1) == capi.RUNTIME_ERROR and b"w holds" in L.ttbfp_last_error()
    assert call(b=N * 2 - 1) == capi.RUNTIME_ERROR and b"bias holds" in L.ttbfp_last_error()
    assert call(y=args["y"] - 1) == capi.RUNTIME_ERROR and b"y holds" in L.ttbfp_last_error()
    assert call() == capi.RUNTIME_ERROR and b"NULL device pointer" in L.ttbfp_last_error()
