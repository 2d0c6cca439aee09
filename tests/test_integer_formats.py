"""Integer queues: Int8, UInt16, Int32 and RawUInt8 / RawUInt16 / RawUInt32 tensors are tiled as they are (tile sizes
pybuda/csrc/lower_to_buda/common.cpp:180-186; int32 and int8 torch tensors become Int32 and Int8 descriptors,
pybuda/pybuda/tensor.py:667-670; device_connector.py:204 names the three raw formats).  The oracle is held against a
reshape / transpose statement of the tile and face order; the kernels against the oracle, bit for bit, with random bit
patterns (every 16-bit pattern includes the NaNs and denormals of bf16: nothing may look at the bits)."""
import numpy as np
import pytest
import torch

import oracle as O

FORMATS = [(O.Int8, np.int8), (O.RawUInt8, np.uint8), (O.UInt16, np.int16), (O.RawUInt16, np.int16), (O.Int32, np.int32),
           (O.RawUInt32, np.uint32)]


def random_ints(rng, shape, dtype):
    bits = rng.integers(0, 256, size=(int(np.prod(shape)) * np.dtype(dtype).itemsize,), dtype=np.uint8)
    return bits.view(dtype).reshape(shape)


def tiles_by_reshape(x):
    """[w, z, R, C] -> tiles [w][z][R/32][C/32], each tile four 16 x 16 faces (top-left, top-right, bottom-left, bottom-right)"""
    w, z, R, C = x.shape
    t = x.reshape(w, z, R // 32, 2, 16, C // 32, 2, 16)  # w z tr fr r tc fc c
    return np.ascontiguousarray(t.transpose(0, 1, 2, 5, 3, 6, 4, 7)).reshape(-1)


@pytest.mark.parametrize("fmt,dtype", FORMATS)
def test_oracle_tiles_integers_as_they_are(fmt, dtype):
    rng = np.random.default_rng(fmt)
    x = random_ints(rng, (2, 3, 64, 96), dtype)
    t = O.tilize_pack(x, fmt)
    assert t.nbytes == O.packed_size(fmt, x.shape) == x.nbytes
    assert np.array_equal(t, tiles_by_reshape(x).view(np.uint8))
    assert np.array_equal(O.unpack_untilize(t, fmt, x.shape, fmt).view(dtype), x)
    strided = random_ints(rng, (1, 2, 64, 128), dtype)[:, :, :, ::2]  # element stride 2
    assert np.array_equal(O.tilize_pack(strided, fmt), tiles_by_reshape(np.ascontiguousarray(strided)).view(np.uint8))


def test_oracle_refuses_mixed_integer_pairs():
    x = np.zeros((1, 1, 32, 32), dtype=np.int32)
    out = np.zeros(8192, dtype=np.uint8)
    L = O.lib()
    for src, dst in ((O.Int32, O.RawUInt32), (O.Int32, O.Float32), (O.Float32, O.Int32), (O.Int8, O.RawUInt8), (O.UInt16, O.Float16_b),
                     (O.Int32, O.Bfp8_b)):
        assert L.oracle_tilize_pack(O._ptr(x), src, *O._shape4(x), dst, 0, O._ptr(out), 1) != 0, (src, dst)


@pytest.mark.gpu
@pytest.mark.parametrize("fmt,dtype", FORMATS)
def test_gpu_integer_tiles_match_the_oracle(fmt, dtype):
    from tt_buda_amd import capi
    tdt = {np.int8: torch.int8, np.uint8: torch.uint8, np.int16: torch.int16, np.int32: torch.int32, np.uint32: torch.int32}[dtype]
    rng = np.random.default_rng(100 + fmt)
    x = random_ints(rng, (2, 2, 96, 160), dtype)
    xd = torch.from_numpy(x.view({np.uint32: np.int32}.get(dtype, dtype))).cuda()
    print("[case] integer tiles", fmt, dtype.__name__, flush=True)
    t = capi.tilize_pack(xd, fmt)
    want = O.tilize_pack(x, fmt)
    assert np.array_equal(t.cpu().numpy(), want)
    back = capi.unpack_untilize(t, fmt, x.shape, tdt)
    assert torch.equal(back, xd)
    # a transposed (strided) source takes the general kernels
    xt = xd.transpose(2, 3).contiguous().transpose(2, 3)
    assert np.array_equal(capi.tilize_pack(xt, fmt).cpu().numpy(), want)
    # ragged shape: zero padding inside the launch, narrowing on the way back
    r = random_ints(rng, (1, 2, 50, 70), dtype)
    rd = torch.from_numpy(r.view({np.uint32: np.int32}.get(dtype, dtype))).cuda()
    padded = np.zeros((1, 2, 64, 96), dtype=dtype)
    padded[:, :, :50, :70] = r
    tp = capi.tilize_pack_padded(rd, fmt)
    assert np.array_equal(tp.cpu().numpy(), O.tilize_pack(padded, fmt))
    assert torch.equal(capi.unpack_untilize_narrow(tp, fmt, r.shape, tdt), rd)
    # queue buffers with a grid, micro blocks and tile headers
    lay, olay = capi.QueueLayout(1, 5, 3, 1, 1, 1, 1, 1), O.QueueLayout(1, 5, 3, 1, 1, 1, 1, 1)
    q = capi.tilize_pack_queue(xd, fmt, lay)
    assert np.array_equal(q.cpu().numpy(), O.tiles_to_queue(want, fmt, x.shape, olay))
    assert torch.equal(capi.unpack_untilize_queue(q, fmt, x.shape, lay, dtype=tdt), xd)
    # an integer format pairs with itself only
    with pytest.raises(capi.BackendError, match="pairs with itself only"):
        capi.unpack_untilize(t, fmt, x.shape, torch.float32 if x.itemsize == 4 else torch.bfloat16)
    with pytest.raises(capi.BackendError, match="pairs with itself only"):
        capi.tilize_pack(xd.float(), fmt)


@pytest.mark.gpu
def test_gpu_integer_queues_through_the_host_layer():
    from tt_buda_amd import tensor as T
    from tt_buda_amd._C import DataFormat as DF
    from tt_buda_amd._C import backend_api as B
    from tt_buda_amd.backend import BackendAPI
    OK, ERR = B.BackendStatusCode.Success, B.BackendStatusCode.RuntimeError
    api = BackendAPI(0)
    try:
        rng = np.random.default_rng(7)
        for df, dtype in ((DF.Int8, torch.int8), (DF.Int32, torch.int32)):  # the two integer formats the tensor glue produces
            print("[case] integer queue", df, flush=True)
            q = api.create_queue(f"ints_{df}", df, (2, 64, 96), num_slots=2)
            x = torch.from_numpy(random_ints(rng, (1, 2, 64, 96), {torch.int8: np.int8, torch.int32: np.int32, torch.uint8: np.uint8, torch.int16: np.int16}[dtype]))
            assert B.push_input(q, T.pytorch_tensor_to_tensor_desc(x, df=df), True, 1, -1) == OK, B.last_error()
            out = B.PytorchTensorDesc()
            assert B.get_output(q, out, True, 1, -1) == OK, B.last_error()
            assert out.format == df
            got = T.tensor_desc_to_pytorch_tensor(out).clone()
            assert B.free_tensor(out) == OK and B.pop_output(q, True, 1) == OK
            assert got.dtype == dtype and torch.equal(got, x)
            # a float tensor is refused by an integer queue, and an integer tensor by a float queue
            assert B.push_input(q, T.pytorch_tensor_to_tensor_desc(torch.zeros(1, 2, 64, 96)), True, 1, -1) == ERR
            assert "an integer format goes with queues of the same format" in B.last_error()
    finally:
        api.shutdown()
