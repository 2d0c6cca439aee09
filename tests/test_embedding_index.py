"""Embedding indices: integer tensors in RawUInt32 queues, and the EmbeddingIndex runtime transform.

The reference states the transform as a chain of torch pads, views and one transpose (pybuda/pybuda/tensor.py:1382-1408).
The glue in tt_buda_amd/tensor.py restates that chain; the oracle states where each element lands by index arithmetic;
the two are held to each other and to a case placed by hand.  RawUInt32 tiles are a pure permutation of 32-bit elements.
"""
import numpy as np
import pytest
import torch

import oracle as O
from tt_buda_amd import tensor as T
from tt_buda_amd._C import DataFormat as DF
from tt_buda_amd._C import backend_api as B


def queue_desc(q_rt, cols_tiles):
    q = B.DramIODesc()
    q.bufq_target_format = DF.RawUInt32
    q.mblock_m, q.mblock_n, q.t = q_rt, cols_tiles, 1
    return q


@pytest.mark.parametrize("n,valid,q_rt", [(32, 32, 1), (100, 100, 1), (128, 70, 1), (2048, 2048, 2), (4096, 4000, 4), (33, 33, 1), (40, 50, 1), (40, 64, 1)])
def test_glue_and_oracle_agree(n, valid, q_rt):
    rng = np.random.default_rng(n + valid)
    idx = rng.integers(0, 50000, (2, n), dtype=np.int32)
    want = O.embedding_index(idx, valid, q_rt)
    q = queue_desc(q_rt, want.shape[3] // 32)
    got = T._embedding_index(torch.from_numpy(idx), (1, 1, valid), q)
    assert tuple(got.shape) == want.shape and got.dtype == torch.int32
    assert np.array_equal(got.numpy().view(np.uint32), want)
    one = T._embedding_index(torch.from_numpy(idx[0]), (valid,), q)  # a single vector
    assert np.array_equal(one.numpy().view(np.uint32), want[:1])


def test_by_hand():
    # 70 indices 1..70: padded to 96 with all-ones, three rows of 32, one tile row: row l sits in row l of the result
    idx = np.arange(1, 71, dtype=np.uint32)
    out = O.embedding_index(idx, 70, 1)
    assert out.shape == (1, 1, 32, 32)
    assert out[0, 0, 0].tolist() == list(range(1, 33)) and out[0, 0, 1].tolist() == list(range(33, 65))
    assert out[0, 0, 2, :6].tolist() == [65, 66, 67, 68, 69, 70] and (out[0, 0, 2, 6:] == 0xFFFFFFFF).all()
    assert not out[0, 0, 3:].any()
    # an original shape longer than the vector (40 indices, original length 50): the reference zero-pads to 64 first and
    # then overwrites positions 50.. with all-ones, so positions 40..49 stay zero
    idx = np.arange(1, 41, dtype=np.uint32)
    out = O.embedding_index(idx, 50, 1)
    assert out[0, 0, 1, :8].tolist() == list(range(33, 41)) and not out[0, 0, 1, 8:18].any() and (out[0, 0, 1, 18:] == 0xFFFFFFFF).all()
    got = T._embedding_index(torch.from_numpy(idx.astype(np.int32)), (50,), queue_desc(1, 1))
    assert np.array_equal(got.numpy().view(np.uint32), out)
    # 2048 indices over two tile rows: 32 rows of 32 each; element e of the second half goes to tile row 1
    idx = np.arange(2048, dtype=np.uint32)
    out = O.embedding_index(idx, 2048, 2)
    assert out.shape == (1, 1, 64, 32)
    assert out[0, 0, 5, 7] == 5 * 32 + 7 and out[0, 0, 32 + 5, 7] == 1024 + 5 * 32 + 7
    # 33 rows per tile row spill into a second column block: row 32 is row 0 of block 1
    idx = np.arange(33 * 32, dtype=np.uint32)
    out = O.embedding_index(idx, 33 * 32, 1)
    assert out.shape == (1, 1, 32, 64) and out[0, 0, 0, 32 + 3] == 32 * 32 + 3 and not out[0, 0, 1:, 32:].any()


def test_oracle_raw_tiles_are_a_permutation():
    x = np.random.default_rng(1).integers(0, 2 ** 32, (2, 1, 64, 96), dtype=np.uint32)
    t = O.tilize_pack(x, O.RawUInt32)
    assert t.size == x.size * 4
    assert np.array_equal(t, O.tilize_pack(x.view(np.float32), O.Float32))  # the same bytes as Float32 tiles of the same bits
    assert np.array_equal(O.unpack_untilize(t, O.RawUInt32, x.shape, O.RawUInt32), x)
    # raw pairs with raw only
    out = np.empty(x.size * 4, dtype=np.uint8)
    assert O.lib().oracle_tilize_pack(O._ptr(x), O.RawUInt32, *O._shape4(x), O.Bfp8_b, 0, O._ptr(out), 1) != 0


@pytest.mark.gpu
def test_gpu_raw_tiles_and_embedding_queue():
    from tt_buda_amd import capi
    from tt_buda_amd.backend import BackendAPI

    rng = np.random.default_rng(2)
    x = rng.integers(0, 2 ** 31, (2, 1, 64, 96), dtype=np.int32)
    xd = torch.from_numpy(x).to("cuda:0")
    print("[case] raw tiles", flush=True)
    t = capi.tilize_pack(xd, capi.DataFormatCode.RawUInt32)
    assert np.array_equal(t.cpu().numpy(), O.tilize_pack(x.view(np.uint32), O.RawUInt32))
    assert torch.equal(capi.unpack_untilize(t, capi.DataFormatCode.RawUInt32, x.shape, torch.int32), xd)
    with pytest.raises(capi.BackendError):
        capi.tilize_pack(xd, capi.DataFormatCode.Bfp8_b)
    with pytest.raises(capi.BackendError):
        capi.unpack_untilize(t, capi.DataFormatCode.RawUInt32, x.shape, torch.float32)
    lay = capi.QueueLayout(2, 1, 1, 3, 1, 1, 1, 1)
    olay = O.QueueLayout(2, 1, 1, 3, 1, 1, 1, 1)
    q = capi.tilize_pack_queue(xd, capi.DataFormatCode.RawUInt32, lay)
    assert np.array_equal(q.cpu().numpy(), O.tiles_to_queue(O.tilize_pack(x.view(np.uint32), O.RawUInt32), O.Float32, x.shape, olay))
    # through the host boundary: an embedding-index queue of two tile rows
    api = BackendAPI(0)
    try:
        print("[case] embedding queue", flush=True)
        idx = torch.from_numpy(rng.integers(0, 30000, (2, 4096), dtype=np.int32))
        qd = api.create_queue("emb_idx", DF.RawUInt32, (1, 64, 64), num_slots=2, input_count=2)
        laid = T._embedding_index(idx, (1, 1, 4000), qd)
        assert tuple(laid.shape) == (2, 1, 64, 64)
        assert B.push_input(qd, T.pytorch_tensor_to_tensor_desc(laid, df=DF.RawUInt32), False, 1, -1) == B.BackendStatusCode.Success
        out = B.PytorchTensorDesc()
        assert B.get_output(qd, out, False, 1, -1) == B.BackendStatusCode.Success
        assert out.format == DF.RawUInt32
        back = T.tensor_desc_to_pytorch_tensor(out).clone()
        B.free_tensor(out)
        assert torch.equal(back, laid)
        # a float tensor does not go into a raw queue
        assert B.push_input(qd, T.pytorch_tensor_to_tensor_desc(torch.zeros(1, 1, 64, 64)), True, 1, -1) == B.BackendStatusCode.RuntimeError
    finally:
        api.shutdown()
