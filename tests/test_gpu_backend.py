"""GPU tests of the host boundary: descriptors in, queues in HBM, descriptors out, with the
reference's names and status-code behaviour, checked against the CPU oracle."""
import ctypes
import os
import sys
import threading

import numpy as np
import pytest
import torch

import oracle as O
import tt_buda_amd as ttb
from tt_buda_amd import tensor as T
from tt_buda_amd._C import DataFormat as DF
from tt_buda_amd._C import backend_api as B
from tt_buda_amd.backend import BackendAPI

pytestmark = pytest.mark.gpu
OK, ERR, TIMEOUT = B.BackendStatusCode.Success, B.BackendStatusCode.RuntimeError, B.BackendStatusCode.TimeoutError
ORACLE_FMT = {DF.Bfp8_b: O.Bfp8_b, DF.Bfp4_b: O.Bfp4_b, DF.Bfp2_b: O.Bfp2_b, DF.Float16_b: O.Float16_b, DF.Float32: O.Float32}


def say(*a):
    print("[case]", *a, flush=True)
    sys.stdout.flush()


@pytest.fixture(scope="module")
def api():
    a = BackendAPI(0)
    yield a
    a.shutdown()


def host_bytes(ptr, n):
    return np.ctypeslib.as_array((ctypes.c_uint8 * n).from_address(ptr)).copy()


def bf16_bits(t):
    return t.contiguous().view(torch.int16).numpy().view(np.uint16).reshape(-1)


def same(a, b):
    """Bit-equality of two arrays, flattened; a short message instead of a dump on mismatch."""
    a, b = np.asarray(a).reshape(-1), np.asarray(b).reshape(-1)
    if a.shape != b.shape:
        print(f"size mismatch {a.shape} vs {b.shape}")
        return False
    bad = np.flatnonzero(a != b)
    if bad.size:
        print(f"{bad.size} mismatches, first at {bad[:5]}: {a[bad[:5]]} vs {b[bad[:5]]}")
    return bad.size == 0


@pytest.mark.parametrize("fmt", [DF.Bfp8_b, DF.Bfp4_b, DF.Bfp2_b, DF.Float16_b])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_tilize_tensor_matches_oracle(api, fmt, dtype):
    say("tilize_tensor", fmt, dtype)
    torch.manual_seed(1)
    x = (torch.randn(2, 3, 64, 96) * 3).to(dtype)
    q = B.DramIODesc()
    q.bufq_target_format = fmt
    desc = B.tilize_tensor(q, T.pytorch_tensor_to_tensor_desc(x))
    src = x.numpy() if dtype == torch.float32 else bf16_bits(x).reshape(tuple(x.shape))
    want = O.tilize_pack(src, ORACLE_FMT[fmt])
    assert desc.format == fmt and desc.num_buffers == 1 and desc.buf_size_bytes == want.size
    assert same(host_bytes(desc.ptr, want.size), want)
    assert B.free_tensor(desc) == OK and desc.ptr == 0
    with pytest.raises(RuntimeError):  # rows not tile aligned: the caller must pad first
        B.tilize_tensor(q, T.pytorch_tensor_to_tensor_desc(torch.zeros(1, 1, 33, 32)))
    with pytest.raises(RuntimeError):  # fp16 sources belong to the 5-bit-exponent formats
        B.tilize_tensor(q, T.pytorch_tensor_to_tensor_desc(torch.zeros(1, 1, 32, 32).half()))


def test_push_get_pop_round_trip_and_ring_wrap(api):
    say("push/get/pop")
    q = api.create_queue("act_bfp8", DF.Bfp8_b, (2, 64, 96), num_slots=3, input_count=2)
    assert (q.name, q.data_format, q.t, q.mblock_m, q.mblock_n, q.input_count) == ("act_bfp8", DF.Bfp8_b, 2, 2, 3, 2)
    assert B.translate_addresses(q) == OK
    torch.manual_seed(2)
    # empty queue: TimeoutError, not a crash (the reference retries this status: backend.py:346-371)
    assert B.get_output(q, B.PytorchTensorDesc(), True, 1, -1) == TIMEOUT
    rounds = [torch.randn(2, 2, 64, 96), torch.randn(1, 2, 64, 96), torch.randn(2, 2, 64, 96).bfloat16().float()]
    # two entries at once, read both back (pop_one False -> input_count entries)
    assert B.push_input(q, T.pytorch_tensor_to_tensor_desc(rounds[0]), False, 1, -1) == OK
    out = B.PytorchTensorDesc()
    assert B.get_output(q, out, False, 1, -1) == OK
    assert (out.shape, out.format, out.itemsize, out.dim) == ([2, 2, 64, 96], DF.Float16_b, 2, 4)
    got = T.tensor_desc_to_pytorch_tensor(out).clone()
    want = O.unpack_untilize(O.tilize_pack(rounds[0].numpy(), O.Bfp8_b), O.Bfp8_b, (2, 2, 64, 96), O.Float16_b)
    assert same(bf16_bits(got), want.reshape(-1))
    assert B.free_tensor(out) == OK
    assert B.pop_output(q, False, 1) == OK
    # one entry, then two more: the second push wraps around the 3-slot ring
    assert B.push_input(q, T.pytorch_tensor_to_tensor_desc(rounds[1]), True, 1, -1) == OK
    assert B.push_input(q, T.pytorch_tensor_to_tensor_desc(rounds[2]), False, 1, -1) == OK
    # full: a fourth entry times out
    assert B.push_input(q, T.pytorch_tensor_to_tensor_desc(rounds[1]), True, 1, -1) == TIMEOUT
    assert "full" in B.last_error()
    out = B.PytorchTensorDesc()
    out.format = DF.Float32  # ask for fp32 floats
    assert B.get_output(q, out, True, 1, -1) == OK
    got = T.tensor_desc_to_pytorch_tensor(out).clone()
    want = O.unpack_untilize(O.tilize_pack(rounds[1].numpy(), O.Bfp8_b), O.Bfp8_b, (1, 2, 64, 96), O.Float32)
    assert same(got.numpy().view(np.uint32), want.view(np.uint32))
    B.free_tensor(out)
    assert B.pop_output(q, True, 1) == OK
    out = B.PytorchTensorDesc()
    out.format = DF.Float32
    assert B.get_output(q, out, False, 1, -1) == OK  # the two wrapped entries, in order
    got = T.tensor_desc_to_pytorch_tensor(out).clone()
    want = O.unpack_untilize(O.tilize_pack(rounds[2].numpy(), O.Bfp8_b), O.Bfp8_b, (2, 2, 64, 96), O.Float32)
    assert same(got.numpy().view(np.uint32), want.view(np.uint32))
    B.free_tensor(out)
    assert B.pop_output(q, False, 1) == OK
    assert B.pop_output(q, True, 1) == TIMEOUT  # nothing left
    # shape mismatch and push_one with two entries are RuntimeErrors
    assert B.push_input(q, T.pytorch_tensor_to_tensor_desc(torch.zeros(1, 2, 64, 64)), True, 1, -1) == ERR
    assert B.push_input(q, T.pytorch_tensor_to_tensor_desc(torch.zeros(2, 2, 64, 96)), True, 1, -1) == ERR


def test_parameter_ram_and_pretilized_reload(api, tmp_path):
    """Weights: push to a RandomAccess queue at ram pointer 0 (backend.py:486-493), or tilize once,
    binarize, debinarize into a fresh descriptor and push the tilized bytes (tti/archive.py:52-147)."""
    say("ram + tbin")
    q = api.create_queue("w_bfp4", DF.Bfp4_b, (1, 128, 64), num_slots=1, io_type=B.IOType.RandomAccess)
    torch.manual_seed(3)
    w = torch.randn(1, 1, 128, 64) * 0.02
    assert B.push_input(q, T.pytorch_tensor_to_tensor_desc(w), True, 1, 0) == OK
    want_packed = O.tilize_pack(w.numpy(), O.Bfp4_b)
    want = O.unpack_untilize(want_packed, O.Bfp4_b, (1, 1, 128, 64), O.Float16_b)
    out = B.PytorchTensorDesc()
    assert B.get_output(q, out, True, 1, 0) == OK
    assert same(bf16_bits(T.tensor_desc_to_pytorch_tensor(out)), want.reshape(-1))
    B.free_tensor(out)
    assert B.pop_output(q, True, 1) == OK  # a RAM has nothing to pop

    tilized = B.tilize_tensor(q, T.pytorch_tensor_to_tensor_desc(w))
    path = str(tmp_path / "w.tbin")
    B.binarize_tensor(tilized, path)
    assert os.path.getsize(path) == want_packed.size
    assert same(np.fromfile(path, dtype=np.uint8), want_packed)
    meta = (tilized.num_buffers, tilized.buf_size_bytes, tilized.format)
    B.free_tensor(tilized)
    reloaded = B.TilizedTensorDesc()
    reloaded.num_buffers, reloaded.buf_size_bytes, reloaded.format = meta
    B.debinarize_tensor(reloaded, path)
    q2 = api.create_queue("w_bfp4_reload", DF.Bfp4_b, (1, 128, 64), num_slots=1, io_type=B.IOType.RandomAccess)
    assert B.push_input(q2, reloaded, 1, 0) == OK
    B.free_tensor(reloaded)
    out = B.PytorchTensorDesc()
    assert B.get_output(q2, out, True, 1, 0) == OK
    assert same(bf16_bits(T.tensor_desc_to_pytorch_tensor(out)), want.reshape(-1))
    B.free_tensor(out)
    # row-major descriptors binarize too
    d = T.pytorch_tensor_to_tensor_desc(w)
    B.binarize_tensor(d, str(tmp_path / "w.bin"))
    assert same(np.fromfile(str(tmp_path / "w.bin"), dtype=np.float32), w.numpy().reshape(-1))
    with pytest.raises(RuntimeError):
        B.debinarize_tensor(B.TilizedTensorDesc(), path)  # size mismatch


def test_device_resident_and_strided_sources(api):
    say("device + strided")
    q = api.create_queue("dev_src", DF.Bfp8_b, (1, 32, 64), num_slots=2)
    torch.manual_seed(4)
    base = torch.randn(1, 1, 32, 128)
    view = base[:, :, :, ::2]  # column stride of two elements
    desc = B.PytorchTensorDesc(view, 4, DF.Float32, 4, list(view.shape), [s * 4 for s in view.stride()])
    assert B.push_input(q, desc, True, 1, -1) == OK
    dev = base.cuda()[:, :, :, ::2]
    ddesc = B.PytorchTensorDesc(dev, 4, DF.Float32, 4, list(dev.shape), [s * 4 for s in dev.stride()])
    assert B.push_input(q, ddesc, True, 1, -1) == OK
    want = O.unpack_untilize(O.tilize_pack(view.numpy(), O.Bfp8_b), O.Bfp8_b, (1, 1, 32, 64), O.Float16_b)
    for _ in range(2):
        out = B.PytorchTensorDesc()
        assert B.get_output(q, out, True, 1, -1) == OK
        assert same(bf16_bits(T.tensor_desc_to_pytorch_tensor(out)), want.reshape(-1))
        B.free_tensor(out)
        assert B.pop_output(q, True, 1) == OK


def test_concurrent_pushers_and_reader(api):
    """The boundary runs without the GIL from several threads (backend_api.cpp:688-701)."""
    say("threads")
    n_threads, per_thread = 4, 6
    queues = [api.create_queue(f"thr{i}", DF.Bfp8_b, (1, 64, 64), num_slots=2) for i in range(n_threads)]
    data = [[torch.randn(1, 1, 64, 64, generator=torch.Generator().manual_seed(100 * i + j)) for j in range(per_thread)]
            for i in range(n_threads)]
    errors = []

    def pusher(i):
        for j in range(per_thread):
            st = TIMEOUT
            for _ in range(20):
                st = B.push_input(queues[i], T.pytorch_tensor_to_tensor_desc(data[i][j]), True, 1, -1)
                if st != TIMEOUT:
                    break
            if st != OK:
                errors.append(("push", i, j, st))

    def reader(i):
        for j in range(per_thread):
            out = B.PytorchTensorDesc()
            out.format = DF.Float32
            st = TIMEOUT
            for _ in range(20):
                st = B.get_output(queues[i], out, True, 1, -1)
                if st != TIMEOUT:
                    break
            if st != OK:
                errors.append(("get", i, j, st))
                return
            got = T.tensor_desc_to_pytorch_tensor(out).clone()
            B.free_tensor(out)
            B.pop_output(queues[i], True, 1)
            want = O.unpack_untilize(O.tilize_pack(data[i][j].numpy(), O.Bfp8_b), O.Bfp8_b, (1, 1, 64, 64), O.Float32)
            if not same(got.numpy().view(np.uint32), want.view(np.uint32)):
                errors.append(("value", i, j))

    threads = [threading.Thread(target=f, args=(i,)) for i in range(n_threads) for f in (pusher, reader)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(60)
    assert not errors, errors
    assert not any(t.is_alive() for t in threads)


def test_python_push_to_queues_and_read_queues_pad_and_narrow(api):
    say("BackendAPI loops")
    q = api.create_queue("py_in", DF.Bfp8_b, (3, 64, 96), num_slots=2)
    torch.manual_seed(5)
    x = torch.randn(1, 3, 50, 70)  # not tile aligned: padded on push, narrowed on read
    api.push_to_queues([q], [x], single_input=True)
    (y,) = api.read_queues([q], [x.shape], single_output=True, fp32_output=True)
    api.pop_queues([q], single_output=True)
    padded = T.pad_pytorch_tensor_to_buda(x, [])
    want = O.unpack_untilize(O.tilize_pack(padded.numpy(), O.Bfp8_b), O.Bfp8_b, tuple(padded.shape), O.Float32)
    assert y.shape == x.shape and same(y.numpy().view(np.uint32), want[:, :, :50, :70].view(np.uint32))
    with pytest.raises(RuntimeError, match="Timeout while reading"):
        api.read_queues([q], [x.shape], single_output=True, shutdown_event=threading.Event())


def hstack_reference(x, f):
    """pybuda/pybuda/op/eval/buda/tm.py:114-122"""
    w, z, r, c = x.shape
    return x.reshape(-1, z // f, f, r, c).permute(0, 1, 3, 2, 4).reshape(w, z // f, r, c * f)


def vstack_reference(x, f):
    """pybuda/pybuda/op/eval/buda/tm.py:131-137"""
    w, z, r, c = x.shape
    return x.reshape(w, z // f, r * f, c)


@pytest.mark.parametrize("h,v,row_major", [(2, 1, 1), (4, 1, 1), (1, 2, 1), (1, 4, 0), (2, 2, 1), (2, 2, 0)])
def test_get_output_applies_hstack_and_vstack(api, h, v, row_major):
    """The output host transforms of the queue descriptor (backend.py:294-302): single factors against
    the reference's own reshape/permute definitions; both at once as their composition, hstack first
    when stack_row_major is set (the combined order is this build's reading, the reference pins only
    the single transforms)."""
    say("output host tm", h, v, row_major)
    name = "out_tm_%d_%d_%d" % (h, v, row_major)
    q = api.create_queue(name, DF.Float16_b, (4, 32, 64), num_slots=4, input_count=3)
    torch.manual_seed(10 * h + v)
    x = torch.randn(3, 4, 32, 64).bfloat16()
    assert B.push_input(q, T.pytorch_tensor_to_tensor_desc(x), False, 1, -1) == OK
    q.hstack_factor, q.vstack_factor, q.stack_row_major = h, v, row_major
    out = B.PytorchTensorDesc()
    assert B.get_output(q, out, False, 1, -1) == OK, B.last_error()
    got = T.tensor_desc_to_pytorch_tensor(out).clone()
    B.free_tensor(out)
    if row_major or v == 1:
        want = vstack_reference(hstack_reference(x, h) if h > 1 else x, v) if v > 1 else hstack_reference(x, h)
    else:
        want = hstack_reference(vstack_reference(x, v), h) if h > 1 else vstack_reference(x, v)
    assert list(got.shape) == [3, 4 // (h * v), 32 * v, 64 * h]
    assert torch.equal(got, want)
    q.hstack_factor = 3  # 4 slices cannot be stacked by 3
    q.vstack_factor = 1
    assert B.get_output(q, B.PytorchTensorDesc(), False, 1, -1) == B.BackendStatusCode.RuntimeError


def test_half_family_queue_round_trip(api):
    """Queues with a 5-bit exponent take Float16 tensors and read back as Float16
    (pybuda/pybuda/device_connector.py:188-192, pybuda/pybuda/tensor.py:602-618)."""
    say("half family queue")
    q = api.create_queue("act_bfp8a", DF.Bfp8, (1, 32, 64), num_slots=2, input_count=2)
    torch.manual_seed(21)
    x = torch.randn(2, 1, 32, 64).half()
    assert B.push_input(q, T.pytorch_tensor_to_tensor_desc(x), False, 1, -1) == OK, B.last_error()
    out = B.PytorchTensorDesc()
    assert B.get_output(q, out, False, 1, -1) == OK, B.last_error()
    assert (out.shape, out.format, out.itemsize) == ([2, 1, 32, 64], DF.Float16, 2)
    got = T.tensor_desc_to_pytorch_tensor(out).clone()
    B.free_tensor(out)
    want = O.unpack_untilize(O.tilize_pack(x.numpy(), O.Bfp8), O.Bfp8, (2, 1, 32, 64), O.Float16)
    assert got.dtype == torch.float16 and np.array_equal(got.numpy().view(np.uint16), want.view(np.uint16))
    # a bf16 or fp32 tensor does not go into such a queue, and a half tensor not into a Bfp8_b queue
    assert B.push_input(q, T.pytorch_tensor_to_tensor_desc(x.float()), False, 1, -1) == ERR
    qb = api.create_queue("act_bfp8b_for_half", DF.Bfp8_b, (1, 32, 64), num_slots=2, input_count=2)
    assert B.push_input(qb, T.pytorch_tensor_to_tensor_desc(x), False, 1, -1) == ERR


def test_ffn_through_queues(api):
    """Bfp8_b weights pushed as parameters, activations through Float16_b queues, two matmul ops."""
    say("ffn program")
    M, H, I = 128, 256, 512
    torch.manual_seed(6)
    x = torch.randn(1, 1, M, H).bfloat16()
    w1, w2 = torch.randn(1, 1, H, I) * 0.02, torch.randn(1, 1, I, H) * 0.02
    b1 = T.pad_pytorch_tensor_to_buda((torch.randn(1, I) * 0.02).bfloat16(), [-2])
    b2 = T.pad_pytorch_tensor_to_buda((torch.randn(1, H) * 0.02).bfloat16(), [-2])
    ram = B.IOType.RandomAccess
    qx = api.create_queue("ffn_x", DF.Float16_b, (1, M, H))
    qh = api.create_queue("ffn_h", DF.Float16_b, (1, M, I))
    qy = api.create_queue("ffn_y", DF.Float16_b, (1, M, H))
    qw1 = api.create_queue("ffn_w1", DF.Bfp8_b, (1, H, I), 1, ram)
    qw2 = api.create_queue("ffn_w2", DF.Bfp8_b, (1, I, H), 1, ram)
    qb1 = api.create_queue("ffn_b1", DF.Float16_b, (1, 32, I), 1, ram)
    qb2 = api.create_queue("ffn_b2", DF.Float16_b, (1, 32, H), 1, ram)
    for q, t in ((qw1, w1), (qw2, w2), (qb1, b1), (qb2, b2)):
        api.push_input(q, T.pytorch_tensor_to_tensor_desc(t), True, 1, 0)
    api.push_to_queues([qx], [x], single_input=True)
    assert api.be_api.run_matmul("ffn_x", "ffn_w1", "ffn_b1", "ffn_h", gelu=True) == OK
    assert api.be_api.run_matmul("ffn_h", "ffn_w2", "ffn_b2", "ffn_y", gelu=False) == OK
    (y,) = api.read_queues([qy], [(1, 1, M, H)], single_output=True)
    api.pop_queues([qy], single_output=True)
    assert B.get_output(qx, B.PytorchTensorDesc(), True, 1, -1) == TIMEOUT  # the op consumed its input
    dq = lambda w, K, N: torch.from_numpy(O.dequant_weight(O.tilize_pack(w.numpy(), O.Bfp8_b), K, N))
    h = torch.nn.functional.gelu(x[0, 0].float() @ dq(w1, H, I) + b1[0, 0, 0].float()).bfloat16()
    want = (h.float() @ dq(w2, I, H) + b2[0, 0, 0].float()).bfloat16()
    err = float((y[0, 0].double() - want.double()).norm() / want.double().norm())
    assert err < 1e-3, err
    # the tanh form of the activation, and a mode the reference does not know either
    api.push_to_queues([qx], [x], single_input=True)
    assert api.be_api.run_matmul("ffn_x", "ffn_w1", "ffn_b1", "ffn_h", gelu=True, approximate="tanh") == OK
    (ht,) = api.read_queues([qh], [(1, 1, M, I)], single_output=True)
    api.pop_queues([qh], single_output=True)
    want_t = torch.nn.functional.gelu(x[0, 0].float() @ dq(w1, H, I) + b1[0, 0, 0].float(), approximate="tanh").bfloat16()
    assert float((ht[0, 0].double() - want_t.double()).norm() / want_t.double().norm()) < 1e-3
    assert not torch.equal(ht[0, 0].cpu(), h)
    assert api.be_api.run_matmul("ffn_x", "ffn_w1", "ffn_b1", "ffn_h", gelu=True, approximate="quick") == ERR
    assert "does not support" in B.last_error()
    assert api.be_api.run_matmul("ffn_x", "ffn_w1", "", "ffn_h", False, 1) == TIMEOUT  # no input entry
    assert api.be_api.run_matmul("ffn_x", "nope", "", "ffn_h") == ERR


def test_op_module_matmul_and_ffn():
    say("op module")
    from tt_buda_amd import op

    torch.manual_seed(7)
    x = torch.randn(2, 64, 128).bfloat16()
    w1, w2 = op.BfpWeight(torch.randn(128, 256) * 0.02), op.BfpWeight(torch.randn(256, 128) * 0.02)
    b1 = T.pad_pytorch_tensor_to_buda((torch.randn(1, 256) * 0.02).bfloat16(), [-2])  # 4-D tile-padded bias
    b2 = (torch.randn(128) * 0.02).bfloat16()
    y = op.ffn(x, w1, b1, w2, b2, out_dtype=torch.float32).cpu()
    h = torch.nn.functional.gelu(x.float() @ w1.dequantize().cpu() + b1[0, 0, 0].float()).bfloat16()
    want = h.float() @ w2.dequantize().cpu() + b2.float()
    assert y.shape == (2, 64, 128)
    assert float((y - want).norm() / want.norm()) < 1e-3


@pytest.mark.parametrize("bias_scale", [None, 0.02, 0.03], ids=["nobias", "bias", "bias_inexact_sum"])
def test_op_module_weight_stack_and_accumulate(bias_scale):
    """The golden evaluation of a matmul over stacks (pybuda/pybuda/op/eval/buda/matmul.py:244-249,306-307):
    torch.matmul pairs x[z] with w[z], adds row 0 of the bias, and `accumulate` sums the results over z with keepdim."""
    say("op module stack", bias_scale)
    from tt_buda_amd import op

    torch.manual_seed(11)
    Z, M, K, N = 3, 64, 96, 160
    x = torch.randn(1, Z, M, K).bfloat16()
    w = op.BfpWeight(torch.randn(1, Z, K, N) * 0.05)
    assert w.Z == Z and w.dequantize().shape == (Z, K, N)
    wd = w.dequantize().cpu()
    if bias_scale is None:
        bias = None
    elif bias_scale == 0.02:  # multiples of 1/64 up to 8/64: Z times the bias is a bf16 value
        bias = (torch.randint(-8, 9, (1, 1, 32, N)).float() / 64).bfloat16()
    else:  # Z times the bias needs more than eight significant bits: it rides in the GEMM's epilogue as an fp32 bias
        bias = (torch.randn(1, 1, 32, N) * bias_scale).bfloat16()
        assert not torch.equal((bias.float() * Z).bfloat16().float(), bias.float() * Z)
    golden = torch.matmul(x.float(), wd)
    if bias is not None:
        golden = golden + bias[:, :, 0:1, :].float()
    y = op.matmul(x, w, bias, out_dtype=torch.float32).cpu()
    assert y.shape == (1, Z, M, N) and float((y - golden).norm() / golden.norm()) < 1e-5
    for z in range(Z):  # every member is the plain product with that matrix
        one = op.matmul(x[0, z], op.BfpWeight(wd[z]), bias, out_dtype=torch.float32).cpu()
        assert torch.equal(one, y[0, z])
    acc = torch.sum(golden, dim=-3, keepdim=True)
    got = op.matmul(x, w, bias, out_dtype=torch.float32, accumulate=True).cpu()
    assert got.shape == (1, 1, M, N) and float((got - acc).norm() / acc.norm()) < 1e-5
    got16 = op.matmul(x, w, bias, accumulate=True).cpu()
    assert float((got16.float() - acc.bfloat16().float()).norm() / acc.norm()) < 1e-3
    gact = op.matmul(x, w, bias, gelu="tanh", out_dtype=torch.float32, accumulate=True).cpu()
    want = torch.nn.functional.gelu(acc, approximate="tanh")
    assert float((gact - want).norm() / want.norm()) < 1e-5


@pytest.mark.parametrize("grid,ublock,order,header", [((2, 2), (2, 1), "c", True), ((1, 3), (1, 2), "r", False),
                                                       ((2, 1), (1, 3), "c", False)])
def test_queue_geometry_push_get_tilize(api, grid, ublock, order, header):
    """A queue cut over a grid of buffers with micro blocks: what comes back is what a plain queue gives, and the
    tilized bytes are the oracle's tiles moved to the slots TileLayout::map names (balancer/types.cpp:629-648)."""
    name = "geo_%d%d_%d%d_%s%d" % (grid + ublock + (order, header))
    say("geometry", name)
    t, R, C = 2, 128, 192
    q = api.create_queue(name, DF.Bfp8_b, (t, R, C), num_slots=3, input_count=2, grid=grid, ublock=ublock, ublock_order=order,
                         tile_header=header)
    assert (q.bufq_grid_dim_r, q.bufq_grid_dim_c, q.ublock_rt, q.ublock_ct, q.ublock_order, q.tile_header) == (
        grid[0], grid[1], ublock[0], ublock[1], order, header)
    assert (q.mblock_m * grid[0] * ublock[0], q.mblock_n * grid[1] * ublock[1]) == (R // 32, C // 32)
    lay = O.QueueLayout(grid[0], grid[1], q.mblock_m, q.mblock_n, ublock[0], ublock[1], int(order == "c"), int(header))
    assert q.bufq_entry_size == lay.buffer_bytes(O.Bfp8_b, 1, t) and len(q.bufq_start_addr_channel) == grid[0] * grid[1]
    assert q.bufq_entry_size + 32 == B.get_io_size_in_bytes(DF.Bfp8_b, False, ublock[1], ublock[0], q.mblock_m, q.mblock_n, t, 1) or not header
    torch.manual_seed(12)
    a, b = torch.randn(2, t, R, C), torch.randn(2, t, R, C) * 8
    flat = lambda x: O.unpack_untilize(O.tilize_pack(x.numpy(), O.Bfp8_b), O.Bfp8_b, tuple(x.shape), O.Float32)

    def read(n_entries):
        out = B.PytorchTensorDesc()
        out.format = DF.Float32
        assert B.get_output(q, out, n_entries == 1, 1, -1) == OK
        got = T.tensor_desc_to_pytorch_tensor(out).clone()
        B.free_tensor(out)
        assert B.pop_output(q, n_entries == 1, 1) == OK
        return got

    assert B.push_input(q, T.pytorch_tensor_to_tensor_desc(a), False, 1, -1) == OK
    assert same(read(2).numpy().view(np.uint32), flat(a).view(np.uint32))
    # slots 2, 0 next: the ring wraps inside every buffer
    assert B.push_input(q, T.pytorch_tensor_to_tensor_desc(b), False, 1, -1) == OK
    assert same(read(1).numpy().view(np.uint32), flat(b[:1]).view(np.uint32))
    assert same(read(1).numpy().view(np.uint32), flat(b[1:]).view(np.uint32))

    # tilize once on the host side, push the tilized buffers: same entries
    tz = B.tilize_tensor(q, T.pytorch_tensor_to_tensor_desc(a))
    per = lay.buffer_bytes(O.Bfp8_b, 2, t)
    assert (tz.num_buffers, tz.buf_size_bytes) == (grid[0] * grid[1], per)
    want = O.tiles_to_queue(O.tilize_pack(a.numpy(), O.Bfp8_b), O.Bfp8_b, (2, t, R, C), lay)
    assert same(host_bytes(tz.ptr, per * tz.num_buffers), want)
    assert B.push_input(q, tz, 1, -1) == OK
    B.free_tensor(tz)
    assert same(read(2).numpy().view(np.uint32), flat(a).view(np.uint32))
    with pytest.raises(RuntimeError):  # the descriptor's entry is [2, 128, 192]
        B.tilize_tensor(q, T.pytorch_tensor_to_tensor_desc(torch.zeros(1, 1, R, C)))
    # hstack on the way out reads runs of z slices out of every buffer
    assert B.push_input(q, T.pytorch_tensor_to_tensor_desc(a[:1]), True, 1, -1) == OK
    q.hstack_factor = 2
    got = read(1)
    q.hstack_factor = 1
    fa = torch.from_numpy(flat(a[:1]))
    assert got.shape == (1, 1, R, 2 * C) and torch.equal(got[0, 0], torch.cat([fa[0, 0], fa[0, 1]], dim=1))


def test_matmul_over_queues_with_geometry(api):
    """Activation and result queues may use any geometry; the weight queue must hold row-major tiles."""
    say("matmul geometry")
    M, K, N = 64, 128, 192
    torch.manual_seed(13)
    x, w = torch.randn(1, 1, M, K).bfloat16(), torch.randn(1, 1, K, N) * 0.05
    ram = B.IOType.RandomAccess
    qx = api.create_queue("mg_x", DF.Float16_b, (1, M, K), grid=(2, 2), ublock=(1, 2), ublock_order="c", tile_header=True)
    qy = api.create_queue("mg_y", DF.Float16_b, (1, M, N), grid=(1, 3), ublock=(2, 1), ublock_order="c")
    qw = api.create_queue("mg_w", DF.Bfp8_b, (1, K, N), 1, ram, ublock=(1, 3))  # r order, one-tile-high micro blocks
    qbad = api.create_queue("mg_w_bad", DF.Bfp8_b, (1, K, N), 1, ram, ublock=(2, 3))
    api.push_input(qw, T.pytorch_tensor_to_tensor_desc(w), True, 1, 0)
    api.push_input(qbad, T.pytorch_tensor_to_tensor_desc(w), True, 1, 0)
    api.push_to_queues([qx], [x], single_input=True)
    assert api.be_api.run_matmul("mg_x", "mg_w_bad", "", "mg_y") == ERR and "row-major" in B.last_error()
    assert api.be_api.run_matmul("mg_x", "mg_w", "", "mg_y") == OK
    (y,) = api.read_queues([qy], [(1, 1, M, N)], single_output=True)
    api.pop_queues([qy], single_output=True)
    want = (x[0, 0].float() @ torch.from_numpy(O.dequant_weight(O.tilize_pack(w.numpy(), O.Bfp8_b), K, N))).bfloat16()
    err = float((y[0, 0].double() - want.double()).norm() / want.double().norm())
    assert err < 1e-3, err


@pytest.mark.parametrize("out_df", [DF.Float16_b, DF.Bfp8_b], ids=["bfloat", "bfp8b"])
@pytest.mark.parametrize("input_df", [DF.Float16_b, DF.Bfp8_b, DF.Bfp4_b], ids=["bfloat", "bfp8b", "bfp4b"])
def test_data_formats_like_the_reference(api, input_df, out_df):
    """The reference's own data-format test (pybuda/test/data_formats/test_df.py:103-138): a 64x64 matmul with inputs and
    parameters in the block formats (it leaves results in the default format; the matmul here takes Bfp8_b weights
    only), accepted by its rule (pybuda/pybuda/op/eval/common.py:154-299):
    allclose with atol = 0.1 max|golden|, or a Pearson correlation of at least 0.99 with the fp32 golden result."""
    say("data formats", input_df, out_df)
    name = f"df_{int(input_df)}_{int(out_df)}"
    torch.manual_seed(int(input_df) * 16 + int(out_df))
    act, w = torch.rand(1, 1, 64, 64), torch.rand(1, 1, 64, 64)  # the reference draws uniform inputs
    qa = api.create_queue(name + "_a", input_df, (1, 64, 64))
    qw = api.create_queue(name + "_w", DF.Bfp8_b, (1, 64, 64), 1, B.IOType.RandomAccess)
    qo = api.create_queue(name + "_o", out_df, (1, 64, 64))
    api.push_input(qw, T.pytorch_tensor_to_tensor_desc(w), True, 1, 0)
    api.push_to_queues([qa], [act], single_input=True)
    assert api.be_api.run_matmul(name + "_a", name + "_w", "", name + "_o") == OK
    (y,) = api.read_queues([qo], [(1, 1, 64, 64)], single_output=True)
    api.pop_queues([qo], single_output=True)
    golden, got = (act[0, 0] @ w[0, 0]), y[0, 0].float()
    close = torch.allclose(golden, got, rtol=0.0, atol=0.1 * float(golden.abs().max()))
    pcc = float(np.min(np.corrcoef(golden.numpy().reshape(-1), got.numpy().reshape(-1))))
    assert close or pcc >= 0.99, (close, pcc)
    assert pcc >= 0.99, pcc  # in fact both hold for every combination


def test_matmul_with_many_rows_uses_the_panel_path(api):
    """4096 rows x 3072 columns qualifies for the two-pass GEMM (weight converted once into scratch memory): same result."""
    say("matmul panel")
    M, K, N = 4096, 64, 3072
    assert ttb.capi.gemm_workspace_bytes(M, N, K) == 2 * K * N
    torch.manual_seed(14)
    x, w = torch.randn(1, 1, M, K).bfloat16(), torch.randn(1, 1, K, N) * 0.05
    qx = api.create_queue("mp_x", DF.Float16_b, (1, M, K))
    qy = api.create_queue("mp_y", DF.Float16_b, (1, M, N))
    qw = api.create_queue("mp_w", DF.Bfp8_b, (1, K, N), 1, B.IOType.RandomAccess)
    api.push_input(qw, T.pytorch_tensor_to_tensor_desc(w), True, 1, 0)
    api.push_to_queues([qx], [x], single_input=True)
    assert api.be_api.run_matmul("mp_x", "mp_w", "", "mp_y") == OK
    (y,) = api.read_queues([qy], [(1, 1, M, N)], single_output=True)
    api.pop_queues([qy], single_output=True)
    wp = ttb.capi.tilize_pack(w.cuda(), ttb.capi.DataFormatCode.Bfp8_b)
    fused = ttb.capi.gemm_bfp8b(x[0, 0].cuda(), wp, N).cpu()
    assert torch.equal(y[0, 0], fused)
