"""The library's host-memory twins of the conversions (``ttbfp_*_cpu``): same datum rules as the kernels, compiled for the
host.  Held bit for bit against the oracle and the committed golden vectors here (no GPU needed), and against the device
entry points on the GPU.  No device entry point calls them: that is checked too."""
import os
import re

import numpy as np
import pytest
import torch

import oracle as O
from tt_buda_amd import capi

F = capi.DataFormatCode
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def heavy_tailed(rng, shape):
    x = rng.standard_normal(shape).astype(np.float32)
    x *= np.exp2(rng.integers(-20, 21, size=(shape[0], shape[1], shape[2], 1))).astype(np.float32)
    x[rng.random(shape) < 0.01] = 0.0
    x[rng.random(shape) < 0.001] = 1e4
    x[0, 0, 0, :8] = [0.0, -0.0, 1e-40, -1e-40, np.inf, -np.inf, 3.4e38, 1.2e-38]
    return x


@pytest.mark.parametrize("fmt", [F.Bfp8_b, F.Bfp4_b, F.Bfp2_b, F.Float16_b, F.Float32])
@pytest.mark.parametrize("rounding", [capi.ROUND_TRUNCATE, capi.ROUND_NEAREST])
@pytest.mark.parametrize("source", ["fp32", "bf16"])
def test_cpu_twin_pack_and_unpack_match_the_oracle(fmt, rounding, source):
    rng = np.random.default_rng(fmt * 7 + rounding)
    x = heavy_tailed(rng, (2, 2, 64, 96))
    t = torch.from_numpy(x)
    if source == "bf16":
        t = t.bfloat16()
        x = t.view(torch.int16).numpy().view(np.uint16)
    packed = capi.tilize_pack_cpu(t, fmt, rounding)
    want = O.tilize_pack(x, fmt, rounding)
    assert np.array_equal(packed.numpy(), want)
    for dt, ofmt in ((torch.float32, O.Float32), (torch.bfloat16, O.Float16_b)):
        if fmt == F.Float32 and dt != torch.float32:
            continue
        back = capi.unpack_untilize_cpu(packed, fmt, x.shape, dt)
        want_back = O.unpack_untilize(want, fmt, x.shape, ofmt)
        got = back.numpy() if dt == torch.float32 else back.view(torch.int16).numpy().view(np.uint16)
        assert np.array_equal(got.view(want_back.dtype), want_back)
    # any strides: a transposed view
    tt = t.transpose(2, 3).contiguous().transpose(2, 3)
    assert np.array_equal(capi.tilize_pack_cpu(tt, fmt, rounding).numpy(), want)


@pytest.mark.parametrize("fmt", [F.Bfp8, F.Bfp4, F.Bfp2, F.Float16])
def test_cpu_twin_half_family(fmt):
    rng = np.random.default_rng(fmt)
    x = (rng.standard_normal((1, 2, 64, 64)) * np.exp2(rng.integers(-12, 12, size=(1, 2, 64, 1)))).astype(np.float16)
    x[0, 0, 0, :4] = [0.0, -0.0, 6e-8, 65504.0]
    for rounding in (capi.ROUND_TRUNCATE, capi.ROUND_NEAREST):
        packed = capi.tilize_pack_cpu(torch.from_numpy(x), fmt, rounding)
        want = O.tilize_pack(x, fmt, rounding)
        assert np.array_equal(packed.numpy(), want)
        back = capi.unpack_untilize_cpu(packed, fmt, x.shape, torch.float16)
        assert np.array_equal(back.numpy().view(np.uint16), O.unpack_untilize(want, fmt, x.shape, O.Float16).view(np.uint16))
    with pytest.raises(capi.BackendError):
        capi.tilize_pack_cpu(torch.from_numpy(x), F.Bfp8_b)


def test_cpu_twin_integers_and_errors():
    rng = np.random.default_rng(5)
    for fmt, dtype in ((F.Int8, torch.int8), (F.UInt16, torch.int16), (F.Int32, torch.int32), (F.RawUInt32, torch.int32)):
        x = torch.from_numpy(rng.integers(-100, 100, size=(1, 2, 64, 32)).astype({torch.int8: np.int8, torch.int16: np.int16, torch.int32: np.int32}[dtype]))
        packed = capi.tilize_pack_cpu(x, fmt)
        assert np.array_equal(packed.numpy(), O.tilize_pack(x.numpy(), fmt))
        assert torch.equal(capi.unpack_untilize_cpu(packed, fmt, x.shape, dtype), x)
    with pytest.raises(capi.BackendError, match="multiples of the 32x32 tile"):
        capi.tilize_pack_cpu(torch.zeros(1, 1, 33, 32), F.Bfp8_b)
    with pytest.raises(capi.BackendError, match="pairs with itself only"):
        capi.tilize_pack_cpu(torch.zeros(1, 1, 32, 32), F.Int32)


def test_cpu_twin_golden_vectors():
    """The committed float64 statement of the format (tests/golden/bfp_vectors.npz) holds for the twins as it does for the
    oracle and the kernels."""
    vec = np.load(os.path.join(ROOT, "tests", "golden", "bfp_vectors.npz"))
    checked = 0
    for name in ("normal", "heavy_tail", "hand_placed"):
        x = torch.from_numpy(np.ascontiguousarray(vec["in_" + name]))
        for fmt_name, fmt in (("bfp8b", F.Bfp8_b), ("bfp4b", F.Bfp4_b), ("bfp2b", F.Bfp2_b)):
            for rname, rounding in (("trunc", capi.ROUND_TRUNCATE), ("near", capi.ROUND_NEAREST)):
                key = "%s_%s_%s" % (name, fmt_name, rname)
                packed = capi.tilize_pack_cpu(x, fmt, rounding)
                assert np.array_equal(packed.numpy(), vec[key + "_packed"]), key
                back = capi.unpack_untilize_cpu(packed, fmt, x.shape, torch.float32)
                assert np.array_equal(back.numpy().view(np.uint32), vec[key + "_floats"].view(np.uint32)), key
                checked += 1
    assert checked == 18


@pytest.mark.parametrize("epilogue", [capi.EPILOGUE_NONE, capi.EPILOGUE_GELU, capi.EPILOGUE_GELU_TANH])
def test_cpu_twin_gemm(epilogue):
    rng = np.random.default_rng(11 + epilogue)
    M, K, N = 64, 128, 96
    w = torch.from_numpy((rng.standard_normal((1, 1, K, N)) * 0.02).astype(np.float32))
    x = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).bfloat16()
    bias = torch.from_numpy((rng.standard_normal(N) * 0.02).astype(np.float32))
    wp = capi.tilize_pack_cpu(w, F.Bfp8_b)
    wd = capi.unpack_untilize_cpu(wp, F.Bfp8_b, w.shape, torch.float32)[0, 0]
    ref = x.float().double() @ wd.double() + bias.double()
    if epilogue == capi.EPILOGUE_GELU:
        ref = torch.nn.functional.gelu(ref)
    elif epilogue == capi.EPILOGUE_GELU_TANH:
        ref = torch.nn.functional.gelu(ref, approximate="tanh")
    got = capi.gemm_bfp8b_cpu(x, wp, N, bias=bias, epilogue=epilogue, out_dtype=torch.float32)
    assert float((got.double() - ref).norm() / ref.norm()) < 1e-6
    got16 = capi.gemm_bfp8b_cpu(x, wp, N, bias=bias.bfloat16(), epilogue=epilogue)
    ref16 = x.float().double() @ wd.double() + bias.bfloat16().double()
    if epilogue == capi.EPILOGUE_GELU:
        ref16 = torch.nn.functional.gelu(ref16)
    elif epilogue == capi.EPILOGUE_GELU_TANH:
        ref16 = torch.nn.functional.gelu(ref16, approximate="tanh")
    assert float((got16.double() - ref16).norm() / ref16.norm()) < 4e-3


def test_no_device_entry_point_calls_a_twin():
    """The twins are leaves: the sources of the device path never name them."""
    device = os.path.join(ROOT, "tt-buda_amd", "csrc", "device")
    host = os.path.join(ROOT, "tt-buda_amd", "csrc", "host")
    for d in (device, host):
        for f in os.listdir(d):
            if not f.endswith((".hip", ".hpp", ".cpp")) or f in ("cpu_twins.hip", "launch.hpp"):
                continue
            text = open(os.path.join(d, f)).read()
            calls = re.findall(r"\bcpu_(?:tilize_pack|unpack_untilize|gemm_bfp8b)\s*\(", text)
            if f == "c_abi.hip":  # its three _cpu entry points, one call each
                assert len(calls) == 3
                for fn in re.findall(r"int32_t (ttbfp_\w+)\([^)]*\)\s*\{(.*?)\n\}", text, re.S):
                    if "cpu_" in fn[1]:
                        assert fn[0].endswith("_cpu"), fn[0]
            else:
                assert not calls, f
    for f in ("backend.py", "op.py", "tensor.py", "tti.py"):
        assert "_cpu(" not in open(os.path.join(ROOT, "tt-buda_amd", f)).read(), f


@pytest.mark.gpu
def test_cpu_twins_equal_the_device_entry_points():
    rng = np.random.default_rng(21)
    x = torch.from_numpy(heavy_tailed(rng, (2, 1, 96, 160)))
    for fmt in (F.Bfp8_b, F.Bfp4_b, F.Bfp2_b, F.Float16_b):
        for rounding in (capi.ROUND_TRUNCATE, capi.ROUND_NEAREST):
            print("[case] cpu twin against the device", fmt, rounding, flush=True)
            host = capi.tilize_pack_cpu(x, fmt, rounding)
            dev = capi.tilize_pack(x.cuda(), fmt, rounding)
            assert torch.equal(dev.cpu(), host)
            assert torch.equal(capi.unpack_untilize(dev, fmt, x.shape, torch.bfloat16).cpu().view(torch.int16),
                               capi.unpack_untilize_cpu(host, fmt, x.shape, torch.bfloat16).view(torch.int16))
    M, K, N = 128, 256, 192
    w = torch.from_numpy((rng.standard_normal((1, 1, K, N)) * 0.02).astype(np.float32))
    a = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).bfloat16()
    wp = capi.tilize_pack_cpu(w, F.Bfp8_b)
    host = capi.gemm_bfp8b_cpu(a, wp, N, out_dtype=torch.float32)
    dev = capi.gemm_bfp8b(a.cuda(), wp.cuda(), N, out_dtype=torch.float32).cpu()
    assert float((dev - host).norm() / host.norm()) < 1e-6
