"""GPU parity: the HIP kernels, called through the C ABI (libttbfp.so), against the CPU oracle.

Integer/byte work (packed tiles, round-trip floats) must be bit-exact.  The GEMM is floating point:
relative Frobenius error <= 1e-3 against dequantize-then-fp32-matmul, the tolerance the benchmark
definition states; the fp32-output path is far tighter and is checked at 1e-5.
"""
import sys

import numpy as np
import pytest
import torch

import oracle as O
import tt_buda_amd as ttb
from tt_buda_amd import capi

pytestmark = pytest.mark.gpu

F = capi.DataFormatCode
BFP = [F.Bfp8_b, F.Bfp4_b, F.Bfp2_b]
DEV = "cuda:0"


def say(*a):
    print("[case]", *a, flush=True)
    sys.stdout.flush()


def to_dev(a):
    """numpy float32 or uint16(bf16 bits) array -> device tensor, strides preserved for views."""
    if a.dtype == np.uint16:
        return torch.from_numpy(a.view(np.int16)).to(DEV).view(torch.bfloat16)
    return torch.from_numpy(a).to(DEV)


def to_np(t):
    t = t.cpu()
    if t.dtype == torch.bfloat16:
        return t.view(torch.int16).numpy().view(np.uint16)
    return t.numpy()


def bits(a):
    return a.view(np.uint32) if a.dtype == np.float32 else a


def make_input(rng, shape, kind, dtype):
    x = rng.standard_normal(shape).astype(np.float32)
    if kind == "scaled":
        x *= np.exp2(rng.integers(-20, 21, (shape[0], shape[1], shape[2], 1))).astype(np.float32)
    elif kind == "edge":
        flat = x.reshape(-1)
        n = flat.size
        flat[rng.integers(0, n, n // 50)] = 0.0
        flat[rng.integers(0, n, n // 50)] = -0.0
        flat[rng.integers(0, n, n // 100)] = np.float32(1e-41)   # denormals
        flat[rng.integers(0, n, n // 100)] = np.float32(-3e-39)
        flat[rng.integers(0, n, n // 1000 + 1)] = np.float32(1e4)
        flat[rng.integers(0, n, n // 1000 + 1)] = np.float32(3.3e38)
        flat[rng.integers(0, n, n // 2000 + 1)] = np.float32(np.inf)
        flat[rng.integers(0, n, n // 2000 + 1)] = np.float32(np.nan)
        flat[: 64] = 0.0  # whole zero blocks
    if dtype == np.uint16:
        return O.f32_to_bf16_bits(x).reshape(shape)
    return x


SHAPES = [(1, 1, 32, 32), (1, 1, 64, 96), (2, 3, 32, 544), (1, 2, 96, 288)]


@pytest.mark.parametrize("dtype", [np.float32, np.uint16], ids=["fp32", "bf16"])
@pytest.mark.parametrize("fmt", BFP + [F.Float16_b, F.Float32])
@pytest.mark.parametrize("rounding", [0, 1], ids=["trunc", "nearest"])
def test_tilize_pack_bit_exact(dtype, fmt, rounding):
    widen = fmt == F.Float32 and dtype == np.uint16  # exact: the Float32 tiles of the same values held as fp32
    rng = np.random.default_rng(1000 + fmt + rounding)
    for shape in SHAPES:
        for kind in ("normal", "scaled", "edge"):
            say("tilize_pack", dtype.__name__, fmt, rounding, shape, kind)
            a = make_input(rng, shape, kind, dtype)
            want = O.tilize_pack((a.astype(np.uint32) << 16).view(np.float32) if widen else a, fmt, rounding)
            got = to_np(capi.tilize_pack(to_dev(a), fmt, rounding))
            assert got.size == want.size
            assert np.array_equal(got, want), f"{shape} {kind}: first diff at {np.flatnonzero(got != want)[:8]}"


@pytest.mark.parametrize("out", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
@pytest.mark.parametrize("fmt", BFP + [F.Float16_b, F.Float32])
def test_unpack_untilize_bit_exact(out, fmt):
    if fmt == F.Float32 and out == torch.bfloat16:
        pytest.skip("Float32 tiles are read back as Float32 only")
    rng = np.random.default_rng(2000 + fmt)
    ofmt = F.Float32 if out == torch.float32 else F.Float16_b
    for shape in SHAPES:
        # arbitrary bytes: every exponent/datum combination, including ones the packer never emits
        # (denormal results, exponent 255); for plain tiles random floats
        say("unpack_untilize", out, fmt, shape)
        n = O.packed_size(fmt, shape)
        if fmt in BFP:
            packed = rng.integers(0, 256, n, dtype=np.uint8)
            packed.reshape(-1, O.tile_bytes(fmt))[::3, :64] = rng.integers(0, 9, 64, dtype=np.uint8)  # tiny exponents
        else:
            packed = O.tilize_pack(make_input(rng, shape, "edge", np.float32), fmt).copy()
        want = O.unpack_untilize(packed, fmt, shape, ofmt)
        got = to_np(capi.unpack_untilize(torch.from_numpy(packed).to(DEV), fmt, shape, out))
        assert np.array_equal(bits(got), bits(want)), f"{shape}: diff at {np.argwhere(bits(got) != bits(want))[:4]}"
        if fmt in BFP:
            # mid-range exponents with arbitrary datums (signed zero magnitudes among them): whole
            # wavefronts then stay on the multiply-based path
            packed.reshape(-1, O.tile_bytes(fmt))[:, :64] = rng.integers(8, 255, (n // O.tile_bytes(fmt), 64), dtype=np.uint8)
            want = O.unpack_untilize(packed, fmt, shape, ofmt)
            got = to_np(capi.unpack_untilize(torch.from_numpy(packed).to(DEV), fmt, shape, out))
            assert np.array_equal(bits(got), bits(want)), f"{shape}: diff at {np.argwhere(bits(got) != bits(want))[:4]}"


# ------------------------------------------------------------------------------------------------
# the family with the 5-bit exponent of IEEE half (Float16 sources, Float16 results)
# ------------------------------------------------------------------------------------------------

A_FAMILY = [F.Bfp8, F.Bfp4, F.Bfp2, F.Float16]


def make_half_input(rng, shape, kind):
    x = rng.standard_normal(shape).astype(np.float32)
    if kind == "scaled":
        x *= np.exp2(rng.integers(-12, 10, (shape[0], shape[1], shape[2], 1))).astype(np.float32)
    elif kind == "edge":
        flat = x.reshape(-1)
        n = flat.size
        flat[rng.integers(0, n, n // 40)] = 0.0
        flat[rng.integers(0, n, n // 40)] = -0.0
        flat[rng.integers(0, n, n // 60)] = np.float32(3e-6)     # half denormals
        flat[rng.integers(0, n, n // 500 + 1)] = np.float32(65504.0)
        flat[rng.integers(0, n, n // 1000 + 1)] = np.float32(np.inf)
        flat[rng.integers(0, n, n // 1000 + 1)] = np.float32(np.nan)
        flat[:64] = 0.0
    with np.errstate(over="ignore"):
        return x.astype(np.float16)


@pytest.mark.parametrize("fmt", A_FAMILY)
@pytest.mark.parametrize("rounding", [0, 1], ids=["trunc", "nearest"])
def test_half_family_tilize_pack_bit_exact(fmt, rounding):
    rng = np.random.default_rng(3000 + fmt + rounding)
    for shape in SHAPES:
        for kind in ("normal", "scaled", "edge"):
            say("tilize_pack half", fmt, rounding, shape, kind)
            a = make_half_input(rng, shape, kind)
            want = O.tilize_pack(a, fmt, rounding)
            got = to_np(capi.tilize_pack(torch.from_numpy(a).to(DEV), fmt, rounding))
            assert np.array_equal(got, want), f"{shape} {kind}: first diff at {np.flatnonzero(got != want)[:8]}"
    # strided view -> the general kernel
    base = make_half_input(rng, (1, 2, 64, 128), "edge")
    view = base[:, :, :, ::2]
    got = to_np(capi.tilize_pack(torch.from_numpy(base).to(DEV)[:, :, :, ::2], fmt, rounding))
    assert np.array_equal(got, O.tilize_pack(view, fmt, rounding))


@pytest.mark.parametrize("fmt", A_FAMILY)
def test_half_family_unpack_untilize_bit_exact(fmt):
    rng = np.random.default_rng(4000 + fmt)
    for shape in SHAPES:
        say("unpack_untilize half", fmt, shape)
        n = O.packed_size(fmt, shape)
        if fmt == F.Float16:
            packed = O.tilize_pack(make_half_input(rng, shape, "edge"), fmt).copy()
        else:
            packed = rng.integers(0, 256, n, dtype=np.uint8)  # any exponent byte, any datum
        want = O.unpack_untilize(packed, fmt, shape, O.Float16)
        got = capi.unpack_untilize(torch.from_numpy(packed).to(DEV), fmt, shape, torch.float16).cpu().numpy()
        assert np.array_equal(got.view(np.uint16), want.view(np.uint16)), f"{shape}"
        # strided destination -> the general kernel
        out = torch.zeros(shape[0], shape[1], shape[2], shape[3] * 2, dtype=torch.float16, device=DEV)[:, :, :, ::2]
        capi.unpack_untilize(torch.from_numpy(packed).to(DEV), fmt, shape, torch.float16, out=out)
        assert np.array_equal(out.contiguous().cpu().numpy().view(np.uint16), want.view(np.uint16))


def test_half_family_format_pairs_are_enforced():
    x16 = torch.zeros(1, 1, 32, 32, dtype=torch.float16, device=DEV)
    x32 = torch.zeros(1, 1, 32, 32, dtype=torch.float32, device=DEV)
    with pytest.raises(capi.BackendError):
        capi.tilize_pack(x16, F.Bfp8_b)   # half sources do not feed the 8-bit exponent formats
    with pytest.raises(capi.BackendError):
        capi.tilize_pack(x32, F.Bfp8)     # and the 5-bit exponent formats take nothing but half
    packed = capi.tilize_pack(x16, F.Bfp4)
    with pytest.raises(capi.BackendError):
        capi.unpack_untilize(packed, F.Bfp4, x16.shape, torch.float32)


@pytest.mark.parametrize("fmt", BFP + [F.Float16_b])
def test_strided_and_unaligned_views_take_the_general_kernels(fmt):
    rng = np.random.default_rng(3000 + fmt)
    base = make_input(rng, (1, 2, 64, 200), "scaled", np.float32)
    views = {
        "column-strided": base[:, :, :, ::2][:, :, :, :96],
        "transposed": np.ascontiguousarray(base[:, :, :, :64]).transpose(0, 1, 3, 2),
        "offset-by-one-element": base[:, :, :, 1:161],
    }
    for name, v in views.items():
        say("general path", fmt, name, v.shape, v.strides)
        want = O.tilize_pack(v, fmt)
        dev_base = to_dev(base)
        if name == "column-strided":
            dv = dev_base[:, :, :, ::2][:, :, :, :96]
        elif name == "transposed":
            dv = dev_base[:, :, :, :64].contiguous().permute(0, 1, 3, 2)
        else:
            dv = dev_base[:, :, :, 1:161]
        assert tuple(dv.shape) == v.shape
        got = capi.tilize_pack(dv, fmt)
        assert np.array_equal(to_np(got), want)
        # and back into a strided destination
        for dt, ofmt in ((torch.float32, F.Float32), (torch.bfloat16, F.Float16_b)):
            want_rt = O.unpack_untilize(want, fmt, v.shape, ofmt)
            holder = torch.zeros((1, 2, v.shape[2], v.shape[3] * 2 + 1), dtype=dt, device=DEV)
            dst = holder[:, :, :, 1::2]
            capi.unpack_untilize(got, fmt, v.shape, out=dst)
            assert np.array_equal(bits(to_np(dst.contiguous())), bits(want_rt))
            assert float(holder[:, :, :, 0::2].abs().sum()) == 0.0  # nothing written between the elements


@pytest.mark.parametrize("dtype", [np.float32, np.uint16], ids=["fp32", "bf16"])
@pytest.mark.parametrize("fmt", BFP + [F.Float16_b])
def test_unit_stride_views_that_start_anywhere_stay_bit_exact(dtype, fmt):
    """Sliced views of a row-major tensor (pybuda/pybuda/tensor.py:707-717): unit element stride, but a first element and a
    row pitch that are multiples of the element size only.  They run on the row kernels (16-byte accesses that start
    anywhere) and must give the bytes of the contiguous copy; on the way back nothing around the view may be touched."""
    rng = np.random.default_rng(int(fmt) * 3 + (dtype == np.uint16))
    tdt = torch.float32 if dtype == np.float32 else torch.bfloat16
    # (holder columns, first column, columns): one element off; an odd row pitch; several segments with a partial last one
    for width, c0, cols in ((192, 1, 160), (163, 2, 160), (1127, 3, 1120), (613, 7, 544)):
        shape = (2, 2, 64, width)
        base = make_input(rng, shape, "scaled", dtype)
        view = base[:, :, :, c0:c0 + cols]
        say("unaligned unit-stride view", fmt, dtype.__name__, width, c0, cols)
        want = O.tilize_pack(np.ascontiguousarray(view), fmt)
        dv = to_dev(base)[:, :, :, c0:c0 + cols]
        assert dv.data_ptr() % 16 != 0 or (width * dv.element_size()) % 16 != 0
        got = capi.tilize_pack(dv, fmt)
        assert np.array_equal(to_np(got), want)
        for dt, ofmt in ((torch.float32, F.Float32), (torch.bfloat16, F.Float16_b)):
            want_rt = O.unpack_untilize(want, fmt, view.shape, ofmt)
            holder = torch.full(shape, -77.0, dtype=dt, device=DEV)
            capi.unpack_untilize(got, fmt, view.shape, out=holder[:, :, :, c0:c0 + cols])
            assert np.array_equal(bits(to_np(holder[:, :, :, c0:c0 + cols].contiguous())), bits(want_rt))
            assert bool((holder[:, :, :, :c0] == -77.0).all()) and bool((holder[:, :, :, c0 + cols:] == -77.0).all())
        # ragged rows and columns of such a view: padding inside the pack launch, narrowing inside the unpack launch
        rv, cv = 50, cols - 8
        ragged = dv[:, :, :rv, :cv]
        pad = np.zeros((2, 2, 64, cols), dtype=dtype)
        pad[:, :, :rv, :cv] = view[:, :, :rv, :cv]
        want_p = O.tilize_pack(pad, fmt)
        got_p = capi.tilize_pack_padded(ragged, fmt)
        assert np.array_equal(to_np(got_p), want_p)
        holder = torch.full(shape, -77.0, dtype=tdt, device=DEV)
        capi.unpack_untilize_narrow(got_p, fmt, (2, 2, rv, cv), out=holder[:, :, :rv, c0:c0 + cv])
        want_n = O.unpack_untilize(want_p, fmt, (2, 2, 64, cols), F.Float32 if dtype == np.float32 else F.Float16_b)[:, :, :rv, :cv]
        assert np.array_equal(bits(to_np(holder[:, :, :rv, c0:c0 + cv].contiguous())), bits(np.ascontiguousarray(want_n)))
        holder[:, :, :rv, c0:c0 + cv] = -77.0
        assert bool((holder == -77.0).all())


def test_config1_bfp8_round_trip_1024():
    """fp32 [1,1,1024,1024] N(0,1) seed 0: packed bytes and round-trip floats bit-exact."""
    torch.manual_seed(0)
    x = torch.randn(1, 1, 1024, 1024)
    say("config 1")
    xd = x.to(DEV)
    packed = capi.tilize_pack(xd, F.Bfp8_b)
    assert packed.numel() == 1_114_112
    want = O.tilize_pack(x.numpy(), F.Bfp8_b)
    assert np.array_equal(to_np(packed), want)
    rt = capi.unpack_untilize(packed, F.Bfp8_b, x.shape, torch.float32)
    want_rt = O.unpack_untilize(want, F.Bfp8_b, tuple(x.shape), O.Float32)
    assert np.array_equal(to_np(rt).view(np.uint32), want_rt.view(np.uint32))
    # pack(unpack(pack(x))) == pack(x)
    assert torch.equal(capi.tilize_pack(rt, F.Bfp8_b), packed)


def config2_input():
    g = torch.Generator().manual_seed(1)
    x = torch.randn(1, 1, 4096, 4096, generator=g)
    k = torch.randint(-20, 21, (128,), generator=g)
    x = x * torch.exp2(k.float()).repeat_interleave(32).view(1, 1, 4096, 1)
    x[torch.rand(x.shape, generator=g) < 0.01] = 0.0
    out = torch.rand(x.shape, generator=g) < 0.001
    sign = torch.where(torch.rand(x.shape, generator=g) < 0.5, -1.0, 1.0)
    x[out] = (sign * 1e4)[out]
    return x


@pytest.mark.parametrize("fmt", [F.Bfp4_b, F.Bfp2_b])
def test_config2_heavy_tailed_4096(fmt):
    x = config2_input()
    say("config 2", fmt)
    packed = capi.tilize_pack(x.to(DEV), fmt)
    assert packed.numel() == {F.Bfp4_b: 9_437_184, F.Bfp2_b: 5_242_880}[fmt]
    want = O.tilize_pack(x.numpy(), fmt, nthreads=8)
    assert np.array_equal(to_np(packed), want)
    rt = capi.unpack_untilize(packed, fmt, x.shape, torch.float32)
    want_rt = O.unpack_untilize(want, fmt, tuple(x.shape), O.Float32, nthreads=8)
    assert np.array_equal(to_np(rt).view(np.uint32), want_rt.view(np.uint32))


def test_config3_streaming_shape_properties_and_slice_parity():
    """bf16 [8,1,8192,8192] U(-8,8): full-size invariants, oracle parity on one w-slice."""
    say("config 3 generate")
    g = torch.Generator(device=DEV).manual_seed(2)
    x = (torch.rand(8, 1, 8192, 8192, generator=g, device=DEV) * 16 - 8).bfloat16()
    say("config 3 pack")
    packed = capi.tilize_pack(x, F.Bfp8_b)
    assert packed.numel() == 570_425_344
    say("config 3 unpack")
    rt = capi.unpack_untilize(packed, F.Bfp8_b, x.shape, torch.bfloat16)
    # truncation never grows a magnitude; error below the block step (|x| <= 8 after bf16
    # rounding, so the shared exponent is at most 3 and the step at most 2^(3-6))
    never_grows = bool((rt.abs() <= x.abs()).all())
    worst = float((x.float() - rt.float()).abs().max())
    assert never_grows
    assert worst < 2.0 ** -3, worst
    # idempotence at full size
    say("config 3 repack")
    assert torch.equal(capi.tilize_pack(rt, F.Bfp8_b), packed)
    # the tile order puts w outermost: slice w=5 is a contiguous eighth of the packed buffer
    say("config 3 oracle slice")
    w = 5
    xs = to_np(x[w:w + 1])
    want = O.tilize_pack(xs, F.Bfp8_b, nthreads=8)
    per_w = packed.numel() // 8
    assert np.array_equal(to_np(packed[w * per_w:(w + 1) * per_w]), want)
    want_rt = O.unpack_untilize(want, F.Bfp8_b, xs.shape, O.Float16_b, nthreads=8)
    assert np.array_equal(to_np(rt[w:w + 1]), want_rt)


def test_tensor_beyond_4_gib_properties_and_far_end_parity():
    """bf16 [5,2,16384,16384]: 5 GiB of source and 2.7 GiB of tiles, so byte offsets pass 2^32 on both sides.  Full-size
    invariants, and oracle parity on the last tile rows of the last slice, where a 32-bit offset would have wrapped."""
    shape = (5, 2, 16384, 16384)
    say("beyond 4 GiB generate")
    x = torch.empty(shape, dtype=torch.bfloat16, device=DEV)
    g = torch.Generator(device=DEV).manual_seed(77)
    for w in range(shape[0]):
        for z in range(shape[1]):
            x[w, z] = (torch.randn(shape[2:], generator=g, device=DEV) * float(2 ** (w - z))).bfloat16()
    say("beyond 4 GiB pack")
    packed = capi.tilize_pack(x, F.Bfp4_b)
    assert packed.numel() == capi.packed_size(F.Bfp4_b, shape) == 5 * 2 * 512 * 512 * 576
    say("beyond 4 GiB unpack")
    rt = capi.unpack_untilize(packed, F.Bfp4_b, shape, torch.bfloat16)
    assert bool((rt.abs() <= x.abs()).all())                       # truncation never grows a magnitude
    assert bool(((rt == 0) | (torch.sign(rt) == torch.sign(x))).all())  # signs survive unless the magnitude is zero
    say("beyond 4 GiB repack")
    assert torch.equal(capi.tilize_pack(rt, F.Bfp4_b), packed)     # idempotence at full size
    say("beyond 4 GiB oracle on the far end")
    rows = 64                                                      # the last two tile rows of the last slice
    xs = to_np(x[4:5, 1:2, -rows:, :])
    want = O.tilize_pack(xs, O.Bfp4_b, nthreads=8)
    assert np.array_equal(to_np(packed[-want.size:]), want)
    want_rt = O.unpack_untilize(want, O.Bfp4_b, xs.shape, O.Float16_b, nthreads=8)
    assert np.array_equal(to_np(rt[4:5, 1:2, -rows:, :]), want_rt)
    # the queue form at the same size: a 4 x 4 grid of buffers, 0.67 GiB apart
    lay = capi.QueueLayout(4, 4, 16, 32, 8, 4, 1, 0)
    say("beyond 4 GiB queue form")
    q = capi.tilize_pack_queue(x, F.Bfp4_b, lay)
    assert q.numel() == packed.numel()
    assert torch.equal(capi.unpack_untilize_queue(q, F.Bfp4_b, shape, lay, dtype=torch.bfloat16), rt)
    olay = O.QueueLayout(4, 4, 16, 32, 8, 4, 1, 0)
    gr, gc, addr = O.queue_map(olay, 1, 511, 511)                  # the very last tile: buffer (3, 3), last address of slice z = 1
    per_buffer = q.numel() // 16
    at = (gr * 4 + gc) * per_buffer + ((4 * 2) * (16 * 32 * 8 * 4) + addr) * 576
    assert at + 576 == q.numel() and torch.equal(q[at:at + 576], packed[-576:])


# ------------------------------------------------------------------------------------------------
# GEMM with Bfp8_b weights
# ------------------------------------------------------------------------------------------------

def rel_fro(a, b):
    a, b = a.double(), b.double()
    return float((a - b).norm() / b.norm())


def packed_weight(K, N, seed, std=0.02):
    g = torch.Generator().manual_seed(seed)
    w = torch.randn(K, N, generator=g) * std
    wp = capi.tilize_pack(w.view(1, 1, K, N).to(DEV), F.Bfp8_b)
    # the packed bytes themselves are oracle-checked, so the dequantized matrix is the oracle's
    want = O.tilize_pack(w.view(1, 1, K, N).numpy(), F.Bfp8_b, nthreads=8)
    assert np.array_equal(to_np(wp), want)
    wdq = torch.from_numpy(O.dequant_weight(want, K, N))
    return wp, wdq


def test_gemm_small_against_the_c_oracle():
    rng = np.random.default_rng(5)
    M, K, N = 64, 96, 160
    w = (rng.standard_normal((1, 1, K, N)) * 0.02).astype(np.float32)
    wp = O.tilize_pack(w, F.Bfp8_b)
    x = O.f32_to_bf16_bits(rng.standard_normal((M, K)).astype(np.float32))
    b = O.f32_to_bf16_bits((rng.standard_normal(N) * 0.02).astype(np.float32))
    xd, wd, bd = to_dev(x), torch.from_numpy(wp).to(DEV), to_dev(b)
    for bias, epi in ((None, 0), (b, 0), (b, 1), (b, 2)):
        say("gemm small", "bias" if bias is not None else "nobias", epi)
        want = torch.from_numpy(O.gemm_bfp(x, wp, N, bias_bf16=bias, epilogue=epi))
        got32 = capi.gemm_bfp8b(xd, wd, N, bias=bd if bias is not None else None, epilogue=epi, out_dtype=torch.float32)
        assert rel_fro(got32.cpu(), want) < 1e-5
        got16 = capi.gemm_bfp8b(xd, wd, N, bias=bd if bias is not None else None, epilogue=epi)
        assert rel_fro(got16.cpu().float(), want.bfloat16().float()) < 1e-3
        assert rel_fro(got16.cpu().float(), want) < 4e-3  # bf16 output rounding alone is ~1.5e-3


@pytest.mark.parametrize("shape", [(32, 96, 160), (32, 1024, 64), (32, 2048, 64), (32, 3072, 32), (64, 3072, 64), (64, 160, 96), (64, 2080, 32), (96, 1504, 192), (128, 256, 384),
                                   (128, 4096, 4096), (160, 96, 224), (224, 128, 256), (608, 192, 384), (416, 160, 96), (256, 512, 256), (384, 192, 640), (512, 1024, 1024),
                                   (768, 128, 16384), (256, 64, 64), (384, 1088, 192), (128 * 17, 128 * 17, 256), (128, 64, 128), (640, 1600, 192), (1024, 2112, 320), (640, 1600, 384), (2048, 1152, 256),
                                   (1024, 4096, 128), (3072, 4096, 192), (6144, 2048, 64),
                                   # K an odd number of tile rows (half a slab at the end) in every form of the macro-tiled kernel, and N an odd
                                   # number of tiles (the last tile column goes to one-row-tile workgroups of the weight-streaming kernel)
                                   (256, 96, 64), (256, 160, 128), (256, 288, 96), (4224, 96, 576), (3072, 160, 1024), (2176, 96, 2176),
                                   (3072, 96, 4096), (768, 160, 16384), (416, 224, 224),
                                   # 192 x 64 macro tiles with two pipelines (16 x 16 and 8 x 32 of them; the first above with half a slab
                                   # at the end), and 128 x 128 with two pipelines where 192 does not divide M
                                   (1536, 256, 2048), (3072, 128, 1024), (2048, 160, 1536), (2048, 256, 1536), (512, 4096, 4128), (512, 4128, 4096), (8192, 4128, 4128)])
def test_gemm_kernel_selection_shapes(shape):
    """One shape per kernel path: one to four tile rows (weight streaming; K that splits unevenly over the wavefronts,
    fewer tile rows of W than wavefronts, slices of one, two, three and four whole tile pairs and of odd counts), ragged (general kernel), 128 x 64
    macro tiles (fewer than 256 tiles of 128 x 128; up to 256 of them in the form with rings - one pipeline where K is an odd number of slabs:
    one, three; two pipelines else: one slab each, two, three; N = 64, N a multiple of 64 only - more in the two-stage form: 33 x 8 tiles),
    128 x 128 macro tiles with two pipelines (16 x 9 and 8 x 32 of them, two slabs and one slab per pipeline), 192 x 64 macro tiles with
    two pipelines, 384 x 128 macro tiles
    (8 x 32 and 16 x 16 of them, where they fill the CUs better than 256 x 256: three slabs, one slab), 128 x 128 macro tiles (17 x 17 of them), and
    enough tiles for the 256 x 256 macro tiles (M = 768); all against
    dequantize-then-fp32-matmul with bias and GELU in both of the reference's forms."""
    M, K, N = shape
    rng = np.random.default_rng(M + K + N)
    w = (rng.standard_normal((1, 1, K, N)) * 0.05).astype(np.float32)
    wp = O.tilize_pack(w, F.Bfp8_b, nthreads=4)
    wdq = torch.from_numpy(O.dequant_weight(wp, K, N))
    x = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).bfloat16()
    b = torch.from_numpy((rng.standard_normal(N) * 0.05).astype(np.float32)).bfloat16()
    xd, wd, bd = x.to(DEV), torch.from_numpy(wp).to(DEV), b.to(DEV)
    base = x.float() @ wdq
    b3 = b.float() * 3 + 1e-3  # an fp32 bias that is no bf16 value (TTBFP_EPILOGUE_BIAS_F32): three times a bias, as the accumulate form adds it
    b3d = b3.to(DEV)
    for bias, epi in ((None, 0), (b, 0), (b, 1), (None, 2), (b3, 0), (b3, 2)):
        say("gemm shapes", shape, "bias" if bias is not None else "nobias", epi)
        want = base + (bias.float() if bias is not None else 0.0)
        if bias is b3:
            bd = b3d
        if epi:  # the two forms of pybuda/pybuda/op/eval/pybuda/eltwise_unary.py:42-49
            want = torch.nn.functional.gelu(want, approximate="tanh" if epi == 2 else "none")
        got32 = capi.gemm_bfp8b(xd, wd, N, bias=bd if bias is not None else None, epilogue=epi, out_dtype=torch.float32).cpu()
        got16 = capi.gemm_bfp8b(xd, wd, N, bias=bd if bias is not None else None, epilogue=epi).cpu()
        e32, e16 = rel_fro(got32, want), rel_fro(got16.float(), want.bfloat16().float())
        assert e32 < 1e-5 and e16 < 1e-3, (shape, epi, e32, e16)


@pytest.mark.parametrize("M", [32, 64, 512, 8192])
def test_config4_gemm_4096(M):
    """W fp32 [4096,4096] N(0,0.02) seed 3 -> Bfp8_b; X bf16 [M,4096] N(0,1) seed 4."""
    K = N = 4096
    say("config 4 weights", M)
    wp, wdq = packed_weight(K, N, seed=3)
    g = torch.Generator().manual_seed(4)
    x = torch.randn(M, K, generator=g).bfloat16()
    say("config 4 reference matmul", M)
    want = x.float() @ wdq  # dequantize-then-fp32-matmul on the host
    say("config 4 gemm", M)
    got32 = capi.gemm_bfp8b(x.to(DEV), wp, N, out_dtype=torch.float32).cpu()
    got16 = capi.gemm_bfp8b(x.to(DEV), wp, N).cpu()
    e32, e16 = rel_fro(got32, want), rel_fro(got16.float(), want.bfloat16().float())
    e16u = rel_fro(got16.float(), want)  # against the un-rounded reference: output rounding alone is ~1.5e-3, a biased rounding would show
    print(f"M={M}: rel-Frobenius fp32-out {e32:.3e}, bf16-out vs bf16-rounded reference {e16:.3e}, vs un-rounded {e16u:.3e}, "
          f"max-abs {float((got32 - want).abs().max()):.3e}", flush=True)
    assert e32 < 1e-3 and e16 < 1e-3 and e16u < 4e-3


def test_config5_bert_large_ffn():
    """GELU(X W1 + b1) W2 + b2, X bf16 [3072,1024], W1 [1024,4096], W2 [4096,1024] in Bfp8_b."""
    say("config 5")
    g = torch.Generator().manual_seed(5)
    x = torch.randn(3072, 1024, generator=g).bfloat16()
    w1p, w1 = packed_weight(1024, 4096, seed=51)
    w2p, w2 = packed_weight(4096, 1024, seed=52)
    b1 = (torch.randn(4096, generator=g) * 0.02).bfloat16()
    b2 = (torch.randn(1024, generator=g) * 0.02).bfloat16()
    # reference: golden matmul + bias row, exact gelu, bf16 between the two matmuls as on the device
    h = torch.nn.functional.gelu(x.float() @ w1 + b1.float()).bfloat16()
    want = h.float() @ w2 + b2.float()
    hd = capi.gemm_bfp8b(x.to(DEV), w1p, 4096, bias=b1.to(DEV), epilogue=capi.EPILOGUE_GELU)
    assert rel_fro(hd.cpu().float(), h.float()) < 1e-3
    y32 = capi.gemm_bfp8b(hd, w2p, 1024, bias=b2.to(DEV), out_dtype=torch.float32).cpu()
    y16 = capi.gemm_bfp8b(hd, w2p, 1024, bias=b2.to(DEV)).cpu()
    e32, e16, e16u = rel_fro(y32, want), rel_fro(y16.float(), want.bfloat16().float()), rel_fro(y16.float(), want)
    print(f"FFN: rel-Frobenius fp32-out {e32:.3e}, bf16-out {e16:.3e}, bf16-out vs un-rounded {e16u:.3e}", flush=True)
    assert e32 < 1e-3 and e16 < 1e-3 and e16u < 4e-3


def test_north_star_gemm_8192_cubed():
    """The shape the GEMM target is quoted on: W fp32 [8192,8192] N(0,0.02) -> Bfp8_b (bytes oracle-checked), X bf16
    [8192,8192] N(0,1); the fused kernel and the workspace (bf16 panel) form, Float32 and Float16_b results.  Checked
    against dequantize-then-fp32-matmul on the host (pybuda/pybuda/op/eval/buda/matmul.py:233-249) on 256 rows: eight in
    each of the 32 rows of 256 x 256 macro tiles, placed so that both wavefront rows, every 32-row MFMA block and both
    lane halves are hit, over all of N - so every macro tile and every block of tiles an XCD works on is compared."""
    M = N = K = 8192
    say("north star weights")
    wp, wdq = packed_weight(K, N, seed=8)
    g = torch.Generator().manual_seed(9)
    x = torch.randn(M, K, generator=g).bfloat16()
    inside = torch.tensor([0, 37, 70, 103, 128 + 5, 128 + 58, 128 + 91, 255])
    rows = (torch.arange(32).view(32, 1) * 256 + inside.view(1, 8)).reshape(-1)
    say("north star reference matmul on", rows.numel(), "rows")
    want = x[rows].float() @ wdq
    xd = x.to(DEV)
    need = capi.gemm_workspace_bytes(M, N, K)
    assert need == 2 * K * N
    ws = torch.empty(need, dtype=torch.uint8, device=DEV)
    for out_dtype in (torch.float32, torch.bfloat16):
        say("north star gemm", out_dtype)
        fused = capi.gemm_bfp8b(xd, wp, N, out_dtype=out_dtype)
        two = capi.gemm_bfp8b(xd, wp, N, out_dtype=out_dtype, workspace=ws)
        assert torch.equal(fused, two)
        got = fused[rows.to(DEV)].cpu()
        if out_dtype == torch.float32:
            e = rel_fro(got, want)
            print(f"8192^3 fp32-out: rel-Frobenius {e:.3e}, max-abs {float((got - want).abs().max()):.3e}", flush=True)
            assert e < 1e-5
        else:
            e, eu = rel_fro(got.float(), want.bfloat16().float()), rel_fro(got.float(), want)
            print(f"8192^3 bf16-out: rel-Frobenius vs bf16-rounded {e:.3e}, vs un-rounded {eu:.3e}", flush=True)
            assert e < 1e-3 and eu < 4e-3


def test_errors_are_status_codes_not_crashes():
    x = torch.zeros(1, 1, 33, 32, device=DEV)
    with pytest.raises(capi.BackendError) as ei:
        out = torch.empty(4096, dtype=torch.uint8, device=DEV)
        capi.check(capi.lib().ttbfp_tilize_pack(x.data_ptr(), 0, (capi.ctypes.c_uint32 * 4)(1, 1, 33, 32),
                                                (capi.ctypes.c_uint64 * 4)(4224, 4224, 128, 4), F.Bfp8_b, 0,
                                                out.data_ptr(), 4096, None))
    assert ei.value.status == capi.RUNTIME_ERROR and "multiples" in str(ei.value)
    with pytest.raises(capi.BackendError):  # destination too small
        capi.tilize_pack(torch.zeros(1, 1, 32, 32, device=DEV), F.Bfp8_b, out=torch.empty(100, dtype=torch.uint8, device=DEV))
    with pytest.raises(capi.BackendError):  # unsupported format (Bfp8 with 5-bit exponent)
        capi.tilize_pack(torch.zeros(1, 1, 32, 32, device=DEV), 2)
    assert ttb.capi.lib().ttbfp_init(0) == capi.SUCCESS


def test_sized_entry_points_match_the_plain_ones_and_guard_the_buffers():
    """ttbfp_unpack_untilize_sized / ttbfp_gemm_bfp8b_bf16_sized run the same launches as the entry points without sizes
    and refuse a destination that is one element short, leaving it untouched."""
    say("sized entry points")
    rng = np.random.default_rng(77)
    shape = (2, 1, 64, 96)
    x = to_dev(rng.standard_normal(shape).astype(np.float32))
    packed = capi.tilize_pack(x, F.Bfp8_b)
    want = capi.unpack_untilize(packed, F.Bfp8_b, shape, torch.bfloat16)
    assert torch.equal(capi.unpack_untilize_sized(packed, F.Bfp8_b, shape, torch.bfloat16), want)
    ragged = (2, 1, 50, 70)
    assert torch.equal(capi.unpack_untilize_sized(packed, F.Bfp8_b, ragged, torch.bfloat16), want[:, :, :50, :70])
    lay = capi.QueueLayout(2, 3, 1, 1, 1, 1, 1, 1)
    qmem = capi.tilize_pack_queue(x, F.Bfp8_b, lay)
    assert torch.equal(capi.unpack_untilize_sized(qmem, F.Bfp8_b, shape, torch.bfloat16, layout=lay), want)
    short = torch.zeros(x.numel() - 1, dtype=torch.bfloat16, device=DEV)
    st = [s * 2 for s in want.stride()]
    code = capi.lib().ttbfp_unpack_untilize_sized(packed.data_ptr(), packed.numel(), F.Bfp8_b, (capi.ctypes.c_uint32 * 4)(*shape), None, 0,
                                                  F.Float16_b, (capi.ctypes.c_uint64 * 4)(*st), short.data_ptr(), short.numel() * 2, None)
    torch.cuda.synchronize()
    assert code == capi.RUNTIME_ERROR and "destination holds" in capi.lib().ttbfp_last_error().decode() and not short.any()
    with pytest.raises(capi.BackendError):  # fewer tiles than the shape needs
        capi.unpack_untilize_sized(packed[:-1], F.Bfp8_b, shape, torch.bfloat16)

    M, K, N = 96, 128, 160
    wp = capi.tilize_pack(to_dev((rng.standard_normal((1, 1, K, N)) * 0.05).astype(np.float32)), F.Bfp8_b)
    a = to_dev(rng.standard_normal((M, K)).astype(np.float32)).bfloat16()
    b = to_dev(rng.standard_normal(N).astype(np.float32)).bfloat16()
    assert torch.equal(capi.gemm_bfp8b(a, wp, N, bias=b, epilogue=1, sized=True), capi.gemm_bfp8b(a, wp, N, bias=b, epilogue=1))
    y = torch.zeros(M * N - 1, dtype=torch.bfloat16, device=DEV)
    code = capi.lib().ttbfp_gemm_bfp8b_bf16_sized(M, N, K, a.data_ptr(), M * K * 2, wp.data_ptr(), wp.numel(), None, 0, 0, y.data_ptr(),
                                                  y.numel() * 2, F.Float16_b, None, 0, None)
    torch.cuda.synchronize()
    assert code == capi.RUNTIME_ERROR and "y holds" in capi.lib().ttbfp_last_error().decode() and not y.any()


@pytest.mark.parametrize("shape", [(0, 1, 32, 32), (1, 0, 64, 64), (1, 1, 32, 32), (1, 1, 32, 32 * 17), (1, 1, 32 * 9, 32), (5, 3, 32, 96),
                                   (1, 1, 64, 32 * 129)])
def test_empty_single_tile_and_ragged_shapes(shape):
    """No entries at all, one tile, and widths that end inside a workgroup's 8- or 16-tile segment."""
    rng = np.random.default_rng(sum(shape))
    for dtype, odtype in ((torch.float32, np.float32), (torch.bfloat16, np.uint16)):
        say("edge shape", shape, dtype)
        host = rng.standard_normal(shape).astype(np.float32)
        x = torch.from_numpy(host).to(DEV).to(dtype)
        src = host if dtype == torch.float32 else O.f32_to_bf16_bits(x.float().cpu().numpy())
        for fmt, ofmt in ((F.Bfp8_b, O.Bfp8_b), (F.Bfp2_b, O.Bfp2_b)):
            packed = capi.tilize_pack(x, fmt)
            assert packed.numel() == capi.packed_size(fmt, shape)
            if packed.numel() == 0:
                assert capi.unpack_untilize(packed, fmt, shape, dtype).numel() == 0
                continue
            want = O.tilize_pack(src.reshape(shape), ofmt)
            assert np.array_equal(packed.cpu().numpy(), want)
            back = capi.unpack_untilize(packed, fmt, shape, dtype)
            want_back = O.unpack_untilize(want, ofmt, shape, O.Float32 if dtype == torch.float32 else O.Float16_b)
            got = back.cpu().numpy() if dtype == torch.float32 else back.view(torch.int16).cpu().numpy().view(np.uint16)
            assert np.array_equal(got.view(want_back.dtype), want_back)


@pytest.mark.parametrize("shape", [(4096, 3072, 64), (4096, 3072, 320), (4096, 4096, 128), (8192, 4096, 4096), (6144, 1024, 64), (6144, 1024, 448),
                                   (6144, 1152, 4096)])
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32], ids=["bf16", "fp32"])
def test_gemm_with_a_workspace_is_bit_identical(shape, out_dtype):
    """The two-pass form (W converted once into a bf16 panel in the caller's workspace) feeds the MFMAs the same operand
    values in the same order as the fused kernel: equal bits, and the oracle's tolerance on a sample of rows."""
    M, N, K = shape
    say("gemm workspace", shape, out_dtype)
    g = torch.Generator(device=DEV).manual_seed(M + N + K)
    w = torch.randn(1, 1, K, N, generator=g, device=DEV) * 0.02
    x = torch.randn(M, K, generator=g, device=DEV).bfloat16()
    bias = (torch.randn(N, generator=g, device=DEV) * 0.02).bfloat16()
    wp = capi.tilize_pack(w, F.Bfp8_b)
    need = capi.gemm_workspace_bytes(M, N, K)
    assert need == 2 * K * N
    ws = torch.empty(need, dtype=torch.uint8, device=DEV)
    for epi, b in ((capi.EPILOGUE_NONE, None), (capi.EPILOGUE_GELU, bias), (capi.EPILOGUE_GELU_TANH, bias)):
        fused = capi.gemm_bfp8b(x, wp, N, bias=b, epilogue=epi, out_dtype=out_dtype)
        two = capi.gemm_bfp8b(x, wp, N, bias=b, epilogue=epi, out_dtype=out_dtype, workspace=ws)
        if K % 128 == 0 and (M // 128) * (N // 128) <= 256:
            # the fused kernel adds the two halves of K in workgroups with two pipelines: the same products, another order of
            # the fp32 additions
            assert rel_fro(fused.float().cpu(), two.float().cpu()) < (1e-6 if out_dtype == torch.float32 else 2e-4)
        else:
            assert torch.equal(fused, two)
    # a workspace that is too small, or a shape that does not qualify, falls back to the fused kernel
    small = capi.gemm_bfp8b(x, wp, N, out_dtype=out_dtype, workspace=ws[:need - 16])
    assert torch.equal(small, capi.gemm_bfp8b(x, wp, N, out_dtype=out_dtype))
    assert capi.gemm_workspace_bytes(128, 4096, 4096) == 0 and capi.gemm_workspace_bytes(4096, 3072, 96) == 0
    if K <= 320:  # against dequantize-then-matmul in fp32 on a few rows
        rows = torch.arange(0, M, M // 8, device=DEV)
        wd = capi.unpack_untilize(wp, F.Bfp8_b, (1, 1, K, N))[0, 0]
        ref = x[rows].float() @ wd
        got = capi.gemm_bfp8b(x, wp, N, out_dtype=torch.float32, workspace=ws)[rows]
        assert float((got - ref).norm() / ref.norm()) < 1e-5


@pytest.mark.parametrize("shape", [(256, 4096, 4096), (256, 1024, 4096), (1024, 1024, 4096), (512, 1024, 4096), (384, 1024, 8192),
                                   (256, 512, 2048), (256, 512, 2560),  # these two: runs of four and of five (an odd number of) slabs
                                   (128, 1024, 4096), (128, 2048, 8192)])  # one tile row: instead of the weight-streaming kernel
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32], ids=["bf16", "fp32"])
def test_gemm_split_over_k_with_a_workspace(shape, out_dtype):
    """Shapes whose 128 x 128 tiles leave CUs idle: with a workspace K is cut into runs whose fp32 partial tiles are added
    in a fixed order by a second kernel.  The sum is grouped differently from the fused kernel's, so the bar is the
    oracle's tolerance against dequantize-then-fp32-matmul, and two calls must agree bit for bit."""
    M, N, K = shape
    say("gemm split k", shape, out_dtype)
    g = torch.Generator(device=DEV).manual_seed(M + N + K)
    w = torch.randn(1, 1, K, N, generator=g, device=DEV) * 0.02
    x = torch.randn(M, K, generator=g, device=DEV).bfloat16()
    bias = (torch.randn(N, generator=g, device=DEV) * 0.02).bfloat16()
    wp = capi.tilize_pack(w, F.Bfp8_b)
    need = capi.gemm_workspace_bytes(M, N, K)
    splits = need // (M * N * 4)
    assert need > 0 and need == splits * M * N * 4 and 2 <= splits <= 8 and (M // 128) * (N // 128) * splits <= 512
    ws = torch.full((need,), 0xFF, dtype=torch.uint8, device=DEV)  # NaN patterns: every partial must be written before it is read
    wd = capi.unpack_untilize(wp, F.Bfp8_b, (1, 1, K, N))[0, 0]
    base = x.float() @ wd
    bias32 = bias.float() * 2 + 1e-3  # an fp32 bias that is no bf16 value
    for epi, b in ((capi.EPILOGUE_NONE, None), (capi.EPILOGUE_NONE, bias), (capi.EPILOGUE_GELU, bias), (capi.EPILOGUE_GELU_TANH, bias),
                   (capi.EPILOGUE_GELU, bias32)):
        want = base + (b.float() if b is not None else 0.0)
        if epi != capi.EPILOGUE_NONE:
            want = torch.nn.functional.gelu(want, approximate="tanh" if epi == capi.EPILOGUE_GELU_TANH else "none")
        got = capi.gemm_bfp8b(x, wp, N, bias=b, epilogue=epi, out_dtype=out_dtype, workspace=ws)
        again = capi.gemm_bfp8b(x, wp, N, bias=b, epilogue=epi, out_dtype=out_dtype, workspace=ws)
        assert torch.equal(got, again)
        if out_dtype == torch.float32:
            assert float((got - want).norm() / want.norm()) < 1e-5
        else:
            assert float((got.float() - want.bfloat16().float()).norm() / want.norm()) < 1e-3
        fused = capi.gemm_bfp8b(x, wp, N, bias=b, epilogue=epi, out_dtype=torch.float32)
        if out_dtype == torch.float32:
            assert float((got - fused).norm() / fused.norm()) < 1e-6
    # too small a workspace: the fused kernel runs
    small = capi.gemm_bfp8b(x, wp, N, out_dtype=out_dtype, workspace=ws[:need - 16])
    assert torch.equal(small, capi.gemm_bfp8b(x, wp, N, out_dtype=out_dtype))


def test_gelu_tanh_form_through_the_op_layer():
    """`approximate="tanh"` (pybuda/pybuda/op/eval/pybuda/eltwise_unary.py:45-47) against the reference's formula written
    out in float64, on values that reach both tails; any other mode raises as it does there."""
    import math
    from tt_buda_amd import op
    say("gelu tanh op layer")
    K, N = 32, 64
    w = torch.zeros(K, N)
    w[0, :] = 1.0  # Y[m, n] = X[m, 0]: the epilogue sees the activations themselves
    x = torch.zeros(64, K)
    x[:, 0] = torch.linspace(-12.0, 12.0, 64)
    x = x.bfloat16()
    got = op.matmul(x, op.BfpWeight(w), gelu="tanh", out_dtype=torch.float32).cpu().double()
    v = x[:, 0:1].double().expand(64, N)
    want = 0.5 * v * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (v + 0.044715 * torch.pow(v, 3.0))))
    # the exponent of the far negative tail carries the fp32 rounding of u times |2u|: a few 1e-6 relative
    assert torch.allclose(got, want, rtol=1e-5, atol=1e-12), float((got - want).abs().max())
    exact = op.matmul(x, op.BfpWeight(w), gelu="none", out_dtype=torch.float32).cpu()
    assert torch.equal(exact, op.matmul(x, op.BfpWeight(w), gelu=True, out_dtype=torch.float32).cpu())
    assert not torch.equal(exact.double(), got)
    with pytest.raises(RuntimeError, match="does not support"):
        op.matmul(x, op.BfpWeight(w), gelu="quick")


def test_entry_points_replay_from_a_hip_graph():
    """The conversion and GEMM entry points only launch kernels on the caller's stream (no allocation, no wait, no memset),
    so a serving loop may record them into a HIP graph once and replay it.  Several replays, with new inputs written and
    the outputs cleared by eager work in between, each checked bit for bit against the eager calls on the same inputs."""
    say("hip graph replay")
    shape = (1, 2, 256, 512)
    M, K, N = 256, 4096, 1024  # with a workspace this shape is split over K
    g = torch.Generator(device=DEV).manual_seed(77)
    x = torch.empty(shape, dtype=torch.bfloat16, device=DEV)
    a = torch.empty((M, K), dtype=torch.bfloat16, device=DEV)
    a32 = torch.empty((32, K), dtype=torch.bfloat16, device=DEV)
    wp = capi.tilize_pack(torch.randn(1, 1, K, N, generator=g, device=DEV) * 0.02, F.Bfp8_b)
    bias = (torch.randn(N, generator=g, device=DEV) * 0.02).bfloat16()
    need = capi.gemm_workspace_bytes(M, N, K)
    assert need > 0
    ws = torch.empty(need, dtype=torch.uint8, device=DEV)
    packed = torch.empty(capi.packed_size(F.Bfp4_b, shape), dtype=torch.uint8, device=DEV)
    back = torch.empty(shape, dtype=torch.float32, device=DEV)
    y = torch.empty((M, N), dtype=torch.bfloat16, device=DEV)
    y_ws = torch.empty((M, N), dtype=torch.float32, device=DEV)
    y32 = torch.empty((32, N), dtype=torch.bfloat16, device=DEV)
    outs = (packed, back, y, y_ws, y32)

    def fill(seed):
        gg = torch.Generator(device=DEV).manual_seed(seed)
        x.copy_((torch.randn(shape, generator=gg, device=DEV) * 3).bfloat16())
        a.copy_(torch.randn((M, K), generator=gg, device=DEV).bfloat16())
        a32.copy_(torch.randn((32, K), generator=gg, device=DEV).bfloat16())

    def work():
        capi.tilize_pack(x, F.Bfp4_b, capi.ROUND_NEAREST, out=packed)
        capi.unpack_untilize(packed, F.Bfp4_b, shape, out=back)
        capi.gemm_bfp8b(a, wp, N, bias=bias, epilogue=capi.EPILOGUE_GELU, out=y)
        capi.gemm_bfp8b(a, wp, N, bias=bias, epilogue=capi.EPILOGUE_GELU_TANH, out=y_ws, workspace=ws)
        capi.gemm_bfp8b(a32, wp, N, out=y32)

    fill(1)
    work()  # the first calls also set kernel attributes once; that must not fall into the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        work()
    for seed in (2, 3, 4):
        fill(seed)
        work()
        torch.cuda.synchronize()
        want = [o.clone() for o in outs]
        for o in outs:
            o.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for o, wnt in zip(outs, want):
            assert torch.equal(o, wnt), seed
        assert float(back.abs().max()) > 0 and float(y_ws.abs().max()) > 0


@pytest.mark.parametrize("dtype,fmt", [(torch.float32, F.Float32), (torch.bfloat16, F.Float16_b), (torch.float32, F.Bfp4_b), (torch.bfloat16, F.Bfp2_b)],
                         ids=["fp32_tiles", "bf16_tiles", "fp32_bfp4b", "bf16_bfp2b"])
def test_large_grids_of_every_tile_size(dtype, fmt):
    """Grids of 8192 workgroups and more are launched with extra dynamic LDS that caps the workgroups per CU; the amount
    depends on the tile size.  Plain tiles are a pure permutation (the view/permute statement of the tile order), packed
    ones must round-trip idempotently and agree with the oracle on a slice."""
    say("large grid", dtype, fmt)
    shape = (2, 1, 8192, 8192) if dtype == torch.float32 else (4, 1, 8192, 8192)
    g = torch.Generator(device=DEV).manual_seed(99)
    x = torch.randn(shape, generator=g, device=DEV).to(dtype)
    packed = capi.tilize_pack(x, fmt)
    back = capi.unpack_untilize(packed, fmt, shape, dtype)
    if fmt in (F.Float32, F.Float16_b):
        W, Z, R, C = shape
        tiles = x.view(W, Z, R // 32, 2, 16, C // 32, 2, 16).permute(0, 1, 2, 5, 3, 6, 4, 7).contiguous()
        assert torch.equal(packed.view(dtype).view(-1), tiles.view(-1))
        assert torch.equal(back, x)
    else:
        again = capi.tilize_pack(back, fmt)
        assert torch.equal(again, packed)  # pack o unpack o pack = pack
        rows = slice(4096, 4096 + 64)
        want = O.tilize_pack(x[1:2, :, rows].float().cpu().numpy() if dtype == torch.float32 else
                             x[1:2, :, rows].view(torch.int16).cpu().numpy().view(np.uint16), int(fmt), nthreads=8)
        per_row_of_tiles = (shape[3] // 32) * (packed.numel() // (shape[0] * shape[2] // 32 * (shape[3] // 32)))
        first = (1 * (shape[2] // 32) + 4096 // 32) * per_row_of_tiles
        assert np.array_equal(packed[first:first + want.size].cpu().numpy(), want.reshape(-1))


def test_large_grid_with_a_partial_last_segment():
    """8224 columns = 257 tiles: the last segment of every band holds one tile, so most lanes of its workgroup lie past the
    last column (they re-fetch the row's last chunk and store nothing) and the unpack kernel takes its rolled load loop -
    on a grid large enough for the capped residency.  Bytes against the oracle on two row bands, and the round trip."""
    say("large grid, ragged columns")
    shape = (1, 1, 16384, 8224)
    g = torch.Generator(device=DEV).manual_seed(123)
    x = (torch.randn(shape, generator=g, device=DEV) * 4).bfloat16()
    packed = capi.tilize_pack(x, F.Bfp8_b)
    back = capi.unpack_untilize(packed, F.Bfp8_b, shape, torch.bfloat16)
    band_bytes = (shape[3] // 32) * 1088
    for r0 in (0, 16384 - 32):
        rows = x[:, :, r0:r0 + 32].view(torch.int16).cpu().numpy().view(np.uint16)
        want = O.tilize_pack(rows, O.Bfp8_b)
        got = packed[(r0 // 32) * band_bytes:(r0 // 32 + 1) * band_bytes].cpu().numpy()
        assert np.array_equal(got, want.reshape(-1)), r0
        want_back = O.unpack_untilize(want, O.Bfp8_b, (1, 1, 32, shape[3]), O.Float16_b)
        assert np.array_equal(back[:, :, r0:r0 + 32].view(torch.int16).cpu().numpy().view(np.uint16), want_back), r0
    assert torch.equal(capi.tilize_pack(back, F.Bfp8_b), packed)
