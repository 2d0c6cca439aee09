"""Padding to whole tiles and narrowing back, inside the pack / unpack launches (``ttbfp_tilize_pack_padded``,
``ttbfp_unpack_untilize_narrow``), against the reference's host-side statement of the same thing:
``pad_pytorch_tensor_to_buda`` pads rows and columns with ``torch.nn.functional.pad`` in "constant" mode, or "replicate"
for a dimension of one that is broadcast to its tile (pybuda/pybuda/tensor.py:805-877); ``narrow_buda_tensor_to_pytorch``
takes the corner back out (tensor.py:879-954).  Expected bytes = the oracle's packing of the numpy-padded tensor."""
import sys

import numpy as np
import pytest
import torch

import oracle as O
from tt_buda_amd import capi

pytestmark = pytest.mark.gpu

F = capi.DataFormatCode
DEV = "cuda:0"


def say(*a):
    print("[case]", *a, flush=True)
    sys.stdout.flush()


def np_pad(a, rep_r, rep_c):
    r, c = a.shape[2], a.shape[3]
    pr, pc = (-r) % 32, (-c) % 32
    a = np.pad(a, ((0, 0), (0, 0), (0, 0), (0, pc)), mode="edge" if rep_c else "constant")
    return np.pad(a, ((0, 0), (0, 0), (0, pr), (0, 0)), mode="edge" if rep_r else "constant")


def as_source(x):
    """device tensor -> what the oracle takes: fp32 array, or uint16 bf16 bits"""
    if x.dtype == torch.bfloat16:
        return x.cpu().view(torch.int16).numpy().view(np.uint16)
    return x.cpu().numpy()


# shape, dtype, replicate rows, replicate cols.  Row strides of 280 and 2 bytes take the general kernel; 1536, 144 and 192
# bytes the fast one (rows past the end; columns past the end in whole 16-byte chunks; a replicated single row).
CASES = [((1, 3, 50, 70), torch.float32, False, False),
         ((2, 1, 1028, 384), torch.float32, False, False),
         ((1, 2, 40, 72), torch.bfloat16, False, False),
         ((3, 1, 33, 520), torch.bfloat16, False, False),
         ((1, 2, 1, 96), torch.bfloat16, True, False),
         ((1, 1, 1, 44), torch.float32, True, False),
         ((2, 1, 64, 1), torch.float32, False, True),
         ((1, 1, 1, 1), torch.bfloat16, True, True),
         ((1, 1, 1, 1), torch.float32, False, False)]


@pytest.mark.parametrize("fmt", [F.Bfp8_b, F.Bfp4_b, F.Bfp2_b, F.Float16_b])
@pytest.mark.parametrize("case", CASES, ids=[f"{'x'.join(map(str, c[0]))}-{str(c[1])[6:]}-{int(c[2])}{int(c[3])}" for c in CASES])
def test_pack_pads_and_unpack_narrows_inside_the_launch(case, fmt):
    shape, dtype, rep_r, rep_c = case
    say("pad/narrow", shape, dtype, rep_r, rep_c, fmt)
    g = torch.Generator(device=DEV).manual_seed(sum(shape) + fmt)
    x = (torch.randn(shape, generator=g, device=DEV) * 3).to(dtype)
    padded = np_pad(as_source(x), rep_r, rep_c)
    tiled = tuple(padded.shape)
    for rounding in (capi.ROUND_TRUNCATE, capi.ROUND_NEAREST):
        want = O.tilize_pack(padded, int(fmt), rounding)
        got = capi.tilize_pack_padded(x, fmt, rep_r, rep_c, rounding)
        assert got.numel() == capi.packed_size(fmt, tiled)
        assert np.array_equal(got.cpu().numpy(), want.reshape(-1)), np.flatnonzero(got.cpu().numpy() != want.reshape(-1))[:8]
    # the same bytes as padding on the host and packing the tile-aligned tensor
    host_padded = torch.from_numpy(padded.view(np.int16) if dtype == torch.bfloat16 else padded).to(DEV)
    if dtype == torch.bfloat16:
        host_padded = host_padded.view(torch.bfloat16)
    packed = capi.tilize_pack_padded(x, fmt, rep_r, rep_c)
    assert torch.equal(packed, capi.tilize_pack(host_padded, fmt))
    # narrowing: the corner of the full read-back, nothing outside it touched
    for out_dtype in (torch.float32, torch.bfloat16):
        full = capi.unpack_untilize(packed, fmt, tiled, out_dtype)
        canvas = torch.full(tiled, -7.0, dtype=out_dtype, device=DEV)
        view = canvas[:, :, :shape[2], :shape[3]]
        capi.unpack_untilize_narrow(packed, fmt, shape, out=view)
        assert torch.equal(view, full[:, :, :shape[2], :shape[3]])
        untouched = canvas.clone()
        untouched[:, :, :shape[2], :shape[3]] = -7.0
        assert bool((untouched == -7.0).all())
        tight = capi.unpack_untilize_narrow(packed, fmt, shape, out_dtype)  # a contiguous result of the logical shape
        assert tight.shape == tuple(shape) and torch.equal(tight, full[:, :, :shape[2], :shape[3]])


def test_pad_and_narrow_into_the_buffers_of_a_queue():
    """The padded pack with a queue geometry (grid 2 x 3 of 1 x 2-tile micro blocks, column-major, with tile headers)."""
    say("pad/narrow queue")
    shape = (2, 2, 100, 370)  # tiles: 4 x 12
    lay = capi.QueueLayout(2, 3, 2, 2, 1, 2, 1, 1)
    g = torch.Generator(device=DEV).manual_seed(5)
    x = torch.randn(shape, generator=g, device=DEV)
    padded = torch.zeros((2, 2, 128, 384), device=DEV)
    padded[:, :, :100, :370] = x
    want = capi.tilize_pack_queue(padded, F.Bfp8_b, lay)
    got = capi.tilize_pack_padded(x, F.Bfp8_b, layout=lay)
    assert torch.equal(got, want)
    back = capi.unpack_untilize_narrow(got, F.Bfp8_b, shape, torch.float32, layout=lay)
    assert torch.equal(back, capi.unpack_untilize_queue(want, F.Bfp8_b, (2, 2, 128, 384), lay)[:, :, :100, :370])


def test_pad_argument_errors():
    x = torch.zeros(1, 1, 5, 7, device=DEV)
    with pytest.raises(capi.BackendError, match="only a dimension of size 1"):
        capi.tilize_pack_padded(x, F.Bfp8_b, replicate_rows=True)
    with pytest.raises(capi.BackendError, match="only a dimension of size 1"):
        capi.tilize_pack_padded(x, F.Bfp8_b, replicate_cols=True)
    with pytest.raises(capi.BackendError, match="needed"):
        capi.tilize_pack_padded(x, F.Bfp8_b, out=torch.empty(1087, dtype=torch.uint8, device=DEV))
