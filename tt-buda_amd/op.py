"""Matmul / GELU / FFN with Bfp8_b weights on device tensors.

Semantics follow the golden evaluation (``pybuda/pybuda/op/eval/buda/matmul.py:233-249``:
``matmul(a, b)`` plus the first row of a tile-padded bias; ``op/eval/pybuda/eltwise_unary.py:42-49``:
GELU in its exact or its tanh form; FFN structure ``pybuda/test/bert/modules.py:133-158``), evaluated by the HIP GEMM with
the weight operand in Bfp8_b tiles.
"""
from typing import Optional

import torch

from . import capi

F = capi.DataFormatCode


class BfpWeight:
    """A weight ``[K, N]``, or a stack ``[Z, K, N]`` / ``[1, Z, K, N]`` of them, resident in HBM as Bfp8_b tiles.

    Tiles lie in ``[z][tile_row][tile_col]`` order, so the packed bytes of a stack are also those of the one matrix
    ``[Z K, N]`` made by setting its members on top of each other, which is what ``matmul(..., accumulate=True)`` uses."""

    def __init__(self, w: torch.Tensor, rounding: int = capi.ROUND_TRUNCATE):
        assert w.dim() in (2, 3, 4) and w.shape[-2] % 32 == 0 and w.shape[-1] % 32 == 0, "weights must be [.., K, N], tile aligned"
        assert w.dim() < 4 or w.shape[0] == 1, "one stack of matrices ([1, Z, K, N])"
        assert w.dtype in (torch.float32, torch.bfloat16)
        self.K, self.N = w.shape[-2:]
        self.Z = w.shape[-3] if w.dim() >= 3 else 1
        self.packed = capi.tilize_pack(w.cuda().reshape(1, self.Z, self.K, self.N), F.Bfp8_b, rounding)

    def dequantize(self, dtype=torch.float32) -> torch.Tensor:
        w = capi.unpack_untilize(self.packed, F.Bfp8_b, (1, self.Z, self.K, self.N), dtype)
        return w.view(self.K, self.N) if self.Z == 1 else w.view(self.Z, self.K, self.N)

    def member(self, z: int) -> torch.Tensor:
        """The packed tiles of matrix ``z`` of the stack (a view)."""
        n = self.packed.numel() // self.Z
        return self.packed[z * n:(z + 1) * n]


def _bias_row(bias: Optional[torch.Tensor], N: int) -> Optional[torch.Tensor]:
    if bias is None:
        return None
    if bias.dim() > 1:  # tile-padded 4-D bias: the reference adds bias[:, :, 0:1, :]
        bias = bias.reshape(-1, bias.shape[-1])[0]
    assert bias.numel() == N
    return bias.to(device="cuda", dtype=torch.bfloat16).contiguous()


def _epilogue(gelu) -> int:
    """``gelu``: False / True (exact form), or the reference's ``approximate`` attribute, "none" or "tanh"
    (``op/eval/pybuda/eltwise_unary.py:42-49``; any other string raises as it does there)."""
    if gelu is False or gelu is None:
        return capi.EPILOGUE_NONE
    if gelu is True or gelu == "none":
        return capi.EPILOGUE_GELU
    if gelu == "tanh":
        return capi.EPILOGUE_GELU_TANH
    raise RuntimeError(f"Gelu does not support {gelu} approximation mode.")


def matmul(x: torch.Tensor, w: BfpWeight, bias: Optional[torch.Tensor] = None, gelu=False,
           out_dtype=torch.bfloat16, accumulate: bool = False) -> torch.Tensor:
    """``x @ dequant(w) (+ bias row) (-> GELU)``; ``gelu``: see ``_epilogue``.

    One matrix (``w.Z == 1``): leading dims of ``x`` are flattened into M.  A stack (``w.Z > 1``): ``x`` is
    ``[.., Z, M, K]`` and member z multiplies ``x[.., z, :, :]``, as ``torch.matmul`` pairs them in the golden
    evaluation; with ``accumulate`` (first attribute of the reference's matmul, ``op/eval/buda/matmul.py:236,306-307``) the
    products are summed over z with ``keepdim``, which is the single product ``[M, Z K] x [Z K, N]`` and runs as one GEMM
    with fp32 accumulation over all of it."""
    epilogue = _epilogue(gelu)
    if w.Z == 1:
        assert not accumulate or x.dim() < 3 or x.shape[-3] == 1, "accumulate sums over the z of a weight stack"
        lead = x.shape[:-1]
        x2 = x.reshape(-1, x.shape[-1]).to(device="cuda", dtype=torch.bfloat16).contiguous()
        assert x2.shape[1] == w.K and x2.shape[0] % 32 == 0, "activations must be [.., K] with a tile-aligned row count"
        y = capi.gemm_bfp8b(x2, w.packed, w.N, bias=_bias_row(bias, w.N), epilogue=epilogue, out_dtype=out_dtype)
        return y.view(*lead, w.N)
    assert x.dim() >= 3 and x.shape[-3] == w.Z and x.shape[-1] == w.K and x.shape[-2] % 32 == 0, "activations must be [.., Z, M, K]"
    assert x.dim() == 3 or all(d == 1 for d in x.shape[:-3]), "one stack of activations"
    M = x.shape[-2]
    xs = x.reshape(w.Z, M, w.K).to(device="cuda", dtype=torch.bfloat16)
    brow = _bias_row(bias, w.N)
    if accumulate:
        # sum_z (x_z w_z + b) = [x_0 .. x_{Z-1}] [w_0; ..; w_{Z-1}] + Z b; Z b is not a bf16 value in general, so it rides in the
        # GEMM's epilogue as an fp32 bias
        x2 = xs.permute(1, 0, 2).reshape(M, w.Z * w.K).contiguous()
        total = None if brow is None else (brow.float() * w.Z).contiguous()
        y = capi.gemm_bfp8b(x2, w.packed, w.N, bias=total, epilogue=epilogue, out_dtype=out_dtype)
        return y.view(*x.shape[:-3], 1, M, w.N)
    y = torch.empty((w.Z, M, w.N), dtype=out_dtype, device="cuda")
    for z in range(w.Z):
        capi.gemm_bfp8b(xs[z].contiguous(), w.member(z), w.N, bias=brow, epilogue=epilogue, out=y[z])
    return y.view(*x.shape[:-1], w.N)


def ffn(x: torch.Tensor, w1: BfpWeight, b1: torch.Tensor, w2: BfpWeight, b2: torch.Tensor,
        out_dtype=torch.bfloat16, gelu="none") -> torch.Tensor:
    """``GELU(x W1 + b1) W2 + b2`` with a bf16 intermediate, as two device matmuls would leave it."""
    return matmul(matmul(x, w1, b1, gelu=gelu), w2, b2, out_dtype=out_dtype)
