"""Runtime I/O on top of the pybind boundary: the push/read/pop loops pybuda keeps in
``BackendAPI`` (``pybuda/pybuda/backend.py:326-456``), against queues that live in MI355X HBM."""
from typing import List, Optional, Sequence, Tuple, Union

import torch

from ._C import DataFormat
from ._C.backend_api import (BackendApi, BackendConfig, BackendDevice, BackendStatusCode, BackendType, DeviceMode, DramIODesc, IOType,
                             PytorchTensorDesc, TilizedTensorDesc, free_tensor, get_output, last_error, pop_output, push_input,
                             translate_addresses)
from .tensor import (convert_tensor_for_tilize, narrow_buda_tensor_to_pytorch, pad_pytorch_tensor_to_buda,
                     pytorch_tensor_to_tensor_desc, tensor_desc_to_pytorch_tensor)


class BackendAPI:
    """Owns one device backend and moves tensors in and out of its queues."""

    def __init__(self, device: int = 0, golden_ignore_df_precision: bool = False, opt_level: int = 0, output_dir: str = "",
                 performance_trace: str = "", runtime_args: str = ""):
        """``golden_ignore_df_precision`` is the reference's switch of the same name (pybuda/pybuda/backend.py:46,78,
        pybuda/pybuda/verify/config.py:67,166-167): False keeps every queue quantized to its DataFormat, True keeps queues in
        full precision and evaluates the matmul in fp32.  The environment variable TT_BACKEND_GOLDEN_QUANTIZE forces False, as
        it does there."""
        import os
        if "TT_BACKEND_GOLDEN_QUANTIZE" in os.environ:
            golden_ignore_df_precision = False
        bcfg = BackendConfig(BackendType.Hip, BackendDevice.MI355X, DeviceMode.CompileAndRun, opt_level, output_dir, "", "")
        bcfg.set_golden_ignore_df_precision(golden_ignore_df_precision)
        bcfg.set_performance_trace_args(performance_trace)
        bcfg.set_runtime_args(runtime_args)
        self.be_api = BackendApi(device, bcfg)
        status = self.be_api.initialize()
        if status != BackendStatusCode.Success:
            raise RuntimeError("Failed to initialize the backend: " + last_error())

    def shutdown(self):
        if self.be_api is not None:
            self.be_api.finish()
            self.be_api = None

    def create_queue(self, name: str, data_format: DataFormat, shape: Sequence[int], num_slots: int = 2,
                     io_type: IOType = IOType.Queue, input_count: int = 1, grid: Sequence[int] = (1, 1),
                     ublock: Sequence[int] = (1, 1), ublock_order: str = "r", tile_header: bool = False) -> DramIODesc:
        """Queue whose entries are ``shape = (t, rows, cols)`` with rows/cols multiples of 32, cut over ``grid`` buffers of
        macro blocks of ``ublock``-sized micro blocks (the netlist queue line's grid_size / mblock / ublock / ublock_order,
        pybuda/csrc/lower_to_buda/queue.cpp:11-67).  The defaults give one buffer of row-major tiles."""
        t, rows, cols = shape
        assert rows % 32 == 0 and cols % 32 == 0, "queue rows/cols must be tile aligned"
        assert ublock_order in ("r", "c"), "ublock_order is 'r' or 'c'"
        rt, ct = rows // 32, cols // 32
        assert rt % (grid[0] * ublock[0]) == 0 and ct % (grid[1] * ublock[1]) == 0, "grid x ublock must divide the entry's tiles"
        return self.be_api.create_queue(name, data_format, t, rt // (grid[0] * ublock[0]), ct // (grid[1] * ublock[1]), ublock[0],
                                        ublock[1], num_slots, io_type, input_count, grid[0], grid[1], int(ublock_order == "c"),
                                        tile_header)

    def get_ordered_queues(self, names: List[str]) -> List[DramIODesc]:
        out = []
        for name in names:
            desc = self.be_api.get_queue_descriptor(name)
            assert translate_addresses(desc) == BackendStatusCode.Success, f"Failed to translate addresses: {desc.name}"
            out.append(desc)
        return out

    @classmethod
    def push_input(cls, queue_desc: DramIODesc, tensor_desc: Union[PytorchTensorDesc, TilizedTensorDesc],
                   single_input: bool = True, timeout_secs: int = 1, ram_address: int = 0,
                   tile_broadcast_r: bool = False, tile_broadcast_c: bool = False):
        if isinstance(tensor_desc, TilizedTensorDesc):
            status = push_input(queue_desc, tensor_desc, timeout_secs, ram_address)
            assert status == BackendStatusCode.Success, "Error while pushing tilized inputs: " + last_error()
        else:
            status = push_input(queue_desc, tensor_desc, single_input, timeout_secs, ram_address, tile_broadcast_r, tile_broadcast_c)
            assert status == BackendStatusCode.Success, "Error while pushing inputs: " + last_error()

    @classmethod
    def push_to_queues(cls, ordered_input_queues: List[DramIODesc], tensors: List[torch.Tensor], single_input: bool,
                       tile_broadcast_dims: Optional[List[Sequence[int]]] = None):
        """Legalise dtype, describe, push: the direct-pusher path (pybuda/pybuda/device_connector.py:228-311).  Where the
        reference pads rows and columns to whole tiles on the host first (``pad_pytorch_tensor_to_buda``: zeros, or copies
        of a dimension of one listed in that input's ``tile_broadcast_dims``), the tensor goes to the backend as it is and
        the pack launch pads it."""
        assert len(tensors) == len(ordered_input_queues), (
            f"Incorrect number of tensors provided on input: tensors:{len(tensors)} vs "
            f"ordered_input_queues:{len(ordered_input_queues)}")
        for i, (q, t) in enumerate(zip(ordered_input_queues, tensors)):
            bcast_r = bcast_c = False
            if not isinstance(t, (PytorchTensorDesc, TilizedTensorDesc)):
                dims = tile_broadcast_dims[i] if tile_broadcast_dims else []
                bcast_c = -1 in dims or 3 in dims
                bcast_r = -2 in dims or 2 in dims
                t = convert_tensor_for_tilize(t, q.data_format)
                if t.dim() == 0:
                    t = t.reshape(1, 1, 1, 1)
                while t.dim() < 4:  # the rank rule of pad_pytorch_tensor_to_buda for a microbatch of one
                    t = t.unsqueeze(1 if t.shape[0] == 1 else 0)
                if bcast_c:
                    assert t.shape[-1] == 1, "Trying to broadcast to tile dim a dimension that's not 1"
                if bcast_r:
                    assert t.shape[-2] == 1, "Trying to broadcast to tile dim a dimension that's not 1"
                t = pytorch_tensor_to_tensor_desc(t)
            cls.push_input(q, t, single_input, 1, -1, bcast_r, bcast_c)

    @classmethod
    def read_queues(cls, queues: List[DramIODesc], original_shapes: List[Tuple[int, ...]], single_output: bool,
                    rd_ptr: int = -1, shutdown_event=None, clone: bool = True, has_microbatch_dim: bool = True,
                    fp32_output: bool = False) -> List[torch.Tensor]:
        """get_output with the reference's retry-on-timeout policy (backend.py:346-371), then view,
        narrow to the original shape, clone and free.  Where the original rows and columns only need the tile padding cut off
        (the common case of ``narrow_buda_tensor_to_pytorch``), the unpack launch writes just that corner and only it is
        copied back; the general narrowing then has nothing left to cut."""
        ret = []
        for outq, shape in zip(queues, original_shapes):
            out_desc = PytorchTensorDesc()
            if fp32_output:
                out_desc.format = DataFormat.Float32
            narrow_r = narrow_c = 0
            rows, cols = outq.bufq_grid_dim_r * outq.mblock_m * outq.ublock_rt * 32, outq.bufq_grid_dim_c * outq.mblock_n * outq.ublock_ct * 32
            if shape is not None and len(shape) >= 2 and outq.hstack_factor <= 1 and outq.vstack_factor <= 1:
                r, c = int(shape[-2]), int(shape[-1])
                if 0 < r <= rows and 0 < c <= cols and (r + 31) // 32 * 32 == rows and (c + 31) // 32 * 32 == cols and (r, c) != (rows, cols):
                    narrow_r, narrow_c = r, c
            resp = BackendStatusCode.RuntimeError
            for _ in range(10):
                resp = get_output(outq, out_desc, single_output, 1, rd_ptr, narrow_r, narrow_c)
                if resp != BackendStatusCode.TimeoutError:
                    break
                if shutdown_event is not None and shutdown_event.is_set():
                    break
            if resp == BackendStatusCode.TimeoutError:
                if shutdown_event is not None:
                    shutdown_event.set()
                raise RuntimeError("Timeout while reading " + outq.name)
            assert resp == BackendStatusCode.Success, "Error while reading output: " + last_error()
            t = tensor_desc_to_pytorch_tensor(out_desc)
            if shape is not None:
                t = narrow_buda_tensor_to_pytorch(t, list(shape), has_microbatch_dim=has_microbatch_dim)
            if clone:
                t = t.clone()
                free_tensor(out_desc)
            ret.append(t)
        return ret

    @classmethod
    def pop_queues(cls, queues: List[DramIODesc], single_output: bool):
        for outq in queues:
            assert pop_output(outq, single_output, 1) == BackendStatusCode.Success, "Error while popping output"
