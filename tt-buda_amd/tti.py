"""Tensor entries of a saved device image: the ``device.json`` side of ``.bin`` / ``.tbin`` payloads.

pybuda saves every parameter and constant of a compiled model next to a JSON entry that says how to read it back
(``pybuda/pybuda/tti/archive.py:52-147``; formats ``pybuda/pybuda/config.py:121-144``): with the ``BACKEND`` dump format
the row-major bytes (``.bin``), with ``BACKEND_TILIZED`` the tiles ``tilize_tensor`` makes for the tensor's queue
(``.tbin``), so that a reload pushes pre-packed weights without converting them again.  The entry's keys are
``bin, itemsize, shape, strides, dim, format`` plus, for tiles, ``num_buffers, buf_size_bytes`` (``format`` is then the
tiles' format).  Names and keys follow the reference; the payloads go through this backend's ``binarize_tensor`` /
``debinarize_tensor``.  Only tensor entries are handled: the rest of a device image (compiled graph state, netlists,
device configuration) belongs to the compiler.
"""
import functools
import json
import os
from enum import Enum
from typing import Any, Callable, Dict, Optional

import torch

from ._C import DataFormat
from ._C.backend_api import PytorchTensorDesc, TilizedTensorDesc, binarize_tensor, debinarize_tensor, free_tensor, tilize_tensor
from .tensor import pytorch_tensor_to_tensor_desc

TTI_VERSION = "1.1.0"  # the version from which tensors are stored through the backend (pybuda/pybuda/tti/tti.py:37)


class TTIDumpFormat(Enum):
    """Serialization of tensor data in a device image (pybuda/pybuda/config.py:121-144)."""

    DEFAULT = "DEFAULT"
    BACKEND = "BACKEND"
    BACKEND_TILIZED = "BACKEND_TILIZED"

    def extension(self) -> str:
        return {TTIDumpFormat.DEFAULT: "pkl", TTIDumpFormat.BACKEND: "bin", TTIDumpFormat.BACKEND_TILIZED: "tbin"}[self]

    @classmethod
    def to_json(cls, value):
        return value.name

    @classmethod
    def from_json(cls, value):
        return cls[value.upper()]


def load_tensor_from_disk(filepath: str, value: Dict[str, Any]):
    """JSON entry + payload file -> a descriptor that ``push_input`` takes: a ``TilizedTensorDesc`` for ``.tbin``, a
    ``PytorchTensorDesc`` otherwise (archive.py:52-66).  The payload lands in backend-owned memory: ``free_tensor`` it."""
    if filepath.endswith(TTIDumpFormat.BACKEND_TILIZED.extension()):
        desc = TilizedTensorDesc()
        desc.format = DataFormat.from_json(value["format"])
        desc.num_buffers = value["num_buffers"]
        desc.buf_size_bytes = value["buf_size_bytes"]
    else:
        desc = PytorchTensorDesc()
        desc.itemsize = value["itemsize"]
        desc.format = DataFormat.from_json(value["format"])
        desc.shape = value["shape"]
        desc.strides = value["strides"]
        if "dim" in value:
            desc.dim = value["dim"]
    debinarize_tensor(desc, filepath)
    return desc


def tensor_file_name(key: str, tti_dump_format: TTIDumpFormat) -> str:
    return os.path.join("tensors", f"torch.Tensor.{key}.{tti_dump_format.extension()}".replace("/", "_"))


class TTDeviceImageJsonEncoder(json.JSONEncoder):
    """Writes tensor payloads beside the JSON and replaces the tensors in the dictionary by their entries."""

    @staticmethod
    def encode_descriptor(filename: str, tensor_desc: PytorchTensorDesc, tilized_tensor_desc: Optional[TilizedTensorDesc] = None):
        encoding = {"bin": filename, "itemsize": tensor_desc.itemsize, "shape": list(tensor_desc.shape),
                    "strides": list(tensor_desc.strides), "dim": tensor_desc.dim, "format": tensor_desc.format}
        if tilized_tensor_desc:
            encoding.update({"format": tilized_tensor_desc.format, "num_buffers": tilized_tensor_desc.num_buffers,
                             "buf_size_bytes": tilized_tensor_desc.buf_size_bytes})
        return encoding

    @staticmethod
    def rehash_tensor_as_pickled_object(d, key, object_value, base_directory):
        filename = tensor_file_name(key, TTIDumpFormat.DEFAULT)
        torch.save(object_value, os.path.join(base_directory, filename))
        d[key] = filename

    @staticmethod
    def rehash_tensor_as_bin_object(d, key, object_value, base_directory, tti_dump_format: TTIDumpFormat, backend_api=None):
        """Payload through the backend: row-major bytes, or with BACKEND_TILIZED the tiles of the queue named ``key``."""
        assert isinstance(object_value, torch.Tensor), "rehash_tensor_as_bin_object expects a torch.Tensor"
        filename = tensor_file_name(key, tti_dump_format)
        tensor = object_value.contiguous()
        tensor_desc = pytorch_tensor_to_tensor_desc(tensor)
        tilized = None
        if tti_dump_format == TTIDumpFormat.BACKEND_TILIZED:
            qdesc = backend_api.be_api.get_queue_descriptor(key)
            tilized = tilize_tensor(qdesc, tensor_desc)
        binarize_tensor(tilized if tilized else tensor_desc, os.path.join(base_directory, filename))
        d[key] = TTDeviceImageJsonEncoder.encode_descriptor(filename, tensor_desc, tilized)
        if tilized:
            free_tensor(tilized)

    @staticmethod
    def preprocess_keys(d, base_directory: str, tti_dump_format: Optional[TTIDumpFormat] = None, backend_api=None):
        """Every tensor in ``d`` (nested dictionaries included) becomes a payload file and an entry."""
        os.makedirs(os.path.join(base_directory, "tensors"), exist_ok=True)
        for key, value in list(d.items()):
            if isinstance(value, torch.Tensor):
                if tti_dump_format in (TTIDumpFormat.BACKEND, TTIDumpFormat.BACKEND_TILIZED) and key != "cpueval_outputs":
                    TTDeviceImageJsonEncoder.rehash_tensor_as_bin_object(d, key, value, base_directory, tti_dump_format, backend_api)
                else:
                    TTDeviceImageJsonEncoder.rehash_tensor_as_pickled_object(d, key, value, base_directory)
            elif isinstance(value, dict):
                d[key] = TTDeviceImageJsonEncoder.preprocess_keys(value, base_directory, tti_dump_format, backend_api)
        return d

    def default(self, obj):
        if hasattr(obj, "to_json"):
            return obj.to_json()
        try:
            return json.JSONEncoder.default(self, obj)
        except TypeError as e:
            raise RuntimeError(f"JSON Serialization failed: {e}. {obj.__class__.__name__}.to_json(..) method needs to be implemented.")


class TTDeviceImageJsonDecoder(json.JSONDecoder):
    @staticmethod
    def rehash_as_tensor(value, directory) -> Callable[[], Any]:
        """A callable that loads the entry when the tensor is first wanted (archive.py:213-220)."""
        return functools.partial(load_tensor_from_disk, os.path.join(directory, value["bin"]), value)

    @staticmethod
    def postprocess_keys(d, directory):
        for key, value in list(d.items()):
            if isinstance(value, dict):
                d[key] = TTDeviceImageJsonDecoder.rehash_as_tensor(value, directory) if "bin" in value else \
                    TTDeviceImageJsonDecoder.postprocess_keys(value, directory)
            elif isinstance(value, str) and value.endswith(".pkl"):
                # files this module wrote itself (the DEFAULT dump format)
                d[key] = torch.load(os.path.join(directory, value), weights_only=True)
        return d


def save_tensors(tensors: Dict[str, Any], directory: str, tti_dump_format: TTIDumpFormat = TTIDumpFormat.BACKEND_TILIZED,
                 backend_api=None, json_name: str = "device.json") -> str:
    """Writes ``tensors`` (name -> torch tensor, possibly nested) under ``directory`` and the entries into ``json_name``."""
    os.makedirs(directory, exist_ok=True)

    def copy_of(d):  # preprocess_keys rewrites the dictionaries it is given: work on copies, the caller keeps its tensors
        return {k: copy_of(v) if isinstance(v, dict) else v for k, v in d.items()}

    entries = TTDeviceImageJsonEncoder.preprocess_keys(copy_of(tensors), directory, tti_dump_format, backend_api)
    path = os.path.join(directory, json_name)
    with open(path, "w") as f:
        json.dump({"tti_version": TTI_VERSION, "tti_dump_format": TTIDumpFormat.to_json(tti_dump_format), "tensors": entries}, f,
                  cls=TTDeviceImageJsonEncoder, indent=2)
    return path


def load_tensors(directory: str, json_name: str = "device.json") -> Dict[str, Any]:
    """name -> callable that loads the descriptor (or the tensor itself for pickled entries)."""
    with open(os.path.join(directory, json_name)) as f:
        doc = json.load(f, cls=TTDeviceImageJsonDecoder)
    return TTDeviceImageJsonDecoder.postprocess_keys(doc["tensors"], directory)
