"""Where a model's tensors come from: a folder of safetensors files, or a dictionary.

Reference: minivllm/models/loader.py:17-21 opens every ``*.safetensors`` file of the folder
and yields ``(name, tensor)``; it does not use an index file. Here the files are opened once
(sorted), their headers give names, shapes and dtypes without reading data, and tensors are
read one at a time by name.

Storage rule: a tensor stored in bfloat16 stays bfloat16, one stored in 32-bit (or wider)
floating point stays float32, integer tensors become int32. Any other stored type (float16,
8-bit floats) is refused: the engine computes in bfloat16 or float32 and converts nothing
behind the user's back.
"""
from __future__ import annotations

import glob
import os
import weakref
from typing import Dict, List, Tuple

import torch


class TensorSource:
    """Names, shapes and data of a model's tensors."""

    def names(self) -> List[str]:
        raise NotImplementedError

    def shape(self, name: str) -> Tuple[int, ...]:
        raise NotImplementedError

    def is_integer(self, name: str) -> bool:
        raise NotImplementedError

    def stored_type(self, name: str) -> str:
        """The stored element type by its safetensors name ("BF16", "F32", "F16", "I64", ...)."""
        raise NotImplementedError

    def read(self, name: str) -> torch.Tensor:
        """The tensor on the CPU, as stored."""
        raise NotImplementedError


_INT_DTYPES = {"I8", "I16", "I32", "I64", "U8", "U16", "U32", "U64", "BOOL"}
# stored floating types the engine keeps (bfloat16 as it is, the wide ones as float32)
KEPT_FLOAT_TYPES = {"BF16", "F32", "F64"}
_TORCH_TYPE_NAMES = {torch.bfloat16: "BF16", torch.float32: "F32", torch.float64: "F64", torch.float16: "F16",
                     torch.int8: "I8", torch.int16: "I16", torch.int32: "I32", torch.int64: "I64",
                     torch.uint8: "U8", torch.bool: "BOOL"}


class SafetensorsSource(TensorSource):
    def __init__(self, model_dir: str):
        from safetensors import safe_open
        files = sorted(glob.glob(os.path.join(model_dir, "*.safetensors")))
        if not files:
            raise FileNotFoundError(f"{model_dir!r} holds no *.safetensors file")
        self._handles = []
        self._where: Dict[str, int] = {}
        self._shapes: Dict[str, Tuple[int, ...]] = {}
        self._dtypes: Dict[str, str] = {}
        for path in files:
            h = safe_open(path, "pt", "cpu")
            self._handles.append(h)
            for name in h.keys():
                if name in self._where:
                    raise ValueError(f"tensor {name!r} appears in more than one safetensors file of {model_dir!r}")
                self._where[name] = len(self._handles) - 1
                sl = h.get_slice(name)
                self._shapes[name] = tuple(sl.get_shape())
                self._dtypes[name] = str(sl.get_dtype())

    def names(self) -> List[str]:
        return list(self._where)

    def shape(self, name: str) -> Tuple[int, ...]:
        return self._shapes[name]

    def is_integer(self, name: str) -> bool:
        return self._dtypes[name].upper() in _INT_DTYPES

    def stored_type(self, name: str) -> str:
        return self._dtypes[name].upper()

    def read(self, name: str) -> torch.Tensor:
        return self._handles[self._where[name]].get_tensor(name)


class DictSource(TensorSource):
    def __init__(self, tensors: Dict[str, torch.Tensor]):
        self._tensors = dict(tensors)

    def names(self) -> List[str]:
        return list(self._tensors)

    def shape(self, name: str) -> Tuple[int, ...]:
        return tuple(self._tensors[name].shape)

    def is_integer(self, name: str) -> bool:
        t = self._tensors[name]
        return not (t.is_floating_point() or t.is_complex())

    def stored_type(self, name: str) -> str:
        dt = self._tensors[name].dtype
        return _TORCH_TYPE_NAMES.get(dt, str(dt).replace("torch.", "").upper())

    def read(self, name: str) -> torch.Tensor:
        return self._tensors[name]


def storage_dtype(t: torch.Tensor) -> torch.dtype:
    """The dtype a stored tensor is kept in on the device."""
    if not t.is_floating_point():
        return torch.int32
    if t.dtype in (torch.float32, torch.float64):
        return torch.float32
    if t.dtype == torch.bfloat16:
        return torch.bfloat16
    raise TypeError(f"tensors stored as {t.dtype} are not supported (bfloat16 and float32 are)")


class DeviceTensors:
    """Hands tensors to the model by name, on the device, in their kept dtype. The same name
    gives the same tensor object while someone still holds it, so a tied head and the embedding
    share their memory."""

    def __init__(self, source: TensorSource, device: torch.device):
        self.source = source
        self.device = device
        self._alive: "weakref.WeakValueDictionary[str, torch.Tensor]" = weakref.WeakValueDictionary()

    def get(self, name: str) -> torch.Tensor:
        t = self._alive.get(name)
        if t is not None:
            return t
        cpu = self.source.read(name)
        t = cpu.to(device=self.device, dtype=storage_dtype(cpu)).contiguous()
        if t.data_ptr() == cpu.data_ptr():      # already there in the kept dtype: do not alias the source
            t = t.clone()
        self._alive[name] = t
        return t
