"""Stage-hop wire format (deserve_utils/serde.py:12-46, identical copy in
deserve_worker/model/utils.py:12-46; sent by
deserve_worker/engine/pipeline/processor.py:224 and forwarded unchanged by the
network layer):

    [u32 big-endian: length of the pickled metadata][pickled metadata][safetensors container]

with one quirk kept: a tensor without elements travels as a one-element tensor
of the same dtype under the name ``"#" + name`` (the reference's container
writer of the time refused empty tensors) and comes back as ``empty((0,))``.

The safetensors container is written and parsed here directly - it is a u64
little-endian header length, a JSON header ``{name: {dtype, shape,
data_offsets}}`` padded with spaces to a multiple of 8 bytes, then the tensors'
bytes back to back - so the hop needs no third-party package; the tests hold
this writer and parser against the ``safetensors`` package in both directions.

Metadata is unpickled with an allow-list: plain containers and scalars, and
``SamplingParams`` (this package's, or the reference's pydantic model of the
same fields, which is mapped onto it).  Anything else in the stream raises
``pickle.UnpicklingError`` instead of being imported: a stage must not execute
what a peer sends.
"""
from __future__ import annotations

import io
import json
import pickle
import struct
from typing import Any, Dict, Tuple

import numpy as np
import torch

from deserve_amd.task import SamplingParams

_DTYPE_NAMES = {
    torch.float64: "F64", torch.float32: "F32", torch.float16: "F16", torch.bfloat16: "BF16",
    torch.int64: "I64", torch.int32: "I32", torch.int16: "I16", torch.int8: "I8",
    torch.uint8: "U8", torch.bool: "BOOL",
}
_NAMED_DTYPES = {v: k for k, v in _DTYPE_NAMES.items()}


def _raw_bytes(t: torch.Tensor) -> bytes:
    t = t.detach().to("cpu").contiguous()
    return t.view(torch.uint8).numpy().tobytes() if t.dtype != torch.bool else \
        t.to(torch.uint8).numpy().tobytes()


def save_container(tensors: Dict[str, torch.Tensor]) -> bytes:
    """A safetensors container holding `tensors` (little-endian, C order)."""
    header: Dict[str, Any] = {}
    chunks = []
    offset = 0
    # widest element type first, then by name: keeps every tensor aligned to its element size
    for name in sorted(tensors, key=lambda k: (-tensors[k].element_size(), k)):
        t = tensors[name]
        if t.dtype not in _DTYPE_NAMES:
            raise ValueError(f"tensor {name!r}: dtype {t.dtype} has no safetensors name")
        raw = _raw_bytes(t)
        header[name] = {"dtype": _DTYPE_NAMES[t.dtype], "shape": list(t.shape),
                        "data_offsets": [offset, offset + len(raw)]}
        chunks.append(raw)
        offset += len(raw)
    text = json.dumps(header, separators=(",", ":")).encode("utf-8")
    text += b" " * (-len(text) % 8)
    return struct.pack("<Q", len(text)) + text + b"".join(chunks)


def load_container(b: bytes) -> Dict[str, torch.Tensor]:
    """Tensors of a safetensors container (copies; the buffer may be released)."""
    if len(b) < 8:
        raise ValueError("safetensors container shorter than its length field")
    (n,) = struct.unpack("<Q", b[:8])
    if 8 + n > len(b):
        raise ValueError(f"safetensors header of {n} bytes exceeds the buffer")
    header = json.loads(b[8: 8 + n].decode("utf-8"))
    data = memoryview(b)[8 + n:]
    out: Dict[str, torch.Tensor] = {}
    for name, info in header.items():
        if name == "__metadata__":
            continue
        dtype = _NAMED_DTYPES.get(info["dtype"])
        if dtype is None:
            raise ValueError(f"tensor {name!r}: unknown dtype {info['dtype']!r}")
        begin, end = info["data_offsets"]
        shape = tuple(int(s) for s in info["shape"])
        count = int(np.prod(shape, dtype=np.int64)) if shape else 1
        size = torch.empty((), dtype=dtype).element_size()
        if not (0 <= begin <= end <= len(data)) or end - begin != count * size:
            raise ValueError(f"tensor {name!r}: offsets {begin}:{end} do not match shape {shape}")
        raw = torch.frombuffer(bytearray(data[begin:end]), dtype=torch.uint8) if count else \
            torch.empty((0,), dtype=torch.uint8)
        t = raw.to(torch.bool) if dtype == torch.bool else raw.view(dtype)
        out[name] = t.reshape(shape)
    return out


class _MetadataUnpickler(pickle.Unpickler):
    _ALLOWED = {("builtins", n) for n in ("dict", "list", "tuple", "set", "frozenset", "str", "int",
                                          "float", "bool", "bytes", "complex", "NoneType")}

    def find_class(self, module: str, name: str):
        if (module, name) in (("deserve_amd.task", "SamplingParams"),
                              ("deserve_worker.task", "SamplingParams")):
            return SamplingParams
        if (module, name) == ("copyreg", "_reconstructor") or (module, name) == ("builtins", "object"):
            return super().find_class(module, name)
        if (module, name) in self._ALLOWED:
            return super().find_class(module, name)
        raise pickle.UnpicklingError(f"metadata names {module}.{name}, which a stage does not load")


def dumps(tensors: Dict[str, torch.Tensor], metadata: Dict[str, Any]) -> bytes:
    metadata_bytes = pickle.dumps(metadata)
    sharp: Dict[str, torch.Tensor] = {}
    for k, v in tensors.items():
        if v.numel() == 0:
            sharp[f"#{k}"] = torch.ones((1,), dtype=v.dtype)
        else:
            sharp[k] = v
    return len(metadata_bytes).to_bytes(4, byteorder="big") + metadata_bytes + save_container(sharp)


def loads(b: bytes) -> Tuple[Dict[str, torch.Tensor], Dict[str, Any]]:
    if len(b) < 4:
        raise ValueError("message shorter than its length field")
    n = int.from_bytes(b[:4], byteorder="big")
    if 4 + n > len(b):
        raise ValueError(f"metadata of {n} bytes exceeds the message")
    metadata = _MetadataUnpickler(io.BytesIO(b[4: 4 + n])).load()
    tensors: Dict[str, torch.Tensor] = {}
    for k, v in load_container(b[4 + n:]).items():
        if k.startswith("#"):
            tensors[k[1:]] = torch.empty((0,), dtype=v.dtype)
        else:
            tensors[k] = v
    return tensors, metadata
