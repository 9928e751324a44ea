"""Checkpoint reading: a model folder holds config.json and model.safetensors.  The safetensors container is read
here directly (8-byte little-endian header length, a JSON header name -> {dtype, shape, data_offsets}, then the raw
little-endian tensor data) through a memory map, so that nothing of the file is copied before the tensor that wants it
asks (the role of the reference's safetensors_weights_iterator, python/sglang/srt/model_loader/weight_utils.py)."""
import json
import mmap
import os
import struct
import warnings
from typing import Dict, Iterator, Tuple

import torch

_DTYPES = {"BF16": torch.bfloat16, "F16": torch.float16, "F32": torch.float32, "F64": torch.float64, "I64": torch.int64,
           "I32": torch.int32, "I16": torch.int16, "I8": torch.int8, "U8": torch.uint8, "BOOL": torch.bool}


def safetensors_weights_iterator(path: str) -> Iterator[Tuple[str, torch.Tensor]]:
    with open(path, "rb") as f:
        (n,) = struct.unpack("<Q", f.read(8))
        header = json.loads(f.read(n).decode("utf-8"))
        mm = mmap.mmap(f.fileno(), 0, access=mmap.ACCESS_READ)
    base = 8 + n
    buf = memoryview(mm)
    for name, meta in header.items():
        if name == "__metadata__":
            continue
        if meta["dtype"] not in _DTYPES:
            raise ValueError(f"{path}: tensor {name} has dtype {meta['dtype']}, which this loader does not read")
        lo, hi = meta["data_offsets"]
        shape = tuple(meta["shape"])
        if hi == lo:
            yield name, torch.empty(shape, dtype=_DTYPES[meta["dtype"]])
            continue
        # clone(): the tensor must outlive the map, and the map is read-only
        with warnings.catch_warnings():
            warnings.simplefilter("ignore", UserWarning)      # "the given buffer is not writable": it is cloned at once
            t = torch.frombuffer(buf[base + lo: base + hi], dtype=_DTYPES[meta["dtype"]]).reshape(shape).clone()
        yield name, t


def load_weights(model_path: str) -> Dict[str, torch.Tensor]:
    files = sorted(f for f in os.listdir(model_path) if f.endswith(".safetensors"))
    if not files:
        raise FileNotFoundError(f"{model_path}: no .safetensors file")
    out: Dict[str, torch.Tensor] = {}
    for f in files:
        out.update(safetensors_weights_iterator(os.path.join(model_path, f)))
    return out
