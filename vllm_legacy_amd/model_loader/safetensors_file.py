"""Reader of the safetensors container: 8 bytes of little-endian header length, that many bytes
of JSON (name -> dtype, shape, data_offsets relative to the end of the header), then raw
little-endian data.  Nothing in the file is executed; tensors are copied out of a memory map."""
import json
import mmap
import struct
from typing import Dict

import torch

_DTYPES = {"BF16": torch.bfloat16, "F16": torch.float16, "F32": torch.float32, "F64": torch.float64,
           "I64": torch.int64, "I32": torch.int32, "I16": torch.int16, "I8": torch.int8,
           "U8": torch.uint8, "BOOL": torch.bool}


def load_safetensors(path: str) -> Dict[str, torch.Tensor]:
    out: Dict[str, torch.Tensor] = {}
    with open(path, "rb") as f:
        (n, ) = struct.unpack("<Q", f.read(8))
        header = json.loads(f.read(n).decode("utf-8"))
        base = 8 + n
        with mmap.mmap(f.fileno(), 0, access=mmap.ACCESS_READ) as m:
            size = len(m)
            for name, info in header.items():
                if name == "__metadata__":
                    continue
                dtype = _DTYPES.get(info["dtype"])
                if dtype is None:
                    raise ValueError(f"{name}: unsupported dtype {info['dtype']}")
                lo, hi = info["data_offsets"]
                shape = tuple(int(s) for s in info["shape"])
                count = 1
                for s in shape:
                    count *= s
                if not (0 <= lo <= hi and base + hi <= size) or hi - lo != count * dtype.itemsize:
                    raise ValueError(f"{name}: data offsets do not fit its shape or the file")
                if count == 0:
                    out[name] = torch.empty(shape, dtype=dtype)
                    continue
                buf = bytearray(m[base + lo:base + hi])
                out[name] = torch.frombuffer(buf, dtype=dtype, count=count).reshape(shape)
    return out
