"""Reader of .safetensors checkpoints: 8-byte little-endian header length, JSON header (name -> dtype, shape,
data_offsets), raw little-endian data.  The file is memory-mapped and every tensor is copied to the device from the map."""
import json
import mmap
import struct
import warnings

import torch

_DT = {"BF16": torch.bfloat16, "F16": torch.float16, "F32": torch.float32, "F64": torch.float64, "I64": torch.int64,
       "I32": torch.int32, "I16": torch.int16, "I8": torch.int8, "U8": torch.uint8, "BOOL": torch.bool}


def read_header(path):
    with open(path, "rb") as f:
        (n,) = struct.unpack("<Q", f.read(8))
        if n > (1 << 28):
            raise ValueError(f"{path}: implausible header length {n}")
        meta = json.loads(f.read(n).decode("utf-8"))
    meta.pop("__metadata__", None)
    return meta, 8 + n


def load(path, device="cpu", names=None):
    """name -> tensor (on `device`) of every tensor of the file (or of `names`)."""
    meta, base = read_header(path)
    out = {}
    with open(path, "rb") as f:
        mm = mmap.mmap(f.fileno(), 0, access=mmap.ACCESS_READ)
        try:
            for name, m in meta.items():
                if names is not None and name not in names:
                    continue
                if m["dtype"] not in _DT:
                    raise ValueError(f"{path}: tensor {name!r} has unsupported dtype {m['dtype']}")
                lo, hi = m["data_offsets"]
                dtype, shape = _DT[m["dtype"]], list(m["shape"])
                count = 1
                for d in shape:
                    count *= d
                if hi - lo != count * torch.empty(0, dtype=dtype).element_size():
                    raise ValueError(f"{path}: tensor {name!r}: {hi - lo} bytes for shape {shape}")
                if count == 0:
                    t = torch.empty(shape, dtype=dtype)
                else:
                    with warnings.catch_warnings():  # the map is read-only; the tensor is copied at once
                        warnings.simplefilter("ignore", UserWarning)
                        t = torch.frombuffer(mm, dtype=dtype, count=count, offset=base + lo).reshape(shape).clone()
                out[name] = t.to(device)
        finally:
            try:
                mm.close()
            except BufferError:  # a view of the map is still alive: the map goes with it
                pass
    return out
