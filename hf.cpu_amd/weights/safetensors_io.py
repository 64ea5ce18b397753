"""Reading and writing the safetensors container.

Layout: an unsigned 64-bit little-endian header length, that many bytes of JSON
mapping each tensor name to ``{"dtype", "shape", "data_offsets": [begin, end]}``
(offsets relative to the end of the header), then the data. Tensors are found by
name, as the reference finds GGUF tensors by name (src/model.c:52-93).
"""
import json
import os
import struct

import numpy as np
import torch

from ..status import EFORMAT, EIO, fail

# container dtype -> (numpy dtype used to carry the bytes, torch dtype they mean)
DTYPES = {
    "F32": (np.dtype("<f4"), torch.float32),
    "BF16": (np.dtype("<u2"), torch.bfloat16),
    "F16": (np.dtype("<f2"), torch.float16),
    "F64": (np.dtype("<f8"), torch.float64),
    "I64": (np.dtype("<i8"), torch.int64),
    "I32": (np.dtype("<i4"), torch.int32),
    "I16": (np.dtype("<i2"), torch.int16),
    "I8": (np.dtype("i1"), torch.int8),
    "U8": (np.dtype("u1"), torch.uint8),
    "BOOL": (np.dtype("u1"), torch.bool),
}
_NAME_OF = {torch.float32: "F32", torch.bfloat16: "BF16", torch.float16: "F16", torch.float64: "F64",
            torch.int64: "I64", torch.int32: "I32", torch.int16: "I16", torch.int8: "I8",
            torch.uint8: "U8", torch.bool: "BOOL"}
MAX_HEADER = 100 << 20


class TensorEntry:
    __slots__ = ("name", "dtype", "shape", "begin", "end", "file")

    def __init__(self, name, dtype, shape, begin, end, file):
        self.name, self.dtype, self.shape, self.begin, self.end, self.file = name, dtype, shape, begin, end, file


class SafetensorsFile:
    """The directory of one file; ``read(name)`` returns a CPU tensor that owns its memory."""

    def __init__(self, path):
        self.path = path
        try:
            size = os.path.getsize(path)
            with open(path, "rb") as f:
                head = f.read(8)
                if len(head) != 8:
                    fail(EFORMAT, f"{path}: shorter than a safetensors header")
                (n,) = struct.unpack("<Q", head)
                if n > MAX_HEADER or 8 + n > size:
                    fail(EFORMAT, f"{path}: header length {n} does not fit the file")
                raw = f.read(n)
        except OSError as e:
            fail(EIO, f"cannot read {path}: {e.strerror}")
        try:
            header = json.loads(raw.decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            fail(EFORMAT, f"{path}: header is not JSON: {e}")
        if not isinstance(header, dict):
            fail(EFORMAT, f"{path}: header is not a JSON object")
        self.data_start = 8 + n
        self.metadata = header.pop("__metadata__", None) or {}
        self.entries = {}
        for name, info in header.items():
            try:
                dtype, shape = info["dtype"], tuple(int(d) for d in info["shape"])
                begin, end = (int(v) for v in info["data_offsets"])
            except (KeyError, TypeError, ValueError):
                fail(EFORMAT, f"{path}: entry of tensor '{name}' is malformed")
            if dtype in DTYPES:
                count = int(np.prod(shape, dtype=np.int64)) if shape else 1
                if begin < 0 or end < begin or self.data_start + end > size \
                        or end - begin != count * DTYPES[dtype][0].itemsize:
                    fail(EFORMAT, f"{path}: data of tensor '{name}' does not match its shape or the file")
            self.entries[name] = TensorEntry(name, dtype, shape, begin, end, self)
        self._map = None

    def names(self):
        return list(self.entries)

    def read(self, name):
        e = self.entries[name]
        if e.dtype not in DTYPES:
            fail(EFORMAT, f"{self.path}: tensor '{name}' has dtype {e.dtype}, which is not readable")
        np_dtype, t_dtype = DTYPES[e.dtype]
        if self._map is None:
            self._map = np.memmap(self.path, dtype=np.uint8, mode="r")
        raw = np.array(self._map[self.data_start + e.begin:self.data_start + e.end])   # owned copy
        arr = raw.view(np_dtype).reshape(e.shape)
        if t_dtype == torch.bfloat16:
            return torch.from_numpy(arr.view(np.int16)).view(torch.bfloat16)
        if t_dtype == torch.bool:
            return torch.from_numpy(arr).to(torch.bool)
        return torch.from_numpy(arr)


def open_model_tensors(model_dir):
    """name -> TensorEntry over ``model.safetensors`` or, if an index file is there,
    over the files it names."""
    single = os.path.join(model_dir, "model.safetensors")
    index = os.path.join(model_dir, "model.safetensors.index.json")
    if os.path.exists(single):
        return dict(SafetensorsFile(single).entries)
    if os.path.exists(index):
        from ..config.reader import read_json_file
        wm = read_json_file(index).get("weight_map")
        if not isinstance(wm, dict):
            fail(EFORMAT, f"{index}: no 'weight_map'")
        files, out = {}, {}
        for name, fname in wm.items():
            if fname not in files:
                files[fname] = SafetensorsFile(os.path.join(model_dir, fname))
            if name not in files[fname].entries:
                fail(EFORMAT, f"{index}: tensor '{name}' is not in {fname}")
            out[name] = files[fname].entries[name]
        return out
    fail(EIO, f"cannot read {single}: no such file")


def write_safetensors(path, tensors, metadata=None):
    """Writes ``tensors`` (name -> CPU tensor, or a callable returning one so that large
    models are made one tensor at a time) in the order given. Callables must come with
    their dtype and shape: ``(dtype, shape, fn)``."""
    header, offset, plan = {}, 0, []
    for name, t in tensors.items():
        if isinstance(t, tuple):
            dtype, shape, fn = t
        else:
            dtype, shape, fn = t.dtype, tuple(t.shape), (lambda t=t: t)
        count = int(np.prod(shape, dtype=np.int64)) if shape else 1
        nbytes = count * torch.empty((), dtype=dtype).element_size()
        header[name] = {"dtype": _NAME_OF[dtype], "shape": list(shape), "data_offsets": [offset, offset + nbytes]}
        offset += nbytes
        plan.append((name, dtype, tuple(shape), nbytes, fn))
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    raw = json.dumps(header, separators=(",", ":")).encode("utf-8")
    raw += b" " * (-len(raw) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(raw)))
        f.write(raw)
        for name, dtype, shape, nbytes, fn in plan:
            t = fn().contiguous()
            if t.dtype != dtype or tuple(t.shape) != shape:
                raise ValueError(f"tensor '{name}' came out as {t.dtype} {tuple(t.shape)}, declared {dtype} {shape}")
            if dtype == torch.bfloat16:
                t = t.view(torch.int16)
            elif dtype == torch.bool:
                t = t.to(torch.uint8)
            data = t.numpy().tobytes()
            assert len(data) == nbytes
            f.write(data)
