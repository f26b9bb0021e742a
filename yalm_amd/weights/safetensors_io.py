"""Reader and writer of the safetensors container: a little-endian u64 header
length, a JSON header {name: {dtype, shape, data_offsets}} (+ "__metadata__"),
then the raw data.  The checks are those of the reference's codec
(src/codec.cpp:39-155): known dtype, at most 4 dimensions, integer sizes, two
offsets with start <= end <= size of the file, and bytes == elements * size.
Errors are exceptions that name the file and the tensor."""
import json
import mmap
import os
import struct

import numpy as np
import torch


class SafetensorsError(ValueError):
    pass


# name -> (numpy dtype to view the bytes with, torch dtype, bytes per element)
_DTYPES = {
    "F32": (np.float32, torch.float32, 4),
    "F16": (np.float16, torch.float16, 2),
    "BF16": (np.uint16, torch.bfloat16, 2),
    "F64": (np.float64, torch.float64, 8),
    "I64": (np.int64, torch.int64, 8),
    "I32": (np.int32, torch.int32, 4),
    "I16": (np.int16, torch.int16, 2),
    "I8": (np.int8, torch.int8, 1),
    "U8": (np.uint8, torch.uint8, 1),
}
_NAMES = {torch.float32: "F32", torch.float16: "F16", torch.bfloat16: "BF16", torch.float64: "F64",
          torch.int64: "I64", torch.int32: "I32", torch.int16: "I16", torch.int8: "I8", torch.uint8: "U8"}
MAX_DIMS = 4


class TensorEntry:
    __slots__ = ("name", "dtype_name", "shape", "start", "end")

    def __init__(self, name, dtype_name, shape, start, end):
        self.name, self.dtype_name, self.shape, self.start, self.end = name, dtype_name, shape, start, end

    @property
    def torch_dtype(self):
        return _DTYPES[self.dtype_name][1]


class SafetensorsFile:
    """One file, memory-mapped read-only; tensors are views until copied."""

    def __init__(self, path):
        self.path = path
        size = os.path.getsize(path)
        if size < 8:
            raise SafetensorsError("%s: too short to be a safetensors file" % path)
        self._fh = open(path, "rb")
        self._map = mmap.mmap(self._fh.fileno(), 0, access=mmap.ACCESS_READ)
        (hlen,) = struct.unpack("<Q", self._map[:8])
        if hlen <= 0 or 8 + hlen > size:
            raise SafetensorsError("%s: header length %d does not fit the file (%d bytes)" % (path, hlen, size))
        try:
            header = json.loads(self._map[8:8 + hlen].decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise SafetensorsError("%s: the header is not JSON: %s" % (path, e)) from None
        if not isinstance(header, dict):
            raise SafetensorsError("%s: the header is not a JSON object" % path)
        self._base = 8 + hlen
        data_size = size - self._base
        self.metadata = {}
        self.entries = {}
        for name, meta in header.items():
            if name == "__metadata__":
                self.metadata = meta if isinstance(meta, dict) else {}
                continue
            self.entries[name] = self._entry(name, meta, data_size)

    def _entry(self, name, meta, data_size):
        where = "%s: tensor %r" % (self.path, name)
        if not isinstance(meta, dict):
            raise SafetensorsError("%s: its header entry is not an object" % where)
        dt = meta.get("dtype")
        if dt not in _DTYPES:
            raise SafetensorsError("%s: dtype %r is not supported" % (where, dt))
        shape = meta.get("shape")
        if not isinstance(shape, list) or len(shape) > MAX_DIMS:
            raise SafetensorsError("%s: shape %r must be a list of at most %d sizes" % (where, shape, MAX_DIMS))
        if any(not isinstance(s, int) or isinstance(s, bool) or s < 0 for s in shape):
            raise SafetensorsError("%s: shape %r holds a size that is no non-negative integer" % (where, shape))
        off = meta.get("data_offsets")
        if (not isinstance(off, list) or len(off) != 2
                or any(not isinstance(o, int) or isinstance(o, bool) for o in off)):
            raise SafetensorsError("%s: data_offsets %r must be two integers" % (where, off))
        start, end = off
        if start < 0 or end < start or end > data_size:
            raise SafetensorsError("%s: data_offsets %r do not lie inside the data (%d bytes)"
                                   % (where, off, data_size))
        numel = 1
        for s in shape:
            numel *= s
        if numel * _DTYPES[dt][2] != end - start:
            raise SafetensorsError("%s: %d elements of %s need %d bytes, the offsets give %d"
                                   % (where, numel, dt, numel * _DTYPES[dt][2], end - start))
        return TensorEntry(name, dt, tuple(shape), start, end)

    def tensor(self, name):
        """A CPU tensor over the mapped bytes (read-only memory: copy before writing)."""
        e = self.entries[name]
        np_dt, torch_dt, _ = _DTYPES[e.dtype_name]
        count = (e.end - e.start) // _DTYPES[e.dtype_name][2]
        arr = np.frombuffer(self._map, dtype=np_dt, count=count, offset=self._base + e.start)
        import warnings
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")                  # torch warns that the array is not writable
            t = torch.from_numpy(arr)
        if torch_dt == torch.bfloat16:
            t = t.view(torch.bfloat16)
        return t.reshape(e.shape)

    def close(self):
        # tensors handed out keep the mapping alive through numpy; closing is best effort
        try:
            self._map.close()
        except (BufferError, ValueError):
            pass
        self._fh.close()


def write_file(path, tensors, metadata=None):
    """Writes CPU tensors (name -> tensor) as one safetensors file."""
    header = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    offset = 0
    order = sorted(tensors)
    for name in order:
        t = tensors[name]
        if t.dtype not in _NAMES:
            raise SafetensorsError("tensor %r: dtype %s cannot be written" % (name, t.dtype))
        if t.dim() > MAX_DIMS:
            raise SafetensorsError("tensor %r: more than %d dimensions" % (name, MAX_DIMS))
        nbytes = t.numel() * t.element_size()
        header[name] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape), "data_offsets": [offset, offset + nbytes]}
        offset += nbytes
    blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
    blob += b" " * ((8 - len(blob) % 8) % 8)
    tmp = path + ".tmp%d" % os.getpid()
    with open(tmp, "wb") as f:
        f.write(struct.pack("<Q", len(blob)))
        f.write(blob)
        for name in order:
            t = tensors[name].detach().cpu().contiguous()
            if t.dtype == torch.bfloat16:
                t = t.view(torch.int16)
            f.write(t.numpy().tobytes())
    os.replace(tmp, path)
