"""Reader and writer of the safetensors container.

Layout (as the reference reads it, src/utils/safetensors_reader.cpp:69-99):
an unsigned 64-bit little-endian header length, a JSON header
``{name: {"dtype", "shape", "data_offsets": [begin, end]}, "__metadata__": ...}``
and the raw data section.  A folder holds either ``model.safetensors`` or the
shards named by ``model.safetensors.index.json`` (``weight_map`` values;
src/utils/safetensors_reader.cpp:15-42).  Files are memory-mapped and tensors
are handed out one by one, so a large file is never held twice.
"""
from __future__ import annotations

import json
import mmap
import os
import struct
from typing import Dict, Iterator, List, Tuple

import torch

# container dtype -> (torch dtype, bytes per element)
DTYPES = {
    "F32": (torch.float32, 4),
    "BF16": (torch.bfloat16, 2),
    "F16": (torch.float16, 2),
    "F64": (torch.float64, 8),
    "I64": (torch.int64, 8),
    "I32": (torch.int32, 4),
    "I16": (torch.int16, 2),
    "I8": (torch.int8, 1),
    "U8": (torch.uint8, 1),
    "BOOL": (torch.bool, 1),
}
_NAMES = {v[0]: k for k, v in DTYPES.items()}


class SafetensorsError(ValueError):
    pass


class SafetensorsFile:
    """One memory-mapped .safetensors file."""

    def __init__(self, path: str):
        self.path = path
        size = os.path.getsize(path)
        if size < 8:
            raise SafetensorsError("%s: too short to be a safetensors file" % path)
        self._f = open(path, "rb")
        self._mm = mmap.mmap(self._f.fileno(), 0, access=mmap.ACCESS_READ)
        (hlen,) = struct.unpack("<Q", self._mm[:8])
        if 8 + hlen > size:
            raise SafetensorsError("%s: header length %d exceeds the file size %d" % (path, hlen, size))
        try:
            header = json.loads(self._mm[8:8 + hlen].decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise SafetensorsError("%s: header is not valid JSON (%s)" % (path, e)) from None
        self.metadata = header.pop("__metadata__", None)
        self._data0 = 8 + hlen
        self.entries: Dict[str, dict] = {}
        data_size = size - self._data0
        for name, ent in header.items():
            dt = ent.get("dtype")
            if dt not in DTYPES:
                raise SafetensorsError("%s: tensor %r has unknown dtype %r" % (path, name, dt))
            shape = ent.get("shape")
            b, e = ent.get("data_offsets", (None, None))
            numel = 1
            for s in shape:
                numel *= int(s)
            if not (isinstance(b, int) and isinstance(e, int) and 0 <= b <= e <= data_size):
                raise SafetensorsError("%s: tensor %r has data_offsets %r outside the data section of %d bytes"
                                       % (path, name, ent.get("data_offsets"), data_size))
            if e - b != numel * DTYPES[dt][1]:
                raise SafetensorsError("%s: tensor %r: %d bytes stored, shape %r of %s needs %d"
                                       % (path, name, e - b, shape, dt, numel * DTYPES[dt][1]))
            self.entries[name] = {"dtype": dt, "shape": [int(s) for s in shape], "offsets": (b, e)}

    def names(self) -> List[str]:
        return list(self.entries)

    def info(self, name: str) -> Tuple[torch.dtype, List[int]]:
        ent = self.entries[name]
        return DTYPES[ent["dtype"]][0], ent["shape"]

    def tensor(self, name: str) -> torch.Tensor:
        """A CPU tensor that views the mapping (read-only memory; copy before writing)."""
        ent = self.entries[name]
        tdtype, _ = DTYPES[ent["dtype"]]
        b, e = ent["offsets"]
        if e == b:
            return torch.empty(ent["shape"], dtype=tdtype)
        buf = memoryview(self._mm)[self._data0 + b:self._data0 + e]
        import warnings
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")  # torch warns that the buffer is not writable
            flat = torch.frombuffer(buf, dtype=tdtype)
        return flat.view(ent["shape"])

    def close(self) -> None:
        try:
            self._mm.close()
        except BufferError:
            pass  # tensors that still view the mapping keep it alive
        self._f.close()


def shard_files(folder: str) -> List[str]:
    """Files that make up the model in ``folder`` (index.json shards, else model.safetensors)."""
    index = os.path.join(folder, "model.safetensors.index.json")
    if os.path.isfile(index):
        with open(index) as f:
            wm = json.load(f).get("weight_map", {})
        files = sorted(set(wm.values()))
        if not files:
            raise SafetensorsError("%s: empty weight_map" % index)
        return [os.path.join(folder, x) for x in files]
    single = os.path.join(folder, "model.safetensors")
    if not os.path.isfile(single):
        raise SafetensorsError("no model.safetensors (or model.safetensors.index.json) in %s" % folder)
    return [single]


def open_folder(folder: str) -> List[SafetensorsFile]:
    return [SafetensorsFile(p) for p in shard_files(folder)]


def write_file(path: str, tensors: Dict[str, torch.Tensor], metadata: Dict[str, str] = None) -> None:
    """Write tensors (CPU, contiguous) in the order given."""
    header = {}
    if metadata:
        header["__metadata__"] = metadata
    off = 0
    for name, t in tensors.items():
        if t.dtype not in _NAMES:
            raise SafetensorsError("tensor %r: dtype %s cannot be stored" % (name, t.dtype))
        n = t.numel() * t.element_size()
        header[name] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape), "data_offsets": [off, off + n]}
        off += n
    hbytes = json.dumps(header, separators=(",", ":")).encode("utf-8")
    hbytes += b" " * ((8 - len(hbytes) % 8) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(hbytes)))
        f.write(hbytes)
        for name, t in tensors.items():
            t = t.detach().cpu().contiguous()
            if t.numel():
                f.write(t.view(torch.uint8).numpy().tobytes() if t.dim() else t.reshape(1).view(torch.uint8).numpy().tobytes())
