"""Reading and writing the safetensors container.

Layout: 8 bytes little-endian header length, a JSON header {name: {dtype, shape,
data_offsets}} (plus an optional "__metadata__"), then one byte buffer.  The
checks are those of the reference's reader (ferrox-safetensors/src/lib.rs:168-243):
header of at most 100 MB, entries sorted by offset contiguous from 0, byte count
= product(shape) x element size, data filling the file exactly.  Tensors are
views into a memory map; nothing is copied until it is uploaded.  A folder may
hold one `model.safetensors` or an index `model.safetensors.index.json` with a
`weight_map` over several files (lib.rs:279-328).
"""
from __future__ import annotations

import json
import mmap
import os
import struct

import torch

MAX_HEADER = 100 * 1024 * 1024
DTYPES = {
    "F64": (torch.float64, 8), "F32": (torch.float32, 4), "F16": (torch.float16, 2), "BF16": (torch.bfloat16, 2),
    "I64": (torch.int64, 8), "I32": (torch.int32, 4), "I16": (torch.int16, 2), "I8": (torch.int8, 1),
    "U8": (torch.uint8, 1), "BOOL": (torch.bool, 1),
}
NAMES = {v[0]: k for k, v in DTYPES.items()}


class SafetensorsError(ValueError):
    pass


class SafetensorsFile:
    def __init__(self, path: str):
        self.path = path
        size = os.path.getsize(path)
        if size < 8:
            raise SafetensorsError(f"{path}: too small to hold a header length")
        self._fh = open(path, "rb")
        (n,) = struct.unpack("<Q", self._fh.read(8))
        if n > MAX_HEADER or 8 + n > size:
            raise SafetensorsError(f"{path}: header length {n} is not plausible for a file of {size} bytes")
        try:
            header = json.loads(self._fh.read(n).decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise SafetensorsError(f"{path}: header is not valid JSON ({e})") from e
        if not isinstance(header, dict):
            raise SafetensorsError(f"{path}: header must be a JSON object")
        self.metadata = header.pop("__metadata__", None) or {}
        self.data_start = 8 + n
        self.entries: dict[str, tuple] = {}
        expect = 0
        for name, e in sorted(header.items(), key=lambda kv: kv[1].get("data_offsets", [0, 0])[0]
                              if isinstance(kv[1], dict) else 0):
            if not isinstance(e, dict) or not {"dtype", "shape", "data_offsets"} <= set(e):
                raise SafetensorsError(f"{path}: entry '{name}' lacks dtype, shape or data_offsets")
            if e["dtype"] not in DTYPES:
                raise SafetensorsError(f"{path}: tensor '{name}' has unsupported dtype {e['dtype']}")
            dt, esize = DTYPES[e["dtype"]]
            shape = tuple(int(d) for d in e["shape"])
            begin, end = (int(v) for v in e["data_offsets"])
            count = 1
            for d in shape:
                count *= d
            if end - begin != count * esize:
                raise SafetensorsError(f"{path}: tensor '{name}' {e['dtype']}{list(shape)} needs {count * esize} "
                                       f"bytes but its offsets span {end - begin}")
            if begin != expect:
                raise SafetensorsError(f"{path}: tensor '{name}' starts at byte {begin}, expected {expect} "
                                       f"(entries must be contiguous)")
            expect = end
            self.entries[name] = (dt, shape, begin, end)
        if self.data_start + expect != size:
            raise SafetensorsError(f"{path}: data ends at byte {self.data_start + expect} but the file has {size}")
        self._map = mmap.mmap(self._fh.fileno(), 0, access=mmap.ACCESS_READ) if size > 0 else None

    def names(self):
        return list(self.entries)

    def info(self, name: str):
        dt, shape, _, _ = self.entries[name]
        return dt, shape

    def tensor(self, name: str) -> torch.Tensor:
        """A CPU tensor viewing the file's bytes (read-only: copy before writing to it)."""
        dt, shape, begin, end = self.entries[name]
        if end == begin:
            return torch.empty(shape, dtype=dt)
        count = (end - begin) // DTYPES[NAMES[dt]][1]
        import warnings
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")    # torch warns that the buffer is not writable
            flat = torch.frombuffer(self._map, dtype=dt, count=count, offset=self.data_start + begin)
        return flat.reshape(shape)


class Checkpoint:
    """All tensors of a model folder, from one file or from an index over shards."""

    def __init__(self, folder: str):
        self.folder = folder
        index = os.path.join(folder, "model.safetensors.index.json")
        single = os.path.join(folder, "model.safetensors")
        self._files: dict[str, SafetensorsFile] = {}
        self._where: dict[str, str] = {}
        if os.path.isfile(single):
            f = self._open(single)
            for n in f.names():
                self._where[n] = single
        elif os.path.isfile(index):
            with open(index) as fh:
                try:
                    wm = json.load(fh)["weight_map"]
                except (json.JSONDecodeError, KeyError, TypeError) as e:
                    raise SafetensorsError(f"{index}: no usable weight_map ({e})") from e
            for n, fname in wm.items():
                path = os.path.join(folder, fname)
                f = self._open(path)
                if n not in f.entries:
                    raise SafetensorsError(f"{index}: tensor '{n}' is not in {fname}")
                self._where[n] = path
        else:
            raise SafetensorsError(f"{folder}: neither model.safetensors nor model.safetensors.index.json")

    def _open(self, path):
        if path not in self._files:
            if not os.path.isfile(path):
                raise SafetensorsError(f"{path}: file named by the index is missing")
            self._files[path] = SafetensorsFile(path)
        return self._files[path]

    def names(self):
        return list(self._where)

    def info(self, name):
        return self._files[self._where[name]].info(name)

    def tensor(self, name):
        return self._files[self._where[name]].tensor(name)


def write_safetensors(path: str, tensors, metadata: dict | None = None) -> None:
    """`tensors`: an iterable of (name, make) or a dict name -> tensor; `make()` returns the CPU
    tensor when it is its turn, so a large model is never held whole."""
    items = list(tensors.items()) if isinstance(tensors, dict) else list(tensors)
    header, offset, plan = {}, 0, []
    for name, t in items:
        if callable(t):
            dt, shape = t.dtype, tuple(t.shape)     # a lazy tensor announces dtype and shape
        else:
            dt, shape = t.dtype, tuple(t.shape)
        if dt not in NAMES:
            raise SafetensorsError(f"cannot store tensor '{name}' of dtype {dt}")
        count = 1
        for d in shape:
            count *= d
        nbytes = count * DTYPES[NAMES[dt]][1]
        header[name] = {"dtype": NAMES[dt], "shape": list(shape), "data_offsets": [offset, offset + nbytes]}
        plan.append((name, t, nbytes))
        offset += nbytes
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
    blob += b" " * ((8 - len(blob) % 8) % 8)
    tmp = path + ".tmp"
    with open(tmp, "wb") as f:
        f.write(struct.pack("<Q", len(blob)))
        f.write(blob)
        for name, t, nbytes in plan:
            if callable(t):
                t = t()
            t = t.detach().contiguous().cpu()
            raw = t.view(torch.uint8) if t.numel() else t
            if t.numel():
                f.write(raw.numpy().tobytes())
    os.replace(tmp, path)


class LazyTensor:
    """dtype and shape now, values when called."""

    def __init__(self, dtype, shape, make):
        self.dtype, self.shape, self._make = dtype, tuple(shape), make

    def __call__(self):
        return self._make()
