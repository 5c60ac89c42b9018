"""Reading and writing of the safetensors container, by tensor name.

Container layout as the reference reads it: an 8-byte little-endian header length,
a JSON object ``{name: {dtype, shape, data_offsets}}`` with an optional
``__metadata__`` entry, then the raw data (/root/reference/src/engine/tq_model.c:185-305
header, :667-732 shard, :624-658 mmap).  The tensor table is a dictionary, not the
reference's fixed 2048-entry array (tq_model.c:77), so models with thousands of
expert tensors fit.  Shards are found like the reference does
(``model.safetensors`` or ``model-*-of-*.safetensors``, tq_model.c:750-842).
"""
from __future__ import annotations

import glob
import json
import mmap
import os
import struct
import warnings
from dataclasses import dataclass

import torch

DTYPES = {
    "F32": (torch.float32, 4),
    "BF16": (torch.bfloat16, 2),
    "F16": (torch.float16, 2),
    "I32": (torch.int32, 4),
    "I64": (torch.int64, 8),
}
NAMES = {v[0]: k for k, v in DTYPES.items()}


class SafetensorsError(ValueError):
    pass


@dataclass(frozen=True)
class TensorEntry:
    name: str
    dtype: str
    shape: tuple[int, ...]
    begin: int
    end: int
    shard: int


class SafetensorsFolder:
    """All shards of a model folder (or the given files), memory-mapped; tensors are read by name.  ``metadata``
    holds the files' ``__metadata__`` entries."""

    def __init__(self, model_dir: str, files: list[str] | None = None):
        self.model_dir = model_dir
        if files is None:
            files = find_shards(model_dir)
            if not files:
                raise SafetensorsError(f"no model.safetensors (or model-*-of-*.safetensors) in {model_dir!r}")
        self.files = files
        self.metadata: dict[str, str] = {}
        self._maps: list[mmap.mmap] = []
        self._handles = []
        self._data_start: list[int] = []
        self.entries: dict[str, TensorEntry] = {}
        for i, path in enumerate(files):
            self._open_shard(i, path)

    def _open_shard(self, index: int, path: str) -> None:
        size = os.path.getsize(path)
        if size < 8:
            raise SafetensorsError(f"{path}: file too small to be safetensors ({size} bytes)")
        f = open(path, "rb")
        self._handles.append(f)
        m = mmap.mmap(f.fileno(), 0, access=mmap.ACCESS_READ)
        self._maps.append(m)
        (hlen,) = struct.unpack("<Q", m[:8])
        if 8 + hlen > size:
            raise SafetensorsError(f"{path}: header of {hlen} bytes reaches beyond the file ({size} bytes)")
        try:
            header = json.loads(m[8:8 + hlen].decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise SafetensorsError(f"{path}: header is not valid JSON ({e})") from e
        start = 8 + hlen
        self._data_start.append(start)
        for name, info in header.items():
            if name == "__metadata__":
                self.metadata.update(info or {})
                continue
            dtype = info.get("dtype")
            if dtype not in DTYPES:
                raise SafetensorsError(f"{path}: tensor {name!r} has unsupported dtype {dtype!r}")
            shape = tuple(int(s) for s in info["shape"])
            begin, end = (int(o) for o in info["data_offsets"])
            count = 1
            for s in shape:
                count *= s
            if end - begin != count * DTYPES[dtype][1] or start + end > size:
                raise SafetensorsError(f"{path}: tensor {name!r} data range [{begin},{end}) does not fit shape {shape} {dtype} or the file")
            if name in self.entries:
                raise SafetensorsError(f"tensor {name!r} appears in more than one shard")
            self.entries[name] = TensorEntry(name, dtype, shape, begin, end, index)

    def names(self):
        return self.entries.keys()

    def read(self, name: str) -> torch.Tensor:
        """A CPU tensor that views the mapped file (no copy); keep the folder open while it is used."""
        e = self.entries[name]
        dtype = DTYPES[e.dtype][0]
        count = (e.end - e.begin) // DTYPES[e.dtype][1]
        if count == 0:
            return torch.empty(e.shape, dtype=dtype)
        with warnings.catch_warnings():
            warnings.simplefilter("ignore", UserWarning)     # the map is read-only; the tensor is only read
            t = torch.frombuffer(self._maps[e.shard], dtype=dtype, count=count,
                                 offset=self._data_start[e.shard] + e.begin)
        return t.view(e.shape)

    def close(self) -> None:
        for m in self._maps:
            try:
                m.close()
            except BufferError:
                pass  # a tensor still views the map; the map goes when the tensor does
        for f in self._handles:
            f.close()
        self._maps, self._handles = [], []

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()


def find_shards(model_dir: str) -> list[str]:
    single = os.path.join(model_dir, "model.safetensors")
    if os.path.isfile(single):
        return [single]
    return sorted(glob.glob(os.path.join(model_dir, "model-*-of-*.safetensors")))


class SafetensorsWriter:
    """Streams tensors into one file.  Shapes and dtypes are declared first so the header can
    be written before the data; tensors are then appended in the declared order."""

    def __init__(self, path: str, table: list[tuple[str, tuple[int, ...], torch.dtype]], metadata: dict | None = None):
        self.path = path
        self.table = table
        header: dict = {}
        if metadata:
            header["__metadata__"] = {k: str(v) for k, v in metadata.items()}
        offset = 0
        for name, shape, dtype in table:
            n = 1
            for s in shape:
                n *= s
            nbytes = n * DTYPES[NAMES[dtype]][1]
            header[name] = {"dtype": NAMES[dtype], "shape": list(shape), "data_offsets": [offset, offset + nbytes]}
            offset += nbytes
        blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
        blob += b" " * ((8 - len(blob) % 8) % 8)
        self._f = open(path, "wb")
        self._f.write(struct.pack("<Q", len(blob)))
        self._f.write(blob)
        self._next = 0

    def append(self, name: str, tensor: torch.Tensor) -> None:
        want_name, shape, dtype = self.table[self._next]
        if name != want_name or tuple(tensor.shape) != tuple(shape) or tensor.dtype != dtype:
            raise SafetensorsError(f"writer expected {want_name} {shape} {dtype}, got {name} {tuple(tensor.shape)} {tensor.dtype}")
        t = tensor.detach().contiguous().cpu()
        if t.numel():
            self._f.write(t.view(torch.uint8).numpy().tobytes() if t.dim() else t.reshape(1).view(torch.uint8).numpy().tobytes())
        self._next += 1

    def close(self) -> None:
        if self._next != len(self.table):
            raise SafetensorsError(f"{self.path}: {len(self.table) - self._next} declared tensors were never written")
        self._f.close()

    def __enter__(self):
        return self

    def __exit__(self, exc_type, *exc):
        if exc_type is None:
            self.close()
        else:
            self._f.close()


def write_safetensors(path: str, tensors: dict[str, torch.Tensor], metadata: dict | None = None) -> None:
    table = [(n, tuple(t.shape), t.dtype) for n, t in tensors.items()]
    with SafetensorsWriter(path, table, metadata) as w:
        for n, t in tensors.items():
            w.append(n, t)
