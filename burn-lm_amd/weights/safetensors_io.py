"""Reading and writing the safetensors container: an 8-byte little-endian header length, a JSON
header ``{name: {dtype, shape, data_offsets}}``, then the raw little-endian data.  Files are
memory-mapped and tensors are copied out one at a time, so a checkpoint larger than host memory
still loads.  A folder may hold one ``model.safetensors`` or shards listed by
``model.safetensors.index.json``."""
from __future__ import annotations

import json
import mmap
import os
import struct
import warnings
from typing import Dict, Iterable, Tuple

import torch

DTYPES = {"F32": torch.float32, "BF16": torch.bfloat16, "F16": torch.float16, "F64": torch.float64,
          "I64": torch.int64, "I32": torch.int32, "I16": torch.int16, "I8": torch.int8, "U8": torch.uint8,
          "BOOL": torch.bool}
NAMES = {v: k for k, v in DTYPES.items()}


class SafetensorsError(ValueError):
    pass


class SafetensorsFile:
    def __init__(self, path: str):
        self.path = path
        try:
            self._f = open(path, "rb")
        except FileNotFoundError:
            raise SafetensorsError(f"{path} not found") from None
        size = os.fstat(self._f.fileno()).st_size
        if size < 8:
            raise SafetensorsError(f"{path} is too short to be a safetensors file")
        (n,) = struct.unpack("<Q", self._f.read(8))
        if n > size - 8:
            raise SafetensorsError(f"{path}: header length {n} exceeds the file size {size}")
        try:
            header = json.loads(self._f.read(n))
        except (json.JSONDecodeError, UnicodeDecodeError) as e:
            raise SafetensorsError(f"{path}: header is not valid JSON: {e}") from None
        self.metadata = header.pop("__metadata__", {})
        self.entries: Dict[str, dict] = header
        self._data_start = 8 + n
        self._mm = mmap.mmap(self._f.fileno(), 0, access=mmap.ACCESS_READ) if size > 0 else None
        for name, e in self.entries.items():
            a, b = e["data_offsets"]
            if e["dtype"] not in DTYPES:
                raise SafetensorsError(f"{path}: tensor {name} has unknown dtype {e['dtype']}")
            count = 1
            for s in e["shape"]:
                count *= s
            if b - a != count * DTYPES[e["dtype"]].itemsize or self._data_start + b > size:
                raise SafetensorsError(f"{path}: tensor {name} has data offsets that do not fit its shape or the file")

    def names(self):
        return list(self.entries)

    def shape(self, name) -> Tuple[int, ...]:
        return tuple(self.entries[name]["shape"])

    def dtype(self, name) -> torch.dtype:
        return DTYPES[self.entries[name]["dtype"]]

    def tensor(self, name) -> torch.Tensor:
        """A CPU tensor that views the mapped file; copy or move it before the file is closed."""
        e = self.entries[name]
        a, _ = e["data_offsets"]
        count = 1
        for s in e["shape"]:
            count *= s
        if count == 0:
            return torch.empty(e["shape"], dtype=DTYPES[e["dtype"]])
        with warnings.catch_warnings():
            warnings.simplefilter("ignore", UserWarning)  # the map is read-only; nothing writes through the view
            t = torch.frombuffer(self._mm, dtype=DTYPES[e["dtype"]], count=count, offset=self._data_start + a)
        return t.reshape(e["shape"])

    def close(self):
        # The map is not closed by hand: tensors made by tensor() may still view it, and each of
        # them keeps the map alive; it is unmapped when the last of them is gone.
        self._mm = None
        self._f.close()


def open_folder(folder: str) -> Dict[str, SafetensorsFile]:
    """name -> the file that holds it, for a model folder (single file or sharded)."""
    index = os.path.join(folder, "model.safetensors.index.json")
    single = os.path.join(folder, "model.safetensors")
    out: Dict[str, SafetensorsFile] = {}
    if os.path.exists(single):
        f = SafetensorsFile(single)
        return {n: f for n in f.names()}
    if os.path.exists(index):
        with open(index) as fh:
            wm = json.load(fh).get("weight_map", {})
        files = {}
        for name, fn in wm.items():
            if fn not in files:
                files[fn] = SafetensorsFile(os.path.join(folder, fn))
            if name not in files[fn].entries:
                raise SafetensorsError(f"{index} places {name} in {fn}, which does not hold it")
            out[name] = files[fn]
        return out
    raise SafetensorsError(f"{folder} holds neither model.safetensors nor model.safetensors.index.json")


def write_file(path: str, tensors: Iterable[Tuple[str, torch.Tensor]], metadata=None) -> None:
    """Write (name, tensor) pairs in the order given.  Tensors are taken one at a time, so the
    iterable may make them lazily; the header is written last-known-size first by a dry pass
    over shapes, hence the iterable is consumed once into a list of CPU tensors' bytes on disk."""
    tmp_data = path + ".data.tmp"
    header = {}
    offset = 0
    with open(tmp_data, "wb") as df:
        for name, t in tensors:
            t = t.detach().to("cpu").contiguous()
            if t.dtype not in NAMES:
                raise SafetensorsError(f"cannot store dtype {t.dtype} of {name}")
            raw = t.reshape(-1).view(torch.uint8).numpy().tobytes() if t.numel() else b""
            df.write(raw)
            header[name] = {"dtype": NAMES[t.dtype], "shape": list(t.shape), "data_offsets": [offset, offset + len(raw)]}
            offset += len(raw)
    if metadata:
        header = {"__metadata__": {str(k): str(v) for k, v in metadata.items()}, **header}
    hb = json.dumps(header, separators=(",", ":")).encode()
    hb += b" " * ((8 - len(hb) % 8) % 8)
    with open(path, "wb") as f, open(tmp_data, "rb") as df:
        f.write(struct.pack("<Q", len(hb)))
        f.write(hb)
        while True:
            chunk = df.read(1 << 24)
            if not chunk:
                break
            f.write(chunk)
    os.remove(tmp_data)
