"""Reading and writing safetensors files.

The format: 8 bytes little-endian header length, a JSON header
``{name: {"dtype", "shape", "data_offsets": [begin, end]}}``, then the tensors' raw
little-endian data.  Files are memory-mapped, so a tensor's bytes are paged in only
when it is copied to the device.  The reference reads the same format through the
safetensors package in its converter (scripts/convert_hf_checkpoint.py:84-90).
"""
import json
import mmap
import os
from typing import Dict, List, Tuple

import torch

_DTYPES = {
    "F64": torch.float64, "F32": torch.float32, "F16": torch.float16,
    "BF16": torch.bfloat16, "I64": torch.int64, "I32": torch.int32,
    "I16": torch.int16, "I8": torch.int8, "U8": torch.uint8, "BOOL": torch.bool,
}
_NAMES = {v: k for k, v in _DTYPES.items()}


class SafetensorsFile:
    """One memory-mapped file; ``entries`` maps a tensor name to (dtype name, shape)."""

    def __init__(self, path: str):
        self.path = path
        with open(path, "rb") as f:
            size = os.fstat(f.fileno()).st_size
            if size < 8:
                raise ValueError(f"{path}: too short for a safetensors file")
            self._map = mmap.mmap(f.fileno(), 0, access=mmap.ACCESS_READ)
        n = int.from_bytes(self._map[:8], "little")
        if 8 + n > size:
            raise ValueError(f"{path}: header length {n} exceeds the file")
        header = json.loads(self._map[8:8 + n].decode("utf-8"))
        self._base = 8 + n
        self._meta = {k: v for k, v in header.items() if k != "__metadata__"}
        self.entries: Dict[str, Tuple[str, Tuple[int, ...]]] = {}
        for name, m in self._meta.items():
            if m["dtype"] not in _DTYPES:
                raise ValueError(f"{path}: tensor {name} has unknown dtype {m['dtype']}")
            lo, hi = m["data_offsets"]
            count = 1
            for s in m["shape"]:
                count *= s
            width = torch.empty((), dtype=_DTYPES[m["dtype"]]).element_size()
            if hi - lo != count * width or self._base + hi > size:
                raise ValueError(f"{path}: tensor {name} has inconsistent offsets")
            self.entries[name] = (m["dtype"], tuple(m["shape"]))

    def tensor(self, name: str) -> torch.Tensor:
        """A CPU tensor that views the mapped bytes (read-only; copy before writing)."""
        m = self._meta[name]
        lo, hi = m["data_offsets"]
        dtype = _DTYPES[m["dtype"]]
        count = 1
        for s in m["shape"]:
            count *= s
        if count == 0:
            return torch.empty(m["shape"], dtype=dtype)
        import warnings
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")     # "buffer is not writable"
            t = torch.frombuffer(self._map, dtype=dtype, count=count,
                                 offset=self._base + lo)
        return t.reshape(m["shape"])


def open_model_files(folder: str) -> List[SafetensorsFile]:
    """The safetensors files of a model folder: those named by
    ``model.safetensors.index.json`` if there is one, else ``model.safetensors``
    (the reference looks for the index first, scripts/convert_hf_checkpoint.py:35-53)."""
    index = os.path.join(folder, "model.safetensors.index.json")
    if os.path.isfile(index):
        with open(index) as f:
            names = sorted(set(json.load(f)["weight_map"].values()))
        return [SafetensorsFile(os.path.join(folder, n)) for n in names]
    single = os.path.join(folder, "model.safetensors")
    if os.path.isfile(single):
        return [SafetensorsFile(single)]
    raise FileNotFoundError(
        f"{folder}: neither model.safetensors.index.json nor model.safetensors")


def write_safetensors(path: str, tensors: Dict[str, torch.Tensor]) -> None:
    """Write CPU tensors under their names, data in the order given."""
    header = {}
    offset = 0
    blobs = []
    for name, t in tensors.items():
        t = t.detach().contiguous().cpu()
        if t.dtype not in _NAMES:
            raise ValueError(f"{name}: dtype {t.dtype} cannot be stored")
        n = t.numel() * t.element_size()
        header[name] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape),
                        "data_offsets": [offset, offset + n]}
        offset += n
        blobs.append(t)
    raw = json.dumps(header, separators=(",", ":")).encode("utf-8")
    raw += b" " * ((8 - len(raw) % 8) % 8)
    with open(path, "wb") as f:
        f.write(len(raw).to_bytes(8, "little"))
        f.write(raw)
        for t in blobs:
            if t.numel():
                f.write(t.reshape(-1).view(torch.uint8).numpy().data)      # the bytes as they lie, no copy
