"""Reading and writing safetensors files by tensor name.

Layout: 8 bytes little-endian header length, a JSON header
{name: {dtype, shape, data_offsets}} ("__metadata__" ignored), then the raw
little-endian tensor bytes; a model folder may hold several such files. It is
the layout the reference's own oracle reads (tools/quant_bench/ref_qwen3.py:45-62).
Files are memory-mapped, so a tensor's bytes are only touched when it is fetched.
"""
from __future__ import annotations

import glob
import json
import os
import struct

import numpy as np
import torch


class WeightsError(RuntimeError):
    pass


# safetensors dtype -> (numpy dtype to map the bytes, torch dtype of the result)
_DTYPES = {
    "F32": (np.float32, torch.float32),
    "F16": (np.float16, torch.float16),
    "BF16": (np.uint16, torch.bfloat16),
    "I32": (np.int32, torch.int32),
    "I64": (np.int64, torch.int64),
    "U8": (np.uint8, torch.uint8),
}
_TORCH_TO_ST = {torch.float32: "F32", torch.float16: "F16", torch.bfloat16: "BF16",
                torch.int32: "I32", torch.int64: "I64", torch.uint8: "U8"}


class SafetensorsFile:
    def __init__(self, path: str):
        self.path = path
        size = os.path.getsize(path)
        with open(path, "rb") as f:
            head = f.read(8)
            if len(head) < 8:
                raise WeightsError(f"{path}: truncated (no header length)")
            (n,) = struct.unpack("<Q", head)
            if n <= 0 or 8 + n > size:
                raise WeightsError(f"{path}: header length {n} does not fit the file of {size} bytes")
            try:
                header = json.loads(f.read(n))
            except (json.JSONDecodeError, UnicodeDecodeError) as exc:
                raise WeightsError(f"{path}: header is not valid JSON: {exc}") from None
        header.pop("__metadata__", None)
        self.data_start = 8 + n
        self.entries: dict[str, dict] = {}
        for name, e in header.items():
            if e.get("dtype") not in _DTYPES:
                raise WeightsError(f"{path}: tensor '{name}' has unsupported dtype {e.get('dtype')!r}")
            try:
                a, b = (int(x) for x in e["data_offsets"])
            except (KeyError, TypeError, ValueError):
                raise WeightsError(f"{path}: tensor '{name}' has no valid data_offsets") from None
            if a < 0 or a > b:
                raise WeightsError(f"{path}: tensor '{name}' has data_offsets [{a}, {b}]")
            count = int(np.prod(e["shape"], dtype=np.int64)) if e["shape"] else 1
            want = count * np.dtype(_DTYPES[e["dtype"]][0]).itemsize
            if b - a != want:
                raise WeightsError(f"{path}: tensor '{name}' spans {b - a} bytes, its shape "
                                   f"{e['shape']} and dtype {e['dtype']} need {want}")
            if self.data_start + b > size:
                raise WeightsError(f"{path}: truncated, tensor '{name}' ends at byte "
                                   f"{self.data_start + b} of {size}")
            self.entries[name] = e
        self._map = None

    def names(self):
        return self.entries.keys()

    def shape(self, name: str) -> tuple:
        return tuple(self.entries[name]["shape"])

    def stored_dtype(self, name: str) -> torch.dtype:
        return _DTYPES[self.entries[name]["dtype"]][1]

    def tensor(self, name: str) -> torch.Tensor:
        """The tensor as stored, on the CPU, backed by the file mapping."""
        e = self.entries[name]
        if self._map is None:
            self._map = np.memmap(self.path, dtype=np.uint8, mode="r")
        np_dtype, t_dtype = _DTYPES[e["dtype"]]
        a, b = e["data_offsets"]
        raw = self._map[self.data_start + a:self.data_start + b]
        arr = np.frombuffer(raw, dtype=np_dtype).reshape(e["shape"])
        import warnings
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")  # the mapping is read-only; it is never written through
            t = torch.from_numpy(arr)
        return t.view(torch.bfloat16) if e["dtype"] == "BF16" else t


def open_model_files(model_dir: str) -> list[SafetensorsFile]:
    """Every *.safetensors of the folder; with model.safetensors.index.json the
    shards it names must all be present."""
    index = os.path.join(model_dir, "model.safetensors.index.json")
    paths = sorted(glob.glob(os.path.join(model_dir, "*.safetensors")))
    if os.path.exists(index):
        with open(index) as f:
            wanted = sorted(set(json.load(f).get("weight_map", {}).values()))
        missing = [w for w in wanted if not os.path.exists(os.path.join(model_dir, w))]
        if missing:
            raise WeightsError(f"{model_dir}: shards named by the index are missing: {missing}")
    if not paths:
        raise WeightsError(f"{model_dir}: no .safetensors file found")
    return [SafetensorsFile(p) for p in paths]


def write_safetensors(path: str, tensors: dict[str, torch.Tensor], metadata: dict | None = None) -> None:
    header: dict = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    offset = 0
    blobs = []
    for name, t in tensors.items():
        t = t.detach().cpu().contiguous()
        if t.dtype not in _TORCH_TO_ST:
            raise WeightsError(f"cannot store tensor '{name}' of dtype {t.dtype}")
        raw = (t.view(torch.uint16) if t.dtype == torch.bfloat16 else t).numpy().tobytes()
        header[name] = {"dtype": _TORCH_TO_ST[t.dtype], "shape": list(t.shape),
                        "data_offsets": [offset, offset + len(raw)]}
        offset += len(raw)
        blobs.append(raw)
    head = json.dumps(header, separators=(",", ":")).encode()
    head += b" " * ((8 - len(head) % 8) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(head)))
        f.write(head)
        for raw in blobs:
            f.write(raw)
