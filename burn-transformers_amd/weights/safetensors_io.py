"""Reading and writing safetensors files without any tensor library's model code.

Format: 8 bytes little-endian header length, a JSON header {name: {dtype, shape, data_offsets}},
then the payload.  The header is checked completely (every byte range has the size its shape
and dtype give, ranges do not overlap and stay inside the file) before any payload is read
(the reference does the same, src/checkpoint/artifact.rs:1-11).
"""

import json
import math
import mmap
import os
import struct

import numpy as np
import torch

MAX_HEADER_BYTES = 100 * 10 ** 6     # src/checkpoint/options.rs:69-81
MAX_TENSORS = 10 * 10 ** 6
MAX_RANK = 32

DTYPES = {
    "F64": (8, torch.float64), "F32": (4, torch.float32), "F16": (2, torch.float16),
    "BF16": (2, torch.bfloat16), "I64": (8, torch.int64), "I32": (4, torch.int32),
    "I16": (2, torch.int16), "I8": (1, torch.int8), "U8": (1, torch.uint8), "BOOL": (1, torch.bool),
}
FLOAT_DTYPES = ("F64", "F32", "F16", "BF16")
_NAMES = {torch_dtype: name for name, (_, torch_dtype) in DTYPES.items()}
_NUMPY_VIEW = {1: np.uint8, 2: np.int16, 4: np.int32, 8: np.int64}


class SafetensorsError(ValueError):
    """The file is not a well-formed safetensors file."""


class Entry:
    """One tensor of one file: name, dtype name, shape, byte range in the payload."""
    __slots__ = ("name", "dtype", "shape", "begin", "end", "path", "payload_start")

    def __init__(self, name, dtype, shape, begin, end, path, payload_start):
        self.name, self.dtype, self.shape = name, dtype, tuple(shape)
        self.begin, self.end, self.path, self.payload_start = begin, end, path, payload_start


def read_header(path):
    """All entries of a file, validated; no payload byte is touched."""
    size = os.path.getsize(path)
    with open(path, "rb") as handle:
        prefix = handle.read(8)
        if len(prefix) != 8:
            raise SafetensorsError(f"{path}: shorter than its 8-byte header length")
        (header_len,) = struct.unpack("<Q", prefix)
        if header_len > MAX_HEADER_BYTES or 8 + header_len > size:
            raise SafetensorsError(f"{path}: header length {header_len} does not fit the file")
        try:
            header = json.loads(handle.read(header_len))
        except ValueError as error:
            raise SafetensorsError(f"{path}: header is not JSON ({error})") from error
    if not isinstance(header, dict):
        raise SafetensorsError(f"{path}: header must be an object")
    if len(header) > MAX_TENSORS:
        raise SafetensorsError(f"{path}: {len(header)} tensors, at most {MAX_TENSORS} are read")
    payload_start = 8 + header_len
    payload_size = size - payload_start
    entries, ranges = {}, []
    for name, info in header.items():
        if name == "__metadata__":
            continue
        try:
            dtype, shape, (begin, end) = info["dtype"], info["shape"], info["data_offsets"]
        except (KeyError, TypeError, ValueError) as error:
            raise SafetensorsError(f"{path}: malformed entry for {name!r}") from error
        if dtype not in DTYPES:
            raise SafetensorsError(f"{path}: tensor {name!r} has unsupported dtype {dtype!r}")
        if len(shape) > MAX_RANK or any((not isinstance(s, int)) or s < 0 for s in shape):
            raise SafetensorsError(f"{path}: tensor {name!r} has a bad shape {shape!r}")
        want = math.prod(shape) * DTYPES[dtype][0]
        if not (0 <= begin <= end <= payload_size) or end - begin != want:
            raise SafetensorsError(
                f"{path}: tensor {name!r} {dtype}{list(shape)} needs {want} bytes, its range is [{begin}, {end})")
        entries[name] = Entry(name, dtype, shape, begin, end, path, payload_start)
        ranges.append((begin, end, name))
    # the ranges tile the payload: they start at its first byte, follow each other without overlap
    # or gap, and end at its last (src/checkpoint/artifact.rs:1-11)
    ranges.sort()
    for (_, end_a, name_a), (begin_b, _, name_b) in zip(ranges, ranges[1:]):
        if begin_b < end_a:
            raise SafetensorsError(f"{path}: tensors {name_a!r} and {name_b!r} overlap")
        if begin_b > end_a:
            raise SafetensorsError(f"{path}: {begin_b - end_a} bytes between tensors {name_a!r} and {name_b!r} belong to no tensor")
    if ranges and (ranges[0][0] != 0 or ranges[-1][1] != payload_size):
        raise SafetensorsError(f"{path}: the tensors cover bytes [{ranges[0][0]}, {ranges[-1][1]}) of a payload of {payload_size}")
    return entries


class PayloadReader:
    """Memory-maps the files of a checkpoint and hands out tensors one at a time."""

    def __init__(self):
        self._maps = {}

    def tensor(self, entry):
        """A CPU torch tensor that owns a copy of the entry's bytes."""
        mapped = self._maps.get(entry.path)
        if mapped is None:
            with open(entry.path, "rb") as handle:
                mapped = mmap.mmap(handle.fileno(), 0, access=mmap.ACCESS_READ)
            self._maps[entry.path] = mapped
        itemsize, torch_dtype = DTYPES[entry.dtype]
        count = math.prod(entry.shape)
        raw = np.frombuffer(mapped, dtype=_NUMPY_VIEW[itemsize], count=count,
                            offset=entry.payload_start + entry.begin)
        tensor = torch.from_numpy(raw.copy())
        if torch_dtype == torch.bool:
            tensor = tensor.view(torch.uint8).to(torch.bool)
        else:
            tensor = tensor.view(torch_dtype)
        return tensor.reshape(entry.shape)

    def close(self):
        for mapped in self._maps.values():
            mapped.close()
        self._maps.clear()


def write_safetensors(path, tensors, metadata=None):
    """Writes CPU tensors (name -> tensor) in name order."""
    header, offset, blobs = {}, 0, []
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    for name in sorted(tensors):
        tensor = tensors[name].detach().cpu().contiguous()
        if tensor.dtype not in _NAMES:
            raise SafetensorsError(f"cannot store {name!r} of dtype {tensor.dtype}")
        itemsize = DTYPES[_NAMES[tensor.dtype]][0]
        view = tensor.view(torch.uint8) if tensor.dtype == torch.bool else tensor
        data = view.reshape(-1).view({1: torch.uint8, 2: torch.int16, 4: torch.int32, 8: torch.int64}[itemsize])
        blob = data.numpy().tobytes()
        header[name] = {"dtype": _NAMES[tensor.dtype], "shape": list(tensor.shape),
                        "data_offsets": [offset, offset + len(blob)]}
        offset += len(blob)
        blobs.append(blob)
    encoded = json.dumps(header, separators=(",", ":")).encode()
    encoded += b" " * (-len(encoded) % 8)
    with open(path, "wb") as handle:
        handle.write(struct.pack("<Q", len(encoded)))
        handle.write(encoded)
        for blob in blobs:
            handle.write(blob)


def discover(model_dir):
    """The safetensors files of a model folder: an index, ``model.safetensors``, or the one
    ``*.safetensors`` file there is (src/checkpoint/options.rs:86-110).  Returns
    (list of file paths, set of names that the index lists without a file holding them)."""
    root = os.path.realpath(model_dir)
    index = os.path.join(root, "model.safetensors.index.json")
    if os.path.isfile(index):
        with open(index) as handle:
            weight_map = json.load(handle).get("weight_map", {})
        files = []
        for shard in sorted(set(weight_map.values())):
            path = os.path.realpath(os.path.join(root, shard))
            if os.path.commonpath([root, path]) != root:
                raise SafetensorsError(f"{index}: shard {shard!r} leaves the model folder")
            files.append(path)
        return files, set(weight_map)
    single = os.path.join(root, "model.safetensors")
    if os.path.isfile(single):
        return [single], set()
    found = sorted(f for f in os.listdir(root) if f.endswith(".safetensors"))
    if len(found) == 1:
        return [os.path.join(root, found[0])], set()
    raise FileNotFoundError(
        f"{model_dir}: expected model.safetensors, an index, or exactly one .safetensors file; found {found}")
