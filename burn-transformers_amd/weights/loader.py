"""Loads a checkpoint into GPU tensors under the model's own tensor names.

Two passes, like the reference (src/models/auto/load.rs:175-204): headers of every file are
read and checked against the family's contract first; only then are payloads read, one tensor
at a time, converted once (round to nearest even when narrowing) and placed on the device.
"""

from dataclasses import replace

import torch

from .contract import WeightError, check
from .safetensors_io import PayloadReader, discover, read_header

COMPUTE_DTYPES = {"float32": torch.float32, "fp32": torch.float32, "f32": torch.float32,
                  "bfloat16": torch.bfloat16, "bf16": torch.bfloat16}


def compute_dtype(name):
    """torch dtype of a ``--dtype`` value."""
    if isinstance(name, torch.dtype):
        if name in (torch.float32, torch.bfloat16):
            return name
    elif name in COMPUTE_DTYPES:
        return COMPUTE_DTYPES[name]
    raise ValueError(f"dtype must be bfloat16 or float32, got {name!r}")


class WeightStore(dict):
    """name -> tensor on the device, in the layout the parts use; remembers how to undo it, and
    what loading did (``report``: the reference's LoadReport, src/checkpoint/report.rs)."""

    def __init__(self, dtype, device):
        super().__init__()
        self.dtype, self.device, self.layouts = dtype, device, {}
        # namespace: the prefix the checkpoint's names carry; applied: tensors placed; converted:
        # {"F32->bfloat16": count, ...} of those whose precision changed; aliased: stored names that
        # are tied to an owner and were only compared with it; ignored: stored names the family
        # lets be (legacy buffers)
        self.report = {"namespace": "", "applied": 0, "converted": {}, "aliased": [], "ignored": []}

    def export(self):
        """The tensors back in checkpoint layout (float32, CPU), for tests and for saving."""
        out = {}
        for name, tensor in self.items():
            value = tensor.detach().to("cpu", torch.float32)
            out[name] = value.t().contiguous() if self.layouts[name] == "in_out" else value
        return out


def place(store, spec, tensor):
    """Converts one CPU tensor in checkpoint layout and puts it into the store."""
    tensor = tensor.to(store.device)
    if spec.layout == "vector":
        value = tensor.to(torch.float32)
    elif spec.layout == "int":
        value = tensor.to(torch.int32)
    elif spec.layout == "in_out":
        value = tensor.to(store.dtype).t().contiguous()
    else:
        value = tensor.to(store.dtype).contiguous()
    store[spec.name] = value
    store.layouts[spec.name] = spec.layout
    store.report["applied"] += 1
    if value.dtype != tensor.dtype:
        change = f"{str(tensor.dtype).replace('torch.', '')}->{str(value.dtype).replace('torch.', '')}"
        store.report["converted"][change] = store.report["converted"].get(change, 0) + 1


def store_from_tensors(tensors, contract, dtype, device, where="tensors"):
    """Builds the store from in-memory CPU tensors under checkpoint names (no prefix)."""
    class _Held:
        def __init__(self, tensor):
            self.shape = tuple(tensor.shape)
            self.dtype = {torch.float32: "F32", torch.bfloat16: "BF16", torch.float16: "F16",
                          torch.float64: "F64", torch.int32: "I32", torch.int64: "I64"}.get(tensor.dtype, "U8")
    bare = replace(contract, prefixes=("",))
    check({name: _Held(t) for name, t in tensors.items()}, bare, where)
    store = WeightStore(dtype, device)
    for spec in contract.tensors:
        place(store, spec, tensors[spec.name])
    return store


def load_checkpoint(model_dir, contract, dtype, device):
    """The model's tensors from the safetensors files of ``model_dir``."""
    files, listed = discover(model_dir)
    entries = {}
    for path in files:
        for name, entry in read_header(path).items():
            if name in entries:
                raise WeightError(model_dir, other=[f"tensor {name} is stored in two files"])
            entries[name] = entry
    prefix, by_spec, stored_aliases = check(entries, contract, model_dir, listed - set(entries))
    reader = PayloadReader()
    try:
        for alias, owner in stored_aliases:        # before anything is placed on the device
            alias_tensor = reader.tensor(entries[alias])
            owner_tensor = reader.tensor(by_spec[owner])
            if alias_tensor.dtype != owner_tensor.dtype or not torch.equal(
                    alias_tensor.view(torch.uint8), owner_tensor.view(torch.uint8)):
                raise WeightError(model_dir, other=[
                    f"{alias} is stored separately and differs from {owner}, to which it must be tied"])
        store = WeightStore(dtype, device)
        for spec in contract.tensors:
            place(store, spec, reader.tensor(by_spec[spec.name]))
    finally:
        reader.close()
    used = {prefix + spec.name for spec in contract.tensors} | {alias for alias, _ in stored_aliases}
    store.report.update(namespace=prefix, aliased=sorted(alias for alias, _ in stored_aliases),
                        ignored=sorted(set(entries) - used))
    return store
