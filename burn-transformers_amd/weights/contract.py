"""The contract between a checkpoint and a model: which tensors, which shapes, which layout.

A family states its contract as a list of :class:`TensorSpec`.  The check compares it with the
headers of the files and raises ONE error that lists every missing tensor, every unexpected
tensor and every wrong shape or dtype, before any payload is read or any tensor is placed on
the GPU (the reference validates strictly and completely before the first write as well,
src/checkpoint/mapping.rs:480-588, src/models/gpt2/model_tests.rs:700-737).
"""

import re
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Tuple

from .safetensors_io import FLOAT_DTYPES

# How a tensor is held once loaded:
#   "in_out"  a projection stored [in, out] (GPT-2's Conv1D); held transposed, [out, in], in the
#             compute dtype, because every matrix product here reads K-contiguous rows
#   "out_in"  a projection stored [out, in]; held as stored, compute dtype
#   "table"   an embedding table [rows, width]; held as stored, compute dtype
#   "vector"  a bias or a norm's scale or shift; always held in float32 (exact for any storage)
#   "int"     an integer table; held as int32
LAYOUTS = ("in_out", "out_in", "table", "vector", "int")


@dataclass(frozen=True)
class TensorSpec:
    name: str
    shape: Tuple[int, ...]
    layout: str

    def __post_init__(self):
        if self.layout not in LAYOUTS:
            raise ValueError(f"unknown layout {self.layout!r}")


@dataclass
class Contract:
    tensors: List[TensorSpec]
    # the same tensors may sit below one of these prefixes; exactly one must hold the anchor
    prefixes: Tuple[str, ...] = ("",)
    anchor: Optional[str] = None
    # regular expressions (full match, prefix removed) of tensors that are skipped when present
    ignored: Tuple[str, ...] = ()
    # alias name -> owner name: if the alias is stored it must be bit-equal to its owner
    aliases: Dict[str, str] = field(default_factory=dict)


class WeightError(ValueError):
    """The checkpoint does not fit the model.  ``missing``, ``unexpected`` and ``mismatched``
    hold the details that the message lists."""

    def __init__(self, where, missing=(), unexpected=(), mismatched=(), other=()):
        self.missing, self.unexpected = list(missing), list(unexpected)
        self.mismatched, self.other = list(mismatched), list(other)
        lines = [f"{where}: the checkpoint does not fit the model"]
        if self.other:
            lines += [f"  {text}" for text in self.other]
        if self.missing:
            lines.append(f"  missing tensors ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected tensors ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        if self.mismatched:
            lines.append(f"  wrong shape or dtype ({len(self.mismatched)}):")
            lines += [f"    {text}" for text in self.mismatched]
        super().__init__("\n".join(lines))


def detect_prefix(names, contract, where):
    """The one namespace that holds the anchor tensor (src/models/gpt2/checkpoint.rs:61-71)."""
    if contract.anchor is None:
        return contract.prefixes[0]
    holding = [p for p in contract.prefixes if p + contract.anchor in names]
    if len(holding) != 1:
        tried = ", ".join(f"`{p}{contract.anchor}`" for p in contract.prefixes)
        raise WeightError(where, other=[
            f"expected exactly one of {tried}, found {len(holding)}"])
    return holding[0]


def check(entries, contract, where, listed_only=()):
    """Compares the entries of the files (name -> Entry) with the contract.

    Returns (prefix, {spec name: entry}, [stored alias names]).  ``listed_only`` are names an
    index lists although no file holds them (a tied head may be recorded that way).
    """
    names = set(entries)
    prefix = detect_prefix(names, contract, where)
    ignored = [re.compile(pattern) for pattern in contract.ignored]
    wanted = {prefix + spec.name: spec for spec in contract.tensors}
    missing = [name for name in wanted if name not in names]
    unexpected, mismatched, stored_aliases = [], [], []
    for name in sorted(names):
        if name in wanted:
            spec, entry = wanted[name], entries[name]
            if tuple(entry.shape) != tuple(spec.shape):
                mismatched.append(f"{name}: stored {entry.dtype}{list(entry.shape)}, the model needs {list(spec.shape)}")
            elif spec.layout == "int" and entry.dtype in FLOAT_DTYPES:
                mismatched.append(f"{name}: an integer table is stored as {entry.dtype}")
            elif spec.layout != "int" and entry.dtype not in FLOAT_DTYPES:
                mismatched.append(f"{name}: parameters must be floating point, stored as {entry.dtype}")
            continue
        bare = name[len(prefix):] if name.startswith(prefix) else name
        if bare in contract.aliases or name in contract.aliases:
            alias = bare if bare in contract.aliases else name
            owner = wanted.get(prefix + contract.aliases[alias])
            if owner is not None and tuple(entries[name].shape) != tuple(owner.shape):
                mismatched.append(f"{name}: stored {list(entries[name].shape)}, its owner "
                                  f"{owner.name} is {list(owner.shape)}")
            stored_aliases.append((name, contract.aliases[alias]))
            continue
        if name.startswith(prefix) and any(p.fullmatch(bare) for p in ignored):
            continue
        unexpected.append(name)
    for name in listed_only:
        bare = name[len(prefix):] if name.startswith(prefix) else name
        if name not in names and bare not in contract.aliases and name not in contract.aliases \
                and name not in wanted:
            unexpected.append(name + " (listed in the index only)")
    if missing or unexpected or mismatched:
        raise WeightError(where, sorted(missing), unexpected, mismatched)
    return prefix, {spec.name: entries[prefix + spec.name] for spec in contract.tensors}, stored_aliases
