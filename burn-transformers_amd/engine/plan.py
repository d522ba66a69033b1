"""A model as data: which parts each layer is made of and in which order layers run.

A family turns its configuration into a :class:`ModelPlan`; the builder (``engine/model.py``)
turns the plan into parts by looking every ``kind`` up in the part registries.  Nothing here
knows an architecture.
"""

from dataclasses import dataclass, field
from typing import Dict, List, Optional


@dataclass
class PartSpec:
    """One part: its kind (a name in a part registry), its sizes and constants, and the names of
    the tensors it uses (role -> name in the weight store)."""
    kind: str
    params: Dict[str, object] = field(default_factory=dict)
    tensors: Dict[str, str] = field(default_factory=dict)


@dataclass
class LayerPlan:
    """One layer: the arrangement of its parts (a block kind) and the parts themselves."""
    block: str
    parts: Dict[str, PartSpec]


@dataclass
class ScheduleEntry:
    """One run of a layer.  ``cache`` numbers the cache entry its mixer uses; two schedule entries
    with the same number share keys and values, and only the one with ``writes`` fills them."""
    layer: int
    cache: Optional[int]
    writes: bool = True


@dataclass
class ModelPlan:
    width: int
    vocab_size: int
    max_positions: int
    embedding: PartSpec
    layers: List[LayerPlan]
    schedule: List[ScheduleEntry]
    final_norm: PartSpec
    readout: PartSpec
