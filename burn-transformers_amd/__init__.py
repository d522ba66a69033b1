"""burn_transformers_amd: a small causal-LM generation library for one AMD MI355X GPU.

    import burn_transformers_amd as bt
    model = bt.load_model("path/to/model", dtype="bfloat16")     # class chosen by config.json
    engine = bt.Engine(model, max_tokens=8192)
    out = bt.generate(engine, [[464, 1115, 4165]], bt.GenerationConfig(max_new_tokens=32))

The configuration, the registry, the weight contract, the cache ledger and the generation
bookkeeping import without a GPU; models, engines and kernels need one and say so.
"""

from . import architectures  # noqa: F401  (registers GPT-2)
from .cache.ledger import CacheFull, CacheLedger
from .config import (ConfigError, Family, GPT2Config, UnsupportedArchitecture, read_config_json,
                     register_family, resolve_family, supported_names, unregister_family)
from .engine.plan import LayerPlan, ModelPlan, PartSpec, ScheduleEntry
from .sampling import (FinishReason, GeneratedSequence, GenerationConfig, GenerationError,
                       GenerationTracker)
from .weights import (Contract, TensorSpec, WeightError, random_tensors, write_random_model,
                      write_safetensors)

__version__ = "0.1.0"

_LAZY = {
    "Engine": ("engine.engine", "Engine"), "StepError": ("engine.engine", "StepError"),
    "CausalLM": ("engine.model", "CausalLM"), "load_model": ("engine.model", "load_model"),
    "model_from_tensors": ("engine.model", "model_from_tensors"),
    "generate": ("engine.generate", "generate"), "generate_batch": ("engine.generate", "generate_batch"),
    "Replay": ("engine.replay", "Replay"), "Cache": ("cache.storage", "Cache"),
    "KVSpec": ("cache.storage", "KVSpec"), "StateSpec": ("cache.storage", "StateSpec"),
    "Sampler": ("sampling.sampler", "Sampler"),
}


def __getattr__(name):
    if name in _LAZY:
        import importlib
        module, attribute = _LAZY[name]
        return getattr(importlib.import_module(f"{__name__}.{module}"), attribute)
    raise AttributeError(f"module {__name__!r} has no attribute {name!r}")
