"""Builds a model from a plan and a weight store, and runs its forward pass for one step.

The model is what the registry hands out for an architecture name: embedding, the layers made
of registered parts, the schedule in which they run, the final norm and the readout.  It holds
no sizes of its own; everything comes from the plan (and so from config.json).
"""

from ..config.base import read_config_json
from ..config.registry import resolve_family
from ..kernels import library as K
from ..parts import Memory, lookup
from ..parts.base import offers_chunked
from ..weights.loader import compute_dtype, load_checkpoint, store_from_tensors


def build_part(role, spec, store):
    missing = [name for name in spec.tensors.values() if name not in store]
    if missing:
        raise KeyError(f"{role} {spec.kind!r} asks for tensors the weight store does not hold: {missing}")
    return lookup(role, spec.kind)(spec.params, {r: store[name] for r, name in spec.tensors.items()})


class CausalLM:
    def __init__(self, plan, store, config=None, family=None):
        self.plan, self.store, self.config, self.family = plan, store, config, family
        self.dtype, self.device = store.dtype, store.device
        self.load_report = getattr(store, "report", None)      # what loading did with the checkpoint's tensors
        self.width, self.vocab_size, self.max_positions = plan.width, plan.vocab_size, plan.max_positions
        self.embedding = build_part("embedding", plan.embedding, store)
        self.blocks = []
        for layer in plan.layers:
            block_class = lookup("block", layer.block)
            unknown = set(layer.parts) - set(block_class.ROLES)
            absent = set(block_class.ROLES) - set(layer.parts)
            if unknown or absent:
                raise ValueError(f"block {layer.block!r} takes parts {sorted(block_class.ROLES)}, "
                                 f"the plan gives {sorted(layer.parts)}")
            self.blocks.append(block_class({name: build_part(block_class.ROLES[name], spec, store)
                                            for name, spec in layer.parts.items()}))
        self.final_norm = build_part("norm", plan.final_norm, store)
        self.readout = build_part("readout", plan.readout, store)
        self.schedule = list(plan.schedule)
        self._check_schedule()
        # a step of this model can be kept as a launch list if every part only launches kernels
        self.recordable = all(block.recordable() for block in self.blocks) and \
            all(part.only_launches_kernels for part in (self.embedding, self.final_norm, self.readout))
        parts = [self.embedding, self.final_norm, self.readout] + [p for block in self.blocks for p in block.parts.values()]
        K.prepare(self.dtype, sorted({name for part in parts for name in part.kernel_modules(self.dtype)}))

    def _check_schedule(self):
        """Every cache entry has exactly one writer, which runs before any reader, and readers keep
        what the writer keeps."""
        writers = {}
        for position, entry in enumerate(self.schedule):
            if not (0 <= entry.layer < len(self.blocks)):
                raise ValueError(f"schedule entry {position} names layer {entry.layer}, "
                                 f"the model has {len(self.blocks)}")
            if entry.cache is None:
                continue
            specs = self.blocks[entry.layer].cache_needs()
            if entry.writes:
                if entry.cache in writers:
                    raise ValueError(f"cache entry {entry.cache} has two writers in the schedule")
                writers[entry.cache] = specs
            elif entry.cache not in writers:
                raise ValueError(f"schedule entry {position} reads cache entry {entry.cache} before it is written")
            elif writers[entry.cache] != specs:
                raise ValueError(f"schedule entry {position} reads cache entry {entry.cache}, "
                                 f"whose keys and values have another shape")
        self.cache_entries = max(writers) + 1 if writers else 0
        self.kv_specs = [writers.get(i, (None, None))[0] for i in range(self.cache_entries)]
        self.state_specs = [writers.get(i, (None, None))[1] for i in range(self.cache_entries)]

    def forward(self, step, cache, readout=True):
        """Logits (float32 [len(step.sel_rows), vocab]) of the step's wanted rows; with
        ``readout=False`` the layers only fill the cache and nothing is returned."""
        with K.one_stream():          # the hundreds of launches below ask for the current stream once
            stream = self.embedding.embed(step)
            for entry in self.schedule:
                memory = Memory(cache, entry.cache, entry.writes, step) if entry.cache is not None else None
                self.blocks[entry.layer].forward(stream, step, memory)
            if not readout:
                return None
            if self.readout.takes_deferred_norm and offers_chunked(self.final_norm):
                hidden = self.final_norm.apply(stream, step, rows=step.sel_rows, chunked=True)
            else:
                hidden = self.final_norm.apply(stream, step, rows=step.sel_rows)
            return self.readout.logits(hidden, step)


    # --- the short way round ----------------------------------------------------------------
    @classmethod
    def from_pretrained(cls, model_dir, dtype="bfloat16", device=None):
        """``load_model`` under the name such loaders usually carry."""
        return load_model(model_dir, dtype, device)

    @classmethod
    def random(cls, config_json, seed=0, dtype="bfloat16", device=None):
        """A model with the random weights ``write_random_model`` writes for this seed (rounded to
        bfloat16 as it stores them), without the folder."""
        import torch
        from ..weights.random_init import random_tensors
        _, tensors = random_tensors(config_json, seed)
        return model_from_tensors(config_json, {k: v.to(torch.bfloat16) for k, v in tensors.items()}, dtype, device)

    def engine(self, max_tokens, **options):
        """An engine (cache and step function) for this model."""
        from .engine import Engine
        return Engine(self, max_tokens, **options)

    def generate(self, prompts, config=None, max_tokens=None, **options):
        """Generates for the prompts with an engine whose cache is as large as they need (or
        ``max_tokens``); see ``engine.generate.generate`` for the options."""
        from ..cache.ledger import BLOCK
        from ..sampling.config import GenerationConfig
        from .generate import generate
        config = config or GenerationConfig()
        if max_tokens is None:
            grows_to = lambda n: min(n + config.max_new_tokens, options.get("total_length") or self.max_positions)
            max_tokens = sum((grows_to(len(p)) + BLOCK - 1) // BLOCK * BLOCK for p in prompts)
        return generate(self.engine(max_tokens), prompts, config, **options)

    def export_weights(self):
        """The tensors back under their checkpoint names and layouts (float32, CPU)."""
        return self.store.export()


def _device(device):
    import torch
    K.require_gpu()
    return torch.device(device if device is not None else "cuda:0")


def load_model(model_dir, dtype="bfloat16", device=None):
    """The model of a folder with config.json and safetensors weights; the class of model is the
    one config.json names."""
    config_json = read_config_json(model_dir)
    family = resolve_family(config_json)
    config = family.config_class.from_dict(config_json)
    store = load_checkpoint(model_dir, family.contract(config), compute_dtype(dtype), _device(device))
    return CausalLM(family.plan(config), store, config, family)


def model_from_tensors(config_json, tensors, dtype="bfloat16", device=None):
    """The same model from in-memory tensors under checkpoint names (random weights, tests)."""
    family = resolve_family(config_json)
    config = family.config_class.from_dict(config_json)
    store = store_from_tensors(tensors, family.contract(config), compute_dtype(dtype), _device(device))
    return CausalLM(family.plan(config), store, config, family)
