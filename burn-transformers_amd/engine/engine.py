"""The engine: a model, its cache and the ONE step function that everything above it uses
(generation, replay, benchmarks).

    engine = Engine(model, max_tokens=4096)
    slot = engine.open()                            # a sequence's handle
    logits = engine.step([(slot, [5, 17, 3])], want=[[0, 2]])   # float32 [2, vocab]
    logits = engine.step([(slot, [9])])             # one more token, logits of it
    engine.close(slot)                              # gives the slot and its blocks back

A step runs exactly the tokens it is given, as one packed batch without padding, against what
earlier steps left in the cache, and returns the logits of the wanted places.  Sequences of a
step may bring different numbers of tokens and stand at different lengths; whole prompts,
chunks of prompts and single tokens all take this path (the reference's forward_cached does
the same behind prefill and decode, src/models/llama/model/decode.rs:630-684).  Everything is
validated before anything changes, lengths advance only after the forward pass was launched
without error (decode.rs:38-41).

Steps are replayed from HIP graphs where their shape repeats: a step is hundreds of kernels,
and launching them one by one costs the host several microseconds each, more than the short
kernels of a decode step take to run.  A graph belongs to a shape (tokens, sequences, wanted
rows, most tokens of one sequence); what differs between steps of one shape (ids, positions,
block tables, wanted rows) lives in device tables that are filled before each replay.  A step
that is not replayed runs from its launch list, which a C++ loop walks: with that, and with the
host kept one step behind the GPU while decoding, a graph pays only where the kernels are so short
that launching them takes longer than running them (small models, small steps).  So a shape that
repeats is measured once from its list and captured only if the host was the limit.
"""

import time

import numpy as np
import torch

from ..cache.ledger import BLOCK
from ..cache.storage import Cache
from ..kernels import library as K
from .step import BufferPool, Step, StepLayout, StepPlan

_PINNED_RING = 4
_MAX_GRAPHS = 48           # graphs kept; the one that was used longest ago goes first
_MAX_PROGRAMS = 1024       # launch lists kept (a few hundred small structures each)
_META_WORDS = 1 << 16      # first size of the device buffer of a step's integer tables
_PROBES = 3                # steps of a shape that are measured before it is captured or left to its list


def launch_bound(samples):
    """From measured steps of one shape, each (seconds the GPU took from the step's first kernel
    to its last, seconds the host took to walk its launch list): True if the GPU is the limit, so
    that a graph would gain nothing.  Where the host is the limit the GPU waits for every launch
    and both times are about equal; where the kernels outlast their launches the GPU's time is the
    longer one.  The median ratio decides, so one odd sample (a first use, a clock still rising)
    does not."""
    ratios = sorted(gpu / max(host, 1e-9) for gpu, host in samples)
    return ratios[len(ratios) // 2] > 1.1


class StepError(ValueError):
    """The step was refused before anything ran; the cache is as it was."""


class Engine:
    def __init__(self, model, max_tokens, max_slots=None, graphs=True, programs=True):
        self.model = model
        self.device, self.dtype = model.device, model.dtype
        self.cache = Cache(model.kv_specs, model.state_specs, max_tokens, model.max_positions,
                           model.dtype, model.device, max_slots)
        self.pool = BufferPool(self.device)
        # a mixer that plans work on the host per step cannot be replayed from a graph
        # graphs: True (capture a repeating shape where a graph pays: see _graph_pays), "always"
        # (capture every repeating shape) or False
        self.use_graphs = bool(graphs) and all(mixer.graph_safe for block in model.blocks for mixer in block.mixers())
        self._graphs_always = graphs == "always"
        # Steps that are not replayed from a graph are kept as launch lists, one per shape, and walked
        # in C++ (kernels.library.Program), if every part of the model only launches kernels
        self.use_programs = programs and getattr(model, "recordable", False)
        self._programs = {}                # shape -> (Program, logits), in order of last use
        self._programs_generation = -1     # the workspace generation the lists were recorded for
        self.program_runs = 0
        self.programs_recorded = 0         # steps that ran from the parts and left a launch list
        self.last_program = None           # the launch list of the latest step, if it ran from one or left one
        self._meta = None                  # device int32 buffer of eager steps
        self._pinned = []                  # ring of (pinned int32 tensor, event)
        self._pinned_next = 0
        self._graphs = {}                  # shape -> dict(graph, meta, logits, generation), in order of last use
        self._seen = {}                    # shape -> times it came without a graph
        # shape -> True (its launch list keeps the GPU busy: no graph), False (the host is the limit:
        # graph), or the measurements under way: [(host seconds of the walk, start event, end event)]
        self._launch_bound = {}
        self._walk_seconds = None          # host time of the latest walk of a launch list
        self.graphs_declined = 0           # shapes that were measured and left to their launch lists
        self.steps_run = 0
        self.graph_replays = 0

    # --- sequences -------------------------------------------------------------------------
    def open(self):
        """A slot for a new sequence."""
        return self.cache.acquire()

    def close(self, slot):
        """Ends a sequence: its slot and its blocks can be used again."""
        self.cache.release(slot)

    def length(self, slot):
        return self.cache.length(slot)

    def truncate(self, slot, length):
        """Rewinds a sequence to its first ``length`` tokens; later steps go on from there."""
        self.cache.truncate(slot, length)

    def reset(self):
        """Ends every sequence (the reference's reset, src/architecture/traits.rs:64)."""
        for slot in self.cache.ledger.live_slots():
            self.cache.release(slot)

    # --- the step function -----------------------------------------------------------------
    def plan(self, entries, want=None):
        """Validates a step and lays its tables out on the host.  Changes nothing.

        An entry that brings no token is idle: it runs nothing, writes nothing and keeps its length
        (the reference's decode rows without a valid token, src/models/llama/model/decode.rs:43-44).
        ``active`` names the entries that bring tokens, ``idle_rows`` the places in the step's
        logits that idle entries take (one row of zeros each when the places are not given:
        decode.rs:730-751)."""
        ledger = self.cache.ledger
        slots, starts, counts, ids, active = [], [], [], [], []
        limit = min(self.model.max_positions, self.cache.max_sequence_length)
        vocab = self.model.vocab_size
        if want is not None and len(want) != len(entries):
            raise StepError("`want` needs one list of places per sequence")
        seen = set()
        for index, (slot, tokens) in enumerate(entries):
            if not ledger.live(slot):
                raise StepError(f"slot {slot} is not open")
            if slot in seen:
                raise StepError(f"slot {slot} appears twice in one step")
            seen.add(slot)
            if type(tokens) is list and len(tokens) == 1 and type(tokens[0]) is int:
                size, low, high = 1, tokens[0], tokens[0]      # a decode step's entry: no array is made for it
                ids.append(tokens[0])
            else:
                tokens = np.asarray(tokens)
                if tokens.size and tokens.dtype.kind not in "iu":
                    raise StepError(f"token ids of slot {slot} are {tokens.dtype} values, expected integers")
                tokens = tokens.astype(np.int64).reshape(-1)
                size = int(tokens.size)
                if size == 0:
                    if want is not None and len(want[index]):
                        raise StepError(f"wanted place {want[index][0]} of slot {slot} is outside its 0 tokens")
                    continue
                low, high = int(tokens.min()), int(tokens.max())
                ids.extend(tokens.tolist())
            if low < 0 or high >= vocab:
                raise StepError(f"token ids of slot {slot} lie in {low}..={high}, "
                                f"expected token values in 0..{vocab}")
            start = ledger.lengths[slot]
            if start + size > limit:
                raise StepError(f"slot {slot} would reach {start + size} tokens, "
                                f"the limit is {limit}")
            active.append(index)
            slots.append(slot)
            starts.append(start)
            counts.append(size)
        offsets = np.concatenate([[0], np.cumsum(counts)]) if counts else np.zeros(1, dtype=np.int64)
        idle_rows = None
        if want is None:
            wanted = [int(offsets[i + 1] - 1) for i in range(len(active))]
            if len(active) != len(entries):         # a row of zeros for every idle entry, where its logits would be
                idle_rows = [i for i in range(len(entries)) if i not in set(active)]
        else:
            wanted = []
            for i, index in enumerate(active):
                for place in want[index]:
                    if not (0 <= place < counts[i]):
                        raise StepError(f"wanted place {place} of slot {slots[i]} is outside its "
                                        f"{counts[i]} tokens")
                    wanted.append(int(offsets[i] + place))
        new_lengths = {s: st + c for s, st, c in zip(slots, starts, counts)}
        try:
            ledger.check_growth(new_lengths)
        except RuntimeError as error:
            raise StepError(str(error)) from error
        # block rows are read after the reservation, in `step`
        return dict(slots=slots, starts=starts, counts=counts, ids=ids, wanted=wanted, new_lengths=new_lengths,
                    active=active, idle_rows=idle_rows, n_entries=len(entries))

    def step(self, entries, want=None, device_tokens=None):
        """Runs one step; returns float32 logits [wanted places, vocab] on the GPU, valid until the
        next step.  ``entries``: [(slot, token ids)], ``want``: per entry the places among its
        tokens whose logits are wanted (default: each entry's last token).

        ``device_tokens``: for a step of one token per sequence, an int32 tensor on the GPU that
        holds the tokens themselves, in the order of the entries (whose own token is then only a
        placeholder): what a selection kernel has just chosen can feed the next step before the
        host has read it, so the host's work on a step overlaps the GPU's work on the one before.
        The ids are not validated (a selection cannot choose outside the vocabulary)."""
        checked = self.plan(entries, want)
        if device_tokens is not None:
            if len(checked["active"]) != len(entries) or max(checked["counts"], default=0) != 1 or \
                    device_tokens.numel() != len(entries) or \
                    device_tokens.dtype != torch.int32 or device_tokens.device != self.device:
                raise StepError("device_tokens: one int32 token on this GPU for each sequence of a step of single tokens")
        if not checked["active"]:
            # No entry brings a token: nothing runs and nothing is committed; the logits are exact
            # zeros of the shape asked for (src/models/llama/model/decode.rs:648-650, 730-751)
            return torch.zeros((len(checked["idle_rows"] or ()), self.model.vocab_size), dtype=torch.float32,
                               device=self.device)
        ledger = self.cache.ledger
        for slot, length in checked["new_lengths"].items():
            ledger.reserve(slot, length)
        try:
            plan = StepPlan(checked["slots"], checked["starts"], checked["counts"], checked["ids"],
                            checked["wanted"], self.cache.block_rows(checked["slots"]), self.cache.max_blocks)
            plan.device_tokens = device_tokens
            if self.use_graphs:
                logits = self._run_from_graph(plan, readout=bool(checked["wanted"]))
            else:
                logits = self._run_eager(plan, want_logits=bool(checked["wanted"]))
        except BaseException:
            # A pass that fails half-way (a kernel refuses its operands, a workspace cannot grow, the
            # library reports an error) leaves every sequence as long as it was: the blocks reserved
            # for this step go back, and what the pass wrote lies beyond the committed lengths, where
            # nothing reads (src/models/llama/model/decode.rs:38-41; the reference's test of it is
            # decode_tests.rs:762).  Fixed-size state is written by a mixer only after its own
            # kernels were launched; a model that keeps such state is told to drop the sequences.
            for slot in checked["new_lengths"]:
                ledger.truncate(slot, ledger.lengths[slot])
            raise
        for slot, length in checked["new_lengths"].items():
            ledger.commit(slot, length)
        self.steps_run += 1
        if checked["idle_rows"]:          # rows of zeros where idle entries' logits would be
            whole = torch.zeros((checked["n_entries"], self.model.vocab_size), dtype=torch.float32, device=self.device)
            whole[torch.tensor(checked["active"], device=self.device)] = logits
            return whole
        return logits

    # --- running ---------------------------------------------------------------------------
    def _upload(self, host, device_meta):
        """One copy of the step's tables to the GPU through a pinned staging buffer."""
        if len(self._pinned) < _PINNED_RING:
            self._pinned.append([torch.empty(max(host.size, 4096), dtype=torch.int32, pin_memory=True),
                                 torch.cuda.Event()])
        entry = self._pinned[self._pinned_next % len(self._pinned)]
        self._pinned_next += 1
        entry[1].synchronize()                       # the copy that last used this buffer is done
        if entry[0].numel() < host.size:
            entry[0] = torch.empty(host.size * 2, dtype=torch.int32, pin_memory=True)
        entry[0][:host.size].numpy()[:] = host
        device_meta[:host.size].copy_(entry[0][:host.size], non_blocking=True)
        entry[1].record()

    def _upload_plan(self, plan, device_meta):
        """The step's tables, and over their token ids the tokens that are on the GPU already."""
        self._upload(plan.host, device_meta)
        if plan.device_tokens is not None:
            offset, size = plan.layout.sections["tok_ids"]
            device_meta[offset:offset + size].copy_(plan.device_tokens, non_blocking=True)

    def _run_eager(self, plan, want_logits=True):
        if self._meta is None or self._meta.numel() < plan.layout.total:
            self._meta = torch.empty(max(plan.layout.total * 2, _META_WORDS), dtype=torch.int32, device=self.device)
            self._programs.clear()                        # they name the old tables
        self._upload_plan(plan, self._meta)
        if self.use_programs:
            return self._run_program(plan, want_logits)
        step = Step(plan.layout, self._meta, self.pool, self.dtype, plan)
        if not want_logits:       # a step whose logits nobody wants still has to fill the cache
            self.model.forward(step, self.cache, readout=False)
            return torch.empty((0, self.model.vocab_size), dtype=torch.float32, device=self.device)
        return self.model.forward(step, self.cache)

    def _run_program(self, plan, readout):
        """The step from its launch list.  The first time a class of steps comes (``token_capacity``:
        a step of up to 64 tokens is a class of its own) the parts run as always and launch as they
        go (the GPU starts at once), and every kernel call is kept as well; from then on the list is
        walked in C++, for any step of the class: the counts in its calls are set to the step's
        (``Program.set_shape``), everything else in them (addresses of weights, workspaces and
        tables, pitches, kernels chosen) is the same for the whole class.  A list names workspaces
        by address, so a workspace that had to grow makes all lists stale, and a list recorded while
        one grew is not kept."""
        if self._programs_generation != self.pool.generation:
            self._programs.clear()
            self._programs_generation = self.pool.generation
            # (measurements under way were of lists that are gone; decisions taken stay)
            self._launch_bound = {k: v for k, v in self._launch_bound.items() if isinstance(v, bool)}
        layout = plan.layout
        exact = (layout.key(), plan.max_count, readout, plan.context_limit)
        # a step of more than 64 tokens that is not one of single tokens shares its list with its class
        shared = (layout.class_key(), readout, plan.context_limit) if layout.tokens > BLOCK and plan.max_count > 1 else None
        key = shared if shared is not None and shared in self._programs else exact
        held = self._programs.pop(key, None)
        if held is not None:
            program, logits = held
            if program.patches is not None:
                program.set_shape(layout.tokens, plan.max_count)
            self._programs[key] = held                    # (again) the most recently used
            self.last_program = program
            began = time.perf_counter()
            try:
                program.run()
            except K.KernelError:
                if program.patches is None:
                    raise
                # a kernel refused the counts of this step of the class (the vendor's library has no
                # algorithm for its rows, say): the list is dropped and the step runs from the parts
                self._programs.pop(key, None)
                return self._run_program(plan, readout)
            self._walk_seconds = time.perf_counter() - began
            self.program_runs += 1
            return logits
        step = Step(layout, self._meta, self.pool, self.dtype, plan)
        generation = self.pool.generation
        program = K.Program()
        with program.recording(launch=True):
            logits = self.model.forward(step, self.cache, readout=readout)
        if not readout:
            logits = torch.empty((0, self.model.vocab_size), dtype=torch.float32, device=self.device)
        self.last_program = None
        self.programs_recorded += 1
        if self.pool.generation != generation:
            # A workspace grew while the step ran.  The launches themselves were in order and are
            # right, but calls recorded before the growth name the old address, and so do all
            # older lists: none is kept, and the shape records again when it next comes (the
            # workspaces are then large enough from the start).
            self._programs.clear()
            self._programs_generation = self.pool.generation
            return logits
        key = exact
        if shared is not None and program.for_any_step_of_its_class(layout.tokens, plan.max_count, layout.rows):
            key = shared
        while len(self._programs) >= _MAX_PROGRAMS:
            self._programs.pop(next(iter(self._programs)))
        self._programs[key] = (program, logits)
        self.last_program = program
        return logits

    def _run_from_graph(self, plan, readout):
        # (parts plan by the class of context: how many runs the keys of a decode step or of a chunk are cut into)
        key = (plan.layout.key(), plan.max_count, readout, plan.context_limit)
        held = self._graphs.pop(key, None)
        if held is not None and held["generation"] != self.pool.generation:
            held = None                                   # a workspace moved: the graph is stale
        if held is None:
            if self._launch_bound.get(key) is True:       # measured: a graph would gain nothing here
                return self._run_eager(plan, want_logits=readout)
            # the first times a shape comes it runs eagerly, which also sizes the workspaces
            seen = self._seen.get(key, 0)
            if seen < (1 if plan.decode else 2):
                if len(self._seen) > 4096:
                    self._seen.clear()
                self._seen[key] = seen + 1
                return self._run_eager(plan, want_logits=readout)
            if self.use_programs and not self._graphs_always and not self._graph_pays(key, plan, readout):
                return self._latest_logits
            held = self._capture(plan, readout)
            while len(self._graphs) >= _MAX_GRAPHS:
                self._graphs.pop(next(iter(self._graphs)))
        self._graphs[key] = held                          # (again) the most recently used
        self._upload_plan(plan, held["meta"])
        held["graph"].replay()
        self.graph_replays += 1
        return held["logits"]

    def _graph_pays(self, key, plan, readout):
        """Whether the shape should be captured, found out by measuring its launch list.

        A graph removes the host's cost of launching a step's kernels.  That cost is hidden anyway
        where the kernels keep the GPU busy for longer than the host needs to launch them (every
        dependent kernel takes the GPU some microseconds however little it does, and the C++ walk
        launches one in about three): then a graph gains nothing and costs its capture, a stall of
        the pipeline, and memory.  So the steps that would have been captured run from their list
        between two events while the host's time for the walk alone is taken (not the upload of the
        step's tables, which may wait for an older copy); after ``_PROBES`` such steps the GPU's
        times are read (one wait, shorter than a capture's) and ``launch_bound`` decides by the
        median.  Returns False when it ran the step itself (the logits are in ``_latest_logits``)."""
        probe = self._launch_bound.get(key)
        if probe is False:
            return True
        if probe is None:
            if len(self._launch_bound) > 4096:
                self._launch_bound.clear()
            probe = self._launch_bound[key] = []
        shared = (plan.layout.class_key(), readout, plan.context_limit)
        if key not in self._programs and shared not in self._programs and self._seen.get(key, 0) < 8:
            # the shape has no list (its first step made a workspace grow, or the lists were dropped
            # since): this step would be launched from Python and say nothing about the list; it
            # records, the next one is measured
            self._seen[key] = self._seen.get(key, 0) + 1
            self._latest_logits = self._run_eager(plan, want_logits=readout)
            return False
        if len(probe) < _PROBES:
            start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record()
            self._walk_seconds = None
            self._latest_logits = self._run_eager(plan, want_logits=readout)
            end.record()
            if self._walk_seconds is not None:        # (None: the step recorded its list anew and says nothing)
                probe.append((self._walk_seconds, start, end))
            return False
        samples = []
        for host_seconds, start, end in probe:
            end.synchronize()
            samples.append((start.elapsed_time(end) * 1e-3, host_seconds))
        self._launch_bound[key] = launch_bound(samples)
        if self._launch_bound[key]:
            self.graphs_declined += 1
            self._latest_logits = self._run_eager(plan, want_logits=readout)
            return False
        return True

    def _capture(self, plan, readout):
        meta = torch.empty(plan.layout.total, dtype=torch.int32, device=self.device)
        self._upload(plan.host, meta)
        step = Step(plan.layout, meta, self.pool, self.dtype, plan)
        torch.cuda.synchronize(self.device)
        graph = torch.cuda.CUDAGraph()
        self.pool.frozen = True
        try:
            with torch.cuda.graph(graph):
                logits = self.model.forward(step, self.cache, readout=readout)
        finally:
            self.pool.frozen = False
        if not readout:
            logits = torch.empty((0, self.model.vocab_size), dtype=torch.float32, device=self.device)
        return dict(graph=graph, meta=meta, logits=logits, generation=self.pool.generation)
